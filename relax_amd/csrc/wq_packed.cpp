// TVM PackedFunc boundary (include/mi355x_wq_packed.h): unpacks DLPack tensors
// handed over by Relax's VM, validates them and forwards to the C ABI.
#include <dlfcn.h>
#include <hip/hip_runtime_api.h>

#include <cstdio>
#include <cstring>

#include "../../include/mi355x_wq.h"
#include "../../include/mi355x_wq_packed.h"
#include "wq_internal.h"

namespace {

thread_local void* g_stream = nullptr;

// Report through TVM's error slot when the host process has one, so that the
// loader's `LOG(FATAL) << TVMGetLastError()` shows our message.
int fail() {
  typedef void (*set_last_error_t)(const char*);
  static set_last_error_t fn =
      reinterpret_cast<set_last_error_t>(dlsym(RTLD_DEFAULT, "TVMAPISetLastError"));
  if (fn != nullptr) fn(mi355x_wq_last_error());
  return -1;
}

struct Dtype {
  uint8_t code, bits;
  const char* name;
};
constexpr Dtype kF16{2, 16, "float16"};
constexpr Dtype kU32{1, 32, "uint32"};
constexpr Dtype kU8{1, 8, "uint8"};

// Checks one tensor argument; on success stores the (byte_offset adjusted) pointer.
// `vector_ok`: the tensor may be 1-d [N] (reported as rows = 1, cols = N).
// `fold_leading`: any rank from 1 on, compact row-major; the extents before the last are folded into the rows
// (x[B, S, K] is B * S rows of K: relax.matmul broadcasts the leading extents of x over a 2-d weight,
// src/relax/op/tensor/linear_algebra.cc:46-114).
bool take_tensor(mi355x_tvm_value* args, int* type_codes, int idx, const char* role, Dtype want,
                 int device_id_expected, const mi355x_dl_tensor** out, void** ptr,
                 bool vector_ok = false, int64_t* rows = nullptr, int64_t* cols = nullptr, bool fold_leading = false) {
  const int tc = type_codes[idx];
  if (tc != MI355X_TVM_DLTENSOR_HANDLE && tc != MI355X_TVM_NDARRAY_HANDLE) {
    wq::set_error("argument %d (%s): expected a tensor (type code 7 or 13), got type code %d", idx,
                  role, tc);
    return false;
  }
  const mi355x_dl_tensor* t = static_cast<const mi355x_dl_tensor*>(args[idx].v_handle);
  if (t == nullptr) {
    wq::set_error("argument %d (%s): NULL tensor handle", idx, role);
    return false;
  }
  if (vector_ok && t->ndim == 1 && t->shape != nullptr) {
    if (t->dtype.code != want.code || t->dtype.bits != want.bits || t->dtype.lanes != 1) {
      wq::set_error("argument %d (%s): expected dtype %s, got code=%d bits=%d lanes=%d", idx, role,
                    want.name, t->dtype.code, t->dtype.bits, t->dtype.lanes);
      return false;
    }
    if (t->device.device_type != MI355X_DL_ROCM ||
        (device_id_expected >= 0 && t->device.device_id != device_id_expected)) {
      wq::set_error("argument %d (%s): expected a ROCm tensor on device %d, got device type %d id %d",
                    idx, role, device_id_expected, t->device.device_type, t->device.device_id);
      return false;
    }
    if (t->shape[0] < 0 || (t->strides != nullptr && t->shape[0] > 1 && t->strides[0] != 1) ||
        (t->data == nullptr && t->shape[0] != 0)) {
      wq::set_error("argument %d (%s): a 1-d tensor must be compact with a data pointer", idx, role);
      return false;
    }
    *out = t;
    *ptr = static_cast<char*>(t->data) + t->byte_offset;
    if (rows != nullptr) *rows = 1;
    if (cols != nullptr) *cols = t->shape[0];
    return true;
  }
  if (fold_leading && t->shape != nullptr && t->ndim >= 1 && t->ndim != 2) {
    if (t->dtype.code != want.code || t->dtype.bits != want.bits || t->dtype.lanes != 1) {
      wq::set_error("argument %d (%s): expected dtype %s, got code=%d bits=%d lanes=%d", idx, role,
                    want.name, t->dtype.code, t->dtype.bits, t->dtype.lanes);
      return false;
    }
    if (t->device.device_type != MI355X_DL_ROCM ||
        (device_id_expected >= 0 && t->device.device_id != device_id_expected)) {
      wq::set_error("argument %d (%s): expected a ROCm tensor on device %d, got device type %d id %d",
                    idx, role, device_id_expected, t->device.device_type, t->device.device_id);
      return false;
    }
    if (t->ndim > 8) {
      wq::set_error("argument %d (%s): at most 8 dimensions, got %d", idx, role, t->ndim);
      return false;
    }
    int64_t lead = 1, expect = 1;
    bool compact = true;
    for (int d = t->ndim - 1; d >= 0; --d) {
      if (t->shape[d] < 0 || (d < t->ndim - 1 && t->shape[d] != 0 && lead > (int64_t)0x7FFFFFFF / t->shape[d])) {
        wq::set_error("argument %d (%s): negative or oversized extent", idx, role);
        return false;
      }
      if (t->strides != nullptr && t->shape[d] > 1 && t->strides[d] != expect) compact = false;
      expect *= t->shape[d];
      if (d < t->ndim - 1) lead *= t->shape[d];
    }
    if (!compact) {
      wq::set_error("argument %d (%s): a %d-d tensor must be compact row-major", idx, role, t->ndim);
      return false;
    }
    if (t->data == nullptr && expect != 0) {
      wq::set_error("argument %d (%s): NULL data pointer", idx, role);
      return false;
    }
    *out = t;
    *ptr = static_cast<char*>(t->data) + t->byte_offset;
    if (rows != nullptr) *rows = lead;
    if (cols != nullptr) *cols = t->shape[t->ndim - 1];
    return true;
  }
  if (t->ndim != 2 || t->shape == nullptr) {
    wq::set_error("argument %d (%s): expected a 2-d tensor, got ndim=%d", idx, role, t->ndim);
    return false;
  }
  if (t->dtype.code != want.code || t->dtype.bits != want.bits || t->dtype.lanes != 1) {
    wq::set_error("argument %d (%s): expected dtype %s, got code=%d bits=%d lanes=%d", idx, role,
                  want.name, t->dtype.code, t->dtype.bits, t->dtype.lanes);
    return false;
  }
  if (t->device.device_type != MI355X_DL_ROCM) {
    wq::set_error("argument %d (%s): expected a ROCm tensor (device type 10), got device type %d",
                  idx, role, t->device.device_type);
    return false;
  }
  if (device_id_expected >= 0 && t->device.device_id != device_id_expected) {
    wq::set_error("argument %d (%s): on device %d but the first tensor is on device %d", idx, role,
                  t->device.device_id, device_id_expected);
    return false;
  }
  if (t->shape[0] < 0 || t->shape[1] < 0) {
    wq::set_error("argument %d (%s): negative extent", idx, role);
    return false;
  }
  if (t->strides != nullptr) {
    // only compact row-major; a stride is irrelevant where the extent is 1
    const bool ok1 = t->shape[1] <= 1 || t->strides[1] == 1;
    const bool ok0 = t->shape[0] <= 1 || t->strides[0] == t->shape[1];
    if (!ok0 || !ok1) {
      wq::set_error("argument %d (%s): strides (%lld, %lld) are not compact row-major for shape (%lld, %lld)",
                    idx, role, (long long)t->strides[0], (long long)t->strides[1],
                    (long long)t->shape[0], (long long)t->shape[1]);
      return false;
    }
  }
  if (t->data == nullptr && t->shape[0] * t->shape[1] != 0) {
    wq::set_error("argument %d (%s): NULL data pointer", idx, role);
    return false;
  }
  *out = t;
  *ptr = static_cast<char*>(t->data) + t->byte_offset;
  if (rows != nullptr) *rows = t->shape[0];
  if (cols != nullptr) *cols = t->shape[1];
  return true;
}

}  // namespace

extern "C" {

void mi355x_wq_packed_set_stream(void* stream) { g_stream = stream; }
void* mi355x_wq_packed_get_stream(void) { return g_stream; }

int mi355x_wq_packed_call(const mi355x_wq_callspec* spec, mi355x_tvm_value* args, int* type_codes,
                          int num_args) {
  return wq::packed_call_with_weights(spec, args, type_codes, num_args, nullptr, nullptr);
}

int mi355x_wq_packed_call_scratch(const mi355x_wq_callspec* spec, mi355x_tvm_value* args, int* type_codes,
                                  int num_args) {
  return wq::packed_call_with_weights(spec, args, type_codes, num_args, nullptr, nullptr, true);
}

}  // extern "C"

int wq::packed_fail() { return fail(); }

int wq::packed_call_with_weights(const mi355x_wq_callspec* spec, mi355x_tvm_value* args, int* type_codes,
                                 int num_args, const void* wq_tiled, const void* scales_tiled, bool library_scratch,
                                 void* workspace, int64_t workspace_bytes) {
  if (spec == nullptr) {
    wq::set_error("call spec is NULL");
    return fail();
  }
  const bool is_matmul = spec->op == 0;
  if (spec->op != 0 && spec->op != 1) {
    wq::set_error("call spec: unknown op %d", spec->op);
    return fail();
  }
  const bool has_bias = is_matmul && spec->arg_bias >= 0;
  const bool has_res = is_matmul && spec->arg_residual >= 0;
  if (!is_matmul && (spec->arg_bias >= 0 || spec->arg_residual >= 0 || spec->activation != 0)) {
    wq::set_error("call spec: dequantize takes no fused operands");
    return fail();
  }
  const int expect = (is_matmul ? 4 : 3) + (has_bias ? 1 : 0) + (has_res ? 1 : 0);
  if (num_args != expect || spec->num_args != expect) {
    wq::set_error("%s expects %d arguments, got %d", is_matmul ? "matmul" : "dequantize", expect,
                  num_args);
    return fail();
  }
  if (args == nullptr || type_codes == nullptr) {
    wq::set_error("NULL argument array");
    return fail();
  }
  // role indices must be a permutation of 0..expect-1
  int roles[6] = {spec->arg_wq, spec->arg_scales, spec->arg_out, 0, 0, 0};
  int nroles = 3;
  if (is_matmul) roles[nroles++] = spec->arg_x;
  if (has_bias) roles[nroles++] = spec->arg_bias;
  if (has_res) roles[nroles++] = spec->arg_residual;
  unsigned seen = 0;
  for (int i = 0; i < nroles; ++i) {
    if (roles[i] < 0 || roles[i] >= expect || (seen & (1u << roles[i]))) {
      wq::set_error("call spec: argument roles are not a permutation of 0..%d", expect - 1);
      return fail();
    }
    seen |= 1u << roles[i];
  }

  const mi355x_dl_tensor *tx = nullptr, *tw = nullptr, *ts = nullptr, *to = nullptr;
  void *px = nullptr, *pw = nullptr, *ps = nullptr, *po = nullptr;
  if (!take_tensor(args, type_codes, spec->arg_wq, "wq", kU32, -1, &tw, &pw)) return fail();
  const int dev = tw->device.device_id;
  if (!take_tensor(args, type_codes, spec->arg_scales, "scales", kF16, dev, &ts, &ps)) return fail();
  int64_t out_rows = 0, out_cols = 0, x_rows = 0, x_cols = 0;
  if (!take_tensor(args, type_codes, spec->arg_out, is_matmul ? "y" : "wd", kF16, dev, &to, &po, false, &out_rows, &out_cols,
                   is_matmul))
    return fail();
  if (is_matmul && !take_tensor(args, type_codes, spec->arg_x, "x", kF16, dev, &tx, &px, false, &x_rows, &x_cols, true))
    return fail();
  // the output (and the residual) repeat the leading extents of x
  auto same_leading = [](const mi355x_dl_tensor* a, const mi355x_dl_tensor* b) {
    if (a->ndim != b->ndim) return false;
    for (int d = 0; d + 1 < a->ndim; ++d)
      if (a->shape[d] != b->shape[d]) return false;
    return true;
  };

  const int per_word = 32 / (spec->bits == 8 ? 8 : 4);
  mi355x_wq_desc d;
  memset(&d, 0, sizeof(d));
  d.bits = spec->bits;
  d.zero_point = spec->zero_point;
  d.n = tw->shape[0];
  d.k = tw->shape[1] * per_word;
  if (ts->shape[0] != d.n) {
    wq::set_error("scales has %lld rows but wq has %lld", (long long)ts->shape[0], (long long)d.n);
    return fail();
  }
  if (spec->group > 0) {
    d.group = spec->group;
    if (d.k % d.group != 0 || ts->shape[1] != d.k / d.group) {
      wq::set_error("scales shape (%lld, %lld) does not match K=%lld / group=%d", (long long)ts->shape[0],
                    (long long)ts->shape[1], (long long)d.k, d.group);
      return fail();
    }
  } else {
    if (ts->shape[1] <= 0 || d.k % ts->shape[1] != 0) {
      wq::set_error("cannot infer the group size: K=%lld, scales has %lld columns", (long long)d.k,
                    (long long)ts->shape[1]);
      return fail();
    }
    d.group = (int32_t)(d.k / ts->shape[1]);
  }

  int64_t m = 0;
  if (is_matmul) {
    m = x_rows;
    if (x_cols != d.k) {
      wq::set_error("x has %lld columns but the weights have K=%lld", (long long)x_cols,
                    (long long)d.k);
      return fail();
    }
    // the gated tail halves the output: y[M, N/2] = multiply(nn.silu(gate), up)
    const bool gated_out = spec->activation == MI355X_WQ_ACT_SILU_MUL;
    if (gated_out && d.n % 2 != 0) {
      wq::set_error("the gated tail (silu_mul) needs an even N, got %lld", (long long)d.n);
      return fail();
    }
    const int64_t want_cols = gated_out ? d.n / 2 : d.n;
    if (out_rows != m || out_cols != want_cols || !same_leading(to, tx)) {
      wq::set_error("y has shape (%lld, %lld), expected (%lld, %lld)%s", (long long)out_rows,
                    (long long)out_cols, (long long)m, (long long)want_cols,
                    same_leading(to, tx) ? "" : " with the leading extents of x");
      return fail();
    }
  } else if (to->shape[0] != d.n || to->shape[1] != d.k) {
    wq::set_error("wd has shape (%lld, %lld), expected (%lld, %lld)", (long long)to->shape[0],
                  (long long)to->shape[1], (long long)d.n, (long long)d.k);
    return fail();
  }
  mi355x_wq_epilogue ep;
  memset(&ep, 0, sizeof(ep));
  ep.activation = spec->activation;
  if (has_bias) {
    const mi355x_dl_tensor* tb = nullptr;
    void* pb = nullptr;
    int64_t br = 0, bc = 0;
    if (!take_tensor(args, type_codes, spec->arg_bias, "bias", kF16, dev, &tb, &pb, true, &br, &bc, true))
      return fail();
    if (br != 1 || bc != d.n) {
      wq::set_error("bias has shape (%lld, %lld), expected (%lld) or (1, %lld)", (long long)br,
                    (long long)bc, (long long)d.n, (long long)d.n);
      return fail();
    }
    ep.bias = pb;
  }
  if (has_res) {
    const mi355x_dl_tensor* tr = nullptr;
    void* pr = nullptr;
    int64_t rr = 0, rc = 0;
    if (!take_tensor(args, type_codes, spec->arg_residual, "residual", kF16, dev, &tr, &pr, false, &rr, &rc, true))
      return fail();
    if (rr != m || rc != d.n || !same_leading(tr, tx)) {
      wq::set_error("residual has shape (%lld, %lld), expected (%lld, %lld)%s", (long long)rr,
                    (long long)rc, (long long)m, (long long)d.n, same_leading(tr, tx) ? "" : " with the leading extents of x");
      return fail();
    }
    ep.residual = pr;
  }
  if (mi355x_wq_check(&d, m) != 0) return fail();
  if (d.n == 0 || (is_matmul && m == 0)) return 0;  // nothing to compute

  int cur = -1;
  if (hipGetDevice(&cur) != hipSuccess) {
    (void)hipGetLastError();
    wq::set_error("no usable HIP device in this process");
    return fail();
  }
  if (cur != dev) {
    wq::set_error("tensors live on ROCm device %d but the current HIP device is %d", dev, cur);
    return fail();
  }
  if (workspace != nullptr && is_matmul) {
    // a workspace the caller (the subgraph module) owns: the K split of decode and prefill calls where it pays;
    // anything else, and a workspace that is too small, runs as the plain call
    const bool tiled = wq_tiled != nullptr;
    return mi355x_wq_matmul_ws(&d, px, tiled ? wq_tiled : pw, tiled ? scales_tiled : ps, &ep, po, m, g_stream,
                               tiled ? 1 : 0, workspace, workspace_bytes) == 0 ? 0 : fail();
  }
  if (library_scratch && is_matmul) {
    // decode calls may split K across workgroups on the library's own scratch array (no allocation); a split
    // that would need more than the array holds runs unsplit -- the option is a speed-up, never a reason to fail
    const bool tiled = wq_tiled != nullptr;
    if (mi355x_wq_workspace_bytes(&d, m, tiled ? 1 : 0) <= mi355x_wq_static_ws_bytes())
      return mi355x_wq_matmul_static_ws(&d, px, tiled ? wq_tiled : pw, tiled ? scales_tiled : ps, &ep, po, m, g_stream,
                                        tiled ? 1 : 0) == 0 ? 0 : fail();
  }
  if (wq_tiled != nullptr && is_matmul)
    return mi355x_wq_matmul_tiled(&d, px, wq_tiled, scales_tiled, &ep, po, m, g_stream) == 0 ? 0 : fail();
  const int rc = is_matmul ? mi355x_wq_matmul_fused(&d, px, pw, ps, &ep, po, m, g_stream)
                           : mi355x_wq_dequantize(&d, pw, ps, po, g_stream);
  return rc == 0 ? 0 : fail();
}

extern "C" {

// Fixed-name entries: arguments in the canonical order x, wq, scales, [bias | residual], out.
#define MI355X_FIXED_ENTRY(NAME, OP, BITS, ZP, BIAS, RES, ACT)                                      \
  int NAME(mi355x_tvm_value* args, int* type_codes, int num_args, mi355x_tvm_value*, int*, void*) { \
    static const mi355x_wq_callspec spec = {                                                        \
        OP, BITS, 0, ZP, 0, (OP) == 0 ? 1 : 0, (OP) == 0 ? 2 : 1,                                   \
        ((OP) == 0 ? 3 : 2) + (BIAS) + (RES), ((OP) == 0 ? 4 : 3) + (BIAS) + (RES),                 \
        (BIAS) ? 3 : -1, (RES) ? 3 : -1, ACT};                                                      \
    return mi355x_wq_packed_call(&spec, args, type_codes, num_args);                                \
  }
MI355X_FIXED_ENTRY(mi355x_q4f16_matmul, 0, 4, 7, 0, 0, 0)
MI355X_FIXED_ENTRY(mi355x_q8f16_matmul, 0, 8, 0, 0, 0, 0)
MI355X_FIXED_ENTRY(mi355x_q4f16_matmul_bias, 0, 4, 7, 1, 0, 0)
MI355X_FIXED_ENTRY(mi355x_q8f16_matmul_bias, 0, 8, 0, 1, 0, 0)
MI355X_FIXED_ENTRY(mi355x_q4f16_matmul_bias_relu, 0, 4, 7, 1, 0, MI355X_WQ_ACT_RELU)
MI355X_FIXED_ENTRY(mi355x_q8f16_matmul_bias_relu, 0, 8, 0, 1, 0, MI355X_WQ_ACT_RELU)
MI355X_FIXED_ENTRY(mi355x_q4f16_matmul_bias_gelu, 0, 4, 7, 1, 0, MI355X_WQ_ACT_GELU)
MI355X_FIXED_ENTRY(mi355x_q8f16_matmul_bias_gelu, 0, 8, 0, 1, 0, MI355X_WQ_ACT_GELU)
MI355X_FIXED_ENTRY(mi355x_q4f16_matmul_residual, 0, 4, 7, 0, 1, 0)
MI355X_FIXED_ENTRY(mi355x_q8f16_matmul_residual, 0, 8, 0, 0, 1, 0)
MI355X_FIXED_ENTRY(mi355x_q4f16_matmul_silu_mul, 0, 4, 7, 0, 0, MI355X_WQ_ACT_SILU_MUL)
MI355X_FIXED_ENTRY(mi355x_q8f16_matmul_silu_mul, 0, 8, 0, 0, 0, MI355X_WQ_ACT_SILU_MUL)
MI355X_FIXED_ENTRY(mi355x_q4f16_dequantize, 1, 4, 7, 0, 0, 0)
MI355X_FIXED_ENTRY(mi355x_q8f16_dequantize, 1, 8, 0, 0, 0, 0)
#undef MI355X_FIXED_ENTRY

// ---- tile-major layout: the one-off transform and the matmul on its output ----------------
// tile_weights(wq[N,K*bits/32], scales[N,K/group], wq_tiled[Np,K*bits/32], scales_tiled[Np,K/group])
// matmul_tiled(x[M,K], wq_tiled[Np,...], scales_tiled[Np,...], y[M,N]) with Np = N rounded up to 16:
// the tile-major buffers are passed as tensors of the canonical shape with whole tiles of rows.
static int packed_tiled(bool is_matmul, int bits, int zero_point, mi355x_tvm_value* args, int* type_codes,
                        int num_args) {
  if (num_args != 4 || args == nullptr || type_codes == nullptr) {
    wq::set_error("%s expects 4 tensor arguments, got %d", is_matmul ? "matmul_tiled" : "tile_weights", num_args);
    return fail();
  }
  const int iw = is_matmul ? 1 : 0, is = is_matmul ? 2 : 1;  // the weight / scale tensor that fixes K and group
  const mi355x_dl_tensor *t0 = nullptr, *tw = nullptr, *ts = nullptr, *t3 = nullptr, *t2 = nullptr;
  void *p0 = nullptr, *pw = nullptr, *ps = nullptr, *p3 = nullptr, *p2 = nullptr;
  if (!take_tensor(args, type_codes, iw, is_matmul ? "wq_tiled" : "wq", kU32, -1, &tw, &pw)) return fail();
  const int dev = tw->device.device_id;
  if (!take_tensor(args, type_codes, is, is_matmul ? "scales_tiled" : "scales", kF16, dev, &ts, &ps)) return fail();
  mi355x_wq_desc d;
  memset(&d, 0, sizeof(d));
  d.bits = bits;
  d.zero_point = zero_point;
  d.k = tw->shape[1] * (32 / bits);
  if (ts->shape[0] != tw->shape[0] || ts->shape[1] <= 0 || d.k % ts->shape[1] != 0) {
    wq::set_error("scales shape (%lld, %lld) does not match weights of %lld rows and K=%lld", (long long)ts->shape[0],
                  (long long)ts->shape[1], (long long)tw->shape[0], (long long)d.k);
    return fail();
  }
  d.group = (int32_t)(d.k / ts->shape[1]);
  int64_t m = 0;
  if (is_matmul) {
    if (!take_tensor(args, type_codes, 0, "x", kF16, dev, &t0, &p0)) return fail();
    if (!take_tensor(args, type_codes, 3, "y", kF16, dev, &t3, &p3)) return fail();
    m = t0->shape[0];
    d.n = t3->shape[1];
    if (t0->shape[1] != d.k || t3->shape[0] != m || tw->shape[0] != (d.n + 15) / 16 * 16) {
      wq::set_error("matmul_tiled: x (%lld, %lld), tiled weights of %lld rows and K=%lld, y (%lld, %lld) do not fit "
                    "(tiled rows must be N rounded up to 16)", (long long)t0->shape[0], (long long)t0->shape[1],
                    (long long)tw->shape[0], (long long)d.k, (long long)t3->shape[0], (long long)t3->shape[1]);
      return fail();
    }
  } else {
    d.n = tw->shape[0];
    if (!take_tensor(args, type_codes, 2, "wq_tiled", kU32, dev, &t2, &p2)) return fail();
    if (!take_tensor(args, type_codes, 3, "scales_tiled", kF16, dev, &t3, &p3)) return fail();
    const int64_t np = (d.n + 15) / 16 * 16;
    if (t2->shape[0] != np || t2->shape[1] != tw->shape[1] || t3->shape[0] != np || t3->shape[1] != ts->shape[1]) {
      wq::set_error("tile_weights: outputs must have the input shapes with %lld rows (N rounded up to 16)",
                    (long long)np);
      return fail();
    }
  }
  if (mi355x_wq_check(&d, m) != 0) return fail();
  if (d.n == 0 || (is_matmul && m == 0)) return 0;
  int cur = -1;
  if (hipGetDevice(&cur) != hipSuccess) {
    (void)hipGetLastError();
    wq::set_error("no usable HIP device in this process");
    return fail();
  }
  if (cur != dev) {
    wq::set_error("tensors live on ROCm device %d but the current HIP device is %d", dev, cur);
    return fail();
  }
  const int rc = is_matmul ? mi355x_wq_matmul_tiled(&d, p0, pw, ps, nullptr, p3, m, g_stream)
                           : mi355x_wq_tile_weights(&d, pw, ps, p2, p3, g_stream);
  return rc == 0 ? 0 : fail();
}

#define MI355X_TILED_ENTRY(NAME, IS_MATMUL, BITS, ZP)                                               \
  int NAME(mi355x_tvm_value* args, int* type_codes, int num_args, mi355x_tvm_value*, int*, void*) { \
    return packed_tiled(IS_MATMUL, BITS, ZP, args, type_codes, num_args);                           \
  }
MI355X_TILED_ENTRY(mi355x_q4f16_tile_weights, false, 4, 7)
MI355X_TILED_ENTRY(mi355x_q8f16_tile_weights, false, 8, 0)
MI355X_TILED_ENTRY(mi355x_q4f16_matmul_tiled, true, 4, 7)
MI355X_TILED_ENTRY(mi355x_q8f16_matmul_tiled, true, 8, 0)
#undef MI355X_TILED_ENTRY

// ---- decode with a workspace tensor: matmul_ws(x[M,K], wq[N,...], scales[N,...], workspace[bytes] u8, y[M,N])
static int packed_ws(int bits, int zero_point, mi355x_tvm_value* args, int* type_codes, int num_args) {
  if (num_args != 5 || args == nullptr || type_codes == nullptr) {
    wq::set_error("matmul_ws expects 5 tensor arguments (x, wq, scales, workspace, y), got %d", num_args);
    return fail();
  }
  const mi355x_dl_tensor *tx = nullptr, *tw = nullptr, *ts = nullptr, *tk = nullptr, *ty = nullptr;
  void *px = nullptr, *pw = nullptr, *ps = nullptr, *pk = nullptr, *py = nullptr;
  if (!take_tensor(args, type_codes, 1, "wq", kU32, -1, &tw, &pw)) return fail();
  const int dev = tw->device.device_id;
  int64_t wr = 0, wbytes = 0;
  if (!take_tensor(args, type_codes, 0, "x", kF16, dev, &tx, &px) ||
      !take_tensor(args, type_codes, 2, "scales", kF16, dev, &ts, &ps) ||
      !take_tensor(args, type_codes, 3, "workspace", kU8, dev, &tk, &pk, true, &wr, &wbytes) ||
      !take_tensor(args, type_codes, 4, "y", kF16, dev, &ty, &py))
    return fail();
  mi355x_wq_desc d;
  memset(&d, 0, sizeof(d));
  d.bits = bits;
  d.zero_point = zero_point;
  d.n = tw->shape[0];
  d.k = tw->shape[1] * (32 / bits);
  const int64_t m = tx->shape[0];
  if (ts->shape[0] != d.n || ts->shape[1] <= 0 || d.k % ts->shape[1] != 0 || tx->shape[1] != d.k ||
      ty->shape[0] != m || ty->shape[1] != d.n) {
    wq::set_error("matmul_ws: x (%lld, %lld), wq of %lld rows and K=%lld, scales (%lld, %lld), y (%lld, %lld) do not fit",
                  (long long)tx->shape[0], (long long)tx->shape[1], (long long)d.n, (long long)d.k,
                  (long long)ts->shape[0], (long long)ts->shape[1], (long long)ty->shape[0], (long long)ty->shape[1]);
    return fail();
  }
  d.group = (int32_t)(d.k / ts->shape[1]);
  if (mi355x_wq_check(&d, m) != 0) return fail();
  if (d.n == 0 || m == 0) return 0;
  int cur = -1;
  if (hipGetDevice(&cur) != hipSuccess) {
    (void)hipGetLastError();
    wq::set_error("no usable HIP device in this process");
    return fail();
  }
  if (cur != dev) {
    wq::set_error("tensors live on ROCm device %d but the current HIP device is %d", dev, cur);
    return fail();
  }
  return mi355x_wq_matmul_ws(&d, px, pw, ps, nullptr, py, m, g_stream, 0, wr * wbytes > 0 ? pk : nullptr, wr * wbytes) == 0
             ? 0
             : fail();
}
int mi355x_q4f16_matmul_ws(mi355x_tvm_value* args, int* type_codes, int num_args, mi355x_tvm_value*, int*, void*) {
  return packed_ws(4, 7, args, type_codes, num_args);
}
int mi355x_q8f16_matmul_ws(mi355x_tvm_value* args, int* type_codes, int num_args, mi355x_tvm_value*, int*, void*) {
  return packed_ws(8, 0, args, type_codes, num_args);
}

// ---- registration in TVM's global table through its C API -----------------------
typedef int (*backend_fn_t)(mi355x_tvm_value*, int*, int, mi355x_tvm_value*, int*, void*);

// TVMPackedCFunc has (args, type_codes, num_args, ret, resource_handle); the
// resource handle carries the backend-style entry to call.
static int registry_adapter(mi355x_tvm_value* args, int* type_codes, int num_args, void* /*ret*/,
                            void* resource_handle) {
  backend_fn_t fn = reinterpret_cast<backend_fn_t>(resource_handle);
  return fn(args, type_codes, num_args, nullptr, nullptr, nullptr);
}

int mi355x_wq_register_tvm_globals(int allow_override) {
  typedef int (*adapter_t)(mi355x_tvm_value*, int*, int, void*, void*);
  typedef int (*create_t)(adapter_t, void*, void (*)(void*), void**);
  typedef int (*register_t)(const char*, void*, int);
  create_t create = reinterpret_cast<create_t>(dlsym(RTLD_DEFAULT, "TVMFuncCreateFromCFunc"));
  register_t reg = reinterpret_cast<register_t>(dlsym(RTLD_DEFAULT, "TVMFuncRegisterGlobal"));
  if (create == nullptr || reg == nullptr) {
    wq::set_error("no TVM runtime is loaded in this process (TVMFuncCreateFromCFunc not found)");
    return -1;
  }
  struct Entry {
    const char* name;
    backend_fn_t fn;
  };
  const Entry entries[] = {{"mi355x.q4f16_matmul", mi355x_q4f16_matmul},
                           {"mi355x.q8f16_matmul", mi355x_q8f16_matmul},
                           {"mi355x.q4f16_matmul_bias", mi355x_q4f16_matmul_bias},
                           {"mi355x.q8f16_matmul_bias", mi355x_q8f16_matmul_bias},
                           {"mi355x.q4f16_matmul_bias_relu", mi355x_q4f16_matmul_bias_relu},
                           {"mi355x.q8f16_matmul_bias_relu", mi355x_q8f16_matmul_bias_relu},
                           {"mi355x.q4f16_matmul_bias_gelu", mi355x_q4f16_matmul_bias_gelu},
                           {"mi355x.q8f16_matmul_bias_gelu", mi355x_q8f16_matmul_bias_gelu},
                           {"mi355x.q4f16_matmul_residual", mi355x_q4f16_matmul_residual},
                           {"mi355x.q8f16_matmul_residual", mi355x_q8f16_matmul_residual},
                           {"mi355x.q4f16_matmul_silu_mul", mi355x_q4f16_matmul_silu_mul},
                           {"mi355x.q8f16_matmul_silu_mul", mi355x_q8f16_matmul_silu_mul},
                           {"mi355x.q4f16_dequantize", mi355x_q4f16_dequantize},
                           {"mi355x.q8f16_dequantize", mi355x_q8f16_dequantize},
                           {"mi355x.q4f16_tile_weights", mi355x_q4f16_tile_weights},
                           {"mi355x.q8f16_tile_weights", mi355x_q8f16_tile_weights},
                           {"mi355x.q4f16_matmul_tiled", mi355x_q4f16_matmul_tiled},
                           {"mi355x.q8f16_matmul_tiled", mi355x_q8f16_matmul_tiled},
                           {"mi355x.q4f16_matmul_ws", mi355x_q4f16_matmul_ws},
                           {"mi355x.q8f16_matmul_ws", mi355x_q8f16_matmul_ws}};
  int count = 0;
  for (const Entry& e : entries) {
    void* handle = nullptr;
    if (create(registry_adapter, reinterpret_cast<void*>(e.fn), nullptr, &handle) != 0 ||
        reg(e.name, handle, allow_override) != 0) {
      wq::set_error("registering %s in the TVM global table failed", e.name);
      return -1;
    }
    ++count;
  }
  return count;
}

}  // extern "C"
