// Runtime module of one offloaded subgraph (include/mi355x_wq_module.h): constant binding at load
// time, the call with the remaining arguments, and the binary form that survives export / load.
#include <dlfcn.h>
#include <hip/hip_runtime_api.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <atomic>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/mi355x_wq.h"
#include "../../include/mi355x_wq_module.h"
#include "wq_internal.h"

namespace {

constexpr int kMaxArgs = 6;  // x, wq, scales, bias, residual, out
constexpr int64_t kMaxString = 1 << 20;
constexpr uint64_t kMaxConsts = 3;  // wq, scales, bias

struct BoundConst {
  mi355x_dl_tensor tensor;  // header handed to the packed call; shape points into `shape`
  int64_t shape[2];
  void* owned;  // device copy of a host constant, or NULL when the caller's device tensor is borrowed
};

}  // namespace

struct mi355x_wq_module {
  std::string symbol, init_name, json;
  mi355x_wq_callspec spec;
  std::vector<std::string> const_names;
  std::vector<int32_t> const_args;
  int32_t flags = 0;
  std::mutex mutex;
  std::atomic<bool> initialized{false};  // set last in init, read without the lock by calls
  std::vector<BoundConst> bound;
  void* wq_tiled = nullptr;
  void* scales_tiled = nullptr;
  int32_t workspace_rows = 0;  // MI355X_WQ_MODULE_OWN_WORKSPACE: calls of up to this many rows may split K
  void* workspace = nullptr;
  int64_t workspace_bytes = 0;
  int device = -1;
};

namespace {

const char* op_name(int op) { return op == 0 ? "matmul" : "dequantize"; }

std::string make_json(const mi355x_wq_module& m) {
  char buf[512];
  const mi355x_wq_callspec& s = m.spec;
  int n = snprintf(buf, sizeof(buf),
                   "{\"version\": 1, \"op\": \"%s\", \"bits\": %d, \"group\": %d, \"zero_point\": %d, "
                   "\"num_args\": %d, \"arg_x\": %d, \"arg_wq\": %d, \"arg_scales\": %d, \"arg_out\": %d, "
                   "\"arg_bias\": %d, \"arg_residual\": %d, \"activation\": %d, \"flags\": %d, \"workspace_rows\": %d, "
                   "\"const_args\": [",
                   op_name(s.op), s.bits, s.group, s.zero_point, s.num_args, s.arg_x, s.arg_wq, s.arg_scales,
                   s.arg_out, s.arg_bias, s.arg_residual, s.activation, m.flags, m.workspace_rows);
  std::string out(buf, n);
  for (size_t i = 0; i < m.const_args.size(); ++i) {
    out += (i ? ", " : "") + std::to_string(m.const_args[i]);
  }
  out += "]}";
  return out;
}

// A reader for the one shape of JSON this module writes: a flat object whose values are integers,
// strings or arrays of integers.  Anything else is an error; nothing is read past the text.
struct JsonReader {
  const char* p;
  const char* end;
  void skip() {
    while (p < end && (*p == ' ' || *p == '\n' || *p == '\t' || *p == '\r')) ++p;
  }
  bool eat(char c) {
    skip();
    if (p < end && *p == c) {
      ++p;
      return true;
    }
    return false;
  }
  bool string(std::string* out) {
    skip();
    if (p >= end || *p != '"') return false;
    const char* q = ++p;
    while (q < end && *q != '"' && *q != '\\') ++q;
    if (q >= end || *q != '"') return false;
    out->assign(p, q);
    p = q + 1;
    return true;
  }
  bool integer(int64_t* out) {
    skip();
    const char* q = p;
    bool neg = false;
    if (q < end && *q == '-') {
      neg = true;
      ++q;
    }
    if (q >= end || *q < '0' || *q > '9') return false;
    int64_t v = 0;
    int digits = 0;
    while (q < end && *q >= '0' && *q <= '9') {
      if (++digits > 9) return false;
      v = v * 10 + (*q - '0');
      ++q;
    }
    *out = neg ? -v : v;
    p = q;
    return true;
  }
};

bool parse_json(const std::string& text, mi355x_wq_callspec* spec, std::vector<int32_t>* const_args, int32_t* flags,
                int32_t* workspace_rows) {
  JsonReader r{text.data(), text.data() + text.size()};
  memset(spec, 0, sizeof(*spec));
  spec->op = -1;
  spec->arg_bias = spec->arg_residual = -1;
  int64_t version = 0;
  bool have_const_args = false;
  if (!r.eat('{')) return false;
  bool first = true;
  while (true) {
    if (r.eat('}')) break;
    if (!first && !r.eat(',')) return false;
    first = false;
    std::string key;
    if (!r.string(&key) || !r.eat(':')) return false;
    if (key == "op") {
      std::string v;
      if (!r.string(&v)) return false;
      if (v == "matmul") spec->op = 0;
      else if (v == "dequantize") spec->op = 1;
      else return false;
    } else if (key == "const_args") {
      if (!r.eat('[')) return false;
      have_const_args = true;
      while (!r.eat(']')) {
        int64_t v;
        if (!const_args->empty() && !r.eat(',')) return false;
        if (!r.integer(&v) || const_args->size() >= kMaxConsts) return false;
        const_args->push_back((int32_t)v);
      }
    } else {
      int64_t v;
      if (!r.integer(&v)) return false;
      int32_t* field = key == "bits" ? &spec->bits : key == "group" ? &spec->group
                     : key == "zero_point" ? &spec->zero_point : key == "num_args" ? &spec->num_args
                     : key == "arg_x" ? &spec->arg_x : key == "arg_wq" ? &spec->arg_wq
                     : key == "arg_scales" ? &spec->arg_scales : key == "arg_out" ? &spec->arg_out
                     : key == "arg_bias" ? &spec->arg_bias : key == "arg_residual" ? &spec->arg_residual
                     : key == "activation" ? &spec->activation : key == "flags" ? flags
                     : key == "workspace_rows" ? workspace_rows : nullptr;
      if (key == "version") version = v;
      else if (field != nullptr) *field = (int32_t)v;
      else return false;
    }
  }
  r.skip();
  return r.p == r.end && version == 1 && spec->op >= 0 && have_const_args;
}

// dmlc::Stream's encoding of std::string and std::vector<std::string>: uint64 sizes, little endian.
struct ByteWriter {
  uint8_t* out;
  int64_t capacity, size = 0;
  void raw(const void* p, int64_t n) {
    if (out != nullptr && size + n <= capacity) memcpy(out + size, p, n);
    size += n;
  }
  void u64(uint64_t v) { raw(&v, 8); }
  void str(const std::string& s) {
    u64(s.size());
    raw(s.data(), (int64_t)s.size());
  }
};

struct ByteReader {
  const uint8_t* in;
  int64_t size, pos = 0;
  bool u64(uint64_t* v) {
    if (size - pos < 8) return false;
    memcpy(v, in + pos, 8);
    pos += 8;
    return true;
  }
  bool str(std::string* s) {
    uint64_t n;
    if (!u64(&n) || n > (uint64_t)kMaxString || (int64_t)n > size - pos) return false;
    s->assign(reinterpret_cast<const char*>(in + pos), n);
    pos += (int64_t)n;
    return true;
  }
};

bool validate(const char* symbol, const mi355x_wq_callspec* spec, const int32_t* const_args, int32_t num_consts,
              int32_t flags) {
  if (symbol == nullptr || symbol[0] == 0) {
    wq::set_error("module: empty symbol name");
    return false;
  }
  if (spec == nullptr) {
    wq::set_error("module: call spec is NULL");
    return false;
  }
  if (spec->op != 0 && spec->op != 1) {
    wq::set_error("module: unknown op %d", spec->op);
    return false;
  }
  if (spec->bits != 4 && spec->bits != 8) {
    wq::set_error("module: bits must be 4 or 8, got %d", spec->bits);
    return false;
  }
  const bool is_matmul = spec->op == 0;
  const int expect = (is_matmul ? 4 : 3) + (is_matmul && spec->arg_bias >= 0) + (is_matmul && spec->arg_residual >= 0);
  if (spec->num_args != expect || expect > kMaxArgs) {
    wq::set_error("module: %s with these fused operands has %d arguments, the spec says %d", op_name(spec->op), expect,
                  spec->num_args);
    return false;
  }
  if (num_consts < 0 || num_consts > (int32_t)kMaxConsts || (num_consts > 0 && const_args == nullptr)) {
    wq::set_error("module: between 0 and %d constants, got %d", (int)kMaxConsts, num_consts);
    return false;
  }
  if ((flags & ~(MI355X_WQ_MODULE_TILE_WEIGHTS | MI355X_WQ_MODULE_LIBRARY_SCRATCH | MI355X_WQ_MODULE_OWN_WORKSPACE)) != 0) {
    wq::set_error("module: unknown flags 0x%x", flags);
    return false;
  }
  bool has_wq = false, has_scales = false;
  for (int i = 0; i < num_consts; ++i) {
    const int a = const_args[i];
    const bool allowed = a == spec->arg_wq || a == spec->arg_scales || (is_matmul && spec->arg_bias >= 0 && a == spec->arg_bias);
    if (a < 0 || a >= expect || !allowed) {
      wq::set_error("module: constant %d binds slot %d, which is not the slot of wq, scales or bias", i, a);
      return false;
    }
    for (int j = 0; j < i; ++j) {
      if (const_args[j] == a) {
        wq::set_error("module: slot %d is bound by two constants", a);
        return false;
      }
    }
    has_wq |= a == spec->arg_wq;
    has_scales |= a == spec->arg_scales;
  }
  if ((flags & MI355X_WQ_MODULE_TILE_WEIGHTS) && !(is_matmul && has_wq && has_scales)) {
    wq::set_error("module: tile-major conversion needs a matmul whose wq and scales are both constants");
    return false;
  }
  if ((flags & MI355X_WQ_MODULE_OWN_WORKSPACE) && !(is_matmul && has_wq && has_scales)) {
    wq::set_error("module: a workspace is sized from N and K at init, which needs a matmul whose wq and scales are both constants");
    return false;
  }
  return true;
}

mi355x_wq_module* build(const char* symbol, const mi355x_wq_callspec* spec, const std::vector<std::string>& names,
                        const int32_t* const_args, int32_t flags) {
  mi355x_wq_module* m = new mi355x_wq_module();
  m->symbol = symbol;
  m->init_name = std::string("__init_") + symbol;
  m->spec = *spec;
  m->const_names = names;
  m->const_args.assign(const_args, const_args + names.size());
  m->flags = flags;
  m->json = make_json(*m);
  m->initialized = names.empty();
  return m;
}

void release_device_memory(mi355x_wq_module* m) {
  for (BoundConst& b : m->bound) {
    if (b.owned != nullptr) (void)hipFree(b.owned);
  }
  m->bound.clear();
  if (m->wq_tiled != nullptr) (void)hipFree(m->wq_tiled);
  if (m->scales_tiled != nullptr) (void)hipFree(m->scales_tiled);
  if (m->workspace != nullptr) (void)hipFree(m->workspace);
  m->wq_tiled = m->scales_tiled = m->workspace = nullptr;
  m->workspace_bytes = 0;
}

bool hip_ok(hipError_t e, const char* what) {
  if (e == hipSuccess) return true;
  (void)hipGetLastError();
  wq::set_error("module init: %s failed: %s", what, hipGetErrorString(e));
  return false;
}

// Binds the constants (called once, under the module's mutex).
bool bind_constants(mi355x_wq_module* m, const mi355x_dl_tensor* const* consts, int32_t num_consts) {
  if (num_consts != (int32_t)m->const_names.size() || (num_consts > 0 && consts == nullptr)) {
    wq::set_error("__init_%s expects %d constants, got %d", m->symbol.c_str(), (int)m->const_names.size(), num_consts);
    return false;
  }
  int cur = -1;
  if (!hip_ok(hipGetDevice(&cur), "hipGetDevice")) return false;
  m->bound.resize(num_consts);
  for (BoundConst& b : m->bound) b.owned = nullptr;
  for (int i = 0; i < num_consts; ++i) {
    const mi355x_dl_tensor* t = consts[i];
    const char* name = m->const_names[i].c_str();
    if (t == nullptr || t->shape == nullptr || t->ndim < 1 || t->ndim > 2) {
      wq::set_error("constant '%s': expected a 1-d or 2-d tensor", name);
      return false;
    }
    if (t->data == nullptr && t->shape[0] != 0 && t->shape[t->ndim - 1] != 0) {
      wq::set_error("constant '%s': NULL data pointer", name);
      return false;
    }
    if (t->strides != nullptr) {
      int64_t expect = 1;
      for (int d = t->ndim - 1; d >= 0; --d) {
        if (t->shape[d] != 1 && t->strides[d] != expect) {
          wq::set_error("constant '%s': not compact row-major", name);
          return false;
        }
        expect *= t->shape[d];
      }
    }
    BoundConst& b = m->bound[i];
    b.tensor = *t;
    b.shape[0] = t->shape[0];
    b.shape[1] = t->ndim == 2 ? t->shape[1] : 1;
    b.tensor.shape = b.shape;
    b.tensor.strides = nullptr;
    if (t->device.device_type == MI355X_DL_CPU) {
      int64_t elems = 1;
      for (int d = 0; d < t->ndim; ++d) elems *= t->shape[d];
      const int64_t bytes = elems * ((t->dtype.bits + 7) / 8) * t->dtype.lanes;
      if (elems < 0 || bytes > ((int64_t)1 << 31)) {
        wq::set_error("constant '%s': %lld bytes is beyond the 2 GiB an operand may have", name, (long long)bytes);
        return false;
      }
      if (!hip_ok(hipMalloc(&b.owned, bytes > 0 ? bytes : 16), "hipMalloc")) return false;
      if (bytes > 0 && !hip_ok(hipMemcpy(b.owned, static_cast<const char*>(t->data) + t->byte_offset, bytes,
                                         hipMemcpyHostToDevice), "hipMemcpy"))
        return false;
      b.tensor.data = b.owned;
      b.tensor.byte_offset = 0;
      b.tensor.device.device_type = MI355X_DL_ROCM;
      b.tensor.device.device_id = cur;
    } else if (t->device.device_type != MI355X_DL_ROCM) {
      wq::set_error("constant '%s': expected a host (1) or ROCm (10) tensor, got device type %d", name,
                    t->device.device_type);
      return false;
    } else if (t->device.device_id != cur) {
      wq::set_error("constant '%s' lives on ROCm device %d but the current HIP device is %d", name,
                    t->device.device_id, cur);
      return false;
    }
  }
  m->device = cur;
  if (!(m->flags & (MI355X_WQ_MODULE_TILE_WEIGHTS | MI355X_WQ_MODULE_OWN_WORKSPACE))) return true;

  // N, K and the group of the bound weights (both flags need wq and scales among the constants)
  const BoundConst *bw = nullptr, *bs = nullptr;
  for (int i = 0; i < num_consts; ++i) {
    if (m->const_args[i] == m->spec.arg_wq) bw = &m->bound[i];
    if (m->const_args[i] == m->spec.arg_scales) bs = &m->bound[i];
  }
  const mi355x_dl_tensor &tw = bw->tensor, &ts = bs->tensor;
  if (tw.ndim != 2 || ts.ndim != 2 || tw.dtype.code != 1 || tw.dtype.bits != 32 || ts.dtype.code != 2 ||
      ts.dtype.bits != 16 || ts.shape[0] != tw.shape[0] || ts.shape[1] <= 0) {
    wq::set_error("module init: wq must be uint32 [N, K*bits/32] and scales float16 [N, K/group]");
    return false;
  }
  mi355x_wq_desc d;
  memset(&d, 0, sizeof(d));
  d.bits = m->spec.bits;
  d.zero_point = m->spec.zero_point;
  d.n = tw.shape[0];
  d.k = tw.shape[1] * (32 / d.bits);
  d.group = m->spec.group > 0 ? m->spec.group : (int32_t)(d.k / ts.shape[1]);
  if (d.group <= 0 || d.k % d.group != 0 || ts.shape[1] != d.k / d.group) {
    wq::set_error("module init: scales shape (%lld, %lld) does not match K=%lld", (long long)ts.shape[0],
                  (long long)ts.shape[1], (long long)d.k);
    return false;
  }
  if (d.n == 0) return true;
  // One-off conversion to the tile-major layout; the canonical tensors stay bound for validation.
  // The flag is a request, not a promise: where the tile-major layout is not defined for this
  // (bits, group, K) -- e.g. int4 with K not a multiple of 256 -- or for this composite -- the gated tail is
  // computed on canonical weights only -- the canonical constants stay bound and calls run on them, exactly as
  // they would without the flag.
  if ((m->flags & MI355X_WQ_MODULE_TILE_WEIGHTS) && m->spec.activation != MI355X_WQ_ACT_SILU_MUL &&
      wq::tiled_layout_defined(d.bits, d.group, d.k)) {
    int64_t wq_bytes = 0, sc_bytes = 0;
    if (mi355x_wq_tiled_sizes(&d, &wq_bytes, &sc_bytes) != 0) return false;
    if (!hip_ok(hipMalloc(&m->wq_tiled, wq_bytes), "hipMalloc") || !hip_ok(hipMalloc(&m->scales_tiled, sc_bytes), "hipMalloc"))
      return false;
    const void* pw = static_cast<const char*>(tw.data) + tw.byte_offset;
    const void* ps = static_cast<const char*>(ts.data) + ts.byte_offset;
    if (mi355x_wq_tile_weights(&d, pw, ps, m->wq_tiled, m->scales_tiled, nullptr) != 0) return false;
    if (!hip_ok(hipStreamSynchronize(nullptr), "hipStreamSynchronize")) return false;
    // The module's own canonical copies (of host constants) are not read again: calls take N, K and the
    // group from the headers and the data from the tile-major buffers, which have at least as many rows.
    for (int i = 0; i < num_consts; ++i) {
      BoundConst& b = m->bound[i];
      const bool is_wq = m->const_args[i] == m->spec.arg_wq, is_scales = m->const_args[i] == m->spec.arg_scales;
      if (b.owned == nullptr || !(is_wq || is_scales)) continue;
      (void)hipFree(b.owned);
      b.owned = nullptr;
      b.tensor.data = is_wq ? m->wq_tiled : m->scales_tiled;
    }
  }
  // The K split's workspace, where this projection has a use for one at any row count up to workspace_rows:
  // allocated and zeroed here, once, so that calls allocate nothing (what the reference's generated host code
  // does per call, python/tvm/contrib/cutlass/gemm_operation.py:294-295).
  if ((m->flags & MI355X_WQ_MODULE_OWN_WORKSPACE) && m->workspace_rows > 0) {
    const int tiled = m->wq_tiled != nullptr ? 1 : 0;
    int64_t need = 0;
    for (int64_t rows = 1; rows <= m->workspace_rows; ++rows) {
      const int64_t b = mi355x_wq_workspace_bytes(&d, rows, tiled);
      if (b < 0) return false;
      if (b > need) need = b;
    }
    if (need > 0) {
      if (!hip_ok(hipMalloc(&m->workspace, need), "hipMalloc")) return false;
      if (!hip_ok(hipMemset(m->workspace, 0, need), "hipMemset") || !hip_ok(hipDeviceSynchronize(), "hipDeviceSynchronize"))
        return false;
      m->workspace_bytes = need;
    }
  }
  return true;
}

void set_int_return(void* ret, int64_t v) {
  typedef int (*set_return_t)(void*, mi355x_tvm_value*, int*, int);
  static set_return_t fn = reinterpret_cast<set_return_t>(dlsym(RTLD_DEFAULT, "TVMCFuncSetReturn"));
  if (fn == nullptr || ret == nullptr) return;
  mi355x_tvm_value value;
  value.v_int64 = v;
  int tcode = 0;  // kTVMArgInt
  (void)fn(ret, &value, &tcode, 1);
}

int packed_init(mi355x_tvm_value* args, int* type_codes, int num_args, void* ret, void* resource) {
  mi355x_wq_module* m = static_cast<mi355x_wq_module*>(resource);
  const mi355x_dl_tensor* consts[kMaxConsts] = {nullptr, nullptr, nullptr};
  if (m == nullptr || num_args < 0 || num_args > (int)kMaxConsts || (num_args > 0 && (args == nullptr || type_codes == nullptr))) {
    wq::set_error("__init_<symbol>: expected one tensor per constant, got %d arguments", num_args);
    return wq::packed_fail();
  }
  for (int i = 0; i < num_args; ++i) {
    if (type_codes[i] != MI355X_TVM_DLTENSOR_HANDLE && type_codes[i] != MI355X_TVM_NDARRAY_HANDLE) {
      wq::set_error("__init_%s: argument %d is not a tensor (type code %d)", m->symbol.c_str(), i, type_codes[i]);
      return wq::packed_fail();
    }
    consts[i] = static_cast<const mi355x_dl_tensor*>(args[i].v_handle);
  }
  if (mi355x_wq_module_init(m, consts, num_args) != 0) return wq::packed_fail();
  set_int_return(ret, 0);
  return 0;
}

int packed_run(mi355x_tvm_value* args, int* type_codes, int num_args, void* /*ret*/, void* resource) {
  return mi355x_wq_module_call(static_cast<mi355x_wq_module*>(resource), args, type_codes, num_args);
}

}  // namespace

extern "C" {

const char* mi355x_wq_module_type_key(void) { return "mi355x_wq"; }

int mi355x_wq_module_create(const char* symbol, const mi355x_wq_callspec* spec, const char* const* const_names,
                            const int32_t* const_args, int32_t num_consts, int32_t flags, mi355x_wq_module** out) {
  if (out == nullptr) {
    wq::set_error("module: output pointer is NULL");
    return -1;
  }
  *out = nullptr;
  if (!validate(symbol, spec, const_args, num_consts, flags)) return -1;
  std::vector<std::string> names;
  for (int i = 0; i < num_consts; ++i) {
    if (const_names == nullptr || const_names[i] == nullptr || const_names[i][0] == 0) {
      wq::set_error("module: constant %d has no name", i);
      return -1;
    }
    names.emplace_back(const_names[i]);
  }
  *out = build(symbol, spec, names, const_args, flags);
  return 0;
}

void mi355x_wq_module_destroy(mi355x_wq_module* mod) {
  if (mod == nullptr) return;
  release_device_memory(mod);
  delete mod;
}

const char* mi355x_wq_module_symbol(const mi355x_wq_module* mod) { return mod ? mod->symbol.c_str() : nullptr; }
int32_t mi355x_wq_module_num_consts(const mi355x_wq_module* mod) { return mod ? (int32_t)mod->const_names.size() : -1; }
const char* mi355x_wq_module_const_name(const mi355x_wq_module* mod, int32_t i) {
  return mod && i >= 0 && i < (int32_t)mod->const_names.size() ? mod->const_names[i].c_str() : nullptr;
}
const char* mi355x_wq_module_json(const mi355x_wq_module* mod) { return mod ? mod->json.c_str() : nullptr; }
int32_t mi355x_wq_module_initialized(const mi355x_wq_module* mod) { return mod && mod->initialized.load() ? 1 : 0; }

int mi355x_wq_module_get_function(mi355x_wq_module* mod, const char* name, mi355x_wq_packed_cfunc* func,
                                  void** resource_handle) {
  if (mod == nullptr || name == nullptr || func == nullptr || resource_handle == nullptr) {
    wq::set_error("module get_function: NULL argument");
    return -1;
  }
  *resource_handle = mod;
  if (mod->symbol == name) *func = packed_run;
  else if (mod->init_name == name) *func = packed_init;
  else {
    *func = nullptr;
    *resource_handle = nullptr;
  }
  return 0;
}

int mi355x_wq_module_init(mi355x_wq_module* mod, const mi355x_dl_tensor* const* consts, int32_t num_consts) {
  if (mod == nullptr) {
    wq::set_error("module is NULL");
    return -1;
  }
  std::lock_guard<std::mutex> guard(mod->mutex);
  if (mod->initialized) return 0;
  if (!bind_constants(mod, consts, num_consts)) {
    release_device_memory(mod);
    return -1;
  }
  mod->initialized = true;
  return 0;
}

int mi355x_wq_module_call(mi355x_wq_module* mod, mi355x_tvm_value* args, int* type_codes, int num_args) {
  if (mod == nullptr) {
    wq::set_error("module is NULL");
    return wq::packed_fail();
  }
  if (!mod->initialized) {
    wq::set_error("%s: The module has not been initialized", mod->symbol.c_str());
    return wq::packed_fail();
  }
  const int total = mod->spec.num_args, nconst = (int)mod->const_names.size();
  if (num_args != total - nconst || (num_args > 0 && (args == nullptr || type_codes == nullptr))) {
    wq::set_error("%s expects %d arguments (%d of the composite's %d are bound constants), got %d",
                  mod->symbol.c_str(), total - nconst, nconst, total, num_args);
    return wq::packed_fail();
  }
  mi355x_tvm_value full[kMaxArgs];
  int codes[kMaxArgs];
  int next = 0;
  for (int slot = 0; slot < total; ++slot) {
    int c = -1;
    for (int i = 0; i < nconst; ++i) {
      if (mod->const_args[i] == slot) c = i;
    }
    if (c >= 0) {
      full[slot].v_handle = &mod->bound[c].tensor;
      codes[slot] = MI355X_TVM_DLTENSOR_HANDLE;
    } else {
      full[slot] = args[next];
      codes[slot] = type_codes[next];
      ++next;
    }
  }
  // (a call of more rows than the workspace was sized for runs as the plain call)
  int64_t rows = 0;
  if (mod->workspace != nullptr && mod->spec.op == 0) {
    const int tc = codes[mod->spec.arg_x];
    const mi355x_dl_tensor* tx = (tc == MI355X_TVM_DLTENSOR_HANDLE || tc == MI355X_TVM_NDARRAY_HANDLE)
                                     ? static_cast<const mi355x_dl_tensor*>(full[mod->spec.arg_x].v_handle) : nullptr;
    if (tx != nullptr && tx->shape != nullptr && tx->ndim >= 1 && tx->ndim <= 8) {
      rows = 1;
      for (int d = 0; d + 1 < tx->ndim; ++d) rows = tx->shape[d] > 0 && rows <= mod->workspace_rows ? rows * tx->shape[d] : rows;
    }
  }
  const bool use_ws = mod->workspace != nullptr && rows >= 1 && rows <= mod->workspace_rows;
  return wq::packed_call_with_weights(&mod->spec, full, codes, total, mod->wq_tiled, mod->scales_tiled,
                                      (mod->flags & MI355X_WQ_MODULE_LIBRARY_SCRATCH) != 0,
                                      use_ws ? mod->workspace : nullptr, use_ws ? mod->workspace_bytes : 0);
}

int64_t mi355x_wq_module_save_to_binary(const mi355x_wq_module* mod, void* buffer, int64_t capacity) {
  if (mod == nullptr || capacity < 0) {
    wq::set_error("module save: NULL module or negative capacity");
    return -1;
  }
  ByteWriter w{static_cast<uint8_t*>(buffer), capacity};
  w.str(mod->symbol);
  w.str(mod->json);
  w.u64(mod->const_names.size());
  for (const std::string& s : mod->const_names) w.str(s);
  return w.size;
}

int mi355x_wq_module_load_from_binary(const void* buffer, int64_t size, int64_t* consumed, mi355x_wq_module** out) {
  if (buffer == nullptr || size < 0 || out == nullptr) {
    wq::set_error("module load: NULL argument");
    return -1;
  }
  *out = nullptr;
  ByteReader r{static_cast<const uint8_t*>(buffer), size};
  std::string symbol, json;
  uint64_t count = 0;
  if (!r.str(&symbol)) {
    wq::set_error("module load: Loading symbol name failed");
    return -1;
  }
  if (!r.str(&json)) {
    wq::set_error("module load: Loading graph json failed");
    return -1;
  }
  std::vector<std::string> names;
  bool ok = r.u64(&count) && count <= kMaxConsts;
  for (uint64_t i = 0; ok && i < count; ++i) {
    std::string s;
    ok = r.str(&s);
    names.push_back(s);
  }
  if (!ok) {
    wq::set_error("module load: Loading the const name list failed");
    return -1;
  }
  std::vector<const char*> name_ptrs;
  for (const std::string& s : names) name_ptrs.push_back(s.c_str());
  if (mi355x_wq_module_create_from_json(symbol.c_str(), json.c_str(), name_ptrs.data(), (int32_t)names.size(), out) != 0)
    return -1;
  if (consumed != nullptr) *consumed = r.pos;
  return 0;
}

int mi355x_wq_module_create_from_json(const char* symbol, const char* json, const char* const* const_names,
                                      int32_t num_consts, mi355x_wq_module** out) {
  if (json == nullptr || out == nullptr) {
    wq::set_error("module: NULL argument");
    return -1;
  }
  *out = nullptr;
  mi355x_wq_callspec spec;
  std::vector<int32_t> const_args;
  int32_t flags = 0, workspace_rows = 0;
  if (!parse_json(json, &spec, &const_args, &flags, &workspace_rows)) {
    wq::set_error("module load: the call description is not one this library wrote: %.200s", json);
    return -1;
  }
  if ((int32_t)const_args.size() != num_consts) {
    wq::set_error("module load: %d constant names for %d constant slots", num_consts, (int)const_args.size());
    return -1;
  }
  if (mi355x_wq_module_create(symbol, &spec, const_names, const_args.data(), num_consts, flags, out) != 0) return -1;
  if (workspace_rows != 0 && mi355x_wq_module_set_workspace_rows(*out, workspace_rows) != 0) {
    mi355x_wq_module_destroy(*out);
    *out = nullptr;
    return -1;
  }
  return 0;
}

int mi355x_wq_module_set_workspace_rows(mi355x_wq_module* mod, int32_t rows) {
  if (mod == nullptr) {
    wq::set_error("module is NULL");
    return -1;
  }
  std::lock_guard<std::mutex> guard(mod->mutex);
  if (!(mod->flags & MI355X_WQ_MODULE_OWN_WORKSPACE)) {
    wq::set_error("module: workspace rows go with MI355X_WQ_MODULE_OWN_WORKSPACE");
    return -1;
  }
  if (rows < 0 || rows > (1 << 20)) {
    wq::set_error("module: workspace rows must be between 0 and %d, got %d", 1 << 20, rows);
    return -1;
  }
  if (mod->initialized && !mod->const_names.empty()) {
    wq::set_error("module: the workspace is sized at init; set the rows before __init_%s runs", mod->symbol.c_str());
    return -1;
  }
  mod->workspace_rows = rows;
  mod->json = make_json(*mod);
  return 0;
}

}  // extern "C"
