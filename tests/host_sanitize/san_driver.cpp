// Host-side checks of the C ABI under AddressSanitizer and UndefinedBehaviorSanitizer.
//
// The three host translation units of the library (argument validation and dispatch, the
// PackedFunc boundary, the subgraph module with its binary loader and JSON reader) are compiled
// with -fsanitize=address,undefined and linked with the ordinary kernel objects into this
// program.  Nothing here needs a GPU: every call either ends in the validation layer or in the
// module's host logic.  The loader is the part that parses bytes it does not control, so it gets
// every truncation of a good module and several thousand random corruptions of it.
//
// Exit status 0 = every expectation held and the sanitizers reported nothing.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "../../include/mi355x_wq.h"
#include "../../include/mi355x_wq_module.h"
#include "../../include/mi355x_wq_packed.h"

static int g_failures = 0;
#define EXPECT(cond)                                                              \
  do {                                                                            \
    if (!(cond)) {                                                                \
      std::fprintf(stderr, "%s:%d: expectation failed: %s (last error: %s)\n", __FILE__, __LINE__, #cond, \
                   mi355x_wq_last_error());                                       \
      ++g_failures;                                                               \
    }                                                                             \
  } while (0)

static bool error_has(const char* what) { return std::strstr(mi355x_wq_last_error(), what) != nullptr; }

static void check_descriptors() {
  mi355x_wq_desc d{4, 32, 7, 0, 4096, 4096};
  EXPECT(mi355x_wq_check(&d, 1) == 0);
  EXPECT(mi355x_wq_check(nullptr, 1) == -1 && error_has("NULL"));
  mi355x_wq_desc b = d;
  b.bits = 5;
  EXPECT(mi355x_wq_check(&b, 1) == -1 && error_has("bits"));
  b = d;
  b.group = 48;
  EXPECT(mi355x_wq_check(&b, 1) == -1 && error_has("group"));
  b = d;
  b.zero_point = 16;
  EXPECT(mi355x_wq_check(&b, 1) == -1 && error_has("zero_point"));
  b = d;
  b.reserved = 3;
  EXPECT(mi355x_wq_check(&b, 1) == -1 && error_has("reserved"));
  b = d;
  b.k = 4100;
  EXPECT(mi355x_wq_check(&b, 1) == -1 && error_has("multiple"));
  b = d;
  b.n = -1;
  EXPECT(mi355x_wq_check(&b, 1) == -1 && error_has("negative"));
  b = d;
  b.n = int64_t(1) << 40;
  EXPECT(mi355x_wq_check(&b, 1) == -1 && error_has("too large"));
  EXPECT(mi355x_wq_check(&d, int64_t(1) << 40) == -1);
  // pointer checks end before any launch
  const uintptr_t ok = 0x10000;
  EXPECT(mi355x_wq_matmul(&d, nullptr, (void*)ok, (void*)ok, (void*)ok, 1, nullptr) == -1 && error_has("x is NULL"));
  EXPECT(mi355x_wq_matmul(&d, (void*)ok, (void*)(ok + 4), (void*)ok, (void*)ok, 1, nullptr) == -1 && error_has("aligned"));
  EXPECT(mi355x_wq_dequantize(&d, (void*)ok, nullptr, (void*)ok, nullptr) == -1);
  mi355x_wq_epilogue ep{(void*)(ok + 1), nullptr, 0, 0};
  EXPECT(mi355x_wq_matmul_fused(&d, (void*)ok, (void*)ok, (void*)ok, &ep, (void*)ok, 1, nullptr) == -1);
  ep = mi355x_wq_epilogue{nullptr, nullptr, 7, 0};
  EXPECT(mi355x_wq_matmul_fused(&d, (void*)ok, (void*)ok, (void*)ok, &ep, (void*)ok, 1, nullptr) == -1);
  // selection and sizes are pure host arithmetic
  for (int64_t m : {int64_t(1), int64_t(8), int64_t(16), int64_t(17), int64_t(64), int64_t(65), int64_t(2048)}) {
    const int k = mi355x_wq_select_kernel(&d, m);
    EXPECT(k == MI355X_WQ_KERNEL_GEMV || k == MI355X_WQ_KERNEL_GEMM || k == MI355X_WQ_KERNEL_SKINNY);
  }
  int64_t wb = 0, sb = 0;
  EXPECT(mi355x_wq_tiled_sizes(&d, &wb, &sb) == 0 && wb == 4096 * 2048 && sb == 4096 * 128 * 2);
  mi355x_wq_desc odd{4, 32, 7, 0, 100, 352};
  EXPECT(mi355x_wq_tiled_sizes(&odd, &wb, &sb) == -1);
  mi355x_wq_desc q8{8, 128, 0, 0, 5120, 13824};
  EXPECT(mi355x_wq_workspace_bytes(&q8, 8, 0) > 0);
  EXPECT(mi355x_wq_workspace_bytes(&q8, 1, 0) == 0);
  EXPECT(mi355x_wq_workspace_bytes(&d, 1, 0) == 0);
  EXPECT(mi355x_wq_matmul_ws(&d, (void*)ok, (void*)ok, (void*)ok, nullptr, (void*)ok, 4, nullptr, 0, (void*)(ok + 4),
                             1 << 20) == -1);
  EXPECT(mi355x_wq_version() > 0);
}

struct Tensor {
  mi355x_dl_tensor t;
  int64_t shape[2];
  int64_t strides[2];
  Tensor(void* data, int dev, int code, int bits, int64_t r, int64_t c) {
    shape[0] = r;
    shape[1] = c;
    strides[0] = c;
    strides[1] = 1;
    t.data = data;
    t.device.device_type = dev;
    t.device.device_id = 0;
    t.ndim = 2;
    t.dtype.code = (uint8_t)code;
    t.dtype.bits = (uint8_t)bits;
    t.dtype.lanes = 1;
    t.shape = shape;
    t.strides = nullptr;
    t.byte_offset = 0;
  }
};

static void check_packed_boundary() {
  void* const p = (void*)0x20000;
  const int64_t m = 2, n = 64, k = 256;
  auto call = [&](Tensor& x, Tensor& wq, Tensor& s, Tensor& y, int nargs = 4, int code0 = MI355X_TVM_DLTENSOR_HANDLE) {
    mi355x_tvm_value args[4];
    int codes[4] = {code0, MI355X_TVM_NDARRAY_HANDLE, MI355X_TVM_DLTENSOR_HANDLE, MI355X_TVM_DLTENSOR_HANDLE};
    args[0].v_handle = &x.t;
    args[1].v_handle = &wq.t;
    args[2].v_handle = &s.t;
    args[3].v_handle = &y.t;
    mi355x_tvm_value ret;
    int ret_code = MI355X_TVM_NULLPTR;
    const int rc = mi355x_q4f16_matmul(args, codes, nargs, &ret, &ret_code, nullptr);
    EXPECT(ret_code == MI355X_TVM_NULLPTR);
    return rc;
  };
  auto good = [&](Tensor*& x, Tensor*& wq, Tensor*& s, Tensor*& y) {
    x = new Tensor(p, MI355X_DL_ROCM, 2, 16, m, k);
    wq = new Tensor(p, MI355X_DL_ROCM, 1, 32, n, k / 8);
    s = new Tensor(p, MI355X_DL_ROCM, 2, 16, n, k / 32);
    y = new Tensor(p, MI355X_DL_ROCM, 2, 16, m, n);
  };
  Tensor *x, *wq, *s, *y;
  auto drop = [&] {
    delete x;
    delete wq;
    delete s;
    delete y;
  };
  good(x, wq, s, y);
  EXPECT(call(*x, *wq, *s, *y, 3) == -1 && error_has("argument"));
  EXPECT(call(*x, *wq, *s, *y, 4, 0 /* an int, not a tensor */) == -1);
  x->t.device.device_type = MI355X_DL_CPU;
  EXPECT(call(*x, *wq, *s, *y) == -1 && error_has("device"));
  drop();
  good(x, wq, s, y);
  x->t.dtype.bits = 32;
  EXPECT(call(*x, *wq, *s, *y) == -1 && error_has("float16"));
  drop();
  good(x, wq, s, y);
  wq->t.dtype.code = 0;
  EXPECT(call(*x, *wq, *s, *y) == -1);
  drop();
  good(x, wq, s, y);
  x->t.ndim = 3;
  EXPECT(call(*x, *wq, *s, *y) == -1);
  drop();
  good(x, wq, s, y);
  x->strides[0] = k + 8;  // not compact
  x->t.strides = x->strides;
  EXPECT(call(*x, *wq, *s, *y) == -1 && error_has("compact"));
  x->strides[0] = k;  // compact strides are accepted: the call then ends in a pointer or launch check, not here
  drop();
  good(x, wq, s, y);
  x->t.byte_offset = 6;  // misaligned view (with a GPU the message names the alignment; without one the device check comes first)
  EXPECT(call(*x, *wq, *s, *y) == -1);
  drop();
  good(x, wq, s, y);
  y->shape[1] = n + 1;
  EXPECT(call(*x, *wq, *s, *y) == -1);
  drop();
  good(x, wq, s, y);
  s->shape[1] = 5;  // K / 5 is no group size
  EXPECT(call(*x, *wq, *s, *y) == -1);
  drop();
  good(x, wq, s, y);
  x->t.data = nullptr;
  EXPECT(call(*x, *wq, *s, *y) == -1);
  // a call description whose slots fall outside the argument list
  mi355x_tvm_value args[4];
  int codes[4] = {7, 7, 7, 7};
  args[0].v_handle = &x->t;
  args[1].v_handle = &wq->t;
  args[2].v_handle = &s->t;
  args[3].v_handle = &y->t;
  mi355x_wq_callspec spec{0, 4, 0, 7, 0, 1, 2, 3, 4, -1, -1, 0};
  spec.arg_out = 9;
  EXPECT(mi355x_wq_packed_call(&spec, args, codes, 4) == -1);
  spec.arg_out = 3;
  spec.arg_bias = 4;
  EXPECT(mi355x_wq_packed_call(&spec, args, codes, 4) == -1);
  spec.arg_bias = -1;
  spec.arg_x = 1;  // two roles in one slot
  EXPECT(mi355x_wq_packed_call(&spec, args, codes, 4) == -1);
  EXPECT(mi355x_wq_packed_call(nullptr, args, codes, 4) == -1);
  drop();
  mi355x_wq_packed_set_stream((void*)0x30);
  EXPECT(mi355x_wq_packed_get_stream() == (void*)0x30);
  mi355x_wq_packed_set_stream(nullptr);
}

static uint64_t g_rng = 0x9E3779B97F4A7C15ull;
static uint32_t rnd() {
  g_rng ^= g_rng << 13;
  g_rng ^= g_rng >> 7;
  g_rng ^= g_rng << 17;
  return (uint32_t)(g_rng >> 16);
}

static void check_module() {
  EXPECT(std::strcmp(mi355x_wq_module_type_key(), "mi355x_wq") == 0);
  mi355x_wq_callspec spec{0, 4, 0, 7, 2, 0, 1, 3, 4, -1, -1, 0};
  const char* names[] = {"fused_decode_q4f16_matmul_mi355x_const_0", "fused_decode_q4f16_matmul_mi355x_const_1"};
  const int32_t slots[] = {0, 1};
  mi355x_wq_module* mod = nullptr;
  EXPECT(mi355x_wq_module_create("fused_decode_q4f16_matmul_mi355x", &spec, names, slots, 2, 0, &mod) == 0 && mod);
  if (!mod) return;
  EXPECT(mi355x_wq_module_num_consts(mod) == 2 && std::strcmp(mi355x_wq_module_const_name(mod, 1), names[1]) == 0);
  EXPECT(mi355x_wq_module_const_name(mod, 2) == nullptr && mi355x_wq_module_const_name(mod, -1) == nullptr);
  EXPECT(mi355x_wq_module_initialized(mod) == 0);
  // a call before init: the reference's message
  mi355x_tvm_value args[2];
  int codes[2] = {7, 7};
  Tensor x((void*)0x20000, MI355X_DL_ROCM, 2, 16, 1, 256), y((void*)0x20000, MI355X_DL_ROCM, 2, 16, 1, 64);
  args[0].v_handle = &x.t;
  args[1].v_handle = &y.t;
  EXPECT(mi355x_wq_module_call(mod, args, codes, 2) == -1 && error_has("has not been initialized"));
  // GetFunction
  mi355x_wq_packed_cfunc fn = nullptr;
  void* handle = nullptr;
  EXPECT(mi355x_wq_module_get_function(mod, "__init_fused_decode_q4f16_matmul_mi355x", &fn, &handle) == 0 && fn);
  EXPECT(mi355x_wq_module_get_function(mod, "no_such_function", &fn, &handle) == 0 && fn == nullptr);
  EXPECT(mi355x_wq_module_get_function(mod, nullptr, &fn, &handle) == -1);
  // init with the wrong count, with NULL tensors, with constants of the wrong shape (all host checks)
  const mi355x_dl_tensor* none[2] = {nullptr, nullptr};
  EXPECT(mi355x_wq_module_init(mod, none, 1) == -1);
  EXPECT(mi355x_wq_module_init(mod, none, 2) == -1);
  std::vector<uint32_t> wq_host(64 * 32);
  std::vector<uint16_t> s_host(64 * 8);
  Tensor wq(wq_host.data(), MI355X_DL_CPU, 1, 32, 64, 32), sc(s_host.data(), MI355X_DL_CPU, 2, 16, 64, 5);
  const mi355x_dl_tensor* bad[2] = {&wq.t, &sc.t};
  EXPECT(mi355x_wq_module_init(mod, bad, 2) == -1);  // K / 5: no group size (or no device here: also -1)
  EXPECT(mi355x_wq_module_initialized(mod) == 0);

  // creation refuses inconsistent descriptions
  mi355x_wq_module* other = nullptr;
  const int32_t x_slot[] = {2, 1};
  EXPECT(mi355x_wq_module_create("f", &spec, names, x_slot, 2, 0, &other) == -1 && other == nullptr);
  const int32_t dup[] = {0, 0};
  EXPECT(mi355x_wq_module_create("f", &spec, names, dup, 2, 0, &other) == -1);
  EXPECT(mi355x_wq_module_create("f", &spec, names, slots, 1, MI355X_WQ_MODULE_TILE_WEIGHTS, &other) == -1);
  EXPECT(mi355x_wq_module_create("", &spec, names, slots, 2, 0, &other) == -1);
  EXPECT(mi355x_wq_module_create("f", nullptr, names, slots, 2, 0, &other) == -1);

  // SaveToBinary / LoadFromBinary
  const int64_t need = mi355x_wq_module_save_to_binary(mod, nullptr, 0);
  EXPECT(need > 0);
  std::vector<unsigned char> blob((size_t)need);
  EXPECT(mi355x_wq_module_save_to_binary(mod, blob.data(), need - 1) == need);  // too small: size only
  EXPECT(mi355x_wq_module_save_to_binary(mod, blob.data(), need) == need);
  int64_t used = 0;
  mi355x_wq_module* back = nullptr;
  EXPECT(mi355x_wq_module_load_from_binary(blob.data(), need, &used, &back) == 0 && back && used == need);
  if (back) {
    EXPECT(std::strcmp(mi355x_wq_module_json(back), mi355x_wq_module_json(mod)) == 0);
    EXPECT(std::strcmp(mi355x_wq_module_symbol(back), mi355x_wq_module_symbol(mod)) == 0);
    mi355x_wq_module_destroy(back);
  }
  // every truncation, in a heap buffer of exactly that size (a read past the end is an ASan report)
  for (int64_t cut = 0; cut < need; ++cut) {
    std::vector<unsigned char> part(blob.begin(), blob.begin() + cut);
    back = nullptr;
    EXPECT(mi355x_wq_module_load_from_binary(part.data(), cut, &used, &back) == -1 && back == nullptr);
  }
  // random corruptions: one to four bytes changed, or a length field blown up
  int loaded = 0;
  for (int it = 0; it < 6000; ++it) {
    std::vector<unsigned char> bad_blob(blob);
    const int edits = 1 + (int)(rnd() % 4);
    for (int e = 0; e < edits; ++e) bad_blob[rnd() % bad_blob.size()] = (unsigned char)rnd();
    if (it % 7 == 0) std::memset(bad_blob.data() + (rnd() % (bad_blob.size() - 8)), 0xFF, 8);
    back = nullptr;
    const int rc = mi355x_wq_module_load_from_binary(bad_blob.data(), (int64_t)bad_blob.size(), &used, &back);
    EXPECT((rc == 0) == (back != nullptr));
    if (back) {
      ++loaded;
      EXPECT(used <= (int64_t)bad_blob.size());
      (void)mi355x_wq_module_json(back);
      mi355x_wq_module_destroy(back);
    }
  }
  std::printf("module loader: %lld truncations refused, 6000 corruptions survived (%d of them still valid modules)\n",
              (long long)need, loaded);
  // the JSON reader on its own
  const std::string good_json = mi355x_wq_module_json(mod);
  other = nullptr;
  EXPECT(mi355x_wq_module_create_from_json("f", good_json.c_str(), names, 2, &other) == 0 && other);
  if (other) mi355x_wq_module_destroy(other);
  const char* broken[] = {"", "{", "}", "[]", "{\"op\":}", "{\"op\":0,,}", "{\"op\":\"matmul\"}", "{\"bits\":99999999999999999999}",
                          "{\"op\":0,\"bits\":4", "nul", "{\"a\":{\"b\":{\"c\":{\"d\":1}}}}", "{\"op\":0,\"bits\":4,\"bits\":8}"};
  for (const char* j : broken) {
    other = nullptr;
    EXPECT(mi355x_wq_module_create_from_json("f", j, names, 2, &other) == -1 && other == nullptr);
  }
  for (size_t cut = 0; cut < good_json.size(); ++cut) {
    other = nullptr;
    const std::string part = good_json.substr(0, cut);
    EXPECT(mi355x_wq_module_create_from_json("f", part.c_str(), names, 2, &other) == -1 && other == nullptr);
  }
  for (int it = 0; it < 3000; ++it) {
    std::string j = good_json;
    j[rnd() % j.size()] = (char)(32 + rnd() % 95);
    other = nullptr;
    const int rc = mi355x_wq_module_create_from_json("f", j.c_str(), names, 2, &other);
    EXPECT((rc == 0) == (other != nullptr));
    if (other) mi355x_wq_module_destroy(other);
  }
  mi355x_wq_module_destroy(mod);
  mi355x_wq_module_destroy(nullptr);
}

int main() {
  check_descriptors();
  check_packed_boundary();
  check_module();
  if (g_failures != 0) {
    std::fprintf(stderr, "%d expectation(s) failed\n", g_failures);
    return 1;
  }
  std::printf("host sanitizer run: ok\n");
  return 0;
}
