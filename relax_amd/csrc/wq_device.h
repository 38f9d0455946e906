// Device-side building blocks shared by the gfx950 kernels: vector types, raw
// buffer loads (out-of-range lanes read 0, which removes every tail branch from
// the hot loops) and the exact int4/int8 -> float16 conversions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace wq {

typedef _Float16 half_t;
typedef half_t half2_t __attribute__((ext_vector_type(2)));
typedef half_t half4_t __attribute__((ext_vector_type(4)));
typedef half_t half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// An offset no buffer of this library can contain (sizes are checked < 2^31 on
// the host): a lane that must not load uses it and receives zeros.
constexpr uint32_t kOobOffset = 0x80000000u;

__device__ __forceinline__ half2_t as_h2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }
__device__ __forceinline__ uint32_t as_u32(half2_t h) { return __builtin_bit_cast(uint32_t, h); }
__device__ __forceinline__ half2_t bcast_h2(half_t s) { return half2_t{s, s}; }

// ---- raw buffer access ------------------------------------------------------
typedef __amdgpu_buffer_rsrc_t rsrc_t;

__device__ __forceinline__ rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  // dword3 0x00020000: 32-bit untyped data format, raw (stride 0) addressing.
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}
__device__ __forceinline__ u32x4 load_b128(rsrc_t r, uint32_t voff) {
  return __builtin_amdgcn_raw_buffer_load_b128(r, voff, 0, 0);
}
__device__ __forceinline__ u32x2 load_b64(rsrc_t r, uint32_t voff) {
  return __builtin_amdgcn_raw_buffer_load_b64(r, voff, 0, 0);
}
__device__ __forceinline__ uint32_t load_b32(rsrc_t r, uint32_t voff) {
  return __builtin_amdgcn_raw_buffer_load_b32(r, voff, 0, 0);
}
__device__ __forceinline__ uint32_t load_b16(rsrc_t r, uint32_t voff) {
  return __builtin_amdgcn_raw_buffer_load_b16(r, voff, 0, 0);
}

// (a & mask) | bits in one VALU op; mask must be wave-uniform (SGPR operand).
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t bits) {
  uint32_t d;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "s"(mask), "v"(bits));
  return d;
}

// ---- exact integer -> float16 conversions -------------------------------------
// A float16 with exponent field 25 (0x6400) has a unit in the last place of 1:
// OR-ing a 4-bit field into mantissa bits 0..3 yields exactly 1024 + field, and
// into bits 4..7 exactly 1024 + 16*field.  Subtracting the offset (and the zero
// point) is exact because the result is a small integer, so the only rounding in
// the whole dequantization is the final multiply by the scale -- the same single
// rounding the CPU path performs.
struct Q4Consts {
  uint32_t magic;   // 0x64006400, kept in a VGPR (gfx9 VOP3 reads one SGPR)
  half2_t sub_lo;   // 1024 + zero_point, both halves
  half2_t mul_hi;   // 1/16
  half2_t sub_hi;   // 64 + zero_point
  half2_t mix_mul;  // (1, 1/16)
  half2_t mix_sub;  // (1024 + zp, 64 + zp)
};

__device__ __forceinline__ Q4Consts make_q4_consts(int zero_point) {
  Q4Consts c;
  c.magic = 0x64006400u;
  asm volatile("" : "+v"(c.magic));  // keep it a register, not a literal
  half_t lo = (half_t)(1024 + zero_point), hi = (half_t)(64 + zero_point);
  c.sub_lo = half2_t{lo, lo};
  c.mul_hi = half2_t{(half_t)0.0625f, (half_t)0.0625f};
  c.sub_hi = half2_t{hi, hi};
  c.mix_mul = half2_t{(half_t)1.0f, (half_t)0.0625f};
  c.mix_sub = half2_t{lo, hi};
  return c;
}

// One packed word -> 4 half2 holding (field - zp) * scale, in the pair order
// (k0,k4) (k1,k5) (k2,k6) (k3,k7).  13 VALU ops per word.
__device__ __forceinline__ void q4_word_paired(uint32_t w, half2_t s2, const Q4Consts& c,
                                               half2_t out[4]) {
  uint32_t w8 = w >> 8;
  half2_t a0 = as_h2(and_or(w, 0x000F000Fu, c.magic)) - c.sub_lo;
  half2_t a1 = __builtin_elementwise_fma(as_h2(and_or(w, 0x00F000F0u, c.magic)), c.mul_hi, -c.sub_hi);
  half2_t a2 = as_h2(and_or(w8, 0x000F000Fu, c.magic)) - c.sub_lo;
  half2_t a3 = __builtin_elementwise_fma(as_h2(and_or(w8, 0x00F000F0u, c.magic)), c.mul_hi, -c.sub_hi);
  out[0] = a0 * s2;
  out[1] = a1 * s2;
  out[2] = a2 * s2;
  out[3] = a3 * s2;
}

// One packed word -> 4 half2 in natural order (k0,k1) (k2,k3) (k4,k5) (k6,k7).
// Byte i of the word is copied under both halves (v_perm), the low half keeps
// field 2i at mantissa bits 0..3 and the high half field 2i+1 at bits 4..7.
// 16 VALU ops per word.
__device__ __forceinline__ void q4_word_natural(uint32_t w, half2_t s2, const Q4Consts& c,
                                                half2_t out[4]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    uint32_t t = __builtin_amdgcn_perm(0u, w, 0x0c000c00u | (uint32_t)i | ((uint32_t)i << 16));
    half2_t h = as_h2(and_or(t, 0x00F0000Fu, c.magic));
    out[i] = __builtin_elementwise_fma(h, c.mix_mul, -c.mix_sub) * s2;
  }
}

// int8 -> float16 in one instruction per weight: v_cvt_f16_i16 with a sub-dword source select
// (byte BYTE of the word, sign-extended) writing the low half (upper half zeroed) or the high half
// (low half kept) of the destination.  Exact for every int8 value.
template <int BYTE>
__device__ __forceinline__ uint32_t cvt_i8_lo(uint32_t w) {
  static_assert(BYTE >= 0 && BYTE < 4, "byte of a 32-bit word");
  uint32_t d;
  if constexpr (BYTE == 0) asm("v_cvt_f16_i16_sdwa %0, sext(%1) dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:BYTE_0" : "=v"(d) : "v"(w));
  else if constexpr (BYTE == 1) asm("v_cvt_f16_i16_sdwa %0, sext(%1) dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:BYTE_1" : "=v"(d) : "v"(w));
  else if constexpr (BYTE == 2) asm("v_cvt_f16_i16_sdwa %0, sext(%1) dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:BYTE_2" : "=v"(d) : "v"(w));
  else asm("v_cvt_f16_i16_sdwa %0, sext(%1) dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:BYTE_3" : "=v"(d) : "v"(w));
  return d;
}
template <int BYTE>
__device__ __forceinline__ uint32_t cvt_i8_hi(uint32_t d, uint32_t w) {
  static_assert(BYTE >= 0 && BYTE < 4, "byte of a 32-bit word");
  if constexpr (BYTE == 0) asm("v_cvt_f16_i16_sdwa %0, sext(%1) dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_0" : "+v"(d) : "v"(w));
  else if constexpr (BYTE == 1) asm("v_cvt_f16_i16_sdwa %0, sext(%1) dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_1" : "+v"(d) : "v"(w));
  else if constexpr (BYTE == 2) asm("v_cvt_f16_i16_sdwa %0, sext(%1) dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_2" : "+v"(d) : "v"(w));
  else asm("v_cvt_f16_i16_sdwa %0, sext(%1) dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_3" : "+v"(d) : "v"(w));
  return d;
}

// int8: one word -> 2 half2, natural order: two conversions and the scale multiply per pair.
// 6 VALU ops per word.
__device__ __forceinline__ void q8_word_natural(uint32_t w, half2_t s2, half2_t out[2]) {
  out[0] = as_h2(cvt_i8_hi<1>(cvt_i8_lo<0>(w), w)) * s2;
  out[1] = as_h2(cvt_i8_hi<3>(cvt_i8_lo<2>(w), w)) * s2;
}

__device__ __forceinline__ half8_t pack_h8(half2_t a, half2_t b, half2_t c, half2_t d) {
  return half8_t{a[0], a[1], b[0], b[1], c[0], c[1], d[0], d[1]};
}

// Operations fused behind the float16 cast of the accumulator, in the order the composite
// applies them: bias add, activation, residual add -- each a single float16 operation with
// one rounding, as the CPU path executes them on float16 tensors.
struct Epilogue {
  const half_t* bias;      // [N], or nullptr
  const half_t* residual;  // [M,N], or nullptr; may be the output buffer itself
  int activation;          // 0 none, 1 relu, 2 gated: y[M, N/2] = multiply(nn.silu(gate), up), see store_gated; 3 gelu
};
constexpr int kActGated = 2;
constexpr int kActGelu = 3;

// nn.gelu on a float16 value as its legalized form x * (0.5 + erf(x * sqrt(0.5)) * 0.5) runs on float16 tensors
// (python/tvm/relax/transform/legalize_ops.py:495-503): every operation rounded once, the constants rounded
// to float16 first, erf evaluated in float32 and rounded.
__device__ __forceinline__ half_t gelu_f16(half_t h) {
  const half_t a = h * (half_t)0.70710678118654752440f;
  const half_t e = (half_t)erff((float)a);
  const half_t b = e * (half_t)0.5f;
  const half_t c = (half_t)0.5f + b;
  return h * c;
}

// Gated tail of a fused gate+up projection.  The weight matrix holds the gate rows 0 .. N/2-1 and the up
// rows N/2 .. N-1; kernels that fuse the tail walk the rows in the interleaved order
// gate 0, up 0, gate 1, up 1, ... (logical row r = physical row r/2 + (r odd ? N/2 : 0)), so that the two
// accumulators of an output land in one lane or in adjacent lanes.
__device__ __forceinline__ int gated_physical_row(int logical, int N) { return (logical >> 1) + ((logical & 1) ? (N >> 1) : 0); }

// multiply(nn.silu(g), u) on float16 values, every operation rounded once as the CPU path executes them:
// e = f16(exp(-g)) (evaluated in float32), d = f16(1 + e), s = f16(1 / d), t = f16(g * s), y = f16(t * u).
// The float32 quotient is correctly rounded and its second rounding to float16 is innocuous.
__device__ __forceinline__ half_t silu_mul(half_t g, half_t u) {
  const half_t e = (half_t)expf(-(float)g);
  const half_t d = (half_t)1 + e;
  const half_t s = (half_t)(1.0f / (float)d);
  const half_t t = g * s;
  return t * u;
}

// y[m, j] of the gated output [M, N/2] from the accumulators of gate row j and up row j
__device__ __forceinline__ void store_gated(half_t* y, int m, int j, int half_n, float acc_gate, float acc_up) {
  y[(size_t)m * half_n + j] = silu_mul((half_t)acc_gate, (half_t)acc_up);
}

// (GELU = false: a build without the gelu branch, for kernels whose register budget it would break;
// their launcher applies gelu in a pass of its own)
template <bool GELU = true>
__device__ __forceinline__ void store_out(const Epilogue& ep, half_t* y, int m, int n, int N, float acc) {
  half_t h = (half_t)acc;
  const size_t idx = (size_t)m * N + n;
  if (ep.bias != nullptr) h = h + ep.bias[n];
  if (ep.activation == 1) h = h > (half_t)0 ? h : (half_t)0;  // max(h, 0) as select(h > 0, h, 0)
  if (GELU && ep.activation == kActGelu) h = gelu_f16(h);
  if (ep.residual != nullptr) h = h + ep.residual[idx];
  y[idx] = h;
}

// Whether rows of y (and of the epilogue operands) can be written two adjacent columns at a
// time with 4-byte accesses: even row length and 4-byte aligned bases (the C ABI only asks for
// 2-byte alignment of y, bias and residual).
__device__ __forceinline__ bool pair_store_ok(const Epilogue& ep, const half_t* y, int N) {
  const uintptr_t bits = reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(ep.bias) |
                         reinterpret_cast<uintptr_t>(ep.residual);
  return ((N & 1) == 0) && ((bits & 3u) == 0);
}

// Columns n (even) and n + 1 of row m; `paired` comes from pair_store_ok.  Same per-element
// arithmetic as store_out.
template <bool GELU = true>
__device__ __forceinline__ void store_out2(const Epilogue& ep, half_t* y, int m, int n, int N, float a0, float a1,
                                           bool paired) {
  if (paired && n + 1 < N) {
    half2_t h = half2_t{(half_t)a0, (half_t)a1};
    const size_t idx = (size_t)m * N + n;
    if (ep.bias != nullptr) h = h + *reinterpret_cast<const half2_t*>(ep.bias + n);
    if (ep.activation == 1) {
      h[0] = h[0] > (half_t)0 ? h[0] : (half_t)0;
      h[1] = h[1] > (half_t)0 ? h[1] : (half_t)0;
    }
    if (GELU && ep.activation == kActGelu) h = half2_t{gelu_f16(h[0]), gelu_f16(h[1])};
    if (ep.residual != nullptr) h = h + *reinterpret_cast<const half2_t*>(ep.residual + idx);
    *reinterpret_cast<half2_t*>(y + idx) = h;
  } else {
    if (n < N) store_out<GELU>(ep, y, m, n, N, a0);
    if (n + 1 < N) store_out<GELU>(ep, y, m, n + 1, N, a1);
  }
}

}  // namespace wq
