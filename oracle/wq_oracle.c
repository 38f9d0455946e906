/*
 * CPU oracle for the weight-only-quantized dequantize + matmul path, plain C.
 *
 * TEST INFRASTRUCTURE ONLY: the shipped library never links or loads this file.
 * It is the checker for the HIP kernels and the host-CPU baseline of the
 * benchmark.
 *
 * Each function walks the loop nest the reference's llvm target executes for the
 * canonical (unscheduled, unfused) module: `decode` materialises the float16
 * weight matrix, `matmul` is a scalar triple loop with float32 products summed
 * sequentially over ascending k, the final cast rounds to nearest even.
 *
 *   unpack / shifts / casts : src/target/llvm/codegen_llvm.cc:1271-1285, 820-852
 *   matmul loop nest        : python/tvm/relax/transform/legalize_ops.py:203-264,
 *                             tests/python/relax/test_transform_legalize_ops_index_linear_algebra.py:283-313
 *   astype                  : python/tvm/relax/transform/legalize_ops.py:157-162
 *
 * float16 is handled in software (bit-exact IEEE binary16, round-to-nearest-even)
 * so the result does not depend on the host's F16C support.  A float16 multiply
 * is "extend both to float32, multiply (exact: 11+11 significand bits), round
 * once to float16", which is what LLVM emits for `fmul half` on a CPU without
 * native half arithmetic.
 *
 * Build: gcc -O2 -ffp-contract=off -fno-fast-math -fopenmp -shared -fPIC
 * (no reassociation, no fused multiply-add: the float32 sum must stay sequential).
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#if defined(_OPENMP)
#include <omp.h>
#endif

static inline float bits_to_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static inline uint32_t f32_to_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}

/* binary16 -> binary32, exact. */
float wq_oracle_f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1Fu;
  uint32_t man = h & 0x3FFu;
  if (exp == 0) {
    if (man == 0) return bits_to_f32(sign);
    /* subnormal: value = man * 2^-24; normalise */
    int e = -1;
    do {
      man <<= 1;
      ++e;
    } while (!(man & 0x400u));
    man &= 0x3FFu;
    return bits_to_f32(sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13));
  }
  if (exp == 31) return bits_to_f32(sign | 0x7F800000u | (man << 13));
  return bits_to_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/* binary32 -> binary16, round to nearest, ties to even. */
uint16_t wq_oracle_f32_to_f16(float f) {
  uint32_t x = f32_to_bits(f);
  uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  uint32_t ax = x & 0x7FFFFFFFu;
  if (ax >= 0x7F800000u) { /* inf / nan */
    if (ax == 0x7F800000u) return (uint16_t)(sign | 0x7C00u);
    return (uint16_t)(sign | 0x7E00u | ((ax >> 13) & 0x3FFu)); /* quiet nan, keep payload top bits */
  }
  if (ax >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u); /* >= 65520 rounds to inf */
  if (ax < 0x33000001u) return sign;                        /* <= 2^-25 rounds to zero (tie -> even 0) */
  int32_t e = (int32_t)(ax >> 23) - 127;
  uint32_t man = (ax & 0x7FFFFFu) | 0x800000u; /* 24-bit significand */
  uint32_t shift;
  uint32_t base;
  if (e < -14) { /* subnormal result: unit is 2^-24 */
    shift = (uint32_t)(13 + (-14 - e));
    base = 0;
  } else {
    shift = 13;
    base = ((uint32_t)(e + 15) << 10) - 0x400u; /* hidden bit of man>>13 adds the 0x400 back */
  }
  uint32_t q = man >> shift;
  uint32_t rem = man & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1u))) ++q;
  return (uint16_t)(sign | (uint16_t)(base + q)); /* carry into exponent is the correct result */
}

/* ---- decode, integer part ------------------------------------------------ */
void wq_oracle_unpack_q4(const uint32_t* wq, int64_t n_rows, int64_t k, uint8_t* out) {
  for (int64_t n = 0; n < n_rows; ++n)
    for (int64_t kk = 0; kk < k; ++kk)
      out[n * k + kk] = (uint8_t)((wq[n * (k / 8) + kk / 8] >> ((uint32_t)(kk % 8) * 4u)) & 15u);
}

void wq_oracle_unpack_q8(const uint32_t* wq, int64_t n_rows, int64_t k, int8_t* out) {
  for (int64_t n = 0; n < n_rows; ++n)
    for (int64_t kk = 0; kk < k; ++kk)
      out[n * k + kk] = (int8_t)(uint8_t)((wq[n * (k / 4) + kk / 4] >> ((uint32_t)(kk % 4) * 8u)) & 255u);
}

/* ---- decode, float16 part ------------------------------------------------ */
/* bits = 4: Wd = (f16(w) - f16(7)) * S[n, k/group];  bits = 8: Wd = f16(int8 w) * S[n, k/group]. */
int wq_oracle_dequant(int bits, int64_t group, const uint32_t* wq, const uint16_t* s, int64_t n_rows,
                      int64_t k, uint16_t* wd, int nthreads) {
  if ((bits != 4 && bits != 8) || group <= 0 || k % group != 0 || k % (32 / bits) != 0) return -1;
  const int64_t per_word = 32 / bits;
  const int64_t kw = k / per_word, kg = k / group;
  (void)nthreads;
#if defined(_OPENMP)
#pragma omp parallel for num_threads(nthreads > 0 ? nthreads : 1) schedule(static)
#endif
  for (int64_t n = 0; n < n_rows; ++n) {
    for (int64_t kk = 0; kk < k; ++kk) {
      uint32_t word = wq[n * kw + kk / per_word];
      float centred;
      if (bits == 4) {
        uint32_t w = (word >> ((uint32_t)(kk % 8) * 4u)) & 15u;
        /* f16(w) - f16(7): both exact, difference exact in float16 */
        centred = wq_oracle_f16_to_f32(wq_oracle_f32_to_f16((float)w - 7.0f));
      } else {
        int8_t w = (int8_t)(uint8_t)((word >> ((uint32_t)(kk % 4) * 8u)) & 255u);
        centred = (float)w; /* |w| <= 128 is exact in float16 */
      }
      float scale = wq_oracle_f16_to_f32(s[n * kg + kk / group]);
      wd[n * k + kk] = wq_oracle_f32_to_f16(centred * scale);
    }
  }
  return 0;
}

/* ---- matmul: y32[m,n] = sum_k f32(x[m,k]) * f32(Wd[n,k]), sequential in k ---- */
void wq_oracle_matmul_f32acc(const uint16_t* x, const uint16_t* wd, int64_t m_rows, int64_t n_rows,
                             int64_t k, float* y32, int nthreads) {
  (void)nthreads;
#if defined(_OPENMP)
#pragma omp parallel for num_threads(nthreads > 0 ? nthreads : 1) schedule(static)
#endif
  for (int64_t n = 0; n < n_rows; ++n) {
    for (int64_t m = 0; m < m_rows; ++m) {
      float acc = 0.0f;
      for (int64_t kk = 0; kk < k; ++kk)
        acc = acc + wq_oracle_f16_to_f32(x[m * k + kk]) * wq_oracle_f16_to_f32(wd[n * k + kk]);
      y32[m * n_rows + n] = acc;
    }
  }
}

void wq_oracle_cast_f16(const float* y32, int64_t count, uint16_t* y) {
  for (int64_t i = 0; i < count; ++i) y[i] = wq_oracle_f32_to_f16(y32[i]);
}

/* ---- whole path; `wd_scratch` is [N,K] float16, `y32_scratch` is [M,N] float32 ---- */
int wq_oracle_wq_matmul(int bits, int64_t group, const uint16_t* x, const uint32_t* wq,
                        const uint16_t* s, int64_t m_rows, int64_t n_rows, int64_t k,
                        uint16_t* wd_scratch, float* y32_scratch, uint16_t* y, int nthreads) {
  if (wq_oracle_dequant(bits, group, wq, s, n_rows, k, wd_scratch, nthreads) != 0) return -1;
  wq_oracle_matmul_f32acc(x, wd_scratch, m_rows, n_rows, k, y32_scratch, nthreads);
  wq_oracle_cast_f16(y32_scratch, m_rows * n_rows, y);
  return 0;
}

/* ---- fused tail: y[m,n] = (relu?)(y[m,n] + bias[n]) + residual[m,n], each add one float16
 * rounding (float32 sum of two float16 values, rounded to float16: the double rounding is
 * innocuous because float32 carries 24 >= 2*11 + 2 significand bits); relu is
 * select(t > 0, t, 0) -- src/target/llvm/codegen_llvm.cc:1500-1504.  bias / residual may be
 * NULL. ---- */
static uint16_t gelu_f16(uint16_t h);

void wq_oracle_epilogue(uint16_t* y, int64_t m_rows, int64_t n_rows, const uint16_t* bias, int activation,
                        const uint16_t* residual) {
  const int relu = activation == 1, gelu = activation == 3;
  for (int64_t m = 0; m < m_rows; ++m)
    for (int64_t n = 0; n < n_rows; ++n) {
      uint16_t h = y[m * n_rows + n];
      if (bias) h = wq_oracle_f32_to_f16(wq_oracle_f16_to_f32(h) + wq_oracle_f16_to_f32(bias[n]));
      if (relu) h = (wq_oracle_f16_to_f32(h) > 0.0f) ? h : (uint16_t)0;
      if (gelu) h = gelu_f16(h);
      if (residual)
        h = wq_oracle_f32_to_f16(wq_oracle_f16_to_f32(h) + wq_oracle_f16_to_f32(residual[m * n_rows + n]));
      y[m * n_rows + n] = h;
    }
}

/* ---- nn.gelu on one float16 value: the legalized form x * (0.5 + erf(x * sqrt(0.5)) * 0.5) of
 * python/tvm/relax/transform/legalize_ops.py:495-503 evaluated on float16, one rounding per operation:
 * a = f16(x * f16(sqrt(0.5))), e = f16(erff(a)), b = f16(e * 0.5), c = f16(0.5 + b), out = f16(x * c).
 * (The reference's CPU path gives float16 erf no extern name, src/target/intrin_rule.h:39-48; evaluating it
 * in float32 and rounding is what the float16 exp of the same path does.) ---- */
static uint16_t gelu_f16(uint16_t h) {
  const float x = wq_oracle_f16_to_f32(h);
  const float c0 = wq_oracle_f16_to_f32(wq_oracle_f32_to_f16(0.70710678118654752440f));
  const float a = wq_oracle_f16_to_f32(wq_oracle_f32_to_f16(x * c0));
  const float e = wq_oracle_f16_to_f32(wq_oracle_f32_to_f16(erff(a)));
  const float b = wq_oracle_f16_to_f32(wq_oracle_f32_to_f16(e * 0.5f));
  const float c = wq_oracle_f16_to_f32(wq_oracle_f32_to_f16(0.5f + b));
  return wq_oracle_f32_to_f16(x * c);
}

/* ---- gated tail: out[m, j] = multiply(nn.silu(y[m, j]), y[m, j + n/2]) for j < n/2, the float16
 * operation sequence of python/tvm/relax/transform/legalize_ops.py:506-510 and
 * src/target/intrin_rule.cc:135-141: e = f16(expf(-g)), d = f16(1 + e), s = f16(1 / d),
 * t = f16(g * s), out = f16(t * u).  Sum, quotient and products of float16 values rounded through
 * float32 equal one rounding (24 >= 2*11 + 2 significand bits). ---- */
void wq_oracle_silu_mul(const uint16_t* y, int64_t m_rows, int64_t n_rows, uint16_t* out) {
  const int64_t half = n_rows / 2;
  for (int64_t m = 0; m < m_rows; ++m)
    for (int64_t j = 0; j < half; ++j) {
      const float g = wq_oracle_f16_to_f32(y[m * n_rows + j]);
      const float u = wq_oracle_f16_to_f32(y[m * n_rows + half + j]);
      const float e = wq_oracle_f16_to_f32(wq_oracle_f32_to_f16(expf(-g)));
      const float d = wq_oracle_f16_to_f32(wq_oracle_f32_to_f16(1.0f + e));
      const float s = wq_oracle_f16_to_f32(wq_oracle_f32_to_f16(1.0f / d));
      const float t = wq_oracle_f16_to_f32(wq_oracle_f32_to_f16(g * s));
      out[m * half + j] = wq_oracle_f32_to_f16(t * u);
    }
}

int wq_oracle_max_threads(void) {
#if defined(_OPENMP)
  return omp_get_max_threads();
#else
  return 1;
#endif
}
