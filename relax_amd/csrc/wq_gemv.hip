// GEMV kernel for decode batches (M <= 16): y[M,N] = x[M,K] @ dequant(Wq,S)^T.
//
// Bound: HBM bandwidth.  Every byte of packed weight is read exactly once with
// 16-byte buffer loads; the activations are staged once per workgroup in LDS, so
// that the only long-latency traffic in the loop is the weight stream and its
// prefetch depth is not tied to activation registers (LDS reads are counted by a
// different wait counter than global loads).
//
// Work split: a workgroup owns R tiles of 16 weight rows; its WAVES wavefronts
// split K in "super steps" of 4*D chunks (chunk = the k covered by one 16-byte
// lane load: 32 for int4, 16 for int8).  Lane (col = lane % 16, kq = lane / 16)
// owns weight row `col` of each tile and the D consecutive chunks kq*D .. kq*D+D-1
// of the super step, so its group scales are one contiguous load per super step.
// Chunk d of all four kq feeds NJ v_mfma_f32_16x16x32_f16 (A = activations,
// B = the weights dequantized in registers to exactly the float16 value the CPU
// path materialises).  Super steps are double buffered in registers: the loads of
// the next one are in flight while the current one is consumed.  The K split is
// reduced through LDS; rows of the MFMA tile beyond M carry unspecified values
// that only reach output rows which are never stored.
//
// The int4 activations are written to LDS already in the pair order
// (k0,k4)(k1,k5)(k2,k6)(k3,k7) the nibble unpack produces, so the loop has no
// permutes at all.
#include "wq_device.h"
#include "wq_internal.h"

namespace wq {

template <int BITS, int R, int D, int SPL>
struct GemvBuf {
  u32x4 w[R][D];
  uint32_t sc[R][SPL > 1 ? SPL / 2 : 1];  // SPL float16 scales, packed two per register
};

template <int BITS, int R, int WAVES, int D, int SPL>
__global__ __launch_bounds__(WAVES * 64) void wq_gemv_kernel(
    const half_t* __restrict__ x, const uint32_t* __restrict__ wq, const half_t* __restrict__ scales,
    half_t* __restrict__ y, int M, int N, int K, int group_shift, int zero_point, int lds_stride) {
  constexpr int CH = 128 / BITS;  // k per 16-byte lane load
  constexpr int NJ = CH / 8;      // MFMAs per lane load
  static_assert(SPL == 1 || SPL == D, "one scale per super step, or one per chunk");
  static_assert(SPL == 1 || (SPL % 2 == 0 && SPL <= 8), "scale vector is 4, 8 or 16 bytes");
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keeps loop control scalar
  const int col = lane & 15, kq = lane >> 4;

  extern __shared__ __attribute__((aligned(16))) unsigned char wq_gemv_smem[];
  half_t* xs = reinterpret_cast<half_t*>(wq_gemv_smem);  // [M][lds_stride] halves
  __shared__ float red[WAVES][R][4][64];

  const uint32_t row_bytes = (uint32_t)K * BITS / 8;
  const int nchunks = K / CH;
  const int nsuper = (nchunks + 4 * D - 1) / (4 * D);
  const int per_wave = (nsuper + WAVES - 1) / WAVES;
  const int ss_begin = wave * per_wave;
  const int ss_end = min(ss_begin + per_wave, nsuper);
  const uint32_t groups_per_row = (uint32_t)nchunks >> group_shift;

  const rsrc_t rw = make_rsrc(wq, (uint32_t)N * row_bytes);
  const rsrc_t rs = make_rsrc(scales, (uint32_t)N * groups_per_row * 2u);

  uint32_t wbase[R], sbase[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int n = min((int)(blockIdx.x * R + r) * 16 + col, N - 1);  // rows past N: computed, not stored
    wbase[r] = (uint32_t)n * row_bytes;
    sbase[r] = (uint32_t)n * groups_per_row * 2u;
  }

  auto load_super = [&](GemvBuf<BITS, R, D, SPL>& b, int ss) {
    const int chunk0 = ss * 4 * D + kq * D;
    // D > 1 is only launched when K is a multiple of 4*D chunks, so a lane's D
    // chunks are valid together; D == 1 checks its single chunk.
    const bool ok = (ss < ss_end) && (chunk0 < nchunks);
    const uint32_t winc = ok ? (uint32_t)chunk0 * 16u : kOobOffset;
    const uint32_t sinc = ok ? ((uint32_t)chunk0 >> group_shift) * 2u : kOobOffset;
#pragma unroll
    for (int r = 0; r < R; ++r) {
#pragma unroll
      for (int d = 0; d < D; ++d) b.w[r][d] = load_b128(rw, wbase[r] + winc + d * 16u);
      if constexpr (SPL == 1) {
        b.sc[r][0] = load_b16(rs, sbase[r] + sinc);
      } else if constexpr (SPL == 2) {
        b.sc[r][0] = load_b32(rs, sbase[r] + sinc);
      } else if constexpr (SPL == 4) {
        const u32x2 v = load_b64(rs, sbase[r] + sinc);
        b.sc[r][0] = v[0];
        b.sc[r][1] = v[1];
      } else {
        const u32x4 v = load_b128(rs, sbase[r] + sinc);
#pragma unroll
        for (int i = 0; i < 4; ++i) b.sc[r][i] = v[i];
      }
    }
  };

  // ---- stage the activations in LDS (whole K, zero padded to a k-step) ----------
  // The first two activation vectors per thread are requested before the first
  // weights and stored after them: global loads retire in order, so this keeps the
  // LDS fill from waiting on the (much slower) first weight loads.
  GemvBuf<BITS, R, D, SPL> b0, b1;
  {
    const int kpad = ((K + 4 * CH - 1) / (4 * CH)) * (4 * CH);
    const int vec_per_row = kpad / 8;
    const int total = M * vec_per_row;
    const rsrc_t rx = make_rsrc(x, (uint32_t)M * (uint32_t)K * 2u);
    auto x_load = [&](int idx) -> u32x4 {
      const int m = idx / vec_per_row, kv = idx - m * vec_per_row;
      const bool ok = idx < total && kv * 8 < K;
      return load_b128(rx, ok ? ((uint32_t)m * (uint32_t)K + (uint32_t)kv * 8u) * 2u : kOobOffset);
    };
    auto x_store = [&](int idx, u32x4 v) {
      if (idx >= total) return;
      const int m = idx / vec_per_row, kv = idx - m * vec_per_row;
      if constexpr (BITS == 4) {
        u32x4 p;
        p[0] = __builtin_amdgcn_perm(v[2], v[0], 0x05040100u);
        p[1] = __builtin_amdgcn_perm(v[2], v[0], 0x07060302u);
        p[2] = __builtin_amdgcn_perm(v[3], v[1], 0x05040100u);
        p[3] = __builtin_amdgcn_perm(v[3], v[1], 0x07060302u);
        v = p;
      }
      *reinterpret_cast<u32x4*>(xs + (size_t)m * lds_stride + kv * 8) = v;
    };
    constexpr int NT = WAVES * 64;
    const u32x4 x0 = x_load(tid), x1 = x_load(tid + NT);
    __builtin_amdgcn_sched_barrier(0);
    load_super(b0, ss_begin);
    __builtin_amdgcn_sched_barrier(0);
    x_store(tid, x0);
    x_store(tid + NT, x1);
    for (int idx = tid + 2 * NT; idx < total; idx += NT) x_store(idx, x_load(idx));
  }
  __syncthreads();

  float4_t acc[R];
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = float4_t{0.f, 0.f, 0.f, 0.f};
  const Q4Consts qc = make_q4_consts(zero_point);
  // lanes of MFMA rows beyond M read row 0: their products land in rows that are not stored
  const half_t* xrow = xs + (size_t)(col < M ? col : 0) * lds_stride;

  auto compute_super = [&](const GemvBuf<BITS, R, D, SPL>& b, int ss) {
    const half_t* xp = xrow + (ss * 4 * D + kq * D) * CH;
    half8_t a[2][NJ];  // activations of chunk d+1 are read from LDS while chunk d is consumed
#pragma unroll
    for (int j = 0; j < NJ; ++j) a[0][j] = *reinterpret_cast<const half8_t*>(xp + j * 8);
#pragma unroll
    for (int d = 0; d < D; ++d) {
      if (d + 1 < D) {
#pragma unroll
        for (int j = 0; j < NJ; ++j)
          a[(d + 1) & 1][j] = *reinterpret_cast<const half8_t*>(xp + (d + 1) * CH + j * 8);
      }
#pragma unroll
      for (int r = 0; r < R; ++r) {
        uint32_t sbits;
        if constexpr (SPL == 1) sbits = b.sc[r][0];
        else sbits = (d & 1) ? (b.sc[r][d >> 1] >> 16) : b.sc[r][d >> 1];
        const half2_t s2 = bcast_h2(__builtin_bit_cast(half_t, (uint16_t)sbits));
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
          half8_t bm;
          if constexpr (BITS == 4) {
            half2_t h[4];
            q4_word_paired(b.w[r][d][j], s2, qc, h);
            bm = pack_h8(h[0], h[1], h[2], h[3]);
          } else {
            half2_t h0[2], h1[2];
            q8_word_natural(b.w[r][d][2 * j], s2, h0);
            q8_word_natural(b.w[r][d][2 * j + 1], s2, h1);
            bm = pack_h8(h0[0], h0[1], h1[0], h1[1]);
          }
          acc[r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[d & 1][j], bm, acc[r], 0, 0, 0);
        }
      }
    }
  };

  // Two super steps per trip, unconditionally: with an early exit between them the
  // compiler sinks the prefetch below the compute.  A trailing odd step loads
  // zeros (out-of-range offsets) and multiplies them with valid activations.
  for (int ss = ss_begin; ss < ss_end; ss += 2) {
    load_super(b1, ss + 1);
    __builtin_amdgcn_sched_barrier(0);
    compute_super(b0, ss);
    __builtin_amdgcn_sched_barrier(0);
    load_super(b0, ss + 2);
    __builtin_amdgcn_sched_barrier(0);
    compute_super(b1, min(ss + 1, nsuper - 1));
    __builtin_amdgcn_sched_barrier(0);
  }

  // ---- reduce the K split across wavefronts, convert, store -----------------------
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[wave][r][i][lane] = acc[r][i];
  __syncthreads();
  for (int idx = tid; idx < R * 256; idx += WAVES * 64) {
    const int r = idx >> 8, i = (idx >> 6) & 3, l = idx & 63;
    const int m = 4 * (l >> 4) + i;
    const int n = (blockIdx.x * R + r) * 16 + (l & 15);
    if (m < M && n < N) {
      float sum = 0.f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) sum += red[w][r][i][l];
      y[(size_t)m * N + n] = (half_t)sum;
    }
  }
}

namespace {

constexpr size_t kMaxXLdsBytes = 100 * 1024;

size_t x_lds_stride(const Problem& p) {
  const int ch = 128 / p.bits;
  const int64_t kpad = ((p.k + 4 * ch - 1) / (4 * ch)) * (4 * ch);
  return (size_t)kpad + 8;  // +16 bytes: consecutive rows start 4 banks apart
}

template <int BITS, int R, int WAVES, int D, int SPL>
void launch_one(const Problem& p, int group_shift) {
  const int tiles = (int)((p.n + 15) / 16);
  const size_t stride = x_lds_stride(p);
  const size_t lds = (size_t)p.m * stride * sizeof(half_t);
  dim3 grid((tiles + R - 1) / R), block(WAVES * 64);
  static bool attr_set = false;  // idempotent; a race only repeats the same call
  if (!attr_set) {
    (void)hipFuncSetAttribute((const void*)wq_gemv_kernel<BITS, R, WAVES, D, SPL>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxXLdsBytes);
    attr_set = true;
  }
  hipLaunchKernelGGL((wq_gemv_kernel<BITS, R, WAVES, D, SPL>), grid, block, lds, p.stream,
                     (const half_t*)p.x, (const uint32_t*)p.wq, (const half_t*)p.scales,
                     (half_t*)p.y, (int)p.m, (int)p.n, (int)p.k, group_shift, p.zero_point,
                     (int)stride);
}

// D chunks per lane need K to be a multiple of 4*D chunks, and the lane's D
// chunks to share one scale (SPL = 1) or to have one each (SPL = D).
template <int BITS, int R, int WAVES, int D>
bool try_launch(const Problem& p, int group_shift) {
  const int ch = 128 / BITS;
  if (D > 1 && p.k % (4 * D * ch) != 0) return false;
  if (group_shift == 0) {
    launch_one<BITS, R, WAVES, D, D>(p, group_shift);
    return true;
  }
  if ((1 << group_shift) >= D) {
    launch_one<BITS, R, WAVES, D, 1>(p, group_shift);
    return true;
  }
  return false;
}

template <int BITS>
bool dispatch(const Problem& p, int gs, int variant) {
  switch (variant) {
    case 1: return try_launch<BITS, 1, 8, 1>(p, gs);
    case 2: return try_launch<BITS, 1, 8, 2>(p, gs);
    case 3: return try_launch<BITS, 1, 8, 4>(p, gs);
    case 4: return try_launch<BITS, 2, 8, 1>(p, gs);
    case 5: return try_launch<BITS, 2, 8, 2>(p, gs);
    case 6: return try_launch<BITS, 2, 8, 4>(p, gs);
    case 7: return try_launch<BITS, 1, 4, 2>(p, gs);
    case 8: return try_launch<BITS, 1, 4, 4>(p, gs);
    case 9: return try_launch<BITS, 2, 4, 2>(p, gs);
    case 10: return try_launch<BITS, 2, 4, 4>(p, gs);
    case 11: return try_launch<BITS, 1, 16, 1>(p, gs);
    case 12: return try_launch<BITS, 1, 16, 2>(p, gs);
    case 13: return try_launch<BITS, 2, 16, 1>(p, gs);
    case 14: return try_launch<BITS, 2, 16, 2>(p, gs);
    case 15: return try_launch<BITS, 4, 8, 1>(p, gs);
    case 16: return try_launch<BITS, 4, 8, 2>(p, gs);
    default: return false;
  }
}

}  // namespace

bool gemv_applicable(const Problem& p) {
  return p.m <= 16 && (size_t)p.m * x_lds_stride(p) * sizeof(half_t) <= kMaxXLdsBytes;
}

int launch_gemv(const Problem& p, int variant) {
  const int ch = 128 / p.bits;
  int ratio = p.group / ch, gs = 0;
  while ((1 << gs) < ratio) ++gs;
  if (ratio < 1 || (1 << gs) != ratio || p.group % ch != 0) {
    set_error("gemv kernel: group %d must be %d times a power of two", p.group, ch);
    return -1;
  }
  if (!gemv_applicable(p)) {
    set_error("gemv kernel: M=%lld, K=%lld activations do not fit the %zu-byte LDS staging area",
              (long long)p.m, (long long)p.k, kMaxXLdsBytes);
    return -1;
  }
  bool ok;
  if (variant == 0) {
    // Measured on MI355X (Llama-2-7B shapes): decode batches up to 4 rows run best
    // with one row tile per 4-wave workgroup; larger batches re-read the staged
    // activations per workgroup, so they take 4 tiles per 8-wave workgroup.  The
    // two-chunk variants need K to be a multiple of 8 chunks; otherwise fall back.
    const int first = p.m <= 4 ? 7 : 16, second = p.m <= 4 ? 1 : 15;
    ok = p.bits == 4 ? (dispatch<4>(p, gs, first) || dispatch<4>(p, gs, second))
                     : (dispatch<8>(p, gs, first) || dispatch<8>(p, gs, second));
  } else {
    ok = p.bits == 4 ? dispatch<4>(p, gs, variant) : dispatch<8>(p, gs, variant);
  }
  if (!ok) {
    set_error("gemv kernel: variant %d does not apply to K=%lld group=%d", variant, (long long)p.k,
              p.group);
    return -1;
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("gemv kernel launch failed: %s", hipGetErrorString(e));
    return -1;
  }
  return 0;
}

}  // namespace wq
