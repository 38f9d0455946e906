// Skinny (GEMV-class) kernel for M <= 64: y[M,N] = x[M,K] @ dequant(Wq,S)^T.
//
// Bound: HBM bandwidth.  Each byte of packed weight is read exactly once with a
// 16-byte buffer load per lane, dequantized in registers (exactly the float16
// value the CPU path materialises) and consumed by v_mfma_f32_16x16x32_f16 with
// the activations as the other operand, so the same kernel serves M = 1 .. 64
// without the VALU ever becoming the limit at large M.
//
// Work split: a workgroup owns R row tiles of 16 output features; its WAVES
// wavefronts split K between them and add their partial tiles through LDS.
// Inside a wavefront, lane (col = lane % 16, kq = lane / 16) owns weight row
// `col` of the tile and the kq-th 16-byte chunk of every 64-byte row segment, so
// one load instruction covers 16 rows x 64 contiguous bytes.
//
// TILED: weights and scales are addressed in the tile-major layout (wq_tiled.hip); a load
// instruction then reads two runs of 512 contiguous bytes.
//
// Tails never branch: activation rows >= M, chunks >= K and k-steps past the
// wavefront's share are loaded from an out-of-range buffer offset, which returns
// zeros (zero scale => zero weight, zero activation); weight rows >= N are
// clamped to the last row and their results are not stored.
#include "wq_device.h"
#include "wq_internal.h"

namespace wq {

__device__ __forceinline__ bool m_ok_row(int row, int M) { return row < M; }

// The wavefront-private LDS exchanges below (activations, canonical weights, scales) rely on two things: the
// hardware executes a wavefront's LDS instructions in order, and every exchange is "all 64 lanes store, then all
// load" with unconditional stores of the loaded type's size or more, which the compiler cannot move the loads
// across or forward from (it must assume they alias).  Wavefront-scope fences between stores and loads state the
// same explicitly but cost 2 - 4 % here (they also stop the scheduler from interleaving the exchanges of
// neighbouring k-steps); the staged builds are pinned bit for bit against the direct ones by the tests instead.
template <int BITS, int R, int MT, int U>
struct SkinnyBatch {
  static constexpr int NJ = (128 / BITS) / 8;
  u32x4 w[U][R];
  uint32_t sc[U][R];
  u32x2 ss[U][(R + 3) / 4];  // staged scales: a k-step's scales of 64 rows per load (canonical staged builds)
  u32x4 xa[U][MT][NJ];
};

// XST: the activations of a k-step reach the MFMA operand registers through a wavefront-private LDS area
// instead of directly.  Directly, lane (row m, chunk kq) loads the 16-byte pieces of its own row: 64 pieces
// from 16 rows per instruction, 64 tag lookups in the L1.  Staged, a load instruction covers 1 KB of four
// rows (8 lines), the wavefront stores the pieces to LDS as loaded and every lane reads back the pieces of
// its operand; which piece a lane loads is XOR-swizzled with the row on the global side so that the
// reads of 16 rows at one position fall on 16 different bank groups.
template <int BITS, int R, int MT, int WAVES, int U, bool TILED, bool XST = false>
__global__ __launch_bounds__(WAVES * 64) void wq_skinny_kernel(
    const half_t* __restrict__ x, const uint32_t* __restrict__ wq, const half_t* __restrict__ scales,
    half_t* y, int M, int N, int K, int group_shift, int zero_point, const Epilogue ep, int slice_rows) {
  constexpr int CH = 128 / BITS;  // k covered by one 16-byte lane load: 32 / 16
  // more than 64 rows: blockIdx.y picks a slice of slice_rows (<= 16 MT) rows; every slice walks all weights
  const int m0 = (int)blockIdx.y * slice_rows;
  constexpr int NJ = CH / 8;      // MFMAs fed by one lane load: 4 / 2
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform loop control
  const int col = lane & 15;
  const int kq = lane >> 4;

  const uint32_t row_bytes = (uint32_t)K * BITS / 8;
  const int nchunks = K / CH;
  const int nsteps = (nchunks + 3) >> 2;
  const int per_wave = (nsteps + WAVES - 1) / WAVES;
  const int ks_begin = wave * per_wave;
  const int ks_end = min(ks_begin + per_wave, nsteps);
  const uint32_t groups_per_row = (uint32_t)nchunks >> group_shift;

  // (tile-major buffers hold whole 16-row tiles, zero filled past N)
  const uint32_t n_stored = TILED ? ((uint32_t)N + 15u) / 16u * 16u : (uint32_t)N;
  const uint32_t nsuper = row_bytes / 128u;  // 128-byte super steps per weight row (tile-major addressing)
  const rsrc_t rw = make_rsrc(wq, n_stored * row_bytes);
  const rsrc_t rs = make_rsrc(scales, n_stored * groups_per_row * 2u);
  const rsrc_t rx = make_rsrc(x, (uint32_t)M * (uint32_t)K * 2u);

  // per-lane row bases.  Weight rows past N are clamped to the last row (their
  // results are never stored); activation rows past M read zeros.
  uint32_t wbase[R], sbase[R], xbase[MT];
  bool xrow_ok[MT];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int n = min((int)(blockIdx.x * R + r) * 16 + col, (int)n_stored - 1);
    if constexpr (TILED) {
      // chunk c of row n: ((tile*S + c/8)*2 + c%2)*1024 + ((c%8)/2*16 + n%16)*16; its scale (int4) is
      // half c%2 of the 4-byte pair at ((tile*S + c/8)*64 + (c%8)/2*16 + n%16)*4, (int8) the float16 at
      // ((tile*S + c/8)*16 + n%16)*2
      const uint32_t tile = (uint32_t)n >> 4, c16 = (uint32_t)n & 15u;
      wbase[r] = tile * nsuper * 2048u + c16 * 16u;
      sbase[r] = BITS == 4 ? (tile * nsuper * 64u + c16) * 4u : (tile * nsuper * 16u + c16) * 2u;
    } else {
      wbase[r] = (uint32_t)n * row_bytes;
      sbase[r] = (uint32_t)n * groups_per_row * 2u;
    }
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = m0 + mt * 16 + col;
    xrow_ok[mt] = m < M;
    xbase[mt] = (uint32_t)m * (uint32_t)K * 2u;
  }

  // staged activations: ROWB bytes of every row per k-step, MT * 4 KB (int4) per wavefront
  constexpr int ROWB = 4 * CH * 2;            // 256 (int4) / 128 (int8)
  constexpr int PIECES = ROWB / 16;           // 16-byte pieces per row and k-step
  constexpr int RPI = 64 / PIECES;            // rows one load instruction covers: 4 / 8
  constexpr int XI = MT * 16 / RPI;           // load instructions per k-step (= MT * NJ)
  static_assert(XI == MT * NJ, "the staged form uses the registers of the direct one");
  // (canonical weights take the same way: a k-step's 64 bytes of 16 R rows, 16 rows per load instruction
  // instead of 64 pieces from 16 rows each; R KB per wavefront)
  constexpr bool WST = XST && !TILED;
  // (and so do their scales: a lane loads the 8 bytes -- int4, four groups -- or 2 bytes -- int8, one group -- that a
  // row contributes to a k-step, one row per lane, instead of every lane its own 2 bytes from 16 rows per tile:
  // a quarter of the scale loads.  The launcher admits these builds for the standard quantizations only, int4 with
  // whole k-steps.)
  constexpr int NSI = (R + 3) / 4;  // scale load instructions per k-step
  constexpr int kWaveStage = MT * 16 * ROWB + (WST ? R * 1024 + NSI * 512 : 0);
  constexpr size_t kRedBytes = (size_t)WAVES * R * MT * 1024, kStageBytes = XST ? (size_t)WAVES * kWaveStage : 0;
  __shared__ __attribute__((aligned(16))) unsigned char smem[kRedBytes > kStageBytes ? kRedBytes : kStageBytes];
  unsigned char* const xst = smem + (size_t)wave * kWaveStage;
  unsigned char* const wst = xst + MT * 16 * ROWB;
  unsigned char* const sst = wst + R * 1024;
  uint32_t sl_base[NSI];
  bool sl_ok[NSI];
  if constexpr (WST) {
#pragma unroll
    for (int i = 0; i < NSI; ++i) {
      const int row = i * 64 + lane;  // among the workgroup's R * 16 rows
      sl_ok[i] = row < R * 16;
      sl_base[i] = (uint32_t)min((int)(blockIdx.x * R) * 16 + row, (int)n_stored - 1) * groups_per_row * 2u;
    }
  }
  const uint32_t ss_rd = BITS == 4 ? (uint32_t)(col * 8 + kq * 2) : (uint32_t)(col * 2);
  // loader: instruction t reads rows 16 t + lane / 4 of the workgroup's R tiles, piece (lane % 4) ^ (row / 4 % 4);
  // operand lane (col, kq) of tile r finds its piece at position kq ^ (col / 4 % 4) of row 16 r + col
  uint32_t wl_base[R];
  int wl_piece = 0;
  if constexpr (WST) {
    wl_piece = (lane & 3) ^ ((lane >> 4) & 3);
#pragma unroll
    for (int t = 0; t < R; ++t) {
      const int n = min((int)(blockIdx.x * R + t) * 16 + (lane >> 2), (int)n_stored - 1);
      wl_base[t] = (uint32_t)n * row_bytes + (uint32_t)wl_piece * 16u;
    }
  }
  const uint32_t ws_rd = (uint32_t)(col * 64 + ((kq ^ ((col >> 2) & 3)) * 16));
  // (256-byte rows span all 64 banks: 16 rows need 16 positions; 128-byte rows alternate between the bank halves,
  // so a pair of rows shares a position)
  auto swz = [](int row) { return PIECES == 16 ? (row & 15) : ((row >> 1) & 7); };
  uint32_t xs_rd[MT][NJ];  // where lane (col, kq) finds piece kq * NJ + j of row mt * 16 + col
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
      xs_rd[mt][j] = (uint32_t)((mt * 16 + col) * ROWB + (((kq * NJ + j) ^ swz(mt * 16 + col)) * 16));
  // the row and the piece this lane loads in instruction t: row t * RPI + lane / PIECES, stored piece lane % PIECES
  uint32_t xl_base[XI];
#pragma unroll
  for (int t = 0; t < XI; ++t) {
    const int local = t * RPI + lane / PIECES, row = m0 + local;
    const int piece = (lane % PIECES) ^ swz(local);
    xl_base[t] = (m_ok_row(row, M)) ? (uint32_t)row * (uint32_t)K * 2u + (uint32_t)piece * 16u : kOobOffset;
  }

  float4_t acc[R][MT];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[r][mt] = float4_t{0.f, 0.f, 0.f, 0.f};

  Q4Consts qc = make_q4_consts(zero_point);

  auto load_batch = [&](SkinnyBatch<BITS, R, MT, U>& b, int ks0) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int ks = ks0 + u;
      const int chunk = ks * 4 + kq;
      const bool ok = (ks < ks_end) && (chunk < nchunks);
      const uint32_t uc = (uint32_t)chunk, c8 = uc & 7u;
      const uint32_t winc = !ok ? kOobOffset
                            : TILED ? (uc >> 3) * 2048u + (c8 & 1u) * 1024u + (c8 >> 1) * 256u : uc * 16u;
      const uint32_t sinc = !ok ? kOobOffset
                            : !TILED ? (uc >> group_shift) * 2u
                            : BITS == 4 ? (uc >> 3) * 256u + (c8 >> 1) * 64u + (c8 & 1u) * 2u : (uc >> 3) * 32u;
      const uint32_t xinc = (uint32_t)chunk * (CH * 2u);
      if constexpr (WST) {
        const bool okw = (ks < ks_end) && (ks * 4 + wl_piece < nchunks);
#pragma unroll
        for (int t = 0; t < R; ++t) b.w[u][t] = load_b128(rw, okw ? wl_base[t] + (uint32_t)ks * 64u : kOobOffset);
#pragma unroll
        for (int i = 0; i < NSI; ++i) {
          const bool oks = sl_ok[i] && ks < ks_end;
          if constexpr (BITS == 4) {
            b.ss[u][i] = load_b64(rs, oks ? sl_base[i] + (uint32_t)ks * 8u : kOobOffset);
          } else {
            b.ss[u][i][0] = load_b16(rs, oks ? sl_base[i] + ((uint32_t)ks >> 1) * 2u : kOobOffset);
          }
        }
      } else {
#pragma unroll
        for (int r = 0; r < R; ++r) {
          b.w[u][r] = load_b128(rw, wbase[r] + winc);  // valid base < 2^31: the sum cannot wrap
          b.sc[u][r] = load_b16(rs, sbase[r] + sinc);
        }
      }
      if constexpr (XST) {
        // line by line: instruction t reads ROWB bytes of RPI rows; a k-step past the end reads zeros
        const uint32_t kinc = (uint32_t)ks * ROWB;
#pragma unroll
        for (int t = 0; t < XI; ++t)
          b.xa[u][t / NJ][t % NJ] = load_b128(rx, (ks < ks_end && xl_base[t] != kOobOffset) ? xl_base[t] + kinc : kOobOffset);
      } else {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          const uint32_t xo = (ok && xrow_ok[mt]) ? xbase[mt] + xinc : kOobOffset;
#pragma unroll
          for (int j = 0; j < NJ; ++j) b.xa[u][mt][j] = load_b128(rx, xo + j * 16u);
        }
      }
    }
  };

  auto compute_batch = [&](const SkinnyBatch<BITS, R, MT, U>& b) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      half8_t a[MT][NJ];
      if constexpr (XST) {
#pragma unroll
        for (int t = 0; t < XI; ++t)
          *reinterpret_cast<u32x4*>(xst + t * 1024 + lane * 16) = b.xa[u][t / NJ][t % NJ];
      }
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
          u32x4 v;
          if constexpr (XST) v = *reinterpret_cast<const u32x4*>(xst + xs_rd[mt][j]);
          else v = b.xa[u][mt][j];
          if constexpr (BITS == 4) {
            // activations follow the weight pair order (k0,k4)(k1,k5)(k2,k6)(k3,k7)
            u32x4 p;
            p[0] = __builtin_amdgcn_perm(v[2], v[0], 0x05040100u);
            p[1] = __builtin_amdgcn_perm(v[2], v[0], 0x07060302u);
            p[2] = __builtin_amdgcn_perm(v[3], v[1], 0x05040100u);
            p[3] = __builtin_amdgcn_perm(v[3], v[1], 0x07060302u);
            a[mt][j] = __builtin_bit_cast(half8_t, p);
          } else {
            a[mt][j] = __builtin_bit_cast(half8_t, v);
          }
        }
      if constexpr (WST) {
#pragma unroll
        for (int t = 0; t < R; ++t) *reinterpret_cast<u32x4*>(wst + t * 1024 + lane * 16) = b.w[u][t];
#pragma unroll
        for (int i = 0; i < NSI; ++i) {
          // every lane stores, also those past the workgroup's rows (the area holds 64 entries per instruction):
          // behind a store under a condition the compiler may reuse the previous k-step's read for the lanes
          // that do not store -- it does not know that other lanes' stores feed them
          if constexpr (BITS == 4) *reinterpret_cast<u32x2*>(sst + (i * 64 + lane) * 8) = b.ss[u][i];
          else *reinterpret_cast<uint16_t*>(sst + (i * 64 + lane) * 2) = (uint16_t)b.ss[u][i][0];
        }
      }
#pragma unroll
      for (int r = 0; r < R; ++r) {
        uint16_t sbits;
        if constexpr (WST) sbits = *reinterpret_cast<const uint16_t*>(sst + r * (BITS == 4 ? 128 : 32) + ss_rd);
        else sbits = (uint16_t)b.sc[u][r];
        const half2_t s2 = bcast_h2(__builtin_bit_cast(half_t, sbits));
        u32x4 wv;
        if constexpr (WST) wv = *reinterpret_cast<const u32x4*>(wst + r * 1024 + ws_rd);
        else wv = b.w[u][r];
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
          half8_t bm;
          if constexpr (BITS == 4) {
            half2_t h[4];
            q4_word_paired(wv[j], s2, qc, h);
            bm = pack_h8(h[0], h[1], h[2], h[3]);
          } else {
            half2_t h0[2], h1[2];
            q8_word_natural(wv[2 * j], s2, h0);
            q8_word_natural(wv[2 * j + 1], s2, h1);
            bm = pack_h8(h0[0], h0[1], h1[0], h1[1]);
          }
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            acc[r][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[mt][j], bm, acc[r][mt], 0, 0, 0);
        }
      }
    }
  };

  // register double buffering: the next batch is in flight while this one is consumed
  SkinnyBatch<BITS, R, MT, U> b0, b1;
  load_batch(b0, ks_begin);
  for (int ks = ks_begin; ks < ks_end; ks += 2 * U) {
    load_batch(b1, ks + U);
    __builtin_amdgcn_sched_barrier(0);
    compute_batch(b0);
    __builtin_amdgcn_sched_barrier(0);
    load_batch(b0, ks + 2 * U);
    __builtin_amdgcn_sched_barrier(0);
    compute_batch(b1);
    __builtin_amdgcn_sched_barrier(0);
  }

  // cross-wave reduction of the K split
  if constexpr (XST) __syncthreads();  // (the staging areas are about to become the reduction buffer)
  float (*red)[R * MT][4][64] = reinterpret_cast<float (*)[R * MT][4][64]>(smem);
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[wave][r * MT + mt][i][lane] = acc[r][mt][i];
  __syncthreads();
  for (int idx = threadIdx.x; idx < R * MT * 256; idx += WAVES * 64) {
    const int t = idx >> 8, i = (idx >> 6) & 3, l = idx & 63;
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) sum += red[w][t][i][l];
    const int r = t / MT, mt = t % MT;
    const int m = m0 + mt * 16 + 4 * (l >> 4) + i;
    const int n = (blockIdx.x * R + r) * 16 + (l & 15);
    if (m < M && n < N) store_out(ep, y, m, n, N, sum);
  }
}

namespace {

// Rows per grid slice: up to 64 rows one slice; above, equal slices of whole 16-row blocks (80 rows: 2 x 48).
int skinny_slice_rows(int64_t m) {
  const int64_t slices = (m + 63) / 64;
  return (int)(((m + slices - 1) / slices + 15) / 16 * 16);
}

template <int BITS, int R, int MT, int WAVES, int U, bool TILED = false, bool XST = false>
void launch_one(const Problem& p, int group_shift) {
  const int tiles = (int)((p.n + 15) / 16);
  const int slice_rows = skinny_slice_rows(p.m);
  dim3 grid((tiles + R - 1) / R, (unsigned)((p.m + slice_rows - 1) / slice_rows)), block(WAVES * 64);
  hipLaunchKernelGGL((wq_skinny_kernel<BITS, R, MT, WAVES, U, TILED, XST>), grid, block, 0, p.stream,
                     (const half_t*)p.x, (const uint32_t*)p.wq, (const half_t*)p.scales,
                     (half_t*)p.y, (int)p.m, (int)p.n, (int)p.k, group_shift, p.zero_point,
                     Epilogue{(const half_t*)p.bias, (const half_t*)p.residual, p.activation}, slice_rows);
}

template <int BITS, int MT>
bool dispatch_variant(const Problem& p, int group_shift, int variant) {
  // the staged builds on canonical weights load a k-step's scales by row: standard quantizations, whole k-steps;
  // anything else runs the direct form of the same shape
  if (variant > 20 && !p.tiled && (group_shift != (BITS == 4 ? 0 : 3) || (BITS == 4 && p.k % 128 != 0))) variant -= 20;
  // (so does int4 at four row blocks with eight wavefronts on four tiles: its staging areas exceed the LDS)
  if (variant == 28 && !p.tiled && BITS == 4 && MT == 4) variant = 8;
  if (variant > 20) {  // staged activations (two row blocks and more), both layouts
    if (p.tiled) {
      switch (variant - 20) {
        case 1: launch_one<BITS, 1, MT, 4, 2, true, true>(p, group_shift); return true;
        case 2: launch_one<BITS, 2, MT, 4, 2, true, true>(p, group_shift); return true;
        case 5: launch_one<BITS, 2, MT, 8, 1, true, true>(p, group_shift); return true;
        case 7: launch_one<BITS, 4, MT, 4, 1, true, true>(p, group_shift); return true;
        case 8: launch_one<BITS, 4, MT, 8, 1, true, true>(p, group_shift); return true;
        case 6: launch_one<BITS, 1, MT, 8, 1, true, true>(p, group_shift); return true;
        case 11: launch_one<BITS, 8, MT, 4, 1, true, true>(p, group_shift); return true;
        default: return false;
      }
    }
    switch (variant - 20) {
      case 1: launch_one<BITS, 1, MT, 4, 2, false, true>(p, group_shift); return true;
      case 2: launch_one<BITS, 2, MT, 4, 2, false, true>(p, group_shift); return true;
      case 5: launch_one<BITS, 2, MT, 8, 1, false, true>(p, group_shift); return true;
      case 7: launch_one<BITS, 4, MT, 4, 1, false, true>(p, group_shift); return true;
      case 8:
        // (int4 at four row blocks: the staging areas of eight wavefronts would not fit the LDS)
        if constexpr (BITS == 8 || MT <= 3) {
          launch_one<BITS, 4, MT, 8, 1, false, true>(p, group_shift);
          return true;
        }
        return false;
      case 6: launch_one<BITS, 1, MT, 8, 1, false, true>(p, group_shift); return true;
      case 11: launch_one<BITS, 8, MT, 4, 1, false, true>(p, group_shift); return true;
      default: return false;
    }
  }
  if (p.tiled) {  // the variants the default choice uses, reading the tile-major layout
    switch (variant) {
      case 1: launch_one<BITS, 1, MT, 4, 2, true>(p, group_shift); return true;
      case 2: launch_one<BITS, 2, MT, 4, 2, true>(p, group_shift); return true;
      case 5: launch_one<BITS, 2, MT, 8, 1, true>(p, group_shift); return true;
      case 7: launch_one<BITS, 4, MT, 4, 1, true>(p, group_shift); return true;
      case 9: launch_one<BITS, 4, MT, 2, 1, true>(p, group_shift); return true;
      case 11: launch_one<BITS, 8, MT, 4, 1, true>(p, group_shift); return true;
      default: return false;
    }
  }
  switch (variant) {
    case 1: launch_one<BITS, 1, MT, 4, 2>(p, group_shift); return true;
    case 2: launch_one<BITS, 2, MT, 4, 2>(p, group_shift); return true;
    case 3: launch_one<BITS, 1, MT, 8, 2>(p, group_shift); return true;
    case 4: launch_one<BITS, 1, MT, 4, 4>(p, group_shift); return true;
    case 5: launch_one<BITS, 2, MT, 8, 1>(p, group_shift); return true;
    case 6: launch_one<BITS, 1, MT, 8, 1>(p, group_shift); return true;
    case 7: launch_one<BITS, 4, MT, 4, 1>(p, group_shift); return true;
    case 8: launch_one<BITS, 4, MT, 8, 1>(p, group_shift); return true;
    case 9: launch_one<BITS, 4, MT, 2, 1>(p, group_shift); return true;
    case 10: launch_one<BITS, 2, MT, 2, 2>(p, group_shift); return true;
    case 11: launch_one<BITS, 8, MT, 4, 1>(p, group_shift); return true;
    default: return false;
  }
}

}  // namespace

int launch_skinny(const Problem& p, int variant) {
  const int ch = 128 / p.bits;
  int ratio = p.group / ch, group_shift = 0;
  while ((1 << group_shift) < ratio) ++group_shift;
  if (ratio < 1 || (1 << group_shift) != ratio || p.group % ch != 0) {
    set_error("skinny kernel: group %d must be %d times a power of two", p.group, ch);
    return -1;
  }
  if (p.m > kSkinnyMaxM) {
    set_error("skinny kernel: M = %lld exceeds %lld", (long long)p.m, (long long)kSkinnyMaxM);
    return -1;
  }
  const int mt = (int)((std::min<int64_t>(p.m, skinny_slice_rows(p.m)) + 15) / 16);
  if (variant == 0) {
    // Measured on MI355X (q4f16, Llama-2-7B shapes, M = 4 .. 64): the number of workgroups is what
    // matters: as few tiles per workgroup as still give every CU at most one workgroup.
    // At most one row tile per CU: one tile per 4-wave workgroup; up to two per CU: two
    // tiles per workgroup, eight wavefronts for int4 and four for int8 (a second, mostly empty
    // round of workgroups costs more: 5120 x 13824 at 64 rows 114 -> 67 us); more: four
    // tiles per workgroup; many: two tiles per 8-wave workgroup for one row block, else four.
    // (above 64 rows the grid has two to four slices of rows: what counts is tiles x slices -- 4096 x 4096 at 96 rows:
    // two tiles per eight-wavefront workgroup 12.5 us, one tile 19.4)
    const int64_t slices = (p.m + skinny_slice_rows(p.m) - 1) / skinny_slice_rows(p.m);
    const int64_t tiles = (p.n + 15) / 16 * slices;
    // From 17 rows on the activations are staged through LDS (variants 21 ...: the same shapes with
    // line-by-line activation loads): 10 - 30 % faster from 32 rows on (4096 x 11008 at 64 rows 46 -> 35 us,
    // int8 5120 x 13824 at 64 rows 72 -> 53 us), level at 17.  With staged loads more wavefronts per
    // workgroup pay: eight on one int4 tile (4096 x 4096 at 32 rows 8.9 -> 8.0 us, 4096 x 11008 at 64 rows
    // 36.7 -> 30.4), eight on four tiles with 513 - 1024 tiles (12288 x 4096 at 48 rows 21.8 -> 20.6; not at
    // four row blocks of int4, whose staging areas fill the LDS; there tile-major weights keep the direct loads).
    // One row block (up to 16 rows, where the decode kernel does not apply): the staged loads pay on the two
    // ends -- at most one tile per CU from 9 rows on and for int8 (2048 x 2048 int8: 4.7 - 5.9 -> 4.2 - 4.6 us),
    // and with several rounds of workgroups (a 152064 x 4096 vocabulary projection: 108 - 153 -> 91 - 102 us,
    // tile-major 75 - 106 -> 70 - 76).
    const bool staged = mt >= 2;
    if (tiles <= 256) variant = staged ? (p.bits == 4 ? 26 : 21) : (p.bits == 8 || p.m >= 9) ? 26 : 1;
    // (one tile per workgroup is 1.5 - 1.8x slower here; int8 at up to 4 rows on tile-major weights:
    // eight wavefronts, 3 - 5 % ahead)
    else if (tiles <= 512) variant = (staged || p.m >= 9) ? 25 : ((p.bits == 4 || (p.tiled && p.m <= 4)) ? 5 : 2);
    else if (tiles <= 1024) {
      if (!staged) variant = 7;
      else if (p.bits == 8 || mt <= 3) variant = 28;
      else variant = p.tiled ? 7 : 27;  // (the same wavefront split on both layouts: their results are bit-equal)
    }
    // several rounds of workgroups: eight tiles share one pass over the activations; staged from 17 rows
    // on for int8 (27648 x 5120 tile-major at 32 rows 43.4 -> 38.5 us) and for canonical int4 up to 48 rows
    else if (!staged) variant = 27;
    else if (p.bits == 8) variant = slices > 1 ? 27 : 31;  // (10240 x 5120 at 96 rows: 36 against 44 us)
    else variant = (!p.tiled && mt <= 3) ? 27 : 11;
  }
  bool ok;
  if (p.bits == 4) {
    ok = mt <= 1   ? dispatch_variant<4, 1>(p, group_shift, variant)
         : mt == 2 ? dispatch_variant<4, 2>(p, group_shift, variant)
         : mt == 3 ? dispatch_variant<4, 3>(p, group_shift, variant)
                   : dispatch_variant<4, 4>(p, group_shift, variant);
  } else {
    ok = mt <= 1   ? dispatch_variant<8, 1>(p, group_shift, variant)
         : mt == 2 ? dispatch_variant<8, 2>(p, group_shift, variant)
         : mt == 3 ? dispatch_variant<8, 3>(p, group_shift, variant)
                   : dispatch_variant<8, 4>(p, group_shift, variant);
  }
  if (!ok) {
    set_error("skinny kernel: unknown variant %d", variant);
    return -1;
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("skinny kernel launch failed: %s", hipGetErrorString(e));
    return -1;
  }
  return 0;
}

}  // namespace wq
