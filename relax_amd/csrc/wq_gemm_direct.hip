// MFMA GEMM for prefill (M > 64) whose weight operand never touches LDS:
// y[M,N] = x[M,K] @ dequant(Wq,S)^T.
//
// Bound: dense float16 MFMA; the design goal is to keep LDS traffic well below the matrix
// pipe's appetite.  A workgroup owns a BM x 256 output tile (BM = 128, or 64 when M is too
// small to give every CU a 128-row tile); all wavefronts share the same BM activation rows
// (staged in LDS) and each owns 64 distinct weight rows, i.e. a BM x 64 sub-tile of 32x32x16
// MFMAs.  The two 32-column MFMA tiles of a wavefront hold the even and the odd columns of
// its 64 (lane col: columns 2 col and 2 col + 1), so a lane finishes with two adjacent outputs
// of a row and stores them with one 4-byte access.  The
// MFMA B operand of lane (col = lane % 32, kh = lane / 32) for 16-wide k slice kk is
// the 8 weights k = k0 + (kh*4 + kk)*8 .. +8 of its row -- exactly one packed int4
// word, or two int8 words -- so a lane loads the 16 bytes (int4) it needs for a whole
// 64-wide K step straight from global memory with one buffer load, together with the
// one group scale that covers them, and dequantizes word by word in registers, to
// exactly the float16 values the CPU path materialises.  No wavefront dequantizes a
// weight twice, and LDS carries only the activations: BM*128 B written and
// WAVES*BM*128 B read per K step.
//
// The A operand follows the same k assignment: lane (row, kh) reads chunk kh*4 + kk
// of its activation row.  LDS rows are 128 bytes, their eight 16-byte chunks
// XOR-swizzled with ((row >> 1) & 7).  The LDS of this part has 64 banks (256 bytes per
// cycle): a 16-byte access is served 16 lanes at a time, and 16 consecutive rows reading the
// same chunk then cover every bank once (two rows of opposite parity share a swizzle term and
// split the 256 bytes between them); with (row & 7) rows r and r + 8 collide and the counters
// show 38 % of the LDS cycles lost to bank conflicts.  Row-contiguous writes are conflict-free.
//
// Pipeline per K step t (four activation stages in LDS; program order is issue order, a
// handful of independent instructions after every MFMA, fenced with sched_barrier):
//   global -> registers : activations of step t+4 (t+3 with one register set), packed weights
//                         of step t+3 (t+2 with two register sets), scales per four steps
//   registers -> LDS    : activations of step t+2
//   LDS -> registers    : A fragments of the next k slice (of step t+1 at the end)
//   dequantize          : one stage each of four pair conversions per MFMA slot
//
// K groups (GROUPS = 2): eight wavefronts, two per SIMD.  Wavefronts 0-3 accumulate the
// first half of K and wavefronts 4-7 the second half of the same 128 x 256 tile, each group
// with its own activation stages; at the end the second group hands its partial sums to the
// first through LDS.  A stall of one wavefront (barrier, memory wait) is covered by the
// other one on its SIMD, and a tile takes half as many sequential K steps, which is what
// counts when M is too small to give every CU a tile.
//
// With two wavefronts on a SIMD the one further back in its step gets the higher priority
// (s_setprio per k slice), so that both reach the step's barrier together.
//
// TILED: the packed weights and scales are in the tile-major layout (wq_tiled.hip); only the
// address arithmetic of the weight and scale loads changes -- 16 lanes then read 256
// contiguous bytes instead of 16 rows' worth of 16-byte pieces.
//
// Shape requirements (checked by the launcher): K a multiple of 256 (at least 512 for K
// groups), group 32 (int4) or 128 (int8), operands < 1 GiB; other shapes use the other GEMM
// kernels.
#include <atomic>
#include <algorithm>
#include <type_traits>

#include "wq_device.h"
#include "wq_internal.h"

namespace wq {

namespace {
constexpr int64_t kGemmSplitMaxTiles = 4096;                      // arrival counters at the head of a workspace
constexpr int64_t kGemmSplitCounterBytes = kGemmSplitMaxTiles * 4;  // (the decode kernel's split uses the same head)
constexpr uint32_t kRowOobD = 0x80000000u;   // offset of a row that must read zeros
constexpr uint32_t kStepOobD = 0x40000000u;  // added for a K step past K: beyond any buffer < 1 GiB

template <int B, int E, class F>
__device__ __forceinline__ void static_for_d(F&& f) {
  if constexpr (B < E) {
    f(std::integral_constant<int, B>{});
    static_for_d<B + 1, E>(f);
  }
}
}  // namespace

template <int BITS>
struct RawB {
  static constexpr int NV = BITS == 4 ? 1 : 2;  // 16-byte loads per 32 k of one row
  u32x4 w[2][NV];                               // [column tile][load]
};

template <int BITS, int GROUPS, int TM, int WAVES, bool TILED, bool KSPLIT = false, bool HOP = false>
__global__ __launch_bounds__(GROUPS * WAVES * 64, 1) void wq_gemm_direct_kernel(
    const half_t* __restrict__ x, const uint32_t* __restrict__ wq, const half_t* __restrict__ scales,
    int M, int N, int K, int shift_and_zero, int tiles_m, int tiles_n, int tile_n0, half_t* y,
    const Epilogue ep, int ksplit, float* partials, unsigned int* counters) {
  // (argument order: the first 14 dwords are preloaded into SGPRs at wavefront launch, later ones are
  // a scalar load at the start of the kernel; what the K loop needs comes first, y and the epilogue last)
  const int group_shift = shift_and_zero & 0xFF, zero_point = (shift_and_zero >> 8) & 0xFF;
  const bool gated = (shift_and_zero >> 16) & 1;  // fused multiply(nn.silu(gate), up): rows walked interleaved
  constexpr int BK = 64;
  static_assert(TM == 4 || TM == 2, "row blocks of 32 per wavefront: 128- or 64-row tile");
  static_assert(WAVES == 4 || WAVES == 2, "wavefronts per K group: 256 or 128 output columns");
  static_assert(GROUPS == 1 || GROUPS == 2 || GROUPS == 4, "K groups");
  static_assert(!HOP || (BITS == 8 && !TILED && TM == 2), "the line-wise weight loads are built for int8, canonical layout, 64-row tiles");
  constexpr int BM = TM * 32;
  constexpr int NT = WAVES * 64;   // threads of one K group
  constexpr int CH = 128 / BITS;   // k per 16-byte packed chunk
  constexpr int NV = RawB<BITS>::NV;
  constexpr int XL = BM * 8 / NT;  // 16-byte activation chunks per thread per step
  constexpr int STAGE = BM * 128;  // bytes per LDS stage
  // register sets: two wavefronts per SIMD leave 128 VGPRs beside the accumulators and hide
  // latency by themselves, so the K-group variants prefetch only one step deep (deeper rings
  // were measured with the 64-row tile, where registers would allow them: no gain)
  constexpr int RB = (TM == 2 || (BITS == 4 && GROUPS == 1)) ? 4 : 2;  // packed weights
  constexpr int XS = (TM == 2 || GROUPS == 1) ? 2 : 1;  // activations (1, 2 or 4; four sets measured: no gain)
  static_assert(XL >= 1 && XL <= 2 * TM, "activation chunks per thread must fit the MFMA slots of one k slice");

  extern __shared__ __attribute__((aligned(16))) unsigned char wq_gemm_direct_smem[];

  // XCD-aware tile order.  Consecutive workgroup ids land on different XCDs; regroup them so
  // that each XCD owns a contiguous range of the tile list, and order the list in column
  // panels of eight tiles, row-major inside a panel: the 32 workgroups an XCD runs at a time
  // then cover 4 activation row blocks x 8 weight column tiles and walk K together, so its L2
  // serves every activation block eight times and every weight tile four times per fetch.
  // K split across workgroups (caller workspace): S consecutive workgroup ids share a tile, each on its
  // own window of K; S = 1 otherwise.
  const int S = KSPLIT ? ksplit : 1;  // (a build of its own: the plain kernel keeps its registers)
  const int nblocks = tiles_m * tiles_n;
  int bid = blockIdx.x;
  const int ks = S > 1 ? bid % S : 0;
  if (S > 1) bid /= S;
  const int tile_lin = bid;  // the tile's slot in the workspace
  if (S == 1 && (nblocks & 7) == 0) bid = (bid & 7) * (nblocks >> 3) + (bid >> 3);
  constexpr int PANEL = 8;
  const int full = tiles_n / PANEL;                 // panels of full width
  const int in_full = bid / (tiles_m * PANEL);      // panel index if inside the full ones
  const int panel = min(in_full, full);
  const int width = panel < full ? PANEL : tiles_n - full * PANEL;
  const int rest = bid - panel * tiles_m * PANEL;
  // (tile_n0: first column tile of this launch, when a matrix is covered by two launches)
  const int tile_m = rest / width, tile_n = tile_n0 + panel * PANEL + rest % width;
  const int m0 = tile_m * BM, n0 = tile_n * (WAVES * 64);

  const int lane = threadIdx.x & 63;
  const int wave_id = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int grp = GROUPS == 1 ? 0 : wave_id / WAVES;  // K group of this wavefront
  const int wave = wave_id % WAVES;                   // 64-column slice of the tile
  const int tid = threadIdx.x & (NT - 1);          // thread index inside the K group
  const int fr = lane & 31, fh = lane >> 5;
  unsigned char* const lds = wq_gemm_direct_smem + grp * (4 * STAGE);  // the group's four stages

  // K range of this group, in 64-wide steps; both groups run the same number of steps and
  // the shorter one reads zeros (out-of-range offsets) past its end.
  // (with a K split the same inside this workgroup's window of whole 256-wide macro steps)
  const int ksteps = K / BK;
  const int macro_per = (ksteps / 4 + S - 1) / S;
  const int win_begin = min(ks * macro_per * 4, ksteps), win_end = min((ks + 1) * macro_per * 4, ksteps);
  const int wsteps = win_end - win_begin;
  const int nloop = GROUPS == 1 ? wsteps : 4 * ((wsteps / 4 + GROUPS - 1) / GROUPS);
  const int kbase = win_begin + grp * nloop;
  const int kend = min(kbase + nloop, win_end);

  const uint32_t row_bytes = (uint32_t)K * BITS / 8;
  const uint32_t groups_per_row = ((uint32_t)K / CH) >> group_shift;
  // (tile-major buffers hold whole 16-row tiles, zero filled past N)
  const uint32_t n_stored = TILED ? ((uint32_t)N + 15u) / 16u * 16u : (uint32_t)N;
  const uint32_t nsuper = row_bytes / 128u;  // 128-byte super steps per weight row (tile-major addressing)
  const rsrc_t rw = make_rsrc(wq, n_stored * row_bytes);
  const rsrc_t rs = make_rsrc(scales, n_stored * groups_per_row * 2u);
  const rsrc_t rx = make_rsrc(x, (uint32_t)M * (uint32_t)K * 2u);

  // ---- activations: global offsets and LDS store address of this thread ---------------
  uint32_t xg[XL];
  const int x_row0 = tid >> 3, x_c = tid & 7;
#pragma unroll
  for (int i = 0; i < XL; ++i) {
    const int m = m0 + x_row0 + i * (NT / 8);
    xg[i] = m < M ? (uint32_t)m * (uint32_t)K * 2u + (uint32_t)x_c * 16u : kRowOobD;
  }
  const uint32_t x_lds = (uint32_t)x_row0 * 128u + (uint32_t)((x_c ^ ((x_row0 >> 1) & 7)) << 4);

  // ---- weights: this lane's two rows (column tiles j = 0, 1) --------------------------
  uint32_t wg[2], sg[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    // column tile j of the MFMA holds the tile's columns of parity j (lane fr: column 2 fr + j), so
    // that a lane ends up with two adjacent outputs of a row and a wavefront stores whole 128-byte lines
    int n = min(n0 + wave * 64 + 2 * fr + j, (int)n_stored - 1);  // rows past N: computed, not stored
    if (gated) n = gated_physical_row(n, N);  // column parity j: gate row / up row of output (n0 + wave*64)/2 + fr
    if constexpr (TILED) {
      // chunk c of row n sits at ((tile*S + c/8)*2 + c%2)*1024 + ((c%8)/2*16 + n%16)*16; the lane's chunks
      // of step kt are 2 kt + fh (int4) or 4 kt + 2 fh + v (int8), which leaves these lane constants
      const uint32_t tile = (uint32_t)n >> 4, col = (uint32_t)n & 15u;
      wg[j] = tile * nsuper * 2048u + (uint32_t)fh * (BITS == 4 ? 1024u : 256u) + col * 16u;
      sg[j] = BITS == 4 ? (tile * nsuper * 64u + col) * 4u : (tile * nsuper * 16u + col) * 2u;
    } else {
      wg[j] = (uint32_t)n * row_bytes + (uint32_t)fh * (32u * BITS / 8);
      sg[j] = (uint32_t)n * groups_per_row * 2u;
    }
  }

  // ---- A fragment read addresses: row fr, chunk fh*4 + kk ------------------------------
  uint32_t a_rd[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk)
    a_rd[kk] = (uint32_t)fr * 128u + (uint32_t)(((fh * 4 + kk) ^ ((fr >> 1) & 7)) << 4);

  // ---- HOP: packed weights by whole cache lines, through a wavefront-private LDS area -------------------
  // Loaded directly, lane (column, kh) reads 16 bytes of its own row: the 64 lanes of a request touch 32 rows,
  // i.e. 32 cache lines, for 32 bytes each, and -- a row of int8 weights being a multiple of 512 bytes -- all of
  // them in the same bank of the L1's tag memory: the lookups go one per clock where contiguous lines go four
  // (TCP_READ_TAGCONFLICT_STALL_CYCLES: 13 - 30 % of the kernel's time on the 5120-wide shapes).  Here a request
  // covers 8 rows x one whole 128-byte line (lane l: row l / 8, 16-byte chunk l % 8), a quarter of the lookups
  // for the same bytes: four requests bring the 32 rows of a column tile for two K steps, the wavefront stores them
  // into its own 4 KB of LDS (rows of 128 bytes, chunks XOR-swizzled like the activation rows: stores and loads
  // conflict-free) and every lane reads back the four chunks of its row in the order the direct loads deliver.
  // The hardware executes a wavefront's LDS instructions in order; the fences state the order for the compiler.
  // (int4 was built the same way -- a line is four K steps there, the block stored twice -- and measured: bit-equal,
  // -6 ... +3.5 % on the 4096- to 22016-row shapes at 128 to 512 rows; it has half the requests per k to begin with.)
  unsigned char* const hop = wq_gemm_direct_smem + GROUPS * 4 * STAGE + wave_id * 4096;
  uint32_t hg[2][4];   // global offset of this lane's chunk for request i4 of column tile j
  uint32_t hop_wr[2];  // LDS store offset for even / odd i4 (+ i4 * 1024)
  uint32_t hop_rd[4];  // LDS load offsets: chunk (step parity) * 4 + kh * 2 + v of row fr
  u32x4 hb[2][4];      // a block (two K steps) of both column tiles on its way: global -> registers -> LDS
  if constexpr (HOP) {
    const int hr = lane >> 3, hc = lane & 7;
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        int n = min(n0 + wave * 64 + 2 * (8 * i4 + hr) + j, (int)n_stored - 1);
        if (gated) n = gated_physical_row(n, N);
        hg[j][i4] = (uint32_t)n * row_bytes + (uint32_t)hc * 16u;
      }
    // row 8 i4 + hr: swizzle term ((row >> 1) & 7) = (4 i4 + (hr >> 1)) & 7
#pragma unroll
    for (int odd = 0; odd < 2; ++odd)
      hop_wr[odd] = (uint32_t)hr * 128u + (uint32_t)((hc ^ (hr >> 1) ^ (odd * 4)) << 4);
#pragma unroll
    for (int c = 0; c < 4; ++c)
      hop_rd[c] = (uint32_t)fr * 128u + (uint32_t)(((((c >> 1) * 4) + fh * 2 + (c & 1)) ^ ((fr >> 1) & 7)) << 4);
  }
  // requests of column tile j's rows for the block that starts at (even) step kt
  auto hop_load = [&](u32x4 (&dst)[4], int j, int kt) {
    const uint32_t koff = kt < kend ? (uint32_t)kt * (BK * BITS / 8) : kStepOobD;
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) dst[i4] = load_b128(rw, hg[j][i4] + koff);
  };
  auto hop_store = [&](const u32x4 (&src)[4]) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");  // (behind the loads of the tile before)
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4)
      *reinterpret_cast<u32x4*>(hop + hop_wr[i4 & 1] + (uint32_t)i4 * 1024u) = src[i4];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  };
  // column tile j of the block in the LDS area -> the register sets of its two steps
  auto hop_fetch = [&](RawB<BITS>& b_even, RawB<BITS>& b_odd, int j) {
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    b_even.w[j][0] = *reinterpret_cast<const u32x4*>(hop + hop_rd[0]);
    b_even.w[j][NV - 1] = *reinterpret_cast<const u32x4*>(hop + hop_rd[1]);
    b_odd.w[j][0] = *reinterpret_cast<const u32x4*>(hop + hop_rd[2]);
    b_odd.w[j][NV - 1] = *reinterpret_cast<const u32x4*>(hop + hop_rd[3]);
  };

  const Q4Consts qc = make_q4_consts(zero_point);

  auto load_x = [&](u32x4 (&xr)[XL], int kt, auto ic) {
    constexpr int i = decltype(ic)::value;
    const uint32_t xk = kt < kend ? (uint32_t)kt * BK * 2u : kStepOobD;
    xr[i] = load_b128(rx, xg[i] + xk);
  };
  auto store_x = [&](const u32x4 (&xr)[XL], uint32_t stage_base, auto ic) {
    constexpr int i = decltype(ic)::value;
    *reinterpret_cast<u32x4*>(lds + stage_base + x_lds + (uint32_t)i * (NT / 8) * 128u) = xr[i];
  };
  // piece c of the packed-weight loads of step kt
  auto load_b = [&](RawB<BITS>& b, int kt, auto cc) {
    constexpr int c = decltype(cc)::value, j = c / NV, v = c % NV;
    if constexpr (TILED) {
      const uint32_t ukt = (uint32_t)kt;
      const uint32_t step = BITS == 4 ? (ukt >> 2) * 2048u + (ukt & 3u) * 256u : (ukt >> 1) * 2048u + (ukt & 1u) * 512u;
      b.w[j][v] = load_b128(rw, wg[j] + (kt < kend ? step : kStepOobD) + v * 1024u);
    } else {
      const uint32_t k0 = (uint32_t)kt * BK;
      b.w[j][v] = load_b128(rw, wg[j] + (kt < kend ? k0 * BITS / 8 : kStepOobD) + v * 16u);
    }
  };
  constexpr int PBL = 2 * NV;  // packed-weight load pieces per step

  // Group scales are fetched once per four K steps (256 k of a row): eight float16 for
  // int4 / group 32, two for int8 / group 128.  2-byte loads per step would touch 32 cache
  // lines per instruction for 128 useful bytes and dominate the L1 pipeline.
  constexpr int SW = BITS == 4 ? 4 : 1;  // 32-bit words of scales per row and macro step
  uint32_t sc_cur[2][SW], sc_nxt[2][SW];
  auto load_scales_of = [&](uint32_t (&sc)[2][SW], int kt0, auto jc) {
    // kt0: first step of the macro step (a multiple of 4); jc: column tile
    constexpr int j = decltype(jc)::value;
    if constexpr (TILED) {
      if constexpr (BITS == 4) {
        // the eight scales of (row, super step) are four 4-byte pairs, one per kq, 64 bytes apart
        const uint32_t base = kt0 < kend ? sg[j] + ((uint32_t)kt0 >> 2) * 256u : kStepOobD;
#pragma unroll
        for (int q = 0; q < 4; ++q) sc[j][q] = load_b32(rs, base + (uint32_t)q * 64u);
      } else {
        // one float16 per (row, super step); a macro step of 256 k spans two of them
        const uint32_t base = kt0 < kend ? sg[j] + ((uint32_t)kt0 >> 1) * 32u : kStepOobD;
        sc[j][0] = load_b16(rs, base) | (load_b16(rs, base + 32u) << 16);
      }
      return;
    }
    const uint32_t off = kt0 < kend ? sg[j] + (uint32_t)kt0 * BK / (BITS == 4 ? 32 : 128) * 2u : kStepOobD;
    if constexpr (BITS == 4) {
      const u32x4 v = load_b128(rs, off);
#pragma unroll
      for (int q = 0; q < 4; ++q) sc[j][q] = v[q];
    } else {
      sc[j][0] = load_b32(rs, off);
    }
  };
  // scale of (column tile j, step t of the macro step) in the low half of a register
  auto pick_scale = [&](const uint32_t (&sc)[2][SW], int j, int t) -> uint32_t {
    if constexpr (BITS == 4) return __builtin_amdgcn_alignbit(sc[j][t], sc[j][t], (uint32_t)fh * 16u);
    else return t < 2 ? sc[j][0] : sc[j][0] >> 16;
  };
  uint32_t s_step[2][2];  // [step parity][column tile]

  // The conversion of one pair of weights is a chain of four dependent VALU ops (byte
  // permute, and-or, fma, scale multiply; int8: convert low, convert high, scale multiply -- three).  The chain is software-pipelined over four
  // MFMA slots -- every slot advances four different pairs by one stage -- so no slot
  // contains dependent instructions.  Pair g (counted from the start of the K step)
  // belongs to B fragment g/4 = slice (g/8), column tile (g/4)%2, position g%4.
  auto stage_perm = [&](const RawB<BITS>& b, auto gc) -> uint32_t {
    constexpr int g = decltype(gc)::value, kk = (g / 8) & 3, j = (g / 4) & 1, pp = g & 3;
    if constexpr (BITS == 4) {
      return __builtin_amdgcn_perm(0u, b.w[j][0][kk], 0x0c000c00u | (uint32_t)pp | ((uint32_t)pp << 16));
    } else {
      // int8: the first weight of the pair, converted into the low half (upper half zero)
      return cvt_i8_lo<(pp & 1) * 2>(b.w[j][kk >> 1][(kk & 1) * 2 + (pp >> 1)]);
    }
  };
  // (int8: the second weight of pair g of `b`, converted into the high half of v -- the chain reads the
  // packed word in two consecutive slots, so a register set is reloaded no earlier than the slot after
  // its last pair entered, and a slot converts before it loads)
  auto stage_bits = [&](uint32_t v, const RawB<BITS>& b, auto gc) -> uint32_t {
    constexpr int g = decltype(gc)::value, kk = (g / 8) & 3, j = (g / 4) & 1, pp = g & 3;
    if constexpr (BITS == 4) return and_or(v, 0x00F0000Fu, qc.magic);
    else return cvt_i8_hi<(pp & 1) * 2 + 1>(v, b.w[j][kk >> 1][(kk & 1) * 2 + (pp >> 1)]);
  };
  auto stage_center = [&](uint32_t v) -> half2_t {
    if constexpr (BITS == 4) return __builtin_elementwise_fma(as_h2(v), qc.mix_mul, -qc.mix_sub);
    else return as_h2(v);  // the conversion is complete: this stage is empty for int8
  };
  auto stage_scale = [&](int parity, half2_t v, auto gc) -> uint32_t {
    constexpr int g = decltype(gc)::value, j = (g / 4) & 1;
    return as_u32(v * bcast_h2(__builtin_bit_cast(half_t, (uint16_t)s_step[parity][j])));
  };

  // A B fragment (four pairs) feeds TM MFMAs, so PPS = 4 / TM pairs enter and leave the
  // conversion pipeline per MFMA slot; a pair leaves LEAD slots before its fragment's first use.
  constexpr int PPS = 4 / TM;
  constexpr int LEAD = TM == 4 ? 5 : 3;
  half8_t fa[2][TM];
  u32x4 fbq[4];  // ring of B fragments (fragment q of a step lives in fbq[q % 4])
  uint32_t t_perm[PPS], t_bits[PPS];  // pipeline registers of the pair conversion
  half2_t t_center[PPS];
  auto read_a = [&](int buf, uint32_t base, auto ic) {
    constexpr int i = decltype(ic)::value;
    fa[buf][i] = *reinterpret_cast<const half8_t*>(lds + base + (uint32_t)i * 4096u);
  };

  float16_t acc[TM][2];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  // ---- prologue ---------------------------------------------------------------------------
  // activations of step T: global -> register set T%XS late in step T-2-XS (one set: in step
  // T-3), registers -> LDS stage T%4 early in step T-2, multiplied in step T;  packed weights
  // of step T: loaded into set T%RB three steps ahead (four sets), or late in step T-2 (two
  // sets).  Step numbers are relative to the K group's first step.
  u32x4 xr[XS][XL];
  RawB<BITS> rb[RB];
  // Every request of the prologue goes out before the first wait (one memory round trip, not one
  // per dependent step).  First what is consumed before the loop: weights and scales of step 0,
  // activations of steps 0 and 1 (in registers of their own: the loop's sets already receive the
  // steps after them).
  u32x4 xp[2][XL];
  if constexpr (HOP) {
    // the first block (steps 0, 1) into the hop registers; the second (steps 2, 3), which the loop's first step
    // moves through the LDS area, into the register sets of steps 2 and 3 for now
    static_for_d<0, 2>([&](auto jc) { hop_load(hb[decltype(jc)::value], decltype(jc)::value, kbase); });
  } else {
    static_for_d<0, PBL>([&](auto cc) { load_b(rb[0], kbase, cc); });
  }
  static_for_d<0, 2>([&](auto jc) { load_scales_of(sc_cur, kbase, jc); });
  static_for_d<0, 2>([&](auto tc) {
    constexpr int T = decltype(tc)::value;
    static_for_d<0, XL>([&](auto ic) { load_x(xp[T], kbase + T, ic); });
  });
  // Then what is still in flight at loop entry, requested in the order the loop itself requests
  // it before its back edge: the wait counts the compiler derives for the loop head are then the
  // steady-state ones instead of a full drain of the memory pipeline every fourth step.
  u32x4 hnext[2][4];  // (HOP: the second block until the hop registers are free)
  if constexpr (HOP) {
    static_assert(RB == 4, "the line-wise loads fill the register sets of two steps at a time");
    static_for_d<2, 2 + XS>([&](auto tc) {
      constexpr int T = decltype(tc)::value;
      static_for_d<0, XL>([&](auto ic) { load_x(xr[T % XS], kbase + T, ic); });
    });
    static_for_d<0, 2>([&](auto jc) { hop_load(hnext[decltype(jc)::value], decltype(jc)::value, kbase + 2); });
  } else if constexpr (RB == 4) {
    static_for_d<0, PBL>([&](auto cc) { load_b(rb[1], kbase + 1, cc); });
    static_for_d<0, XL>([&](auto ic) { load_x(xr[2 % XS], kbase + 2, ic); });
    static_for_d<0, PBL>([&](auto cc) { load_b(rb[2], kbase + 2, cc); });
    static_for_d<3, 2 + XS>([&](auto tc) {
      constexpr int T = decltype(tc)::value;
      static_for_d<0, XL>([&](auto ic) { load_x(xr[T % XS], kbase + T, ic); });
    });
  } else {
    static_for_d<2, 2 + XS>([&](auto tc) {
      constexpr int T = decltype(tc)::value;
      static_for_d<0, XL>([&](auto ic) { load_x(xr[T % XS], kbase + T, ic); });
    });
    static_for_d<0, PBL>([&](auto cc) { load_b(rb[1], kbase + 1, cc); });
  }
  __builtin_amdgcn_sched_barrier(0);
  static_for_d<0, 2>([&](auto tc) {
    constexpr int T = decltype(tc)::value;
    static_for_d<0, XL>([&](auto ic) { store_x(xp[T], (uint32_t)(T * STAGE), ic); });
  });
  if constexpr (HOP) {
    // block 0 through the LDS area into the sets of steps 0 and 1; then the hop registers take the second block
    static_for_d<0, 2>([&](auto jc) {
      constexpr int j = decltype(jc)::value;
      hop_store(hb[j]);
      hop_fetch(rb[0], rb[1], j);
    });
  }
  __syncthreads();
  if constexpr (HOP) {
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) hb[j][i4] = hnext[j][i4];
  }
  static_for_d<0, TM>([&](auto ic) { read_a(0, a_rd[0], ic); });
#pragma unroll
  for (int j = 0; j < 2; ++j) s_step[0][j] = pick_scale(sc_cur, j, 0);
  // prime the conversion pipeline: the first PPS * LEAD pairs complete, then PPS pairs each
  // three, two and one stage in
  static_for_d<0, PPS * LEAD>([&](auto gc) {
    constexpr int g = decltype(gc)::value;
    fbq[g / 4][g & 3] = stage_scale(0, stage_center(stage_bits(stage_perm(rb[0], gc), rb[0], gc)), gc);
  });
  static_for_d<0, PPS>([&](auto pc) {
    constexpr int pp = decltype(pc)::value;
    constexpr std::integral_constant<int, PPS * LEAD + pp> g1{};
    constexpr std::integral_constant<int, PPS * (LEAD + 1) + pp> g2{};
    t_center[pp] = stage_center(stage_bits(stage_perm(rb[0], g1), rb[0], g1));
    t_bits[pp] = stage_bits(stage_perm(rb[0], g2), rb[0], g2);
    t_perm[pp] = stage_perm(rb[0], std::integral_constant<int, PPS * (LEAD + 2) + pp>{});
  });

  // One K step, P = (step number in the group) % 4 fixes every register set and LDS stage at
  // compile time.
  constexpr int NMFMA = TM * 2 * 4;
  auto step = [&](auto pc, int kt) {
    constexpr int P = decltype(pc)::value;
    RawB<BITS>& bcur = rb[P % RB];
    RawB<BITS>& bnxt = rb[(P + 1) % RB];
    RawB<BITS>& bload = rb[(P + RB - 1) % RB];   // receives step kt + RB - 1
    constexpr uint32_t st_rd = (uint32_t)(P * STAGE), st_next = (uint32_t)(((P + 1) & 3) * STAGE);
    constexpr uint32_t st_wr = (uint32_t)(((P + 2) & 3) * STAGE);
    // scales of the next step (its first pairs are converted at the end of this one)
#pragma unroll
    for (int j = 0; j < 2; ++j)
      s_step[(P + 1) & 1][j] = P < 3 ? pick_scale(sc_cur, j, P + 1) : pick_scale(sc_nxt, j, 0);
    __builtin_amdgcn_sched_barrier(0);
    static_for_d<0, NMFMA>([&](auto sc) {
      constexpr int s = decltype(sc)::value;
      constexpr int kk = s / (2 * TM), j = (s / TM) % 2, i = s % TM;
      constexpr int q = kk * 2 + j;  // index of the B fragment in use
      // Two wavefronts share a SIMD (K groups): the one further back in its step gets the issue slots,
      // so that both reach the step's barrier together instead of one idling there.
      if constexpr (GROUPS > 1 && s % (2 * TM) == 0) __builtin_amdgcn_s_setprio(3 - kk);
      const half8_t bm = __builtin_bit_cast(half8_t, fbq[q & 3]);
      acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[kk & 1][i], bm, acc[i][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      // pair conversion pipeline: slot s finishes pairs PPS*(s+LEAD).. and starts the pairs three
      // slots behind them (pairs 32.. belong to the next step's packed weights)
      static_for_d<0, PPS>([&](auto pc) {
        constexpr int pp = decltype(pc)::value;
        constexpr int gd = PPS * (s + LEAD) + pp, ga = gd + 3 * PPS, gb = ga - PPS;
        fbq[(gd / 4) & 3][gd & 3] = stage_scale(gd < 32 ? (P & 1) : ((P + 1) & 1), t_center[pp],
                                                std::integral_constant<int, gd & 31>{});
        t_center[pp] = stage_center(t_bits[pp]);
        t_bits[pp] = gb < 32 ? stage_bits(t_perm[pp], bcur, std::integral_constant<int, gb & 31>{})
                             : stage_bits(t_perm[pp], bnxt, std::integral_constant<int, gb & 31>{});
        t_perm[pp] = ga < 32 ? stage_perm(bcur, std::integral_constant<int, ga & 31>{})
                             : stage_perm(bnxt, std::integral_constant<int, ga & 31>{});
      });
      // A fragments of the next slice (slice 0 of the next stage at the end), one per slot
      if constexpr (j == 0)
        read_a((kk + 1) & 1, a_rd[(kk + 1) & 3] + (kk == 3 ? st_next : st_rd), std::integral_constant<int, i>{});
      // activations: registers -> LDS (step kt+2), then the same registers <- global (step kt+4)
      constexpr int sq = 2 * TM - 1 - (j * TM + i);  // slot index inside the slice, from its end
      // (the activations of step s live in register set s % XS)
      if constexpr (kk == 0 && sq < XL) store_x(xr[(P + 2) % XS], st_wr, std::integral_constant<int, sq>{});
      if constexpr (XS >= 2) {
        if constexpr (kk == 2 && sq < XL) load_x(xr[(P + 2) % XS], kt + 2 + XS, std::integral_constant<int, sq>{});
      } else {
        if constexpr (kk == 1 && sq < XL) load_x(xr[0], kt + 3, std::integral_constant<int, sq>{});
      }
      // packed weights of step kt + RB - 1, into the set whose last use has passed
      if constexpr (HOP) {
        // even steps: the block of steps kt + 2, kt + 3 leaves the hop registers for the LDS area and the register
        // sets of its two steps (both free: their steps kt - 2, kt - 1 are through), column tile by column tile;
        // the registers are requested again at once, for the block of steps kt + 4, kt + 5 (two steps of latency)
        if constexpr (P % 2 == 0) {
          if constexpr (s == 4) hop_store(hb[0]);
          if constexpr (s == 5) hop_load(hb[0], 0, kt + 4);
          if constexpr (s == 6) hop_fetch(rb[(P + 2) % RB], rb[(P + 3) % RB], 0);
          if constexpr (s == 7) hop_store(hb[1]);
          if constexpr (s == 8) hop_load(hb[1], 1, kt + 4);
          if constexpr (s == 9) hop_fetch(rb[(P + 2) % RB], rb[(P + 3) % RB], 1);
        }
      } else if constexpr (RB == 4) {
        if constexpr (kk == 1 && j * TM + i < PBL) load_b(bload, kt + 3, std::integral_constant<int, j * TM + i>{});
      } else {
        // two sets: the current step's set is free once its last pair has entered the pipeline
        // (slot NMFMA - LEAD - 3 - 1 at the latest, i.e. before the last slice)
        if constexpr (kk == 3 && j * TM + i < PBL) load_b(bcur, kt + 2, std::integral_constant<int, j * TM + i>{});
      }
      // scales of the next macro step: requested in its first step, first used in its last
      // (a request just before the back edge would be waited for at once: the loop-carried
      // copy of the loaded words drains the memory pipeline)
      if constexpr (P == 0 && kk == 2 && j * TM + i < 2)
        load_scales_of(sc_nxt, kt + 4, std::integral_constant<int, j * TM + i>{});
      __builtin_amdgcn_sched_barrier(0);
    });
    __syncthreads();
  };

  for (int kt = kbase; kt < kbase + nloop; kt += 4) {
    step(std::integral_constant<int, 0>{}, kt);
    step(std::integral_constant<int, 1>{}, kt + 1);
    step(std::integral_constant<int, 2>{}, kt + 2);
    step(std::integral_constant<int, 3>{}, kt + 3);
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int q = 0; q < SW; ++q) sc_cur[j][q] = sc_nxt[j][q];
  }

  int mrow0 = m0, nrb = TM;  // first row and row blocks this wavefront finishes (a K split's sum shares them out)
  // ---- K groups: the other groups hand their partial sums to the first through LDS ---------
  // Rounds of 16 KB per wavefront (two row blocks each); a wavefront and its partners hold the
  // same elements in the same lanes, so the exchange is lane-contiguous 16-byte vectors.
  if constexpr (GROUPS > 1) {
    float4_t* const xch = reinterpret_cast<float4_t*>(wq_gemm_direct_smem) + wave * (16 * 64) + lane;
#pragma unroll
    for (int g = 1; g < GROUPS; ++g) {
#pragma unroll
      for (int h = 0; h < TM / 2; ++h) {
        if (grp == g) {
#pragma unroll
          for (int il = 0; il < 2; ++il)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
              for (int v4 = 0; v4 < 4; ++v4) {
                const float16_t& a = acc[h * 2 + il][j];
                xch[((il * 2 + j) * 4 + v4) * 64] = float4_t{a[v4 * 4], a[v4 * 4 + 1], a[v4 * 4 + 2], a[v4 * 4 + 3]};
              }
        }
        __syncthreads();
        if (grp == 0) {
#pragma unroll
          for (int il = 0; il < 2; ++il)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
              for (int v4 = 0; v4 < 4; ++v4) {
                const float4_t o = xch[((il * 2 + j) * 4 + v4) * 64];
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[h * 2 + il][j][v4 * 4 + e] += o[e];
              }
        }
        __syncthreads();
      }
    }
    if (!KSPLIT && grp != 0) return;
  }
  if constexpr (KSPLIT) {
    // K split: every workgroup writes the float32 partial tile of its window to the workspace (lane-contiguous
    // 16-byte vectors) and counts itself in; the one that finds S - 1 others counted adds the S partials in the
    // order of their windows -- whoever arrives last, the sum is the same -- and goes on to the epilogue; it
    // returns the counter to zero for the next launch.  Partials and counters are only touched by accesses that
    // are performed at the memory side of the chip's L2s (sc1), and a workgroup's stores have completed before
    // the barrier after which its count goes out.
    // What would break it: one plain load or store (no sc1) of a partial or a counter word, here or in any kernel
    // that shares the workspace -- it may be served from a stale line of the reader's L2 or stay dirty in the
    // writer's.  A source-level test refuses such an access.
    const bool owner = GROUPS == 1 || grp == 0;
    constexpr uint32_t kWaveFloats = TM * 2 * 16 * 64;  // accumulators of one wavefront
    const rsrc_t rp = make_rsrc(partials + (size_t)tile_lin * S * WAVES * kWaveFloats, (uint32_t)S * WAVES * kWaveFloats * 4u);
    if (owner) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int v4 = 0; v4 < 4; ++v4) {
            const float16_t& a = acc[i][j];
            const u32x4 bits = __builtin_bit_cast(u32x4, float4_t{a[v4 * 4], a[v4 * 4 + 1], a[v4 * 4 + 2], a[v4 * 4 + 3]});
            __builtin_amdgcn_raw_buffer_store_b128(bits, rp, ((uint32_t)(ks * WAVES + wave) * (TM * 8) + (i * 2 + j) * 4 + v4) * 1024u + lane * 16u, 0, 0x10);
          }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    int* const last = reinterpret_cast<int*>(wq_gemm_direct_smem);
    if (threadIdx.x == 0)
      *last = __hip_atomic_fetch_add(&counters[tile_lin], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == (unsigned)(S - 1);
    __syncthreads();
    if (!*last) return;
    if (threadIdx.x == 0) __hip_atomic_store(&counters[tile_lin], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // The K groups share the sum: the first RG of them take TM / RG of the tile's row blocks each and finish
    // those rows themselves.  With one row block per group four windows' vectors are in flight together
    // (one trip to the memory side instead of S); with two, one window at a time (two measured no faster).
    constexpr int RG = (TM % GROUPS == 0) ? GROUPS : ((GROUPS % TM == 0) ? TM : 1);
    constexpr int RPG = TM / RG;           // row blocks per reducing group
    constexpr int WIN = RPG == 1 ? 4 : 1;  // windows in flight
    if (grp >= RG) return;
    nrb = RPG;
    const int i0 = grp * RPG;
    mrow0 = m0 + i0 * 32;
#pragma unroll
    for (int i = 0; i < RPG; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
    auto load_window = [&](int q, u32x4 (&buf)[RPG][2][4]) {
      // (windows past the last read zeros: the offset is out of the buffer's range)
      const uint32_t base = q < S ? (uint32_t)(q * WAVES + wave) * (TM * 8) * 1024u : kRowOobD;
#pragma unroll
      for (int i = 0; i < RPG; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int v4 = 0; v4 < 4; ++v4)
            buf[i][j][v4] = __builtin_amdgcn_raw_buffer_load_b128(
                rp, base + (((i0 + i) * 2 + j) * 4 + v4) * 1024u + lane * 16u, 0, 0x10);
    };
    auto add_window = [&](const u32x4 (&buf)[RPG][2][4]) {
#pragma unroll
      for (int i = 0; i < RPG; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int v4 = 0; v4 < 4; ++v4) {
            const float4_t o = __builtin_bit_cast(float4_t, buf[i][j][v4]);
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[i][j][v4 * 4 + e] += o[e];
          }
    };
    u32x4 win[WIN][RPG][2][4];
    for (int q = 0; q < S; q += WIN) {  // windows are added in their order, whoever arrived last
#pragma unroll
      for (int w = 0; w < WIN; ++w) load_window(q + w, win[w]);
#pragma unroll
      for (int w = 0; w < WIN; ++w) add_window(win[w]);  // (+ 0.0 for a window past the last: no change)
    }
  }

  // ---- epilogue: lane holds columns 2 (lane % 32), + 1 and rows 8*(v/4) + 4*(lane/32) + v%4 ------
  const int n = n0 + wave * 64 + 2 * fr;
  if (gated) {
    // the lane's two columns are the gate and the up accumulator of output column n / 2
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = mrow0 + i * 32 + (v >> 2) * 8 + fh * 4 + (v & 3);
        if (i < nrb && m < M && n + 1 < N) store_gated(y, m, n >> 1, N >> 1, acc[i][0][v], acc[i][1][v]);
      }
    return;
  }
  const bool paired = pair_store_ok(ep, y, N);
  if (paired && m0 + BM <= M && n0 + WAVES * 64 <= N) {
    // Tile inside the matrix, 4-byte accesses allowed: the tail's shape is decided once, outside the
    // unrolled stores (per-element tests of the three epilogue fields cost more than the stores).
    half_t* const y0 = y + (size_t)(mrow0 + fh * 4) * N + n;
    auto store_tile = [&](auto has_bias, auto relu, auto has_res) {
      half2_t b2 = half2_t{(half_t)0, (half_t)0};
      if constexpr (decltype(has_bias)::value) b2 = *reinterpret_cast<const half2_t*>(ep.bias + n);
      const half_t* const r0 = decltype(has_res)::value ? ep.residual + (size_t)(mrow0 + fh * 4) * N + n : nullptr;
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          if (i >= nrb) continue;
          half2_t res[4];
          if constexpr (decltype(has_res)::value) {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              res[e] = *reinterpret_cast<const half2_t*>(r0 + (size_t)(i * 32 + g * 8 + e) * N);
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            half2_t h = half2_t{(half_t)acc[i][0][g * 4 + e], (half_t)acc[i][1][g * 4 + e]};
            if constexpr (decltype(has_bias)::value) h = h + b2;
            if constexpr (decltype(relu)::value) {
              h[0] = h[0] > (half_t)0 ? h[0] : (half_t)0;
              h[1] = h[1] > (half_t)0 ? h[1] : (half_t)0;
            }
            if constexpr (decltype(has_res)::value) h = h + res[e];
            *reinterpret_cast<half2_t*>(y0 + (size_t)(i * 32 + g * 8 + e) * N) = h;
          }
        }
    };
    using T = std::true_type;
    using F = std::false_type;
    const bool hb = ep.bias != nullptr, hr = ep.residual != nullptr, ra = ep.activation == 1;
    if (!hb && !ra && !hr) store_tile(F{}, F{}, F{});
    else if (hb && !ra && !hr) store_tile(T{}, F{}, F{});
    else if (hb && ra && !hr) store_tile(T{}, T{}, F{});
    else if (!hb && !ra && hr) store_tile(F{}, F{}, T{});
    else if (hb && !ra && hr) store_tile(T{}, F{}, T{});
    else if (hb && ra && hr) store_tile(T{}, T{}, T{});
    else if (!hb && ra && !hr) store_tile(F{}, T{}, F{});
    else store_tile(F{}, T{}, T{});
    return;
  }
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int m = mrow0 + i * 32 + (v >> 2) * 8 + fh * 4 + (v & 3);
      if (i < nrb && m < M) store_out2<false>(ep, y, m, n, N, acc[i][0][v], acc[i][1][v], paired);
    }
}

namespace {

// Column tiles [tile_n0, tile_n0 + tile_count) of the matrix (tile_count < 0: all of them).
template <int BITS, int GROUPS, int TM, int WAVES, bool TILED, bool KSPLIT = false, bool HOP = false>
bool launch_direct(const Problem& p, int group_shift, int tile_n0 = 0, int tile_count = -1, int ksplit = 1,
                   void* workspace = nullptr) {
  constexpr int BM = TM * 32, BN = WAVES * 64;
  const int tiles_m = (int)((p.m + BM - 1) / BM);
  const int tiles_n = tile_count >= 0 ? tile_count : (int)((p.n + BN - 1) / BN);
  if (tiles_n == 0) return true;
  dim3 grid(tiles_m * tiles_n * ksplit), block(GROUPS * WAVES * 64);
  // workspace of the K split: arrival counters at its head (shared with the decode kernel's split), then
  // [tiles][ksplit] float32 partial tiles
  unsigned int* const counters = static_cast<unsigned int*>(workspace);
  float* const partials = reinterpret_cast<float*>(static_cast<char*>(workspace) + kGemmSplitCounterBytes);
  // four activation stages per K group; the K-group exchange needs 16 KB per wavefront of a group
  // (HOP: 4 KB per wavefront behind the stages, for the weights' way from whole-line loads to the lanes)
  constexpr size_t stages = (size_t)GROUPS * 4 * BM * 128 + (HOP ? (size_t)GROUPS * WAVES * 4096 : 0);
  constexpr size_t exchange = GROUPS > 1 ? (size_t)WAVES * 16384 : 0;
  constexpr size_t lds_bytes = stages > exchange ? stages : exchange;
  static_assert(lds_bytes <= 160 * 1024, "LDS per workgroup");
  static std::atomic<bool> lds_ok[kMaxDevices];
  if (!ensure_dynamic_lds((const void*)wq_gemm_direct_kernel<BITS, GROUPS, TM, WAVES, TILED, KSPLIT, HOP>, (int)lds_bytes, lds_ok))
    return false;
  hipLaunchKernelGGL((wq_gemm_direct_kernel<BITS, GROUPS, TM, WAVES, TILED, KSPLIT, HOP>), grid, block, lds_bytes, p.stream,
                     (const half_t*)p.x, (const uint32_t*)p.wq, (const half_t*)p.scales, (int)p.m, (int)p.n,
                     (int)p.k, group_shift | (p.zero_point << 8) | (p.activation == kActGated ? 1 << 16 : 0), tiles_m, tiles_n, tile_n0, (half_t*)p.y,
                     Epilogue{(const half_t*)p.bias, (const half_t*)p.residual, p.activation}, ksplit, partials, counters);
  return true;
}

// `direct_loads`: the 64-row tiles on canonical int8 weights with every lane loading its own row's pieces, as all
// other builds do, instead of whole cache lines through LDS (kept to pin the two against each other, bit for bit)
template <int GROUPS, int TM, int WAVES>
bool launch_bits(const Problem& p, int group_shift, int tile_n0 = 0, int tile_count = -1, bool direct_loads = false) {
  if constexpr (TM == 2) {
    if (!p.tiled && p.bits == 8 && !direct_loads)
      return launch_direct<8, GROUPS, TM, WAVES, false, false, true>(p, group_shift, tile_n0, tile_count);
  }
  if (p.tiled)
    return p.bits == 4 ? launch_direct<4, GROUPS, TM, WAVES, true>(p, group_shift, tile_n0, tile_count)
                       : launch_direct<8, GROUPS, TM, WAVES, true>(p, group_shift, tile_n0, tile_count);
  return p.bits == 4 ? launch_direct<4, GROUPS, TM, WAVES, false>(p, group_shift, tile_n0, tile_count)
                     : launch_direct<8, GROUPS, TM, WAVES, false>(p, group_shift, tile_n0, tile_count);
}

// The K-split builds: 128 x 256 tiles with two K groups above 64 rows, 64 x 128 tiles with four K groups up to 64.
template <int GROUPS, int TM, int WAVES>
bool launch_split_shape(const Problem& p, int group_shift, int ksplit, void* workspace) {
  if (p.tiled)
    return p.bits == 4 ? launch_direct<4, GROUPS, TM, WAVES, true, true>(p, group_shift, 0, -1, ksplit, workspace)
                       : launch_direct<8, GROUPS, TM, WAVES, true, true>(p, group_shift, 0, -1, ksplit, workspace);
  if constexpr (TM == 2) {
    if (p.bits == 8) return launch_direct<8, GROUPS, TM, WAVES, false, true, true>(p, group_shift, 0, -1, ksplit, workspace);
  }
  return p.bits == 4 ? launch_direct<4, GROUPS, TM, WAVES, false, true>(p, group_shift, 0, -1, ksplit, workspace)
                     : launch_direct<8, GROUPS, TM, WAVES, false, true>(p, group_shift, 0, -1, ksplit, workspace);
}

bool launch_split_bits(const Problem& p, int group_shift, int ksplit, void* workspace) {
  return p.m > 64 ? launch_split_shape<2, 4, 4>(p, group_shift, ksplit, workspace)
                  : launch_split_shape<4, 2, 2>(p, group_shift, ksplit, workspace);
}

// Whether, and how many ways, to split K across workgroups for `p` (128 x 256 tiles, two K groups inside
// the workgroup): where those tiles would leave at least half of the CUs without one -- the cases the
// default selection answers with smaller tiles, whose workgroups then move two to four times the bytes
// per output.  Every window costs a round trip through the workspace (partial tile out, count, the last
// one reads them all), so the windows must stay long: measured on the Llama-2 projections, int8 weights
// gain from windows of four macro steps (K 1024) on, int4 weights -- whose small-tile kernels are better --
// only from eight macro steps on, with at least four windows and tiles on at most an eighth of the CUs.
int gemm_split_ways(const Problem& p) {
  if (p.m <= 16 || p.k % 256 != 0 || p.group != (p.bits == 4 ? 32 : 128) || !gemm_pipe_applicable(p)) return 1;
  if (p.activation == kActGated || p.activation == kActGelu) return 1;
  const int64_t cu = cu_count(), macro = p.k / 256;
  if (p.m <= 64) {
    // 17 .. 64 rows: one row of 64 x 128 tiles (four K groups, so a window is at least four macro steps); without
    // the split these shapes run on a fraction of the CUs or through the register-activation kernel, whose time
    // grows with the rows.  The split costs the same from 17 to 64 rows -- about 16 us on a 4096 x 4096
    // projection, 22 us on 4096 x 11008, 34 us on 5120 x 13824 int8, most of it start-up and the exchange -- so it
    // takes over where the other kernels have grown past it (measured on the Llama-2 7B / 13B projections):
    // with K of at least 8192 from 33 rows on (three row blocks in the register-activation kernel; int8 on
    // canonical weights: from 25); with shorter K only for int4 on canonical weights at more than 48 rows and
    // 96 or more column tiles (12288 x 4096 at 64 rows 24.7 -> 23.1 us).
    const int64_t tiles128 = (p.n + 127) / 128;
    if (p.k >= 8192) {
      if (p.m < ((!p.tiled && p.bits == 8) ? 25 : 33)) return 1;
    } else if (p.tiled || p.bits != 4 || p.m <= 48 || tiles128 < 96) {
      return 1;
    }
    const int64_t tiles = (p.n + 127) / 128;
    if (tiles * 2 > cu || tiles > kGemmSplitMaxTiles) return 1;
    const int64_t ways = std::min<int64_t>({cu / tiles, macro / 4, 8});
    if (ways < 2) return 1;
    const int64_t per = (macro + ways - 1) / ways;
    return (int)((macro + per - 1) / per);
  }
  const int64_t tiles = ((p.m + 127) / 128) * ((p.n + 255) / 256);
  if (tiles * (p.bits == 4 ? 8 : 2) > cu || tiles > kGemmSplitMaxTiles) return 1;
  // (int8 in the canonical layout: since the plain call's 64-row tiles load the weight rows by whole cache lines,
  // the split's 128-row tiles, which do not, only win with long K -- at 256 rows 5120 x 13824 64 against 78 us,
  // but 15360 x 5120 59 against 60 and 5120 x 5120 34.1 against 33.5)
  if (!p.tiled && p.bits == 8 && p.k < 8192) return 1;
  // (not where the plain call's 64 x 128 tiles fill three quarters of the CUs or more in one round:
  // 15360 x 5120 int8 at 128 rows, 240 tiles, 46 us plain against 49 us split)
  const int64_t plain = ((p.m + 63) / 64) * ((p.n + 127) / 128);
  if (p.m <= 128 && plain <= cu && plain * 4 >= cu * 3) return 1;
  const int64_t ways = std::min<int64_t>({cu / tiles, macro / (p.bits == 4 ? 8 : 4), 8});
  if (ways < (p.bits == 4 ? 4 : 2)) return 1;
  const int64_t per = (macro + ways - 1) / ways;  // macro steps per window; drop windows that would be empty
  return (int)((macro + per - 1) / per);
}

}  // namespace

// variant 1: 128 x 256 tile, four wavefronts (one per SIMD); 2: the same tile, eight wavefronts in
// two K groups (two per SIMD), each group accumulating half of K; 3 / 4: the same with 64 rows per
// workgroup -- twice the tiles and about half the time per K step, for M too small to give every CU
// a 128-row tile; 5: 64 x 128 tile, eight wavefronts in four K groups, for problems that leave CUs
// idle even with 64 x 256 tiles; 6: variant 2 for whole rounds of tiles plus variant 4 for the rest.
bool launch_gemm_direct(const Problem& p, int group_shift, int variant) {
  if (!gemm_pipe_applicable(p)) return false;
  // scales are fetched per 256 k: the kernel is laid out for the two benchmark quantizations
  if (p.k % 256 != 0 || p.group != (p.bits == 4 ? 32 : 128)) return false;
  if ((variant == 2 || variant == 4) && p.k < 512) return false;
  if (variant == 5 && p.k < 1024) return false;
  switch (variant) {
    case 1: return launch_bits<1, 4, 4>(p, group_shift);
    case 2: return launch_bits<2, 4, 4>(p, group_shift);
    case 3: return launch_bits<1, 2, 4>(p, group_shift);
    case 4: return launch_bits<2, 2, 4>(p, group_shift);
    case 5: return launch_bits<4, 2, 2>(p, group_shift);
    // 7, 8, 9: variants 3, 4, 5 without the line-wise weight loads that int8 weights in the canonical layout get there
    case 7: return launch_bits<1, 2, 4>(p, group_shift, 0, -1, true);
    case 8: return p.k >= 512 && launch_bits<2, 2, 4>(p, group_shift, 0, -1, true);
    case 9: return p.k >= 1024 && launch_bits<4, 2, 2>(p, group_shift, 0, -1, true);
    case 6: {
      // 128 x 256 tiles for the column tiles that fill whole rounds of the CUs, 64 x 256 tiles for the
      // rest, as a second launch: the last, partly filled round then takes about half as long
      // (2048 x 22016: 1376 tiles = 5.4 rounds of 256 -> five rounds and 192 half tiles: 372 -> 346 us
      // when launches come with pauses, no difference when they run back to back for milliseconds --
      // the part is power limited then, and CUs that idle in a last round let the others clock higher;
      // 512 x 22016: 2 - 7 % either way).  Applies when the rest is at most half a round and its
      // 64-row tiles fit one.
      if (p.k < 512) return false;
      const int64_t cu = cu_count(), tm128 = (p.m + 127) / 128, tm64 = (p.m + 63) / 64, tn = (p.n + 255) / 256;
      const int64_t full_cols = (tm128 * tn / cu) * cu / tm128;  // column tiles inside whole rounds
      const int64_t rest_cols = tn - full_cols;
      if (full_cols < 1 || rest_cols < 1 || rest_cols * tm128 * 2 > cu || rest_cols * tm64 > cu) return false;
      return launch_bits<2, 4, 4>(p, group_shift, 0, (int)full_cols) &&
             launch_bits<2, 2, 4>(p, group_shift, (int)full_cols, (int)rest_cols);
    }
    default: return false;
  }
}


// Bytes of caller workspace the K split of the direct-weight GEMM needs for `p`, 0 where it does not apply.
int64_t gemm_split_workspace_bytes(const Problem& p) {
  const int ways = gemm_split_ways(p);
  if (ways < 2) return 0;
  if (p.m <= 64) return kGemmSplitCounterBytes + ((p.n + 127) / 128) * ways * (64 * 128 * 4);
  const int64_t tiles = ((p.m + 127) / 128) * ((p.n + 255) / 256);
  return kGemmSplitCounterBytes + tiles * ways * (128 * 256 * 4);
}

// 1 = launched with the K split, 0 = the split does not apply or the workspace is too small, -1 = failure
int launch_gemm_split(const Problem& p, void* workspace, int64_t workspace_bytes) {
  const int64_t need = gemm_split_workspace_bytes(p);
  if (need == 0 || workspace == nullptr || workspace_bytes < need) return 0;
  const int ch = 128 / p.bits;
  int ratio = p.group / ch, group_shift = 0;
  while ((1 << group_shift) < ratio) ++group_shift;
  if (!launch_split_bits(p, group_shift, gemm_split_ways(p), workspace)) return -1;
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("gemm kernel (K split) launch failed: %s", hipGetErrorString(e));
    return -1;
  }
  return 1;
}

}  // namespace wq
