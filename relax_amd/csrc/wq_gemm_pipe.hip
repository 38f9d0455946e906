// Software-pipelined MFMA GEMM for prefill (M > 64): y[M,N] = x[M,K] @ dequant(Wq,S)^T.
//
// Bound: dense float16 MFMA.  A workgroup owns a BM x BN output tile and walks K in
// steps of 64.  Its wavefronts hold (BM/WM) x (BN/WN) sub-tiles as 32x32 MFMA
// accumulators (v_mfma_f32_32x32x16_f16, float32).  Per step and wavefront the
// MFMA pipe needs TM*TN*4 instructions of 32 cycles; everything else -- global
// loads of the next-but-two step, the int4/int8 -> float16 dequantization of the
// next-but-one step, LDS stores, LDS operand reads -- is interleaved between them
// (sched_group_barrier) so that the matrix pipe is the only critical resource.
//
// Pipeline (step t is being multiplied):
//   global -> registers : step t+3, issued at the top of the iteration (two register
//                         sets, so a load has a full iteration to arrive);
//   registers -> LDS    : step t+2, dequantized to exactly the float16 values the
//                         CPU path materialises, written between the MFMAs;
//   LDS -> registers    : operand fragments of the next 16-wide k slice, and at the
//                         end of the step the first slice of step t+1.
// LDS holds three stages, so the stage read by step t+1 was completed before the
// previous barrier and one barrier per step suffices.
//
// LDS layout per stage: activations [BM][64] then weights [BN][64] float16, rows of
// 128 bytes whose eight 16-byte chunks are XOR-swizzled with ((row >> 1) & 7): the
// 16-byte operand reads of 16 consecutive lanes (16 consecutive rows, same chunk)
// then cover all 64 banks exactly once, without padding.
//
// Shape requirements (checked by the launcher; other shapes use the generic GEMM
// kernel): K a multiple of 64, every operand below 1 GiB.
#include <atomic>
#include <type_traits>

#include "wq_device.h"
#include "wq_internal.h"

namespace wq {

namespace {
constexpr uint32_t kRowOob = 0x80000000u;   // offset of a row that must read zeros
constexpr uint32_t kStepOob = 0x40000000u;  // added for a k step past K: beyond any buffer < 1 GiB
}  // namespace

// Compile-time loop: f(std::integral_constant<int, B>{}), ..., f(std::integral_constant<int, E-1>{}).
template <int B, int E, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (B < E) {
    f(std::integral_constant<int, B>{});
    static_for<B + 1, E>(f);
  }
}

template <int XL, int WL>
struct GemmStage {
  u32x4 x[XL];
  u32x4 w[WL];
  uint32_t s[WL];
};

template <int BITS, int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(WM * WN * 64, 1) void wq_gemm_pipe_kernel(
    const half_t* __restrict__ x, const uint32_t* __restrict__ wq, const half_t* __restrict__ scales,
    half_t* y, int M, int N, int K, int group_shift, int zero_point, int tiles_m, int tiles_n,
    const Epilogue ep) {
  constexpr int BK = 64;
  constexpr int NT = WM * WN * 64;
  constexpr int CH = 128 / BITS;          // k per 16-byte packed chunk: 32 / 16
  constexpr int TM = BM / WM / 32;        // 32x32 accumulator tiles per wavefront along M
  constexpr int TN = BN / WN / 32;
  constexpr int XL = BM * 8 / NT;         // 16-byte activation chunks per thread per step
  constexpr int WL = BN * (BK / CH) / NT; // 16-byte packed weight chunks per thread per step
  constexpr int WPC = CH / 8;             // 16-byte float16 chunks produced per packed chunk: 4 / 2
  constexpr int STAGE = (BM + BN) * 128;  // bytes per LDS stage
  static_assert(BM * 8 % NT == 0 && BN * (BK / CH) % NT == 0 && XL >= 1 && WL >= 1, "tile/thread split");
  static_assert(XL % 4 == 0 && (WL * WPC) % 4 == 0, "stores are spread over the four k slices of a step");

  extern __shared__ __attribute__((aligned(16))) unsigned char wq_gemm_pipe_smem[];
  unsigned char* const lds = wq_gemm_pipe_smem;

  // XCD-aware tile order: consecutive workgroup ids land on different XCDs, so regroup
  // them to keep the tiles that share a weight column block on one L2.
  const int nblocks = tiles_m * tiles_n;
  int bid = blockIdx.x;
  if ((nblocks & 7) == 0) bid = (bid & 7) * (nblocks >> 3) + (bid >> 3);
  const int tile_m = bid % tiles_m;
  const int tile_n = bid / tiles_m;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;

  const uint32_t row_bytes = (uint32_t)K * BITS / 8;
  const uint32_t groups_per_row = ((uint32_t)K / CH) >> group_shift;
  const rsrc_t rw = make_rsrc(wq, (uint32_t)N * row_bytes);
  const rsrc_t rs = make_rsrc(scales, (uint32_t)N * groups_per_row * 2u);
  const rsrc_t rx = make_rsrc(x, (uint32_t)M * (uint32_t)K * 2u);

  // ---- per-thread global offsets and LDS store addresses ----------------------------
  uint32_t xg[XL];  // byte offset of this thread's chunk in row (m0 + row) at k = 0
  const int x_row0 = tid >> 3, x_c = tid & 7;
#pragma unroll
  for (int i = 0; i < XL; ++i) {
    const int m = m0 + x_row0 + i * (NT / 8);
    xg[i] = m < M ? (uint32_t)m * (uint32_t)K * 2u + (uint32_t)x_c * 16u : kRowOob;
  }
  // NT/8 is a multiple of 16, so the swizzle term is the same for every i
  const uint32_t x_lds = (uint32_t)x_row0 * 128u + (uint32_t)((x_c ^ ((x_row0 >> 1) & 7)) << 4);

  uint32_t wg[WL], sg[WL], w_lds[WL][WPC];
  int w_kofs[WL];  // k offset of the packed chunk inside the step
#pragma unroll
  for (int i = 0; i < WL; ++i) {
    const int c = tid + i * NT;
    const int row = c / (BK / CH), q = c % (BK / CH);
    const int n = min(n0 + row, N - 1);  // rows past N are computed but never stored
    wg[i] = (uint32_t)n * row_bytes + (uint32_t)q * 16u;
    sg[i] = (uint32_t)n * groups_per_row * 2u;
    w_kofs[i] = q * CH;
#pragma unroll
    for (int j = 0; j < WPC; ++j) {
      const int chunk = q * WPC + j;
      w_lds[i][j] = (uint32_t)BM * 128u + (uint32_t)row * 128u + (uint32_t)((chunk ^ ((row >> 1) & 7)) << 4);
    }
  }

  // ---- per-lane LDS operand read addresses, one per 16-wide k slice -----------------
  const int fr = lane & 31, fh = lane >> 5;
  uint32_t a_rd[4], b_rd[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) {
    const uint32_t swz = (uint32_t)(((kk * 2 + fh) ^ ((fr >> 1) & 7)) << 4);
    a_rd[kk] = (uint32_t)(wm * (BM / WM) + fr) * 128u + swz;
    b_rd[kk] = (uint32_t)BM * 128u + (uint32_t)(wn * (BN / WN) + fr) * 128u + swz;
  }

  const Q4Consts qc = make_q4_consts(zero_point);
  const int ksteps = K / BK;
  const int ksteps_even = (ksteps + 1) & ~1;  // the loop is unrolled by two register sets

  // ---- the pieces of work that are slotted between the MFMAs of a step ------------------
  // global -> registers, piece c of step kt: activation chunk c, or packed weights + scale
  auto load_piece = [&](GemmStage<XL, WL>& g, uint32_t xk, uint32_t wk, uint32_t k0, bool ok, auto cc) {
    constexpr int c = decltype(cc)::value;
    if constexpr (c < XL) {
      g.x[c] = load_b128(rx, xg[c] + xk);
    } else {
      constexpr int i = c - XL;
      g.w[i] = load_b128(rw, wg[i] + wk);
      const uint32_t sk = ok ? (((k0 + (uint32_t)w_kofs[i]) / CH) >> group_shift) * 2u : kStepOob;
      g.s[i] = load_b16(rs, sg[i] + sk);
    }
  };
  constexpr int PC = XL + WL;  // load pieces per step
  auto issue_global = [&](GemmStage<XL, WL>& g, int kt) {
    const uint32_t k0 = (uint32_t)kt * BK;
    const bool ok = kt < ksteps;
    const uint32_t xk = ok ? k0 * 2u : kStepOob, wk = ok ? k0 * BITS / 8 : kStepOob;
    static_for<0, PC>([&](auto cc) { load_piece(g, xk, wk, k0, ok, cc); });
  };

  // registers -> LDS, piece b: for every float16 chunk of dequantized weights four
  // pair conversions and one 16-byte store, then the activation chunk stores
  constexpr int NCH = WL * WPC;         // float16 chunks of weights per thread per step
  constexpr int PB = 5 * NCH + XL;      // store pieces per step
  half2_t hq[4];
  auto store_piece = [&](const GemmStage<XL, WL>& g, uint32_t stage_base, auto bc) {
    constexpr int b = decltype(bc)::value;
    if constexpr (b < 5 * NCH) {
      constexpr int c = b / 5, pp = b % 5, wi = c / WPC, wj = c % WPC;
      if constexpr (pp < 4) {
        const half2_t s2 = bcast_h2(__builtin_bit_cast(half_t, (uint16_t)g.s[wi]));
        if constexpr (BITS == 4) {
          const uint32_t tt = __builtin_amdgcn_perm(0u, g.w[wi][wj], 0x0c000c00u | (uint32_t)pp | ((uint32_t)pp << 16));
          const half2_t h = as_h2(and_or(tt, 0x00F0000Fu, qc.magic));
          hq[pp] = __builtin_elementwise_fma(h, qc.mix_mul, -qc.mix_sub) * s2;
        } else {
          const half2_t off = half2_t{(half_t)1152.0f, (half_t)1152.0f};
          const uint32_t word = g.w[wi][2 * wj + pp / 2];
          const uint32_t tt = __builtin_amdgcn_perm(0u, word, (pp & 1) ? 0x0c030c02u : 0x0c010c00u) ^ 0x64806480u;
          hq[pp] = (as_h2(tt) - off) * s2;
        }
      } else {
        *reinterpret_cast<u32x4*>(lds + stage_base + w_lds[wi][wj]) =
            u32x4{as_u32(hq[0]), as_u32(hq[1]), as_u32(hq[2]), as_u32(hq[3])};
      }
    } else {
      constexpr int i = b - 5 * NCH;
      *reinterpret_cast<u32x4*>(lds + stage_base + x_lds + (uint32_t)i * (NT / 8) * 128u) = g.x[i];
    }
  };
  auto store_all = [&](const GemmStage<XL, WL>& g, uint32_t stage_base) {
    static_for<0, PB>([&](auto bc) { store_piece(g, stage_base, bc); });
  };

  // LDS -> operand fragments of k slice `kk` of a stage, fragment f in the order the
  // MFMAs need them: A0, B0 .. B(TN-1), A1 .. A(TM-1)
  half8_t fa[2][TM], fb[2][TN];
  auto read_piece = [&](int buf, uint32_t a_base, uint32_t b_base, auto fc) {
    constexpr int f = decltype(fc)::value;
    if constexpr (f == 0) {
      fa[buf][0] = *reinterpret_cast<const half8_t*>(lds + a_base);
    } else if constexpr (f <= TN) {
      fb[buf][f - 1] = *reinterpret_cast<const half8_t*>(lds + b_base + (uint32_t)(f - 1) * 4096u);
    } else {
      fa[buf][f - TN] = *reinterpret_cast<const half8_t*>(lds + a_base + (uint32_t)(f - TN) * 4096u);
    }
  };

  float16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  // ---- prologue: steps 0 and 1 into LDS, step 2 into registers ----------------------
  GemmStage<XL, WL> g0, g1;
  issue_global(g0, 0);
  issue_global(g1, 1);
  store_all(g0, 0u);
  issue_global(g0, 2);
  store_all(g1, (uint32_t)STAGE);
  __syncthreads();
  static_for<0, TM + TN>([&](auto fc) { read_piece(0, a_rd[0], b_rd[0], fc); });

  // One step.  `cur` holds step kt+2 (stored to stage st_wr between the MFMAs), `nxt`
  // receives step kt+3.  Program order is the intended issue order: after every MFMA
  // (32 cycles of the matrix pipe, 4 of the issue port) a handful of independent
  // instructions; sched_barrier keeps the compiler from regrouping them.
  constexpr int NMFMA = TM * TN * 4;
  auto step = [&](GemmStage<XL, WL>& cur, GemmStage<XL, WL>& nxt, int kt, uint32_t st_rd,
                  uint32_t st_next, uint32_t st_wr) {
    const uint32_t k0n = (uint32_t)(kt + 3) * BK;
    const bool okn = kt + 3 < ksteps;
    const uint32_t xk = okn ? k0n * 2u : kStepOob, wk = okn ? k0n * BITS / 8 : kStepOob;
    uint32_t a_cur[4], b_cur[4];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      a_cur[kk] = a_rd[kk] + (kk == 0 ? st_next : st_rd);  // slice 0 is pre-read for the next step
      b_cur[kk] = b_rd[kk] + (kk == 0 ? st_next : st_rd);
    }
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, NMFMA>([&](auto sc) {
      constexpr int s = decltype(sc)::value;
      constexpr int kk = s / (TM * TN), tix = s % (TM * TN), i = tix / TN, j = tix % TN;
      acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[kk & 1][i], fb[kk & 1][j], acc[i][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (tix < TM + TN) {
        constexpr int nk = (kk + 1) & 3;  // next slice: kk+1 of this stage, or 0 of the next
        read_piece((kk + 1) & 1, a_cur[nk], b_cur[nk], std::integral_constant<int, tix>{});
      }
      static_for<s * PB / NMFMA, (s + 1) * PB / NMFMA>([&](auto bc) { store_piece(cur, st_wr, bc); });
      static_for<s * PC / NMFMA, (s + 1) * PC / NMFMA>(
          [&](auto cc) { load_piece(nxt, xk, wk, k0n, okn, cc); });
      __builtin_amdgcn_sched_barrier(0);
    });
    __syncthreads();
  };

  uint32_t st_rd = 0u, st_next = (uint32_t)STAGE, st_wr = 2u * STAGE;
  for (int kt = 0; kt < ksteps_even; kt += 2) {
    step(g0, g1, kt, st_rd, st_next, st_wr);
    step(g1, g0, kt + 1, st_next, st_wr, st_rd);
    const uint32_t r0 = st_rd;  // two steps later the three stages have rotated by two
    st_rd = st_wr;
    st_wr = st_next;
    st_next = r0;
  }

  // ---- epilogue: lane holds column (lane % 32) and rows 8*(v/4) + 4*(lane/32) + v%4 ---
  // the tail's shape is tested once, not per element
  const bool plain = ep.bias == nullptr && ep.residual == nullptr && ep.activation == 0;
  auto store_tiles = [&](auto plain_c) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int n = n0 + wn * (BN / WN) + j * 32 + fr;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int m = m0 + wm * (BM / WM) + i * 32 + (v >> 2) * 8 + fh * 4 + (v & 3);
          if (m < M && n < N) {
            if constexpr (decltype(plain_c)::value) y[(size_t)m * N + n] = (half_t)acc[i][j][v];
            else store_out(ep, y, m, n, N, acc[i][j][v]);
          }
        }
      }
  };
  if (plain) store_tiles(std::true_type{});
  else store_tiles(std::false_type{});
}

namespace {

template <int BITS, int BM, int BN, int WM, int WN>
bool launch_pipe(const Problem& p, int group_shift) {
  const int tiles_m = (int)((p.m + BM - 1) / BM);
  const int tiles_n = (int)((p.n + BN - 1) / BN);
  dim3 grid(tiles_m * tiles_n), block(WM * WN * 64);
  constexpr size_t lds_bytes = 3 * (size_t)(BM + BN) * 128;
  static_assert(lds_bytes <= 160 * 1024, "three stages must fit the 160 KB LDS");
  static std::atomic<bool> lds_ok[kMaxDevices];
  if (!ensure_dynamic_lds((const void*)wq_gemm_pipe_kernel<BITS, BM, BN, WM, WN>, (int)lds_bytes, lds_ok)) return false;
  hipLaunchKernelGGL((wq_gemm_pipe_kernel<BITS, BM, BN, WM, WN>), grid, block, lds_bytes, p.stream,
                     (const half_t*)p.x, (const uint32_t*)p.wq, (const half_t*)p.scales,
                     (half_t*)p.y, (int)p.m, (int)p.n, (int)p.k, group_shift, p.zero_point, tiles_m,
                     tiles_n, Epilogue{(const half_t*)p.bias, (const half_t*)p.residual, p.activation});
  return true;
}

}  // namespace

bool gemm_pipe_applicable(const Problem& p) {
  const int64_t lim = 0x40000000ll;
  return p.k % 64 == 0 && p.k >= 64 && p.m * p.k * 2 < lim && p.n * (p.k * p.bits / 8) < lim;
}

// variant: 1 = 256x128 tile, 2 = 128x128, 3 = 128x256 (BM x BN), four wavefronts each
bool launch_gemm_pipe(const Problem& p, int group_shift, int variant) {
  if (!gemm_pipe_applicable(p)) return false;
#define WQ_PIPE_CASE(ID, BM, BN, WM, WN)                             \
  case ID:                                                           \
    return p.bits == 4 ? launch_pipe<4, BM, BN, WM, WN>(p, group_shift) \
                       : launch_pipe<8, BM, BN, WM, WN>(p, group_shift);
  switch (variant) {
    WQ_PIPE_CASE(1, 256, 128, 2, 2)
    WQ_PIPE_CASE(2, 128, 128, 2, 2)
    WQ_PIPE_CASE(3, 128, 256, 2, 2)
    default: return false;
  }
#undef WQ_PIPE_CASE
}

}  // namespace wq
