// GEMV kernel for decode batches (M <= 16): y[M,N] = x[M,K] @ dequant(Wq,S)^T.
//
// Bound: HBM bandwidth.  Every byte of packed weight is read exactly once with
// 16-byte buffer loads.  The kernel is persistent: the grid is sized to the chip
// (a few workgroups per CU) and every workgroup walks a strided list of 16-row
// weight tiles, so that
//   * the activations are staged in LDS once per workgroup instead of once per
//     tile (LDS reads are counted by a different wait counter than global loads,
//     so the weight prefetch depth is not tied to activation registers);
//   * the weight stream of a wavefront is one software pipeline across all its
//     tiles: while it consumes one "super step" the next one -- possibly of the
//     next tile -- is already in flight.
//
// Work split inside a workgroup: its WAVES wavefronts split K.  K is walked in
// super steps of 4*D chunks (chunk = the k covered by one 16-byte lane load: 32
// for int4, 16 for int8).  Lane (col = lane % 16, kq = lane / 16) owns weight row
// `col` of the tile and the D consecutive chunks kq*D .. kq*D+D-1 of the super
// step, so its group scales are one contiguous load per super step.  Chunk d of
// all four kq feeds NJ v_mfma_f32_16x16x32_f16 (A = activations from LDS, B = the
// weights dequantized in registers to exactly the float16 value the CPU path
// materialises).  Rows of the MFMA tile beyond M read activation row 0; their
// results are never stored.
//
// When M*K does not fit the LDS staging area, K is processed in phases: stage a
// K range, run every tile of the workgroup over it, restage.  Each wavefront adds
// its partial tile to a private LDS slot (no atomics, deterministic order); the
// slots are summed over wavefronts, converted and stored once at the end.
//
// The int4 activations are written to LDS already in the pair order
// (k0,k4)(k1,k5)(k2,k6)(k3,k7) the nibble unpack produces, so the loop has no
// permutes.
//
// TILED: weights and scales are in the tile-major layout (wq_tiled.hip), whose blocks are
// exactly what a wavefront reads per instruction (D = 2): every load of the weight stream
// is 1 KB contiguous.  Same lanes, same chunks, same order: bit-identical results.
//
// XS: how the first phase's activations reach LDS, a build each -- the start-up of a launch runs on a cold
// instruction cache, and every alternative it has to jump over costs a fetch from memory (with all of them in one
// build a batch-1 launch took 0.3 us longer).  0: a flat index over (row, 16-byte column) of any shape, up to
// three requests per thread ahead of the first weights, the rest in a loop (batch 1 - 2, or rows longer than
// the workgroup has threads); 1, 2, 3: the same for exactly that many requests per thread and rows of at least as
// many vectors as the workgroup has threads (K >= 4096 with eight wavefronts) -- straight-line code, no division;
// 4, 8, 16: a thread stages its own column of up to that many rows, the first four or eight requested ahead of the
// first weights.
//
// KSPLIT: K is split over R workgroups per tile list as well (caller workspace): each writes a
// float32 partial tile, the last to arrive adds them in the order of the K windows and stores.
#include <algorithm>
#include <atomic>
#include <type_traits>

#include "wq_device.h"
#include "wq_internal.h"

namespace wq {

// Measurement build (-DWQ_GEMV_STAMPS, linked into a library of its own that only bench.py --stamps loads): every
// wavefront records the 100 MHz real-time counter at eight points of its life -- entry, first requests issued,
// activations staged, first super step computed, end of the weight stream, before and after the barrier ahead of the
// slot sum, stores acknowledged -- into a device array with one slot per launch modulo four, so that the last four
// launches of a replayed graph can be read back.  In the product build the hooks expand to nothing.
#ifdef WQ_GEMV_STAMPS
constexpr int kStampLaunches = 4, kStampWaves = 4096, kStampPoints = 8;
__device__ unsigned long long g_gemv_stamps[kStampLaunches * kStampWaves * kStampPoints];
#define WQ_STAMP(i) (stamps_[i] = __builtin_amdgcn_s_memrealtime())
#else
#define WQ_STAMP(i) ((void)0)
#endif

template <int D, int SPL>
struct GemvBuf {
  u32x4 w[D];
  uint32_t sc[SPL > 1 ? SPL / 2 : 1];  // SPL float16 scales, packed two per register
};

// What a wavefront walks in one K phase: of every tile of its workgroup the super steps start .. start + cnt - 1
// (the phase's super steps dealt out evenly: the first `nsuper % WAVES` wavefronts take one more).
struct GemvCtx {
  int chunk_base;  // first chunk of the phase
  int nsuper;      // super steps of the phase
  int start, cnt;
};

// The kernel's argument segment as a struct (arguments are laid out in order with their natural alignment):
// the kernel reads the arguments that only its last section needs -- the output, the epilogue, the K split's
// workspace -- through the segment pointer, at a place of the kernel's choosing (fetch_late_arguments).  Left to
// itself the compiler fetches them at the top of the kernel and, in the builds that run short of scalar registers,
// waits for that fetch (a trip to host-visible memory) to spill them: ahead of the first weight request.
struct GemvKernArgs {
  const half_t* x;
  const uint32_t* wq;
  const half_t* scales;
  int M, N, K, shift_and_zero, max_tiles, phase_chunks, ksplit, grid;
  half_t* y;
  Epilogue ep;
  float* partials;
  unsigned int* counters;
};

template <int BITS, int WAVES, int D, int SPL, bool TILED, int XS, bool KSPLIT, bool PHASES>
// PHASES: the launch walks K in more than one phase (activations beyond the LDS).  The host knows; as a template
// flag it keeps the second phase description out of the build that runs the common launches, whose first memory
// requests otherwise wait behind that bookkeeping (and behind the late kernel arguments, which the compiler
// fetched early and spilled when the scalar registers ran out).
// Scalar kernel arguments instead of one struct, and in this order: the first 14 dwords of the
// argument segment are preloaded into SGPRs at wavefront launch (16 user SGPRs less the segment
// pointer); anything after them is fetched by a scalar load from host-visible memory.
// Everything the staging and the weight stream need -- the three input pointers, the shape, the
// plan and the grid size (gridDim.x is itself a load from the end of the segment), 14 dwords --
// therefore comes first, and what only the final store needs (y, the epilogue, the K split's
// workspace) after it.
// (at least two wavefronts per SIMD as far as registers go, also for the 4-wavefront builds: with 512
// registers to hand the compiler keeps the accumulator in AGPRs and copies it to and from VGPRs around the
// stream loop, and a copy out of the AGPRs that a taken branch puts right behind the last MFMA reads the
// registers before the MFMA has written them -- the wait states are missing on that path; the 4-wavefront
// builds lost part of a super step's sum in two of four accumulator registers that way)
__global__ __launch_bounds__(WAVES * 64) __attribute__((amdgpu_waves_per_eu(2, 8))) void wq_gemv_kernel(
    const half_t* x_, const uint32_t* wq_, const half_t* scales_, int M_, int N_, int K_,
    int shift_and_zero_, int max_tiles_, int phase_chunks_, int ksplit_, int grid_, half_t* y_late, const Epilogue ep_late,
    float* partials_late, unsigned int* counters_late) {
  static_assert(!KSPLIT || !PHASES, "the cross-workgroup K split walks one window of K");
  static_assert(XS == 0 || XS == 1 || XS == 2 || XS == 3 || XS == 4 || XS == 8 || XS == 16, "staging mode");
  constexpr bool ROWS = XS >= 4;
  constexpr bool XPRE = PHASES && (XS == 4 || XS == 8);  // (up to eight rows) a phase's activations are requested a phase ahead
  const int group_shift_ = shift_and_zero_ & 0xFF, zero_point_ = (shift_and_zero_ >> 8) & 0xFF;
  const bool gated = (shift_and_zero_ >> 16) & 1;  // fused multiply(nn.silu(gate), up): rows walked interleaved
  // Weight rows per tile, 8 .. 16 (16 on tile-major weights, with the gated tail and with the K split): a tile is
  // always 16 MFMA columns, of which the first tile_rows carry rows -- the host shortens the tiles where 16-row
  // tiles would leave the workgroups unevenly loaded (5120 rows: 320 tiles on 256 workgroups, two for some and one
  // for the others; 512 tiles of 10 rows: two for each).
  const int tile_rows = (shift_and_zero_ >> 20) & 0x1F;
  constexpr int CH = 128 / BITS;  // k per 16-byte lane load
  constexpr int NJ = CH / 8;      // MFMAs per lane load
  constexpr int NT = WAVES * 64;
  const int lds_stride = phase_chunks_ * CH + 8;  // halves per staged row (launch_one's plan)
  static_assert(SPL == 1 || SPL == D, "one scale per super step, or one per chunk");
  static_assert(!TILED || D == 2, "the tile-major layout is written for super steps of eight chunks");
  static_assert(SPL == 1 || (SPL % 2 == 0 && SPL <= 8), "scale vector is 4, 8 or 16 bytes");
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keeps loop control scalar
  const int col = lane & 15, kq = lane >> 4;
#ifdef WQ_GEMV_STAMPS
  unsigned long long stamps_[kStampPoints] = {};
#endif
  WQ_STAMP(0);
  const int M = M_, N = N_, K = K_;

  extern __shared__ __attribute__((aligned(16))) unsigned char wq_gemv_smem[];
  // [max_tiles][WAVES][4][64] float partial tiles, then [M][lds_stride] staged activations
  float* slots = reinterpret_cast<float*>(wq_gemv_smem);
  half_t* xs = reinterpret_cast<half_t*>(wq_gemv_smem + (size_t)max_tiles_ * WAVES * 1024);

  const uint32_t row_bytes = (uint32_t)K * BITS / 8;
  const int nchunks = K / CH;
  const uint32_t groups_per_row = (uint32_t)nchunks >> group_shift_;
  // (the tile-major buffers hold whole tiles: rows up to the next multiple of 16, zero filled)
  const uint32_t n_stored = TILED ? (uint32_t)((N_ + 15) >> 4) * 16u : (uint32_t)N;
  const rsrc_t rw = make_rsrc(wq_, n_stored * row_bytes);
  const rsrc_t rs = make_rsrc(scales_, n_stored * groups_per_row * 2u);
  const rsrc_t rx = make_rsrc(x_, (uint32_t)M * (uint32_t)K * 2u);

  // XS = 1, 2, 3: the activation requests ahead of everything else -- they need nothing but the thread index and the
  // shape.  Vector q of this thread is index tid + q * NT of the flat order, in row 0, 1 or 2 (rows have at least
  // NT vectors, launch_one checks); one phase: a vector inside K is inside the phase.
  constexpr int XQ = (XS >= 1 && XS <= 3) ? XS : 1;
  int mq[XQ], kvq[XQ];
  u32x4 xq[XQ];
  if constexpr (XS >= 1 && XS <= 3) {
    const int vec_per_row = (nchunks + 4 * D - 1) / (4 * D) * (4 * D) * CH / 8;
#pragma unroll
    for (int q = 0; q < XS; ++q) {
      mq[q] = q == 0 ? 0 : (tid + q * NT >= vec_per_row ? 1 : 0) + (tid + q * NT >= 2 * vec_per_row ? 1 : 0);
      kvq[q] = tid + q * NT - mq[q] * vec_per_row;
      const bool ok = mq[q] < M && kvq[q] * 8 < K;
      xq[q] = load_b128(rx, ok ? ((uint32_t)mq[q] * (uint32_t)K + (uint32_t)(kvq[q] * 8)) * 2u : kOobOffset);
    }
    __builtin_amdgcn_sched_barrier(0);
  }

  // Tiles of this workgroup: tile0, tile0 + tstride, ...  With the K split, R consecutive workgroups
  // share a tile list and each walks its own window of K (phase_chunks chunks from kr * phase_chunks).
  const int G = grid_;
  const int R = KSPLIT ? ksplit_ : 1;
  const int kr = KSPLIT ? (int)blockIdx.x % R : 0;
  const int tile0 = KSPLIT ? (int)blockIdx.x / R : (int)blockIdx.x;
  const int tstride = KSPLIT ? G / R : G;
  // (= ceil((tiles - tile0) / tstride) without the division: max_tiles is the ceiling for tile0 = 0)
  const int my_tiles = max_tiles_ - ((tile0 + (max_tiles_ - 1) * tstride) * tile_rows >= N ? 1 : 0);

  const Q4Consts qc = make_q4_consts(zero_point_);
  const half_t* xrow = xs + (size_t)(col < M ? col : 0) * lds_stride;

  auto make_ctx = [&](int chunk_base) -> GemvCtx {
    GemvCtx c;
    c.chunk_base = chunk_base;
    const int ph_chunks = min(phase_chunks_, nchunks - chunk_base);
    c.nsuper = ph_chunks > 0 ? (ph_chunks + 4 * D - 1) / (4 * D) : 0;
    const int base = c.nsuper / WAVES, extra = c.nsuper % WAVES;
    c.cnt = base + (wave < extra ? 1 : 0);
    c.start = wave * base + min(wave, extra);
    return c;
  };
  const GemvCtx dead_ctx = GemvCtx{nchunks, 0, 0, 0};
  // the items of a phase in the order a wavefront walks them: (tile index i, step s); i = my_tiles: no item
  auto first_tile = [&](const GemvCtx& c) { return c.cnt > 0 ? 0 : my_tiles; };
  auto advance = [&](const GemvCtx& c, int& i, int& s) {
    if (++s >= c.cnt) {
      s = 0;
      ++i;
    }
  };

  // weights of item (i, s) of phase `c` -> registers; anything that is no item loads zeros
  auto load_super = [&](GemvBuf<D, SPL>& b, const GemvCtx& c, int i, int s) {
    const int ss = c.start + s;  // super step within the phase
    const int tile = tile0 + i * tstride;
    bool ok = i < my_tiles;
    if constexpr (TILED) {
      // Tile-major stream: the D 1 KB blocks of (tile, super step) are consecutive and lane l owns
      // bytes 16 l .. 16 l + 15 of each -- every load instruction of the wavefront reads 1 KB
      // contiguously.  Scales: int4 / group 32 one 4-byte pair per lane, int8 / group 128 one
      // float16 per (row, super step).
      const uint32_t nsuper_all = (uint32_t)nchunks / (4 * D);
      const uint32_t item = (uint32_t)tile * nsuper_all + (uint32_t)(c.chunk_base / (4 * D) + ss);
      ok = ok && (c.chunk_base + ss * 4 * D < nchunks);
      const uint32_t woff = ok ? item * (D * 1024u) + (uint32_t)lane * 16u : kOobOffset;
#pragma unroll
      for (int d = 0; d < D; ++d) b.w[d] = load_b128(rw, woff + d * 1024u);
      if constexpr (SPL == 1) b.sc[0] = load_b16(rs, ok ? (item * 16u + (uint32_t)col) * 2u : kOobOffset);
      else b.sc[0] = load_b32(rs, ok ? (item * 64u + (uint32_t)lane) * 4u : kOobOffset);
      return;
    }
    int n = min(tile * tile_rows + col, N - 1);  // rows past N: computed, not stored
    ok = ok && col < tile_rows;                  // columns past the tile's rows: zeros, no request
    if (gated) n = gated_physical_row(n, N);  // even columns of a tile: gate rows, odd columns: their up rows
    const int chunk0 = c.chunk_base + ss * 4 * D + kq * D;
    // D > 1 is only launched when K is a multiple of 4*D chunks, so a lane's D
    // chunks are valid together; D == 1 checks its single chunk.
    ok = ok && (chunk0 < nchunks);
    const uint32_t woff = ok ? (uint32_t)n * row_bytes + (uint32_t)chunk0 * 16u : kOobOffset;
    const uint32_t soff =
        ok ? ((uint32_t)n * groups_per_row + ((uint32_t)chunk0 >> group_shift_)) * 2u : kOobOffset;
#pragma unroll
    for (int d = 0; d < D; ++d) b.w[d] = load_b128(rw, woff + d * 16u);
    if constexpr (SPL == 1) {
      b.sc[0] = load_b16(rs, soff);
    } else if constexpr (SPL == 2) {
      b.sc[0] = load_b32(rs, soff);
    } else if constexpr (SPL == 4) {
      const u32x2 v = load_b64(rs, soff);
      b.sc[0] = v[0];
      b.sc[1] = v[1];
    } else {
      const u32x4 v = load_b128(rs, soff);
#pragma unroll
      for (int q = 0; q < 4; ++q) b.sc[q] = v[q];
    }
  };

  // staged activations of step s of the phase
  auto x_of = [&](const GemvCtx& c, int s) -> const half_t* { return xrow + ((c.start + s) * 4 * D + kq * D) * CH; };

  float4_t acc = float4_t{0.f, 0.f, 0.f, 0.f};

  // one super step of MFMAs on the staged activations at xp
  auto compute_super = [&](const GemvBuf<D, SPL>& b, const half_t* xp) {
    half8_t av[2][NJ];  // activations of chunk d+1 are read from LDS while chunk d is consumed
#pragma unroll
    for (int j = 0; j < NJ; ++j) av[0][j] = *reinterpret_cast<const half8_t*>(xp + j * 8);
#pragma unroll
    for (int d = 0; d < D; ++d) {
      if (d + 1 < D) {
#pragma unroll
        for (int j = 0; j < NJ; ++j)
          av[(d + 1) & 1][j] = *reinterpret_cast<const half8_t*>(xp + (d + 1) * CH + j * 8);
      }
      uint32_t sbits;
      if constexpr (SPL == 1) sbits = b.sc[0];
      else sbits = (d & 1) ? (b.sc[d >> 1] >> 16) : b.sc[d >> 1];
      const half2_t s2 = bcast_h2(__builtin_bit_cast(half_t, (uint16_t)sbits));
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        half8_t bm;
        if constexpr (BITS == 4) {
          half2_t h[4];
          q4_word_paired(b.w[d][j], s2, qc, h);
          bm = pack_h8(h[0], h[1], h[2], h[3]);
        } else {
          half2_t h0[2], h1[2];
          q8_word_natural(b.w[d][2 * j], s2, h0);
          q8_word_natural(b.w[d][2 * j + 1], s2, h1);
          bm = pack_h8(h0[0], h0[1], h1[0], h1[1]);
        }
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[d & 1][j], bm, acc, 0, 0, 0);
      }
    }
  };

  // adds the finished partial tile to this wavefront's private slot and clears it
  auto flush_tile = [&](int i, bool first_phase) {
    float* s = slots + ((size_t)(i * WAVES + wave) * 4) * 64 + lane;
#pragma unroll
    for (int r = 0; r < 4; ++r) s[r * 64] = first_phase ? acc[r] : s[r * 64] + acc[r];
    acc = float4_t{0.f, 0.f, 0.f, 0.f};
  };

  // The weight stream is one software pipeline over all K phases: the register set that a phase's last trip
  // frees is filled with the first item of the next phase, so that the phase boundary (a barrier, the
  // activations of the next K range into LDS, a barrier) does not find the memory pipeline empty.
  GemvBuf<D, SPL> b0, b1;
  // (the late arguments: fetched from the argument segment by fetch_late_arguments, see GemvKernArgs and below)
  half_t* y_ = nullptr;
  Epilogue ep_ = Epilogue{nullptr, nullptr, 0};
  float* partials_ = nullptr;
  unsigned int* counters_ = nullptr;
  u32x4 xn[XPRE ? 8 : 1];  // XPRE: this thread's column of the next phase's activations, requested a phase ahead

  auto permute_x = [&](u32x4 v) -> u32x4 {
    if constexpr (BITS == 4) {
      u32x4 p;
      p[0] = __builtin_amdgcn_perm(v[2], v[0], 0x05040100u);
      p[1] = __builtin_amdgcn_perm(v[2], v[0], 0x07060302u);
      p[2] = __builtin_amdgcn_perm(v[3], v[1], 0x05040100u);
      p[3] = __builtin_amdgcn_perm(v[3], v[1], 0x07060302u);
      return p;
    } else {
      return v;
    }
  };
  // 16-byte vector kv of activation row m in the phase that starts at chunk `chunk_base` (zeros past the
  // phase, the row or K), and its place in LDS
  auto x_load_of = [&](const GemvCtx& c, int m, int kv) -> u32x4 {
    const int kbase = c.chunk_base * CH;
    const int vec_per_row = ((c.nsuper * 4 * D + 3) / 4) * 4 * CH / 8;
    const bool ok = m < M && kv < vec_per_row && kbase + kv * 8 < K;
    return load_b128(rx, ok ? ((uint32_t)m * (uint32_t)K + (uint32_t)(kbase + kv * 8)) * 2u : kOobOffset);
  };
  auto x_store_of = [&](const GemvCtx& c, int m, int kv, u32x4 v) {
    const int vec_per_row = ((c.nsuper * 4 * D + 3) / 4) * 4 * CH / 8;
    if (m >= M || kv >= vec_per_row) return;
    *reinterpret_cast<u32x4*>(xs + (size_t)m * lds_stride + kv * 8) = permute_x(v);
  };

  auto fetch_late_arguments = [&]() {
    typedef const __attribute__((address_space(4))) GemvKernArgs* kernarg_ptr_t;
    kernarg_ptr_t late = (kernarg_ptr_t)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(late));
    y_ = late->y;
    ep_ = Epilogue{late->ep.bias, late->ep.residual, late->ep.activation};
    if constexpr (KSPLIT) {
      partials_ = late->partials;
      counters_ = late->counters;
    }
  };

  // Where the fetch goes.  The loads are plain loads from constant memory, which the compiler moves freely: placed
  // behind the first weight requests they sank below the first activation store, i.e. behind the wait for the
  // first activations, and the barrier that ends the staging then waited for a scalar load issued a memory trip
  // late (0.5 us per launch on a 4096 x 4096 projection at batch 1).  The builds that walk K in one phase have the
  // scalar registers to hold the seven values from the top of the kernel, so they fetch there, and an empty asm
  // ahead of the staging barrier names the values as inputs: the loads cannot sink past it, and that barrier's
  // wait for the LDS stores covers them.  The K-phase builds are short of scalar registers (a fetch at the top makes
  // them wait for it and spill the values ahead of their first request): they fetch behind their first requests.
  if constexpr (!PHASES) fetch_late_arguments();
  auto pin_late_arguments = [&]() {
    asm volatile("" ::"s"(y_), "s"(ep_.bias), "s"(ep_.residual), "s"(ep_.activation));
    if constexpr (KSPLIT) asm volatile("" ::"s"(partials_), "s"(counters_));
  };

  // One K phase: stage its activations, stream every tile of the workgroup over it.  The first phase
  // is a copy of its own ahead of the loop over the others: inside a loop the compiler hoists the
  // stream's constants in front of it, i.e. in front of the kernel's first requests.
  // b0_loaded: the previous phase's last trip has requested this phase's first item.
  auto run_phase = [&](const int ph, const GemvCtx& c, const GemvCtx& cn, const bool b0_loaded) {
    // ---- stage this phase's activations (zero padded to a whole k-step) ---------------
    // The first batch of vectors per thread is requested before the first weights and
    // stored after them: global loads retire in order, so the LDS fill does not wait
    // for the much slower first weight loads.
    const int vec_per_row = ((c.nsuper * 4 * D + 3) / 4) * 4 * CH / 8;
    if (ph == 0) {
      if constexpr (XS >= 1 && XS <= 3) {
        // exactly XS vectors per thread, rows of at least NT vectors (launch_one checks): vector q of this thread
        // is index tid + q * NT of the flat order, in row 0, 1 or 2
        static_assert(!PHASES && !KSPLIT, "one phase over all of K");
        // (the requests went out at the top of the kernel)
        load_super(b0, c, first_tile(c), 0);
        __builtin_amdgcn_sched_barrier(0);
        WQ_STAMP(1);
#pragma unroll
        for (int q = 0; q < XS; ++q) x_store_of(c, mq[q], kvq[q], xq[q]);
      } else if constexpr (!ROWS) {
        // one or two rows, or rows longer than the workgroup has threads: a flat index over (row, column),
        // up to three vectors per thread ahead of the weights -- as many as the activations have, each
        // further one under a wave-uniform branch.  (Every request, even one that is masked off, takes its
        // turn in the memory pipeline ahead of the first weights, and a request behind the first weights
        // comes back after them, a cold trip to HBM later: 4096 x 11008 at batch 1 has 2.7 vectors per
        // thread and waited 2.3 us for its activations with two ahead, 1.3 us with three.)
        const int total = M * vec_per_row;
        auto at = [&](int idx, int& m, int& kv) {
          m = idx / vec_per_row;
          kv = idx - m * vec_per_row;
        };
        // (the first vectors without the division when a row has at least as many vectors as the
        // workgroup has threads -- K >= 4096: they are in rows 0 to 2; the start-up of a 5 us kernel is
        // a few hundred instructions, and a division is forty of them)
        const bool wide = vec_per_row >= NT, second = total > NT, third = total > 2 * NT;
        int m0 = 0, kv0 = tid, m1 = 0, kv1 = 0, m2 = 0, kv2 = 0;
        if (!wide) at(tid, m0, kv0);
        const u32x4 x0 = x_load_of(c, m0, kv0);
        u32x4 x1 = u32x4{0u, 0u, 0u, 0u}, x2 = u32x4{0u, 0u, 0u, 0u};
        if (second) {
          if (wide) {
            m1 = tid + NT >= vec_per_row ? 1 : 0;
            kv1 = tid + NT - m1 * vec_per_row;
          } else {
            at(tid + NT, m1, kv1);
          }
          x1 = x_load_of(c, m1, kv1);
        }
        if (third) {
          if (wide) {
            m2 = (tid + 2 * NT >= vec_per_row ? 1 : 0) + (tid + 2 * NT >= 2 * vec_per_row ? 1 : 0);
            kv2 = tid + 2 * NT - m2 * vec_per_row;
          } else {
            at(tid + 2 * NT, m2, kv2);
          }
          x2 = x_load_of(c, m2, kv2);
        }
        __builtin_amdgcn_sched_barrier(0);
        load_super(b0, c, first_tile(c), 0);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (PHASES) fetch_late_arguments();
        WQ_STAMP(1);
        x_store_of(c, m0, kv0, x0);
        if (second) x_store_of(c, m1, kv1, x1);
        if (third) x_store_of(c, m2, kv2, x2);
        for (int idx = tid + 3 * NT; idx < total; idx += 4 * NT) {
          int ma, ka, mb, kb, mc, kc, md, kd;
          at(idx, ma, ka);
          at(idx + NT, mb, kb);
          at(idx + 2 * NT, mc, kc);
          at(idx + 3 * NT, md, kd);
          const u32x4 v0 = x_load_of(c, ma, ka), v1 = x_load_of(c, mb, kb), v2 = x_load_of(c, mc, kc),
                      v3 = x_load_of(c, md, kd);
          x_store_of(c, ma, ka, v0);
          x_store_of(c, mb, kb, v1);
          x_store_of(c, mc, kc, v2);
          x_store_of(c, md, kd, v3);
        }
      } else {
        // more rows, and a phase of at most one vector per thread and row (launch_one checks): a thread
        // stages its column of RM rows per batch.  No address needs a division (with the flat index the
        // divisions alone cost half a microsecond at eight rows), the RM requests of the first batch are
        // in flight together and all go out before the first weights.  (Measured alternatives, all
        // slower: part of the batch behind the weights -- it returns after them, i.e. after a cold trip
        // to HBM; sixteen in flight; requests under per-vector branches, which the wait-count
        // insertion serialises.)
        auto stage = [&](auto rmc) {
          constexpr int RM = decltype(rmc)::value;
          u32x4 xv[RM];
#pragma unroll
          for (int r = 0; r < RM; ++r) xv[r] = x_load_of(c, r, tid);
          __builtin_amdgcn_sched_barrier(0);
          load_super(b0, c, first_tile(c), 0);
          __builtin_amdgcn_sched_barrier(0);
          if constexpr (PHASES) fetch_late_arguments();
          WQ_STAMP(1);
#pragma unroll
          for (int r = 0; r < RM; ++r) x_store_of(c, r, tid, xv[r]);
          if constexpr (XS == 16) {  // rows 8 .. 15
#pragma unroll
            for (int r = 0; r < RM; ++r) xv[r] = x_load_of(c, RM + r, tid);
#pragma unroll
            for (int r = 0; r < RM; ++r) x_store_of(c, RM + r, tid, xv[r]);
          }
        };
        stage(std::integral_constant<int, XS == 4 ? 4 : 8>{});
      }
    } else {
      __syncthreads();  // every wavefront is done reading the previous phase
      auto restage_rows = [&]() {
        for (int m0 = 0; m0 < M; m0 += 8) {
          u32x4 xv[8];
#pragma unroll
          for (int r = 0; r < 8; ++r) xv[r] = x_load_of(c, m0 + r, tid);
#pragma unroll
          for (int r = 0; r < 8; ++r) x_store_of(c, m0 + r, tid, xv[r]);
        }
      };
      if constexpr (XPRE) {
        // (requested at the start of the previous phase: here long since)
#pragma unroll
        for (int r = 0; r < 8; ++r) x_store_of(c, r, tid, xn[r]);
      } else if constexpr (ROWS) {
        restage_rows();
      } else {
        const int total = M * vec_per_row;
        for (int idx = tid; idx < total; idx += 2 * NT) {
          const int ma = idx / vec_per_row, ka = idx - ma * vec_per_row;
          const int mb = (idx + NT) / vec_per_row, kb = idx + NT - mb * vec_per_row;
          const u32x4 v0 = x_load_of(c, ma, ka), v1 = x_load_of(c, mb, kb);
          x_store_of(c, ma, ka, v0);
          x_store_of(c, mb, kb, v1);
        }
      }
      if (!b0_loaded) load_super(b0, c, first_tile(c), 0);
    }
    if (ph == 0) pin_late_arguments();
    __syncthreads();
    if constexpr (XPRE) {
      // the next phase's column of this thread, behind the one item that is in flight
#pragma unroll
      for (int r = 0; r < 8; ++r) xn[r] = x_load_of(cn, r, tid);
      __builtin_amdgcn_sched_barrier(0);
    }

    if (ph == 0) WQ_STAMP(2);
    // ---- the weight stream: a flat software pipeline over (tile, super step) ----------
    // Two items per trip, unconditionally (with an early exit in between, the compiler
    // sinks the prefetch below the compute).  Items past the end load zeros from an
    // out-of-range offset and are not computed.
    const int items = my_tiles * c.cnt;
    int ci = first_tile(c), cs = 0;  // tile / step of the item being consumed
    int pi = ci, ps = 0;             // ... of the item being prefetched
    for (int j = 0; j < items; j += 2) {
      advance(c, pi, ps);
      load_super(b1, c, pi, ps);
      __builtin_amdgcn_sched_barrier(0);
      compute_super(b0, x_of(c, cs));
      if (ph == 0 && j == 0) WQ_STAMP(3);
      if (cs == c.cnt - 1) flush_tile(ci, ph == 0);
      advance(c, ci, cs);
      __builtin_amdgcn_sched_barrier(0);
      // the item after next, or behind the last trip the first item of the next phase
      advance(c, pi, ps);
      if constexpr (PHASES) {
        const bool wrap = j + 2 >= items;
        GemvCtx lc;
        lc.chunk_base = wrap ? cn.chunk_base : c.chunk_base;
        lc.nsuper = wrap ? cn.nsuper : c.nsuper;
        lc.start = wrap ? cn.start : c.start;
        lc.cnt = wrap ? cn.cnt : c.cnt;
        load_super(b0, lc, wrap ? first_tile(cn) : pi, wrap ? 0 : ps);
      } else {
        load_super(b0, c, pi, ps);  // (behind the last trip: no item, zeros)
      }
      __builtin_amdgcn_sched_barrier(0);
      if (ci < my_tiles) {
        compute_super(b1, x_of(c, cs));
        if (cs == c.cnt - 1) flush_tile(ci, ph == 0);
      }
      advance(c, ci, cs);
      __builtin_amdgcn_sched_barrier(0);
    }
    WQ_STAMP(4);
    // a wavefront without work in the first phase still owns slots that the epilogue sums
    if (ph == 0 && c.cnt == 0)
      for (int i = 0; i < my_tiles; ++i) flush_tile(i, true);
    return items > 0;
  };
  if constexpr (!PHASES) {
    run_phase(0, make_ctx(KSPLIT ? kr * phase_chunks_ : 0), dead_ctx, false);
  } else {
    GemvCtx c = phase_chunks_ < nchunks ? make_ctx(phase_chunks_) : dead_ctx;
    bool loaded = run_phase(0, make_ctx(0), c, false);
    for (int ph = 1; ph * phase_chunks_ < nchunks; ++ph) {
      const GemvCtx cn = (ph + 1) * phase_chunks_ < nchunks ? make_ctx((ph + 1) * phase_chunks_) : dead_ctx;
      loaded = run_phase(ph, c, cn, loaded);
      c = cn;
    }
  }

  // ---- sum the wavefronts' partial tiles, convert, store -----------------------------
  WQ_STAMP(5);
  __syncthreads();
  WQ_STAMP(6);
  if constexpr (!KSPLIT) {
    // (the plain store first and on its own: the tails' code -- erf, exp -- is then a block the common launch never
    // enters, instead of four stretches it jumps over on a cold instruction cache)
    const bool plain = !gated && ep_.bias == nullptr && ep_.residual == nullptr && ep_.activation == 0;
    for (int idx = tid; idx < my_tiles * 256; idx += NT) {
      const int i = idx >> 8, r = (idx >> 6) & 3, l = idx & 63;
      const int m = 4 * (l >> 4) + r;
      const int n = (tile0 + i * tstride) * tile_rows + (l & 15);
      if (m < M && n < N && (l & 15) < tile_rows) {
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) sum += slots[((size_t)(i * WAVES + w) * 4 + r) * 64 + l];
        if (plain) {
          y_[(size_t)m * N + n] = (half_t)sum;
        } else if (gated) {
          // adjacent columns of the tile hold a gate / up pair: the even lane also sums its neighbour's
          if ((l & 1) == 0 && n + 1 < N) {
            float up = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) up += slots[((size_t)(i * WAVES + w) * 4 + r) * 64 + l + 1];
            store_gated(y_, m, n >> 1, N >> 1, sum, up);
          }
        } else {
          store_out(ep_, y_, m, n, N, sum);
        }
      }
    }
  } else {
    // K split over R workgroups: every workgroup writes its float32 partial tile (1 KB) to the
    // workspace and counts itself in; the one that finds R - 1 others counted adds the R partials in
    // the order of their K windows -- whoever arrives last, the sum is the same -- applies the
    // epilogue, stores, and returns the counter to zero for the next launch.  Nobody waits for anybody.
    //
    // Ordering.  In the language's memory model the count would be a release (and, for the workgroup
    // that arrives last, an acquire) at agent scope.  On this part both are cache-wide operations -- a
    // write-back and an invalidate of a whole L2 -- and were measured: with acquire-release on the one
    // counter add per workgroup a launch takes 2.8 - 4.9 us longer (4096 x 11008 at 8 rows: 11.3 -> 14.1 us,
    // 5120 x 13824 int8 at batch 1: 18.0 -> 22.9 us), more than the split saves.  The exchange therefore
    // relies on what the hardware guarantees for the accesses it actually makes:
    // Visibility across the chip's eight L2s without cache-wide fences (a device-scope fence writes
    // back and invalidates a whole L2; one per wavefront cost 65 us per launch): the partial tiles and
    // the counters are only ever touched by device-scope atomic stores, loads and adds, which are
    // performed at the memory side of the L2s; a workgroup's stores have completed (vmcnt(0)) before
    // the barrier after which its count goes out.
    // What would break it: one plain (non-atomic, or workgroup-scope) load or store of a partial or a counter
    // word, in this kernel or any other that shares the workspace -- it may be served from a stale line of the
    // reader's L2 or stay dirty in the writer's.  A source-level test refuses such an access.
    for (int idx = tid; idx < my_tiles * 256; idx += NT) {
      const int i = idx >> 8, r = (idx >> 6) & 3, l = idx & 63;
      float sum = 0.f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) sum += slots[((size_t)(i * WAVES + w) * 4 + r) * 64 + l];
      __hip_atomic_store(&partials_[((size_t)(tile0 + i * tstride) * R + kr) * 256 + (idx & 255)], sum,
                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    int* const last = reinterpret_cast<int*>(slots);  // (the slots have been read)
    if (tid < my_tiles)
      last[tid] = __hip_atomic_fetch_add(&counters_[tile0 + tid * tstride], 1u, __ATOMIC_RELAXED,
                                         __HIP_MEMORY_SCOPE_AGENT) == (unsigned)(R - 1);
    __syncthreads();
    for (int idx = tid; idx < my_tiles * 256; idx += NT) {
      const int i = idx >> 8, r = (idx >> 6) & 3, l = idx & 63;
      if (!last[i]) continue;
      const int m = 4 * (l >> 4) + r;
      const int n = (tile0 + i * tstride) * tile_rows + (l & 15);  // (the split runs on 16-row tiles)
      float* const part = partials_ + (size_t)(tile0 + i * tstride) * R * 256 + (idx & 255);
      float sum = 0.f;
      for (int q = 0; q < R; ++q) sum += __hip_atomic_load(part + q * 256, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (m < M && n < N) store_out(ep_, y_, m, n, N, sum);
    }
    __syncthreads();
    if (tid < my_tiles && last[tid])
      __hip_atomic_store(&counters_[tile0 + tid * tstride], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
#ifdef WQ_GEMV_STAMPS
  // (the plain builds do not use ksplit_: the measurement build's launcher passes a launch counter there)
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  WQ_STAMP(7);
  if (!KSPLIT && lane == 0 && (int)blockIdx.x * WAVES + wave < kStampWaves) {
    unsigned long long* t =
        g_gemv_stamps + ((size_t)(ksplit_ & (kStampLaunches - 1)) * kStampWaves + (size_t)blockIdx.x * WAVES + wave) * kStampPoints;
    for (int q = 0; q < kStampPoints; ++q) t[q] = stamps_[q];
  }
#endif
}

namespace {

constexpr size_t kLdsPerCu = 160 * 1024;
constexpr int64_t kSplitMaxTiles = 4096;                 // row tiles a K split handles (N <= 65536)
constexpr int64_t kSplitCounterBytes = kSplitMaxTiles * 4;  // head of the workspace
constexpr size_t kLdsPerWgMax = 159 * 1024;  // of the 160 KB a workgroup can address

struct Plan {
  int grid, max_tiles, phase_chunks, lds_stride;
  size_t lds_bytes;
  int tile_rows = 16;  // weight rows per tile
};

// Rows per tile for N rows on `cap` CUs.  With 16-row tiles a tile count just above a multiple of the CUs leaves most of
// them idle for a whole tile (5120 rows: 320 tiles on 256 CUs -- 64 walk two tiles, 192 one); shorter tiles even that
// out (512 tiles of 10 rows: two each) at the price of load instructions whose lanes past the tile's rows request
// nothing.  Cost of a choice: tiles per CU x (rows + 4) -- a tile costs its bytes plus about four rows' worth of
// per-tile work -- and a shorter tile must win by an eighth.  Measured (us, 16 rows -> the rule's choice): int8
// 5120 x 5120 at 1 / 16 rows 8.80 -> 7.92 / 12.41 -> 11.22, 5120 x 13824 19.44 -> 16.68 / 26.14 -> 24.09, int4
// 5120 x 5120 6.31 -> 5.98; what counts is the balance over CUs, not over workgroups: 12288 rows on two workgroups
// per CU (768 tiles: two for one workgroup, one for the other, three per CU) lose with 12-row tiles (7.36 -> 8.28).
// `forced` (8 .. 16) overrides the rule.
inline int pick_tile_rows(int64_t n, int cap, int forced) {
  if (forced >= 8 && forced <= 16) return forced;
  auto cost = [&](int tr) {
    const int64_t tiles = (n + tr - 1) / tr, grid = std::min<int64_t>(tiles, cap);
    return ((tiles + grid - 1) / grid) * (tr + 4);
  };
  int best = 16;
  int64_t best_cost = cost(16);
  for (int tr = 15; tr >= 8; --tr)
    if (cost(tr) < best_cost) best = tr, best_cost = cost(tr);
  return best_cost * 8 <= cost(16) * 7 ? best : 16;
}

// Chooses the grid (workgroups per CU), the tiles per workgroup and the K phase so
// that partial-tile slots + staged activations fit in LDS.
template <int BITS, int WAVES, int D>
bool make_plan(const Problem& p, int wgs_per_cu, Plan* out, int tile_rows = 0) {
  constexpr int ch = 128 / BITS;
  // (tile-major weights are laid out in 16-row tiles, and the gated tail pairs adjacent columns of one)
  const int tr = (p.tiled || p.activation == kActGated) ? 16 : pick_tile_rows(p.n, cu_count(), tile_rows);
  const int tiles = (int)((p.n + tr - 1) / tr);
  const int nchunks = (int)(p.k / ch);
  const size_t budget = std::min(kLdsPerWgMax, kLdsPerCu / (size_t)wgs_per_cu - 1024);
  const int grid = std::min(tiles, cu_count() * wgs_per_cu);
  const int max_tiles = (tiles + grid - 1) / grid;
  const size_t slot_bytes = (size_t)max_tiles * WAVES * 1024;
  if (slot_bytes + 4096 > budget) return false;
  // largest phase in chunks: a multiple of 4*D*WAVES, so every wavefront gets whole super steps
  const size_t x_budget = budget - slot_bytes;
  const int unit = 4 * D * WAVES;
  const int64_t max_k = (int64_t)(x_budget / (2 * (size_t)p.m)) - 8;
  int phase_chunks = (int)(max_k / ch) / unit * unit;
  if (phase_chunks <= 0) return false;
  const int whole = (nchunks + 4 * D - 1) / (4 * D) * (4 * D);  // K as one phase, padded to a super step
  if (phase_chunks >= whole) {
    phase_chunks = whole;
  } else if (p.m > 2) {
    // K is walked in phases anyway: phases of equal length, and of at most one 16-byte vector per
    // thread and row where that costs at most one phase more, so that the staging takes the
    // column-per-thread path
    const int per_vec = WAVES * 64 * 8 / ch;  // chunks whose vectors one pass of the workgroup covers
    int nph = (nchunks + phase_chunks - 1) / phase_chunks;
    const int capped = per_vec / unit * unit;
    if (capped > 0 && (nchunks + capped - 1) / capped <= nph + 1) nph = (nchunks + capped - 1) / capped;
    phase_chunks = std::min(phase_chunks, ((nchunks + nph - 1) / nph + unit - 1) / unit * unit);
  }
  out->grid = grid;
  out->max_tiles = max_tiles;
  out->tile_rows = tr;
  out->phase_chunks = phase_chunks;
  out->lds_stride = phase_chunks * ch + 8;  // +16 bytes: consecutive rows start 4 banks apart
  out->lds_bytes = slot_bytes + (size_t)p.m * out->lds_stride * sizeof(half_t);
  return out->lds_bytes <= budget;
}

// Launch results of the helpers below: the variant does not fit the problem (try another),
// the kernel was launched, or a runtime call failed (error already set).
enum { kNotApplicable = 0, kLaunched = 1, kFailed = -1 };

#ifdef WQ_GEMV_STAMPS
int g_stamp_launches = 0;  // launches since the last reset: selects the slot a launch records into
#endif

// the kernel's ksplit argument (the measurement build numbers the plain launches there instead)
inline int stamp_slot_or(int ksplit, bool split_build) {
#ifdef WQ_GEMV_STAMPS
  if (!split_build) return g_stamp_launches++;
#endif
  (void)split_build;
  return ksplit;
}

template <int BITS, int WAVES, int D, int SPL, bool TILED = false, bool KSPLIT = false>
int launch_one(const Problem& p, int group_shift, const Plan& plan, int ksplit = 1, void* workspace = nullptr) {
  const Epilogue ep{(const half_t*)p.bias, (const half_t*)p.residual, p.activation};
  // workspace of the K split: kSplitMaxTiles arrival counters at a fixed place -- a workspace shared by
  // projections of different shapes keeps them apart from the partial tiles, whose leftovers are not
  // zero -- then [tiles][ksplit][256] float partial tiles
  unsigned int* const counters = static_cast<unsigned int*>(workspace);
  float* const partials = reinterpret_cast<float*>(static_cast<char*>(workspace) + kSplitCounterBytes);
  // the builds of the kernel: by the way the activations are staged (the kernel's XS) and by whether K is walked in
  // several phases
  auto go = [&](auto xs, auto phases) -> int {
    constexpr int XS = decltype(xs)::value;
    constexpr bool PHASES = decltype(phases)::value;
    static std::atomic<bool> lds_ok[kMaxDevices];
    if (!ensure_dynamic_lds((const void*)wq_gemv_kernel<BITS, WAVES, D, SPL, TILED, XS, KSPLIT, PHASES>, (int)kLdsPerWgMax,
                            lds_ok))
      return kFailed;
    hipLaunchKernelGGL((wq_gemv_kernel<BITS, WAVES, D, SPL, TILED, XS, KSPLIT, PHASES>), dim3(plan.grid), dim3(WAVES * 64),
                       plan.lds_bytes, p.stream, (const half_t*)p.x, (const uint32_t*)p.wq, (const half_t*)p.scales,
                       (int)p.m, (int)p.n, (int)p.k,
                       group_shift | (p.zero_point << 8) | (p.activation == kActGated ? 1 << 16 : 0) | (plan.tile_rows << 20),
                       plan.max_tiles, plan.phase_chunks, stamp_slot_or(ksplit, KSPLIT), plan.grid, (half_t*)p.y, ep,
                       partials, counters);
    return kLaunched;
  };
  using std::integral_constant;
  constexpr int ch = 128 / BITS, NT = WAVES * 64;
  const int phase_vectors = (plan.phase_chunks + 3) / 4 * 4 * ch / 8;  // 16-byte vectors per staged row
  const bool flat = p.m <= 2 || phase_vectors > NT;
  const bool phases = !KSPLIT && (int64_t)plan.phase_chunks * ch < p.k;
  auto with_phases = [&](auto xs) -> int {
    if constexpr (KSPLIT) return go(xs, std::false_type{});
    else return phases ? go(xs, std::true_type{}) : go(xs, std::false_type{});
  };
  if (!flat) {
    if (p.m <= 4) return with_phases(integral_constant<int, 4>{});
    return p.m <= 8 ? with_phases(integral_constant<int, 8>{}) : with_phases(integral_constant<int, 16>{});
  }
  if constexpr (!KSPLIT && WAVES == 8) {
    // (the default shapes only: every exact build is a kernel more)
    const int64_t total = p.m * (int64_t)phase_vectors;
    if (!phases && phase_vectors >= NT && total <= 3 * NT) {
      if (total <= NT) return go(integral_constant<int, 1>{}, std::false_type{});
      if (total <= 2 * NT) return go(integral_constant<int, 2>{}, std::false_type{});
      return go(integral_constant<int, 3>{}, std::false_type{});
    }
  }
  return with_phases(integral_constant<int, 0>{});
}

// D chunks per lane need K to be a multiple of 4*D chunks, and the lane's D
// chunks to share one scale (SPL = 1) or to have one each (SPL = D).
template <int BITS, int WAVES, int D>
int try_launch(const Problem& p, int group_shift, int wgs_per_cu, int tile_rows) {
  constexpr int ch = 128 / BITS;
  if (D > 1 && p.k % (4 * D * ch) != 0) return kNotApplicable;
  Plan plan;
  if (!make_plan<BITS, WAVES, D>(p, wgs_per_cu, &plan, tile_rows)) return kNotApplicable;
  if (p.tiled) {
    // only the layout's own shape: super steps of eight chunks, scales per chunk (int4 / group 32)
    // or per super step (int8 / group 128)
    if constexpr (D == 2) {
      if (BITS == 4 && group_shift == 0) return launch_one<BITS, WAVES, 2, 2, true>(p, group_shift, plan);
      if (BITS == 8 && group_shift == 3) return launch_one<BITS, WAVES, 2, 1, true>(p, group_shift, plan);
    }
    return kNotApplicable;
  }
  if (group_shift == 0) return launch_one<BITS, WAVES, D, D>(p, group_shift, plan);
  if ((1 << group_shift) >= D) return launch_one<BITS, WAVES, D, 1>(p, group_shift, plan);
  return kNotApplicable;
}

// variant = 100 * rows-per-tile (0: the rule's choice, else 8 .. 16) + 10 * workgroups-per-CU + shape index
template <int BITS>
int dispatch(const Problem& p, int gs, int variant) {
  const int tr = variant / 100, wpc = variant % 100 / 10, shape = variant % 10;
  if (wpc < 1 || wpc > 8 || (tr != 0 && (tr < 8 || tr > 16))) return kNotApplicable;
  if (tr != 0 && tr != 16 && (p.tiled || p.activation == kActGated)) return kNotApplicable;
  switch (shape) {
    case 1: return try_launch<BITS, 4, 1>(p, gs, wpc, tr);
    case 2: return try_launch<BITS, 4, 2>(p, gs, wpc, tr);
    case 3: return try_launch<BITS, 4, 4>(p, gs, wpc, tr);
    case 4: return try_launch<BITS, 8, 1>(p, gs, wpc, tr);
    case 5: return try_launch<BITS, 8, 2>(p, gs, wpc, tr);
    case 6: return try_launch<BITS, 8, 4>(p, gs, wpc, tr);
    case 7: return try_launch<BITS, 16, 1>(p, gs, wpc, tr);
    case 8: return try_launch<BITS, 16, 2>(p, gs, wpc, tr);
    default: return kNotApplicable;
  }
}

}  // namespace

namespace {

// The variants the default dispatch tries, in order (see launch_gemv).
const int* default_order(const Problem& p) {
  // Measured on MI355X (Llama-2-7B and 13B shapes): one or two rows of int4 weights run best with two
  // 8-wave workgroups per CU (4096 x 11008 at batch 1: 8.7 against 9.3 us), everything else with one
  // (12288 x 4096 at 4 rows: 8.7 against 9.0 us; int8 15360 x 5120 at batch 1: 18.2 against 19.6 us).
  // Two-chunk super steps first, single chunks (any K) as the fallback.
  static const int small[] = {25, 15, 24, 14}, large[] = {15, 14, 15, 14};
  // (between one and two row tiles per CU a second workgroup per CU only unbalances them:
  // 5120 x 5120, 9.9 against 8.7 us)
  const int64_t tiles = (p.n + 15) / 16;
  const bool fills = tiles <= cu_count() || tiles >= 2 * cu_count();
  return (p.m <= 2 && p.bits == 4 && fills) ? small : large;
}

// Whether `variant` can be launched for p: K divisibility and an LDS plan (partial-tile slots of
// the tiles a workgroup owns + staged activations).  Mirrors dispatch() without launching.
template <int BITS>
bool variant_has_plan(const Problem& p, int gs, int variant) {
  const int wpc = variant / 10, shape = variant % 10;
  constexpr int ch = 128 / BITS;
  const int waves = shape <= 3 ? 4 : (shape <= 6 ? 8 : 16);
  const int d = shape <= 6 ? (1 << ((shape - 1) % 3)) : (shape == 7 ? 1 : 2);
  if (wpc < 1 || wpc > 8 || shape < 1 || shape > 8) return false;
  if (d > 1 && p.k % (4 * d * ch) != 0) return false;
  if (gs != 0 && (1 << gs) < d) return false;
  Plan plan;
  switch (waves * 10 + d) {
    case 41: return make_plan<BITS, 4, 1>(p, wpc, &plan);
    case 42: return make_plan<BITS, 4, 2>(p, wpc, &plan);
    case 44: return make_plan<BITS, 4, 4>(p, wpc, &plan);
    case 81: return make_plan<BITS, 8, 1>(p, wpc, &plan);
    case 82: return make_plan<BITS, 8, 2>(p, wpc, &plan);
    case 84: return make_plan<BITS, 8, 4>(p, wpc, &plan);
    case 161: return make_plan<BITS, 16, 1>(p, wpc, &plan);
    case 162: return make_plan<BITS, 16, 2>(p, wpc, &plan);
    default: return false;
  }
}

}  // namespace

// M <= 16 and one of the default variants fits: with very many row tiles per workgroup (N in the
// hundreds of thousands) the per-tile partial-sum slots outgrow LDS and the caller falls back to
// the register-activation kernel.
bool gemv_applicable(const Problem& p) {
  if (p.m < 1 || p.m > 16) return false;
  const int ch = 128 / p.bits;
  int ratio = p.group / ch, gs = 0;
  while ((1 << gs) < ratio) ++gs;
  if (ratio < 1 || (1 << gs) != ratio) return false;
  const int* order = default_order(p);
  for (int q = 0; q < 4; ++q) {
    const int shape = order[q] % 10;
    if (p.tiled && shape != 2 && shape != 5 && shape != 8) continue;  // tile-major: two-chunk super steps only
    if (p.bits == 4 ? variant_has_plan<4>(p, gs, order[q]) : variant_has_plan<8>(p, gs, order[q])) return true;
  }
  return false;
}

int launch_gemv(const Problem& p, int variant) {
  const int ch = 128 / p.bits;
  int ratio = p.group / ch, gs = 0;
  while ((1 << gs) < ratio) ++gs;
  if (ratio < 1 || (1 << gs) != ratio || p.group % ch != 0) {
    set_error("gemv kernel: group %d must be %d times a power of two", p.group, ch);
    return -1;
  }
  if (p.m < 1 || p.m > 16) {
    set_error("gemv kernel: M=%lld is outside 1..16", (long long)p.m);
    return -1;
  }
  int ok = kNotApplicable;
  if (variant == 0) {
    const int* order = default_order(p);
    for (int q = 0; q < 4; ++q) {
      const int v = order[q];
      ok = p.bits == 4 ? dispatch<4>(p, gs, v) : dispatch<8>(p, gs, v);
      if (ok != kNotApplicable) break;
    }
  } else {
    ok = p.bits == 4 ? dispatch<4>(p, gs, variant) : dispatch<8>(p, gs, variant);
  }
  if (ok == kFailed) return -1;
  if (ok == kNotApplicable) {
    set_error("gemv kernel: variant %d does not apply to M=%lld K=%lld group=%d", variant,
              (long long)p.m, (long long)p.k, p.group);
    return -1;
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("gemv kernel launch failed: %s", hipGetErrorString(e));
    return -1;
  }
  return 0;
}

namespace {

// Cross-workgroup K split of the 8-wavefront, two-chunk kernel (one workgroup per CU).
constexpr int kSplitWaves = 8, kSplitD = 2, kSplitMaxR = 4;

struct SplitPlan {
  int r = 1;
  Plan plan;
  int64_t workspace_bytes = 0;
};

// LDS plan for `r` K windows, or false.  *path = the longest chain of super steps a wavefront walks.
template <int BITS>
bool split_plan_for(const Problem& p, int r, Plan* out, int64_t* path) {
  constexpr int ch = 128 / BITS;
  const int tiles = (int)((p.n + 15) / 16);
  const int nsuper = (int)(p.k / ch) / (4 * kSplitD);
  const int groups = std::min(tiles, std::max(1, cu_count() / r));  // tile lists, each shared by r workgroups
  const int max_tiles = (tiles + groups - 1) / groups;
  const int window = (nsuper + r - 1) / r;  // super steps per K window
  if (window < 1 || (int64_t)(r - 1) * window >= nsuper) return false;
  const size_t slot_bytes = (size_t)max_tiles * kSplitWaves * 1024;
  const int lds_stride = window * 4 * kSplitD * ch + 8;
  const size_t lds_bytes = slot_bytes + (size_t)p.m * lds_stride * sizeof(half_t);
  if (lds_bytes > kLdsPerWgMax) return false;
  out->grid = groups * r;
  out->max_tiles = max_tiles;
  out->phase_chunks = window * 4 * kSplitD;
  out->lds_stride = lds_stride;
  out->lds_bytes = lds_bytes;
  *path = (int64_t)max_tiles * ((window + kSplitWaves - 1) / kSplitWaves);
  return true;
}

// Whether, and how many ways, to split K across workgroups.  What the split buys was measured on MI355X
// by timing problems of the same bytes with K cut and N multiplied: a shorter critical path where the
// tile count leaves CUs idle for whole rounds (5120 rows = 320 tiles on 256 CUs), and less activation
// staging where one tile per CU makes every workgroup stage all of a large x.  What it costs: the last
// workgroup's chain of three trips to the memory side of the L2s (partials out, count, partials in),
// 2 - 3 us.  A super step of a wavefront takes about 0.7 us, so the split must save at least five of
// them on the critical path (5120 x 13824 int8 on 16-row tiles: 28 -> 20 super steps; 22.7 -> 19.8 us at 8 rows,
// 24.1 -> 21.3 us at 16 -- at up to 5 rows, where the activations fit the LDS in one piece, the plain call's 10-row
// tiles do better, 16.7 against 18.4 us at batch 1), or spare a problem with one tile per CU the K phases that activations beyond the LDS
// need (4096 x 11008 int4: 12.9 -> 11.8 us at 10 rows, 13.9 -> 12.9 us at 16, int8 17.4 -> 13.8 us at 8 rows; int4
// at up to 8 rows not: there the phases run with the next phase's activations requested a phase ahead, 10.3
// against 11.1 us).  On tile-major weights
// the register-activation kernel already covers the small batches of these shapes: there only from
// 12 rows on.  Measured and excluded: 4096 x 4096 at 8 - 16 rows (5.7 -> 7.3 us), 5120 x 5120 (10.4 -> 12.1 us).
template <int BITS>
bool choose_split(const Problem& p, int gs, SplitPlan* out) {
  constexpr int ch = 128 / BITS;
  if (p.m < 1 || p.m > 16 || p.k % (4 * kSplitD * ch) != 0) return false;
  if (p.tiled ? !((BITS == 4 && gs == 0) || (BITS == 8 && gs == 3)) : !(gs == 0 || (1 << gs) >= kSplitD)) return false;
  if (p.tiled && p.m < 12) return false;
  const int64_t tiles = (p.n + 15) / 16, cu = cu_count();
  if (tiles > kSplitMaxTiles) return false;
  const int nsuper = (int)(p.k / ch) / (4 * kSplitD);
  // (paths in twentieths of a 16-row super step: the plain call may run shorter tiles, pick_tile_rows, whose super
  // steps cost (rows + 4) / 20 of a 16-row one -- while its activations fit the LDS in one piece; the split's tiles
  // have 16 rows)
  const bool gated = p.activation == kActGated;
  const int tr = (p.tiled || gated || (int64_t)p.m * p.k * 2 + 16384 > (int64_t)kLdsPerWgMax) ? 16 : pick_tile_rows(p.n, (int)cu, 0);
  const int64_t tiles1 = (p.n + tr - 1) / tr;
  const int64_t path1 = ((tiles1 + std::min(tiles1, cu) - 1) / std::min(tiles1, cu)) * ((nsuper + kSplitWaves - 1) / kSplitWaves) * (tr + 4);
  int best = 1;
  int64_t best_path = path1;
  Plan best_plan{};
  for (int r = 2; r <= kSplitMaxR; ++r) {
    Plan plan;
    int64_t path;
    if (!split_plan_for<BITS>(p, r, &plan, &path)) continue;
    if (path * 20 < best_path) {
      best = r;
      best_path = path * 20;
      best_plan = plan;
    }
  }
  if (best == 1 || path1 - best_path < 5 * 20) {
    best = 1;
    if (p.m * p.k * 2 > 160 * 1024 && tiles <= cu && !(BITS == 4 && p.m <= 8)) {
      // the fewest windows whose activations fit, each wavefront keeping at least one super step
      for (int r = 2; r <= kSplitMaxR && best == 1; ++r) {
        Plan plan;
        int64_t path;
        if ((nsuper + r - 1) / r >= kSplitWaves && split_plan_for<BITS>(p, r, &plan, &path)) {
          best = r;
          best_plan = plan;
        }
      }
    }
  }
  if (best == 1) return false;
  out->r = best;
  out->plan = best_plan;
  out->workspace_bytes = kSplitCounterBytes + tiles * best * 1024;
  return true;
}

bool choose_split_any(const Problem& p, SplitPlan* out, int* gs_out) {
  const int ch = 128 / p.bits;
  int ratio = p.group / ch, gs = 0;
  while ((1 << gs) < ratio) ++gs;
  if (ratio < 1 || (1 << gs) != ratio || p.group % ch != 0) return false;
  *gs_out = gs;
  return p.bits == 4 ? choose_split<4>(p, gs, out) : choose_split<8>(p, gs, out);
}

}  // namespace

int64_t gemv_split_workspace_bytes(const Problem& p) {
  SplitPlan sp;
  int gs;
  return choose_split_any(p, &sp, &gs) ? sp.workspace_bytes : 0;
}

// 1 = launched with the K split, 0 = the split does not apply or the workspace is too small (nothing
// launched), -1 = failure
int launch_gemv_split(const Problem& p, void* workspace, int64_t workspace_bytes) {
  SplitPlan sp;
  int gs;
  if (!choose_split_any(p, &sp, &gs) || workspace == nullptr || workspace_bytes < sp.workspace_bytes) return 0;
  int ok;
  if (p.bits == 4) {
    if (p.tiled) ok = launch_one<4, kSplitWaves, kSplitD, 2, true, true>(p, gs, sp.plan, sp.r, workspace);
    else if (gs == 0) ok = launch_one<4, kSplitWaves, kSplitD, kSplitD, false, true>(p, gs, sp.plan, sp.r, workspace);
    else ok = launch_one<4, kSplitWaves, kSplitD, 1, false, true>(p, gs, sp.plan, sp.r, workspace);
  } else {
    if (p.tiled) ok = launch_one<8, kSplitWaves, kSplitD, 1, true, true>(p, gs, sp.plan, sp.r, workspace);
    else if (gs == 0) ok = launch_one<8, kSplitWaves, kSplitD, kSplitD, false, true>(p, gs, sp.plan, sp.r, workspace);
    else ok = launch_one<8, kSplitWaves, kSplitD, 1, false, true>(p, gs, sp.plan, sp.r, workspace);
  }
  if (ok != kLaunched) return -1;
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("gemv kernel (K split) launch failed: %s", hipGetErrorString(e));
    return -1;
  }
  return 1;
}

// ---- the K split on memory the library owns: an entry point that allocates nothing -------------------
// For callers that cannot allocate (code under HIP graph capture, serving loops, harnesses that forbid
// hipMalloc): the partial tiles and arrival counters of the K split live in a file-scope device array
// instead of a caller workspace.  Every GPU the library runs on holds its own copy of the array, at its
// own address, until the process ends; the host-side name `scratch` is only a handle for
// hipGetSymbolAddress, never an address a kernel may use.  The address is looked up once per device
// (with that device current) and kept; kernels receive it as an argument, exactly as they receive a
// caller's workspace.  The array starts zeroed (device variables are zero-initialised when the code
// object is loaded) and every launch returns its counters to zero, so consecutive calls need no
// clearing; partial tiles are written before they are read.  All calls on one GPU share the array:
// calls that overlap in time on one GPU (different streams, different threads) race.
static __device__ __align__(256) unsigned char scratch[kSplitCounterBytes + 4 * 1024 * 1024];

namespace {

constexpr int64_t kStaticScratchBytes = kSplitCounterBytes + 4 * 1024 * 1024;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

// Device address of the current device's copy of `scratch`, or nullptr with the error set.
void* static_scratch_address() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0) {
    (void)hipGetLastError();
    set_error("no usable HIP device in this process");
    return nullptr;
  }
  const bool cached = dev < kMaxDevices;  // beyond the table: looked up on every call
  if (cached) {
    void* known = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (known != nullptr) return known;
  }
  void* ptr = nullptr;
  const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
  if (e != hipSuccess || ptr == nullptr) {
    (void)hipGetLastError();
    set_error("cannot resolve the library's scratch array on device %d: %s", dev, hipGetErrorString(e));
    return nullptr;
  }
  if (cached) g_scratch_ptr[dev].store(ptr, std::memory_order_release);
  return ptr;
}

}  // namespace

int64_t gemv_static_scratch_bytes() { return kStaticScratchBytes; }

// 1 = launched with the K split on the library's scratch array, 0 = the split does not apply to `p`
// (nothing launched), -1 = failure: the split would need more than the array holds, or a runtime error
int launch_gemv_split_static(const Problem& p) {
  const int64_t need = gemv_split_workspace_bytes(p);
  if (need == 0) return 0;
  if (need > kStaticScratchBytes) {
    set_error("the K split of this problem needs %lld bytes of scratch memory, the library's own array holds %lld: "
              "use mi355x_wq_matmul_ws with a caller workspace", (long long)need, (long long)kStaticScratchBytes);
    return -1;
  }
  void* const ptr = static_scratch_address();
  if (ptr == nullptr) return -1;
  return launch_gemv_split(p, ptr, kStaticScratchBytes);
}

}  // namespace wq

#ifdef WQ_GEMV_STAMPS
// The measurement build's two exports: copy the stamp array to the host (n values), clear it and restart the launch count.
extern "C" __attribute__((visibility("default"))) int mi355x_wq_stamps_read(unsigned long long* host, int n) {
  if (n < 0 || n > wq::kStampLaunches * wq::kStampWaves * wq::kStampPoints) return -1;
  return hipMemcpyFromSymbol(host, HIP_SYMBOL(wq::g_gemv_stamps), (size_t)n * 8) == hipSuccess ? 0 : -1;
}
extern "C" __attribute__((visibility("default"))) int mi355x_wq_stamps_reset() {
  void* p = nullptr;
  if (hipGetSymbolAddress(&p, HIP_SYMBOL(wq::g_gemv_stamps)) != hipSuccess) return -1;
  wq::g_stamp_launches = 0;
  return hipMemset(p, 0, sizeof(unsigned long long) * wq::kStampLaunches * wq::kStampWaves * wq::kStampPoints) == hipSuccess ? 0 : -1;
}
#endif
