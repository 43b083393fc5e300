// Register-staged fp16 GEMM kernel: global -> registers -> LDS -> MFMA.
// Handles every tile shape and the SwiGLU A operand (which needs arithmetic on
// the way into LDS).  See gemm_kernel_dma.h for the variant that moves tiles
// into LDS without passing through registers.
#pragma once

#include "gemm_common.h"

namespace cusync {
namespace gemm {

template<int BM_, int BN_, int BK_, int WM_, int WN_>
struct TileCfg {
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_;
  static constexpr int THREADS = kThreads;
  static constexpr int WTM = BM / WM, WTN = BN / WN;       // wavefront tile
  static constexpr int TM = WTM / 32, TN = WTN / 32;       // MFMA tiles per wavefront
  static constexpr int PA = BK + 8;                         // LDS row pitch of A in halfs (16 B pad)
  static constexpr int PB = BN + 32;                        // LDS row pitch of B in halfs (64 B pad)
  static constexpr int A_HALFS = BM * PA, B_HALFS = BK * PB;
  static constexpr int CA = BM * BK / 8 / kThreads;         // 16-byte chunks of A per thread per K chunk
  static constexpr int CB = BK * BN / 8 / kThreads;
  static constexpr int LDS_BYTES = 2 * (A_HALFS + B_HALFS) * 2;   // two stages
  static_assert(WM * WN == 4, "four wavefronts per workgroup");
  static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wavefront tile is made of 32x32 MFMA tiles");
  static_assert(BM * BK / 8 % kThreads == 0 && BK * BN / 8 % kThreads == 0, "whole chunks per thread");
  static_assert(BK % 16 == 0, "MFMA consumes 16 k per step");
  static_assert(LDS_BYTES <= 160 * 1024, "fits the LDS of one CU");
};

// Software pipeline over K, three chunks deep, one barrier per chunk:
//   iteration kt:  issue global loads of chunk kt+2 into register set kt%2
//                  MFMA on LDS stage kt%2, interleaved with
//                  moving register set (kt+1)%2 into LDS stage (kt+1)%2
//                  barrier
// A global load therefore has one whole iteration of MFMA work to complete
// before anything depends on it.
template<class C, bool SWIGLU>
__global__ __launch_bounds__(kThreads) void gemmKernel(GemmParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  __shared__ uint32_t sTicket, sLast;
  half_t* const sA = reinterpret_cast<half_t*>(smem);
  half_t* const sB = sA + 2 * C::A_HALFS;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / C::WN, wn = wave % C::WN;
  const cusync::DynStage& stage = p.stage;
  constexpr bool swiglu = SWIGLU;

  const __amdgpu_buffer_rsrc_t rA = makeRsrc(p.A, p.M * p.lda * 2);
  const __amdgpu_buffer_rsrc_t rB = makeRsrc(p.B, p.K * p.ldb * 2);

  // Chunk i of a thread is chunk (tid + i*256) of the tile: consecutive lanes take
  // consecutive 16-byte pieces of a row, so a row of the tile is one contiguous run.
  constexpr int A_PER_ROW = C::BK / 8, B_PER_ROW = C::BN / 8;
  constexpr int A_ROW_STEP = kThreads / A_PER_ROW, B_ROW_STEP = kThreads / B_PER_ROW;
  static_assert(kThreads % A_PER_ROW == 0 && kThreads % B_PER_ROW == 0, "row-aligned chunk steps");
  const uint32_t aRow0 = tid / A_PER_ROW, aKc = (tid % A_PER_ROW) * 8;
  const uint32_t bRow0 = tid / B_PER_ROW, bNc = (tid % B_PER_ROW) * 8;

  // LDS addresses of this lane's MFMA fragments inside a stage.
  const int aFragOff = (wm * C::WTM + (lane & 31)) * C::PA + 8 * (lane >> 5);
  const int bFragOff = (8 * (lane >> 5) + ((lane & 15) >> 2)) * C::PB + wn * C::WTN + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

  const uint32_t numTiles = stage.numTiles();
  const bool consumer = stage.isConsumer();
  const uint32_t tmq = consumer ? stage.d.in.tileM : 1, tnq = consumer ? stage.d.in.tileN : 1;
  // Policies that synchronise once per row of tiles (RowSync, ConsecutiveSync) are
  // handled entirely by the pre-loop wait; only the others wait per K chunk.
  const bool chunkSync = consumer && stage.d.in.kind != CUSYNC_POLICY_ROWSYNC &&
                         stage.d.in.kind != CUSYNC_POLICY_CONSECUTIVESYNC;

  // Thread 0 keeps the ticket state: the start count is issued first and settled after the
  // first tile's loads are under way; the draw of the next ticket is issued while a tile is
  // being computed and settled when the tile is done.
  uint32_t dryXcds = 0, nextRaw = 0;
  const uint32_t startToken = tid == 0 ? stage.beginStart() : 0;
  const bool noDraws = stage.noDraws;     // every tile is some workgroup's static first tile
  for (uint32_t round = 0;; round++) {
    if (tid == 0) sTicket = round == 0 ? stage.firstTicket(p.launched, dryXcds, noDraws) : stage.drawFinish(nextRaw, p.launched, round, dryXcds, noDraws);
    __syncthreads();
    const uint32_t ticket = sTicket;
    if (ticket >= numTiles) {
      if (tid == 0 && round == 0) stage.finishStart(startToken, p.launched);
      break;
    }
    const cusync_dim3 t = stage.ticketToTile(ticket);      // x = column tile, y = row tile
    const uint32_t m0 = t.y * C::BM, n0 = t.x * C::BN;
    const uint32_t mEnd = min(m0 + (uint32_t)C::BM, p.M);
    // K range of this slice, in chunks of BK counted from kBegin
    const uint32_t kBegin = t.z * p.kPerSlice, kEnd = min(p.K, kBegin + p.kPerSlice);
    const uint32_t nk = (kEnd - kBegin + C::BK - 1) / C::BK;

    floatx16 acc[C::TM][C::TN];
#pragma unroll
    for (int i = 0; i < C::TM; i++)
#pragma unroll
      for (int j = 0; j < C::TN; j++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    // Two register sets for chunks in flight.
    uint4v gA[2][C::CA], gA2[2][SWIGLU ? C::CA : 1], gB[2][C::CB];
#pragma unroll
    for (int s = 0; s < 2; s++) {
#pragma unroll
      for (int i = 0; i < C::CA; i++) { gA[s][i] = uint4v{0, 0, 0, 0}; if constexpr (swiglu) gA2[s][i] = uint4v{0, 0, 0, 0}; }
#pragma unroll
      for (int i = 0; i < C::CB; i++) gB[s][i] = uint4v{0, 0, 0, 0};
    }

    // ---- consumer side: rows [m0, mEnd) of A are the producer's output ------
    // Wait for every producer tile a K chunk touches before its loads are issued.
    // The semaphore of the next column tile is polled one iteration early (the
    // load returns while MFMAs run), so in steady state no wave ever stalls on a
    // poll; only a tile that is really not there yet makes the wave spin.
    uint32_t nextColTile = kBegin / tnq;   // producer column tiles below this one have been waited for (or are not needed)
    uint32_t nextColTileUp = swiglu ? (p.K + kBegin) / tnq : 0;
    (void)nextColTileUp;
    const bool oneRowBlock = chunkSync && (m0 / tmq == (mEnd - 1) / tmq);
    uint32_t polledTile = 0xffffffffu, polledValue = 0;
    auto waitRows = [&](uint32_t col, uint32_t z) {
      for (uint32_t r = m0; r < mEnd; r = (r / tmq + 1) * tmq) {
        cusync_dim3 w = {r, col, z};
        stage.waitWave(w);
      }
    };
    auto waitColTile = [&](uint32_t ct) {
      if (oneRowBlock && ct == polledTile) {
        cusync_dim3 w = {m0, ct * tnq, 0};
        if (!stage.needsWait(w)) return;
        if (cusync::dev::pollFinish(polledValue) >= stage.waitTarget()) {
          // The early poll was a relaxed load: it still needs the acquire a wait ends with.  Where a
          // producer tile is not a whole number of cache lines of A (a pitch or a base that is not a
          // multiple of 128 bytes) a line can straddle a posted and an unposted tile and sit in this
          // XCD's caches already; only the agent-scope acquire drops it.
          if (stage.lineAligned) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
          else cusync::dev::acquireFence();
          return;
        }
      }
      waitRows(ct * tnq, 0);
    };
    auto waitChunk = [&](uint32_t k0) {
      if (!chunkSync) return;
      const uint32_t kLast = min(k0 + (uint32_t)C::BK, kEnd) - 1;
      for (; nextColTile <= kLast / tnq; nextColTile++) waitColTile(nextColTile);
      if constexpr (swiglu) {
        // The up half lies K columns to the right.  StridedSync folds it onto the
        // gate half's semaphore (which then counts to 2); any other policy guards
        // those columns with semaphores of their own.
        if (stage.d.in.kind != CUSYNC_POLICY_STRIDEDSYNC)
          for (; nextColTileUp <= (p.K + kLast) / tnq; nextColTileUp++) waitRows(nextColTileUp * tnq, 0);
      }
    };
    auto earlyPoll = [&](uint32_t k0) {      // k0: first column of a chunk whose loads come one iteration later
      if (!oneRowBlock || k0 >= kEnd) return;
      const uint32_t ct = k0 / tnq;
      if (ct < nextColTile || ct == polledTile) return;
      cusync_dim3 w = {m0, ct * tnq, 0};
      if (!stage.needsWait(w)) return;
      polledTile = ct;
      polledValue = stage.peekBegin(w);
    };

    auto issue = [&](auto P, uint32_t kt) {
      constexpr int S = decltype(P)::value;
      const uint32_t k0 = kBegin + kt * C::BK;
      // weights first: they need no wait
#pragma unroll
      for (int i = 0; i < C::CB; i++) {
        const uint32_t n = n0 + bNc;
        const uint32_t off = n < p.N ? ((k0 + bRow0 + i * B_ROW_STEP) * p.ldb + n) * 2 : kOutOfRange;
        gB[S][i] = loadChunk(rB, off);
      }
      waitChunk(k0);
#pragma unroll
      for (int i = 0; i < C::CA; i++) {
        const uint32_t k = k0 + aKc;
        const uint32_t off = k < p.K ? ((m0 + aRow0 + i * A_ROW_STEP) * p.lda + k) * 2 : kOutOfRange;
        gA[S][i] = loadChunk(rA, off);
        if constexpr (swiglu) gA2[S][i] = loadChunk(rA, off == kOutOfRange ? off : off + p.K * 2);
      }
    };
    auto stash = [&](auto P) {
      constexpr int S = decltype(P)::value;
      half_t* a = sA + S * C::A_HALFS;
      half_t* b = sB + S * C::B_HALFS;
#pragma unroll
      for (int i = 0; i < C::CA; i++) {
        uint4v v = gA[S][i];
        if constexpr (swiglu) v = swigluChunk(gA[S][i], gA2[S][i]);
        *reinterpret_cast<uint4v*>(a + (aRow0 + i * A_ROW_STEP) * C::PA + aKc) = v;
      }
#pragma unroll
      for (int i = 0; i < C::CB; i++)
        *reinterpret_cast<uint4v*>(b + (bRow0 + i * B_ROW_STEP) * C::PB + bNc) = gB[S][i];
    };
    // MFMA pass over LDS stage P, with register set P^1 moved into stage P^1 on the way.
    auto computeAndStash = [&](auto P) {
      constexpr int S = decltype(P)::value;
      const half_t* a = sA + S * C::A_HALFS + aFragOff;
      const half_t* b = sB + S * C::B_HALFS + bFragOff;
      // Fragments are double-buffered in registers: the LDS reads of k-step kk+1
      // are in flight while the MFMAs of k-step kk execute.
      half8 fa[2][C::TM], fb[2][C::TN];
      auto loadFrags = [&](int slot, int kk) {
#pragma unroll
        for (int i = 0; i < C::TM; i++)
          fa[slot][i] = *reinterpret_cast<const half8*>(a + i * 32 * C::PA + kk * 16);
#pragma unroll
        for (int j = 0; j < C::TN; j++) {
          typedef short4v __attribute__((address_space(3))) * lds_ptr;
          const half_t* q = b + kk * 16 * C::PB + j * 32;
          short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(q));
          short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(q + 4 * C::PB));
          half4 l4 = __builtin_bit_cast(half4, lo), h4 = __builtin_bit_cast(half4, hi);
          fb[slot][j] = __builtin_shufflevector(l4, h4, 0, 1, 2, 3, 4, 5, 6, 7);
        }
      };
      constexpr int KS = C::BK / 16;
      loadFrags(0, 0);
#pragma unroll
      for (int kk = 0; kk < KS; kk++) {
        if (kk + 1 < KS) loadFrags((kk + 1) & 1, kk + 1);
        if (kk == KS / 2) stash(Parity<S ^ 1>{});
#pragma unroll
        for (int i = 0; i < C::TM; i++)
#pragma unroll
          for (int j = 0; j < C::TN; j++)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[kk & 1][j], fa[kk & 1][i], acc[i][j], 0, 0, 0);
      }
      schedPass<KS, C::TM * C::TN, C::TM + 2 * C::TN, C::CA + C::CB>();
    };
    auto step = [&](auto P, uint32_t kt) {
      if (kt + 2 < nk) issue(P, kt + 2);
      earlyPoll(kBegin + (kt + 3) * C::BK);
      __builtin_amdgcn_sched_barrier(0);
      computeAndStash(P);
      __builtin_amdgcn_sched_barrier(0);
      __syncthreads();
    };

    // Pre-loop wait (policies that synchronise once per row of tiles).  It can
    // last as long as the producer runs, so a single wave polls for the
    // workgroup and the others sleep at the barrier.
    if (consumer) {
      cusync_dim3 w = {m0, 0, 1};
      if (stage.needsWait(w)) {
        if (wave == 0) waitRows(0, 1);
        __syncthreads();
      }
    }

    issue(Parity<0>{}, 0);
    if (nk > 1) issue(Parity<1>{}, 1);
    if (tid == 0 && round == 0) stage.finishStart(startToken, p.launched);
    earlyPoll(kBegin + 2 * C::BK);
    stash(Parity<0>{});
    __syncthreads();

    for (uint32_t kt = 0; kt < nk; kt += 2) {
      step(Parity<0>{}, kt);
      if (kt + 1 < nk) step(Parity<1>{}, kt + 1);
    }

    if (tid == 0) nextRaw = stage.drawBegin(dryXcds, noDraws);     // settled after the epilogue
    const bool completed = finishTile<C>(p, acc, t, wm, wn, lane, &sLast, smem);
    cusync_dim3 done = {m0, outputColumn(p, n0), t.z};
    // the post's barrier (or this one) keeps the next tile's LDS writes behind the epilogue's LDS reads
    if (completed && stage.isProducer()) stage.post(done, postsPerTile(p), stage.storesThrough());
    else __syncthreads();
  }
}

}  // namespace gemm
}  // namespace cusync
