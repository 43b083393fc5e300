// fp16 GEMM kernel whose A and B tiles go from global memory straight into LDS
// (buffer_load ... lds, 16 bytes per lane) without passing through registers.
//
// Why: on gfx950 an LDS write issued by a wave (ds_write_b128) costs about 50
// clocks of that wave's LDS issue time, and with the MFMA rate doubled over
// CDNA3 the LDS is the scarce unit.  The direct loads take the write half of the
// LDS traffic off the waves and free the registers a staged copy needs, which
// is what makes a 256x256 tile (256 accumulator registers per lane) fit.
//
// Layout.  A direct load writes one contiguous 1 KiB run of LDS per wave
// instruction, lane l at byte 16*l, so rows cannot be padded.  Bank conflicts
// are avoided by permuting WHICH 16-byte chunk of global memory each lane
// fetches instead (an XOR swizzle):
//   A stage  [BM rows][BK halfs]:   chunk c of row r lives at slot c ^ swzA(r)
//   B stage  [BK rows][BN halfs]:   chunk c of row k lives at slot c ^ 4*(k&1)
// so that the eight lanes the LDS serves together (A fragments: eight rows;
// B transpose reads: four k rows x 64 bytes) fall on distinct bank groups.
// (With BK = 32 the swizzle of A is (r / 4) % 4, see A_SWZ_DIV below.)
//
// Pipeline.  STAGES LDS stages; iteration kt waits for its own chunk
// (s_waitcnt vmcnt), passes one barrier, issues the loads of chunk kt+STAGES-1
// into the stage the previous iteration finished with, and runs the MFMAs of
// chunk kt.  The loads are inline assembly on purpose: the compiler would
// otherwise wait for every outstanding direct load before any LDS read, which
// removes the overlap between prefetch and compute.
//
// Pipelined order (DmaCfg::PIPE, for workgroups that have a CU to themselves and
// so nobody to fill their bubbles).  In the order above the first fragments of a
// chunk can only be read after the barrier, and all wavefronts read them at the
// same moment: the matrix pipes idle for an LDS round trip per chunk.  Here the
// barrier sits between the two k-steps of chunk kt and already covers chunk
// kt+1, so that the fragments of (kt+1, k-step 0) are read under the MFMAs of
// (kt, k-step 1); the loads of chunk kt+STAGES-1 go into the stage of chunk kt-1.
//
// Assembly order (DmaCfg::PINGPONG, the 256x384x32 and 256x192x64 tiles: up to 192 accumulator registers per lane
// leave the compiler no room to schedule a loop around them).  What binds these GEMMs is data moved per MFMA: bytes
// from L2 into LDS through the CU's one vector memory path, which holds a bounded number of requests at once (so both
// operands are fetched in whole 128-byte lines, A 64 columns of K at a time), bytes from LDS into registers, and
// the power both cost; the tile is as large as the register file allows and has its CU to itself.  The K loop is
// one asm statement written by gen_wide_steps.py (gemm_wide_steps.inc): all eight wavefronts run the same stream,
// two per SIMD, so that one wavefront's waits fall under its partner's MFMAs; the fragments of k-step s+1 are read
// from LDS progressively under the MFMAs of step s, every MFMA waiting for its own operands only; one barrier per
// chunk, placed behind the first MFMAs of the preceding chunk's last k-step; the direct loads of the chunks two and
// three ahead are issued between the MFMAs.  (An earlier form ran the wavefronts as two groups half a k-step out of
// phase; the single stream measured 4 % faster.)  A tile-policy consumer waits for all its producer tiles before the
// first load: the loop has no place for a poll.
#pragma once

#include "gemm_tiles.h"

namespace cusync {
namespace gemm {

template<int BM_, int BN_, int BK_, int WM_, int WN_, int STAGES_, int WAVES_PER_SIMD_ = 1, bool BT_ = false, bool PIPE_ = false, bool PINGPONG_ = false>
struct DmaCfg {
  static constexpr bool PIPE = PIPE_;                      // barrier in the middle of a chunk, fragments prefetched across chunks
  static constexpr bool PINGPONG = PINGPONG_;              // K loop in assembly, operands in whole cache lines (see above)
  static constexpr bool BT = BT_;                          // B given as [N][K] (k contiguous), e.g. KRSC filters
  static constexpr int WAVES_PER_SIMD = WAVES_PER_SIMD_;   // register budget: 512 / this per lane
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_, STAGES = STAGES_;
  static constexpr int WTM = BM / WM, WTN = BN / WN;
  static constexpr int TM = WTM / 32, TN = WTN / 32;
  static constexpr int KS = BK / 16;                        // MFMA k-steps per chunk
  static constexpr int A_ROW_BYTES = BK * 2, B_ROW_BYTES = BT ? BK * 2 : BN * 2;
  static constexpr int B_ROWS = BT ? BN : BK;
  static constexpr int A_CPR = A_ROW_BYTES / 16, B_CPR = B_ROW_BYTES / 16;   // 16-byte chunks per row
  static constexpr int A_STAGE = BM * A_ROW_BYTES, B_STAGE = B_ROWS * B_ROW_BYTES;
  static constexpr int WAVES = WM * WN, THREADS = WAVES * 64;
  // 1 KiB wave loads per chunk.  When B's do not divide among the waves the spare ones of the last waves
  // go out of range into a 1 KiB dump behind the stages, so that every wave counts the same loads per chunk.
  static constexpr int A_TOTAL = A_STAGE / 1024, B_TOTAL = B_STAGE / 1024;
  static constexpr int A_LOADS = A_TOTAL / WAVES, B_LOADS = (B_TOTAL + WAVES - 1) / WAVES;   // per wave per chunk
  static constexpr int LOADS = A_LOADS + B_LOADS;
  static constexpr int A_ROWS_PER_LOAD = 1024 / A_ROW_BYTES;
  static constexpr bool DUMP = B_TOTAL % WAVES != 0;
  static constexpr int DUMP_OFFSET = STAGES * (A_STAGE + B_STAGE);
  // Beyond the pipeline stages: what a k-slice keeps in LDS while the slices of a tile add it up together (the
  // epilogue's buffer plus the fp32 partial sums of half a tile, the share of one of two slices), as far as the
  // workgroup's share of the CU's LDS goes (1 KiB left for the static variables).
  static constexpr int LDS_SHARE = 160 * 1024 / (WAVES_PER_SIMD * 4 / WAVES > 0 ? WAVES_PER_SIMD * 4 / WAVES : 1) - 1024;
  static constexpr int REDUCE_BYTES = (WM * 32 * (BN * 2 + 16) + 1023) / 1024 * 1024 + (BM / 2) * BN * 4;
  static constexpr int PIPE_BYTES = DUMP_OFFSET + (DUMP ? 1024 : 0);
  static constexpr int LDS_BYTES = PIPE_BYTES > LDS_SHARE ? PIPE_BYTES : REDUCE_BYTES < PIPE_BYTES ? PIPE_BYTES : REDUCE_BYTES < LDS_SHARE ? REDUCE_BYTES : LDS_SHARE;
  static_assert(WAVES == 4 || WAVES == 8, "four or eight wavefronts per workgroup");
  static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wavefront tile is made of 32x32 MFMA tiles");
  static_assert(A_CPR == 4 || A_CPR == 8, "BK is 32 or 64");
  static_assert(BT || B_CPR % 8 == 0, "a B row covers whole 128-byte bank sweeps");
  static_assert(BT || WTN % 32 == 0, "MFMA tiles of B start on 64-byte groups");
  static_assert(A_TOTAL % WAVES == 0 && B_STAGE % 1024 == 0, "whole 1 KiB loads per wave");
  static_assert(LDS_BYTES * (WAVES_PER_SIMD * 4 / WAVES) <= 160 * 1024, "fits the LDS of one CU");
  static_assert((STAGES - 1) * LOADS < 64, "outstanding loads fit the vmcnt counter");
  static_assert(KS >= 2, "the loads of the next chunk ride on the LDS reads of k-step 1");
  static_assert(!PIPE || (KS == 2 && STAGES >= 3), "the pipelined order is written for two k-steps per chunk");
  static_assert(!PINGPONG || (WAVES == 8 && !PIPE && !BT && BM == 256 && ((BN == 384 && BK == 32) || (BN == 192 && BK == 64))), "the assembly K loops are written for two tiles");
};

// One direct load: 64 lanes x 16 bytes from buffer `rsrc` at per-lane byte offset
// `voff` into LDS at ldsAddr + 16*lane.  ldsAddr must be wave-uniform.
__device__ __forceinline__ void loadToLds(uint4v rsrc, uint32_t ldsAddr, uint32_t voff) {
  asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
               :: "s"(ldsAddr), "v"(voff), "s"(rsrc) : "memory");
}

// The same for the lower 32 lanes only (512 bytes); the wavefront must be fully active around it.
__device__ __forceinline__ void loadToLdsLowerHalf(uint4v rsrc, uint32_t ldsAddr, uint32_t voff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_mov_b64 exec, 0xffffffff\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds\n\ts_mov_b64 exec, -1"
               :: "s"(ldsAddr), "v"(voff), "s"(rsrc) : "memory");
}

template<int N>
__device__ __forceinline__ void waitVmcnt() { asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory"); }

__device__ __forceinline__ uint4v rawRsrc(const void* base, uint32_t bytes) {
  const uint64_t a = (uint64_t)base;
  uint4v r;
  r.x = __builtin_amdgcn_readfirstlane((uint32_t)a);
  r.y = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32) & 0xffffu);
  r.z = __builtin_amdgcn_readfirstlane(bytes);
  r.w = 0x00020000u;
  return r;
}

// What the assembly K loop of the 256x384x32 tile works on (gemm_wide_steps.inc, written by gen_wide_steps.py): LDS
// addresses of this lane's fragments, byte offsets of its direct loads at K = 0, the operands' descriptors and the
// LDS addresses its wavefront's loads of stage 0 go to.
struct WideOperands {
  uint32_t vA, vB[3];     // LDS: this lane's A fragment (slot 0, first k-step, first row tile) and its three B fragments (stage 0)
  uint32_t a[4], b[3];    // byte offsets of this lane's direct loads at the first column of the tile's K range
  uint4v rA, rB;
  uint32_t m0A, m0B;      // LDS addresses this wavefront's loads of slot / stage 0 go to
  uint32_t dB;            // bytes from one chunk's rows of B to the next chunk's
};
#include "gemm_wide_steps.inc"

// One GEMM: all tiles of stage p.stage that this workgroup draws.  CHUNKS: the stage may be a consumer that waits
// K chunk by K chunk (the tile policies); without it that code is not compiled in (gemm_tiles.h says for which
// tiles that is worth a kernel of its own).
//
// ROUNDS: a GEMM's chunk waits are made once per round of the pipeline (STAGES chunks ahead) instead of once per
// chunk.  The wait's code is inlined where it is called; per chunk that is nine copies of it in the kernel, per
// round two, and the TileSync consumer of the 2048-row MLP is 13 us (2 %) faster for it.  The kernel of several
// GEMMs in one launch keeps the waits per chunk: compiled the other way the 512-row chain, where one launch is the
// best mode, took 212 instead of 208 us (and 222 instead of 212 while the k-slices' reduction was still unrolled
// and the kernel parked ten more registers per lane in scratch for it); it would gain at 2048 rows, 595 -> 588 us,
// where the two launches are ahead anyway.
template<class C, int AMODE, bool CHUNKS, bool ROUNDS>
__device__ __forceinline__ void gemmDmaTiles(const GemmParams& p) {
  constexpr bool conv = AMODE == kAConv;
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  __shared__ uint32_t sTicket, sLast;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / C::WN, wn = wave % C::WN;
  const cusync::DynStage& stage = p.stage;

  const uint4v rA = rawRsrc(p.A, conv ? p.cvN * p.cvH * p.cvW * p.cvC * 2 : p.M * p.lda * 2);
  const uint4v rB = rawRsrc(p.B, (C::BT ? p.N : p.K) * p.ldb * 2);
  const uint32_t ldsBase = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem;

  const uint32_t numTiles = stage.numTiles();
  const bool consumer = stage.isConsumer();
  const uint32_t tmq = consumer ? stage.d.in.tileM : 1, tnq = consumer ? stage.d.in.tileN : 1;
  const bool chunkSync = CHUNKS && consumer && stage.d.in.kind != CUSYNC_POLICY_ROWSYNC &&
                         stage.d.in.kind != CUSYNC_POLICY_CONSECUTIVESYNC;

  // Thread 0 keeps the ticket state: the start count is issued first and settled after the
  // first tile's loads are under way; the draw of the next ticket is issued while a tile is
  // being computed and settled when the tile is done.
  uint32_t dryXcds = 0, nextRaw = 0;
  const unsigned long long tlEntry = p.timeline ? wall_clock64() : 0;
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
    const cusync_dim3 t = stage.ticketToTile(ticket);
    const unsigned long long tl0 = p.timeline ? wall_clock64() : 0;
    const uint32_t m0 = t.y * C::BM, n0 = t.x * C::BN;
    const uint32_t mEnd = min(m0 + (uint32_t)C::BM, p.M);
    const uint32_t kBegin = t.z * p.kPerSlice, kEnd = min(p.K, kBegin + p.kPerSlice);
    const uint32_t nk = (kEnd - kBegin + C::BK - 1) / C::BK;

    // Where this lane's loads and fragments sit.  Worked out per tile from a lane id the compiler cannot see
    // through where the tile's accumulators fill the register file (PINGPONG): it would otherwise keep these
    // fifteen values alive across the main loop for the next tile and reload others from scratch inside it.
    int laneL = lane;
    if constexpr (C::PINGPONG) asm volatile("" : "+v"(laneL));
    // ---- direct-load side: which global chunk this lane fetches ---------------
    // A: load q of this wave fills rows (wave*A_LOADS + q)*A_ROWS_PER_LOAD + lane/A_CPR, slot lane%A_CPR.
    // Rows that share a swizzle value.  A 16-byte-per-lane LDS read is served sixteen lanes at a time over all 64
    // banks: with 64-byte rows the sixteen rows of such a group cover every bank four times over, so rows r, r+4, r+8
    // and r+12 must sit in four different slots (four rows per swizzle value: 5.5 clocks per wave instruction on one
    // CU against 8.0 with two rows per value).
    constexpr int A_SWZ_DIV = C::A_CPR == 4 ? 4 : C::PINGPONG ? 2 : 1;      // (128-byte rows: two rows cover all banks once)
    const uint32_t aLoadRow = wave * C::A_LOADS * C::A_ROWS_PER_LOAD + laneL / C::A_CPR;
    const uint32_t aLoadChunk = (laneL % C::A_CPR) ^ ((aLoadRow / A_SWZ_DIV) & (C::A_CPR - 1));
    // B: the 16-byte slots of a stage are numbered row by row; load q of this wave fills slots
    // (wave*B_LOADS + q)*64 + lane, i.e. row slot / B_CPR, position slot % B_CPR (a row need not be a
    // power of two long: 192 columns are 24 slots).  With B given k-contiguous ([N][K]) its stage is laid
    // out and swizzled exactly like A's.
    uint32_t bLoadRow[C::B_LOADS], bLoadChunk[C::B_LOADS];
#pragma unroll
    for (int q = 0; q < C::B_LOADS; q++) {
      const uint32_t slot = (wave * C::B_LOADS + q) * 64 + laneL;
      bLoadRow[q] = slot / C::B_CPR;                 // >= B_ROWS for a spare load
      const uint32_t pos = slot % C::B_CPR;
      bLoadChunk[q] = C::BT ? pos ^ ((bLoadRow[q] / A_SWZ_DIV) & (C::B_CPR - 1)) : pos ^ (4 * (bLoadRow[q] & 1));
    }
    static_assert(C::PINGPONG || C::A_ROWS_PER_LOAD % (A_SWZ_DIV * C::A_CPR) == 0, "swizzle repeats per load");      // (the assembly loops set their loads up themselves)

    // ---- fragment side: where this lane's MFMA operands sit inside a stage -----
    // A fragment of k-step kk: row (lane&31) of the 32-row MFMA tile, chunk 2*kk + lane/32.
    uint32_t aFrag[C::KS];
    {
      const uint32_t row = wm * C::WTM + (laneL & 31);
      const uint32_t swz = (row / A_SWZ_DIV) & (C::A_CPR - 1);
#pragma unroll
      for (int kk = 0; kk < C::KS; kk++)
        aFrag[kk] = row * C::A_ROW_BYTES + (((2 * kk + (laneL >> 5)) ^ swz) * 16);
    }
    // B fragment: transpose read of rows kk*16 + 8*(lane/32) + 4*t + (lane&15)/4,
    // 4 halfs at column wn*WTN + j*32 + 16*((lane/16)&1) + 4*(lane&3).
    // A stage row is kept as 64-byte groups; the group of MFMA tile j is swapped with its neighbour on odd rows.
    const uint32_t bFlip = (laneL >> 2) & 1;                      // parity of the row this lane reads
    const uint32_t bRowOff = (8 * (laneL >> 5) + ((laneL & 15) >> 2)) * C::B_ROW_BYTES;
    const uint32_t bInGroup = (2 * ((laneL >> 4) & 1) + ((laneL & 3) >> 1)) * 16 + (laneL & 1) * 8;
    uint32_t bFrag[C::TN];
#pragma unroll
    for (int j = 0; j < C::TN; j++) bFrag[j] = bRowOff + (((wn * C::TN + j) ^ bFlip) * 64) + bInGroup;
    // k-contiguous B: same addressing as the A fragment, rows are output columns.
    uint32_t bFragT[C::KS];
    {
      const uint32_t row = wn * C::WTN + (laneL & 31);
      const uint32_t swz = (row / A_SWZ_DIV) & (C::A_CPR - 1);
#pragma unroll
      for (int kk = 0; kk < C::KS; kk++)
        bFragT[kk] = row * C::A_ROW_BYTES + (((2 * kk + (laneL >> 5)) ^ swz) * 16);
    }

    floatx16 acc[C::TM][C::TN];
#pragma unroll
    for (int i = 0; i < C::TM; i++)
#pragma unroll
      for (int j = 0; j < C::TN; j++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    // Per-tile byte offsets of this lane's loads at k0 = 0.
    const uint32_t aVoff0 = ((m0 + aLoadRow) * p.lda + aLoadChunk * 8) * 2;
    const uint32_t aVstep = C::A_ROWS_PER_LOAD * p.lda * 2;
    // B offsets at k0 = 0; columns (or, k-contiguous, rows) outside the matrix are sent out of range.
    uint32_t bVoff0[C::B_LOADS];
#pragma unroll
    for (int q = 0; q < C::B_LOADS; q++) {
      if constexpr (C::BT) bVoff0[q] = bLoadRow[q] < C::B_ROWS ? ((n0 + bLoadRow[q]) * p.ldb + bLoadChunk[q] * 8) * 2 : kOutOfRange;     // rows past N fall outside the buffer
      else bVoff0[q] = (bLoadRow[q] < C::B_ROWS && n0 + bLoadChunk[q] * 8 < p.N) ? (bLoadRow[q] * p.ldb + n0 + bLoadChunk[q] * 8) * 2 : kOutOfRange;
    }

    // Convolution: the pixel each of this lane's A rows stands for.
    int32_t cvIh0[C::A_LOADS], cvIw0[C::A_LOADS];
    uint32_t cvBase[C::A_LOADS];
    if constexpr (conv) {
#pragma unroll
      for (int q = 0; q < C::A_LOADS; q++) {
        const uint32_t m = m0 + aLoadRow + q * C::A_ROWS_PER_LOAD;
        const uint32_t img = m / (p.cvP * p.cvQ), rem = m % (p.cvP * p.cvQ);
        cvIh0[q] = (int32_t)((rem / p.cvQ) * p.cvStride) - (int32_t)p.cvPad;
        cvIw0[q] = (int32_t)((rem % p.cvQ) * p.cvStride) - (int32_t)p.cvPad;
        cvBase[q] = m < p.M ? img * p.cvH * p.cvW * p.cvC : kOutOfRange / 2;
      }
    }

    // ---- consumer side (same protocol as the staged kernel) ------------------
    uint32_t nextColTile = (kBegin & ~(p.waitRound - 1)) / tnq;     // the first chunk's line may begin in the tile before
    const bool oneRowBlock = chunkSync && (m0 / tmq == (mEnd - 1) / tmq);
    uint32_t readyEnd = 0;        // column tiles of the producer below this one are known to be posted (for all row blocks of this tile)
    auto waitRows = [&](uint32_t col, uint32_t z) { stage.waitWaveRows(m0, mEnd - 1, tmq, col, z); };
    // Convolution fed by another convolution: the rows of the producer's output
    // this tile reads are its own pixels plus the filter's halo, and a K chunk
    // (r, s, c0..) lies in the producer's column tile c0 / tileN.  Each column
    // tile is waited for once, for the whole halo range.
    uint32_t cvSeen = 0;
    auto cvRowRange = [&](uint32_t& lo, uint32_t& hi) {
      auto pixelRow = [&](uint32_t m) {
        const uint32_t img = m / (p.cvP * p.cvQ), rem = m % (p.cvP * p.cvQ);
        return (img * p.cvH + (rem / p.cvQ) * p.cvStride) * p.cvW + (rem % p.cvQ) * p.cvStride;
      };
      const uint32_t before = p.cvPad * p.cvW + p.cvPad, after = (p.cvR - 1 - p.cvPad) * p.cvW + (p.cvS - 1 - p.cvPad);
      const uint32_t first = pixelRow(m0), last = pixelRow(mEnd - 1) + after;
      lo = first > before ? first - before : 0;
      hi = min(last, p.cvN * p.cvH * p.cvW - 1);
    };
    auto cvWaitRows = [&](uint32_t policyCol, uint32_t z) {
      uint32_t lo, hi;
      cvRowRange(lo, hi);
      stage.waitWaveRows(lo, hi, tmq, policyCol, z);
    };
    auto waitChunk = [&](uint32_t k0) {
      if constexpr (!CHUNKS) return;
      if (!chunkSync) return;
      if constexpr (conv) {
        const uint32_t ct = (k0 % p.cvC) / tnq;
        if (cvSeen & (1u << ct)) return;
        cvSeen |= 1u << ct;
        // Conv2DTileSync divides the K tile index by R*S to get the channel tile
        cvWaitRows(stage.d.in.kind == CUSYNC_POLICY_CONV2DTILESYNC ? ct * p.cvR * p.cvS * tnq : ct * tnq, 0);
        return;
      }
      // last column whose producer tile must be there: the chunk's last column, or (waitRound) the last column
      // of the 128-byte line it lies in
      const uint32_t kLast = min((min(k0 + (uint32_t)C::BK, kEnd) - 1) | (p.waitRound - 1), p.K - 1);
      for (; nextColTile <= kLast / tnq; nextColTile++) {
        if (nextColTile < readyEnd) continue;            // seen posted by an earlier look-ahead
        const uint32_t left = max(kEnd - 1, kLast) / tnq - nextColTile + 1;      // column tiles this slice still has to see
        if (oneRowBlock) readyEnd = nextColTile + stage.waitWaveAhead(m0, nextColTile * tnq, tnq, left);
        else readyEnd = nextColTile + stage.waitWaveAheadRows(m0, mEnd - 1, tmq, nextColTile * tnq, tnq, left);
      }
    };

    // Direct load number q (B loads first, then A) of chunk kt into stage S.
    // Columns / rows outside the operands or past the end of this K slice are
    // redirected out of range and land in LDS as zeros, so chunks past the end
    // may be issued harmlessly.
    auto issueOne = [&](auto SP, auto QP, uint32_t kt) {
      constexpr int S = decltype(SP)::value;
      constexpr int Q = decltype(QP)::value;
      const uint32_t k0 = kBegin + kt * C::BK;
      if constexpr (Q < C::B_LOADS) {
        uint32_t lds = ldsBase + C::STAGES * C::A_STAGE + S * C::B_STAGE + (wave * C::B_LOADS + Q) * 1024;
        if constexpr (C::DUMP) { if (wave * C::B_LOADS + Q >= C::B_TOTAL) lds = ldsBase + C::DUMP_OFFSET; }
        uint32_t off;
        if constexpr (C::BT) off = (bVoff0[Q] != kOutOfRange && k0 + bLoadChunk[Q] * 8 < kEnd) ? bVoff0[Q] + k0 * 2 : kOutOfRange;
        else off = (bVoff0[Q] != kOutOfRange && k0 < kEnd) ? bVoff0[Q] + k0 * p.ldb * 2 : kOutOfRange;
        loadToLds(rB, __builtin_amdgcn_readfirstlane(lds), off);
      } else {
        constexpr int QA = Q - C::B_LOADS;
        const bool aInRange = k0 + aLoadChunk * 8 < kEnd;   // never touch columns the slice has not waited for
        const uint32_t lds = ldsBase + S * C::A_STAGE + (wave * C::A_LOADS + QA) * 1024;
        uint32_t off = aInRange ? aVoff0 + k0 * 2 + QA * aVstep : kOutOfRange;
        if constexpr (conv) {
          const uint32_t rs = k0 / p.cvC, c0 = k0 % p.cvC;
          const int32_t ih = cvIh0[QA] + (int32_t)(rs / p.cvS), iw = cvIw0[QA] + (int32_t)(rs % p.cvS);
          const bool inside = aInRange && cvBase[QA] != kOutOfRange / 2 && ih >= 0 && ih < (int32_t)p.cvH && iw >= 0 && iw < (int32_t)p.cvW;
          off = inside ? (cvBase[QA] + ((uint32_t)ih * p.cvW + (uint32_t)iw) * p.cvC + c0 + aLoadChunk * 8) * 2 : kOutOfRange;
        }
        loadToLds(rA, __builtin_amdgcn_readfirstlane(lds), off);
      }
    };
    auto issueAll = [&](auto SP, uint32_t kt) {
      staticFor<C::LOADS>([&](auto QP) { issueOne(SP, QP, kt); });
    };

    // MFMA pass over stage S.  The direct loads of chunk ktLoad (into stage SL)
    // are issued one at a time between the LDS reads of the first k-step, so
    // that they trickle into the memory pipeline under the MFMAs instead of
    // arriving as one burst that stalls the wave.
    auto compute = [&](auto SP, auto SLP, uint32_t ktLoad) {
      constexpr int S = decltype(SP)::value;
      const char* sa = smem + S * C::A_STAGE;
      const char* sb = smem + C::STAGES * C::A_STAGE + S * C::B_STAGE;
      half8 fa[2][C::TM], fb[2][C::TN];
      constexpr int R = C::TM + C::TN;                 // fragment loads per k-step (a B fragment is two reads)
      // Fragment f of a k-step: f < TM is A tile f, otherwise B tile f - TM.
      auto loadFrag = [&](auto FP, int slot, int kk) {
        constexpr int F = decltype(FP)::value;
        if constexpr (F < C::TM) {
          fa[slot][F] = *reinterpret_cast<const half8*>(sa + aFrag[kk] + F * 32 * C::A_ROW_BYTES);
        } else {
          constexpr int J = F - C::TM;
          if constexpr (C::BT) {
            fb[slot][J] = *reinterpret_cast<const half8*>(smem + C::STAGES * C::A_STAGE + S * C::B_STAGE + bFragT[kk] + J * 32 * C::B_ROW_BYTES);
            return;
          }
          typedef short4v __attribute__((address_space(3))) * lds_ptr;
          const char* q = sb + bFrag[J] + kk * 16 * C::B_ROW_BYTES;
          short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(q));
          short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(q + 4 * C::B_ROW_BYTES));
          half4 l4 = __builtin_bit_cast(half4, lo), h4 = __builtin_bit_cast(half4, hi);
          fb[slot][J] = __builtin_shufflevector(l4, h4, 0, 1, 2, 3, 4, 5, 6, 7);
        }
      };
      auto loadFrags = [&](int slot, int kk) {
        staticFor<R>([&](auto FP) { loadFrag(FP, slot, kk); });
      };
      // Fragments of k-step 1 with the direct loads spread between them.
      auto loadFragsAndIssue = [&](int slot, int kk) {
        staticFor<R>([&](auto FP) {
          loadFrag(FP, slot, kk);
          staticFor<C::LOADS>([&](auto QP) {
            if constexpr (decltype(QP)::value * R / C::LOADS == decltype(FP)::value) issueOne(SLP, QP, ktLoad);
          });
        });
      };
      loadFrags(0, 0);
#pragma unroll
      for (int kk = 0; kk < C::KS; kk++) {
        if (kk == 0 && C::KS > 1) loadFragsAndIssue(1, 1);
        else if (kk + 1 < C::KS) loadFrags((kk + 1) & 1, kk + 1);
#pragma unroll
        for (int i = 0; i < C::TM; i++)
#pragma unroll
          for (int j = 0; j < C::TN; j++)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[kk & 1][j], fa[kk & 1][i], acc[i][j], 0, 0, 0);
      }
      schedPass<C::KS, C::TM * C::TN, C::TM + (C::BT ? 1 : 2) * C::TN, 0>();
    };

    // Iteration kt on stage S = kt % STAGES.  Chunks kt+1 .. kt+STAGES-2 are the
    // ones this wave still has in flight behind chunk kt.
    auto step = [&](auto SP, uint32_t kt) {
      constexpr int S = decltype(SP)::value;
      waitVmcnt<(C::STAGES - 2) * C::LOADS>();
      __builtin_amdgcn_s_barrier();      // chunk kt is in LDS for everyone; everyone is done with chunk kt-1
      asm volatile("" ::: "memory");
      const uint32_t ktLoad = kt + C::STAGES - 1;
      if constexpr (conv || !ROUNDS) { if (ktLoad < nk) waitChunk(kBegin + ktLoad * C::BK); }
      __builtin_amdgcn_sched_barrier(0);
      compute(SP, Parity<(S + C::STAGES - 1) % C::STAGES>{}, ktLoad);
      __builtin_amdgcn_sched_barrier(0);
    };

    // ---- pipelined order -----------------------------------------------------------
    half8 pfa[2][C::TM], pfb[2][C::TN];
    auto loadFragP = [&](auto SP, auto FP, auto SLOT, int kk) {
      constexpr int S = decltype(SP)::value, F = decltype(FP)::value, slot = decltype(SLOT)::value;
      if constexpr (F < C::TM) {
        pfa[slot][F] = *reinterpret_cast<const half8*>(smem + S * C::A_STAGE + aFrag[kk] + F * 32 * C::A_ROW_BYTES);
      } else {
        constexpr int J = F - C::TM;
        const char* sb = smem + C::STAGES * C::A_STAGE + S * C::B_STAGE;
        if constexpr (C::BT) {
          pfb[slot][J] = *reinterpret_cast<const half8*>(sb + bFragT[kk] + J * 32 * C::B_ROW_BYTES);
        } else {
          typedef short4v __attribute__((address_space(3))) * lds_ptr;
          const char* q = sb + bFrag[J] + kk * 16 * C::B_ROW_BYTES;
          short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(q));
          short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(q + 4 * C::B_ROW_BYTES));
          half4 l4 = __builtin_bit_cast(half4, lo), h4 = __builtin_bit_cast(half4, hi);
          pfb[slot][J] = __builtin_shufflevector(l4, h4, 0, 1, 2, 3, 4, 5, 6, 7);
        }
      }
    };
    auto mfmaP = [&](auto SLOT) {
      constexpr int slot = decltype(SLOT)::value;
#pragma unroll
      for (int i = 0; i < C::TM; i++)
#pragma unroll
        for (int j = 0; j < C::TN; j++)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(pfb[slot][j], pfa[slot][i], acc[i][j], 0, 0, 0);
    };
    auto stepP = [&](auto SP, uint32_t kt) {
      constexpr int S = decltype(SP)::value;
      constexpr int R = C::TM + C::TN;
      constexpr int DS = C::TM + (C::BT ? 1 : 2) * C::TN;
      // k-step 0 (fragments already in slot 0) while the fragments of k-step 1 arrive
      staticFor<R>([&](auto FP) { loadFragP(SP, FP, Parity<1>{}, 1); });
      mfmaP(Parity<0>{});
      schedHalf<C::TM * C::TN, DS>();
      __builtin_amdgcn_sched_barrier(0);
      waitVmcnt<(C::STAGES - 3) * C::LOADS>();     // own part of chunk kt+1
      __builtin_amdgcn_s_barrier();                // chunk kt+1 is in LDS for everyone; everyone is done with chunk kt-1
      asm volatile("" ::: "memory");
      const uint32_t ktLoad = kt + C::STAGES - 1;
      if constexpr (conv || !ROUNDS) { if (ktLoad < nk) waitChunk(kBegin + ktLoad * C::BK); }
      __builtin_amdgcn_sched_barrier(0);
      // k-step 1 while the first fragments of chunk kt+1 arrive and the loads of chunk ktLoad go out
      staticFor<R>([&](auto FP) {
        loadFragP(Parity<(S + 1) % C::STAGES>{}, FP, Parity<0>{}, 0);
        staticFor<C::LOADS>([&](auto QP) {
          if constexpr (decltype(QP)::value * R / C::LOADS == decltype(FP)::value) issueOne(Parity<(S + C::STAGES - 1) % C::STAGES>{}, QP, ktLoad);
        });
      });
      mfmaP(Parity<1>{});
      schedHalf<C::TM * C::TN, DS>();
      __builtin_amdgcn_sched_barrier(0);
    };

    if (consumer) {
      cusync_dim3 w = {m0, 0, 1};
      if (stage.needsWait(w)) {
        if (wave == 0) { if constexpr (conv) cvWaitRows(0, 1); else waitRows(0, 1); }
        __syncthreads();
      }
    }

    // Prologue: chunks 0 .. STAGES-2 (chunks past the end of K load zeros).
    // A GEMM's chunks go through the producer's column tiles in order, so the wait for a chunk covers the chunks
    // before it: with ROUNDS, one wait for the prologue and one per round of the loop below, each for the last
    // chunk whose loads it is in front of.  A convolution's chunks come back to the same channel tiles tap after
    // tap and are always waited for one by one.
    constexpr bool perChunk = conv || !ROUNDS;
    auto waitThrough = [&](uint32_t kt) { waitChunk(kBegin + min(kt, nk - 1) * C::BK); };
    // (the assembly K loop has no place for waits: a stage of a tile policy waits for all its producer tiles here)
    if constexpr (C::PINGPONG) waitThrough(nk - 1);
    else if constexpr (perChunk) waitChunk(kBegin);
    else waitThrough(C::STAGES - 2);
    if constexpr (!C::PINGPONG) issueAll(Parity<0>{}, 0);
    if constexpr (C::STAGES > 2 && !C::PINGPONG) { if constexpr (perChunk) { if (nk > 1) waitChunk(kBegin + C::BK); } issueAll(Parity<1>{}, 1); }
    if constexpr (C::STAGES > 3) { if constexpr (perChunk) { if (nk > 2) waitChunk(kBegin + 2 * C::BK); } issueAll(Parity<2>{}, 2); }
    if constexpr (C::STAGES > 4) { if constexpr (perChunk) { if (nk > 3) waitChunk(kBegin + 3 * C::BK); } issueAll(Parity<3>{}, 3); }
    static_assert(C::STAGES >= 2 && C::STAGES <= 5, "prologue written for 2..5 stages");
    if (tid == 0 && round == 0) stage.finishStart(startToken, p.launched);
    const unsigned long long tl1 = p.timeline ? wall_clock64() : 0;

    if constexpr (C::PINGPONG && C::BN == 384) {
      // The K loop is assembly (gemm_wide_steps.inc); its LDS layout and what it is handed are set up here.  A is
      // kept 64 columns of K at a time, [256 rows][128 bytes] in a ring of two slots, so that every piece fetched
      // from memory is a whole cache line; B in the ring of three 32-row stages behind it.
      static_assert(C::BM == 256 && C::BN == 384 && C::BK == 32 && C::WM == 2 && C::WN == 4 && C::STAGES == 3 && !conv,
                    "the assembly K loop is written for this tile");
      constexpr uint32_t A_SLOT = 256 * 128, B_BASE = 2 * A_SLOT;
      static_assert(B_BASE + 3 * C::B_STAGE <= C::LDS_BYTES, "two A slots and three B stages fit the workgroup's LDS");
      WideOperands w;
      {
        // fragment side: row (laneL & 31) of the wavefront's first MFMA row tile, 16-byte piece (laneL >> 5) of the
        // k-step.  The eight pieces of a row are swizzled with bits 1..3 of the row number: an LDS read serves
        // sixteen lanes at a time, sixteen consecutive rows here, and with 128-byte rows two rows cover all banks once,
        // so rows 2n and 2n+1 take one position and the eight pairs eight different ones.
        const uint32_t row = wm * C::WTM + (laneL & 31);
        w.vA = ldsBase + row * 128 + ((((uint32_t)laneL >> 5) ^ ((row >> 1) & 7)) * 16);
#pragma unroll
        for (int j = 0; j < C::TN; j++) w.vB[j] = ldsBase + B_BASE + bFrag[j];
        // load side: load q of this wavefront fills rows wave * 32 + q * 8 + laneL / 8 of a slot; the lane at piece
        // position p of a row fetches the piece that belongs there under the swizzle
#pragma unroll
        for (int q = 0; q < 4; q++) {
          const uint32_t lrow = q * 8 + ((uint32_t)laneL >> 3), piece = ((uint32_t)laneL & 7) ^ ((lrow >> 1) & 7);
          w.a[q] = ((m0 + wave * 32 + lrow) * p.lda + kBegin + piece * 8) * 2;
        }
#pragma unroll
        for (int q = 0; q < C::B_LOADS; q++) w.b[q] = bVoff0[q] == kOutOfRange ? kOutOfRange : bVoff0[q] + kBegin * p.ldb * 2;
      }
      w.rA = rA; w.rB = rB;
      w.m0A = __builtin_amdgcn_readfirstlane(ldsBase + wave * 4096);
      w.m0B = __builtin_amdgcn_readfirstlane(ldsBase + B_BASE + wave * C::B_LOADS * 1024);
      w.dB = C::BK * p.ldb * 2;
      // A slot 0 and chunks 0 and 1 of B (K is a whole number of slots: at least two chunks)
#pragma unroll
      for (int q = 0; q < 4; q++) loadToLds(rA, __builtin_amdgcn_readfirstlane(w.m0A + q * 1024), w.a[q]);
#pragma unroll
      for (int c = 0; c < 2; c++)
#pragma unroll
        for (int q = 0; q < C::B_LOADS; q++)
          loadToLds(rB, __builtin_amdgcn_readfirstlane(w.m0B + c * C::B_STAGE + q * 1024), w.b[q] == kOutOfRange ? kOutOfRange : w.b[q] + c * w.dB);
      // The loop loads chunk 2 next and moves on chunk by chunk while there is another one.
      const uint32_t soffA = min(2u, nk - 1) * 64;
      wideLoop(acc, w, soffA, nk);
    } else if constexpr (C::PINGPONG) {
      // 256x192 in whole cache lines: A [256 rows][128 bytes = 64 columns of K] in a ring of three slots, B in stages
      // of [32 k rows][384 bytes] in a ring of four behind it; the K loop is assembly (gemm_wide_steps.inc).
      static_assert(C::BN == 192 && C::BK == 64 && C::WM == 4 && C::WN == 2 && !conv, "the assembly K loop is written for this tile");
      constexpr uint32_t B_BASE = 3 * C::A_STAGE, B_STAGE32 = 32 * C::B_ROW_BYTES;
      static_assert(B_BASE + 4 * B_STAGE32 <= C::LDS_BYTES, "three A slots and four B stages fit the workgroup's LDS");
      WideOperands w;
      w.vA = ldsBase + aFrag[0];
#pragma unroll
      for (int j = 0; j < C::TN; j++) w.vB[j] = ldsBase + B_BASE + bFrag[j];
      // A: load q of this wavefront fills rows wave * 32 + q * 8 + laneL / 8 of a slot; the lane at piece position p
      // of a row fetches the piece that belongs there under the swizzle (which differs from load to load)
#pragma unroll
      for (int q = 0; q < 4; q++) {
        const uint32_t lrow = q * 8 + ((uint32_t)laneL >> 3), piece = ((uint32_t)laneL & 7) ^ ((lrow >> 1) & 7);
        w.a[q] = ((m0 + wave * 32 + lrow) * p.lda + kBegin + piece * 8) * 2;
      }
      // B: a stage is 768 pieces of 16 bytes, 96 per wavefront: a load of all 64 lanes and one of the lower 32
#pragma unroll
      for (int q = 0; q < 2; q++) {
        const uint32_t slot = wave * 96 + q * 64 + (uint32_t)laneL, brow = slot / C::B_CPR, piece = (slot % C::B_CPR) ^ (4 * (brow & 1));
        w.b[q] = n0 + piece * 8 < p.N ? ((kBegin + brow) * p.ldb + n0 + piece * 8) * 2 : kOutOfRange;
      }
      w.rA = rA; w.rB = rB;
      w.m0A = __builtin_amdgcn_readfirstlane(ldsBase + wave * 4096);
      w.m0B = __builtin_amdgcn_readfirstlane(ldsBase + B_BASE + wave * 1536);
      w.dB = 32 * p.ldb * 2;
      const uint32_t chunks = 2 * nk, lastSlot = (chunks - 2) * 64;         // nk counts slots of 64 columns
      auto loadA = [&](uint32_t slot) {
#pragma unroll
        for (int q = 0; q < 4; q++) loadToLds(rA, __builtin_amdgcn_readfirstlane(w.m0A + slot * C::A_STAGE + q * 1024), w.a[q] + min(slot * 128, lastSlot));
      };
      auto loadB = [&](uint32_t c) {
        const uint32_t off = min(c, chunks - 1) * w.dB;
        loadToLds(rB, __builtin_amdgcn_readfirstlane(w.m0B + c * B_STAGE32), w.b[0] == kOutOfRange ? kOutOfRange : w.b[0] + off);
        loadToLdsLowerHalf(rB, __builtin_amdgcn_readfirstlane(w.m0B + c * B_STAGE32 + 1024), w.b[1] == kOutOfRange ? kOutOfRange : w.b[1] + off);
      };
      // what the loop finds under way: A slots 0 and 1, chunks 0 to 2 of B, in the order its own loads keep
      loadA(0); loadB(0); loadB(1); loadA(1); loadB(2);
      pairLoop192(acc, w, min(3u, chunks - 1) * 64, chunks, lastSlot);
    } else if constexpr (C::PIPE) {
      waitVmcnt<(C::STAGES - 2) * C::LOADS>();     // chunk 0
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      staticFor<C::TM + C::TN>([&](auto FP) { loadFragP(Parity<0>{}, FP, Parity<0>{}, 0); });
      for (uint32_t kt = 0; kt < nk; kt += C::STAGES) {
        if constexpr (!perChunk) waitThrough(kt + 2 * C::STAGES - 2);      // the loads this round issues
        stepP(Parity<0>{}, kt);
        if (kt + 1 < nk) stepP(Parity<1 % C::STAGES>{}, kt + 1);
        if (C::STAGES > 2 && kt + 2 < nk) stepP(Parity<2 % C::STAGES>{}, kt + 2);
        if (C::STAGES > 3 && kt + 3 < nk) stepP(Parity<3 % C::STAGES>{}, kt + 3);
        if (C::STAGES > 4 && kt + 4 < nk) stepP(Parity<4 % C::STAGES>{}, kt + 4);
      }
    } else {
      for (uint32_t kt = 0; kt < nk; kt += C::STAGES) {
        if constexpr (!perChunk) waitThrough(kt + 2 * C::STAGES - 2);      // the loads this round issues
        step(Parity<0>{}, kt);
        if (kt + 1 < nk) step(Parity<1 % C::STAGES>{}, kt + 1);
        if (C::STAGES > 2 && kt + 2 < nk) step(Parity<2 % C::STAGES>{}, kt + 2);
        if (C::STAGES > 3 && kt + 3 < nk) step(Parity<3 % C::STAGES>{}, kt + 3);
        if (C::STAGES > 4 && kt + 4 < nk) step(Parity<4 % C::STAGES>{}, kt + 4);
      }
    }

    // The loads issued for chunks past the end of K (zeros) may still be on their way into LDS, which the
    // epilogue is about to reuse.
    waitVmcnt<0>();
    const unsigned long long tl2 = p.timeline ? wall_clock64() : 0;
    if (tid == 0) nextRaw = stage.drawBegin(dryXcds, noDraws);     // settled after the epilogue
    const bool completed = finishTile<C, !conv>(p, acc, t, wm, wn, lane, &sLast, smem);

    // All waves must be past their last LDS read before the next tile's loads
    // land in stage 0; the post (or this barrier) provides that.
    cusync_dim3 done = {m0, outputColumn(p, n0), t.z};
    if (completed && stage.isProducer()) stage.post(done, postsPerTile(p), stage.storesThrough());
    else __syncthreads();
    if (tid == 0) recordTile(p, t, round, tlEntry, tl0, tl1, tl2, p.timeline ? wall_clock64() : 0);
  }
}

template<class C, int AMODE = kAPlain, bool CHUNKS = true>
__global__ __launch_bounds__(C::THREADS, C::WAVES_PER_SIMD) void gemmDmaKernel(GemmParams p) {
  gemmDmaTiles<C, AMODE, CHUNKS, true>(p);
}

// Dependent GEMMs of one tile shape in ONE launch: every workgroup works through the tiles of the first
// GEMM it can draw, then those of the second, and so on; a tile of a later GEMM waits on the semaphores
// of the one before exactly as it does when they are separate launches.  No kernel boundary, wait
// kernel or second launch sits between producer and consumer, which is what a chain of short GEMMs
// (few rows: 30 us in the kernel, 10 us around it) pays most for.  Forward progress: the launch has
// no more workgroups than stay resident, and a workgroup only moves on when the GEMM it is on has no
// tile left to hand out, so every tile a consumer tile waits for is in the hands of a running workgroup.
template<class C>
__global__ __launch_bounds__(C::THREADS, C::WAVES_PER_SIMD) void gemmDmaChainKernel(GemmChainParams cp) {
  for (uint32_t g = 0; g < cp.count; g++) {
    gemmDmaTiles<C, kAPlain, true, false>(cp.gemm[g]);
    __syncthreads();        // everyone has read the last ticket of this GEMM before the next one's is written
  }
}

}  // namespace gemm
}  // namespace cusync
