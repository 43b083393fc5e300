// Fused multi-head attention (softmax(mask(Q K^T * scale)) V, fp16 in/out, fp32
// accumulate, head width 128) as a CuSync middle stage: it waits for the tiles
// of the QKV projection that hold its Q rows and each K/V block just before it
// loads them, and posts every finished output tile for the output projection.
//
// One workgroup (four wavefronts) owns 128 query rows of one head; each
// wavefront owns 32 of them.  K and V are walked in blocks of 64 rows that go
// from global memory straight into LDS, two or four stages deep (see the
// kernel's template parameter).  Within a block all K fragments are requested
// up front and the V^T fragments between the MFMAs of the first product, so
// that the second product finds them in registers; the blocks that need the
// causal mask are the last of a range and have their own copy of the loop.
// Under a causal mask the row tiles are taken in descending order: the long
// ones start first.  Measured at 2048 rows x 12 heads, alone: 49-51 us
// (12.9 GFLOP, 260 TFLOP/s); a block of 64 keys takes a workgroup 1.6 us, of
// which the MFMAs and the exponentials are a third (the kernel without them:
// 43 us), the rest being LDS round trips and the remaining vector instructions
// of a single wavefront per SIMD issuing in order.  Computing the scores of
// block j+1 under the softmax of block j was built and was slower (2.4 us per
// block): it needs more than 256 registers, and the compiler then shuttles
// values between the two register files.
//
// Everything is computed transposed so that the softmax needs no shuffles:
//   S^T = K Q^T      (MFMA rows = kv, columns = q)
//   O^T = V^T P^T    (MFMA rows = head dim, columns = q)
// In the 32x32 MFMA result layout a lane holds one column, i.e. one query row:
// its 16 registers per tile are 16 kv positions (or head-dim positions) of that
// query.  Row maximum, row sum and the rescale factor are therefore per-lane
// scalars; only the two half-waves (lanes l and l^32 hold the same query, other
// kv positions) exchange one value per block.  The registers of S^T, converted
// to fp16, already are the B operand of the second product: register e of a
// lane in half-wave h stands for kv position 16u + 8(e/4) + 4h + e%4 of k-step
// u, and the V^T fragment is read (LDS transpose read) in that same order.
//
// Long key ranges can be split (AttnParams::chunk key/value blocks per workgroup, grid z = split
// index): a workgroup that walks all 32 blocks of the last rows of a 2048-row causal problem
// alone is what the whole kernel waits for.  Each split leaves its unnormalised O^T, row maxima
// and row sums in a workspace (register order, so all accesses are coalesced); the split that
// arrives last at the tile's counter rescales and adds them in split order — the result does
// not depend on arrival order — normalises, stores, re-arms the counter and posts the tile.
#pragma once

#include "gemm_kernel_dma.h"

namespace cusync {
namespace attn {

using namespace cusync::gemm;

constexpr int kBQ = 128, kBKV = 64, kHD = 128;
constexpr int kRowBytes = kHD * 2;                  // one K or V row of a head
constexpr int kStageBytes = kBKV * kRowBytes;       // one K or one V block
constexpr int ldsBytes(int stages) { return stages * 2 * kStageBytes; }      // `stages` blocks of K and of V
constexpr int kBlockLoads = 8;                      // 1 KiB direct loads per wavefront and block (four of K, four of V)
constexpr float kMasked = -1.0e30f;

struct AttnParams {
  cusync::DynStage stage;
  uint32_t S, heads;                 // S query rows (= rows the stage produces)
  uint32_t cached;                   // rows of qkv in front of the query rows: the key/value cache
  const half_t* qkv; uint32_t ldq;   // [cached + S][ldq]: Q at column 0, K at heads*128, V at 2*heads*128
  half_t* out; uint32_t ldo;         // [S][ldo]
  float scaleLog2;                   // softmax scale * log2(e)
  uint32_t causal;
  uint32_t launched;
  uint32_t chunk;                    // key/value blocks per split; 0: one workgroup walks the whole range
  float* partO;                      // [heads][row tiles][splits][64][256] unnormalised O^T, register order
  float* partStat;                   // [heads][row tiles][splits][2][256] row maximum, row sum
  uint32_t* arrivals;                // [heads][row tiles] splits finished; 0 between launches
  uint32_t partBytes;                // bytes of partO and partStat together (they are adjacent)
  uint32_t descending;               // row tiles are taken last first
  unsigned long long* timeline;      // diagnosis (cusync_rt_set_timeline), records as the GEMM kernels write them
  uint32_t timelineCap;
};

// kStages blocks of K and V in LDS, kStages - 1 of them in flight behind the one being multiplied: 4 (128 KB, the CU
// to itself) or 2 (64 KB, room for another kernel's workgroups beside it).
template<int kStages>
__global__ __launch_bounds__(kThreads, 2) void attentionKernel(AttnParams p) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  __shared__ uint32_t sTicket, sLast;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t hi = lane >> 5;
  const cusync::DynStage& stage = p.stage;
  const uint32_t E = p.heads * kHD;
  const uint32_t total = p.cached + p.S;               // key/value rows
  const uint32_t bufBytes = total * p.ldq * 2;
  const uint4v rLds = rawRsrc(p.qkv, bufBytes);
  const __amdgpu_buffer_rsrc_t rReg = makeRsrc(p.qkv, bufBytes);
  const uint32_t ldsBase = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem;

  // ---- direct-load side -------------------------------------------------------
  // A block is 64 rows of 256 bytes = 16 loads of 1 KiB; wave w issues loads
  // 4w..4w+3 of K and of V.  Load q of a wave fills rows 16w + 4q + lane/16,
  // 16-byte slot lane%16.  The chunk of the row a lane fetches is permuted so
  // that the fragment reads below are free of bank conflicts:
  //   K: slot = chunk ^ (row & 15)       (row-fragment reads, 32 rows x one chunk)
  //   V: slot = chunk ^ 4*(row & 1)      (transpose reads, 4 rows x 64 bytes)
  const uint32_t ldRow = wave * 16 + (lane >> 4);
  uint32_t kChunk[4];
#pragma unroll
  for (int q = 0; q < 4; q++) kChunk[q] = (lane & 15) ^ ((4 * q + (lane >> 4)) & 15);
  const uint32_t vChunk = (lane & 15) ^ (4 * ((lane >> 4) & 1));

  // ---- fragment side ------------------------------------------------------------
  // K fragment of k-step s (16 head-dim positions): row lane%32 of a 32-row tile, chunk 2s + hi.
  uint32_t kFrag[8];
#pragma unroll
  for (int s = 0; s < 8; s++) kFrag[s] = (lane & 31) * kRowBytes + (((2 * s + hi) ^ (lane & 15)) * 16);
  // V^T fragment of k-step u, head-dim tile t: transpose reads of rows 16u + 4hi + (lane&15)/4 (+8),
  // 4 halfs at column 32t + 16*((lane/16)&1) + 4*(lane&3).
  const uint32_t flip = (lane >> 2) & 1;
  const uint32_t vRowOff = (4 * hi + ((lane & 15) >> 2)) * kRowBytes;
  const uint32_t vColOff = (2 * ((lane >> 4) & 1) + ((lane & 3) >> 1)) * 16 + (lane & 1) * 8;
  const uint32_t vEven = vRowOff + vColOff + 64 * flip;          // tiles t = 0, 2: + 64 t
  const uint32_t vOdd = vRowOff + vColOff + 64 - 64 * flip;      // tiles t = 1, 3: + 64 (t - 1)

  const uint32_t numTiles = stage.numTiles();
  const bool consumer = stage.isConsumer();
  const uint32_t tmq = consumer ? stage.d.in.tileM : 1, tnq = consumer ? stage.d.in.tileN : 1;
  // RowSync and ConsecutiveSync mark their waits with z = 1, the tile policies with z = 0.
  const uint32_t zWait = consumer && (stage.d.in.kind == CUSYNC_POLICY_ROWSYNC ||
                                      stage.d.in.kind == CUSYNC_POLICY_CONSECUTIVESYNC) ? 1 : 0;
  // Every wave waits for itself: each one fetches part of every block.
  // `col`: first of the kHD columns of qkv that are about to be read.  They can lie in more than one of the
  // producer's column tiles (192-wide tiles against 128-wide heads): every one of them is waited for.  The
  // row policies guard whole rows of a third of qkv with one semaphore, so one wait covers all columns.
  auto waitRows = [&](uint32_t rowBegin, uint32_t rowEnd, uint32_t col) {
    if (!consumer || rowBegin >= rowEnd) return;
    for (uint32_t c = col / tnq * tnq; c < col + kHD; c += tnq) {
      stage.waitWaveRows(rowBegin, rowEnd - 1, tmq, c, zWait);
      if (zWait) break;
    }
  };

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
    cusync_dim3 t = stage.ticketToTile(ticket);
    // Tickets are handed out by ascending row tile, and under a causal mask the last row tiles walk the longest key
    // ranges (and are the only ones whose later splits exist at all): taken in descending order the long tiles
    // start first and the tickets left for a second round are the short and the empty ones.  (Measured against
    // the ascending order with every mode of the chain timed in turn: 2048 rows 433 -> 417 us stream-ordered,
    // 426 -> 415 under RowSync; 512 rows 165 -> 161 and 157 -> 155; 1024 and 256 rows within 2 us either way.)
    if (p.descending) t.y = stage.d.grid.y - 1 - t.y;
    const unsigned long long tl0 = p.timeline ? wall_clock64() : 0;
    const uint32_t head = t.x, q0 = t.y * kBQ;
    const uint32_t qEnd = min(q0 + (uint32_t)kBQ, p.S);
    const uint32_t nkv = p.causal ? p.cached + qEnd : total;
    const uint32_t nblk = (nkv + kBKV - 1) / kBKV;
    const uint32_t splits = p.chunk ? (nblk + p.chunk - 1) / p.chunk : 1;
    if (t.z >= splits) {                               // this row tile needs fewer splits than the grid has
      if (tid == 0) nextRaw = stage.drawBegin(dryXcds, noDraws);
      if (tid == 0 && round == 0) stage.finishStart(startToken, p.launched);
      __syncthreads();
      continue;
    }
    const uint32_t jBegin = p.chunk ? t.z * p.chunk : 0;
    const uint32_t jEnd = p.chunk ? min(nblk, jBegin + p.chunk) : nblk;
    const uint32_t qw = q0 + 32 * wave;                 // first query row of this wave
    const uint32_t myq = qw + (lane & 31);
    // positions are rows of qkv: query i sits at cached + i and, when causal, sees keys 0 .. cached + i
    const uint32_t limit = p.causal ? p.cached + min(myq, p.S - 1) : total - 1;   // last kv position this query sees

    // Direct loads of block j into stage st.  Rows past the end of the
    // sequence lie outside the buffer and arrive as zeros.
    // Blocks past the end of the range are issued all the same, out of range (they arrive as zeros), so that the
    // count of loads in flight that the main loop waits for is the same at every block.
    auto issue = [&](uint32_t j, uint32_t st, bool valid) {
      const uint32_t kLds = ldsBase + st * 2 * kStageBytes + wave * 4 * 1024;
      const uint32_t rowOff = (j * kBKV + ldRow) * p.ldq;
#pragma unroll
      for (int q = 0; q < 4; q++)
        loadToLds(rLds, __builtin_amdgcn_readfirstlane(kLds + q * 1024),
                  valid ? (rowOff + q * 4 * p.ldq + E + head * kHD + kChunk[q] * 8) * 2 : kOutOfRange);
#pragma unroll
      for (int q = 0; q < 4; q++)
        loadToLds(rLds, __builtin_amdgcn_readfirstlane(kLds + kStageBytes + q * 1024),
                  valid ? (rowOff + q * 4 * p.ldq + 2 * E + head * kHD + vChunk * 8) * 2 : kOutOfRange);
    };
    // Key/value rows (counted from the first row the producer writes) below these marks are known to be posted, for
    // the K and for the V columns of this head.  A poll is a round trip to memory that the direct loads in flight
    // have to drain behind, so a block that needs rows beyond the mark first looks, without spinning, at all row
    // blocks of the producer that the rest of this tile's key range meets, and spins only if its own rows are
    // still missing: a tile that starts after its producer is done polls twice in all.
    uint32_t seenRows[2] = {0, 0};
    auto waitKV = [&](uint32_t j, uint32_t jLast) {       // blocks j .. jLast
      if (!consumer) return;
      // only the rows behind the cache come from the producer; its tiles count rows from there
      const uint32_t lo = max(j * kBKV, p.cached), hi = min(jLast * kBKV + (uint32_t)kBKV, total);
      if (lo >= hi) return;
      const uint32_t rowLo = lo - p.cached, rowHi = hi - p.cached;             // [rowLo, rowHi)
      const uint32_t rangeEnd = min(jEnd * kBKV, total) - p.cached;            // end of this tile's key range
#pragma unroll
      for (int c = 0; c < 2; c++) {
        if (rowHi <= seenRows[c]) continue;
        const uint32_t col = (c + 1) * E + head * kHD;
        const uint32_t first = max(rowLo, seenRows[c]);
        uint32_t ready = 64;                       // row blocks posted in every producer column tile the head's columns meet
        for (uint32_t ct = col / tnq * tnq; ct < col + kHD; ct += tnq) {
          ready = min(ready, stage.peekWaveRows(first, rangeEnd - 1, tmq, ct, zWait));
          if (zWait) break;
        }
        if (ready) seenRows[c] = min(rangeEnd, (first / tmq + ready) * tmq);
        if (rowHi > seenRows[c]) {
          waitRows(rowLo, rowHi, col);
          seenRows[c] = max(seenRows[c], min(rangeEnd, ((rowHi - 1) / tmq + 1) * tmq));
        }
        // RowSync guards all columns of a row block with one semaphore: what is known of K holds for V (and for Q)
        if (stage.d.in.kind == CUSYNC_POLICY_ROWSYNC) { seenRows[1] = seenRows[0]; break; }
      }
    };

    // The first blocks are requested before Q: they are what the tile waits for longest.  One wait for all of them
    // (the wait's code is inlined where it is called).
    waitKV(jBegin, min(jBegin + (uint32_t)kStages - 2, jEnd - 1));
#pragma unroll
    for (uint32_t a = 0; a < kStages - 1; a++) issue(jBegin + a, a, jBegin + a < jEnd);
    if (tid == 0 && round == 0) stage.finishStart(startToken, p.launched);
    // Q fragments stay in registers for the whole tile: k-step s is head-dim 16s + 8hi .. + 7 of row myq.
    if (!(stage.d.in.kind == CUSYNC_POLICY_ROWSYNC && p.cached == 0 && seenRows[0] >= qEnd)) waitRows(q0, qEnd, head * kHD);
    half8 qf[8];
#pragma unroll
    for (int s = 0; s < 8; s++)
      qf[s] = __builtin_bit_cast(half8, loadChunk(rReg, myq < p.S ? ((p.cached + myq) * p.ldq + head * kHD + 16 * s + 8 * hi) * 2 : kOutOfRange));
    // The fragments are waited for here, once.  Left to the compiler the wait lands in the block loop, in front of
    // each fragment's first use: it counts these eight loads as possibly outstanding on every pass and asks for
    // "at most 7 - s loads in flight" there, and the loads in flight there are the direct loads of the blocks ahead,
    // issued after these and invisible to its count: every block then waits for the blocks it has just requested.
    // (At the benchmark's sizes those land within a block's time and the kernel measures the same either way.)
#pragma unroll
    for (int s = 0; s < 8; s++) asm volatile("" : "+v"(qf[s]));
    const unsigned long long tl1 = p.timeline ? wall_clock64() : 0;

    float rowMax = kMasked, rowSum = 0.0f;      // rowSum: this half-wave's share
    floatx16 o[4];
#pragma unroll
    for (int tt = 0; tt < 4; tt++)
#pragma unroll
      for (int r = 0; r < 16; r++) o[tt][r] = 0.0f;

    // One key/value block in LDS stage st.  MASKED: the block reaches past what some query of this wavefront sees
    // and the scores beyond are masked; as a run-time condition inside the block the compiler turns the mask into
    // selects that every block pays for (a third of its vector instructions).
    auto computeBlock = [&](auto MASKED, uint32_t j, uint32_t st) __attribute__((always_inline)) {
      const char* ks = smem + st * 2 * kStageBytes;
      const char* vs = ks + kStageBytes;

      // S^T = K Q^T for the two 32-row kv tiles of the block.  All K fragments are requested first; the V^T
      // fragments of the second product are requested between the MFMAs, so that they arrive under the softmax
      // instead of holding up the second product (the compiler's own order is read, wait, MFMA, one by one, which
      // with two wavefronts per SIMD leaves the matrix pipe idle for most of an LDS round trip each time).
      typedef short4v __attribute__((address_space(3))) * lds_ptr;
      half8 kf[8][2];
#pragma unroll
      for (int s = 0; s < 8; s++)
#pragma unroll
        for (int a = 0; a < 2; a++) kf[s][a] = *reinterpret_cast<const half8*>(ks + kFrag[s] + a * 32 * kRowBytes);
      floatx16 sacc[2];
#pragma unroll
      for (int a = 0; a < 2; a++)
#pragma unroll
        for (int r = 0; r < 16; r++) sacc[a][r] = 0.0f;
#pragma unroll
      for (int s = 0; s < 8; s++)
#pragma unroll
        for (int a = 0; a < 2; a++) sacc[a] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[s][a], qf[s], sacc[a], 0, 0, 0);
      // V^T fragments of k-steps 0 and 1 now, those of k-steps 2 and 3 under the MFMAs of the first two
      half8 vf[4][4];
      auto readV = [&](int u, int tt) {
        const char* q = vs + ((tt & 1) ? vOdd + (tt - 1) * 64 : vEven + tt * 64) + u * 16 * kRowBytes;
        const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(q));
        const short4v up = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(q + 8 * kRowBytes));
        const half4 l4 = __builtin_bit_cast(half4, lo), u4 = __builtin_bit_cast(half4, up);
        vf[u][tt] = __builtin_shufflevector(l4, u4, 0, 1, 2, 3, 4, 5, 6, 7);
      };
#pragma unroll
      for (int u = 0; u < 2; u++)
#pragma unroll
        for (int tt = 0; tt < 4; tt++) readV(u, tt);
      schedGroup<kSchedDsRead, 16>();
      staticFor<16>([&](auto) { schedGroup<kSchedMfma, 1>(); schedGroup<kSchedDsRead, 1>(); });
      __builtin_amdgcn_sched_barrier(0);

      // mask (only blocks that reach past what some query of this wave sees: MASKED), running maximum of the raw scores
      const uint32_t kvBase = j * kBKV + 4 * hi;
      if constexpr (decltype(MASKED)::value != 0) {
#pragma unroll
        for (int a = 0; a < 2; a++)
#pragma unroll
          for (int r = 0; r < 16; r++)
            if (kvBase + 32 * a + 8 * (r / 4) + (r % 4) > limit) sacc[a][r] = kMasked;
      }
      float blockMax = kMasked;
#pragma unroll
      for (int a = 0; a < 2; a++)
#pragma unroll
        for (int r = 0; r < 16; r += 2) blockMax = __builtin_fmaxf(__builtin_fmaxf(blockMax, sacc[a][r]), sacc[a][r + 1]);
      blockMax = fmaxf(blockMax, __shfl_xor(blockMax, 32));
      const float newMax = fmaxf(rowMax, blockMax);
      const float alpha = __builtin_amdgcn_exp2f((rowMax - newMax) * p.scaleLog2);
      const float shift = newMax * p.scaleLog2;
      rowMax = newMax;

      // P^T = exp2(S^T * scale - max * scale), as fp16 B operands of the second product
      half8 pf[4];
      float blockSum = 0.0f;
#pragma unroll
      for (int a = 0; a < 2; a++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[a][r], p.scaleLog2, -shift));
          blockSum += e;
          pf[2 * a + r / 8][r % 8] = (half_t)e;
        }
      rowSum = rowSum * alpha + blockSum;
      if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
        for (int tt = 0; tt < 4; tt++)
#pragma unroll
          for (int r = 0; r < 16; r++) o[tt][r] *= alpha;
      }

      // O^T += V^T P^T
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int u = 2; u < 4; u++)
#pragma unroll
        for (int tt = 0; tt < 4; tt++) readV(u, tt);
#pragma unroll
      for (int u = 0; u < 4; u++)
#pragma unroll
        for (int tt = 0; tt < 4; tt++) o[tt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[u][tt], pf[u], o[tt], 0, 0, 0);
      staticFor<8>([&](auto) { schedGroup<kSchedMfma, 1>(); schedGroup<kSchedDsRead, 2>(); });
    };

    // The blocks that need the mask are the last ones of the range (a causal mask, or a sequence that ends inside a
    // block): one loop over the blocks before them, one over them, each with its own copy of the block's code.  (One
    // loop that chooses between the two copies per block makes the compiler spill a hundred registers.)
    auto runBlocks = [&](auto MASKED, uint32_t jFrom, uint32_t jTo) __attribute__((always_inline)) {
      for (uint32_t j = jFrom; j < jTo; j++) {
        const uint32_t st = (j - jBegin) % kStages;
        waitVmcnt<(kStages - 2) * kBlockLoads>();      // this wavefront's part of block j
        __builtin_amdgcn_s_barrier();       // block j is in LDS for everyone; everyone is done with block j-1
        asm volatile("" ::: "memory");
        const uint32_t ahead = j + kStages - 1;           // goes into the stage block j-1 has left
        if (ahead < jEnd) waitKV(ahead, ahead);
        issue(ahead, (st + kStages - 1) % kStages, ahead < jEnd);
        if (p.causal && j * kBKV > p.cached + qw + 31) continue;       // wholly in this wave's future (wave-uniform)
        computeBlock(MASKED, j, st);
      }
    };
    // block j needs the mask when its last key, 64 j + 63, lies beyond what the first query of this wavefront sees
    const uint32_t seenByAll = p.causal ? p.cached + min(qw, p.S - 1) : total - 1;
    const uint32_t jMask = min(jEnd, max(jBegin, (seenByAll + 1) / kBKV));
    runBlocks(Parity<0>{}, jBegin, jMask);
    runBlocks(Parity<1>{}, jMask, jEnd);
    waitVmcnt<0>();        // the loads issued past the end of the range may still be on their way into LDS

    const unsigned long long tl2 = p.timeline ? wall_clock64() : 0;
    if (tid == 0) nextRaw = stage.drawBegin(dryXcds, noDraws);     // settled after the epilogue
    rowSum += __shfl_xor(rowSum, 32);
    bool completed = true;
    if (splits > 1) {
      // Leave this split's share in the workspace; the last split to arrive puts the tile together.  The shares are
      // written through to memory as they are stored: left dirty in this XCD's L2 they would be written back by the
      // release below together with everything else that is dirty there, which was measured at 14-20 us per tile
      // when the tiles of half a launch finish together.
      const size_t slot = ((size_t)head * stage.d.grid.y + t.y) * stage.d.grid.z;
      const __amdgpu_buffer_rsrc_t rPart = makeRsrc(p.partO, p.partBytes);
      const uint32_t offO = (uint32_t)(((slot + t.z) * (64 * kThreads) + tid * 4) * sizeof(float));
#pragma unroll
      for (int tt = 0; tt < 4; tt++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
          const floatx4 v = floatx4{o[tt][4 * g], o[tt][4 * g + 1], o[tt][4 * g + 2], o[tt][4 * g + 3]};
          __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uint4v, v), rPart, (int)(offO + (tt * 4 + g) * (kThreads * 16)), 0, 16 /* sc1 */);
        }
      const uint32_t offS = (uint32_t)(((char*)p.partStat - (char*)p.partO) + ((slot + t.z) * (2 * kThreads) + tid) * sizeof(float));
      const float scaledMax = rowMax * p.scaleLog2;      // the running maximum is kept unscaled
      __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, scaledMax), rPart, (int)offS, 0, 16);
      __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, rowSum), rPart, (int)(offS + kThreads * sizeof(float)), 0, 16);
      // The count below is the first thread's, and a workgroup barrier does not wait for stores to memory: every
      // wavefront sees its own through first.
      waitVmcnt<0>();
      __syncthreads();
      uint32_t* counter = p.arrivals + head * stage.d.grid.y + t.y;
      if (tid == 0) {
        const uint32_t before = stage.countIn(counter);      // relaxed: the shares were written through and are acknowledged
        const bool last = before == splits - 1;
        if (last) { cusync::dev::storeRelaxed(counter, 0); stage.countSeen(); }
        sLast = last;
      }
      __syncthreads();
      completed = sLast != 0;
      if (completed) {
        // Splits are added in index order, this one's own share read back like the others, so that the result does
        // not depend on which split arrived last.  The loads are coherent at device scope (sc1) instead of following
        // an acquire fence, which would empty this XCD's L2 under the workgroups still walking their keys; and they
        // are issued two splits at a time: a round trip to memory per split and two more for the row statistics is
        // what this step used to consist of (15 us for two splits).
        auto statOff = [&](uint32_t z) { return (uint32_t)(((char*)p.partStat - (char*)p.partO) + ((slot + z) * (2 * kThreads) + tid) * sizeof(float)); };
        auto loadStat = [&](uint32_t off) { return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rPart, (int)off, 0, 16 /* sc1 */)); };
        float m = kMasked;
        for (uint32_t z = 0; z < splits; z += 4) {
          float a[4];
#pragma unroll
          for (uint32_t q = 0; q < 4; q++) a[q] = z + q < splits ? loadStat(statOff(z + q)) : kMasked;
#pragma unroll
          for (uint32_t q = 0; q < 4; q++) m = fmaxf(m, a[q]);
        }
        rowSum = 0.0f;
#pragma unroll
        for (int tt = 0; tt < 4; tt++)
#pragma unroll
          for (int r = 0; r < 16; r++) o[tt][r] = 0.0f;
        for (uint32_t z = 0; z < splits; z += 2) {
          float sMax[2], sSum[2];
          uint4v v[2][16];
#pragma unroll
          for (uint32_t q = 0; q < 2; q++) {
            const bool valid = z + q < splits;
            const uint32_t zz = valid ? z + q : z;
            sMax[q] = valid ? loadStat(statOff(zz)) : kMasked;
            sSum[q] = loadStat(statOff(zz) + kThreads * sizeof(float));
            const uint32_t off = (uint32_t)(((slot + zz) * (64 * kThreads) + tid * 4) * sizeof(float));
#pragma unroll
            for (int i = 0; i < 16; i++) v[q][i] = __builtin_amdgcn_raw_buffer_load_b128(rPart, (int)(off + i * (kThreads * 16)), 0, 16 /* sc1 */);
          }
#pragma unroll
          for (uint32_t q = 0; q < 2; q++) {
            const float w = __builtin_amdgcn_exp2f(sMax[q] - m);      // 0 for the missing second split of an odd count
            rowSum += w * sSum[q];
#pragma unroll
            for (int tt = 0; tt < 4; tt++)
#pragma unroll
              for (int g = 0; g < 4; g++) {
                const floatx4 f = __builtin_bit_cast(floatx4, v[q][tt * 4 + g]);
#pragma unroll
                for (int e = 0; e < 4; e++) o[tt][4 * g + e] += w * f[e];
              }
          }
        }
      }
    }
    // Normalise and store: register r of tile tt is head-dim 32tt + 8(r/4) + 4hi + r%4 of query myq.
    const float inv = 1.0f / rowSum;
    if (completed && myq < p.S) {
      // written through like the partial results: a post, or another tile's release, then finds nothing to write back
      const __amdgpu_buffer_rsrc_t rOut = makeRsrc(p.out, p.S * p.ldo * 2);
      const uint32_t dst = (myq * p.ldo + head * kHD + 4 * hi) * 2;
#pragma unroll
      for (int tt = 0; tt < 4; tt++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
          half4 v;
#pragma unroll
          for (int e = 0; e < 4; e++) v[e] = (half_t)(o[tt][4 * g + e] * inv);
          __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(uint2v, v), rOut, (int)(dst + (32 * tt + 8 * g) * 2), 0, 16 /* sc1 */);
        }
    }

    // All waves must be past their last LDS read before the next tile's loads
    // land in stage 0; the post (or this barrier) provides that.
    cusync_dim3 done = {q0, head * kHD, 0};
    if (completed && stage.isProducer()) stage.post(done, 1, stage.storesThrough());
    else __syncthreads();
    if (tid == 0) recordTileAt(p.timeline, p.timelineCap, stage, p.launched, t, round, tlEntry, tl0, tl1, tl2, p.timeline ? wall_clock64() : 0);
  }
}

}  // namespace attn
}  // namespace cusync
