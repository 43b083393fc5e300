// Fused multi-head attention (softmax(mask(Q K^T * scale)) V, fp16 in/out, fp32
// accumulate, head width 128) as a CuSync middle stage: it waits for the tiles
// of the QKV projection that hold its Q rows and each K/V block just before it
// loads them, and posts every finished output tile for the output projection.
//
// One workgroup (four wavefronts) owns 128 query rows of one head; each
// wavefront owns 32 of them.  K and V are walked in blocks of 64 rows that go
// from global memory straight into LDS (two stages, the next block loads while
// the current one is multiplied; two workgroups share a CU.  Four stages with
// one workgroup per CU were measured at 2048 rows x 12 heads: 89 us against 70).
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
constexpr int kLdsBytes = 2 * 2 * kStageBytes;      // two stages of K + V
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
};

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
  const uint32_t startToken = tid == 0 ? stage.beginStart() : 0;
  const bool noDraws = stage.allStatic(p.launched);     // every tile is some workgroup's static first tile
  for (uint32_t round = 0;; round++) {
    if (tid == 0) sTicket = round == 0 ? stage.firstTicket(p.launched, dryXcds, noDraws) : stage.drawFinish(nextRaw, p.launched, round, dryXcds, noDraws);
    __syncthreads();
    const uint32_t ticket = sTicket;
    if (ticket >= numTiles) {
      if (tid == 0 && round == 0) stage.finishStart(startToken, p.launched);
      break;
    }
    const cusync_dim3 t = stage.ticketToTile(ticket);
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
    auto issue = [&](uint32_t j, uint32_t st) {
      const uint32_t kLds = ldsBase + st * 2 * kStageBytes + wave * 4 * 1024;
      const uint32_t rowOff = (j * kBKV + ldRow) * p.ldq;
#pragma unroll
      for (int q = 0; q < 4; q++)
        loadToLds(rLds, __builtin_amdgcn_readfirstlane(kLds + q * 1024),
                  (rowOff + q * 4 * p.ldq + E + head * kHD + kChunk[q] * 8) * 2);
#pragma unroll
      for (int q = 0; q < 4; q++)
        loadToLds(rLds, __builtin_amdgcn_readfirstlane(kLds + kStageBytes + q * 1024),
                  (rowOff + q * 4 * p.ldq + 2 * E + head * kHD + vChunk * 8) * 2);
    };
    auto waitKV = [&](uint32_t j) {
      // only the rows behind the cache come from the producer; its tiles count rows from there
      const uint32_t lo = max(j * kBKV, p.cached), hi = min(j * kBKV + (uint32_t)kBKV, total);
      if (lo >= hi) return;
      waitRows(lo - p.cached, hi - p.cached, E + head * kHD);
      waitRows(lo - p.cached, hi - p.cached, 2 * E + head * kHD);
    };

    // Q fragments stay in registers for the whole tile: k-step s is head-dim 16s + 8hi .. + 7 of row myq.
    waitRows(q0, qEnd, head * kHD);
    half8 qf[8];
#pragma unroll
    for (int s = 0; s < 8; s++)
      qf[s] = __builtin_bit_cast(half8, loadChunk(rReg, myq < p.S ? ((p.cached + myq) * p.ldq + head * kHD + 16 * s + 8 * hi) * 2 : kOutOfRange));

    waitKV(jBegin);
    issue(jBegin, 0);
    if (tid == 0 && round == 0) stage.finishStart(startToken, p.launched);

    float rowMax = kMasked, rowSum = 0.0f;      // rowSum: this half-wave's share
    floatx16 o[4];
#pragma unroll
    for (int tt = 0; tt < 4; tt++)
#pragma unroll
      for (int r = 0; r < 16; r++) o[tt][r] = 0.0f;

    for (uint32_t j = jBegin; j < jEnd; j++) {
      const uint32_t st = (j - jBegin) & 1;
      waitVmcnt<0>();
      __builtin_amdgcn_s_barrier();       // block j is in LDS for everyone; everyone is done with block j-1
      asm volatile("" ::: "memory");
      if (j + 1 < jEnd) { waitKV(j + 1); issue(j + 1, st ^ 1); }
      if (p.causal && j * kBKV > p.cached + qw + 31) continue;       // wholly in this wave's future (wave-uniform)

      const char* ks = smem + st * 2 * kStageBytes;
      const char* vs = ks + kStageBytes;

      // S^T = K Q^T for the two 32-row kv tiles of the block
      floatx16 sacc[2];
#pragma unroll
      for (int a = 0; a < 2; a++)
#pragma unroll
        for (int r = 0; r < 16; r++) sacc[a][r] = 0.0f;
#pragma unroll
      for (int s = 0; s < 8; s++)
#pragma unroll
        for (int a = 0; a < 2; a++) {
          const half8 kf = *reinterpret_cast<const half8*>(ks + kFrag[s] + a * 32 * kRowBytes);
          sacc[a] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qf[s], sacc[a], 0, 0, 0);
        }

      // scale, mask, running maximum
      const uint32_t kvBase = j * kBKV + 4 * hi;
      const bool needMask = j * kBKV + kBKV - 1 > (p.causal ? p.cached + min(qw, p.S - 1) : total - 1);
      float blockMax = kMasked;
#pragma unroll
      for (int a = 0; a < 2; a++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          float x = sacc[a][r] * p.scaleLog2;
          if (needMask && kvBase + 32 * a + 8 * (r / 4) + (r % 4) > limit) x = kMasked;
          sacc[a][r] = x;
          blockMax = fmaxf(blockMax, x);
        }
      blockMax = fmaxf(blockMax, __shfl_xor(blockMax, 32));
      const float newMax = fmaxf(rowMax, blockMax);
      const float alpha = __builtin_amdgcn_exp2f(rowMax - newMax);
      rowMax = newMax;

      // P^T = exp2(S^T - max), as fp16 B operands of the second product
      half8 pf[4];
      float blockSum = 0.0f;
#pragma unroll
      for (int a = 0; a < 2; a++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const float e = __builtin_amdgcn_exp2f(sacc[a][r] - newMax);
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
      typedef short4v __attribute__((address_space(3))) * lds_ptr;
#pragma unroll
      for (int u = 0; u < 4; u++)
#pragma unroll
        for (int tt = 0; tt < 4; tt++) {
          const char* q = vs + ((tt & 1) ? vOdd + (tt - 1) * 64 : vEven + tt * 64) + u * 16 * kRowBytes;
          const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(q));
          const short4v up = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(q + 8 * kRowBytes));
          const half4 l4 = __builtin_bit_cast(half4, lo), u4 = __builtin_bit_cast(half4, up);
          const half8 vf = __builtin_shufflevector(l4, u4, 0, 1, 2, 3, 4, 5, 6, 7);
          o[tt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pf[u], o[tt], 0, 0, 0);
        }
    }

    if (tid == 0) nextRaw = stage.drawBegin(dryXcds, noDraws);     // settled after the epilogue
    rowSum += __shfl_xor(rowSum, 32);
    bool completed = true;
    if (splits > 1) {
      // leave this split's share in the workspace; the last split to arrive puts the tile together
      const size_t slot = ((size_t)head * stage.d.grid.y + t.y) * stage.d.grid.z;
      float* po = p.partO + (slot + t.z) * (64 * kThreads) + tid * 4;
#pragma unroll
      for (int tt = 0; tt < 4; tt++)
#pragma unroll
        for (int g = 0; g < 4; g++)
          *reinterpret_cast<floatx4*>(po + (tt * 4 + g) * (kThreads * 4)) = floatx4{o[tt][4 * g], o[tt][4 * g + 1], o[tt][4 * g + 2], o[tt][4 * g + 3]};
      float* ps = p.partStat + (slot + t.z) * (2 * kThreads) + tid;
      ps[0] = rowMax;
      ps[kThreads] = rowSum;
      __syncthreads();
      uint32_t* counter = p.arrivals + head * stage.d.grid.y + t.y;
      if (tid == 0) {
        const uint32_t before = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
        const bool last = before == splits - 1;
        if (last) cusync::dev::storeRelaxed(counter, 0);
        sLast = last;
      }
      __syncthreads();
      completed = sLast != 0;
      if (completed) {
        cusync::dev::acquireFence();
        float m = kMasked;
        for (uint32_t z = 0; z < splits; z++) m = fmaxf(m, p.partStat[(slot + z) * (2 * kThreads) + tid]);
        rowSum = 0.0f;
#pragma unroll
        for (int tt = 0; tt < 4; tt++)
#pragma unroll
          for (int r = 0; r < 16; r++) o[tt][r] = 0.0f;
        for (uint32_t z = 0; z < splits; z++) {
          const float* qs = p.partStat + (slot + z) * (2 * kThreads) + tid;
          const float w = __builtin_amdgcn_exp2f(qs[0] - m);
          rowSum += w * qs[kThreads];
          const float* qo = p.partO + (slot + z) * (64 * kThreads) + tid * 4;
#pragma unroll
          for (int tt = 0; tt < 4; tt++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
              const floatx4 v = *reinterpret_cast<const floatx4*>(qo + (tt * 4 + g) * (kThreads * 4));
#pragma unroll
              for (int e = 0; e < 4; e++) o[tt][4 * g + e] += w * v[e];
            }
        }
      }
    }
    // Normalise and store: register r of tile tt is head-dim 32tt + 8(r/4) + 4hi + r%4 of query myq.
    const float inv = 1.0f / rowSum;
    if (completed && myq < p.S) {
      half_t* dst = p.out + (size_t)myq * p.ldo + head * kHD + 4 * hi;
#pragma unroll
      for (int tt = 0; tt < 4; tt++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
          half4 v;
#pragma unroll
          for (int e = 0; e < 4; e++) v[e] = (half_t)(o[tt][4 * g + e] * inv);
          *reinterpret_cast<half4*>(dst + 32 * tt + 8 * g) = v;
        }
    }

    // All waves must be past their last LDS read before the next tile's loads
    // land in stage 0; the post (or this barrier) provides that.
    cusync_dim3 done = {q0, head * kHD, 0};
    if (completed && stage.isProducer()) stage.post(done);
    else __syncthreads();
  }
}

}  // namespace attn
}  // namespace cusync
