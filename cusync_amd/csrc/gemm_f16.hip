// Sync-aware fp16 GEMM for gfx950 (MI355X):  D = epilogue(A x B), fp32 accumulate.
//
// Stands in for the CUTLASS kernel of the reference
// (src/include/cutlass/cusync-cutlass/include/cutlass/gemm/kernel/cusyncgemm.h:208-399
// and its main loops gemm/threadblock/cusyncmma_multistage.h:943-1200) with the
// same three hooks — next tile at entry, wait before loading a tile of the
// synchronised operand A, post after the epilogue — but is written for CDNA4:
//
//  * 256 threads = 4 wavefronts of 64 lanes in a WM x WN arrangement; each
//    wavefront owns (BM/WM) x (BN/WN) of the output as 32x32 MFMA tiles
//    (v_mfma_f32_32x32x16_f16), accumulators stay in registers.
//  * A and B tiles are fetched with 16-byte buffer loads into registers one K
//    chunk ahead, then staged in LDS.  A is kept [m][k] with a 16-byte row pad;
//    B is kept [k][n] exactly as it lies in memory and read with the LDS
//    transpose load (ds_read_b64_tr_b16), which hands each lane the four
//    consecutive k of one column that the MFMA wants.  No register transposes.
//  * The MFMA is issued with B as its first operand, so a lane ends up with four
//    consecutive columns of one output row and writes 8 bytes at a time.
//  * The launch is persistent: at most as many workgroups as stay resident,
//    each drawing tile tickets until the stage has no tiles left.
//  * Buffer descriptors bound every load to the operand's extent, so ragged M
//    (B = 1, 16, ...) reads zeros instead of faulting.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <utility>
#include <mutex>
#include <string>

#include "../../include/cusync_amd.h"
#include "rt_internal.h"
#include "stage_device.h"

namespace {

typedef _Float16 half_t;
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint2v __attribute__((ext_vector_type(2)));

constexpr int kThreads = 256;
constexpr uint32_t kOutOfRange = 0x80000000u;   // buffer offset beyond any descriptor we build

struct GemmParams {
  cusync::DynStage stage;
  uint32_t M, N, K;
  const half_t* A; uint32_t lda;
  const half_t* B; uint32_t ldb;
  half_t* D; uint32_t ldd;
  int32_t epilogue;
  int32_t a_mode;
  uint32_t launched;       // workgroups in this launch
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t makeRsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

__device__ __forceinline__ uint4v loadChunk(__amdgpu_buffer_rsrc_t r, uint32_t byteOffset) {
  return __builtin_amdgcn_raw_buffer_load_b128(r, (int)byteOffset, 0, 0);
}

// erf by Abramowitz & Stegun 7.1.26 (|error| <= 1.5e-7), enough for an fp16 result
// and a third of the instructions of the library erff.
__device__ __forceinline__ float fastErf(float x) {
  const float ax = __builtin_fabsf(x);
  const float t = __builtin_amdgcn_rcpf(1.0f + 0.3275911f * ax);
  float poly = 1.061405429f;
  poly = poly * t - 1.453152027f;
  poly = poly * t + 1.421413741f;
  poly = poly * t - 0.284496736f;
  poly = poly * t + 0.254829592f;
  poly *= t;
  const float e = __expf(-ax * ax);
  const float r = 1.0f - poly * e;
  return __builtin_copysignf(r, x);
}

__device__ __forceinline__ float applyEpilogue(float v, int epilogue) {
  if (epilogue == CUSYNC_EPILOGUE_GELU) return 0.5f * v * (1.0f + fastErf(v * 0.70710678118654752f));
  if (epilogue == CUSYNC_EPILOGUE_RELU) return v > 0.0f ? v : 0.0f;
  return v;
}

__device__ __forceinline__ float siluf(float x) { return x * __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }

// A[m,k] = silu(gate) * up, element-wise on one 16-byte chunk.
__device__ __forceinline__ uint4v swigluChunk(uint4v gate, uint4v up) {
  half8 g = __builtin_bit_cast(half8, gate);
  half8 u = __builtin_bit_cast(half8, up);
  half8 r;
#pragma unroll
  for (int i = 0; i < 8; i++) r[i] = (half_t)(siluf((float)g[i]) * (float)u[i]);
  return __builtin_bit_cast(uint4v, r);
}

// Instruction-order directives for the scheduler (groups of one kind of
// instruction, placed in the order the directives appear).  Without them the
// compiler serialises "LDS read, wait, two MFMAs", which leaves the matrix
// pipe idle for the whole LDS latency when only one wavefront runs per SIMD.
constexpr int kSchedMfma = 0x008, kSchedDsRead = 0x100, kSchedDsWrite = 0x200;

template<int MASK, int SIZE>
__device__ __forceinline__ void schedGroup() {
  if constexpr (SIZE > 0) __builtin_amdgcn_sched_group_barrier(MASK, SIZE, 0);
}

// Share of `total` items that falls to slot `i` of `slots` when spread evenly.
constexpr int evenShare(int total, int slots, int i) { return (total * (i + 1)) / slots - (total * i) / slots; }

// Order of one pass over an LDS stage: STEPS k-steps of NM MFMAs each.  The R
// LDS reads that fetch the fragments of k-step s+1 are spread between the
// MFMAs of k-step s; the W LDS writes that stage the next K chunk are spread
// over the MFMAs of the second half of the pass, as late as possible so that
// the global loads feeding them have had time to land.
template<int STEPS, int NM, int R, int W, int S = 0, int M = 0>
__device__ __forceinline__ void schedPass() {
  if constexpr (S == 0 && M == 0) schedGroup<kSchedDsRead, R>();        // fragments of k-step 0
  if constexpr (S < STEPS) {
    constexpr int FIRST_W = STEPS / 2;                                  // first k-step that carries writes
    constexpr int W_SLOTS = (STEPS - FIRST_W) * NM;
    schedGroup<kSchedMfma, 1>();
    if constexpr (S + 1 < STEPS) schedGroup<kSchedDsRead, evenShare(R, NM, M)>();
    if constexpr (S >= FIRST_W) schedGroup<kSchedDsWrite, evenShare(W, W_SLOTS, (S - FIRST_W) * NM + M)>();
    if constexpr (M + 1 < NM) schedPass<STEPS, NM, R, W, S, M + 1>();
    else schedPass<STEPS, NM, R, W, S + 1, 0>();
  }
}

template<int BM_, int BN_, int BK_, int WM_, int WN_>
struct TileCfg {
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_;
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

template<int P> struct Parity { static constexpr int value = P; };

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
  __shared__ uint32_t sTicket;
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

  if (tid == 0) stage.announceStart(p.launched);

  const uint32_t numTiles = stage.numTiles();
  const uint32_t nk = (p.K + C::BK - 1) / C::BK;
  const bool consumer = stage.isConsumer();
  const uint32_t tmq = consumer ? stage.d.in.tileM : 1, tnq = consumer ? stage.d.in.tileN : 1;
  // Policies that synchronise once per row of tiles (RowSync, ConsecutiveSync) are
  // handled entirely by the pre-loop wait; only the others wait per K chunk.
  const bool chunkSync = consumer && stage.d.in.kind != CUSYNC_POLICY_ROWSYNC &&
                         stage.d.in.kind != CUSYNC_POLICY_CONSECUTIVESYNC;

  for (uint32_t round = 0;; round++) {
    if (tid == 0) sTicket = stage.drawTicket(p.launched, round);
    __syncthreads();
    const uint32_t ticket = sTicket;
    if (ticket >= numTiles) break;
    const cusync_dim3 t = stage.ticketToTile(ticket);      // x = column tile, y = row tile
    const uint32_t m0 = t.y * C::BM, n0 = t.x * C::BN;
    const uint32_t mEnd = min(m0 + (uint32_t)C::BM, p.M);

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
    uint32_t nextColTile = 0;        // producer column tiles below this one have been waited for
    uint32_t nextColTileUp = swiglu ? p.K / tnq : 0;
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
        if (!stage.needsWait(w) || polledValue >= stage.waitTarget()) return;
      }
      waitRows(ct * tnq, 0);
    };
    auto waitChunk = [&](uint32_t k0) {
      if (!chunkSync) return;
      const uint32_t kLast = min(k0 + (uint32_t)C::BK, p.K) - 1;
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
      if (!oneRowBlock || k0 >= p.K) return;
      const uint32_t ct = k0 / tnq;
      if (ct < nextColTile || ct == polledTile) return;
      cusync_dim3 w = {m0, ct * tnq, 0};
      if (!stage.needsWait(w)) return;
      polledTile = ct;
      polledValue = stage.peek(w);
    };

    auto issue = [&](auto P, uint32_t kt) {
      constexpr int S = decltype(P)::value;
      const uint32_t k0 = kt * C::BK;
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
      earlyPoll((kt + 3) * C::BK);
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
    earlyPoll(2 * C::BK);
    stash(Parity<0>{});
    __syncthreads();

    for (uint32_t kt = 0; kt < nk; kt += 2) {
      step(Parity<0>{}, kt);
      if (kt + 1 < nk) step(Parity<1>{}, kt + 1);
    }

    // Epilogue.  acc[i][j][r] of lane l is output row  m = .. + (l & 31)  and
    // column  n = .. + 8*(r/4) + 4*(l/32) + r%4.
#pragma unroll
    for (int i = 0; i < C::TM; i++) {
      const uint32_t m = m0 + wm * C::WTM + i * 32 + (lane & 31);
#pragma unroll
      for (int j = 0; j < C::TN; j++) {
#pragma unroll
        for (int g = 0; g < 4; g++) {
          const uint32_t n = n0 + wn * C::WTN + j * 32 + 8 * g + 4 * (lane >> 5);
          half4 o;
#pragma unroll
          for (int e = 0; e < 4; e++) o[e] = (half_t)applyEpilogue(acc[i][j][g * 4 + e], p.epilogue);
          if (m < p.M && n < p.N)
            *reinterpret_cast<half4*>(p.D + (size_t)m * p.ldd + n) = o;
        }
      }
    }

    cusync_dim3 done = {m0, n0, t.z};
    stage.post(done);    // barrier inside when the stage is a producer
  }
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------

struct TileInfo {
  uint32_t bm, bn, bk;
  size_t lds;
  void (*kernel[2])(GemmParams);   // [plain A, SwiGLU A]
  int residentPerCU;     // filled lazily
};

#define CUSYNC_TILE(BM, BN, BK, WM, WN) \
  { BM, BN, BK, (size_t)TileCfg<BM, BN, BK, WM, WN>::LDS_BYTES, \
    { gemmKernel<TileCfg<BM, BN, BK, WM, WN>, false>, gemmKernel<TileCfg<BM, BN, BK, WM, WN>, true> }, -1 }

TileInfo g_tiles[CUSYNC_TILE_COUNT] = {
  CUSYNC_TILE(256, 256, 32, 2, 2),   // CUSYNC_TILE_256x256x32
  CUSYNC_TILE(256, 128, 64, 2, 2),   // CUSYNC_TILE_256x128x64
  CUSYNC_TILE(128, 128, 64, 2, 2),   // CUSYNC_TILE_128x128x64
  CUSYNC_TILE(64, 128, 64, 1, 4),    // CUSYNC_TILE_64x128x64
  CUSYNC_TILE(32, 128, 64, 1, 4),    // CUSYNC_TILE_32x128x64
  CUSYNC_TILE(128, 256, 64, 2, 2),   // CUSYNC_TILE_128x256x64
  CUSYNC_TILE(256, 64, 64, 4, 1),    // CUSYNC_TILE_256x64x64
  CUSYNC_TILE(128, 64, 64, 2, 2),    // CUSYNC_TILE_128x64x64
};

std::mutex g_mutex;
int g_numCUs = 0;

TileInfo* tileInfo(int tile) {
  if (tile < 0 || tile >= CUSYNC_TILE_COUNT) return nullptr;
  return &g_tiles[tile];
}

int residentWorkgroups(int tile) {
  TileInfo* ti = tileInfo(tile);
  if (!ti) return 0;
  std::lock_guard<std::mutex> lock(g_mutex);
  if (ti->residentPerCU < 0) {
    if (g_numCUs == 0) {
      int dev = 0;
      hipDeviceProp_t prop;
      if (CUSYNC_HIP(hipGetDevice(&dev)) || CUSYNC_HIP(hipGetDeviceProperties(&prop, dev))) return 0;
      g_numCUs = prop.multiProcessorCount;
    }
    int perCU = 1 << 30;
    for (int v = 0; v < 2; v++) {
      if (CUSYNC_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(ti->kernel[v]),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)ti->lds))) return 0;
      int n = 0;
      if (CUSYNC_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, ti->kernel[v], kThreads, ti->lds))) return 0;
      perCU = std::min(perCU, n);
    }
    ti->residentPerCU = perCU;
  }
  return ti->residentPerCU * g_numCUs;
}

}  // namespace

extern "C" {

int cusync_gemm_tile_shape(int tile, uint32_t* tileM, uint32_t* tileN, uint32_t* tileK) {
  TileInfo* ti = tileInfo(tile);
  if (!ti) return 1;
  if (tileM) *tileM = ti->bm;
  if (tileN) *tileN = ti->bn;
  if (tileK) *tileK = ti->bk;
  return 0;
}

cusync_dim3 cusync_gemm_grid(int tile, uint32_t M, uint32_t N, int split_k) {
  cusync_dim3 g = {0, 0, 0};
  TileInfo* ti = tileInfo(tile);
  if (!ti) return g;
  g.x = (N + ti->bn - 1) / ti->bn;
  g.y = (M + ti->bm - 1) / ti->bm;
  g.z = split_k > 0 ? (uint32_t)split_k : 1;
  return g;
}

int cusync_gemm_max_resident(int tile) { return residentWorkgroups(tile); }

cusync_error cusync_gemm_can_implement(const cusync_gemm_args* a) {
  using cusync::rt::setError;
  if (!a) return CUSYNC_ERROR_NOT_INITIALIZED;
  TileInfo* ti = tileInfo(a->tile);
  if (!ti) { setError("gemm: unknown tile id"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (a->M == 0 || a->N == 0 || a->K == 0) { setError("gemm: empty problem"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (a->K % 8 || a->N % 8) { setError("gemm: K and N must be multiples of 8 (16-byte loads)"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (a->lda % 8 || a->ldb % 8 || a->ldd % 4) { setError("gemm: leading dimensions must keep 16-byte alignment"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  const uint32_t aCols = a->a_mode == CUSYNC_A_SWIGLU ? 2 * a->K : a->K;
  if (a->lda < aCols || a->ldb < a->N || a->ldd < a->N) { setError("gemm: leading dimension smaller than the row"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if ((uint64_t)a->M * a->lda * 2 >= 0x80000000ull || (uint64_t)a->K * a->ldb * 2 >= 0x80000000ull) {
    setError("gemm: operand larger than 2 GiB is not addressable by one buffer descriptor");
    return CUSYNC_ERROR_NOT_INITIALIZED;
  }
  if (((uintptr_t)a->A | (uintptr_t)a->B) % 16 || (uintptr_t)a->D % 8) { setError("gemm: misaligned operand"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (a->split_k > 1) { setError("gemm: split_k > 1 is not built"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (a->a_mode != CUSYNC_A_PLAIN && a->a_mode != CUSYNC_A_SWIGLU) { setError("gemm: unknown a_mode"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (a->epilogue < 0 || a->epilogue > CUSYNC_EPILOGUE_RELU) { setError("gemm: unknown epilogue"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  const cusync_dim3 g = cusync_gemm_grid(a->tile, a->M, a->N, a->split_k);
  const cusync_stage_desc& s = a->stage;
  if (s.grid.x != g.x || s.grid.y != g.y || s.grid.z != g.z) {
    setError("gemm: stage grid does not match cusync_gemm_grid(tile, M, N, split_k)");
    return CUSYNC_ERROR_NOT_INITIALIZED;
  }
  if (!s.tileOrder || !s.tileCounter || !s.startCounter || !s.spinTimeouts) { setError("gemm: stage not allocated"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (s.out.kind != CUSYNC_POLICY_NOSYNC && !s.tileStatusWrite) { setError("gemm: producer stage without semaphores"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (s.in.kind != CUSYNC_POLICY_NOSYNC) {
    if (!s.tileStatusRead) { setError("gemm: consumer stage not paired with a producer"); return CUSYNC_ERROR_NOT_INITIALIZED; }
    if (s.in.tileM == 0 || s.in.tileN == 0) { setError("gemm: input policy with zero tile extent"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  }
  if ((s.opts & CUSYNC_OPT_NO_ATOMIC_ADD) && s.out.kind != CUSYNC_POLICY_NOSYNC &&
      cusync::dyn::waitValue(s.out) != cusync::dyn::postValue(s.out)) {
    setError("gemm: NoAtomicAdd needs a policy whose wait value equals its post value");
    return CUSYNC_ERROR_NOT_INITIALIZED;
  }
  return CUSYNC_SUCCESS;
}

size_t cusync_gemm_workspace_size(const cusync_gemm_args* a) {
  (void)a;
  return 0;
}

cusync_error cusync_gemm_run(const cusync_gemm_args* a, void* stream) {
  cusync_error e = cusync_gemm_can_implement(a);
  if (e != CUSYNC_SUCCESS) return e;
  TileInfo* ti = tileInfo(a->tile);
  const int resident = residentWorkgroups(a->tile);
  if (resident <= 0) { cusync::rt::setError("gemm: kernel does not fit on a CU"); return CUSYNC_ERROR_DEVICE; }
  const cusync_stage_desc& s = a->stage;
  const uint32_t tiles = s.grid.x * s.grid.y * s.grid.z;
  uint32_t launched = std::min<uint32_t>(tiles, (uint32_t)resident);
  if (a->max_workgroups > 0) launched = std::min<uint32_t>(launched, (uint32_t)a->max_workgroups);

  GemmParams p;
  p.stage.d = s;
  // Producer tiles are whole 128-byte lines of A when the row pitch, the base and
  // the producer's tile width all are multiples of 128 bytes (64 halfs).
  p.stage.lineAligned = s.in.kind != CUSYNC_POLICY_NOSYNC && (uintptr_t)a->A % 128 == 0 &&
                        (a->lda * 2) % 128 == 0 && (s.in.tileN * 2) % 128 == 0;
  p.M = a->M; p.N = a->N; p.K = a->K;
  p.A = (const half_t*)a->A; p.lda = a->lda;
  p.B = (const half_t*)a->B; p.ldb = a->ldb;
  p.D = (half_t*)a->D; p.ldd = a->ldd;
  p.epilogue = a->epilogue;
  p.a_mode = a->a_mode;
  p.launched = launched;
  hipLaunchKernelGGL(ti->kernel[a->a_mode == CUSYNC_A_SWIGLU ? 1 : 0], dim3(launched), dim3(kThreads), ti->lds, (hipStream_t)stream, p);
  if (CUSYNC_HIP(hipGetLastError())) return CUSYNC_ERROR_DEVICE;
  return CUSYNC_SUCCESS;
}

}  // extern "C"
