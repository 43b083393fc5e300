// Pieces shared by the fp16 GEMM kernels: parameter block, buffer-descriptor
// loads, epilogue math and the instruction-order directives.
#pragma once

#include <type_traits>

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <utility>

#include "../../include/cusync_amd.h"
#include "stage_device.h"

namespace cusync {
namespace gemm {


typedef _Float16 half_t;
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint2v __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

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
  // split-K: slice z of a tile covers K columns [z*kPerSlice, (z+1)*kPerSlice)
  uint32_t splitK, kPerSlice;
  float* partials;         // [splitK][m-tiles][n-tiles][BM*BN] fp32 partial sums in register order
  uint32_t* arrivals;      // [2][m-tiles * n-tiles] slices that wrote their partial sums / that stored their share, per output tile; 0 between launches
  // Split-K where every k-slice of the launch has a workgroup of its own from the start (one round, all resident):
  // the slices of a tile wait for each other and each adds up and stores a share of the tile (whole 32-row
  // pieces of it), instead of the slice that arrives last doing all of it while the others' CUs idle.  Set by the
  // launcher; needs BM/32 to be a multiple of splitK.
  uint32_t coopReduce;
  uint32_t partialBytes;   // size of `partials`, for the buffer descriptor of the write-through stores
  uint32_t mPad;           // m-tiles * BM
  // Consumer whose producer's tiles are not whole 128-byte lines of A (a tile policy with a tile width that is
  // not a multiple of 64 halfs): 64, and every wait of a K chunk then covers all producer column tiles that
  // reach into the lines the chunk touches, not only the columns it reads.  A line is then never fetched
  // before everything in it has been posted, so no stale line can sit in this XCD's caches and the waits can
  // do without the cache invalidation (DynStage::lineAligned).  1 otherwise.
  uint32_t waitRound;
  // Diagnosis (cusync_rt_set_timeline): null, or a buffer of 64-bit words, word 0 the number of records written
  // so far, then records of eight words per finished tile (see recordTile).
  unsigned long long* timeline;
  uint32_t timelineCap;    // records the buffer holds
  // implicit-GEMM convolution (A is gathered from an NHWC tensor): M = n*P*Q, K = R*S*C, k = (r*S + s)*C + c
  uint32_t cvN, cvH, cvW, cvC, cvP, cvQ, cvR, cvS, cvPad, cvStride;
};

enum { kAPlain = 0, kAConv = 1 };

// One record of the diagnosis timeline, written by the first thread of a workgroup when a tile is done:
// [0] role (1 producer, 2 consumer, 3 both, 0 neither) | workgroup index << 8 | XCD id << 40
// [1] tile x | y << 16 | z << 32 | tiles this workgroup did before << 48
// [2..6] constant-rate 100 MHz clock: tile drawn, first loads issued (the waits of the first chunks are over),
//        main loop done, epilogue and post done, and the clock at kernel entry of this workgroup;  [7] launched
__device__ __forceinline__ void recordTileAt(unsigned long long* timeline, uint32_t timelineCap, const cusync::DynStage& stage,
                                             uint32_t launched, const cusync_dim3& t, uint32_t round,
                                             unsigned long long tEntry, unsigned long long t0, unsigned long long t1,
                                             unsigned long long t2, unsigned long long t3) {
  if (!timeline) return;
  const unsigned long long slot = __hip_atomic_fetch_add(timeline, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (slot >= timelineCap) return;
  unsigned long long* r = timeline + 1 + slot * 8;
  const uint32_t role = (stage.isProducer() ? 1u : 0u) | (stage.isConsumer() ? 2u : 0u);
  const uint32_t xcc = __builtin_amdgcn_s_getreg((3 << 11) | 20);       // HW_REG_XCC_ID, bits 0..3
  r[0] = role | ((unsigned long long)cusync::DynStage::workgroupIndex() << 8) | ((unsigned long long)xcc << 40);
  r[1] = t.x | ((unsigned long long)t.y << 16) | ((unsigned long long)t.z << 32) | ((unsigned long long)round << 48);
  r[2] = t0; r[3] = t1; r[4] = t2; r[5] = t3; r[6] = tEntry; r[7] = launched;
}
__device__ __forceinline__ void recordTile(const GemmParams& p, const cusync_dim3& t, uint32_t round,
                                           unsigned long long tEntry, unsigned long long t0, unsigned long long t1,
                                           unsigned long long t2, unsigned long long t3) {
  recordTileAt(p.timeline, p.timelineCap, p.stage, p.launched, t, round, tEntry, t0, t1, t2, t3);
}

// First output column of the tile whose first column of the product is n0: the SwiGLU epilogue folds pairs of
// column groups, so its tiles are half as wide in the output, and that is what a consumer's policy sees.
__device__ __forceinline__ uint32_t outputColumn(const GemmParams& p, uint32_t n0) {
  return p.epilogue == CUSYNC_EPILOGUE_SWIGLU ? n0 / 2 : n0;
}
// Posts of the output policy one finished tile stands for.  StridedSync folds the tile of the gate columns and
// the tile of the up columns of one column range onto one semaphore that counts to two
// (src/ml-bench/transformer/mlp.cu:76-101); a tile of the SwiGLU epilogue holds both and posts for both.
__device__ __forceinline__ uint32_t postsPerTile(const GemmParams& p) {
  return p.epilogue == CUSYNC_EPILOGUE_SWIGLU && p.stage.d.out.kind == CUSYNC_POLICY_STRIDEDSYNC ? p.stage.d.out.stride : 1;
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t makeRsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

__device__ __forceinline__ uint4v loadChunk(__amdgpu_buffer_rsrc_t r, uint32_t byteOffset) {
  return __builtin_amdgcn_raw_buffer_load_b128(r, (int)byteOffset, 0, 0);
}

// GeLU, 0.5 v (1 + erf(v / sqrt 2)), with the same erf (A&S 7.1.26, |error| <= 1.5e-7) written out for the two signs:
// erf(|x|) = 1 - P e with P = poly(t) t, t = 1 / (1 + p |x|), e = exp(-x^2), so that
//   v >= 0:  0.5 v (2 - P e) = v - 0.5 |v| P e        v < 0:  0.5 v (P e) = -0.5 |v| P e
// i.e. max(v, 0) - |v| (0.5 P) e: eleven full-rate and two transcendental instructions per value instead of fourteen
// and two (the epilogue of a GeLU tile is bound by exactly these: 96 values per lane, two wavefronts per SIMD), and
// without the cancellation of 1 + erf for negative v.
__device__ __forceinline__ float geluErf(float v) {
  const float av = __builtin_fabsf(v);
  const float t = __builtin_amdgcn_rcpf(__builtin_fmaf(0.3275911f * 0.70710678118654752f, av, 1.0f));
  float poly = 0.5f * 1.061405429f;
  poly = __builtin_fmaf(poly, t, 0.5f * -1.453152027f);
  poly = __builtin_fmaf(poly, t, 0.5f * 1.421413741f);
  poly = __builtin_fmaf(poly, t, 0.5f * -0.284496736f);
  poly = __builtin_fmaf(poly, t, 0.5f * 0.254829592f);
  poly *= t;
  const float s = v * 0.84932180028801904f;          // sqrt(0.5 * log2(e)): exp(-v^2 / 2) = exp2(-(s s))
  const float e = __builtin_amdgcn_exp2f(-(s * s));
  return __builtin_fmaf(-(poly * e), av, __builtin_fmaxf(v, 0.0f));
}

// The epilogue kind is a template argument: asked per value at run time, even the plain conversion cost the
// 256x384 tile 8 us per tile in scalar compares and branches (its 192 values per lane), and GeLU 3 us more
// than its arithmetic.  Callers branch once per pass of a tile (TileStore::pass).
template<int EPILOGUE>
__device__ __forceinline__ float applyEpilogue(float v) {
  if constexpr (EPILOGUE == CUSYNC_EPILOGUE_GELU) return geluErf(v);
  else if constexpr (EPILOGUE == CUSYNC_EPILOGUE_RELU) return v > 0.0f ? v : 0.0f;
  else return v;
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

// True for the tile configurations whose K loop is assembly (DmaCfg::PINGPONG).
template<class C, class = void> struct IsAssemblyTile : std::false_type {};
template<class C> struct IsAssemblyTile<C, std::enable_if_t<C::PINGPONG>> : std::true_type {};

// Stores of an output tile.  Final values go through LDS so that global memory sees whole rows: a lane holds 4
// consecutive columns of 32 different rows, which stored directly would be 8-byte pieces scattered over 32 cache
// lines per instruction.  One pass per MFMA row tile: every wave writes its 32 rows x WTN columns (fp16, epilogue
// applied) into a [WM*32][BN] buffer (rows padded by 16 bytes against bank conflicts), then all threads copy the
// buffer out, 16 bytes per lane, consecutive lanes along a row.
// pass(i, rows, value): MFMA row tile i of every wave, value(j, g) its four floats of tile j, group g; bit w of
// `rows` set = the waves of wave row w write their 32 rows of this pass and those rows are stored.
// CUSYNC_EPILOGUE_SWIGLU: the tile's columns are gate and up columns in alternating groups of eight, and in the
// MFMA result layout group g of a lane is columns 8g + 4*(lane/32) + 0..3 of its 32-column tile: groups 0 and 2
// are gate values, groups 1 and 3 the up values of the same output columns.  The tile's output is BN/2 wide.
template<class C>
struct TileStore {
  const GemmParams& p;
  char* lds;
  uint32_t m0, n0;
  int wm, wn, lane;
  uint32_t tid;        // threadIdx.x, opaque to the compiler where the K loop is assembly (see the constructor)
  bool through;
  __amdgpu_buffer_rsrc_t rD;
  static constexpr uint32_t kAllRows = (1u << C::WM) - 1;

  __device__ __forceinline__ TileStore(const GemmParams& p_, const cusync_dim3& t, int wm_, int wn_, int lane_, char* lds_)
      : p(p_), lds(lds_), m0(t.y * C::BM), n0(t.x * C::BN), wm(wm_), wn(wn_), lane(lane_), tid(threadIdx.x), through(p_.stage.storesThrough()),
        rD(makeRsrc(p_.D, p_.M * p_.ldd * 2)) {
    // Everything the copy-out computes per thread (piece index -> row, column, offset) depends on the thread index
    // only, so the compiler works it out once, ahead of the tile loop, and keeps it live across the K loop: where
    // that loop is assembly with most registers named, those values wait in scratch and every tile's epilogue
    // reloads them.  Made opaque here, they are computed where they are used.
    if constexpr (IsAssemblyTile<C>::value) {
      asm volatile("" : "+v"(tid));
      asm volatile("" : "+v"(lane));
    }
  }

  template<class V>
  __device__ __forceinline__ void passPairs(int i, uint32_t rows, V&& value) const {
    constexpr int PITCH = C::BN + 16;                 // BN/2 halfs and the pad
    constexpr int ROWS = C::WM * 32;
    constexpr int CPR = C::BN / 16;
    static_assert(ROWS * PITCH <= C::LDS_BYTES, "epilogue buffer fits the pipeline stages");
    static_assert((ROWS * CPR) % C::THREADS == 0, "whole copy steps");
    constexpr int STEPS = ROWS * CPR / C::THREADS;
    __syncthreads();
    if ((rows >> wm) & 1) {
#pragma unroll
      for (int j = 0; j < C::TN; j++)
#pragma unroll
        for (int gp = 0; gp < 2; gp++) {
          const floatx4 vg = value(j, 2 * gp), vu = value(j, 2 * gp + 1);
          half4 o;
#pragma unroll
          for (int e = 0; e < 4; e++) o[e] = (half_t)(siluf(vg[e]) * vu[e]);
          *reinterpret_cast<half4*>(lds + (wm * 32 + (lane & 31)) * PITCH + (wn * (C::WTN / 2) + j * 16 + 8 * gp + 4 * (lane >> 5)) * 2) = o;
        }
    }
    __syncthreads();
#pragma unroll
    for (int s = 0; s < STEPS; s++) {
      const uint32_t idx = s * C::THREADS + tid;
      const uint32_t lr = idx / CPR, c = idx % CPR;
      const uint32_t m = m0 + (lr / 32) * C::WTM + i * 32 + lr % 32, n = n0 / 2 + c * 8;
      const bool inside = m < p.M && n < p.N / 2 && ((rows >> (lr / 32)) & 1);
      const uint4v v = *reinterpret_cast<const uint4v*>(lds + lr * PITCH + c * 16);
      const int off = inside ? (int)((m * p.ldd + n) * 2) : (int)kOutOfRange;
      if (through) __builtin_amdgcn_raw_buffer_store_b128(v, rD, off, 0, 16 /* sc1 */);
      else __builtin_amdgcn_raw_buffer_store_b128(v, rD, off, 0, 0);
    }
  }

  // This wave's 32 rows x WTN columns of a pass into the buffer, one kind of epilogue applied.
  template<int EPILOGUE, int PITCH, class V>
  __device__ __forceinline__ void writeRows(V&& value) const {
#pragma unroll
    for (int j = 0; j < C::TN; j++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const floatx4 v = value(j, g);
        half4 o;
#pragma unroll
        for (int e = 0; e < 4; e++) o[e] = (half_t)applyEpilogue<EPILOGUE>(v[e]);
        *reinterpret_cast<half4*>(lds + (wm * 32 + (lane & 31)) * PITCH + (wn * C::WTN + j * 32 + 8 * g + 4 * (lane >> 5)) * 2) = o;
      }
  }

  template<class V>
  __device__ __forceinline__ void pass(int i, uint32_t rows, V&& value) const {
    if (p.epilogue == CUSYNC_EPILOGUE_SWIGLU) { passPairs(i, rows, value); return; }
    constexpr int PITCH = C::BN * 2 + 16;
    constexpr int ROWS = C::WM * 32;
    constexpr int CPR = C::BN / 8;
    static_assert(ROWS * PITCH <= C::LDS_BYTES, "epilogue buffer fits the pipeline stages");
    static_assert((ROWS * CPR) % C::THREADS == 0, "whole copy steps");
    __syncthreads();       // the buffer is free: main-loop reads, or the previous pass, are done
    if ((rows >> wm) & 1) {
      if (p.epilogue == CUSYNC_EPILOGUE_GELU) writeRows<CUSYNC_EPILOGUE_GELU, PITCH>(value);
      else if (p.epilogue == CUSYNC_EPILOGUE_RELU) writeRows<CUSYNC_EPILOGUE_RELU, PITCH>(value);
      else writeRows<CUSYNC_EPILOGUE_NONE, PITCH>(value);
    }
    copyOut(i, rows);
  }

  // The same pass for values that are final fp16 already (the epilogue applied and four columns packed into two
  // registers): half4At(j, g).
  template<class V>
  __device__ __forceinline__ void passHalf(int i, uint32_t rows, V&& half4At) const {
    constexpr int PITCH = C::BN * 2 + 16;
    __syncthreads();
    if ((rows >> wm) & 1) {
#pragma unroll
      for (int j = 0; j < C::TN; j++)
#pragma unroll
        for (int g = 0; g < 4; g++)
          *reinterpret_cast<half4*>(lds + (wm * 32 + (lane & 31)) * PITCH + (wn * C::WTN + j * 32 + 8 * g + 4 * (lane >> 5)) * 2) = half4At(j, g);
    }
    copyOut(i, rows);
  }

  // Second half of a pass: all threads copy the buffer out to global memory.
  __device__ __forceinline__ void copyOut(int i, uint32_t rows) const {
    constexpr int PITCH = C::BN * 2 + 16;
    constexpr int ROWS = C::WM * 32;
    constexpr int CPR = C::BN / 8;
    constexpr int STEPS = ROWS * CPR / C::THREADS;
    __syncthreads();
#pragma unroll
    for (int s = 0; s < STEPS; s++) {
      const uint32_t idx = s * C::THREADS + tid;
      const uint32_t lr = idx / CPR, c = idx % CPR;
      const uint32_t m = m0 + (lr / 32) * C::WTM + i * 32 + lr % 32, n = n0 + c * 8;
      // Every thread issues every store, those outside the matrix (or outside `rows`) with an offset the buffer
      // descriptor rejects.  With the read and the store under a condition (a divergent branch around each) and,
      // for a stage that is no producer, the store through a 64-bit pointer, the 2048-row MLP step was 13 us
      // longer (three tiles per workgroup, 4 us each).  Reading all of a pass's pieces from LDS ahead of its
      // first store was measured too: 2 us slower than one after the other.
      const bool inside = m < p.M && n < p.N && ((rows >> (lr / 32)) & 1);
      const uint4v v = *reinterpret_cast<const uint4v*>(lds + lr * PITCH + c * 16);
      const int off = inside ? (int)((m * p.ldd + n) * 2) : (int)kOutOfRange;
      // A producer's output is written through to memory (device scope) as it is stored: the release of the
      // post then finds no dirty lines of it in this XCD's L2.  Left to the post, every one of the workgroups
      // of an XCD that finish together starts a write-back of the whole L2 (measured: the producer of the
      // 2048-row MLP runs 5 us longer than the same kernel without a post).
      if (through) __builtin_amdgcn_raw_buffer_store_b128(v, rD, off, 0, 16 /* sc1 */);
      else __builtin_amdgcn_raw_buffer_store_b128(v, rD, off, 0, 0);
    }
  }
};

// Writes the accumulators of one output tile and tells the caller whether this
// workgroup completed the tile (and therefore posts it).
//
// acc[i][j][r] of lane l is output row  m0 + wm*WTM + i*32 + (l & 31)  and column
// n0 + wn*WTN + j*32 + 8*(r/4) + 4*(l/32) + r%4.
//
// Without split-K the epilogue is applied and the fp16 result stored.  With
// split-K the slice's fp32 partial sums go to the workspace; the slice that
// arrives last (per-tile counter, release/acquire at agent scope because the
// slices ran on different XCDs) adds the slices in index order — so the result
// does not depend on arrival order — applies the epilogue, stores, re-arms the
// counter and posts.  Must be called by all threads of the workgroup.
template<class C>
__device__ __forceinline__ bool finishTileSplit(const GemmParams& p, floatx16 (&acc)[C::TM][C::TN],
                                                const cusync_dim3& t, int wm, int wn, int lane, uint32_t* sLast, char* lds);

// SPLIT = false leaves the k-slices' part out of the kernel (the convolutions never slice K, and code a kernel
// carries without running it still costs it time).
template<class C, bool SPLIT = true>
__device__ __forceinline__ bool finishTile(const GemmParams& p, floatx16 (&acc)[C::TM][C::TN],
                                           const cusync_dim3& t, int wm, int wn, int lane, uint32_t* sLast, char* lds) {
  if constexpr (SPLIT) { if (p.splitK > 1) return finishTileSplit<C>(p, acc, t, wm, wn, lane, sLast, lds); }
  const TileStore<C> store(p, t, wm, wn, lane, lds);
  if constexpr (IsAssemblyTile<C>::value && C::TM * C::TN <= 6) {
    // The 256x192x64 tile (96 accumulators per lane, K loop in assembly): epilogue and conversion come first, for
    // the whole tile at once and in place (two results per register), and the passes move packed values only
    // (GEMM1 of the 2048-row MLP with GeLU: 10.1 -> 8.4 us per tile).  Not for the 256x384 tile: with 192
    // accumulators the same form made the compiler park twice as much in scratch (16 -> 28 us).
    if (p.epilogue != CUSYNC_EPILOGUE_SWIGLU) {
      half4 h[C::TM][C::TN][4];
      auto packAll = [&](auto kind) {
#pragma unroll
        for (int i = 0; i < C::TM; i++)
#pragma unroll
          for (int j = 0; j < C::TN; j++)
#pragma unroll
            for (int g = 0; g < 4; g++)
#pragma unroll
              for (int e = 0; e < 4; e++) h[i][j][g][e] = (half_t)applyEpilogue<decltype(kind)::value>(acc[i][j][g * 4 + e]);
      };
      if (p.epilogue == CUSYNC_EPILOGUE_GELU) packAll(std::integral_constant<int, CUSYNC_EPILOGUE_GELU>{});
      else if (p.epilogue == CUSYNC_EPILOGUE_RELU) packAll(std::integral_constant<int, CUSYNC_EPILOGUE_RELU>{});
      else packAll(std::integral_constant<int, CUSYNC_EPILOGUE_NONE>{});
#pragma unroll
      for (int i = 0; i < C::TM; i++) store.passHalf(i, TileStore<C>::kAllRows, [&](int j, int g) { return h[i][j][g]; });
      return true;
    }
  }
#pragma unroll
  for (int i = 0; i < C::TM; i++)
    store.pass(i, TileStore<C>::kAllRows, [&](int j, int g) {
      return floatx4{acc[i][j][g * 4], acc[i][j][g * 4 + 1], acc[i][j][g * 4 + 2], acc[i][j][g * 4 + 3]};
    });
  return true;
}

// The k-slices' part of finishTile.  Nothing in it may need the accumulators once they are written to the
// workspace: with them alive next to a slice's worth of loads in flight the compiler runs out of registers and
// spills in the main loop of the 256-row tiles (the 512-row GEMM1's k loop went from 73 to 162 us).  As a function
// of its own (not inlined) it costs more still: the kernel then keeps a stack and the same k loop takes 130 us.
template<class C>
__device__ __forceinline__ bool finishTileSplit(const GemmParams& p, floatx16 (&acc)[C::TM][C::TN],
                                                const cusync_dim3& t, int wm, int wn, int lane, uint32_t* sLast, char* lds) {
  const TileStore<C> store(p, t, wm, wn, lane, lds);
  constexpr uint32_t kAllRows = TileStore<C>::kAllRows;
  // Partial sums live in the workspace in register order: value g of MFMA tile (i, j) of every thread is one
  // contiguous run (16 bytes per thread), so slices write and read with fully coalesced accesses; the padding rows
  // and columns of edge tiles are carried along.  They are written through to memory (sc1): the release that
  // follows then has nothing of them to write back, and the slices that read them do so with device-coherent loads.
  constexpr size_t kTileFloats = (size_t)C::BM * C::BN;
  const size_t sliceStride = (size_t)p.stage.d.grid.x * p.stage.d.grid.y * kTileFloats;
  const size_t tileOffset = ((size_t)t.y * p.stage.d.grid.x + t.x) * kTileFloats + (size_t)threadIdx.x * 4;      // in floats
  auto slot = [](int i, int j, int g) { return (size_t)((i * C::TN + j) * 4 + g) * (C::THREADS * 4); };
  const __amdgpu_buffer_rsrc_t rPart = makeRsrc(p.partials, p.partialBytes);
  auto partOffset = [&](uint32_t z, int i, int j, int g) { return (uint32_t)((tileOffset + z * sliceStride + slot(i, j, g)) * sizeof(float)); };
  // Shared reduction: the pieces this slice adds up itself (see below) need not travel through memory.  Their
  // partial sums wait in LDS behind the epilogue's buffer, every lane's own values in a place of its own, if the
  // workgroup's LDS has room for them (a quarter of the partial-sum traffic with four slices, half with two).
  constexpr uint32_t kPieces = C::TM * C::WM;                                   // 32-row pieces of a tile
  constexpr uint32_t kEpiBytes = (C::WM * 32 * (C::BN * 2 + 16) + 1023) / 1024 * 1024;
  constexpr uint32_t kPieceBytes = C::WN * C::TN * 4 * 1024;                    // 32 rows x BN columns of fp32
  const uint32_t perSlice = C::BM >= 128 && p.coopReduce ? kPieces / p.splitK : 0;
  const bool ownInLds = C::BM >= 128 && p.coopReduce && kEpiBytes + perSlice * kPieceBytes <= (uint32_t)C::LDS_BYTES;
  auto ownedPiece = [&](int i) { return ((uint32_t)i * C::WM + (uint32_t)wm) / (perSlice ? perSlice : 1u) == t.z; };      // uniform per wavefront; asked under the shared reduction only
  auto ownSlot = [&](int i, int j, int g) {
    const uint32_t o = (uint32_t)i * C::WM + (uint32_t)wm - t.z * perSlice;
    return lds + kEpiBytes + ((o * C::WN + (uint32_t)wn) * (C::TN * 4) + (uint32_t)(j * 4 + g)) * 1024 + (uint32_t)lane * 16;
  };
  if (ownInLds) __syncthreads();         // every wavefront is out of the main loop and its loads have landed
#pragma unroll
  for (int i = 0; i < C::TM; i++) {
    const bool keep = ownInLds && ownedPiece(i);
#pragma unroll
    for (int j = 0; j < C::TN; j++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const floatx4 v = floatx4{acc[i][j][g * 4], acc[i][j][g * 4 + 1], acc[i][j][g * 4 + 2], acc[i][j][g * 4 + 3]};
        if (keep) *reinterpret_cast<floatx4*>(ownSlot(i, j, g)) = v;
        else __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uint4v, v), rPart, (int)partOffset(t.z, i, j, g), 0, 16 /* sc1 */);
      }
  }
  // the release below is the first thread's and covers its own wavefront's stores; the others see theirs through here
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  const uint32_t tileIndex = t.y * p.stage.d.grid.x + t.x;
  uint32_t* counter = p.arrivals + tileIndex;

  // (the launcher shares the reduction only among tiles of 128 rows and more: the smaller ones do not carry the code)
  if (C::BM >= 128 && p.coopReduce) {
    // ---- every slice adds up and stores its share ---------------------------------------------------------
    // The tile is cut into BM/32 pieces of 32 rows (piece u = i * WM + wm: MFMA row tile i of wave row wm); slice z
    // takes the pieces [z * U/S, (z + 1) * U/S).  A piece is summed over the slices in index order (this slice's
    // own term read back like the others: see above), so the result is the same, bit for bit, whichever way and
    // in whatever order of arrival the tile is put together.
    uint32_t* departures = p.arrivals + p.stage.d.grid.x * p.stage.d.grid.y + tileIndex;
    if (threadIdx.x == 0) {
      // not a release: the partial sums were written through and every wavefront has seen its own acknowledged
      p.stage.countIn(counter);
      if (!dev::pollUntilAtLeast(counter, p.splitK)) dev::countGiveUp(p.stage.d.spinTimeouts);     // the siblings are resident: bounded all the same
      p.stage.countSeen();
    }
    __syncthreads();
    // not unrolled: the sums do not live in the accumulators, so one copy of the pass serves every i
#pragma unroll 1
    for (int i = 0; i < C::TM; i++) {
      const bool owned = ownedPiece(i);
      const uint32_t firstPiece = t.z * perSlice, endPiece = firstPiece + perSlice;
      // wave rows of this pass that belong to this slice
      uint32_t rows = 0;
#pragma unroll
      for (uint32_t w = 0; w < (uint32_t)C::WM; w++) { const uint32_t q = (uint32_t)i * C::WM + w; if (q >= firstPiece && q < endPiece) rows |= 1u << w; }
      if (rows == 0) continue;                                              // uniform per workgroup
      floatx4 sum[C::TN][4];
      if (owned) {
        // two slices' worth of loads in flight at a time; this slice's own term is read back like the others (from
        // LDS or from memory: kept in registers it costs the main loop its registers, see above)
        for (uint32_t z = 0; z < p.splitK; z += 2) {
          uint4v v[2][C::TN][4];
#pragma unroll
          for (uint32_t q = 0; q < 2; q++) {
            if (z + q >= p.splitK) break;
#pragma unroll
            for (int j = 0; j < C::TN; j++)
#pragma unroll
              for (int g = 0; g < 4; g++)
                v[q][j][g] = ownInLds && z + q == t.z ? *reinterpret_cast<const uint4v*>(ownSlot(i, j, g))
                                                      : __builtin_amdgcn_raw_buffer_load_b128(rPart, (int)partOffset(z + q, i, j, g), 0, 16 /* sc1 */);
          }
#pragma unroll
          for (uint32_t q = 0; q < 2; q++) {
            if (z + q >= p.splitK) break;
#pragma unroll
            for (int j = 0; j < C::TN; j++)
#pragma unroll
              for (int g = 0; g < 4; g++) {
                const floatx4 term = __builtin_bit_cast(floatx4, v[q][j][g]);
                sum[j][g] = (z + q == 0) ? term : sum[j][g] + term;
              }
          }
        }
      }
      store.pass(i, rows, [&](int j, int g) { return sum[j][g]; });
    }
    // the slice that stores its share last re-arms the counters and has the tile to post
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
      // A producer's stores must be out before the count that lets the last slice post: they were written through
      // and are acknowledged (the wait above), so the count needs no release, which would only start a write-back of
      // this XCD's L2.  No acquire either: nobody reads another slice's output.
      const uint32_t before = p.stage.countIn(departures);
      const bool last = before == p.splitK - 1;
      if (last) { dev::storeRelaxed(counter, 0); dev::storeRelaxed(departures, 0); }
      *sLast = last;
    }
    __syncthreads();
    return *sLast != 0;
  }

  if (threadIdx.x == 0) {
    // neither release (the partial sums were written through and are acknowledged) nor acquire (the finishing slice
    // reads them with device-coherent loads): either would work on this XCD's whole L2
    const uint32_t before = p.stage.countIn(counter);
    const bool last = before == p.splitK - 1;
    if (last) { dev::storeRelaxed(counter, 0); p.stage.countSeen(); }
    *sLast = last;
  }
  __syncthreads();
  if (!*sLast) return false;
  // The slice that arrived last adds the slices in index order, one row of MFMA tiles at a time: all loads
  // of that row for one slice are issued together (TN * 4 of 16 bytes per thread).  One position at a time
  // would be a chain of round trips to memory as long as the GEMM itself; everything at once, accumulated
  // into `acc`, makes the compiler spill in the main loop.  The loads are coherent at device scope (sc1; the
  // partial sums were written through), which spares the acquire fence that would empty this XCD's L2.
  // Narrow wavefront tiles have few loads per slice: several slices are fetched together (G of them), still
  // added in index order
  constexpr int G = C::BM <= 64 ? 36 / (C::TN * 4) : C::TN * 4 >= 16 ? 1 : 16 / (C::TN * 4);
  // (a real loop over i: one copy of the loads and of the pass)
#pragma unroll 1
  for (int i = 0; i < C::TM; i++) {
    floatx4 sum[C::TN][4];
    for (uint32_t z = 0; z < p.splitK; z += G) {
      floatx4 v[G][C::TN][4];
#pragma unroll
      for (int q = 0; q < G; q++) {
        if (z + q >= p.splitK) break;
#pragma unroll
        for (int j = 0; j < C::TN; j++)
#pragma unroll
          for (int g = 0; g < 4; g++)
            v[q][j][g] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(rPart, (int)partOffset(z + q, i, j, g), 0, 16 /* sc1 */));
      }
#pragma unroll
      for (int q = 0; q < G; q++) {
        if (z + q >= p.splitK) break;
#pragma unroll
        for (int j = 0; j < C::TN; j++)
#pragma unroll
          for (int g = 0; g < 4; g++) sum[j][g] = (z + q == 0) ? v[q][j][g] : sum[j][g] + v[q][j][g];
      }
    }
    store.pass(i, kAllRows, [&](int j, int g) { return sum[j][g]; });
  }
  return true;
}

// Half a pass: NM MFMAs with the R LDS reads of the next k-step's fragments spread between them.
template<int NM, int R, int M = 0>
__device__ __forceinline__ void schedHalf() {
  if constexpr (M < NM) {
    schedGroup<kSchedMfma, 1>();
    schedGroup<kSchedDsRead, evenShare(R, NM, M)>();
    schedHalf<NM, R, M + 1>();
  }
}

template<int P> struct Parity { static constexpr int value = P; };

// Calls f(Parity<0>{}), f(Parity<1>{}), ... f(Parity<N-1>{}): a loop whose index
// is a compile-time constant inside the body.
template<int N, class F>
__device__ __forceinline__ void staticFor(F&& f) {
  [&]<int... I>(std::integer_sequence<int, I...>) { (f(Parity<I>{}), ...); }(std::make_integer_sequence<int, N>{});
}

}  // namespace gemm
}  // namespace cusync
