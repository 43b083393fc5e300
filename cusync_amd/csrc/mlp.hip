// MLP chain: two dependent GEMMs, X*W1 (+activation) -> H, H*W2 -> Y, run either
// stream-ordered (kernel-boundary sync) or as a CuSync producer/consumer pair on
// two streams.  Host code only; the kernels are launched through
// cusync_gemm_run.  Stands in for the hot loops of the reference driver
// (src/ml-bench/transformer/mlp.cu:411-491 runBaselineGPT3, :645-716
// runCuSyncGPT3, :718-862 runCuSyncLLaMA) and for the C surface of
// src/ml-bench/transformer/mlp-lib.cu:555-618.
#include <hip/hip_runtime.h>

#include <string.h>
#include <algorithm>
#include <string>

#include "../../include/cusync_amd.h"
#include "rt_internal.h"
#include "split_choice.h"
#include "gemm_common.h"

struct cusync_mlp {
  cusync_mlp_config cfg;
  const void* w1;
  const void* w2;
  int tile1, tile2;
  int split1, split2;
  void* ws1;
  void* ws2;
  uint32_t n1, k1, n2, k2;          // GEMM1 is [batch,k1]x[k1,n1], GEMM2 is [batch,k2]x[k2,n2]
  uint32_t ldh;                      // row pitch of the intermediate
  void* w1p; void* w2p;              // repack_weights: padded copies of the weights, owned
  uint32_t ldw1, ldw2;               // row pitch of the weights the GEMMs read
  int epilogue1, aMode2;
  cusync_stage_desc prod, cons;
  hipStream_t sProd, sCons;
  hipEvent_t eStart, eMid, eEnd;
  // LLaMA with silu(gate) * up as GEMM1's epilogue: w1p holds W1 with the gate and up columns interleaved in
  // groups of eight, the intermediate is [batch][inner]
  bool fused;
  // LLaMA with the activation as a stage of its own between the GEMMs: silu(gate) * up, once per element
  bool actStage;
  void* act;                         // [batch][inner] fp16, GEMM2's A operand
  cusync_stage_desc mid;
  hipStream_t sMid;
  uint32_t timeoutsSeen;             // sum of the stages' give-up counters when the last run returned
};

namespace {

using cusync::rt::setError;
using cusync::gemm::pickSplit;
using cusync::gemm::half_t;
using cusync::gemm::uint4v;

// ---- silu(gate) * up as a CuSync stage ------------------------------------------------------------
// A = silu(G[:, 0:d]) * G[:, d:2d] in tiles of 128 x 128.  As a consumer of GEMM1 a tile waits for the
// producer tiles that hold its gate and its up columns (under StridedSync both map to one semaphore
// that counts to two); as a producer for GEMM2 it posts the tile.  Fused into GEMM2's A loader the
// same arithmetic is repeated once per column tile of GEMM2 (64 times for the LLaMA shard) and makes
// that kernel three times slower; here every element is computed once.
constexpr uint32_t kActM = 128, kActN = 128, kActThreads = 256;

// dst[row][0..vecs) = src[row][0..vecs) in 16-byte pieces; dst rows are dstPitch pieces apart
__global__ __launch_bounds__(256) void repackRowsKernel(const uint4v* src, uint4v* dst, uint32_t vecs, uint32_t dstPitch) {
  const uint32_t c = blockIdx.x * 256 + threadIdx.x;
  if (c < vecs) dst[(size_t)blockIdx.y * dstPitch + c] = src[(size_t)blockIdx.y * vecs + c];
}

// dst[row] = the gate and up halves of src[row] ([2d] halfs, gate | up) interleaved in 16-byte pieces: piece 2q of
// dst is piece q of the gate half, piece 2q + 1 is piece q of the up half (d / 8 pieces per half); dst rows are
// dstPitch pieces apart.  The layout CUSYNC_EPILOGUE_SWIGLU reads.
__global__ __launch_bounds__(256) void interleaveGateUpKernel(const uint4v* src, uint4v* dst, uint32_t piecesPerHalf, uint32_t dstPitch) {
  const uint32_t j = blockIdx.x * 256 + threadIdx.x;
  if (j < 2 * piecesPerHalf)
    dst[(size_t)blockIdx.y * dstPitch + j] = src[(size_t)blockIdx.y * 2 * piecesPerHalf + (j & 1) * piecesPerHalf + (j >> 1)];
}

struct ActParams {
  cusync::DynStage stage;
  uint32_t M, d;                 // rows, columns of A (= inner)
  const half_t* G; uint32_t ldg; // gate | up, [M][ldg]
  half_t* A; uint32_t lda;
  uint32_t launched;
};

__global__ __launch_bounds__(kActThreads) void swigluStageKernel(ActParams p) {
  __shared__ uint32_t sTicket;
  const cusync::DynStage& stage = p.stage;
  const uint32_t tid = threadIdx.x;
  const uint32_t numTiles = stage.numTiles();
  const bool consumer = stage.isConsumer();
  const uint32_t tmq = consumer ? stage.d.in.tileM : 1, tnq = consumer ? stage.d.in.tileN : 1;
  // the row policies mark their waits with z = 1, the tile policies with z = 0
  const uint32_t zWait = consumer && stage.d.in.kind == CUSYNC_POLICY_ROWSYNC ? 1 : 0;
  uint32_t dryXcds = 0, nextRaw = 0;
  const uint32_t startToken = tid == 0 ? stage.beginStart() : 0;
  const bool noDraws = stage.noDraws;
  for (uint32_t round = 0;; round++) {
    if (tid == 0) sTicket = round == 0 ? stage.firstTicket(p.launched, dryXcds, noDraws) : stage.drawFinish(nextRaw, p.launched, round, dryXcds, noDraws);
    __syncthreads();
    const uint32_t ticket = sTicket;
    if (tid == 0 && round == 0) stage.finishStart(startToken, p.launched);
    if (ticket >= numTiles) break;
    const cusync_dim3 t = stage.ticketToTile(ticket);
    const uint32_t m0 = t.y * kActM, c0 = t.x * kActN;
    const uint32_t mEnd = min(m0 + kActM, p.M), cEnd = min(c0 + kActN, p.d);
    if (consumer) {
      if (tid < 64) {          // one wavefront waits for everybody
        for (uint32_t r = m0; r < mEnd; r = (r / tmq + 1) * tmq)
          for (uint32_t half = 0; half < 2; half++)
            for (uint32_t c = (half * p.d + c0) / tnq * tnq; c < half * p.d + cEnd; c += tnq) {
              cusync_dim3 w = {r, c, zWait};
              stage.waitWave(w);
              if (zWait) break;             // a row policy guards whole rows: one wait per row block
            }
      }
      __syncthreads();
    }
    if (tid == 0) nextRaw = stage.drawBegin(dryXcds, noDraws);     // settled after the tile
#pragma unroll
    for (uint32_t i = 0; i < kActM * kActN / 8 / kActThreads; i++) {
      const uint32_t idx = i * kActThreads + tid;
      const uint32_t m = m0 + idx / (kActN / 8), c = c0 + (idx % (kActN / 8)) * 8;
      if (m < p.M && c < p.d) {
        const uint4v g = *reinterpret_cast<const uint4v*>(p.G + (size_t)m * p.ldg + c);
        const uint4v u = *reinterpret_cast<const uint4v*>(p.G + (size_t)m * p.ldg + p.d + c);
        *reinterpret_cast<uint4v*>(p.A + (size_t)m * p.lda + c) = cusync::gemm::swigluChunk(g, u);
      }
    }
    cusync_dim3 done = {m0, c0, 0};
    if (stage.isProducer()) stage.post(done);
    else __syncthreads();
  }
}

// Workgroups of the activation kernel that stay resident on the device; 0 if the runtime would not say.
// Worked out once (the initialisation of a function-local static is safe against concurrent first calls).
int actResident() {
  static const int resident = [] {
    int dev = 0, perCU = 0;
    hipDeviceProp_t prop;
    if (CUSYNC_HIP(hipGetDevice(&dev)) || CUSYNC_HIP(hipGetDeviceProperties(&prop, dev)) ||
        CUSYNC_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&perCU, swigluStageKernel, (int)kActThreads, 0))) return 0;
    return std::max(1, std::min(perCU, 4)) * prop.multiProcessorCount;
  }();
  return resident;
}

cusync_error runActStage(const cusync_mlp* m, const void* h, void* stream) {
  const int resident = actResident();
  if (resident <= 0) return CUSYNC_ERROR_DEVICE;
  const cusync_stage_desc& s = m->mid;
  ActParams p = {};
  p.stage.d = s;
  p.stage.releaseAll = cusync::rt::forceRelease();
  p.stage.lineAligned = false;       // every wait is followed by an L2 invalidation: tiles of 128 columns of a 2d-wide matrix are not whole lines for every d
  p.M = m->cfg.batch; p.d = m->cfg.inner;
  p.G = (const half_t*)h; p.ldg = m->ldh;
  p.A = (half_t*)m->act; p.lda = m->cfg.inner;
  p.launched = std::min<uint32_t>(s.grid.x * s.grid.y * s.grid.z, (uint32_t)resident);
  p.stage.prepare(p.launched);
  hipLaunchKernelGGL(swigluStageKernel, dim3(p.launched), dim3(kActThreads), 0, (hipStream_t)stream, p);
  if (CUSYNC_HIP(hipGetLastError())) return CUSYNC_ERROR_DEVICE;
  return CUSYNC_SUCCESS;
}

// Built-in choice of tile shapes per batch size for 256 CUs.  Above 128 rows the
// direct-to-LDS tiles are used; below that the M extent follows the batch.  A SwiGLU consumer has
// to use a register-staged tile, and StridedSync needs the gate|up split on a
// tile boundary (2752 = 43 * 64).
void pickTiles(const cusync_mlp_config& c, int sync, bool swiglu, bool fused, int* t1, int* t2) {
  if (fused) {
    // silu(gate) * up in GEMM1's epilogue: both GEMMs have plain operands and run the direct-to-LDS tiles at every
    // batch size; the kernels mask the ragged last column tile of the shard's widths (2 * 2752 and 8192).  The
    // policies count columns of the intermediate, half a GEMM1 tile wide, and no width constrains StridedSync.
    // Measured by the tuner on the LLaMA shard (cusync_amd/tile_sizes_db.py, llama_mlp_mi355x): for GEMM2 the 64-row
    // tiles stay ahead up to 512 rows; GEMM1 from 129 rows on takes 128x192 with a CU to itself, in as many k-slices
    // as fill the device, now that the slices share the reduction (256 rows: 54 -> 49 us against 64x192 in two
    // slices; level at 512 rows).
    int a, b;
    if (c.batch <= 32) a = b = CUSYNC_TILE_D32x128x64;
    else if (c.batch <= 64) { a = CUSYNC_TILE_D64x128x64; b = CUSYNC_TILE_D32x128x64; }     // GEMM2 at 64 rows: 17 us in two slices against 20 on 64x128
    else if (c.batch <= 128) { a = CUSYNC_TILE_D64x192x64; b = CUSYNC_TILE_D64x128x64; }
    else if (c.batch <= 512) { a = CUSYNC_TILE_128x192x32_ALONE; b = CUSYNC_TILE_D64x128x64; }
    else if (c.batch <= 1024) { a = CUSYNC_TILE_128x192x32_ALONE; b = CUSYNC_TILE_128x256x32; }
    else a = b = CUSYNC_TILE_256x256x32;
    // From 257 rows on GEMM1 (K = 8192) takes the 256x192 tile whose K loop is assembly, in as many k-slices as fill
    // the device (the chain under RowSync: 384 rows 106 -> 92 us, 512: 117 -> 103, 768: 166 -> 131, 1024: 176 -> 156,
    // 1536: 236 -> 203, 2048: 263 -> 246; level at 256 rows).  Its last column tile is ragged (5504 = 28.7 x 192).
    if (c.batch > 256 && c.hidden % 64 == 0) a = CUSYNC_TILE_256x192x64;
    // 129 to 256 rows: 128x192 with the operands fetched 64 columns of K at a time (a row of A as one 128-byte line;
    // the chain under RowSync: 160 rows 77 -> 65 us, 256 rows 80 -> 72; level with 256x192x64 at 384 and 512 rows)
    else if (c.batch > 128 && c.hidden % 64 == 0) a = CUSYNC_TILE_D128x192x64;
    *t1 = c.tile1 >= 0 ? c.tile1 : a;
    *t2 = c.tile2 >= 0 ? c.tile2 : b;
    if (c.one_launch && sync != CUSYNC_SYNC_STREAM && c.tile2 < 0) *t2 = *t1;
    return;
  }
  int small;
  if (c.batch <= 32) small = CUSYNC_TILE_32x128x64;
  else if (c.batch <= 64) small = CUSYNC_TILE_64x128x64;
  else small = CUSYNC_TILE_128x128x64;
  const bool big = c.batch > 128;
  // Measured on the GPT-3 shard.  Where the width is a multiple of 192 (6144 and 12288 columns are 32 and
  // 64 tiles: whole rounds on 256 CUs) the 192-wide direct-to-LDS tiles win from 256 rows on.  GEMM1: 256x192
  // with a CU to itself (8 % faster than 128x192 at two workgroups per CU at 1024 and 2048 rows; below that the
  // k-slices fill the device).  GEMM2: the same (from 257 to 512 rows in two k-slices whose workgroups each add up
  // and store half a tile: at 512 rows 106 us against 117 us for 128x192 without slices, at 384 rows 96 against
  // 110 us for 128x192 alone on its CU, which led there while a k-slice's arrival still wrote an L2 back).
  // Other widths (the LLaMA shard: 5504 and 8192 columns; the kernels mask the ragged last column tile): 128x192
  // alone on its CU up to 1024 rows, above that 256x192 for GEMM1 and 256x256 for GEMM2 (at 2048 rows 232 and 256
  // tiles: one round).  Measured against 128x128 / 128x256 at two workgroups per CU: 172 -> 147 us at 512 rows,
  // 232 -> 211 at 1024, 356 -> 304 at 2048.
  const uint32_t n1 = c.model == CUSYNC_MLP_LLAMA ? 2 * c.inner : c.inner, n2 = c.hidden;
  int a = !big ? small : c.batch <= 1024 ? CUSYNC_TILE_128x192x32_ALONE : CUSYNC_TILE_256x192x32;
  int b = !big ? small : swiglu ? CUSYNC_TILE_256x128x64 : c.batch <= 1024 ? CUSYNC_TILE_128x192x32_ALONE : CUSYNC_TILE_256x256x32;
  if (big && n1 % 192 == 0) a = CUSYNC_TILE_256x192x32;
  // (1025 to 1536 rows are five or six row tiles of 256, 320 or 384 tiles of GEMM2 for 256 CUs: there 128x192 at
  // two workgroups per CU fills the second round better: 1152 rows 230 -> 212 us, 1280: 233 -> 217, 1536: 246 -> 236;
  // from 1664 rows on 256x192 leads again, 258 against 285 us)
  if (big && n2 % 192 == 0 && !swiglu) b = c.batch > 1024 && c.batch <= 1536 ? CUSYNC_TILE_128x192x32 : CUSYNC_TILE_256x192x32;
  // Up to 256 rows the GEMMs are bound by streaming the weights: direct-to-LDS tiles with 60-96 KB of loads
  // in flight per workgroup (measured: 104 -> 85 us at 1-32 rows, 127 -> 101 us at 64, 187 -> 158 us at 256).
  // 64x192 makes 32 or 64 column tiles, which 8 or 4 k-slices turn into one workgroup per CU.
  if (c.batch <= 32) {
    a = CUSYNC_TILE_D32x128x64;
    if (!swiglu) b = CUSYNC_TILE_D32x128x64;
  } else if (c.batch <= 128) {
    if (n1 % 192 == 0) a = CUSYNC_TILE_D64x192x64;
    if (n2 % 192 == 0 && !swiglu) b = CUSYNC_TILE_D64x192x64;
  } else if (c.batch <= 256) {
    // two row tiles of 128: 128x192 at two workgroups per CU, in four and two k-slices (256 rows: 78.5 and 72.4 us
    // against 82.7 and 73.5 for 64x192 in two slices and one; the pair 151 against 156 us stream-ordered, 140
    // against 142 under TileSync; 160 rows, where 64x192 makes three row tiles: 130 against 148 us), now that a
    // slice's arrival no longer writes its XCD's L2 back.  At 128 rows 64x192 in four and two slices still leads
    // (106 against 120 us for one row tile of 128 in eight and four).
    if (n1 % 192 == 0) a = CUSYNC_TILE_128x192x32;
    if (n2 % 192 == 0 && !swiglu) b = CUSYNC_TILE_128x192x32;
    // The same tile with both operands fetched 64 columns of K at a time, a CU to itself: a row of A then arrives as
    // one 128-byte line instead of two 64-byte pieces, and what bounds the loop here is the number of requests a CU's
    // memory path holds, not their size (stream-ordered pair / best CuSync, us: 160 rows 126 / 122 -> 121 / 116,
    // 192: 133 / 125 -> 124 / 118, 224: 140 / 131 -> 126 / 120, 256: 148 / 138 -> 128 / 124, on other machines of the
    // same kind 148 / 138 -> 143 / 135; level at 128 rows, and behind 256x192x64 in four and two k-slices from 257
    // rows on: 320 rows 156 against 173).
    if (a == CUSYNC_TILE_128x192x32 && c.hidden % 64 == 0) a = CUSYNC_TILE_D128x192x64;
    if (b == CUSYNC_TILE_128x192x32 && c.inner % 64 == 0) b = CUSYNC_TILE_D128x192x64;
  }
  // StridedSync needs the gate|up split on a column-tile boundary of GEMM1: 128- or 256-wide tiles where the
  // 192-wide ones do not divide `inner`, 64-wide ones where nothing else does (2752 = 43 * 64)
  if (sync == CUSYNC_SYNC_STRIDED) {
    uint32_t tn = 0;
    cusync_gemm_tile_shape(c.tile1 >= 0 ? c.tile1 : a, nullptr, &tn, nullptr);
    if (c.inner % 128 != 0) a = c.batch <= 128 ? CUSYNC_TILE_128x64x64 : CUSYNC_TILE_256x64x64;
    else if (tn == 0 || c.inner % tn != 0) a = c.batch <= 1024 ? CUSYNC_TILE_128x128x32 : CUSYNC_TILE_128x256x32;
  }
  // Where K is a multiple of 64 the 256x192 tile with both operands fetched 64 columns at a time, in whole cache
  // lines, and its K loop in assembly takes over from the 32-column one (GPT-3 shard, same machine, stream-ordered:
  // 512 rows 204 -> 196 us, 1024 rows 330 -> 308, 2048 rows 612 -> 562), and from 1025 rows on GEMM2 runs 256x384
  // tiles, at most one per CU, where its width allows (12288 columns are 32 of them; 2048 rows: 562 -> 557 us; with
  // fewer rows it would need k-slices, whose reduction costs it more than the tile gains).  Both wait for all their
  // producer tiles before the first load, whatever the policy.
  const uint32_t k1 = c.hidden, k2 = c.inner;
  if (a == CUSYNC_TILE_256x192x32 && k1 % 64 == 0) a = CUSYNC_TILE_256x192x64;
  if (b == CUSYNC_TILE_256x192x32 && k2 % 64 == 0) b = CUSYNC_TILE_256x192x64;
  // (1025 to 1536 rows, five or six row tiles: 160 or 192 tiles of 256x384 in one round against 128x192 at two
  // workgroups per CU in one and a half: 1056 rows 397 -> 347 us, 1152: 404 -> 353, 1280: 407 -> 365, 1536: 444 -> 400)
  if (big && c.batch > 1024 && !swiglu && k2 % 64 == 0 && n2 % 384 == 0 && !c.one_launch) b = CUSYNC_TILE_256x384x32;
  *t1 = c.tile1 >= 0 ? c.tile1 : a;
  *t2 = c.tile2 >= 0 ? c.tile2 : b;
  // both GEMMs in one launch share a kernel: the consumer takes the producer's tile
  if (c.one_launch && sync != CUSYNC_SYNC_STREAM && c.tile2 < 0 && !swiglu) *t2 = *t1;
}

cusync_policy_desc noSync() {
  cusync_policy_desc p;
  memset(&p, 0, sizeof p);
  p.kind = CUSYNC_POLICY_NOSYNC;
  p.tileM = p.tileN = 1; p.R = p.S = 1;
  return p;
}

cusync_gemm_args gemmArgs(const cusync_mlp* m, int which, const void* x, void* h, void* y) {
  cusync_gemm_args a;
  memset(&a, 0, sizeof a);
  a.M = m->cfg.batch;
  a.split_k = which == 0 ? m->split1 : m->split2;
  a.workspace = which == 0 ? m->ws1 : m->ws2;
  a.max_workgroups = std::max(0, which == 0 ? m->cfg.max_wg1 : m->cfg.max_wg2);
  a.shared_reduction = 1;       // a consumer of this handle is launched only after its producer is resident
  if (which == 0) {
    a.stage = m->prod;
    a.N = m->n1; a.K = m->k1;
    a.A = x; a.lda = m->k1;
    a.B = m->w1p ? m->w1p : m->w1; a.ldb = m->ldw1;
    a.D = h; a.ldd = m->ldh;
    a.epilogue = m->epilogue1;
    a.a_mode = CUSYNC_A_PLAIN;
    a.tile = m->tile1;
  } else {
    a.stage = m->cons;
    a.N = m->n2; a.K = m->k2;
    a.A = m->actStage ? m->act : h; a.lda = m->actStage ? m->k2 : m->ldh;
    a.B = m->w2p ? m->w2p : m->w2; a.ldb = m->ldw2;
    a.D = y; a.ldd = m->n2;
    a.epilogue = CUSYNC_EPILOGUE_NONE;
    a.a_mode = m->aMode2;
    a.tile = m->tile2;
  }
  return a;
}

// create() failed: gives back what the handle holds so far and keeps the text of the failure
void discard(cusync_mlp* m) {
  const std::string why = cusync_rt_last_error();
  cusync_mlp_destroy(m);
  setError(why);
}

// What a handle for `c` runs with: where the activation is computed, the sync mode after the StridedSync
// substitution, tiles and k-slices.  False (with the error text set) for a configuration no handle can be made of.
struct Choice { bool fused, actStage, oneLaunch; int aMode2, sync, tile1, tile2, split1, split2; };

// Both GEMMs in one launch need the same direct-to-LDS tile for both and a plain A operand in GEMM2.
bool oneLaunchPossible(const Choice& o) {
  uint32_t bk = 0;
  if (cusync_gemm_tile_shape(o.tile1, nullptr, nullptr, &bk)) return false;
  const bool direct = bk == 32 || o.tile1 >= CUSYNC_TILE_D32x128x64;      // the direct-to-LDS tiles
  return o.tile1 == o.tile2 && direct && o.aMode2 == CUSYNC_A_PLAIN && !o.actStage;
}

bool choose(const cusync_mlp_config& given, Choice* o) {
  cusync_mlp_config c = given;
  const bool llama = c.model == CUSYNC_MLP_LLAMA;
  // one_launch < 0: where one launch measured ahead of two on the GPT-3 shard (1 to 64 rows under either policy:
  // 1-5 us of 67-83; 512 to 1024 rows: 1-3 us of 172-284; behind at 256 rows and from 1025 on, and at every size of
  // the LLaMA shard, whose GEMM2 wants a tile of its own) and the tiles are the table's
  const bool automatic = c.one_launch < 0;
  if (automatic) c.one_launch = c.sync != CUSYNC_SYNC_STREAM && !llama && c.tile1 < 0 && c.tile2 < 0 &&
                                (c.batch <= 64 || (c.batch >= 512 && c.batch <= 1024));
  const uint32_t k1 = c.hidden, n1 = llama ? 2 * c.inner : c.inner, k2 = c.inner, n2 = c.hidden;
  const bool swiglu = llama && c.activation;
  // where silu(gate) * up is computed: 2 = GEMM1's epilogue (the built-in choice), -1 = a stage of its own, 1 = GEMM2's A loader
  const int where = !swiglu ? 0 : c.swiglu_in_gemm2 == 0 ? 2 : c.swiglu_in_gemm2;
  if (swiglu && where != 2 && where != -1 && where != 1) { setError("mlp: swiglu_in_gemm2 must be -1, 0, 1 or 2"); return false; }
  o->fused = swiglu && where == 2;
  o->actStage = swiglu && where == -1;
  o->aMode2 = (swiglu && where == 1) ? CUSYNC_A_SWIGLU : CUSYNC_A_PLAIN;
  o->sync = c.sync;
  if (swiglu && !o->fused && o->sync == CUSYNC_SYNC_TILE && c.inner % 128 == 0) o->sync = CUSYNC_SYNC_STRIDED;
  pickTiles(c, o->sync, o->aMode2 == CUSYNC_A_SWIGLU, o->fused, &o->tile1, &o->tile2);
  o->oneLaunch = c.one_launch && o->sync != CUSYNC_SYNC_STREAM;
  if (o->oneLaunch && !oneLaunchPossible(*o)) {
    if (!automatic) {
      setError("mlp: one launch for both GEMMs needs the same direct-to-LDS tile for both and a plain A operand");
      return false;
    }
    c.one_launch = 0;
    o->oneLaunch = false;
    pickTiles(c, o->sync, o->aMode2 == CUSYNC_A_SWIGLU, o->fused, &o->tile1, &o->tile2);
  }
  uint32_t bk1 = 0, bk2 = 0;
  if (cusync_gemm_tile_shape(o->tile1, nullptr, nullptr, &bk1) || cusync_gemm_tile_shape(o->tile2, nullptr, nullptr, &bk2)) {
    setError("mlp: unknown tile id");
    return false;
  }
  const cusync_dim3 flat1 = cusync_gemm_grid(o->tile1, c.batch, n1, 1);
  const cusync_dim3 flat2 = cusync_gemm_grid(o->tile2, c.batch, n2, 1);
  o->split1 = pickSplit(c.split_k1, flat1.x * flat1.y, k1, bk1, cusync_gemm_max_resident(o->tile1));
  o->split2 = pickSplit(c.split_k2, flat2.x * flat2.y, k2, bk2, cusync_gemm_max_resident(o->tile2));
  return true;
}

}  // namespace

extern "C" {

cusync_mlp* cusync_mlp_create(const cusync_mlp_config* cfg, const void* w1, const void* w2) {
  if (!cfg || !w1 || !w2) { setError("mlp: null argument"); return nullptr; }
  if (cfg->batch == 0 || cfg->hidden == 0 || cfg->inner == 0) { setError("mlp: empty shape"); return nullptr; }
  cusync_mlp* m = new cusync_mlp();
  m->cfg = *cfg;
  m->w1 = w1; m->w2 = w2;
  const bool llama = cfg->model == CUSYNC_MLP_LLAMA;
  m->k1 = cfg->hidden;
  m->n1 = llama ? 2 * cfg->inner : cfg->inner;
  m->k2 = cfg->inner;
  m->n2 = cfg->hidden;
  m->ldh = m->n1;
  m->w1p = m->w2p = nullptr;
  m->ldw1 = m->n1; m->ldw2 = m->n2;
  Choice ch;
  if (!choose(*cfg, &ch)) { discard(m); return nullptr; }
  m->cfg.one_launch = ch.oneLaunch;      // settled: the run asks this copy
  m->fused = ch.fused;
  m->actStage = ch.actStage;
  m->aMode2 = ch.aMode2;
  m->epilogue1 = (!llama && cfg->activation) ? CUSYNC_EPILOGUE_GELU : m->fused ? CUSYNC_EPILOGUE_SWIGLU : CUSYNC_EPILOGUE_NONE;
  if (cfg->repack_weights) {
    // rows 256 bytes longer than the data: consecutive k rows of a column tile then fall into consecutive
    // channel classes (address bits 8..11) instead of all into one
    m->ldw1 = m->n1 + 128; m->ldw2 = m->n2 + 128;
    if (CUSYNC_HIP(hipMalloc(&m->w1p, (size_t)m->k1 * m->ldw1 * sizeof(half_t))) ||
        CUSYNC_HIP(hipMalloc(&m->w2p, (size_t)m->k2 * m->ldw2 * sizeof(half_t))) ||
        cusync_mlp_reload_weights(m) != CUSYNC_SUCCESS) {
      discard(m);
      return nullptr;
    }
  }
  if (m->fused) {
    if (cfg->inner % 8 != 0) { setError("mlp: the SwiGLU epilogue needs inner % 8 == 0"); discard(m); return nullptr; }
    m->ldh = cfg->inner;              // the intermediate is silu(gate) * up itself
    if (!m->w1p) {                    // not yet there from repack_weights: the handle's interleaved copy of W1
      m->ldw1 = m->n1;
      if (CUSYNC_HIP(hipMalloc(&m->w1p, (size_t)m->k1 * m->ldw1 * sizeof(half_t))) || cusync_mlp_reload_weights(m) != CUSYNC_SUCCESS) {
        discard(m);
        return nullptr;
      }
    }
  }
  m->act = nullptr;
  m->sMid = nullptr;
  memset(&m->mid, 0, sizeof m->mid);

  const int sync = ch.sync;
  m->tile1 = ch.tile1; m->tile2 = ch.tile2;
  uint32_t tm1 = 0, tn1 = 0;
  cusync_gemm_tile_shape(m->tile1, &tm1, &tn1, nullptr);

  cusync_policy_desc pol = noSync();
  int opts = 0;
  const uint32_t tnOut = m->fused ? tn1 / 2 : tn1;      // width of a GEMM1 tile in columns of the intermediate
  m->split1 = ch.split1; m->split2 = ch.split2;
  m->ws1 = m->ws2 = nullptr;
  const cusync_dim3 g1 = cusync_gemm_grid(m->tile1, cfg->batch, m->n1, m->split1);
  const cusync_dim3 g2 = cusync_gemm_grid(m->tile2, cfg->batch, m->n2, m->split2);
  switch (sync) {
    case CUSYNC_SYNC_STREAM:
      break;
    case CUSYNC_SYNC_ROW:        // RowSync(gridDim1.n()), src/ml-bench/transformer/mlp.cu:1032-1034
      pol.kind = CUSYNC_POLICY_ROWSYNC; pol.order = CUSYNC_ORDER_TRANSPOSE_XY;
      pol.tileM = tm1; pol.tileN = 1; pol.waitValue = g1.x; pol.postValue = 1;
      opts = CUSYNC_OPT_REORDER_TILE_LOADS;      // defined for every policy, mlp.cu:15
      break;
    case CUSYNC_SYNC_TILE:       // TileSync<TransposeXY,kM,kN> + NoAtomicAdd + ReorderTileLoads, mlp.cu:9-16,111
      pol.kind = CUSYNC_POLICY_TILESYNC; pol.order = CUSYNC_ORDER_TRANSPOSE_XY;
      pol.tileM = tm1; pol.tileN = tnOut; pol.waitValue = 1; pol.postValue = 1;
      opts = CUSYNC_OPT_NO_ATOMIC_ADD | CUSYNC_OPT_REORDER_TILE_LOADS;
      break;
    case CUSYNC_SYNC_STRIDED:    // StridedSync<TransposeXY,d,kM,kN,2>, mlp.cu:109; atomic add kept (:9-14)
      if (!llama) { setError("mlp: StridedSync is for the gate|up layout"); discard(m); return nullptr; }
      if (!m->fused && cfg->inner % tn1 != 0) { setError("mlp: StridedSync needs inner % tileN == 0"); discard(m); return nullptr; }
      pol.kind = CUSYNC_POLICY_STRIDEDSYNC; pol.order = CUSYNC_ORDER_TRANSPOSE_XY;
      pol.tileM = tm1; pol.tileN = tnOut; pol.waitValue = 2; pol.postValue = 1;
      // GridN: the width of one group (gate, or up) in whole tiles.  With the epilogue computing silu(gate) * up a
      // workgroup holds the gate tile and the up tile of its column range and posts for both at once; the width
      // is rounded up to whole tiles (the reference rounds its 2731 columns up to 2816, mlp.cu:247-250).
      pol.gridN = m->fused ? (cfg->inner + tnOut - 1) / tnOut * tnOut : cfg->inner; pol.stride = 2;
      opts = CUSYNC_OPT_REORDER_TILE_LOADS;
      break;
    default:
      setError("mlp: unknown sync mode");
      discard(m);
      return nullptr;
  }
  if (cfg->opts >= 0) opts |= cfg->opts;

  // the edge into GEMM2 when the activation is a stage of its own: its 128 x 128 tiles under the same kind of policy
  cusync_policy_desc pol2 = pol;
  const cusync_dim3 gAct = {(cfg->inner + kActN - 1) / kActN, (cfg->batch + kActM - 1) / kActM, 1};
  if (m->actStage && sync != CUSYNC_SYNC_STREAM) {
    pol2 = noSync();
    pol2.order = CUSYNC_ORDER_TRANSPOSE_XY; pol2.postValue = 1;
    if (sync == CUSYNC_SYNC_ROW) { pol2.kind = CUSYNC_POLICY_ROWSYNC; pol2.tileM = kActM; pol2.tileN = 1; pol2.waitValue = gAct.x; }
    else { pol2.kind = CUSYNC_POLICY_TILESYNC; pol2.tileM = kActM; pol2.tileN = kActN; pol2.waitValue = 1; }
  }

  memset(&m->prod, 0, sizeof m->prod);
  memset(&m->cons, 0, sizeof m->cons);
  m->prod.grid = g1; m->prod.tileSize = {1, 1, 1}; m->prod.iter = 1; m->prod.opts = opts;
  m->prod.in = noSync(); m->prod.out = pol;
  m->cons.grid = g2; m->cons.tileSize = {1, 1, 1}; m->cons.iter = 1; m->cons.opts = opts;
  m->cons.in = m->actStage ? pol2 : pol; m->cons.out = noSync();
  if (cusync_stage_create(&m->prod, CUSYNC_ORDER_TRANSPOSE_XY) != CUSYNC_SUCCESS ||
      cusync_stage_create(&m->cons, CUSYNC_ORDER_TRANSPOSE_XY) != CUSYNC_SUCCESS) {
    discard(m);
    return nullptr;
  }
  if (m->actStage) {
    m->mid.grid = gAct; m->mid.tileSize = {1, 1, 1}; m->mid.iter = 1; m->mid.opts = opts;
    m->mid.in = pol; m->mid.out = pol2;
    if (cusync_stage_create(&m->mid, CUSYNC_ORDER_TRANSPOSE_XY) != CUSYNC_SUCCESS ||
        CUSYNC_HIP(hipMalloc(&m->act, (size_t)cfg->batch * cfg->inner * sizeof(half_t))) ||
        CUSYNC_HIP(hipStreamCreateWithFlags(&m->sMid, hipStreamNonBlocking))) {
      discard(m);
      return nullptr;
    }
  }
  if (sync != CUSYNC_SYNC_STREAM) {
    const bool ok = m->actStage ? cusync_set_producer_consumer_pair(&m->prod, &m->mid) == CUSYNC_SUCCESS &&
                                  cusync_set_producer_consumer_pair(&m->mid, &m->cons) == CUSYNC_SUCCESS
                                : cusync_set_producer_consumer_pair(&m->prod, &m->cons) == CUSYNC_SUCCESS;
    if (!ok) {
      setError("mlp: pairing the stages failed");
      discard(m);
      return nullptr;
    }
  }
  for (int which = 0; which < 2; which++) {
    cusync_gemm_args a = gemmArgs(m, which, nullptr, nullptr, nullptr);
    const size_t bytes = cusync_gemm_workspace_size(&a);
    if (bytes == 0) continue;
    void* ws = nullptr;
    if (CUSYNC_HIP(hipMalloc(&ws, bytes)) || CUSYNC_HIP(hipMemset(ws, 0, bytes))) { discard(m); return nullptr; }
    (which == 0 ? m->ws1 : m->ws2) = ws;
  }
  if (CUSYNC_HIP(hipStreamCreateWithFlags(&m->sProd, hipStreamNonBlocking)) ||
      CUSYNC_HIP(hipStreamCreateWithFlags(&m->sCons, hipStreamNonBlocking)) ||
      CUSYNC_HIP(hipEventCreate(&m->eStart)) || CUSYNC_HIP(hipEventCreate(&m->eMid)) ||
      CUSYNC_HIP(hipEventCreate(&m->eEnd))) {
    discard(m);
    return nullptr;
  }
  return m;
}

cusync_error cusync_mlp_reload_weights(cusync_mlp* m) {
  if (!m) return CUSYNC_ERROR_NOT_INITIALIZED;
  if (!m->w1p && !m->w2p) return CUSYNC_SUCCESS;
  // a kernel, not a copy-engine transfer: the GEMMs of the last run may have left lines of the handle's buffers
  // in the L2s, and only a kernel boundary on the device is sure to drop them
  hipStream_t s = nullptr;
  if (CUSYNC_HIP(hipDeviceSynchronize())) return CUSYNC_ERROR_DEVICE;
  const struct { const void* src; void* dst; uint32_t rows, cols, pitch; bool interleave; } job[2] = {
      {m->w1, m->w1p, m->k1, m->n1, m->ldw1, m->fused}, {m->w2, m->w2p, m->k2, m->n2, m->ldw2, false}};
  for (const auto& j : job) {
    if (!j.dst) continue;
    if (j.cols % 8 != 0 || (j.interleave && j.cols % 16 != 0)) { setError("mlp: the handle's copies of the weights need rows of whole 16-byte pieces"); return CUSYNC_ERROR_NOT_INITIALIZED; }
    const uint32_t vecs = j.cols / 8;
    const dim3 grid((vecs + 255) / 256, j.rows, 1);
    if (j.interleave) hipLaunchKernelGGL(interleaveGateUpKernel, grid, dim3(256), 0, s, (const uint4v*)j.src, (uint4v*)j.dst, vecs / 2, j.pitch / 8);
    else hipLaunchKernelGGL(repackRowsKernel, grid, dim3(256), 0, s, (const uint4v*)j.src, (uint4v*)j.dst, vecs, j.pitch / 8);
    if (CUSYNC_HIP(hipGetLastError())) return CUSYNC_ERROR_DEVICE;
  }
  if (CUSYNC_HIP(hipDeviceSynchronize())) return CUSYNC_ERROR_DEVICE;
  return CUSYNC_SUCCESS;
}

// Also the clean-up of a create() that failed half way: every member is null until it has been made
// (the handle is value-initialised), and everything here skips what is null.
void cusync_mlp_destroy(cusync_mlp* m) {
  if (!m) return;
  if (m->sProd) (void)hipStreamSynchronize(m->sProd);
  if (m->sCons) (void)hipStreamSynchronize(m->sCons);
  if (m->sMid) (void)hipStreamSynchronize(m->sMid);
  cusync_stage_free(&m->prod);        // null-safe per member
  cusync_stage_free(&m->cons);
  cusync_stage_free(&m->mid);
  if (m->act) (void)hipFree(m->act);
  if (m->ws1) (void)hipFree(m->ws1);
  if (m->ws2) (void)hipFree(m->ws2);
  if (m->w1p) (void)hipFree(m->w1p);
  if (m->w2p) (void)hipFree(m->w2p);
  if (m->eStart) (void)hipEventDestroy(m->eStart);
  if (m->eMid) (void)hipEventDestroy(m->eMid);
  if (m->eEnd) (void)hipEventDestroy(m->eEnd);
  if (m->sProd) (void)hipStreamDestroy(m->sProd);
  if (m->sCons) (void)hipStreamDestroy(m->sCons);
  if (m->sMid) (void)hipStreamDestroy(m->sMid);
  delete m;
}

cusync_error cusync_mlp_run_split(cusync_mlp* m, const void* x, void* h, void* y, int runs,
                                  double* times_us, double* gemm1_us, double* gemm2_us) {
  if (!m || !x || !h || !y) return CUSYNC_ERROR_NOT_INITIALIZED;
  const bool overlapped = m->prod.out.kind != CUSYNC_POLICY_NOSYNC;
  for (int r = 0; r < runs; r++) {
    cusync_gemm_args a1 = gemmArgs(m, 0, x, h, y);
    cusync_gemm_args a2 = gemmArgs(m, 1, x, h, y);
    cusync_error e;
    if (CUSYNC_HIP(hipEventRecord(m->eStart, m->sProd))) return CUSYNC_ERROR_DEVICE;
    if (overlapped && m->cfg.one_launch) {
      // both GEMMs in one launch: same stages and semaphores, no wait kernel, no second launch
      const cusync_gemm_args both[2] = {a1, a2};
      if ((e = cusync_gemm_chain_run(both, 2, m->sProd)) != CUSYNC_SUCCESS) return e;
      if (CUSYNC_HIP(hipEventRecord(m->eEnd, m->sProd))) return CUSYNC_ERROR_DEVICE;
    } else if ((e = cusync_gemm_run(&a1, m->sProd)) != CUSYNC_SUCCESS) {
      return e;
    } else if (overlapped) {
      // The consumer's stream is held back until every workgroup of the producer has started.  A producer launch
      // that takes every workgroup slot of the device is waited for here on the host (a wait kernel's wave on one
      // of the CUs would keep the last producer workgroup off the device until another retires); for any other
      // the reference's wait kernel goes into the consumer's stream, unordered like the reference's.
      if (m->actStage) {        // GEMM1 -> activation -> GEMM2, a stream and a hold-back per edge
        if ((e = cusync_hold_back(&m->prod, m->sMid)) != CUSYNC_SUCCESS) return e;
        if ((e = runActStage(m, h, m->sMid)) != CUSYNC_SUCCESS) return e;
        if ((e = cusync_invoke_wait_kernel(&m->mid, m->sCons)) != CUSYNC_SUCCESS) return e;
      } else if ((e = cusync_hold_back(&m->prod, m->sCons)) != CUSYNC_SUCCESS) {
        return e;
      }
      if ((e = cusync_gemm_run(&a2, m->sCons)) != CUSYNC_SUCCESS) return e;
      if (CUSYNC_HIP(hipEventRecord(m->eEnd, m->sCons))) return CUSYNC_ERROR_DEVICE;
    } else {
      if (CUSYNC_HIP(hipEventRecord(m->eMid, m->sProd))) return CUSYNC_ERROR_DEVICE;
      if (m->actStage && (e = runActStage(m, h, m->sProd)) != CUSYNC_SUCCESS) return e;     // counted with GEMM2
      if ((e = cusync_gemm_run(&a2, m->sProd)) != CUSYNC_SUCCESS) return e;
      if (CUSYNC_HIP(hipEventRecord(m->eEnd, m->sProd))) return CUSYNC_ERROR_DEVICE;
    }
    if (CUSYNC_HIP(hipEventSynchronize(m->eEnd))) return CUSYNC_ERROR_DEVICE;
    // The consumer finishing implies every producer tile was posted, but the
    // producer kernel itself must have retired before its stage is reused.
    if (overlapped && CUSYNC_HIP(hipStreamSynchronize(m->sProd))) return CUSYNC_ERROR_DEVICE;
    if (overlapped && m->actStage && CUSYNC_HIP(hipStreamSynchronize(m->sMid))) return CUSYNC_ERROR_DEVICE;
    float ms = 0;
    if (times_us) {
      if (CUSYNC_HIP(hipEventElapsedTime(&ms, m->eStart, m->eEnd))) return CUSYNC_ERROR_DEVICE;
      times_us[r] = (double)ms * 1000.0;
    }
    if (!overlapped && gemm1_us) {
      if (CUSYNC_HIP(hipEventElapsedTime(&ms, m->eStart, m->eMid))) return CUSYNC_ERROR_DEVICE;
      gemm1_us[r] = (double)ms * 1000.0;
    }
    if (!overlapped && gemm2_us) {
      if (CUSYNC_HIP(hipEventElapsedTime(&ms, m->eMid, m->eEnd))) return CUSYNC_ERROR_DEVICE;
      gemm2_us[r] = (double)ms * 1000.0;
    }
    m->prod.iter += 1;     // incrementIter on both stages, mlp.cu:709-712
    m->cons.iter += 1;
    m->mid.iter += 1;
  }
  // every run above was synchronised with; a wait that gave up let its kernel go on with unposted data
  const cusync_stage_desc* stages[3] = {&m->prod, &m->cons, &m->mid};
  return cusync::rt::checkSpinTimeouts(stages, 3, &m->timeoutsSeen, "mlp");
}

cusync_error cusync_mlp_run(cusync_mlp* m, const void* x, void* h, void* y, int runs, double* times_us) {
  return cusync_mlp_run_split(m, x, h, y, runs, times_us, nullptr, nullptr);
}

const cusync_stage_desc* cusync_mlp_stage(const cusync_mlp* m, int which) {
  if (!m) return nullptr;
  if (which == 2) return m->actStage ? &m->mid : nullptr;
  return which == 0 ? &m->prod : &m->cons;
}

int cusync_mlp_splits(const cusync_mlp* m, int* split_k1, int* split_k2) {
  if (!m) return 1;
  if (split_k1) *split_k1 = m->split1;
  if (split_k2) *split_k2 = m->split2;
  return 0;
}

int cusync_mlp_choice(const cusync_mlp_config* cfg, int* tile1, int* tile2, int* split_k1, int* split_k2, int* one_launch) {
  if (!cfg || cfg->batch == 0 || cfg->hidden == 0 || cfg->inner == 0) { setError("mlp: empty shape"); return 1; }
  Choice ch;
  if (!choose(*cfg, &ch)) return 1;
  if (tile1) *tile1 = ch.tile1;
  if (tile2) *tile2 = ch.tile2;
  if (split_k1) *split_k1 = ch.split1;
  if (split_k2) *split_k2 = ch.split2;
  if (one_launch) *one_launch = ch.oneLaunch;
  return 0;
}

int cusync_mlp_tiles(const cusync_mlp* m, int* tile1, int* tile2) {
  if (!m) return 1;
  if (tile1) *tile1 = m->tile1;
  if (tile2) *tile2 = m->tile2;
  return 0;
}

}  // extern "C"
