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

#include "gemm_tiles.h"
#include "split_choice.h"

namespace {

using namespace cusync::gemm;

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------

TileInfo g_tiles[CUSYNC_TILE_COUNT];
std::once_flag g_tilesOnce;

std::mutex g_mutex;
int g_numCUs = 0;
uint32_t g_ldsPerCU = 0;

// The kernels are instantiated in several translation units (they take minutes to compile); each fills in
// the entries of the tiles it holds.
TileInfo* tileInfo(int tile) {
  if (tile < 0 || tile >= CUSYNC_TILE_COUNT) return nullptr;
  std::call_once(g_tilesOnce, [] {
    fillStagedTiles(g_tiles);
    fillDmaTilesWide(g_tiles);
    fillDmaTilesMid(g_tiles);
    fillDmaTilesFew(g_tiles);
    fillDmaTilesXWide(g_tiles);
  });
  return &g_tiles[tile];
}

// A consumer stage of a tile policy waits K chunk by K chunk; the row policies wait once per tile, and a stage
// without an input policy not at all (same test as in the kernel).
bool waitsPerChunk(const cusync_stage_desc& s) {
  return s.in.kind != CUSYNC_POLICY_NOSYNC && s.in.kind != CUSYNC_POLICY_ROWSYNC && s.in.kind != CUSYNC_POLICY_CONSECUTIVESYNC;
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
      g_ldsPerCU = (uint32_t)prop.maxSharedMemoryPerMultiProcessor;
    }
    int perCU = 1 << 30;
    for (int v = 0; v < 2; v++) {
      if (!ti->kernel[v]) continue;
      if (CUSYNC_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(ti->kernel[v]),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)std::max<size_t>(ti->lds, g_ldsPerCU / 2)))) return 0;
      int n = 0;
      if (CUSYNC_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, ti->kernel[v], (int)ti->threads, ti->lds))) return 0;
      perCU = std::min(perCU, n);
    }
    const void* others[2] = { reinterpret_cast<const void*>(ti->chainKernel), reinterpret_cast<const void*>(ti->kernelNoChunkWaits) };
    for (const void* k : others) {
      if (!k) continue;
      int n = 0;
      if (CUSYNC_HIP(hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)std::max<size_t>(ti->lds, g_ldsPerCU / 2))) ||
          CUSYNC_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, k, (int)ti->threads, ti->lds))) return 0;
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

static size_t partialBytes(const cusync_gemm_args* a, const TileInfo* ti);

cusync_error cusync_gemm_can_implement(const cusync_gemm_args* a) {
  using cusync::rt::setError;
  if (!a) return CUSYNC_ERROR_NOT_INITIALIZED;
  TileInfo* ti = tileInfo(a->tile);
  if (!ti) { setError("gemm: unknown tile id"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (a->M == 0 || a->N == 0 || a->K == 0) { setError("gemm: empty problem"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (a->K % 8 || a->N % 8) { setError("gemm: K and N must be multiples of 8 (16-byte loads)"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (a->lda % 8 || a->ldb % 8 || a->ldd % 8) { setError("gemm: leading dimensions must keep 16-byte alignment"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  const uint32_t aCols = a->a_mode == CUSYNC_A_SWIGLU ? 2 * a->K : a->K;
  const uint32_t dCols = a->epilogue == CUSYNC_EPILOGUE_SWIGLU ? a->N / 2 : a->N;
  if (a->lda < aCols || a->ldb < a->N || a->ldd < dCols) { setError("gemm: leading dimension smaller than the row"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if ((uint64_t)a->M * a->lda * 2 >= 0x80000000ull || (uint64_t)a->K * a->ldb * 2 >= 0x80000000ull ||
      (uint64_t)a->M * a->ldd * 2 >= 0x80000000ull) {
    setError("gemm: operand larger than 2 GiB is not addressable by one buffer descriptor");
    return CUSYNC_ERROR_NOT_INITIALIZED;
  }
  if (((uintptr_t)a->A | (uintptr_t)a->B | (uintptr_t)a->D) % 16) { setError("gemm: misaligned operand"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (a->a_mode == CUSYNC_A_SWIGLU && !ti->kernel[1]) { setError("gemm: this tile shape has no SwiGLU variant"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (a->split_k < 1) { setError("gemm: split_k must be at least 1"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (a->split_k > 1) {
    if ((uint32_t)a->split_k > (a->K + ti->bk - 1) / ti->bk) { setError("gemm: more k-slices than K chunks"); return CUSYNC_ERROR_NOT_INITIALIZED; }
    if (!everySliceHasAChunk(a->K, ti->bk, (uint32_t)a->split_k)) { setError("gemm: split_k leaves the last k-slice without a K chunk (each slice takes ceil(chunks / split_k) chunks)"); return CUSYNC_ERROR_NOT_INITIALIZED; }
    if (!a->workspace || (uintptr_t)a->workspace % 16) { setError("gemm: split_k > 1 needs a 16-byte aligned workspace of cusync_gemm_workspace_size bytes"); return CUSYNC_ERROR_NOT_INITIALIZED; }
    if (a->N % 4) { setError("gemm: split_k needs N % 4 == 0"); return CUSYNC_ERROR_NOT_INITIALIZED; }
    if (partialBytes(a, ti) >= 0x80000000ull) { setError("gemm: the partial sums of these k-slices exceed 2 GiB, more than one buffer descriptor addresses"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  }
  if (a->tile == CUSYNC_TILE_256x384x32 || a->tile == CUSYNC_TILE_256x192x64) {
    // A is fetched 64 columns of K at a time, and nothing masks a piece that reaches past the end of a row or of a k-slice
    const uint32_t chunks = a->K / 32, slices = (uint32_t)std::max(a->split_k, 1);
    if (a->K % 64 || (a->tile == CUSYNC_TILE_256x384x32 && ((chunks + slices - 1) / slices) % 2)) {
      setError("gemm: the 256x384x32 and 256x192x64 tiles take K 64 columns at a time: K (and with split_k > 1 every k-slice) must be a multiple of 64");
      return CUSYNC_ERROR_NOT_INITIALIZED;
    }
  }
  if (a->a_mode != CUSYNC_A_PLAIN && a->a_mode != CUSYNC_A_SWIGLU) { setError("gemm: unknown a_mode"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (a->epilogue < 0 || a->epilogue > CUSYNC_EPILOGUE_SWIGLU) { setError("gemm: unknown epilogue"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (a->epilogue == CUSYNC_EPILOGUE_SWIGLU && a->N % 16) { setError("gemm: the SwiGLU epilogue pairs groups of eight columns: N must be a multiple of 16"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  const cusync_dim3 g = cusync_gemm_grid(a->tile, a->M, a->N, a->split_k);
  const cusync_stage_desc& s = a->stage;
  if (s.grid.x != g.x || s.grid.y != g.y || s.grid.z != g.z) {
    setError("gemm: stage grid does not match cusync_gemm_grid(tile, M, N, split_k)");
    return CUSYNC_ERROR_NOT_INITIALIZED;
  }
  if (!s.tileOrder || !s.tileCounter || !s.startCounter || !s.spinTimeouts || !s.xcdTickets) { setError("gemm: stage not allocated"); return CUSYNC_ERROR_NOT_INITIALIZED; }
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

// [split_k][m-tiles][n-tiles][BM*BN] fp32 partial sums (each tile in the order its workgroup holds it in
// registers), then two counters per output tile (slices that wrote their partial sums, slices that stored their share).
static size_t partialBytes(const cusync_gemm_args* a, const TileInfo* ti) {
  const cusync_dim3 g = cusync_gemm_grid(a->tile, a->M, a->N, a->split_k);
  return (size_t)a->split_k * g.y * g.x * ti->bm * ti->bn * sizeof(float);
}

// Kernel parameters of one GEMM launched with `launched` workgroups.
static GemmParams gemmParams(const cusync_gemm_args* a, const TileInfo* ti, uint32_t launched) {
  const cusync_stage_desc& s = a->stage;
  GemmParams p;
  p.stage.d = s;
  // Producer tiles are whole 128-byte lines of A when the row pitch, the base and the producer's tile width all
  // are multiples of 128 bytes (64 halfs); the row policies guard whole rows.  With a tile width that is not,
  // the direct-to-LDS kernels make every wait cover whole lines instead (GemmParams::waitRound), which serves
  // the same end: no line of A is fetched before everything in it has been posted.
  const bool rowPolicy = s.in.kind == CUSYNC_POLICY_ROWSYNC || s.in.kind == CUSYNC_POLICY_CONSECUTIVESYNC;
  const bool wholeLineTiles = rowPolicy || (s.in.tileN * 2) % 128 == 0;
  const bool canRound = ti->chainKernel != nullptr && a->a_mode == CUSYNC_A_PLAIN;      // a direct-to-LDS tile
  p.stage.lineAligned = !cusync::rt::forceAcquire() && s.in.kind != CUSYNC_POLICY_NOSYNC && (uintptr_t)a->A % 128 == 0 &&
                        (a->lda * 2) % 128 == 0 && (wholeLineTiles || canRound);
  p.stage.releaseAll = cusync::rt::forceRelease();
  p.waitRound = p.stage.lineAligned && !wholeLineTiles ? 64 : 1;
  p.stage.prepare(launched);
  p.M = a->M; p.N = a->N; p.K = a->K;
  p.A = (const half_t*)a->A; p.lda = a->lda;
  p.B = (const half_t*)a->B; p.ldb = a->ldb;
  p.D = (half_t*)a->D; p.ldd = a->ldd;
  p.epilogue = a->epilogue;
  p.a_mode = a->a_mode;
  p.launched = launched;
  p.splitK = (uint32_t)a->split_k;
  const uint32_t chunks = (a->K + ti->bk - 1) / ti->bk;
  p.kPerSlice = (chunks + p.splitK - 1) / p.splitK * ti->bk;
  p.mPad = s.grid.y * ti->bm;
  cusync::rt::timeline(&p.timeline, &p.timelineCap);
  p.partials = (float*)a->workspace;
  p.arrivals = a->split_k > 1 ? (uint32_t*)((char*)a->workspace + partialBytes(a, ti)) : nullptr;
  p.partialBytes = a->split_k > 1 ? (uint32_t)partialBytes(a, ti) : 0;
  // every k-slice has its own workgroup from the start, and the tile's 32-row pieces divide among the slices.
  // Tiles of 128 rows and more only: with the small tiles of the few-row GEMMs, whose slices finish up to 10 us
  // apart, the same scheme (also cut finer, into 32x32 pieces) ended every launch 6-12 us later than the slice
  // that arrives last doing all of it.  Never under AvoidWaitKernel (see slicesShareReduction).
  const bool direct = ti->chainKernel != nullptr;
  p.coopReduce = slicesShareReduction(a->split_k, a->shared_reduction != 0, direct, p.stage.noDraws, launched,
                                      s.grid.x * s.grid.y * s.grid.z, ti->bm, (s.opts & CUSYNC_OPT_AVOID_WAIT_KERNEL) != 0) &&
                 !getenv("CUSYNC_NO_COOP_REDUCE");
  return p;
}

size_t cusync_gemm_workspace_size(const cusync_gemm_args* a) {
  TileInfo* ti = a ? tileInfo(a->tile) : nullptr;
  if (!ti || a->split_k <= 1) return 0;
  const cusync_dim3 g = cusync_gemm_grid(a->tile, a->M, a->N, a->split_k);
  return partialBytes(a, ti) + 2 * (size_t)g.x * g.y * sizeof(uint32_t);      // partial sums, then two counters per output tile
}

// ---- split-K workspace held by the library itself ------------------------------------------------------------
// cusync_gemm_run_static_workspace takes the k-slices' partial sums and arrival counters from this array instead
// of from memory the caller allocated.  Each device the library runs on holds its own copy until the process ends.
// In host code the array's name is only a handle for hipGetSymbolAddress: the device address it yields, looked up
// once per device, is what kernels and fills are given.
static __device__ __align__(256) unsigned char scratch[CUSYNC_GEMM_STATIC_WORKSPACE_BYTES];

namespace {

constexpr int kMaxDevices = 64;
void* g_scratchPtr[kMaxDevices] = {};      // device address of `scratch` on each device, null until looked up
std::mutex g_scratchMutex;

// Device address of this device's copy of `scratch`; null (and an error text) if the runtime would not give it.
void* scratchOfCurrentDevice() {
  int dev = 0;
  if (CUSYNC_HIP(hipGetDevice(&dev))) return nullptr;
  if (dev < 0 || dev >= kMaxDevices) { cusync::rt::setError("gemm: device index beyond the table of static workspaces"); return nullptr; }
  std::lock_guard<std::mutex> lock(g_scratchMutex);
  if (!g_scratchPtr[dev]) {
    void* p = nullptr;
    if (CUSYNC_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)))) return nullptr;
    g_scratchPtr[dev] = p;
  }
  return g_scratchPtr[dev];
}

// A fill kernel rather than hipMemsetAsync: memset nodes recorded into a captured graph have given wrong
// results on replays, and this entry point is for callers that may be under capture.
__global__ void zeroWordsKernel(uint32_t* p, uint32_t n) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

}  // namespace

cusync_error cusync_gemm_run_static_workspace(const cusync_gemm_args* a, void* stream) {
  if (!a) return CUSYNC_ERROR_NOT_INITIALIZED;
  cusync_gemm_args mine = *a;
  mine.workspace = nullptr;
  if (mine.split_k > 1) {
    TileInfo* ti = tileInfo(mine.tile);
    if (!ti) { cusync::rt::setError("gemm: unknown tile id"); return CUSYNC_ERROR_NOT_INITIALIZED; }
    const size_t need = cusync_gemm_workspace_size(&mine);
    if (need > (size_t)CUSYNC_GEMM_STATIC_WORKSPACE_BYTES) {
      cusync::rt::setError("gemm: this split-K problem needs " + std::to_string(need) + " bytes of workspace, the library's own holds " +
                           std::to_string((size_t)CUSYNC_GEMM_STATIC_WORKSPACE_BYTES) + "; use cusync_gemm_run with a workspace of the caller's");
      return CUSYNC_ERROR_NOT_INITIALIZED;
    }
    void* ws = scratchOfCurrentDevice();
    if (!ws) return CUSYNC_ERROR_DEVICE;
    mine.workspace = ws;
    const cusync_error ok = cusync_gemm_can_implement(&mine);
    if (ok != CUSYNC_SUCCESS) return ok;
    // The arrival counters sit behind the partial sums, at an offset that depends on the problem: what the last
    // call left there is another problem's data.  The partial sums need no clearing (every slice writes its own
    // before anyone adds them up).
    const cusync_dim3 g = cusync_gemm_grid(mine.tile, mine.M, mine.N, mine.split_k);
    const uint32_t counters = 2 * g.x * g.y;
    uint32_t* arrivals = (uint32_t*)((char*)ws + partialBytes(&mine, ti));
    hipLaunchKernelGGL(zeroWordsKernel, dim3((counters + 255) / 256), dim3(256), 0, (hipStream_t)stream, arrivals, counters);
    if (CUSYNC_HIP(hipGetLastError())) return CUSYNC_ERROR_DEVICE;
  }
  return cusync_gemm_run(&mine, stream);
}

cusync_error cusync_gemm_run(const cusync_gemm_args* a, void* stream) {
  cusync_error e = cusync_gemm_can_implement(a);
  if (e != CUSYNC_SUCCESS) return e;
  TileInfo* ti = tileInfo(a->tile);
  const int resident = residentWorkgroups(a->tile);
  if (resident <= 0) {     // keep what the runtime said, if it said anything
    const std::string why = cusync_rt_last_error();
    cusync::rt::setError("gemm: kernel does not fit on a CU" + (why.empty() ? std::string() : " (" + why + ")"));
    return CUSYNC_ERROR_DEVICE;
  }
  const cusync_stage_desc& s = a->stage;
  const uint32_t tiles = s.grid.x * s.grid.y * s.grid.z;
  uint32_t launched = std::min<uint32_t>(tiles, (uint32_t)resident);
  if (a->max_workgroups > 0) launched = std::min<uint32_t>(launched, (uint32_t)a->max_workgroups);

  const GemmParams p = gemmParams(a, ti, launched);
  void (*kernel)(GemmParams) = ti->kernel[a->a_mode == CUSYNC_A_SWIGLU ? 1 : 0];
  // the few-row tiles come with a kernel compiled without the per-chunk waits, for stages that never make them
  if (a->a_mode != CUSYNC_A_SWIGLU && ti->kernelNoChunkWaits && !waitsPerChunk(s)) kernel = ti->kernelNoChunkWaits;
  // A consumer's workgroups are dispatched while the producer's hold their CUs, and where two of them fit a CU the
  // dispatcher packs them in pairs onto the CUs the producer left free: when the producer is done, half the device
  // runs the consumer two to a CU and the other half nothing (LLaMA MLP, 640 to 1024 rows under RowSync: 144-175 us
  // against 140-164 stream-ordered).  A launch of no more workgroups than CUs therefore asks for half a CU's LDS,
  // which with the kernel's few static bytes lets one workgroup onto a CU and leaves the other half to the producer
  // (the same chains: 132-159 us).  A launch of at most half as many workgroups as CUs is left to be packed: it is
  // resident beside the producer at once and leaves whole CUs to the stage after it (measured on the attention
  // kernel, see cusync_attention_run).  Nor a launch under AvoidWaitKernel, which may reach the device before its
  // producer: holding half of every CU it could keep a producer that needs more than the other half off the device.
  size_t lds = ti->lds;
  if (s.in.kind != CUSYNC_POLICY_NOSYNC && !(s.opts & CUSYNC_OPT_AVOID_WAIT_KERNEL) && launched <= (uint32_t)g_numCUs &&
      launched > (uint32_t)g_numCUs / 2 && ti->residentPerCU > 1)
    lds = std::max<size_t>(lds, g_ldsPerCU / 2);
  hipLaunchKernelGGL(kernel, dim3(launched), dim3(ti->threads), lds, (hipStream_t)stream, p);
  if (CUSYNC_HIP(hipGetLastError())) return CUSYNC_ERROR_DEVICE;
  cusync::rt::noteLaunch(s, launched >= (uint32_t)resident);
  return CUSYNC_SUCCESS;
}

int cusync_gemm_fills_device(const cusync_gemm_args* a) {
  if (!a || !tileInfo(a->tile)) return 0;
  const int resident = residentWorkgroups(a->tile);
  if (resident <= 0) return 0;
  const cusync_dim3 g = cusync_gemm_grid(a->tile, a->M, a->N, a->split_k);
  uint32_t launched = std::min<uint32_t>(g.x * g.y * g.z, (uint32_t)resident);
  if (a->max_workgroups > 0) launched = std::min<uint32_t>(launched, (uint32_t)a->max_workgroups);
  return launched >= (uint32_t)resident ? 1 : 0;
}

cusync_error cusync_gemm_chain_run(const cusync_gemm_args* args, int count, void* stream) {
  using cusync::rt::setError;
  if (!args || count < 1 || count > kMaxChainedGemms) { setError("gemm chain: 1 to 4 GEMMs"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  TileInfo* ti = tileInfo(args[0].tile);
  if (!ti || !ti->chainKernel) { setError("gemm chain: needs a direct-to-LDS tile"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  const int resident = residentWorkgroups(args[0].tile);
  if (resident <= 0) { setError("gemm: kernel does not fit on a CU"); return CUSYNC_ERROR_DEVICE; }
  uint32_t launched = (uint32_t)resident, mostTiles = 0;
  for (int i = 0; i < count; i++) {
    const cusync_gemm_args& a = args[i];
    if (a.tile != args[0].tile) { setError("gemm chain: all GEMMs must use the same tile"); return CUSYNC_ERROR_NOT_INITIALIZED; }
    if (a.a_mode != CUSYNC_A_PLAIN) { setError("gemm chain: plain A operands only"); return CUSYNC_ERROR_NOT_INITIALIZED; }
    const cusync_error e = cusync_gemm_can_implement(&a);
    if (e != CUSYNC_SUCCESS) return e;
    if (a.stage.in.kind != CUSYNC_POLICY_NOSYNC && i == 0) { setError("gemm chain: the first GEMM cannot wait on a stage outside the launch"); return CUSYNC_ERROR_NOT_INITIALIZED; }
    mostTiles = std::max<uint32_t>(mostTiles, a.stage.grid.x * a.stage.grid.y * a.stage.grid.z);
    if (a.max_workgroups > 0) launched = std::min<uint32_t>(launched, (uint32_t)a.max_workgroups);
  }
  // As many workgroups as the GEMM with most tiles has (and the device holds at once).  A workgroup without a tile
  // of GEMM i goes straight on to GEMM i+1 and waits there for tiles that running workgroups hold.
  launched = std::min<uint32_t>(launched, mostTiles);
  GemmChainParams cp = {};
  cp.count = (uint32_t)count;
  for (int i = 0; i < count; i++) cp.gemm[i] = gemmParams(&args[i], ti, launched);
  hipLaunchKernelGGL(ti->chainKernel, dim3(launched), dim3(ti->threads), ti->lds, (hipStream_t)stream, cp);
  if (CUSYNC_HIP(hipGetLastError())) return CUSYNC_ERROR_DEVICE;
  return CUSYNC_SUCCESS;
}

}  // extern "C"
