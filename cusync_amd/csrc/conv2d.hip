// Sync-aware NHWC forward convolution as an implicit GEMM
//   [N*P*Q, R*S*C] x [R*S*C, K]  ->  y[N,P,Q,K],   k = (r*S + s)*C + c,
// cross-correlation, fp16 in, fp32 accumulate, fp16 out, optional ReLU.
// Stands in for cutlass::conv::device::CuSyncImplicitGemmConvolution
// (src/include/cutlass/cusync-cutlass/include/cutlass/conv/device/cusyncimplicit_gemm_convolution.h:226-298)
// and its kernel (conv/kernel/implicit_cusyncgemm_convolution.h:287-477,
// conv/threadblock/implicit_cusyncgemm_pipelined.h:313-492).
//
// The kernel is the direct-to-LDS GEMM kernel with two changes: the A operand is
// gathered (a K chunk of a row is one contiguous run of channels of one input
// pixel, or zeros outside the image), and B — the KRSC filter — is already
// k-contiguous, so its stage is laid out like A's and read without transpose.
// A consumer convolution waits for every producer row block that the filter's
// halo reaches, not only for the block of its own rows.
#include <hip/hip_runtime.h>

#include <string.h>
#include <algorithm>
#include <mutex>
#include <vector>

#include "../../include/cusync_amd.h"
#include "rt_internal.h"
#include "gemm_kernel_dma.h"
#include "conv3x3_kernel.h"
#include "split_choice.h"

namespace {

using namespace cusync::gemm;

struct ConvTile {
  uint32_t bm, bn, bk;
  size_t lds;
  void (*kernel)(GemmParams);
  int residentPerCU;
  void (*chainKernel)(ConvChainParams);     // several layers in one launch; halo tiles only
  void (*splitKernel)(GemmParams);          // the same tile with its steps cut into runs (split_k > 1); halo tiles only
};

#define CUSYNC_CONV_TILE(BM, BN, BK, WM, WN, ST, OCC) \
  { BM, BN, BK, (size_t)DmaCfg<BM, BN, BK, WM, WN, ST, OCC, true>::LDS_BYTES, \
    gemmDmaKernel<DmaCfg<BM, BN, BK, WM, WN, ST, OCC, true>, kAConv>, -1, nullptr, nullptr }

using HaloA = Halo3x3Cfg<256, 64, 4, 1, 4, 2>;     // 64 output channels per tile: four waves of 64 x 64 stacked
using HaloB = Halo3x3Cfg<128, 128, 2, 2, 3, 1>;    // 128 output channels per tile
using HaloC = Halo3x3Cfg<64, 128, 2, 2, 3, 1>;     // 64 pixels: what fits beside the halo of 512-channel pixels (7 x 7 images)

ConvTile g_convTiles[CUSYNC_CONV_TILE_COUNT] = {
  CUSYNC_CONV_TILE(128, 64, 32, 2, 2, 4, 3),    // CUSYNC_CONV_TILE_128x64x32
  CUSYNC_CONV_TILE(128, 128, 32, 2, 2, 4, 2),   // CUSYNC_CONV_TILE_128x128x32
  CUSYNC_CONV_TILE(256, 64, 32, 4, 1, 3, 2),    // CUSYNC_CONV_TILE_256x64x32
  // the halo tiles: 3x3 / pad 1 / stride 1 only; LDS size depends on the image width and channels
  { HaloA::BM, HaloA::BN, HaloA::BK, 0, convHalo3x3Kernel<HaloA>, -1, convHalo3x3ChainKernel<HaloA>, convHalo3x3Kernel<HaloA, true> },   // CUSYNC_CONV_TILE_HALO_256x64x64
  { HaloB::BM, HaloB::BN, HaloB::BK, 0, convHalo3x3Kernel<HaloB>, -1, convHalo3x3ChainKernel<HaloB>, convHalo3x3Kernel<HaloB, true> },   // CUSYNC_CONV_TILE_HALO_128x128x64
  { HaloC::BM, HaloC::BN, HaloC::BK, 0, convHalo3x3Kernel<HaloC>, -1, convHalo3x3ChainKernel<HaloC>, convHalo3x3Kernel<HaloC, true> },   // CUSYNC_CONV_TILE_HALO_64x128x64
};

bool isHalo(int tile) { return tile >= CUSYNC_CONV_TILE_HALO_256x64x64 && tile <= CUSYNC_CONV_TILE_HALO_64x128x64; }
uint32_t haloLds(int tile, uint32_t W, uint32_t C) {
  return tile == CUSYNC_CONV_TILE_HALO_256x64x64 ? HaloA::ldsBytes(W, C) : tile == CUSYNC_CONV_TILE_HALO_128x128x64 ? HaloB::ldsBytes(W, C) : HaloC::ldsBytes(W, C);
}
constexpr uint32_t kMaxLds = 160 * 1024 - 1024;      // what one workgroup may ask for (the kernel has 8 bytes of static LDS)

// The halo kernel needs 3x3, pad 1, stride 1, a power-of-two channel count of at least 64, and its tile plus
// halo in LDS.
bool haloEligible(int tile, uint32_t W, uint32_t C, uint32_t R, uint32_t S, uint32_t pad, uint32_t stride) {
  return R == 3 && S == 3 && pad == 1 && stride == 1 && C >= 64 && (C & (C - 1)) == 0 && haloLds(tile, W, C) <= kMaxLds;
}

std::mutex g_convMutex;

ConvTile* convTile(int tile) {
  if (tile < 0 || tile >= CUSYNC_CONV_TILE_COUNT) return nullptr;
  return &g_convTiles[tile];
}

int g_convNumCUs = 0;
uint32_t g_haloLds[CUSYNC_CONV_TILE_COUNT] = {};      // LDS size the cached occupancy of a halo kernel was computed for

int residentConv(ConvTile* ti, size_t lds) {
  std::lock_guard<std::mutex> lock(g_convMutex);
  const int idx = (int)(ti - g_convTiles);
  const bool halo = isHalo(idx);
  if (ti->residentPerCU < 0 || (halo && g_haloLds[idx] != lds)) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (CUSYNC_HIP(hipGetDevice(&dev)) || CUSYNC_HIP(hipGetDeviceProperties(&prop, dev))) return 0;
    g_convNumCUs = prop.multiProcessorCount;
    if (CUSYNC_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(ti->kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, halo ? (int)kMaxLds : (int)lds))) return 0;
    int n = 0;
    if (CUSYNC_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, ti->kernel, kThreads, lds))) return 0;
    if (ti->chainKernel) {
      // the chain kernel is the same code in a loop: it gets the same LDS allowance and must fit as often
      int m = 0;
      if (CUSYNC_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(ti->chainKernel),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLds)) ||
          CUSYNC_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&m, ti->chainKernel, kThreads, lds))) return 0;
      n = std::min(n, m);
    }
    if (ti->splitKernel) {
      int m = 0;
      if (CUSYNC_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(ti->splitKernel),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLds)) ||
          CUSYNC_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&m, ti->splitKernel, kThreads, lds))) return 0;
      n = std::min(n, m);
    }
    ti->residentPerCU = n;
    if (halo) g_haloLds[idx] = (uint32_t)lds;
  }
  return ti->residentPerCU * g_convNumCUs;
}

uint32_t outExtent(uint32_t in, uint32_t filter, uint32_t pad, uint32_t stride) { return (in + 2 * pad - filter) / stride + 1; }

size_t partialBytes(const cusync_conv2d_args* a, const ConvTile* ti) {
  const cusync_dim3 g = cusync_conv2d_grid_split(a->tile, a->N, a->H, a->W, a->K, a->R, a->S, a->pad, a->stride, a->split_k);
  return (size_t)g.z * g.y * g.x * ti->bm * ti->bn * sizeof(float);
}

// Kernel parameters of one convolution launched with `launched` workgroups.
GemmParams convParams(const cusync_conv2d_args* a, const ConvTile* ti, uint32_t launched) {
  const cusync_stage_desc& s = a->stage;
  GemmParams p = {};
  p.stage.d = s;
  p.cvN = a->N; p.cvH = a->H; p.cvW = a->W; p.cvC = a->C;
  p.cvP = outExtent(a->H, a->R, a->pad, a->stride);
  p.cvQ = outExtent(a->W, a->S, a->pad, a->stride);
  p.cvR = a->R; p.cvS = a->S; p.cvPad = a->pad; p.cvStride = a->stride;
  p.M = a->N * p.cvP * p.cvQ; p.N = a->K; p.K = a->R * a->S * a->C;
  p.A = (const half_t*)a->x; p.lda = a->C;
  p.B = (const half_t*)a->w; p.ldb = p.K;
  p.D = (half_t*)a->y; p.ldd = a->K;
  p.epilogue = a->epilogue;
  p.a_mode = CUSYNC_A_PLAIN;
  p.launched = launched;
  p.splitK = (uint32_t)std::max(1, a->split_k);
  const uint32_t chunks = (p.K + ti->bk - 1) / ti->bk;
  p.kPerSlice = (chunks + p.splitK - 1) / p.splitK * ti->bk;
  p.mPad = s.grid.y * ti->bm;
  p.waitRound = 1;
  p.coopReduce = 0; p.partialBytes = 0;
  p.partials = nullptr; p.arrivals = nullptr;
  if (p.splitK > 1) {
    // [split_k][row tiles][column tiles][BM * BN] fp32 partial sums, then two counters per output tile, as the GEMM's
    const size_t bytes = partialBytes(a, ti);
    p.partials = (float*)a->workspace;
    p.arrivals = (uint32_t*)((char*)a->workspace + bytes);
    p.partialBytes = (uint32_t)bytes;
  }
  cusync::rt::timeline(&p.timeline, &p.timelineCap);
  // Producer tiles are whole 128-byte lines of the activation tensor when a pixel's channels are.
  p.stage.lineAligned = !cusync::rt::forceAcquire() && s.in.kind != CUSYNC_POLICY_NOSYNC && (uintptr_t)a->x % 128 == 0 &&
                        (a->C * 2) % 128 == 0 &&
                        (s.in.kind == CUSYNC_POLICY_ROWSYNC || (s.in.tileN * 2) % 128 == 0);
  p.stage.releaseAll = cusync::rt::forceRelease();
  p.stage.prepare(launched);
  // the runs of a tile share the adding up when each has a workgroup of its own from the start (see gemm_f16.hip)
  p.coopReduce = slicesShareReduction((int)p.splitK, true, true, p.stage.noDraws, launched, s.grid.x * s.grid.y * s.grid.z,
                                      ti->bm, (s.opts & CUSYNC_OPT_AVOID_WAIT_KERNEL) != 0);
  return p;
}

}  // namespace

extern "C" {

int cusync_conv2d_tile_shape(int tile, uint32_t* tileM, uint32_t* tileN, uint32_t* tileK) {
  ConvTile* ti = convTile(tile);
  if (!ti) return 1;
  if (tileM) *tileM = ti->bm;
  if (tileN) *tileN = ti->bn;
  if (tileK) *tileK = ti->bk;
  return 0;
}

cusync_dim3 cusync_conv2d_grid_split(int tile, uint32_t N, uint32_t H, uint32_t W, uint32_t K, uint32_t R, uint32_t S,
                                     uint32_t pad, uint32_t stride, int split_k) {
  cusync_dim3 g = {0, 0, 0};
  ConvTile* ti = convTile(tile);
  if (!ti || stride == 0 || H + 2 * pad < R || W + 2 * pad < S) return g;
  const uint32_t M = N * outExtent(H, R, pad, stride) * outExtent(W, S, pad, stride);
  g.x = (K + ti->bn - 1) / ti->bn;
  g.y = (M + ti->bm - 1) / ti->bm;
  g.z = (uint32_t)std::max(1, split_k);
  return g;
}

cusync_dim3 cusync_conv2d_grid(int tile, uint32_t N, uint32_t H, uint32_t W, uint32_t K, uint32_t R, uint32_t S,
                               uint32_t pad, uint32_t stride) {
  return cusync_conv2d_grid_split(tile, N, H, W, K, R, S, pad, stride, 1);
}

size_t cusync_conv2d_workspace_size(const cusync_conv2d_args* a) {
  ConvTile* ti = a ? convTile(a->tile) : nullptr;
  if (!ti || a->split_k <= 1) return 0;
  const cusync_dim3 g = cusync_conv2d_grid_split(a->tile, a->N, a->H, a->W, a->K, a->R, a->S, a->pad, a->stride, a->split_k);
  return partialBytes(a, ti) + 2 * (size_t)g.x * g.y * sizeof(uint32_t);
}

cusync_error cusync_conv2d_can_implement(const cusync_conv2d_args* a) {
  using cusync::rt::setError;
  if (!a) return CUSYNC_ERROR_NOT_INITIALIZED;
  ConvTile* ti = convTile(a->tile);
  if (!ti) { setError("conv2d: unknown tile id"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (!a->N || !a->H || !a->W || !a->C || !a->K || !a->R || !a->S || !a->stride) { setError("conv2d: empty problem"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (a->H + 2 * a->pad < a->R || a->W + 2 * a->pad < a->S) { setError("conv2d: filter larger than the padded image"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (a->pad >= a->R || a->pad >= a->S) { setError("conv2d: padding must be smaller than the filter"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (a->C % ti->bk) { setError("conv2d: channels must be a multiple of the K chunk"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (isHalo(a->tile) && !haloEligible(a->tile, a->W, a->C, a->R, a->S, a->pad, a->stride)) {
    setError("conv2d: the halo tile needs a 3x3 filter, pad 1, stride 1, a power-of-two channel count >= 64 and its rows plus 2W + 2 pixels in LDS");
    return CUSYNC_ERROR_NOT_INITIALIZED;
  }
  if (a->K % 8) { setError("conv2d: output channels must be a multiple of 8"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  const uint64_t outRows = (uint64_t)((a->H + 2 * a->pad - a->R) / a->stride + 1) * ((a->W + 2 * a->pad - a->S) / a->stride + 1) * a->N;
  if ((uint64_t)a->N * a->H * a->W * a->C * 2 >= 0x80000000ull || (uint64_t)a->K * a->R * a->S * a->C * 2 >= 0x80000000ull ||
      outRows * a->K * 2 >= 0x80000000ull) {
    setError("conv2d: operand larger than 2 GiB is not addressable by one buffer descriptor");
    return CUSYNC_ERROR_NOT_INITIALIZED;
  }
  if (((uintptr_t)a->x | (uintptr_t)a->w | (uintptr_t)a->y) % 16) { setError("conv2d: misaligned operand"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (a->epilogue < 0 || a->epilogue > CUSYNC_EPILOGUE_RELU) { setError("conv2d: unknown epilogue"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (a->split_k > 1) {
    if (!ti->splitKernel) { setError("conv2d: split_k > 1 needs a halo tile"); return CUSYNC_ERROR_NOT_INITIALIZED; }
    if ((uint32_t)a->split_k > a->R * a->S * (a->C / ti->bk)) { setError("conv2d: more runs than steps (9 * C / 64)"); return CUSYNC_ERROR_NOT_INITIALIZED; }
    if (!a->workspace || (uintptr_t)a->workspace % 16) { setError("conv2d: split_k > 1 needs a 16-byte aligned workspace of cusync_conv2d_workspace_size bytes"); return CUSYNC_ERROR_NOT_INITIALIZED; }
    if (partialBytes(a, ti) >= 0x80000000ull) { setError("conv2d: partial sums larger than 2 GiB"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  }
  const cusync_dim3 g = cusync_conv2d_grid_split(a->tile, a->N, a->H, a->W, a->K, a->R, a->S, a->pad, a->stride, a->split_k);
  const cusync_stage_desc& s = a->stage;
  if (s.grid.x != g.x || s.grid.y != g.y || s.grid.z != g.z) { setError("conv2d: stage grid does not match cusync_conv2d_grid_split"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (!s.tileOrder || !s.tileCounter || !s.startCounter || !s.spinTimeouts || !s.xcdTickets) { setError("conv2d: stage not allocated"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (s.out.kind != CUSYNC_POLICY_NOSYNC && !s.tileStatusWrite) { setError("conv2d: producer stage without semaphores"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (s.in.kind != CUSYNC_POLICY_NOSYNC) {
    if (!s.tileStatusRead) { setError("conv2d: consumer stage not paired with a producer"); return CUSYNC_ERROR_NOT_INITIALIZED; }
    if (s.in.tileM == 0 || s.in.tileN == 0) { setError("conv2d: input policy with zero tile extent"); return CUSYNC_ERROR_NOT_INITIALIZED; }
    if (s.in.kind != CUSYNC_POLICY_ROWSYNC && a->C / std::max(s.in.tileN, 1u) > 32) { setError("conv2d: more than 32 producer channel tiles"); return CUSYNC_ERROR_NOT_INITIALIZED; }
    if (s.in.kind == CUSYNC_POLICY_CONV2DTILESYNC && (s.in.R != a->R || s.in.S != a->S)) { setError("conv2d: Conv2DTileSync built for another filter size"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  }
  if ((s.opts & CUSYNC_OPT_NO_ATOMIC_ADD) && s.out.kind != CUSYNC_POLICY_NOSYNC &&
      cusync::dyn::waitValue(s.out) != cusync::dyn::postValue(s.out)) {
    setError("conv2d: NoAtomicAdd needs a policy whose wait value equals its post value");
    return CUSYNC_ERROR_NOT_INITIALIZED;
  }
  return CUSYNC_SUCCESS;
}

int cusync_conv2d_max_resident(int tile) {
  ConvTile* ti = convTile(tile);
  if (!ti) return 0;
  return residentConv(ti, isHalo(tile) ? haloLds(tile, 56, 64) : ti->lds);     // the halo tiles: for 56 x 56 x 64 images
}

cusync_error cusync_conv2d_run(const cusync_conv2d_args* a, void* stream) {
  cusync_error e = cusync_conv2d_can_implement(a);
  if (e != CUSYNC_SUCCESS) return e;
  ConvTile* ti = convTile(a->tile);
  const size_t lds = isHalo(a->tile) ? haloLds(a->tile, a->W, a->C) : ti->lds;
  const int resident = residentConv(ti, lds);
  if (resident <= 0) { cusync::rt::setError("conv2d: kernel does not fit on a CU"); return CUSYNC_ERROR_DEVICE; }
  const cusync_stage_desc& s = a->stage;
  const uint32_t tiles = s.grid.x * s.grid.y * s.grid.z;
  uint32_t launched = std::min<uint32_t>(tiles, (uint32_t)resident);
  if (a->max_workgroups > 0) launched = std::min<uint32_t>(launched, (uint32_t)a->max_workgroups);

  GemmParams p = convParams(a, ti, launched);
  hipLaunchKernelGGL(a->split_k > 1 ? ti->splitKernel : ti->kernel, dim3(launched), dim3(kThreads), lds, (hipStream_t)stream, p);
  if (CUSYNC_HIP(hipGetLastError())) return CUSYNC_ERROR_DEVICE;
  cusync::rt::noteLaunch(a->stage, launched >= (uint32_t)resident);
  return CUSYNC_SUCCESS;
}

}  // extern "C"

/* ---- chain of same-shape 3x3 convolutions ------------------------------------------ */

struct cusync_conv_chain {
  cusync_conv_chain_config cfg;
  std::vector<const void*> w;
  std::vector<cusync_stage_desc> st;
  std::vector<hipStream_t> stream;
  std::vector<hipEvent_t> ev;        // layers + 1 events: start, after each layer
  std::vector<void*> ws;             // per layer: partial sums and counters of the runs a tile's steps are cut into
  int splitK = 1;
  uint32_t timeoutsSeen = 0;         // sum of the stages' give-up counters when the last run returned
};

namespace {

// After the runs of a call have been synchronised with: an error if a wait of any layer gave up meanwhile.
cusync_error chainTimeouts(cusync_conv_chain* c) {
  std::vector<const cusync_stage_desc*> stages;
  for (const auto& d : c->st) stages.push_back(&d);
  return cusync::rt::checkSpinTimeouts(stages.data(), (int)stages.size(), &c->timeoutsSeen, "conv chain");
}

cusync_policy_desc noSyncDesc() {
  cusync_policy_desc p;
  memset(&p, 0, sizeof p);
  p.kind = CUSYNC_POLICY_NOSYNC;
  p.tileM = p.tileN = 1; p.R = p.S = 1;
  return p;
}

void freeChain(cusync_conv_chain* c) {
  for (auto s : c->stream) (void)hipStreamSynchronize(s);
  for (auto& d : c->st) cusync_stage_free(&d);
  for (auto w : c->ws) (void)hipFree(w);
  for (auto e : c->ev) (void)hipEventDestroy(e);
  for (auto s : c->stream) (void)hipStreamDestroy(s);
  delete c;
}

}  // namespace

extern "C" {

cusync_conv_chain* cusync_conv_chain_create(const cusync_conv_chain_config* cfg, const void* const* weights) {
  using cusync::rt::setError;
  if (!cfg || !weights) { setError("conv chain: null argument"); return nullptr; }
  if (cfg->layers < 1 || cfg->layers > 16) { setError("conv chain: 1 to 16 layers"); return nullptr; }
  cusync_conv_chain* c = new cusync_conv_chain();
  c->cfg = *cfg;
  if (c->cfg.tile < 0)
    c->cfg.tile = cfg->C % 128 == 0 && haloEligible(CUSYNC_CONV_TILE_HALO_128x128x64, cfg->W, cfg->C, 3, 3, 1, 1) ? CUSYNC_CONV_TILE_HALO_128x128x64
                  : haloEligible(CUSYNC_CONV_TILE_HALO_256x64x64, cfg->W, cfg->C, 3, 3, 1, 1) ? CUSYNC_CONV_TILE_HALO_256x64x64
                  : cfg->C % 128 == 0 && haloEligible(CUSYNC_CONV_TILE_HALO_64x128x64, cfg->W, cfg->C, 3, 3, 1, 1) ? CUSYNC_CONV_TILE_HALO_64x128x64
                  : cfg->C % 128 == 0 ? CUSYNC_CONV_TILE_128x128x32 : CUSYNC_CONV_TILE_256x64x32;
  uint32_t tm = 0, tn = 0;
  if (cusync_conv2d_tile_shape(c->cfg.tile, &tm, &tn, nullptr)) { setError("conv chain: unknown tile id"); delete c; return nullptr; }
  if (c->cfg.fused && cfg->sync != CUSYNC_SYNC_STREAM &&
      (!isHalo(c->cfg.tile) || cfg->layers > (uint32_t)kMaxFusedLayers || !haloEligible(c->cfg.tile, cfg->W, cfg->C, 3, 3, 1, 1))) {
    setError("conv chain: one launch for all layers needs a halo tile that fits and at most 8 layers");
    delete c;
    return nullptr;
  }
  cusync_dim3 g = cusync_conv2d_grid(c->cfg.tile, cfg->N, cfg->H, cfg->W, cfg->C, 3, 3, 1, 1);
  if (g.x == 0 || g.y == 0) { setError("conv chain: empty shape"); delete c; return nullptr; }
  // Layers whose tiles leave most of the device idle (14 x 14 x 256 at batch 32: 98 tiles; 7 x 7 x 512: 100) have the
  // 9 * C / 64 steps of a tile cut into runs, a workgroup each, whose partial sums are put together as the GEMM's
  // k-slices are: as many runs as stay resident together, of at least nine steps each (measured, pairs in us without
  // runs -> with: 32x14x14x256 63 -> 54 in two; 32x7x7x512 82 -> 59 in two; 8x14x14x256 65 -> 50 in four;
  // 1x7x7x512 82 -> 43 in eight; with shorter runs the exchange costs more than the idle CUs: 1x56x56x64 35 -> 50
  // in nine runs of one step), and a number the 32-row pieces of a 128-row tile divide among, so that the runs
  // share the adding up.
  c->splitK = 1;
  if (cfg->split_k > 1) c->splitK = cfg->split_k;
  else if (cfg->split_k == 0 && isHalo(c->cfg.tile) && !(c->cfg.fused && cfg->sync != CUSYNC_SYNC_STREAM)) {
    ConvTile* ti = convTile(c->cfg.tile);
    const int resident = residentConv(ti, haloLds(c->cfg.tile, cfg->W, cfg->C));
    const uint32_t tiles = g.x * g.y, steps = 9 * (cfg->C / 64);
    uint32_t s = resident > 0 && tiles * 2 <= (uint32_t)g_convNumCUs ? std::min<uint32_t>((uint32_t)resident / tiles, steps / 9) : 1u;
    if (tm >= 128) s = s >= 4 ? 4 : s == 3 ? 2 : s;      // a 128-row tile's four pieces divide among two or four runs
    while (s > 1 && (steps + s - 1) / s * (s - 1) >= steps) s--;      // no run without steps
    c->splitK = (int)std::max(1u, s);
  }
  if (c->splitK > 1 && (!isHalo(c->cfg.tile) || (c->cfg.fused && cfg->sync != CUSYNC_SYNC_STREAM))) {
    setError("conv chain: cutting a tile's steps into runs needs a halo tile and one launch per layer");
    delete c;
    return nullptr;
  }
  if (c->splitK > 1 && (uint32_t)c->splitK > 9 * (cfg->C / 64)) {
    setError("conv chain: more runs than a tile has steps (9 * C / 64)");
    delete c;
    return nullptr;
  }
  g.z = (uint32_t)c->splitK;

  // Edge policies: what a layer posts and what the next one waits on
  // (src/ml-bench/volta_conv2d/resnet.cu:107-116; in vgg.cu the middle layers are consumer and producer at once).
  cusync_policy_desc post = noSyncDesc(), wait = noSyncDesc();
  int opts = 0;
  switch (cfg->sync) {
    case CUSYNC_SYNC_STREAM:
      break;
    case CUSYNC_SYNC_ROW:
      post.kind = CUSYNC_POLICY_ROWSYNC; post.order = CUSYNC_ORDER_TRANSPOSE_XY;
      post.tileM = tm; post.tileN = 1; post.waitValue = g.x; post.postValue = 1;
      wait = post;
      break;
    case CUSYNC_SYNC_TILE:
      post.kind = CUSYNC_POLICY_TILESYNC; post.order = CUSYNC_ORDER_TRANSPOSE_XY;
      post.tileM = tm; post.tileN = tn; post.waitValue = 1; post.postValue = 1;
      wait = post;
      wait.kind = CUSYNC_POLICY_CONV2DTILESYNC; wait.R = 3; wait.S = 3;
      opts = CUSYNC_OPT_NO_ATOMIC_ADD | CUSYNC_OPT_REORDER_TILE_LOADS;
      break;
    default:
      setError("conv chain: sync must be STREAM, ROW or TILE");
      delete c;
      return nullptr;
  }
  if (cfg->opts >= 0) opts |= cfg->opts;
  c->st.resize(cfg->layers);
  for (uint32_t i = 0; i < cfg->layers; i++) memset(&c->st[i], 0, sizeof c->st[i]);
  for (uint32_t i = 0; i < cfg->layers; i++) {
    c->w.push_back(weights[i]);
    cusync_stage_desc& d = c->st[i];
    d.grid = g; d.tileSize = {1, 1, 1}; d.iter = 1; d.opts = opts;
    d.in = i == 0 ? noSyncDesc() : wait;
    d.out = i + 1 == cfg->layers ? noSyncDesc() : post;
    if (!weights[i] || cusync_stage_create(&d, CUSYNC_ORDER_TRANSPOSE_XY) != CUSYNC_SUCCESS) { freeChain(c); return nullptr; }
  }
  if (cfg->sync != CUSYNC_SYNC_STREAM)
    for (uint32_t i = 0; i + 1 < cfg->layers; i++)
      if (cusync_set_producer_consumer_pair(&c->st[i], &c->st[i + 1]) != CUSYNC_SUCCESS) { freeChain(c); return nullptr; }
  const uint32_t streams = cfg->sync == CUSYNC_SYNC_STREAM ? 1 : cfg->layers;
  for (uint32_t i = 0; i < streams; i++) {
    hipStream_t s;
    if (CUSYNC_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking))) { freeChain(c); return nullptr; }
    c->stream.push_back(s);
  }
  for (uint32_t i = 0; i <= cfg->layers; i++) {
    hipEvent_t e;
    if (CUSYNC_HIP(hipEventCreate(&e))) { freeChain(c); return nullptr; }
    c->ev.push_back(e);
  }
  if (c->splitK > 1) {
    cusync_conv2d_args a;
    memset(&a, 0, sizeof a);
    a.N = cfg->N; a.H = cfg->H; a.W = cfg->W; a.C = cfg->C; a.K = cfg->C; a.R = a.S = 3; a.pad = 1; a.stride = 1;
    a.tile = c->cfg.tile; a.split_k = c->splitK;
    const size_t bytes = cusync_conv2d_workspace_size(&a);
    for (uint32_t i = 0; i < cfg->layers; i++) {
      void* w = nullptr;
      if (CUSYNC_HIP(hipMalloc(&w, bytes)) || CUSYNC_HIP(hipMemset(w, 0, bytes))) { if (w) (void)hipFree(w); freeChain(c); return nullptr; }
      c->ws.push_back(w);
    }
  }
  return c;
}

void cusync_conv_chain_destroy(cusync_conv_chain* c) {
  if (c) freeChain(c);
}

cusync_error cusync_conv_chain_run(cusync_conv_chain* c, const void* x, void* const* ys, int runs,
                                   double* times_us, double* layer_us) {
  if (!c || !x || !ys) return CUSYNC_ERROR_NOT_INITIALIZED;
  const uint32_t n = c->cfg.layers;
  const bool overlapped = c->cfg.sync != CUSYNC_SYNC_STREAM;
  auto layerArgs = [&](uint32_t i) {
    cusync_conv2d_args a;
    memset(&a, 0, sizeof a);
    a.stage = c->st[i];
    a.N = c->cfg.N; a.H = c->cfg.H; a.W = c->cfg.W; a.C = c->cfg.C; a.K = c->cfg.C;
    a.R = a.S = 3; a.pad = 1; a.stride = 1;
    a.x = i == 0 ? x : ys[i - 1];
    a.w = c->w[i];
    a.y = ys[i];
    a.epilogue = (c->cfg.relu && i + 1 < n) ? CUSYNC_EPILOGUE_RELU : CUSYNC_EPILOGUE_NONE;
    a.tile = c->cfg.tile;
    a.split_k = c->splitK;
    a.workspace = c->splitK > 1 ? c->ws[i] : nullptr;
    return a;
  };
  if (overlapped && c->cfg.fused) {
    // all layers in one launch on the first stream
    ConvTile* ti = convTile(c->cfg.tile);
    const size_t lds = haloLds(c->cfg.tile, c->cfg.W, c->cfg.C);
    const int resident = residentConv(ti, lds);
    if (resident <= 0) { cusync::rt::setError("conv chain: kernel does not fit on a CU"); return CUSYNC_ERROR_DEVICE; }
    const cusync_dim3& g = c->st[0].grid;
    const uint32_t launched = std::min<uint32_t>(g.x * g.y * g.z, (uint32_t)resident);
    for (int r = 0; r < runs; r++) {
      ConvChainParams cp = {};
      cp.layers = n;
      for (uint32_t i = 0; i < n; i++) {
        const cusync_conv2d_args a = layerArgs(i);
        const cusync_error e = cusync_conv2d_can_implement(&a);
        if (e != CUSYNC_SUCCESS) return e;
        cp.layer[i] = convParams(&a, ti, launched);
      }
      if (CUSYNC_HIP(hipEventRecord(c->ev[0], c->stream[0]))) return CUSYNC_ERROR_DEVICE;
      hipLaunchKernelGGL(ti->chainKernel, dim3(launched), dim3(kThreads), lds, c->stream[0], cp);
      if (CUSYNC_HIP(hipGetLastError()) || CUSYNC_HIP(hipEventRecord(c->ev[n], c->stream[0])) ||
          CUSYNC_HIP(hipEventSynchronize(c->ev[n]))) return CUSYNC_ERROR_DEVICE;
      float ms = 0;
      if (times_us) {
        if (CUSYNC_HIP(hipEventElapsedTime(&ms, c->ev[0], c->ev[n]))) return CUSYNC_ERROR_DEVICE;
        times_us[r] = (double)ms * 1000.0;
      }
      for (uint32_t i = 0; i < n; i++) c->st[i].iter += 1;
    }
    return chainTimeouts(c);
  }
  for (int r = 0; r < runs; r++) {
    if (CUSYNC_HIP(hipEventRecord(c->ev[0], c->stream[0]))) return CUSYNC_ERROR_DEVICE;
    for (uint32_t i = 0; i < n; i++) {
      hipStream_t s = c->stream[overlapped ? i : 0];
      const cusync_conv2d_args a = layerArgs(i);
      cusync_error e;
      // overlapped: layer i's stream is held back until layer i - 1 is on the device: by the reference's wait kernel
      // where that layer's launch left workgroup slots free (392 tiles on 512 slots for the benchmark shapes), so
      // that the wait kernel's wave takes nothing from the producer; from this thread where the launch took them all.
      if (overlapped && i > 0 && (e = cusync_hold_back(&c->st[i - 1], s)) != CUSYNC_SUCCESS) return e;
      if ((e = cusync_conv2d_run(&a, s)) != CUSYNC_SUCCESS) return e;
      if ((!overlapped || i + 1 == n) && CUSYNC_HIP(hipEventRecord(c->ev[i + 1], s))) return CUSYNC_ERROR_DEVICE;
    }
    if (CUSYNC_HIP(hipEventSynchronize(c->ev[n]))) return CUSYNC_ERROR_DEVICE;
    if (overlapped)
      for (uint32_t i = 0; i + 1 < n; i++)
        if (CUSYNC_HIP(hipStreamSynchronize(c->stream[i]))) return CUSYNC_ERROR_DEVICE;
    float ms = 0;
    if (times_us) {
      if (CUSYNC_HIP(hipEventElapsedTime(&ms, c->ev[0], c->ev[n]))) return CUSYNC_ERROR_DEVICE;
      times_us[r] = (double)ms * 1000.0;
    }
    if (!overlapped && layer_us)
      for (uint32_t i = 0; i < n; i++) {
        if (CUSYNC_HIP(hipEventElapsedTime(&ms, c->ev[i], c->ev[i + 1]))) return CUSYNC_ERROR_DEVICE;
        layer_us[(size_t)r * n + i] = (double)ms * 1000.0;
      }
    for (uint32_t i = 0; i < n; i++) c->st[i].iter += 1;
  }
  return chainTimeouts(c);
}

const cusync_stage_desc* cusync_conv_chain_stage(const cusync_conv_chain* c, uint32_t which) {
  if (!c || which >= c->cfg.layers) return nullptr;
  return &c->st[which];
}

int cusync_conv_chain_tile(const cusync_conv_chain* c) { return c ? c->cfg.tile : -1; }
int cusync_conv_chain_split(const cusync_conv_chain* c) { return c ? c->splitK : -1; }

}  // extern "C"
