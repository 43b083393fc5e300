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

#include <algorithm>
#include <mutex>

#include "../../include/cusync_amd.h"
#include "rt_internal.h"
#include "gemm_kernel_dma.h"

namespace {

using namespace cusync::gemm;

struct ConvTile {
  uint32_t bm, bn, bk;
  size_t lds;
  void (*kernel)(GemmParams);
  int residentPerCU;
};

#define CUSYNC_CONV_TILE(BM, BN, BK, WM, WN, ST, OCC) \
  { BM, BN, BK, (size_t)DmaCfg<BM, BN, BK, WM, WN, ST, OCC, true>::LDS_BYTES, \
    gemmDmaKernel<DmaCfg<BM, BN, BK, WM, WN, ST, OCC, true>, kAConv>, -1 }

ConvTile g_convTiles[CUSYNC_CONV_TILE_COUNT] = {
  CUSYNC_CONV_TILE(128, 64, 32, 2, 2, 4, 3),    // CUSYNC_CONV_TILE_128x64x32
  CUSYNC_CONV_TILE(128, 128, 32, 2, 2, 4, 2),   // CUSYNC_CONV_TILE_128x128x32
  CUSYNC_CONV_TILE(256, 64, 32, 4, 1, 3, 2),    // CUSYNC_CONV_TILE_256x64x32
};

std::mutex g_convMutex;

ConvTile* convTile(int tile) {
  if (tile < 0 || tile >= CUSYNC_CONV_TILE_COUNT) return nullptr;
  return &g_convTiles[tile];
}

int residentConv(ConvTile* ti) {
  std::lock_guard<std::mutex> lock(g_convMutex);
  int dev = 0;
  hipDeviceProp_t prop;
  if (CUSYNC_HIP(hipGetDevice(&dev)) || CUSYNC_HIP(hipGetDeviceProperties(&prop, dev))) return 0;
  if (ti->residentPerCU < 0) {
    if (CUSYNC_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(ti->kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)ti->lds))) return 0;
    int n = 0;
    if (CUSYNC_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, ti->kernel, kThreads, ti->lds))) return 0;
    ti->residentPerCU = n;
  }
  return ti->residentPerCU * prop.multiProcessorCount;
}

uint32_t outExtent(uint32_t in, uint32_t filter, uint32_t pad, uint32_t stride) { return (in + 2 * pad - filter) / stride + 1; }

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

cusync_dim3 cusync_conv2d_grid(int tile, uint32_t N, uint32_t H, uint32_t W, uint32_t K, uint32_t R, uint32_t S,
                               uint32_t pad, uint32_t stride) {
  cusync_dim3 g = {0, 0, 0};
  ConvTile* ti = convTile(tile);
  if (!ti || stride == 0 || H + 2 * pad < R || W + 2 * pad < S) return g;
  const uint32_t M = N * outExtent(H, R, pad, stride) * outExtent(W, S, pad, stride);
  g.x = (K + ti->bn - 1) / ti->bn;
  g.y = (M + ti->bm - 1) / ti->bm;
  g.z = 1;
  return g;
}

cusync_error cusync_conv2d_can_implement(const cusync_conv2d_args* a) {
  using cusync::rt::setError;
  if (!a) return CUSYNC_ERROR_NOT_INITIALIZED;
  ConvTile* ti = convTile(a->tile);
  if (!ti) { setError("conv2d: unknown tile id"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (!a->N || !a->H || !a->W || !a->C || !a->K || !a->R || !a->S || !a->stride) { setError("conv2d: empty problem"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (a->H + 2 * a->pad < a->R || a->W + 2 * a->pad < a->S) { setError("conv2d: filter larger than the padded image"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (a->pad >= a->R || a->pad >= a->S) { setError("conv2d: padding must be smaller than the filter"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (a->C % ti->bk) { setError("conv2d: channels must be a multiple of the K chunk (32)"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (a->K % 8) { setError("conv2d: output channels must be a multiple of 8"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if ((uint64_t)a->N * a->H * a->W * a->C * 2 >= 0x80000000ull || (uint64_t)a->K * a->R * a->S * a->C * 2 >= 0x80000000ull) {
    setError("conv2d: operand larger than 2 GiB is not addressable by one buffer descriptor");
    return CUSYNC_ERROR_NOT_INITIALIZED;
  }
  if (((uintptr_t)a->x | (uintptr_t)a->w) % 16 || (uintptr_t)a->y % 8) { setError("conv2d: misaligned operand"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (a->epilogue < 0 || a->epilogue > CUSYNC_EPILOGUE_RELU) { setError("conv2d: unknown epilogue"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  const cusync_dim3 g = cusync_conv2d_grid(a->tile, a->N, a->H, a->W, a->K, a->R, a->S, a->pad, a->stride);
  const cusync_stage_desc& s = a->stage;
  if (s.grid.x != g.x || s.grid.y != g.y || s.grid.z != g.z) { setError("conv2d: stage grid does not match cusync_conv2d_grid"); return CUSYNC_ERROR_NOT_INITIALIZED; }
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
  return ti ? residentConv(ti) : 0;
}

cusync_error cusync_conv2d_run(const cusync_conv2d_args* a, void* stream) {
  cusync_error e = cusync_conv2d_can_implement(a);
  if (e != CUSYNC_SUCCESS) return e;
  ConvTile* ti = convTile(a->tile);
  const int resident = residentConv(ti);
  if (resident <= 0) { cusync::rt::setError("conv2d: kernel does not fit on a CU"); return CUSYNC_ERROR_DEVICE; }
  const cusync_stage_desc& s = a->stage;
  const uint32_t tiles = s.grid.x * s.grid.y * s.grid.z;
  uint32_t launched = std::min<uint32_t>(tiles, (uint32_t)resident);
  if (a->max_workgroups > 0) launched = std::min<uint32_t>(launched, (uint32_t)a->max_workgroups);

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
  p.splitK = 1;
  p.kPerSlice = (p.K + ti->bk - 1) / ti->bk * ti->bk;
  p.mPad = s.grid.y * ti->bm;
  // Producer tiles are whole 128-byte lines of the activation tensor when a pixel's channels are.
  p.stage.lineAligned = s.in.kind != CUSYNC_POLICY_NOSYNC && (uintptr_t)a->x % 128 == 0 &&
                        (a->C * 2) % 128 == 0 &&
                        (s.in.kind == CUSYNC_POLICY_ROWSYNC || (s.in.tileN * 2) % 128 == 0);
  hipLaunchKernelGGL(ti->kernel, dim3(launched), dim3(kThreads), ti->lds, (hipStream_t)stream, p);
  if (CUSYNC_HIP(hipGetLastError())) return CUSYNC_ERROR_DEVICE;
  return CUSYNC_SUCCESS;
}

}  // extern "C"
