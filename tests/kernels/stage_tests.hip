// GPU test kernels written against the public C++ API (include/cusync/cusync.h),
// the way a user of the library writes sync-aware kernels.  Built into
// libcusync_stage_tests.so and driven from pytest through extern "C" entry points.
//
// Protocols follow the reference's own tests:
//   run_simple_test  — tests/simple-test.cu:34-105 (two copy kernels synchronised
//                      per block; data and semaphore values checked)
//   run_two_matmuls  — src/examples/twoMatMuls/matrixMul.cu:41-121, 127-272 (two
//                      chained 32x32-tiled fp32 GEMMs, consumer waits per k-tile)
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <vector>

#include <cusync/cusync.h>
#include <cusync/gemm.h>
#include <type_traits>

#define HIP_OK(cmd) do { hipError_t e_ = (cmd); if (e_ != hipSuccess) { \
  printf("HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); return -1; } } while (0)

namespace cusync {
// Same role as tests/cusync-test.h of the reference: a friend of CuStage that
// checks, from inside the consumer kernel, that the semaphore a block waited on
// holds exactly expectedWaitValue * iter.
class CuSyncTest {
public:
  char* semValid;   // device, one flag per stage
  template<typename Stage>
  __device__ void setSemValue(uint32_t stageIdx, dim3 tile, Stage& stage) {
    if (!stage.isConsumer()) return;
    if (threadIdx.x == 0 && threadIdx.y == 0) {
      const bool eq = stage.expectedWaitValue(tile) * (uint32_t)stage.iter == stage.waitSemValue(tile);
      if (!eq) semValid[stageIdx] = 0;
    }
  }
  template<typename Stage> static int iterOf(Stage& s) { return s.iter; }
};
}  // namespace cusync

using namespace cusync;

template<typename Stage>
__global__ void copyKernel(CuSyncTest cutest, Stage stage, int idx, const uint32_t* in, uint32_t* out) {
  __shared__ int tileSh[3];
  dim3 tile = stage.tile((dim3*)&tileSh[0]);
  stage.wait(tile);
  // The block copies the slice that belongs to the tile it was handed, so the
  // data check also covers the ticket -> tile mapping.
  const uint32_t linear = threadIdx.x + tile.x * blockDim.x;
  out[linear] = in[linear];
  stage.post(tile);
  cutest.setSemValue(idx, tile, stage);
}

struct SimpleResult {
  int32_t data_ok, sems_ok, prod_status, cons_status, pair_status, wait_status;
  uint32_t tile_counter_prod, tile_counter_cons, kernel_executed, spin_timeouts;
};

template<typename Prod, typename Cons, typename Sync>
static int runSimple(int iters, uint32_t blocks, SimpleResult* res, uint32_t* semsOut, uint32_t* orderOut) {
  const uint32_t threadsPerBlock = 128;
  const size_t size = (size_t)blocks * threadsPerBlock;
  uint32_t *a1, *a2, *a3;
  HIP_OK(hipMalloc(&a1, size * 4)); HIP_OK(hipMalloc(&a2, size * 4)); HIP_OK(hipMalloc(&a3, size * 4));
  std::vector<uint32_t> host(size);
  for (size_t i = 0; i < size; i++) host[i] = (uint32_t)i;
  HIP_OK(hipMemcpy(a1, host.data(), size * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemset(a2, 0, size * 4)); HIP_OK(hipMemset(a3, 0, size * 4));
  hipStream_t prodStream, consStream;
  HIP_OK(hipStreamCreateWithFlags(&consStream, hipStreamNonBlocking));
  HIP_OK(hipStreamCreateWithFlags(&prodStream, hipStreamNonBlocking));

  dim3 threads(threadsPerBlock, 1, 1), grid(blocks, 1, 1);
  Sync sync;
  Prod prod(grid, threads, NoSync(), sync);
  Cons cons(grid, threads, sync, NoSync());
  res->prod_status = prod.status();
  res->cons_status = cons.status();
  res->pair_status = CuSync::setProducerConsumerPair(prod, cons);

  CuSyncTest cutest;
  HIP_OK(hipMalloc(&cutest.semValid, 1));
  HIP_OK(hipMemset(cutest.semValid, 1, 1));

  res->wait_status = CuSyncSuccess;
  for (int i = 0; i < iters; i++) {
    hipLaunchKernelGGL(copyKernel<Prod>, grid, threads, 0, prodStream, cutest, prod, -1, a1, a2);
    int w = prod.invokeWaitKernel(consStream);
    if (w != CuSyncSuccess) res->wait_status = w;
    hipLaunchKernelGGL(copyKernel<Cons>, grid, threads, 0, consStream, cutest, cons, 0, a2, a3);
    HIP_OK(hipDeviceSynchronize());
    prod.incrementIter();
    cons.incrementIter();
  }

  bool eq = true;
  HIP_OK(hipMemcpy(host.data(), a2, size * 4, hipMemcpyDeviceToHost));
  for (size_t i = 0; i < size; i++) eq = eq && host[i] == (uint32_t)i;
  HIP_OK(hipMemcpy(host.data(), a3, size * 4, hipMemcpyDeviceToHost));
  for (size_t i = 0; i < size; i++) eq = eq && host[i] == (uint32_t)i;
  res->data_ok = eq;
  char valid = 0;
  HIP_OK(hipMemcpy(&valid, cutest.semValid, 1, hipMemcpyDeviceToHost));
  res->sems_ok = valid;

  cusync_stage_desc pd = prod.desc(), cd = cons.desc();
  uint32_t startCounter = 0;
  if (cusync_stage_read_state(&pd, semsOut, (cusync_dim3*)orderOut, &res->tile_counter_prod, &startCounter,
                              &res->kernel_executed, nullptr) != CUSYNC_SUCCESS) return -1;
  if (cusync_stage_read_state(&cd, nullptr, nullptr, &res->tile_counter_cons, nullptr, nullptr,
                              &res->spin_timeouts) != CUSYNC_SUCCESS) return -1;

  prod.destroy(); cons.destroy();
  HIP_OK(hipFree(a1)); HIP_OK(hipFree(a2)); HIP_OK(hipFree(a3)); HIP_OK(hipFree(cutest.semValid));
  HIP_OK(hipStreamDestroy(prodStream)); HIP_OK(hipStreamDestroy(consStream));
  return 0;
}

// ---- two chained fp32 GEMMs on 32x32 tiles (user-written kernel) -------------

const int BLOCK = 32;
using MMSync = TileSync<IdentityOrder, BLOCK, BLOCK>;
using MMProd = CuStage<IdentityOrder, NoSync, MMSync>;
using MMCons = CuStage<IdentityOrder, MMSync, NoSync>;

template<typename Stage>
__global__ void tiledSgemm(Stage stage, float* C, const float* A, const float* B, int wA, int wB) {
  __shared__ int tileSh[3];
  __shared__ float As[BLOCK][BLOCK];
  __shared__ float Bs[BLOCK][BLOCK];
  dim3 t = stage.tile((dim3*)&tileSh[0]);
  const int bx = t.x, by = t.y, tx = threadIdx.x, ty = threadIdx.y;
  float sum = 0;
  for (int k0 = 0; k0 < wA; k0 += BLOCK) {
    // A's tile (columns k0.., rows by*32..) is the producer's output tile {k0/32, by}.
    dim3 need((uint32_t)k0, (uint32_t)by * BLOCK, 1);
    stage.wait(need);
    As[ty][tx] = A[(by * BLOCK + ty) * wA + k0 + tx];
    Bs[ty][tx] = B[(k0 + ty) * wB + bx * BLOCK + tx];
    __syncthreads();
#pragma unroll
    for (int k = 0; k < BLOCK; k++) sum += As[ty][k] * Bs[k][tx];
    __syncthreads();
  }
  C[(by * BLOCK + ty) * wB + bx * BLOCK + tx] = sum;
  stage.post(dim3((uint32_t)bx * BLOCK, (uint32_t)by * BLOCK, 0));
}

extern "C" {

// variant: 0 none, 1 NoAtomicAdd, 2 AvoidCustomOrder (tests/simple-test.cu:107-137)
int run_simple_test(int variant, int iters, uint32_t blocks, SimpleResult* res, uint32_t* semsOut, uint32_t* orderOut) {
  using Sync = TileSync<IdentityOrder, 1, 1>;
  if (variant == 0)
    return runSimple<CuStage<IdentityOrder, NoSync, Sync>, CuStage<IdentityOrder, Sync, NoSync>, Sync>(iters, blocks, res, semsOut, orderOut);
  if (variant == 1)
    return runSimple<CuStage<IdentityOrder, NoSync, Sync, NoAtomicAdd>, CuStage<IdentityOrder, Sync, NoSync>, Sync>(iters, blocks, res, semsOut, orderOut);
  if (variant == 2)
    return runSimple<CuStage<IdentityOrder, NoSync, Sync, AvoidCustomOrder>, CuStage<IdentityOrder, Sync, NoSync>, Sync>(iters, blocks, res, semsOut, orderOut);
  return -2;
}

// C = A*B then E = C*D, all n x n fp32 device pointers supplied by the caller.
// semsOut receives the (n/32)^2 semaphores of the producer.
int run_two_matmuls(int n, const float* A, const float* B, const float* D, float* C, float* E,
                    uint32_t* semsOut, int* statusOut) {
  if (n % BLOCK) return -2;
  hipStream_t prodStream, consStream;
  HIP_OK(hipStreamCreateWithFlags(&consStream, hipStreamNonBlocking));
  HIP_OK(hipStreamCreateWithFlags(&prodStream, hipStreamNonBlocking));
  dim3 threads(BLOCK, BLOCK, 1), grid(n / BLOCK, n / BLOCK, 1);
  MMSync sync;
  MMProd prod(grid, threads, NoSync(), sync);
  MMCons cons(grid, threads, sync, NoSync());
  statusOut[0] = CuSync::setProducerConsumerPair(prod, cons);
  hipLaunchKernelGGL(tiledSgemm<MMProd>, grid, threads, 0, prodStream, prod, C, A, B, n, n);
  statusOut[1] = prod.invokeWaitKernel(consStream);
  hipLaunchKernelGGL(tiledSgemm<MMCons>, grid, threads, 0, consStream, cons, E, (const float*)C, D, n, n);
  HIP_OK(hipDeviceSynchronize());
  prod.incrementIter(); cons.incrementIter();
  cusync_stage_desc pd = prod.desc(), cd = cons.desc();
  uint32_t timeouts = 0;
  if (cusync_stage_read_state(&pd, semsOut, nullptr, nullptr, nullptr, nullptr, nullptr) != CUSYNC_SUCCESS) return -1;
  if (cusync_stage_read_state(&cd, nullptr, nullptr, nullptr, nullptr, nullptr, &timeouts) != CUSYNC_SUCCESS) return -1;
  statusOut[2] = (int)timeouts;
  prod.destroy(); cons.destroy();
  HIP_OK(hipStreamDestroy(prodStream)); HIP_OK(hipStreamDestroy(consStream));
  return 0;
}

// Host-only checks of the error paths (no kernel is launched).
// out[0] pair(consumer-as-producer)  out[1] pair(producer-as-consumer)
// out[2] invokeWaitKernel on a non-producer  out[3] status() of a valid stage
// out[4] pair with a default-constructed producer
int run_error_paths(int* out) {
  using Sync = TileSync<IdentityOrder, 1, 1>;
  using P = CuStage<IdentityOrder, NoSync, Sync>;
  using Cn = CuStage<IdentityOrder, Sync, NoSync>;
  dim3 grid(4, 1, 1), threads(64, 1, 1);
  Sync sync;
  P prod(grid, threads, NoSync(), sync);
  Cn cons(grid, threads, sync, NoSync());
  out[0] = CuSync::setProducerConsumerPair(cons, cons);
  out[1] = CuSync::setProducerConsumerPair(prod, prod);
  out[2] = cons.invokeWaitKernel(nullptr);
  out[3] = prod.status();
  P empty;
  out[4] = CuSync::setProducerConsumerPair(empty, cons);
  prod.destroy(); cons.destroy();
  return 0;
}

// ---- the GPT-3 MLP loop of the reference's driver, on the launcher objects ------------------------------------
// Written after runCuSyncGPT3 (src/ml-bench/transformer/mlp.cu:645-716): Arguments{stage, size, refs, {alpha, beta},
// split_k}, get_workspace_size, can_implement, initialize, and per run  gemm_op1.run(true, NULL, producer_stream),
// prod.invokeWaitKernel(consumer_stream), gemm_op2.run(true, NULL, consumer_stream), then incrementIter on the
// stages and on the launchers' params_.custage.  policy 0: TileSync + NoAtomicAdd (mlp.cu:9-16, 111), 1: RowSync.
// x [M][K1], w1 [K1][N1], h [M][N1], w2 [N1][N2], y [M][N2]: fp16 device pointers.
// out[0] sum of every Status / CuSyncError that was not success (0 = all good)  out[1] spin time-outs
// out[2] producer's wait-kernel flag after the last run  out[3] semaphore mismatches against iters (TileSync) or iters * gN (RowSync)
}  // extern "C"

constexpr int kLauncherTile = CUSYNC_TILE_128x128x32;
using LTileSync = TileSync<TransposeXYOrder, 128, 128>;
using LRowSync = RowSync<128>;

template<typename Sync, int Opts>
static int launcherChainImpl(Sync sync, uint32_t M, uint32_t K1, uint32_t N1, uint32_t N2, const void* x, const void* w1, void* h,
                             const void* w2, void* y, int splitK1, int iters, int* out) {
  using ProdCuStage = CuStage<TransposeXYOrder, NoSync, Sync, Opts>;
  using ConsCuStage = CuStage<TransposeXYOrder, Sync, NoSync, Opts>;
  using Gemm1 = CuSyncGemm<ProdCuStage, kLauncherTile, CUSYNC_EPILOGUE_GELU>;
  using Gemm2 = CuSyncGemm<ConsCuStage, kLauncherTile, CUSYNC_EPILOGUE_NONE>;
  int bad = 0;
  const GemmCoord size1((int)M, (int)N1, (int)K1), size2((int)M, (int)N2, (int)N1);
  const dim3 gridDim1 = Gemm1::get_grid_shape(size1, splitK1), gridDim2 = Gemm2::get_grid_shape(size2, 1);
  ProdCuStage prod(gridDim1, dim3(1, 1, 1), NoSync(), sync);
  ConsCuStage cons(gridDim2, dim3(1, 1, 1), sync, NoSync());
  bad += CuSync::setProducerConsumerPair(prod, cons) != CuSyncSuccess;

  hipStream_t producer_stream, consumer_stream;
  HIP_OK(hipStreamCreateWithFlags(&producer_stream, hipStreamNonBlocking));
  HIP_OK(hipStreamCreateWithFlags(&consumer_stream, hipStreamNonBlocking));

  typename Gemm1::Arguments args1{prod, size1, {(const half_bits*)x, (int)K1}, {(const half_bits*)w1, (int)N1},
                                  {(const half_bits*)h, (int)N1}, {(half_bits*)h, (int)N1}, {1.0f, 0.0f}, splitK1};
  Gemm1 gemm_op1;
  size_t workspace_size = Gemm1::get_workspace_size(args1);
  void* workspace1 = nullptr;
  if (workspace_size) HIP_OK(hipMalloc(&workspace1, workspace_size));
  bad += gemm_op1.can_implement(args1) != Status::kSuccess;
  bad += gemm_op1.initialize(args1, workspace1) != Status::kSuccess;

  typename Gemm2::Arguments args2{cons, size2, {(const half_bits*)h, (int)N1}, {(const half_bits*)w2, (int)N2},
                                  {(const half_bits*)y, (int)N2}, {(half_bits*)y, (int)N2}, {1.0f, 0.0f}, 1};
  Gemm2 gemm_op2;
  bad += Gemm2::get_workspace_size(args2) != 0;
  bad += gemm_op2.can_implement(args2) != Status::kSuccess;
  bad += gemm_op2.initialize(args2, nullptr) != Status::kSuccess;
  // what the launcher refuses: a beta term, and k-slices without a workspace
  typename Gemm2::Arguments withBeta = args2;
  withBeta.epilogue = {1.0f, 1.0f};
  bad += Gemm2::can_implement(withBeta) != Status::kErrorNotSupported;
  typename Gemm1::Arguments sliced = args1;
  sliced.split_k_slices = 2;
  { Gemm1 tmp; bad += tmp.initialize(sliced, nullptr) != Status::kErrorWorkspaceNull; }

  hipEvent_t start, end;
  HIP_OK(hipEventCreate(&start)); HIP_OK(hipEventCreate(&end));
  for (int r = 0; r < iters; r++) {
    HIP_OK(hipEventRecord(start, producer_stream));
    bad += gemm_op1.run(true, NULL, producer_stream) != Status::kSuccess;
    bad += prod.invokeWaitKernel(consumer_stream) != CuSyncSuccess;
    bad += gemm_op2.run(true, NULL, consumer_stream) != Status::kSuccess;
    HIP_OK(hipEventRecord(end, consumer_stream));
    HIP_OK(hipEventSynchronize(end));
    HIP_OK(hipStreamSynchronize(producer_stream));
    prod.incrementIter();
    cons.incrementIter();
    gemm_op2.params_.custage.incrementIter();
    gemm_op1.params_.custage.incrementIter();
  }
  out[0] = bad;
  const cusync_stage_desc pd = prod.desc(), cd = cons.desc();
  const uint32_t tiles = gridDim1.x * gridDim1.y * gridDim1.z;
  std::vector<uint32_t> sems(tiles);
  uint32_t flag = 0, timeouts = 0;
  if (cusync_stage_read_state(&pd, sems.data(), nullptr, nullptr, nullptr, &flag, nullptr) != CUSYNC_SUCCESS) return -1;
  if (cusync_stage_read_state(&cd, nullptr, nullptr, nullptr, nullptr, nullptr, &timeouts) != CUSYNC_SUCCESS) return -1;
  out[1] = (int)timeouts;
  out[2] = (int)flag;
  int mismatches = 0;
  const bool rows = std::is_same<Sync, LRowSync>::value;
  for (uint32_t i = 0; i < tiles; i++) {
    const uint32_t want = rows ? (i < gridDim1.y ? (uint32_t)iters * gridDim1.x : 0u) : (i < gridDim1.x * gridDim1.y ? (uint32_t)iters : 0u);
    mismatches += sems[i] != want;
  }
  out[3] = mismatches;
  prod.destroy(); cons.destroy();
  if (workspace1) HIP_OK(hipFree(workspace1));
  HIP_OK(hipEventDestroy(start)); HIP_OK(hipEventDestroy(end));
  HIP_OK(hipStreamDestroy(producer_stream)); HIP_OK(hipStreamDestroy(consumer_stream));
  return 0;
}

extern "C" {

int run_launcher_mlp(int policy, uint32_t M, uint32_t K1, uint32_t N1, uint32_t N2, const void* x, const void* w1, void* h,
                     const void* w2, void* y, int splitK1, int iters, int* out) {
  if (policy == 0) {
    LTileSync sync;
    return launcherChainImpl<LTileSync, NoAtomicAdd | ReorderTileLoads>(sync, M, K1, N1, N2, x, w1, h, w2, y, splitK1, iters, out);
  }
  const dim3 g1 = CuSyncGemm<CuStage<TransposeXYOrder, NoSync, LRowSync>, kLauncherTile>::get_grid_shape(GemmCoord((int)M, (int)N1, (int)K1), splitK1);
  LRowSync sync(g1.x);
  return launcherChainImpl<LRowSync, NoOptimization>(sync, M, K1, N1, N2, x, w1, h, w2, y, splitK1, iters, out);
}

// ---- the ResNet pair on the convolution launcher (src/ml-bench/volta_conv2d/resnet.cu:107-116, 704-744) -------------
// x [N][H][W][C], w1 and w2 [C][3][3][C], y1 and y2 [N][H][W][C].  out as above (semaphores: TileSync, all == iters).
// splitK > 1: Conv2dProblemSize::split_k_slices (resnet.cu:689), with the workspace get_workspace_size asks for.
extern "C++" {
template<int kTile, int kTileM, int kTileN>
static int launcherConvPairImpl(uint32_t N, uint32_t H, uint32_t W, uint32_t C, const void* x, const void* w1, void* y1, const void* w2, void* y2,
                                int splitK, int iters, int* out) {
  using Sync1 = TileSync<TransposeXYOrder, kTileM, kTileN>;
  using Sync2 = Conv2DTileSync<TransposeXYOrder, 3, 3, kTileM, kTileN>;
  using ProdCuStage = CuStage<TransposeXYOrder, NoSync, Sync1>;
  using ConsCuStage = CuStage<TransposeXYOrder, Sync2, NoSync>;
  using Conv1 = CuSyncImplicitGemmConvolution<ProdCuStage, kTile, CUSYNC_EPILOGUE_RELU>;
  using Conv2 = CuSyncImplicitGemmConvolution<ConsCuStage, kTile, CUSYNC_EPILOGUE_NONE>;
  int bad = 0;
  const Conv2dProblemSize problem((int)N, (int)H, (int)W, (int)C, (int)C, 3, 3, 1, 1, splitK);
  const dim3 grid = Conv1::get_grid_shape(problem);
  Sync1 sync1;
  Sync2 sync2;
  ProdCuStage prod(grid, dim3(1, 1, 1), NoSync(), sync1);
  ConsCuStage cons(grid, dim3(1, 1, 1), sync2, NoSync());
  bad += CuSync::setProducerConsumerPair(prod, cons) != CuSyncSuccess;
  hipStream_t s1, s2;
  HIP_OK(hipStreamCreateWithFlags(&s1, hipStreamNonBlocking));
  HIP_OK(hipStreamCreateWithFlags(&s2, hipStreamNonBlocking));
  typename Conv1::Arguments args1(prod, problem, {(const half_bits*)x, (int)C}, {(const half_bits*)w1, (int)C}, {(const half_bits*)y1, (int)C}, {(half_bits*)y1, (int)C});
  typename Conv2::Arguments args2(cons, problem, {(const half_bits*)y1, (int)C}, {(const half_bits*)w2, (int)C}, {(const half_bits*)y2, (int)C}, {(half_bits*)y2, (int)C});
  Conv1 conv1;
  Conv2 conv2;
  bad += Conv1::can_implement(args1) != Status::kSuccess;
  void *ws1 = nullptr, *ws2 = nullptr;
  const size_t wsBytes = Conv1::get_workspace_size(args1);
  bad += (splitK > 1) != (wsBytes > 0);
  if (wsBytes) {
    bad += conv1.initialize(args1) != Status::kErrorWorkspaceNull;      // runs without a workspace are refused
    HIP_OK(hipMalloc(&ws1, wsBytes)); HIP_OK(hipMalloc(&ws2, wsBytes));
    HIP_OK(hipMemset(ws1, 0, wsBytes)); HIP_OK(hipMemset(ws2, 0, wsBytes));
  }
  bad += conv1.initialize(args1, ws1) != Status::kSuccess;
  bad += conv2.initialize(args2, ws2) != Status::kSuccess;
  for (int r = 0; r < iters; r++) {
    bad += conv1.run(true, NULL, s1) != Status::kSuccess;
    bad += prod.invokeWaitKernel(s2) != CuSyncSuccess;
    bad += conv2.run(true, NULL, s2) != Status::kSuccess;
    HIP_OK(hipDeviceSynchronize());
    prod.incrementIter();
    cons.incrementIter();
    conv1.params_.custage.incrementIter();
    conv2.params_.custage.incrementIter();
  }
  out[0] = bad;
  const cusync_stage_desc pd = prod.desc(), cd = cons.desc();
  const uint32_t tiles = grid.x * grid.y * grid.z;
  std::vector<uint32_t> sems(tiles);
  uint32_t flag = 0, timeouts = 0;
  if (cusync_stage_read_state(&pd, sems.data(), nullptr, nullptr, nullptr, &flag, nullptr) != CUSYNC_SUCCESS) return -1;
  if (cusync_stage_read_state(&cd, nullptr, nullptr, nullptr, nullptr, nullptr, &timeouts) != CUSYNC_SUCCESS) return -1;
  out[1] = (int)timeouts;
  out[2] = (int)flag;
  int mismatches = 0;
  // one post per output tile, whatever the runs: grid.x * grid.y semaphores stand at `iters`, the others were never touched
  uint32_t posted = 0;
  for (uint32_t i = 0; i < tiles; i++) { posted += sems[i] == (uint32_t)iters; mismatches += sems[i] != 0 && sems[i] != (uint32_t)iters; }
  mismatches += posted != grid.x * grid.y;
  out[3] = mismatches;
  prod.destroy(); cons.destroy();
  HIP_OK(hipStreamDestroy(s1)); HIP_OK(hipStreamDestroy(s2));
  if (ws1) HIP_OK(hipFree(ws1));
  if (ws2) HIP_OK(hipFree(ws2));
  return 0;
}
}  // extern "C++"

int run_launcher_conv_pair(uint32_t N, uint32_t H, uint32_t W, uint32_t C, const void* x, const void* w1, void* y1, const void* w2, void* y2,
                           int iters, int* out) {
  return launcherConvPairImpl<CUSYNC_CONV_TILE_128x64x32, 128, 64>(N, H, W, C, x, w1, y1, w2, y2, 1, iters, out);
}

// the same pair on the 128x128 halo tile with every tile's steps in `splitK` runs
int run_launcher_conv_pair_runs(uint32_t N, uint32_t H, uint32_t W, uint32_t C, const void* x, const void* w1, void* y1, const void* w2, void* y2,
                                int splitK, int iters, int* out) {
  return launcherConvPairImpl<CUSYNC_CONV_TILE_HALO_128x128x64, 128, 128>(N, H, W, C, x, w1, y1, w2, y2, splitK, iters, out);
}

}  // extern "C"
