// Launcher objects for the sync-aware kernels, shaped like the reference's
// cutlass::gemm::device::CuSyncGemm (src/include/cutlass/cusync-cutlass/include/cutlass/gemm/device/cusyncgemm.h:
// Arguments :293-350, can_implement :364-386, get_workspace_size :388-404, initialize :407-456, update :458-476,
// run :494-563, public params_ :352) and cutlass::conv::device::CuSyncImplicitGemmConvolution
// (.../conv/device/cusyncimplicit_gemm_convolution.h:226-298), so that the driver loops written against them
// (src/ml-bench/transformer/mlp.cu:645-716: Arguments{stage, size, refs, {alpha, beta}, split_k}, get_workspace_size,
// can_implement, initialize, then per run  op.run(true, NULL, stream)  and  op.params_.custage.incrementIter())
// carry over line by line.  Host code only, C++14, over the C ABI of cusync_amd.h: the kernels are the library's
// hand-written gfx950 kernels, chosen by a tile id instead of a threadblock-shape template.
#pragma once

#include <stddef.h>
#include <stdint.h>

#include "cusync.h"

namespace cusync {

// The values of cutlass::Status the launchers return (cutlass/cutlass.h), by the same names.
enum class Status { kSuccess, kErrorMisalignedOperand, kErrorInvalidProblem, kErrorNotSupported, kErrorWorkspaceNull, kErrorInternal };

inline const char* cusyncGetStatusString(Status s) {
  switch (s) {
    case Status::kSuccess: return "Success";
    case Status::kErrorMisalignedOperand: return "Error Misaligned Operand";
    case Status::kErrorInvalidProblem: return "Error Invalid Problem";
    case Status::kErrorNotSupported: return "Error Not Supported";
    case Status::kErrorWorkspaceNull: return "Error Workspace Null";
    default: return "Error Internal";
  }
}

// cutlass::gemm::GemmCoord: (m, n, k).
struct GemmCoord {
  int m_, n_, k_;
  GemmCoord(int m = 0, int n = 0, int k = 0) : m_(m), n_(n), k_(k) {}
  int m() const { return m_; }
  int n() const { return n_; }
  int k() const { return k_; }
};

// cutlass::TensorRef for a row-major fp16 matrix: a device pointer and the row pitch in elements.
template<typename Element>
struct TensorRef {
  Element* ptr_;
  int stride_;
  TensorRef(Element* ptr = nullptr, int stride = 0) : ptr_(ptr), stride_(stride) {}
  Element* data() const { return ptr_; }
  int stride(int = 0) const { return stride_; }
  void reset(Element* ptr) { ptr_ = ptr; }
};

typedef uint16_t half_bits;      // fp16 storage; the host never computes on it

// EpilogueOutputOp::Params of LinearCombination: D = alpha * accumulator + beta * C.  The kernels compute
// alpha = 1, beta = 0 (what every driver of the reference passes, mlp.cu:244); anything else is refused.
struct LinearCombinationParams {
  float alpha, beta;
  LinearCombinationParams(float a = 1.0f, float b = 0.0f) : alpha(a), beta(b) {}
};

// ThreadblockShape of a tile id at compile time, for the policies whose tile extents are template arguments
// (RowSync<kM>, TileSync<Order, kM, kN>: mlp.cu:1026-1037 takes them from ShapeThreadBlock1).  The same numbers as
// cusync_gemm_tile_shape() returns at run time.
template<int TileId> struct GemmTileShape;
#define CUSYNC_GEMM_TILE_SHAPE(ID, M, N, K) \
  template<> struct GemmTileShape<ID> { static constexpr uint32_t kM = M, kN = N, kK = K; }
CUSYNC_GEMM_TILE_SHAPE(CUSYNC_TILE_256x256x32, 256, 256, 32);
CUSYNC_GEMM_TILE_SHAPE(CUSYNC_TILE_256x128x64, 256, 128, 64);
CUSYNC_GEMM_TILE_SHAPE(CUSYNC_TILE_128x128x64, 128, 128, 64);
CUSYNC_GEMM_TILE_SHAPE(CUSYNC_TILE_64x128x64, 64, 128, 64);
CUSYNC_GEMM_TILE_SHAPE(CUSYNC_TILE_32x128x64, 32, 128, 64);
CUSYNC_GEMM_TILE_SHAPE(CUSYNC_TILE_128x256x64, 128, 256, 64);
CUSYNC_GEMM_TILE_SHAPE(CUSYNC_TILE_256x64x64, 256, 64, 64);
CUSYNC_GEMM_TILE_SHAPE(CUSYNC_TILE_128x64x64, 128, 64, 64);
CUSYNC_GEMM_TILE_SHAPE(CUSYNC_TILE_256x128x32, 256, 128, 32);
CUSYNC_GEMM_TILE_SHAPE(CUSYNC_TILE_128x256x32, 128, 256, 32);
CUSYNC_GEMM_TILE_SHAPE(CUSYNC_TILE_128x128x32, 128, 128, 32);
CUSYNC_GEMM_TILE_SHAPE(CUSYNC_TILE_128x192x32, 128, 192, 32);
CUSYNC_GEMM_TILE_SHAPE(CUSYNC_TILE_256x192x32, 256, 192, 32);
CUSYNC_GEMM_TILE_SHAPE(CUSYNC_TILE_D32x128x64, 32, 128, 64);
CUSYNC_GEMM_TILE_SHAPE(CUSYNC_TILE_D64x128x64, 64, 128, 64);
CUSYNC_GEMM_TILE_SHAPE(CUSYNC_TILE_D64x192x64, 64, 192, 64);
CUSYNC_GEMM_TILE_SHAPE(CUSYNC_TILE_128x192x32_ALONE, 128, 192, 32);
CUSYNC_GEMM_TILE_SHAPE(CUSYNC_TILE_256x384x32, 256, 384, 32);
CUSYNC_GEMM_TILE_SHAPE(CUSYNC_TILE_256x192x64, 256, 192, 64);
CUSYNC_GEMM_TILE_SHAPE(CUSYNC_TILE_D128x192x64, 128, 192, 64);
#undef CUSYNC_GEMM_TILE_SHAPE

// CuSyncGemm<CuStageImpl, TileId, Epilogue>: D = epilogue(A x B), fp16 row-major, fp32 accumulate.
//   TileId    CUSYNC_TILE_*  (stands in for ThreadblockShape / WarpShape / Stages)
//   Epilogue  CUSYNC_EPILOGUE_*  (LinearCombination, LinearCombinationGELU, LinearCombinationRelu, ...)
template<typename CuStageImpl, int TileId, int Epilogue = CUSYNC_EPILOGUE_NONE>
class CuSyncGemm {
 public:
  typedef TensorRef<const half_bits> TensorRefA;
  typedef TensorRef<const half_bits> TensorRefB;
  typedef TensorRef<const half_bits> TensorRefC;
  typedef TensorRef<half_bits> TensorRefD;

  struct Arguments {
    CuStageImpl custage;
    GemmCoord problem_size;
    TensorRefA ref_A;
    TensorRefB ref_B;
    TensorRefC ref_C;          // source of the beta term: unused (beta = 0), kept for the argument order
    TensorRefD ref_D;
    LinearCombinationParams epilogue;
    int split_k_slices;
    Arguments() : split_k_slices(1) {}
    Arguments(CuStageImpl custage_, GemmCoord problem_size_, TensorRefA ref_A_, TensorRefB ref_B_, TensorRefC ref_C_,
              TensorRefD ref_D_, LinearCombinationParams epilogue_ = LinearCombinationParams(), int split_k_slices_ = 1)
        : custage(custage_), problem_size(problem_size_), ref_A(ref_A_), ref_B(ref_B_), ref_C(ref_C_), ref_D(ref_D_),
          epilogue(epilogue_), split_k_slices(split_k_slices_) {}
  };

  // What run() launches with.  `custage` is public as in the reference: the driver loop calls
  // params_.custage.incrementIter() between runs and the next run() picks the new iteration up.
  struct Params {
    CuStageImpl custage;
    GemmCoord problem_size;
    TensorRefA ref_A;
    TensorRefB ref_B;
    TensorRefD ref_D;
    int split_k_slices;
    void* workspace;
    int max_workgroups;        // 0: as many as stay resident
    Params() : split_k_slices(1), workspace(nullptr), max_workgroups(0) {}
  };
  Params params_;

  CuSyncGemm() {}

  // The tile grid the stage given to Arguments must have been built with:
  // CuSyncGemmHorizontalThreadblockSwizzle::get_grid_shape(get_tiled_shape(problem, tile, split_k)).
  static dim3 get_grid_shape(GemmCoord problem_size, int split_k_slices = 1) {
    const cusync_dim3 g = cusync_gemm_grid(TileId, (uint32_t)problem_size.m(), (uint32_t)problem_size.n(), split_k_slices);
    return dim3(g.x, g.y, g.z);
  }

  static Status can_implement(Arguments const& args) {
    if (args.epilogue.alpha != 1.0f || args.epilogue.beta != 0.0f) return Status::kErrorNotSupported;
    cusync_gemm_args a = toArgs(args.custage, args.problem_size, args.ref_A, args.ref_B, args.ref_D, args.split_k_slices,
                                (void*)(uintptr_t)16 /* any aligned non-null pointer: the workspace comes with initialize() */, 0);
    return cusync_gemm_can_implement(&a) == CUSYNC_SUCCESS ? Status::kSuccess : Status::kErrorInvalidProblem;
  }

  static size_t get_workspace_size(Arguments const& args) {
    cusync_gemm_args a = toArgs(args.custage, args.problem_size, args.ref_A, args.ref_B, args.ref_D, args.split_k_slices, nullptr, 0);
    return cusync_gemm_workspace_size(&a);
  }

  // Stores the arguments and, with k-slices, clears the workspace (the reference clears its semaphores the
  // same way, cusyncgemm.h:432-440; here on the calling thread, `stream` is accepted for the signature).
  Status initialize(Arguments const& args, void* workspace = nullptr, void* stream = nullptr) {
    (void)stream;
    if (args.epilogue.alpha != 1.0f || args.epilogue.beta != 0.0f) return Status::kErrorNotSupported;
    if (args.split_k_slices > 1) {
      if (!workspace) return Status::kErrorWorkspaceNull;
      if (cusync_rt_memset(workspace, 0, get_workspace_size(args)) != 0) return Status::kErrorInternal;
    }
    params_.custage = args.custage;
    params_.problem_size = args.problem_size;
    params_.ref_A = args.ref_A;
    params_.ref_B = args.ref_B;
    params_.ref_D = args.ref_D;
    params_.split_k_slices = args.split_k_slices;
    params_.workspace = workspace;
    cusync_gemm_args a = toArgs(params_.custage, params_.problem_size, params_.ref_A, params_.ref_B, params_.ref_D,
                                params_.split_k_slices, params_.workspace, params_.max_workgroups);
    return cusync_gemm_can_implement(&a) == CUSYNC_SUCCESS ? Status::kSuccess : Status::kErrorInvalidProblem;
  }

  // Lightweight update of the operand pointers (cusyncgemm.h:458-491).
  Status update(Arguments const& args, void* workspace = nullptr) {
    if (args.split_k_slices > 1 && !workspace) return Status::kErrorWorkspaceNull;
    params_.ref_A.reset(args.ref_A.data());
    params_.ref_B.reset(args.ref_B.data());
    params_.ref_D.reset(args.ref_D.data());
    params_.workspace = workspace;
    return Status::kSuccess;
  }
  Status updateA(TensorRefA a) { params_.ref_A.reset(a.data()); return Status::kSuccess; }
  Status updateC(TensorRefC) { return Status::kSuccess; }
  Status updateD(TensorRefD d) { params_.ref_D.reset(d.data()); return Status::kSuccess; }

  Status run(void* stream = nullptr) {
    cusync_gemm_args a = toArgs(params_.custage, params_.problem_size, params_.ref_A, params_.ref_B, params_.ref_D,
                                params_.split_k_slices, params_.workspace, params_.max_workgroups);
    return cusync_gemm_run(&a, stream) == CUSYNC_SUCCESS ? Status::kSuccess : Status::kErrorInternal;
  }
  // run(overlap, kernelExecuted, stream) of the reference (cusyncgemm.h:525-563): both flags select the same launch there.
  Status run(bool overlap, int* kernelExecuted, void* stream = nullptr) {
    (void)overlap; (void)kernelExecuted;
    return run(stream);
  }
  Status operator()(void* stream = nullptr) { return run(stream); }
  Status operator()(Arguments const& args, void* workspace = nullptr, void* stream = nullptr) {
    Status s = initialize(args, workspace, stream);
    return s == Status::kSuccess ? run(stream) : s;
  }

 private:
  static cusync_gemm_args toArgs(const CuStageImpl& stage, GemmCoord size, TensorRefA A, TensorRefB B, TensorRefD D, int split_k,
                                 void* workspace, int max_workgroups) {
    cusync_gemm_args a;
    a.stage = stage.desc();
    a.M = (uint32_t)size.m(); a.N = (uint32_t)size.n(); a.K = (uint32_t)size.k();
    a.A = A.data(); a.lda = (uint32_t)A.stride();
    a.B = B.data(); a.ldb = (uint32_t)B.stride();
    a.D = D.data(); a.ldd = (uint32_t)D.stride();
    a.epilogue = Epilogue;
    a.a_mode = CUSYNC_A_PLAIN;
    a.tile = TileId;
    a.split_k = split_k;
    a.workspace = workspace;
    a.max_workgroups = max_workgroups;
    // k-slices add their partial sums up among themselves where the library finds that safe for this launch
    // (cusync_gemm_args::shared_reduction); the reference's reduction is a kernel of its own, cusyncgemm.h:525-563
    a.shared_reduction = 1;
    return a;
  }
};

// cutlass::conv::Conv2dProblemSize for what the kernels do: NHWC input, KRSC filter, cross-correlation, one
// padding and one stride for both directions, no dilation, no groups.
struct Conv2dProblemSize {
  int N, H, W, C, K, R, S, pad, stride;
  int split_k_slices;      // runs the R*S*C/64 steps of a tile are cut into (src/ml-bench/volta_conv2d/resnet.cu:246, 689); 1 = none
  Conv2dProblemSize(int N_ = 0, int H_ = 0, int W_ = 0, int C_ = 0, int K_ = 0, int R_ = 3, int S_ = 3, int pad_ = 1, int stride_ = 1,
                    int split_k_slices_ = 1)
      : N(N_), H(H_), W(W_), C(C_), K(K_), R(R_), S(S_), pad(pad_), stride(stride_), split_k_slices(split_k_slices_) {}
  int P() const { return (H + 2 * pad - R) / stride + 1; }
  int Q() const { return (W + 2 * pad - S) / stride + 1; }
};

// CuSyncImplicitGemmConvolution<CuSyncImpl, kernel>: y = epilogue(conv(x, w)) as an implicit GEMM.
//   TileId    CUSYNC_CONV_TILE_*;  Epilogue  CUSYNC_EPILOGUE_* (the ResNet pair: RELU after the first layer)
template<typename CuStageImpl, int TileId, int Epilogue = CUSYNC_EPILOGUE_NONE>
class CuSyncImplicitGemmConvolution {
 public:
  struct Arguments {
    CuStageImpl custage;
    Conv2dProblemSize problem_size;
    TensorRef<const half_bits> ref_A;     // activations x[N][H][W][C]
    TensorRef<const half_bits> ref_B;     // filters w[K][R][S][C]
    TensorRef<const half_bits> ref_C;     // unused (beta = 0)
    TensorRef<half_bits> ref_D;           // output y[N][P][Q][K]
    LinearCombinationParams output_op;
    Arguments() {}
    Arguments(CuStageImpl& custage_, Conv2dProblemSize const& problem_size_, TensorRef<const half_bits> const& ref_A_,
              TensorRef<const half_bits> const& ref_B_, TensorRef<const half_bits> const& ref_C_, TensorRef<half_bits> const& ref_D_,
              LinearCombinationParams const& output_op_ = LinearCombinationParams())
        : custage(custage_), problem_size(problem_size_), ref_A(ref_A_), ref_B(ref_B_), ref_C(ref_C_), ref_D(ref_D_), output_op(output_op_) {}
  };
  struct Params {
    CuStageImpl custage;
    Conv2dProblemSize problem_size;
    const half_bits* x;
    const half_bits* w;
    half_bits* y;
    int max_workgroups;
    void* workspace;
    Params() : x(nullptr), w(nullptr), y(nullptr), max_workgroups(0), workspace(nullptr) {}
  };
  Params params_;

  static dim3 get_grid_shape(Conv2dProblemSize const& p) {
    const cusync_dim3 g = cusync_conv2d_grid_split(TileId, (uint32_t)p.N, (uint32_t)p.H, (uint32_t)p.W, (uint32_t)p.K, (uint32_t)p.R, (uint32_t)p.S,
                                                  (uint32_t)p.pad, (uint32_t)p.stride, p.split_k_slices);
    return dim3(g.x, g.y, g.z);
  }
  static Status can_implement(Arguments const& args) {
    if (args.output_op.alpha != 1.0f || args.output_op.beta != 0.0f) return Status::kErrorNotSupported;
    // the workspace arrives with initialize(): any aligned address stands in for it here
    cusync_conv2d_args a = toArgs(args.custage, args.problem_size, args.ref_A.data(), args.ref_B.data(), args.ref_D.data(), 0,
                                  args.problem_size.split_k_slices > 1 ? (void*)args.ref_D.data() : nullptr);
    return cusync_conv2d_can_implement(&a) == CUSYNC_SUCCESS ? Status::kSuccess : Status::kErrorInvalidProblem;
  }
  // Bytes initialize() wants for the runs' partial sums and counters (0 without runs).  The caller zeroes the
  // buffer once; the kernels leave the counters at zero.
  static size_t get_workspace_size(Arguments const& args) {
    cusync_conv2d_args a = toArgs(args.custage, args.problem_size, nullptr, nullptr, nullptr, 0, nullptr);
    return cusync_conv2d_workspace_size(&a);
  }
  Status initialize(Arguments const& args, void* workspace = nullptr, void* stream = nullptr) {
    (void)stream;
    const Status s = can_implement(args);
    if (s != Status::kSuccess) return s;
    if (args.problem_size.split_k_slices > 1 && !workspace) return Status::kErrorWorkspaceNull;
    params_.workspace = workspace;
    params_.custage = args.custage;
    params_.problem_size = args.problem_size;
    params_.x = args.ref_A.data(); params_.w = args.ref_B.data(); params_.y = args.ref_D.data();
    return Status::kSuccess;
  }
  Status run(void* stream = nullptr) {
    cusync_conv2d_args a = toArgs(params_.custage, params_.problem_size, params_.x, params_.w, params_.y, params_.max_workgroups,
                                  params_.workspace);
    return cusync_conv2d_run(&a, stream) == CUSYNC_SUCCESS ? Status::kSuccess : Status::kErrorInternal;
  }
  Status run(bool overlap, int* kernelExecuted, void* stream = nullptr) { (void)overlap; (void)kernelExecuted; return run(stream); }
  Status operator()(void* stream = nullptr) { return run(stream); }

 private:
  static cusync_conv2d_args toArgs(const CuStageImpl& stage, Conv2dProblemSize const& p, const half_bits* x, const half_bits* w,
                                   half_bits* y, int max_workgroups, void* workspace) {
    cusync_conv2d_args a;
    a.stage = stage.desc();
    a.N = (uint32_t)p.N; a.H = (uint32_t)p.H; a.W = (uint32_t)p.W; a.C = (uint32_t)p.C;
    a.K = (uint32_t)p.K; a.R = (uint32_t)p.R; a.S = (uint32_t)p.S; a.pad = (uint32_t)p.pad; a.stride = (uint32_t)p.stride;
    a.x = x; a.w = w; a.y = y;
    a.epilogue = Epilogue;
    a.tile = TileId;
    a.max_workgroups = max_workgroups;
    a.split_k = p.split_k_slices;
    a.workspace = workspace;
    return a;
  }
};

}  // namespace cusync
