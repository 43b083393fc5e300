/*
 * cusync_amd.h — C ABI of the MI355X-native CuSync library (libcusync_amd.so).
 *
 * Plain C types only: pointers, sizes and PODs.  Everything above this line of
 * the stack (the C++ CuStage API in include/cusync/, the drivers, the Python
 * test harness) reaches the GPU exclusively through these entry points.
 *
 * Each entry point names the interface of the reference (microsoft/cusync) it
 * stands in for.  Reference paths:
 *   CS = src/include/cusync
 *   CC = src/include/cutlass/cusync-cutlass/include/cutlass
 *   TB = src/ml-bench/transformer     CV = src/ml-bench/volta_conv2d
 */
#ifndef CUSYNC_AMD_H
#define CUSYNC_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------- */
/* PODs                                                                       */
/* ------------------------------------------------------------------------- */

typedef struct cusync_dim3 { uint32_t x, y, z; } cusync_dim3;

/* CS/cusync.h:46-53 — same enumerators in the same order; success is 5. */
typedef enum cusync_error {
  CUSYNC_ERROR_NOT_PRODUCER = 0,
  CUSYNC_ERROR_NOT_CONSUMER = 1,
  CUSYNC_ERROR_NOT_INITIALIZED = 2,
  CUSYNC_ERROR_INVALID_LINEAR_BLOCK_INDEX = 3,
  CUSYNC_ERROR_DEVICE = 4,            /* CuSyncErrorCUDAError */
  CUSYNC_SUCCESS = 5
} cusync_error;

/* CS/cusync.h:69-75 */
enum {
  CUSYNC_OPT_NONE = 0,
  CUSYNC_OPT_NO_ATOMIC_ADD = 1 << 0,
  CUSYNC_OPT_AVOID_WAIT_KERNEL = 1 << 1,
  CUSYNC_OPT_AVOID_CUSTOM_ORDER = 1 << 2,
  CUSYNC_OPT_REORDER_TILE_LOADS = 1 << 3
};

/* CS/tile-orders.h:50-76 */
enum { CUSYNC_ORDER_IDENTITY = 0, CUSYNC_ORDER_TRANSPOSE_XY = 1 };

/* CS/policies.h:18-210; StridedSync TB/mlp.cu:76-101; ConsecutiveSync TB/attention.cu:51-70 */
enum {
  CUSYNC_POLICY_NOSYNC = 0,
  CUSYNC_POLICY_ROWSYNC = 1,
  CUSYNC_POLICY_TILESYNC = 2,
  CUSYNC_POLICY_STRIDEDSYNC = 3,
  CUSYNC_POLICY_CONV2DTILESYNC = 4,
  CUSYNC_POLICY_CONSECUTIVESYNC = 5
};

/* Run-time image of a policy type: its template arguments and its two members. */
typedef struct cusync_policy_desc {
  int32_t kind;
  int32_t order;
  uint32_t tileM, tileN;
  uint32_t waitValue, postValue;
  uint32_t gridN, stride;     /* StridedSync<Order, GridN, TileM, TileN, stride> */
  uint32_t R, S;              /* Conv2DTileSync<Order, R, S, TileM, TileN> */
  uint32_t H;                 /* ConsecutiveSync<Order, H, TileM, TileN> */
} cusync_policy_desc;

/* Run-time image of a CuStage object (CS/cusync.h:93-117): what a kernel gets
 * by value.  Device pointers are owned by whoever called cusync_stage_alloc. */
/* tileOrder[i] == (i % gx, (i / gx) % gy, i / (gx*gy)) for every i: true of both tile orders the reference
 * ships (CS/tile-orders.h:52-75).  The prebuilt kernels then compute a ticket's tile instead of loading it. */
enum { CUSYNC_STAGE_IDENTITY_ORDER = 1 };

/* Semaphore i of a stage lives at tileStatus[i * CUSYNC_SEM_STRIDE]: each on its own 128-byte line, so that the
 * waves polling one semaphore do not queue up behind those polling its neighbours (the reference packs them,
 * CS/cusync.h:186-190).  cusync_stage_read_state returns them packed. */
#define CUSYNC_SEM_STRIDE 32
#define CUSYNC_HOST_FLAG_OFFSET 32

typedef struct cusync_stage_desc {
  cusync_dim3 grid;           /* grid_     : logical tile grid of this stage */
  cusync_dim3 prodGrid;       /* prodGrid_ : logical tile grid of its producer */
  cusync_dim3 tileSize;       /* tileSize_ : stored, never read (as in the reference) */
  int32_t iter;               /* run counter, starts at 1 */
  int32_t opts;               /* CUSYNC_OPT_* bits */
  uint32_t flags;             /* CUSYNC_STAGE_* bits, filled in by cusync_stage_alloc */
  uint32_t reserved;
  cusync_policy_desc in;      /* inputPolicy_  */
  cusync_policy_desc out;     /* outputPolicy_ */
  cusync_dim3 *tileOrder;     /* [numTiles] ticket -> tile */
  uint32_t *tileCounter;      /* ticket dispenser; 0 between runs */
  uint32_t *startCounter;     /* counts workgroups that have begun; 0 between runs */
  uint32_t *xcdTickets;       /* 9 counters, 128 bytes apart: one ticket dispenser per XCD for the prebuilt
                                 kernels plus a count of workgroups that ran dry; all 0 between runs */
  uint32_t *kernelExecuted;   /* wait-kernel flag: == iter once every workgroup of the run has begun */
  uint32_t *spinTimeouts;     /* number of waits of this stage that gave up, 0 in a healthy chain.  Pinned host memory
                                 that the device writes to, so that the host reads it without a copy; the word
                                 CUSYNC_HOST_FLAG_OFFSET words behind it mirrors the wait-kernel flag for
                                 cusync_wait_producer_started (written right after the flag itself), and the word after
                                 that is the launchers' note for cusync_hold_back (host-written only) */
  uint32_t *tileStatusWrite;  /* semaphores this stage posts, CUSYNC_SEM_STRIDE apart */
  uint32_t *tileStatusRead;   /* semaphores this stage waits on (its producer's) */
} cusync_stage_desc;

/* ------------------------------------------------------------------------- */
/* Thin runtime layer (replaces the cudaMalloc/Memset/Memcpy/stream/event     */
/* calls made directly by CS/cusync.h:125-198 and the drivers)                */
/* ------------------------------------------------------------------------- */

const char *cusync_rt_last_error(void);            /* text of the last failed HIP call, "" if none */
/* Diagnosis, off by default.  With a device buffer set (8-byte aligned, zeroed by the caller) the direct-to-LDS GEMM
 * kernels, the 3x3 convolution kernel with the input tile in LDS and the attention kernel append one record of eight 64-bit words per finished tile behind a record count in word 0: role and
 * workgroup and XCD, tile, and the 100 MHz clock at five points of the tile (drawn, first loads issued, main loop
 * done, posted, kernel entry).  This is how the per-workgroup timelines in profiles/ were taken.  NULL switches it
 * off again; when off the kernels pay one test per tile.  No counterpart in the reference. */
cusync_error cusync_rt_set_timeline(void *device_buffer, size_t bytes);
int cusync_rt_device_count(void);
int cusync_rt_device_info(int *num_cus, int *clock_khz, size_t *lds_per_cu, size_t *hbm_bytes,
                          char *name, size_t name_len);
int cusync_rt_malloc(void **ptr, size_t bytes);     /* 0 on success */
int cusync_rt_free(void *ptr);
int cusync_rt_memset(void *ptr, int value, size_t bytes);
int cusync_rt_memcpy_h2d(void *dst, const void *src, size_t bytes);
int cusync_rt_memcpy_d2h(void *dst, const void *src, size_t bytes);
int cusync_rt_memcpy_d2d(void *dst, const void *src, size_t bytes);
int cusync_rt_stream_create(void **stream);         /* non-blocking stream, default priority */
int cusync_rt_stream_destroy(void *stream);
int cusync_rt_stream_sync(void *stream);
int cusync_rt_device_sync(void);
int cusync_rt_event_create(void **event);
int cusync_rt_event_destroy(void *event);
int cusync_rt_event_record(void *event, void *stream);
int cusync_rt_event_sync(void *event);
int cusync_rt_event_elapsed_us(void *start, void *end, double *us);
int cusync_rt_stream_wait_event(void *stream, void *event);

/* ------------------------------------------------------------------------- */
/* Stage life cycle                                                           */
/* ------------------------------------------------------------------------- */

/* Replaces the device half of the CuStage constructor (CS/cusync.h:176-198) and
 * buildScheduleBuffer (:125-157): uploads host_tile_order[numTiles], zeroes the
 * ticket and start counters, and for a producer allocates numTiles zeroed
 * semaphores plus the wait-kernel flag (skipped with AVOID_WAIT_KERNEL).
 * desc->grid/opts/in/out must be filled in; pointer members are written. */
cusync_error cusync_stage_alloc(cusync_stage_desc *desc, const cusync_dim3 *host_tile_order);
/* The reference never frees (no destructor); this does.  Only call on the
 * descriptor that was passed to cusync_stage_alloc, not on copies. */
cusync_error cusync_stage_free(cusync_stage_desc *desc);
/* Environment: CUSYNC_FORCE_ACQUIRE=1 makes every consumer wait of the prebuilt kernels end with the agent-scope
 * acquire (which drops this XCD's cached lines), also where the launcher would skip it because the producer's
 * tiles are whole 128-byte lines of the consumer's operand.  A switch for diagnosis; results do not change. */
/* Same result as cusync_stage_alloc with the tile order generated from
 * desc->grid for one of the two built-in orders. */
cusync_error cusync_stage_create(cusync_stage_desc *desc, int order);
/* CuSync::setProducerConsumerPair (CS/cusync.h:289-298). */
cusync_error cusync_set_producer_consumer_pair(const cusync_stage_desc *prod, cusync_stage_desc *cons);
/* CuStage::invokeWaitKernel (CS/cusync.h:203-209) + src/cusync.cu:11-25:
 * enqueues a one-wave kernel on `stream` that returns once the producer's flag
 * has reached desc->iter.  No-op with AVOID_WAIT_KERNEL. */
cusync_error cusync_invoke_wait_kernel(const cusync_stage_desc *prod, void *stream);
/* Same, but `stream` first waits for `launch_event` (a hipEvent_t the caller recorded on the producer's stream
 * immediately before launching the producer's kernel; NULL = no ordering, i.e. cusync_invoke_wait_kernel).  The two
 * streams are separate hardware queues and the wait kernel's wave can reach the GPU before the producer's
 * workgroups do; behind the event it is dispatched after the producer's launch has begun.  No counterpart in the
 * reference, which launches the wait kernel unordered (src/ml-bench/transformer/mlp.cu:683-699). */
cusync_error cusync_invoke_wait_kernel_after(const cusync_stage_desc *prod, void *stream, void *launch_event);
/* The same hold-back done by the calling host thread instead of a kernel: returns once every workgroup of the
 * producer's run prod->iter has started (the mirror of its flag in host memory, which the device writes to, has
 * reached prod->iter), or CUSYNC_ERROR_DEVICE after timeout_ms (0 = two seconds).  The caller then launches the consumer.
 * Why: a wait kernel is a wave that holds registers on one CU until the flag rises (hipStreamWaitValue32 is such a
 * kernel too on this runtime).  A producer whose workgroups need whole CUs and whose launch fills every CU cannot
 * place its last workgroup on that CU; the flag is then not raised until another workgroup retires and the chain
 * is one producer tile longer (measured on the 2048-row GPT-3 MLP: 720-790 us against 610 in one run out of ten;
 * per-workgroup timestamps show workgroup 249 of 256 entering at 313 us).  The host holds no CU.  The chain
 * handles of this library use it for exactly those producers and the wait kernel for all others (with
 * CUSYNC_WAIT_KERNEL=1 in the environment they use the wait kernel everywhere, for comparison).  No counterpart
 * in the reference. */
cusync_error cusync_wait_producer_started(const cusync_stage_desc *prod, uint32_t timeout_ms);
/* CuStage::invokeWaitKernel as the library's own chains do it (CS/cusync.h:203-209): holds `stream` back until every
 * workgroup of the producer's run prod->iter has started, by whichever of the two ways above suits the producer's last
 * launch.  cusync_gemm_run, cusync_conv2d_run and cusync_attention_run leave a note in the stage's host memory saying
 * whether the launch they just made took every workgroup slot of the device (cusync_gemm_fills_device); for such a
 * launch the calling thread waits (cusync_wait_producer_started) and, should that time out (the producer is queued
 * behind other work), the wait kernel is enqueued after all; for any other launch, for a stream under capture, or with
 * CUSYNC_WAIT_KERNEL=1 in the environment, the wait kernel is enqueued at once.  Call it after the producer's launch
 * call has returned and before the consumer's, as the reference's loop does (src/ml-bench/transformer/mlp.cu:691-699). */
cusync_error cusync_hold_back(const cusync_stage_desc *prod, void *stream);
/* cusync::invokeWaitKernel(sem, value, stream) (CS/wait-kernel.h:10). */
cusync_error cusync_wait_kernel(uint32_t *semaphore, uint32_t value, void *stream);
/* Reads back device state for tests (the reference reaches it through the
 * friend class CuSyncTest, CS/cusync.h:120, tests/cusync-test.h). Any output
 * pointer may be NULL. sems must hold numTiles entries. */
cusync_error cusync_stage_read_state(const cusync_stage_desc *desc, uint32_t *sems, cusync_dim3 *tile_order,
                                     uint32_t *tile_counter, uint32_t *start_counter,
                                     uint32_t *kernel_executed, uint32_t *spin_timeouts);

/* Host evaluation of a policy / tile order, same arithmetic the device uses. */
uint32_t cusync_policy_tile_index(const cusync_policy_desc *p, cusync_dim3 tile, cusync_dim3 grid);
uint32_t cusync_policy_wait_value(const cusync_policy_desc *p, cusync_dim3 tile, cusync_dim3 grid);
uint32_t cusync_policy_post_value(const cusync_policy_desc *p, cusync_dim3 tile, cusync_dim3 grid);
int      cusync_policy_is_sync(const cusync_policy_desc *p, cusync_dim3 tile, cusync_dim3 grid);
uint32_t cusync_order_block_index(int order, cusync_dim3 grid, cusync_dim3 block);
cusync_dim3 cusync_order_tile_to_block(int order, cusync_dim3 tile);

/* ------------------------------------------------------------------------- */
/* Sync-aware fp16 GEMM (replaces cutlass::gemm::device::CuSyncGemm,          */
/* CC/gemm/device/cusyncgemm.h:169-599 and its kernel CC/gemm/kernel/         */
/* cusyncgemm.h:208-399)                                                      */
/* ------------------------------------------------------------------------- */

enum {
  CUSYNC_EPILOGUE_NONE = 0, CUSYNC_EPILOGUE_GELU = 1, CUSYNC_EPILOGUE_RELU = 2,
  /* D[m, 8q + t] = silu(P[m, 16q + t]) * P[m, 16q + 8 + t], P = A*B, t = 0..7: B holds the gate and the up
   * projection of a SwiGLU feed-forward with their columns interleaved in groups of eight (gate columns 8q..8q+7,
   * then up columns 8q..8q+7), so that a workgroup has both factors of an output element in its own registers and
   * the activation costs no pass of its own (LinearCombinationSilu + LinearCombinationSwiGLU of the reference's
   * library build, TB/mlp-lib.cu:122-133, in one epilogue).  D has N/2 columns; N % 16 == 0.  The tile is posted
   * under the output's coordinates {row, n0 / 2}: a consumer's policy counts columns of D. */
  CUSYNC_EPILOGUE_SWIGLU = 3
};
/* How the A operand is formed while it is staged into LDS. */
enum {
  CUSYNC_A_PLAIN = 0,
  CUSYNC_A_SWIGLU = 1          /* A[m,k] = silu(G[m,k]) * G[m,k + K]; G has K*2 valid columns */
};

/* Tile shapes the library was built with.  The ...x32 shapes move their operands from
 * global memory straight into LDS and have no SwiGLU variant; the others stage them
 * through registers.  256x256x32 and 256x192x32 run eight wavefronts per workgroup and
 * one workgroup per CU (such a producer and its consumer cannot share a CU, so a chain
 * on them overlaps nothing); all others run four wavefronts. */
enum {
  CUSYNC_TILE_256x256x32 = 0,
  CUSYNC_TILE_256x128x64 = 1,
  CUSYNC_TILE_128x128x64 = 2,
  CUSYNC_TILE_64x128x64 = 3,
  CUSYNC_TILE_32x128x64 = 4,
  CUSYNC_TILE_128x256x64 = 5,
  CUSYNC_TILE_256x64x64 = 6,
  CUSYNC_TILE_128x64x64 = 7,
  CUSYNC_TILE_256x128x32 = 8,
  CUSYNC_TILE_128x256x32 = 9,
  CUSYNC_TILE_128x128x32 = 10,
  CUSYNC_TILE_128x192x32 = 11,       /* direct-to-LDS; 6144 = 32 x 192, 12288 = 64 x 192: whole waves on 256 CUs */
  CUSYNC_TILE_256x192x32 = 12,
  CUSYNC_TILE_D32x128x64 = 13,       /* direct-to-LDS, 4 stages: few rows, bound by streaming the weights */
  CUSYNC_TILE_D64x128x64 = 14,       /* direct-to-LDS, 3 stages */
  CUSYNC_TILE_D64x192x64 = 15,       /* direct-to-LDS, 4 stages, a CU to itself: 32 or 64 column tiles times 8 or 4 k-slices are 256 */
  CUSYNC_TILE_128x192x32_ALONE = 16, /* 128x192x32 with 4 stages in the pipelined order and a CU to itself: for GEMMs of about one tile per CU */
  CUSYNC_TILE_256x384x32 = 17,       /* direct-to-LDS, eight wavefronts of 128x96 in two alternating groups, 3 stages, a CU to itself:
                                        a third less data moved per MFMA than 256x192; 12288 columns are 32 tiles.  K must be a
                                        multiple of 32; a stage of a tile policy waits for all its producer tiles before its first load */
  CUSYNC_TILE_256x192x64 = 18,       /* 256x192 with both operands fetched 64 columns of K at a time, in whole cache lines (A ring of three
                                        slots, B ring of four 32-row stages, one barrier per 32 columns), K loop in assembly.  K (and every k-slice) a
                                        multiple of 64; a stage of a tile policy waits for all its producer tiles before its first load */
  CUSYNC_TILE_D128x192x64 = 19,      /* 128x192 with both operands fetched 64 columns of K at a time: A in whole cache lines, three
                                        stages of 40 KB, a CU to itself: for 256 rows and thereabouts, where the loop waits on the
                                        number of requests a CU's memory path holds and 64-byte pieces of A rows take as many as lines */
  CUSYNC_TILE_COUNT = 20
};

typedef struct cusync_gemm_args {
  cusync_stage_desc stage;     /* Arguments::custage (cusyncgemm.h:293-350) */
  uint32_t M, N, K;            /* problem_size */
  const void *A; uint32_t lda; /* fp16 row-major [M,K] (or [M,2K] gate|up for CUSYNC_A_SWIGLU) */
  const void *B; uint32_t ldb; /* fp16 row-major [K,N] */
  void *D; uint32_t ldd;       /* fp16 row-major [M,N] ([M,N/2] with CUSYNC_EPILOGUE_SWIGLU); D = epilogue(A*B), alpha = 1, beta = 0 */
  int32_t epilogue;            /* CUSYNC_EPILOGUE_* */
  int32_t a_mode;              /* CUSYNC_A_* */
  int32_t tile;                /* CUSYNC_TILE_* */
  int32_t split_k;             /* k-slices (grid z); > 1 adds the slices' fp32 partial sums through `workspace`.  Every slice takes
                                  ceil(chunks / split_k) K chunks of the tile's depth, and a count that leaves the last slice without
                                  a chunk is refused by cusync_gemm_can_implement (44 chunks in 16 slices) */
  void *workspace;             /* split_k > 1: cusync_gemm_workspace_size bytes, zeroed once by the caller */
  int32_t max_workgroups;      /* 0 = as many as stay resident; else cap on launched workgroups */
  int32_t shared_reduction;    /* split_k > 1.  0: the k-slice of a tile that finishes last adds up all slices and stores
                                  the tile.  1: where every k-slice of the launch has a workgroup of its own from the start
                                  (no more tiles than workgroups stay resident), tileM is at least 128 and tileM/32 is a multiple of split_k, the
                                  slices of a tile wait for each other and each adds up and stores a share; same sums in
                                  the same order, so bit-identical results.  The waiting slices hold their CUs: only for
                                  launches whose workgroups no other kernel keeps off the device while it waits for them
                                  (the chains of this library launch a consumer only after its producer is resident).
                                  Ignored (the last-arriver form runs) for a stage with CUSYNC_OPT_AVOID_WAIT_KERNEL: without
                                  the hold-back a consumer's launch may reach the device first and keep sibling slices off it.
                                  No counterpart in the reference, whose split-K reduction is a kernel of its own
                                  (cusyncgemm.h:525-563). */
} cusync_gemm_args;

/* Tile extents of a CUSYNC_TILE_* id; returns 0 on success. */
int cusync_gemm_tile_shape(int tile, uint32_t *tileM, uint32_t *tileN, uint32_t *tileK);
/* Logical grid (n-tiles, m-tiles, k-slices): CuSyncGemmHorizontalThreadblockSwizzle
 * get_tiled_shape + get_grid_shape (CC/gemm/threadblock/cusync_threadblock_swizzle.h:12-54). */
cusync_dim3 cusync_gemm_grid(int tile, uint32_t M, uint32_t N, int split_k);
/* can_implement (cusyncgemm.h:364-386): CUSYNC_SUCCESS or CUSYNC_ERROR_NOT_INITIALIZED
 * with the reason in cusync_rt_last_error(). */
cusync_error cusync_gemm_can_implement(const cusync_gemm_args *args);
/* get_workspace_size (cusyncgemm.h:388-404). */
size_t cusync_gemm_workspace_size(const cusync_gemm_args *args);
/* Workgroups of this tile shape that stay resident on the device at once. */
int cusync_gemm_max_resident(int tile);
/* 1 when the launch of these arguments takes every workgroup slot the device has for its kernel (as many
 * workgroups as stay resident).  A single wave of another kernel that gets onto a CU first, a wait kernel for
 * instance, then keeps one of the workgroups off the device until another retires; the chains hold such a
 * producer's consumer back from the host instead (cusync_wait_producer_started).  No counterpart in the reference. */
int cusync_gemm_fills_device(const cusync_gemm_args *args);
/* run(stream) (cusyncgemm.h:525-563).  args->stage.iter selects the run. */
cusync_error cusync_gemm_run(const cusync_gemm_args *args, void *stream);
/* cusync_gemm_run for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference, whose split-K workspace always comes
 * from the caller (cusyncgemm.h:388-404, 407-456).  args->workspace is ignored: with split_k > 1 the k-slices'
 * partial sums and arrival counters live in an array the library holds in device memory
 * (CUSYNC_GEMM_STATIC_WORKSPACE_BYTES on every device it runs on, until the process ends); problems whose
 * cusync_gemm_workspace_size exceeds that are refused with CUSYNC_ERROR_NOT_INITIALIZED and a text in
 * cusync_rt_last_error().  The call allocates and frees nothing; it clears the arrival counters it is going to use
 * with a small fill kernel on `stream` (no memset) and launches the same kernel as cusync_gemm_run, so results are
 * bit-identical.  All calls on one device share the one array: two calls with split_k > 1 that overlap in time on
 * a device (different streams, or a graph replayed while another runs) race and give wrong results. */
#define CUSYNC_GEMM_STATIC_WORKSPACE_BYTES (32u << 20)
cusync_error cusync_gemm_run_static_workspace(const cusync_gemm_args *args, void *stream);
/* `count` (1..4) dependent GEMMs of one direct-to-LDS tile shape in ONE launch: every workgroup works through the
 * tiles of args[0] it can draw, then those of args[1], ...; a tile of args[i] waits on the semaphores args[i-1]
 * posts, exactly as in separate launches (the stages are created and paired the same way), but no kernel boundary,
 * wait kernel or second launch sits in between.  No counterpart in the reference, whose consumer is always a launch
 * of its own; here a first dispatch on another stream starts 15-20 us after the producer did, which chains of
 * short kernels cannot afford.  args[0] must not wait on a stage outside the launch. */
cusync_error cusync_gemm_chain_run(const cusync_gemm_args *args, int count, void *stream);

/* ------------------------------------------------------------------------- */
/* Sync-aware NHWC forward convolution as an implicit GEMM (replaces           */
/* cutlass::conv::device::CuSyncImplicitGemmConvolution,                       */
/* CC/conv/device/cusyncimplicit_gemm_convolution.h:226-298, and its kernel    */
/* CC/conv/kernel/implicit_cusyncgemm_convolution.h:287-477)                   */
/* ------------------------------------------------------------------------- */

enum {
  CUSYNC_CONV_TILE_128x64x32 = 0,    /* M x K_out x K chunk */
  CUSYNC_CONV_TILE_128x128x32 = 1,
  CUSYNC_CONV_TILE_256x64x32 = 2,
  CUSYNC_CONV_TILE_HALO_256x64x64 = 3,   /* 3x3, pad 1, stride 1, C a power of two >= 64: the input tile and its halo
                                            stay in LDS, each pixel is fetched once instead of once per filter tap */
  CUSYNC_CONV_TILE_HALO_128x128x64 = 4,
  CUSYNC_CONV_TILE_HALO_64x128x64 = 5,   /* the halo tile that still fits with 512 channels (7 x 7 images) */
  CUSYNC_CONV_TILE_COUNT = 6
};

typedef struct cusync_conv2d_args {
  cusync_stage_desc stage;     /* Arguments::custage; grid = cusync_conv2d_grid(...) */
  uint32_t N, H, W, C;         /* input  x[N,H,W,C]  fp16 NHWC */
  uint32_t K, R, S;            /* filter w[K,R,S,C]  fp16 KRSC, cross-correlation (CV/resnet.cu:678) */
  uint32_t pad, stride;        /* same in both directions; output y[N,P,Q,K], P = (H+2*pad-R)/stride+1 */
  const void *x;
  const void *w;
  void *y;
  int32_t epilogue;            /* CUSYNC_EPILOGUE_* (the ResNet pair uses RELU after the first convolution) */
  int32_t tile;                /* CUSYNC_CONV_TILE_* */
  int32_t max_workgroups;      /* 0 = as many as stay resident */
  int32_t split_k;             /* Conv2dProblemSize::split_k_slices (CV/resnet.cu:246, 689, 765): 0 or 1 = none; n (halo tiles):
                                  the R*S*C/64 steps of a tile in n runs, grid z = n, partial sums added in run order */
  void *workspace;             /* split_k > 1: cusync_conv2d_workspace_size bytes, 16-byte aligned; its counters (the last
                                  2 * tiles words) zero before the first run, the kernel leaves them zero */
} cusync_conv2d_args;

int cusync_conv2d_tile_shape(int tile, uint32_t *tileM, uint32_t *tileN, uint32_t *tileK);
/* Logical grid (K_out tiles, N*P*Q tiles, 1): the implicit-GEMM form of get_tiled_shape
 * (CC/gemm/threadblock/cusync_threadblock_swizzle.h:34-44). */
cusync_dim3 cusync_conv2d_grid(int tile, uint32_t N, uint32_t H, uint32_t W, uint32_t K, uint32_t R, uint32_t S,
                               uint32_t pad, uint32_t stride);
/* The same with the tile's steps cut into split_k runs: (K_out tiles, N*P*Q tiles, split_k), as get_tiled_shape with
 * split_k_slices gives it (CV/resnet.cu:765). */
cusync_dim3 cusync_conv2d_grid_split(int tile, uint32_t N, uint32_t H, uint32_t W, uint32_t K, uint32_t R, uint32_t S,
                                     uint32_t pad, uint32_t stride, int split_k);
/* get_workspace_size (cusyncimplicit_gemm_convolution.h): 0 without runs. */
size_t cusync_conv2d_workspace_size(const cusync_conv2d_args *args);
cusync_error cusync_conv2d_can_implement(const cusync_conv2d_args *args);
int cusync_conv2d_max_resident(int tile);
/* operator()(stream) (cusyncimplicit_gemm_convolution.h:283-298).  A consumer stage waits, per producer
 * channel tile, for every producer row block reached by the filter window of its rows. */
cusync_error cusync_conv2d_run(const cusync_conv2d_args *args, void *stream);

/* Chain of `layers` 3x3, pad 1, stride 1 convolutions with C input and C output channels each:
 * two layers are the ResNet block of CV/resnet.cu:560-830 (producer + consumer), four are the VGG
 * block of CV/vgg.cu, whose middle layers are consumer and producer at once. */
typedef struct cusync_conv_chain_config {
  uint32_t N, H, W, C;
  uint32_t layers;             /* 1..16 */
  int32_t sync;                /* CUSYNC_SYNC_STREAM, _ROW (RowSync both sides) or _TILE (TileSync -> Conv2DTileSync) */
  int32_t tile;                /* CUSYNC_CONV_TILE_*, -1 = built-in choice */
  int32_t opts;                /* extra CUSYNC_OPT_* bits, -1 = none */
  int32_t relu;                /* 1: ReLU after every layer but the last */
  int32_t fused;               /* 1 (sync ROW or TILE, halo tiles, at most 8 layers): all layers in ONE launch whose workgroups
                                  work through layer 0, then layer 1, ... with the same semaphores between them; no wait
                                  kernel and no second launch between a producer and its consumer */
  int32_t split_k;             /* --split_k_slices (CV/resnet.cu:329): runs a tile's steps are cut into; 1 = none; 0 = the
                                  library picks (runs only for layers whose tiles leave more than half the CUs idle) */
} cusync_conv_chain_config;

typedef struct cusync_conv_chain cusync_conv_chain;

/* weights[i]: filter of layer i, [C][3][3][C] fp16 device pointer. */
cusync_conv_chain *cusync_conv_chain_create(const cusync_conv_chain_config *cfg, const void *const *weights);
void cusync_conv_chain_destroy(cusync_conv_chain *chain);
/* x: [N][H][W][C]; ys[i]: output of layer i, same shape.  Synchronises after each of the `runs` runs;
 * times_us[r] = start of the first kernel to end of the last; in the stream-ordered mode
 * layer_us[r*layers + i] receives the time of layer i. */
cusync_error cusync_conv_chain_run(cusync_conv_chain *chain, const void *x, void *const *ys, int runs,
                                   double *times_us, double *layer_us);
const cusync_stage_desc *cusync_conv_chain_stage(const cusync_conv_chain *chain, uint32_t which);
int cusync_conv_chain_tile(const cusync_conv_chain *chain);
int cusync_conv_chain_split(const cusync_conv_chain *chain);      /* runs per tile the chain runs with */

/* ------------------------------------------------------------------------- */
/* Fused multi-head attention stage: O = softmax(mask(Q K^T * scale)) V per    */
/* head, fp16 in/out, fp32 accumulate.  Takes the place of the two inner GEMM  */
/* stages S = Q K^T and O = P V of the reference's attention chain (gemm_op2 / */
/* gemm_op3 with SCuStage / OCuStage, TB/attention.cu:101-104, 797-803): it is */
/* a consumer of the QKV projection and a producer for the output projection.  */
/* ------------------------------------------------------------------------- */

typedef struct cusync_attention_args {
  cusync_stage_desc stage;     /* grid = cusync_attention_grid(seq, heads) */
  uint32_t seq, heads, head_dim;   /* seq query rows; head_dim must be 128 */
  uint32_t cached_rows;        /* rows of qkv in front of the query rows: the key/value cache of TB/attention.cu:272-276
                                  (query i sits at row cached_rows + i and sees keys 0 .. cached_rows + i); 0 = none */
  const void *qkv;             /* [cached_rows + seq][ldqkv] fp16: Q at column 0, K at heads*head_dim, V at 2*heads*head_dim */
  uint32_t ldqkv;
  void *out;                   /* [seq][ldo] fp16, head h in columns h*head_dim .. */
  uint32_t ldo;
  float scale;                 /* softmax scale; 0 selects 1/sqrt(head_dim) */
  int32_t causal;              /* 1: query i sees keys 0..i */
  int32_t max_workgroups;      /* 0 = as many as stay resident */
  uint32_t kv_split_blocks;    /* 0: one workgroup walks all keys of its rows; n: at most n key/value blocks (of 64 rows) per
                                  workgroup, grid = cusync_attention_grid_split, partial results combined through `workspace` */
  void *workspace;             /* kv_split_blocks > 0: cusync_attention_workspace_size bytes, zeroed once by the caller */
} cusync_attention_args;

/* Rows per output tile (128), columns per output tile (= head_dim) and key/value rows per inner step. */
int cusync_attention_tile_shape(uint32_t *tileM, uint32_t *tileN, uint32_t *blockKV);
/* Logical grid (heads, row tiles, 1); an output tile is posted as {row, head*head_dim, 0}. */
cusync_dim3 cusync_attention_grid(uint32_t seq, uint32_t heads);
/* Grid with the key range split: (heads, row tiles, splits of the longest row tile).  Row tiles that see fewer keys
 * (causal) leave their surplus splits empty; a tile is posted once, by the split that completes it. */
cusync_dim3 cusync_attention_grid_split(uint32_t seq, uint32_t heads, uint32_t cached_rows, uint32_t kv_split_blocks);
size_t cusync_attention_workspace_size(const cusync_attention_args *args);
cusync_error cusync_attention_can_implement(const cusync_attention_args *args);
int cusync_attention_max_resident(void);
/* As a consumer (input policy RowSync, TileSync or ConsecutiveSync over the QKV projection's tiles) the
 * kernel waits for the producer tiles holding its Q rows, and for those of each K / V block right
 * before loading it; as a producer it posts each finished output tile. */
cusync_error cusync_attention_run(const cusync_attention_args *args, void *stream);

/* Self-attention chain X Wqkv -> attention -> O Wo (TB/attention.cu:560-830 runBaseline / runCuSync). */
typedef struct cusync_attn_layer_config {
  uint32_t seq;                /* rows of X */
  uint32_t hidden;             /* columns of X and of Y (12288 for the GPT-3 shard) */
  uint32_t heads, head_dim;    /* 12 x 128 per GPU */
  int32_t sync;                /* CUSYNC_SYNC_*; STRIDED = ConsecutiveSync into the attention, RowSync out of it */
  int32_t tile1, tile3;        /* GEMM tile ids, -1 = built-in choice */
  int32_t opts;                /* extra CUSYNC_OPT_* bits, -1 = none */
  int32_t causal;
  uint32_t cached_rows;        /* key/value cache rows in front of the `seq` new ones (the reference's --seqlen with
                                  --batch new rows, TB/attention.cu:265-276); qkv then has cached_rows + seq rows */
  int32_t kv_split_blocks;     /* key/value blocks per attention workgroup: -1 = built-in choice, 0 = no split */
} cusync_attn_layer_config;

typedef struct cusync_attn_layer cusync_attn_layer;

/* wqkv: [hidden][3*heads*head_dim], wo: [heads*head_dim][hidden], both fp16 row-major device pointers. */
cusync_attn_layer *cusync_attn_layer_create(const cusync_attn_layer_config *cfg, const void *wqkv, const void *wo);
void cusync_attn_layer_destroy(cusync_attn_layer *layer);
/* x: [seq][hidden]; qkv: [cached_rows + seq][3*heads*head_dim] (the cache rows filled by the caller); o: [seq][heads*head_dim]; y: [seq][hidden].  Runs `runs`
 * times, synchronising after each; times_us[r] = start of the first kernel to end of the last.  For the
 * stream-ordered mode stage_us[3*r + i] receives the time of stage i. */
cusync_error cusync_attn_layer_run(cusync_attn_layer *layer, const void *x, void *qkv, void *o, void *y, int runs,
                                   double *times_us, double *stage_us);
const cusync_stage_desc *cusync_attn_layer_stage(const cusync_attn_layer *layer, int which);
int cusync_attn_layer_tiles(const cusync_attn_layer *layer, int *tile1, int *tile3);

/* ------------------------------------------------------------------------- */
/* MLP chain (replaces the extern "C" surface of TB/mlp-lib.cu:555-618 and    */
/* the hot loops runBaselineGPT3 / runCuSyncGPT3 / runCuSyncLLaMA,            */
/* TB/mlp.cu:411-491, 645-716, 718-862)                                       */
/* ------------------------------------------------------------------------- */

enum { CUSYNC_MLP_GPT3 = 0, CUSYNC_MLP_LLAMA = 1 };
enum { CUSYNC_SYNC_STREAM = 0,     /* kernel-boundary sync: both GEMMs on one stream */
       CUSYNC_SYNC_ROW = 1, CUSYNC_SYNC_TILE = 2, CUSYNC_SYNC_STRIDED = 3 };

typedef struct cusync_mlp_config {
  int32_t model;               /* CUSYNC_MLP_* */
  uint32_t batch;              /* rows of X */
  uint32_t hidden;             /* H: 12288 (GPT-3) / 8192 (LLaMA) */
  uint32_t inner;              /* columns of H1: 4H/8 = 6144 (GPT-3); d = 2752 or 2816 (LLaMA) */
  int32_t sync;                /* CUSYNC_SYNC_* */
  int32_t tile1, tile2;        /* CUSYNC_TILE_* per GEMM, -1 = pick from the built-in table */
  int32_t opts;                /* extra CUSYNC_OPT_* bits, -1 = the reference's defaults for `sync` */
  int32_t activation;          /* GPT-3: 1 = GeLU fused in GEMM1, 0 = none.  LLaMA: 1 = silu(g)*u fused
                                  in GEMM2's A loader, 0 = GEMM2 reads the gate half as is (TB/mlp.cu:785-792) */
  int32_t split_k1, split_k2;  /* k-slices per GEMM (--split-k1/--split-k2, TB/mlp.cu:880-931); 0 = pick so that
                                  the launch fills the device */
  int32_t max_wg1, max_wg2;    /* workgroups per launch of each GEMM; 0 = built-in choice, -1 = as many as stay resident */
  int32_t one_launch;          /* 1 (with a CuSync mode): both GEMMs in one launch, cusync_gemm_chain_run; needs the same
                                  direct-to-LDS tile for both and a plain A operand in GEMM2.  0: one launch per GEMM on
                                  two streams, as the reference runs them.  -1: whichever measured faster for this
                                  model and batch size with the table's tiles (cusync_mlp_choice reports it) */
  int32_t swiglu_in_gemm2;     /* LLaMA with activation: where silu(gate)*up is computed.
                                  2: in GEMM1's epilogue (CUSYNC_EPILOGUE_SWIGLU).  create() copies w1 into a buffer of its
                                  own with the gate and up columns interleaved in groups of eight (call
                                  cusync_mlp_reload_weights after changing the caller's copy); the intermediate h is then
                                  silu(gate)*up itself, [batch][inner] packed at the front of the caller's buffer, GEMM2
                                  reads it with the direct-to-LDS tiles, and the policies count its columns (a GEMM1 tile
                                  is half as wide there; under StridedSync it posts for its gate half and its up half at
                                  once).  Two kernels, every element once, half the intermediate traffic.
                                  -1: in a stage of its own between the GEMMs (a third kernel and stream; h is gate|up).
                                  1: in GEMM2's A loader as the data passes (repeated for every column tile of GEMM2:
                                  357 against 128 us at 2048 rows; h is gate|up).
                                  0: built-in choice, which is 2 */
  int32_t repack_weights;      /* 1: create() copies w1 and w2 into buffers of its own whose row pitch is 256 bytes longer
                                  than the row, and the GEMMs read those (call cusync_mlp_reload_weights after changing
                                  the caller's copies).  The shards' rows are multiples of 4 KiB, so a column tile of the
                                  caller's layout keeps address bits 8..11 fixed over all its k rows and draws on one
                                  class of memory channels only, one of which delivers a quarter less: at few rows,
                                  where the GEMMs stream the weights, the slowest tiles decide (24 against 18.5 us).
                                  0: read the caller's arrays in place (the reference's behaviour). */
} cusync_mlp_config;

typedef struct cusync_mlp cusync_mlp;   /* opaque */

/* initMLPParams / initCuSyncMLPParams (TB/mlp-lib.cu:555-567, 596-609).
 * w1: [hidden, inner] (GPT-3) or [hidden, 2*inner] gate|up (LLaMA); w2: [inner, hidden]. */
cusync_mlp *cusync_mlp_create(const cusync_mlp_config *cfg, const void *w1, const void *w2);
void cusync_mlp_destroy(cusync_mlp *mlp);
/* With repack_weights: copies the caller's w1 / w2 (the pointers given to create) into the padded buffers again. */
cusync_error cusync_mlp_reload_weights(cusync_mlp *mlp);
/* runLLAMA / runCuSyncLLAMA (TB/mlp-lib.cu:569-576, 611-618): `runs` back-to-back
 * passes x -> h -> y.  h is the intermediate [batch, inner] (GPT-3) or a buffer of
 * [batch, 2*inner] (LLaMA: gate|up, or silu(gate)*up in its first batch*inner elements
 * when the activation is GEMM1's epilogue, see cusync_mlp_config::swiglu_in_gemm2).  If times_us != NULL it receives one elapsed time
 * per run, measured with events start (producer stream) -> end (consumer stream)
 * exactly as TB/mlp.cu:691-708; each run is then followed by an event wait. */
/* Returns CUSYNC_ERROR_DEVICE (text in cusync_rt_last_error) when a wait of one of the chain's stages, the wait
 * kernel's included, gave up after CUSYNC_SPIN_LIMIT polls during the call: the kernel went on with data that
 * had not been posted, so the outputs of the call are not valid.  The same holds for cusync_conv_chain_run and
 * cusync_attn_layer_run.  The launchers that do not synchronise (cusync_gemm_run, cusync_conv2d_run,
 * cusync_attention_run) cannot know: their callers read spin_timeouts with cusync_stage_read_state. */
cusync_error cusync_mlp_run(cusync_mlp *mlp, const void *x, void *h, void *y, int runs, double *times_us);
/* Same, but also reports the two kernels' own durations (stream-ordered mode
 * only; TB/mlp.cu:463-488). */
cusync_error cusync_mlp_run_split(cusync_mlp *mlp, const void *x, void *h, void *y, int runs,
                                  double *times_us, double *gemm1_us, double *gemm2_us);
/* Device state of the two stages for tests (see cusync_stage_read_state). */
const cusync_stage_desc *cusync_mlp_stage(const cusync_mlp *mlp, int which /* 0 producer (GEMM1), 1 consumer (GEMM2), 2 the activation stage or NULL */);
int cusync_mlp_tiles(const cusync_mlp *mlp, int *tile1, int *tile2);
/* The tile table without a handle: the tiles, k-slices and number of launches (*one_launch 1 or 0)
 * cusync_mlp_create would take for `cfg` on this device (fields < 0 / 0 in cfg mean "choose", as there).  What a driver that wires its own stages and launchers looks
 * up per batch size, as the reference's build looks its shapes up in src/ml-bench/transformer/tile_sizes_db.py.
 * Returns 0, or 1 with cusync_rt_last_error() set. */
int cusync_mlp_choice(const cusync_mlp_config *cfg, int *tile1, int *tile2, int *split_k1, int *split_k2, int *one_launch);
int cusync_mlp_splits(const cusync_mlp *mlp, int *split_k1, int *split_k2);

/* ------------------------------------------------------------------------- */
/* Cost of the synchronisation itself (src/examples/sync-overhead/sync-overhead.cu) */
/* ------------------------------------------------------------------------- */

/* The example's experiment (sync-overhead.cu:40-105): a producer kernel that writes one value per thread and a
 * consumer kernel that adds one to it, `blocks` x `threads`, timed from the host over `iters` runs after `warmup`:
 * once with CuStage tile/post/wait per block on two streams, once stream-ordered without any of it.
 * Overhead in percent = (with - without) / without * 100 (:104).  After each of the two legs the consumer's output
 * is checked: every element must be the value the producer wrote in the last run plus one, and no wait may have
 * given up; otherwise CUSYNC_ERROR_DEVICE with the count in cusync_rt_last_error(). */
cusync_error cusync_sync_overhead_pair(uint32_t blocks, uint32_t threads, int warmup, int iters,
                                       double *with_sync_us, double *without_sync_us);
/* The same experiment with the example's own kernels (sync-overhead.cu:40-59, 84-101): the producer's first thread
 * adds one to its block's word of a bare flag array behind a barrier, the consumer's first thread polls word 0, no
 * fences, no tile order, both kernels on ONE stream, so that the flags are up when the consumer starts: the cost of
 * touching the flags, which is what the example's percentage measures.  Same checks as above. */
cusync_error cusync_sync_overhead_bare(uint32_t blocks, uint32_t threads, int warmup, int iters,
                                       double *with_flags_us, double *without_flags_us);
/* Latency of a post -> wait hand-over: workgroup 0 and workgroup `partner` (1..63) of one launch pass a
 * semaphore back and forth `rounds` times.  Workgroups go to the eight XCDs round-robin, so partner 8 shares
 * workgroup 0's XCD and partner 1 does not.  No counterpart in the reference, whose GPUs have one L2. */
cusync_error cusync_sync_overhead_pingpong(uint32_t partner, uint32_t rounds, double *ns_per_round_trip);

/* ------------------------------------------------------------------------- */
/* What the matrix pipes sustain on this machine                              */
/* ------------------------------------------------------------------------- */

/* Runs chains of v_mfma_f32_32x32x16_f16 on register operands (no LDS, no memory) on every SIMD of the device,
 * `launches` untimed launches and then `launches` timed ones of `iters` x 16 MFMAs per wavefront, with all-zero
 * (`random_data` = 0) or random operands, and reports the rate and the shader clock it ran at.  Under such a load
 * the power management lowers the clock, more so the more bits toggle: the result is the ceiling of any fp16 GEMM
 * on the machine, below the published 2.5 PFLOP/s.  No counterpart in the reference; bench.py prints it next to
 * the roofline of the GEMM kernels. */
cusync_error cusync_probe_mfma_rate(int random_data, uint32_t iters, int launches, double *tflops, double *clock_mhz);

#ifdef __cplusplus
}
#endif
#endif /* CUSYNC_AMD_H */
