/*
 * CPU oracle for the CuSync hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * Nothing in the shipped library links, loads or calls this file.  It exists so
 * that tests, the smoke check and the benchmark's cpu_baseline leg can compare
 * the HIP path with an independent, plain-C restatement of what the reference
 * computes.  Every function names the reference file:line it restates
 * (paths are relative to the reference checkout):
 *
 *   CS = src/include/cusync            TB = src/ml-bench/transformer
 *   CC = src/include/cutlass/cusync-cutlass/include/cutlass
 *   CV = src/ml-bench/volta_conv2d     EX = src/examples
 *
 * Pinning status (what checks each function against something other than
 * itself lives in tests/test_oracle_*.py):
 *   tile orders, schedule buffer, policies .... pinned (closed forms, brute force, hand-worked cases)
 *   semaphore end state ....................... pinned (closed forms; tests/simple-test.cu known answer)
 *   fp16 <-> fp32 conversion .................. pinned (numpy float16, exhaustive one way)
 *   GEMM fp32-accumulate ...................... pinned (matrixMul.cu known answer, numpy matmul)
 *   equals() .................................. pinned (hand-worked branches)
 *   conv2d NHWC ............................... pinned (all-ones closed form, 1x1 == GEMM, scipy correlate)
 *   causal multi-head attention ............... pinned (row sums, first-row identity, numpy restatement)
 *   GeLU / SiLU*up / ReLU epilogues ........... pinned to the textbook closed forms only;
 *        PARITY UNPINNED against the reference: its arithmetic for these lives in
 *        NVIDIA CUTLASS (un-vendored submodule, absent) and no reference test covers them.
 */
#ifndef CUSYNC_ORACLE_H
#define CUSYNC_ORACLE_H

#include <stdint.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct { uint32_t x, y, z; } orc_dim3;

/* CS/tile-orders.h:50-76 */
enum { ORC_ORDER_IDENTITY = 0, ORC_ORDER_TRANSPOSE_XY = 1 };

/* CS/policies.h:18-210, TB/mlp.cu:76-101, TB/attention.cu:51-70 */
enum {
  ORC_NOSYNC = 0,
  ORC_ROWSYNC = 1,
  ORC_TILESYNC = 2,
  ORC_STRIDEDSYNC = 3,
  ORC_CONV2DTILESYNC = 4,
  ORC_CONSECUTIVESYNC = 5
};

/* CS/cusync.h:46-53 — the success code is LAST (5), not 0. */
enum {
  ORC_ERR_NOT_PRODUCER = 0,
  ORC_ERR_NOT_CONSUMER = 1,
  ORC_ERR_NOT_INITIALIZED = 2,
  ORC_ERR_INVALID_LINEAR_BLOCK_INDEX = 3,
  ORC_ERR_DEVICE = 4,
  ORC_SUCCESS = 5
};

/* CS/cusync.h:69-75 */
enum {
  ORC_OPT_NONE = 0,
  ORC_OPT_NO_ATOMIC_ADD = 1,
  ORC_OPT_AVOID_WAIT_KERNEL = 2,
  ORC_OPT_AVOID_CUSTOM_ORDER = 4,
  ORC_OPT_REORDER_TILE_LOADS = 8
};

typedef struct {
  int32_t kind;        /* ORC_* policy kind */
  int32_t order;       /* ORC_ORDER_* (ignored by RowSync) */
  uint32_t tileM, tileN;
  uint32_t waitValue, postValue;
  uint32_t gridN;      /* StridedSync: width (elements) of one strided group */
  uint32_t stride;     /* StridedSync: number of groups == wait value */
  uint32_t R, S;       /* Conv2DTileSync filter extent */
  uint32_t H;          /* ConsecutiveSync: hidden size; group width is H/8 elements */
} orc_policy;

/* ---- tile orders -------------------------------------------------------- */
uint32_t orc_block_index(int order, orc_dim3 grid, orc_dim3 block);
orc_dim3 orc_tile_to_block(int order, orc_dim3 tile);
uint32_t orc_tile_index(int order, orc_dim3 tile, orc_dim3 grid);
/* Fills out[numTiles]; returns ORC_SUCCESS or ORC_ERR_INVALID_LINEAR_BLOCK_INDEX. */
int orc_build_schedule(int order, orc_dim3 grid, orc_dim3 *out);

/* ---- policies ----------------------------------------------------------- */
uint32_t orc_policy_wait_value(const orc_policy *p, orc_dim3 tile, orc_dim3 grid);
uint32_t orc_policy_post_value(const orc_policy *p, orc_dim3 tile, orc_dim3 grid);
uint32_t orc_policy_tile_index(const orc_policy *p, orc_dim3 tile, orc_dim3 grid);
int      orc_policy_is_sync(const orc_policy *p, orc_dim3 tile, orc_dim3 grid);

/* ---- protocol end state ------------------------------------------------- */
/* Semaphore array after `iters` complete runs of a producer GEMM/conv kernel
 * whose grid is (n-tiles, m-tiles, k-slices) and whose blocks post
 * {m*kernelTileM, n*kernelTileN, k}; with k-slices > 1 only the last slice posts. */
void orc_expected_sems_gemm(const orc_policy *out_policy, orc_dim3 grid,
                            uint32_t kernelTileM, uint32_t kernelTileN,
                            int iters, int opts, uint32_t *sems /* [gx*gy*gz] */);
/* Semaphore array after `iters` runs of the 1-D copy-kernel producer of
 * tests/simple-test.cu (every block posts its own block index as the tile). */
void orc_expected_sems_blocks(const orc_policy *out_policy, orc_dim3 grid,
                              int iters, int opts, uint32_t *sems);
/* Replays producer and consumer blocks of a two-stage GEMM chain on the CPU with
 * a bounded number of resident slots per stage, tickets drawn in tile order.
 * Returns 1 if every consumer wait was eventually satisfied (no deadlock) and
 * every wait saw exactly value == iter*waitValue at consumer exit, else 0. */
int orc_replay_chain(const orc_policy *policy, orc_dim3 prodGrid, orc_dim3 consGrid,
                     uint32_t prodTileM, uint32_t prodTileN,
                     uint32_t consTileM, uint32_t consTileK, uint32_t consK,
                     int prodSlots, int consSlots, int iters, int opts,
                     uint32_t *sems_out);

/* ---- numerics ----------------------------------------------------------- */
float    orc_h2f(uint16_t h);
uint16_t orc_f2h(float f);
void     orc_h2f_array(const uint16_t *h, float *f, size_t n);
void     orc_f2h_array(const float *f, uint16_t *h, size_t n);

enum { ORC_EPI_NONE = 0, ORC_EPI_GELU = 1, ORC_EPI_RELU = 2 };
float orc_gelu(float x);
float orc_silu(float x);

/* TB/common.h:89-102: row-major, i outer, OpenMP over j, fp32 accumulate in k
 * order, result cast to fp16.  Operands are raw fp16 bit patterns. */
void orc_gemm_f16(uint32_t M, uint32_t N, uint32_t K,
                  const uint16_t *A, uint32_t lda, const uint16_t *B, uint32_t ldb,
                  uint16_t *C, uint32_t ldc, int epilogue);
/* h[r,i] = fp16( silu(gu[r,i]) * gu[r,i+d] ), gu has row pitch ld_gu. */
void orc_swiglu_f16(uint32_t M, uint32_t d, const uint16_t *gu, uint32_t ld_gu,
                    uint16_t *h, uint32_t ld_h);
/* H = silu(A W[:, 0:d]) * (A W[:, d:2d]) with the activation on the fp32 accumulators (one rounding). */
void orc_gemm_swiglu_f16(uint32_t M, uint32_t d, uint32_t K,
                         const uint16_t *A, uint32_t lda, const uint16_t *W, uint32_t ldw,
                         uint16_t *H, uint32_t ldh);
/* Causal multi-head attention over one sequence.  qkv is [S, 3*heads*hd] laid
 * out as [Q | K | V] blocks of heads*hd columns; out is [S, heads*hd]. */
void orc_attention_f16(uint32_t S, uint32_t heads, uint32_t hd,
                       const uint16_t *qkv, uint32_t ld_qkv,
                       uint16_t *out, uint32_t ld_out, int causal);
/* Same with a key/value cache: the S query rows are rows cached..cached+S-1 of qkv ([cached+S, 3*heads*hd]),
 * keys and values rows 0..cached+S-1 (TB/attention.cu:272-276, 289).  Pinned: equals the last S rows of
 * orc_attention_f16 over all cached+S rows when causal. */
void orc_attention_kv_f16(uint32_t S, uint32_t cached, uint32_t heads, uint32_t hd,
                          const uint16_t *qkv, uint32_t ld_qkv,
                          uint16_t *out, uint32_t ld_out, int causal);
/* NHWC fprop, KRSC filter, cross-correlation (CV/resnet.cu:678), fp32 accumulate. */
void orc_conv2d_nhwc_f16(uint32_t N, uint32_t H, uint32_t W, uint32_t C, uint32_t K,
                         uint32_t R, uint32_t S, uint32_t pad, uint32_t stride,
                         const uint16_t *x, const uint16_t *w, uint16_t *y, int epilogue);
/* TB/common.h:104-137 */
int orc_equals_f16(size_t n, const uint16_t *a, const uint16_t *b, float tol);
/* Counts elements with |a-b| > abs_tol + rel_tol*|b| (b is the reference). */
size_t orc_count_mismatch_f16(size_t n, const uint16_t *a, const uint16_t *b,
                              float rel_tol, float abs_tol, float *max_abs_err);
int orc_num_threads(void);

#ifdef __cplusplus
}
#endif
#endif
