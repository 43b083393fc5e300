/*
 * CPU oracle for the CuSync hot path.  TEST INFRASTRUCTURE ONLY — see
 * cusync_oracle.h for the rules on who may call it and for the pinning status
 * of every function.
 */
#include "cusync_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------------ */
/* Tile orders                                                               */
/* ------------------------------------------------------------------------ */

/* CS/tile-orders.h:52-54 (TransposeXYOrder) and :68-70 (IdentityOrder): both
 * orders linearise a block as x + y*gx + z*gx*gy. */
uint32_t orc_block_index(int order, orc_dim3 grid, orc_dim3 block) {
  (void)order;
  return block.x + block.y * grid.x + block.z * grid.x * grid.y;
}

/* CS/tile-orders.h:57-59: TransposeXY maps tile {x,y,z} to block {y,x,z};
 * :73-75: Identity maps it to {x,y,z}. */
orc_dim3 orc_tile_to_block(int order, orc_dim3 tile) {
  orc_dim3 b;
  if (order == ORC_ORDER_TRANSPOSE_XY) {
    b.x = tile.y; b.y = tile.x; b.z = tile.z;
  } else {
    b = tile;
  }
  return b;
}

/* CS/tile-orders.h:39-42 */
uint32_t orc_tile_index(int order, orc_dim3 tile, orc_dim3 grid) {
  return orc_block_index(order, grid, orc_tile_to_block(order, tile));
}

/* CS/cusync.h:125-157.  The reference indexes hTileOrder[id] without checking
 * id < numTiles; the oracle treats an out-of-range id as the same error. */
int orc_build_schedule(int order, orc_dim3 grid, orc_dim3 *out) {
  uint32_t n = grid.x * grid.y * grid.z;
  int err = 0;
  for (uint32_t i = 0; i < n; i++) { out[i].x = n; out[i].y = 0; out[i].z = 0; }
  for (uint32_t z = 0; z < grid.z; z++)
    for (uint32_t y = 0; y < grid.y; y++)
      for (uint32_t x = 0; x < grid.x; x++) {
        orc_dim3 b = {x, y, z};
        uint32_t id = orc_block_index(order, grid, b);
        if (id < n && out[id].x == n) out[id] = b; else err = 1;
      }
  return err ? ORC_ERR_INVALID_LINEAR_BLOCK_INDEX : ORC_SUCCESS;
}

/* ------------------------------------------------------------------------ */
/* Policies                                                                  */
/* ------------------------------------------------------------------------ */

uint32_t orc_policy_wait_value(const orc_policy *p, orc_dim3 tile, orc_dim3 grid) {
  (void)tile; (void)grid;
  switch (p->kind) {
    case ORC_ROWSYNC:         return p->waitValue;            /* CS/policies.h:66-68 */
    case ORC_TILESYNC:        return p->waitValue;            /* CS/policies.h:122-124 */
    case ORC_CONV2DTILESYNC:  return p->waitValue;            /* CS/policies.h:182-184 */
    case ORC_STRIDEDSYNC:     return p->stride;               /* TB/mlp.cu:83-85 */
    case ORC_CONSECUTIVESYNC: return (p->H / 8) / p->tileN;   /* TB/attention.cu:55-57 */
    default:                  return 0;                       /* CS/policies.h:24 */
  }
}

uint32_t orc_policy_post_value(const orc_policy *p, orc_dim3 tile, orc_dim3 grid) {
  (void)tile; (void)grid;
  switch (p->kind) {
    case ORC_ROWSYNC:         return p->postValue;            /* CS/policies.h:91-93 */
    case ORC_TILESYNC:        return p->postValue;            /* CS/policies.h:130-131 */
    case ORC_CONV2DTILESYNC:  return p->postValue;            /* CS/policies.h:190-191 */
    case ORC_STRIDEDSYNC:     return 1;                       /* TB/mlp.cu:87-88 */
    case ORC_CONSECUTIVESYNC: return 1;                       /* TB/attention.cu:59-60 */
    default:                  return 0;                       /* CS/policies.h:30 */
  }
}

uint32_t orc_policy_tile_index(const orc_policy *p, orc_dim3 tile, orc_dim3 grid) {
  orc_dim3 t = {0, 0, 0};
  switch (p->kind) {
    case ORC_ROWSYNC:                                         /* CS/policies.h:74-76 */
      return tile.x / p->tileM;
    case ORC_TILESYNC:                                        /* CS/policies.h:137-139 */
      t.x = tile.x / p->tileM; t.y = tile.y / p->tileN;
      return orc_tile_index(p->order, t, grid);
    case ORC_CONV2DTILESYNC:                                  /* CS/policies.h:197-199 */
      t.x = tile.x / p->tileM; t.y = (tile.y / p->tileN) / (p->R * p->S);
      return orc_tile_index(p->order, t, grid);
    case ORC_STRIDEDSYNC: {                                   /* TB/mlp.cu:90-96 */
      uint32_t ty = tile.y / p->tileN;
      if (ty >= p->gridN / p->tileN) ty -= p->gridN / p->tileN;
      t.x = tile.x / p->tileM; t.y = ty;
      return orc_tile_index(p->order, t, grid);
    }
    case ORC_CONSECUTIVESYNC: {                               /* TB/attention.cu:62-65 */
      uint32_t g = (p->H / 8) / p->tileN;
      orc_dim3 gg = {grid.x / g, grid.y, grid.z};
      t.x = tile.x / p->tileM; t.y = (tile.y / p->tileN) / g;
      return orc_tile_index(p->order, t, gg);
    }
    default:                                                  /* CS/policies.h:26 */
      return 0;
  }
}

int orc_policy_is_sync(const orc_policy *p, orc_dim3 tile, orc_dim3 grid) {
  (void)grid;
  switch (p->kind) {
    case ORC_ROWSYNC:         return tile.z == 1;                               /* CS/policies.h:83-85 */
    case ORC_TILESYNC:        return tile.y % p->tileN == 0;                    /* CS/policies.h:145-147 */
    case ORC_CONV2DTILESYNC:  return (tile.y / p->tileN) % (p->R * p->S) == 0;  /* CS/policies.h:206-208 */
    case ORC_STRIDEDSYNC:     return tile.y % p->tileN == 0;                    /* TB/mlp.cu:98-100 */
    case ORC_CONSECUTIVESYNC: return tile.z == 1;                               /* TB/attention.cu:67-69 */
    default:                  return 0;                                         /* CS/policies.h:28 */
  }
}

/* ------------------------------------------------------------------------ */
/* Protocol end state                                                        */
/* ------------------------------------------------------------------------ */

/* One post: CS/cusync_device_defs.h:55-72.  atomicAdd(sem, postValue), or with
 * NoAtomicAdd a plain store of postValue*iter. */
static void post_one(const orc_policy *p, orc_dim3 tile, orc_dim3 grid, int iter,
                     int opts, uint32_t *sems) {
  uint32_t idx = orc_policy_tile_index(p, tile, grid);
  uint32_t v = orc_policy_post_value(p, tile, grid);
  if (opts & ORC_OPT_NO_ATOMIC_ADD) sems[idx] = v * (uint32_t)iter;
  else sems[idx] += v;
}

/* CC/gemm/kernel/cusyncgemm.h:374-398: the block posts {row offset, column
 * offset, k-slice}; with serial split-K only the last k-slice posts.
 * Grid convention CC/gemm/threadblock/cusync_threadblock_swizzle.h:27-32:
 * x = n-tile, y = m-tile, z = k-slice.  CS/cusync.h:188-189: one semaphore per
 * block of the grid, zero-initialised. */
void orc_expected_sems_gemm(const orc_policy *p, orc_dim3 grid,
                            uint32_t kernelTileM, uint32_t kernelTileN,
                            int iters, int opts, uint32_t *sems) {
  uint32_t n = grid.x * grid.y * grid.z;
  memset(sems, 0, n * sizeof(uint32_t));
  for (int it = 1; it <= iters; it++)
    for (uint32_t z = 0; z < grid.z; z++)
      for (uint32_t y = 0; y < grid.y; y++)
        for (uint32_t x = 0; x < grid.x; x++) {
          if (z + 1 != grid.z) continue;
          orc_dim3 tile = {y * kernelTileM, x * kernelTileN, z};
          post_one(p, tile, grid, it, opts, sems);
        }
}

/* tests/simple-test.cu:14-27: tile = custage.tile(...) is the block index and
 * is posted unchanged. */
void orc_expected_sems_blocks(const orc_policy *p, orc_dim3 grid, int iters,
                              int opts, uint32_t *sems) {
  uint32_t n = grid.x * grid.y * grid.z;
  memset(sems, 0, n * sizeof(uint32_t));
  for (int it = 1; it <= iters; it++)
    for (uint32_t z = 0; z < grid.z; z++)
      for (uint32_t y = 0; y < grid.y; y++)
        for (uint32_t x = 0; x < grid.x; x++) {
          orc_dim3 tile = {x, y, z};
          post_one(p, tile, grid, it, opts, sems);
        }
}

/* CPU replay of CS/cusync_device_defs.h (tile/wait/post) for a two-GEMM chain.
 * Producer blocks run to completion in ticket order; consumer blocks occupy a
 * slot from their first wait to their last.  A consumer's waits are the ones a
 * tile-synchronised main loop issues: once with z=1 before the loop, then one
 * per K chunk with z=0 (CC/gemm/threadblock/cusyncmma_multistage.h:986-994,
 * 1032-1040).  Deadlock = all consumer slots blocked and no producer left that
 * can still run. */
int orc_replay_chain(const orc_policy *p, orc_dim3 prodGrid, orc_dim3 consGrid,
                     uint32_t prodTileM, uint32_t prodTileN,
                     uint32_t consTileM, uint32_t consTileK, uint32_t consK,
                     int prodSlots, int consSlots, int iters, int opts,
                     uint32_t *sems) {
  uint32_t np = prodGrid.x * prodGrid.y * prodGrid.z;
  uint32_t nc = consGrid.x * consGrid.y * consGrid.z;
  orc_dim3 *po = (orc_dim3 *)malloc(np * sizeof(orc_dim3));
  orc_dim3 *co = (orc_dim3 *)malloc(nc * sizeof(orc_dim3));
  int ok = 1;
  if (orc_build_schedule(ORC_ORDER_IDENTITY, prodGrid, po) != ORC_SUCCESS) ok = 0;
  if (orc_build_schedule(ORC_ORDER_IDENTITY, consGrid, co) != ORC_SUCCESS) ok = 0;
  memset(sems, 0, np * sizeof(uint32_t));
  if (consSlots < 1) consSlots = 1;
  if (prodSlots < 1) prodSlots = 1;
  uint32_t nchunks = (consK + consTileK - 1) / consTileK;
  /* per-slot state: consumer ticket and next chunk to wait for (-1 = pre-loop) */
  int64_t *slotTicket = (int64_t *)malloc(sizeof(int64_t) * (size_t)consSlots);
  int64_t *slotChunk = (int64_t *)malloc(sizeof(int64_t) * (size_t)consSlots);
  for (int it = 1; it <= iters && ok; it++) {
    uint32_t pnext = 0, cnext = 0, cdone = 0;
    for (int s = 0; s < consSlots; s++) slotTicket[s] = -1;
    while (cdone < nc && ok) {
      int progressed = 0;
      /* producers: up to prodSlots tiles complete per round, in ticket order */
      for (int s = 0; s < prodSlots && pnext < np; s++, pnext++) {
        orc_dim3 b = po[pnext];
        if (b.z + 1 == prodGrid.z) {
          orc_dim3 tile = {b.y * prodTileM, b.x * prodTileN, b.z};
          post_one(p, tile, prodGrid, it, opts, sems);
        }
        progressed = 1;
      }
      /* consumers */
      for (int s = 0; s < consSlots; s++) {
        if (slotTicket[s] < 0) {
          if (cnext >= nc) continue;
          slotTicket[s] = cnext++; slotChunk[s] = -1; progressed = 1;
        }
        orc_dim3 b = co[slotTicket[s]];
        uint32_t row = b.y * consTileM;
        for (;;) {
          orc_dim3 t;
          t.x = row;
          t.y = slotChunk[s] < 0 ? 0 : (uint32_t)slotChunk[s] * consTileK;
          t.z = slotChunk[s] < 0 ? 1 : 0;
          if (orc_policy_is_sync(p, t, prodGrid)) {
            uint32_t idx = orc_policy_tile_index(p, t, prodGrid);
            uint32_t need = (uint32_t)it * orc_policy_wait_value(p, t, prodGrid);
            if (idx >= np) { ok = 0; break; }
            if (sems[idx] < need) break;          /* still spinning */
            if (sems[idx] != need) ok = 0;        /* tests/cusync-test.h:24 */
          }
          progressed = 1;
          slotChunk[s]++;
          if ((uint32_t)slotChunk[s] >= nchunks) { slotTicket[s] = -1; cdone++; break; }
        }
      }
      if (!progressed) { ok = 0; break; }        /* deadlock */
    }
  }
  free(po); free(co); free(slotTicket); free(slotChunk);
  return ok;
}

/* ------------------------------------------------------------------------ */
/* fp16 <-> fp32                                                             */
/* ------------------------------------------------------------------------ */

float orc_h2f(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else {
      int e = -1;
      do { e++; man <<= 1; } while ((man & 0x400u) == 0);
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

/* Round to nearest, ties to even (IEEE 754 binary32 -> binary16). */
uint16_t orc_f2h(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  uint32_t ax = x & 0x7fffffffu;
  if (ax >= 0x7f800000u) {                        /* inf / nan */
    if (ax > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((ax >> 13) & 0x3ffu));
    return (uint16_t)(sign | 0x7c00u);
  }
  if (ax >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);   /* rounds to >= 65520 -> inf */
  if (ax < 0x33000001u) return sign;                            /* < 2^-25 (or == 2^-25 tie to 0) */
  int32_t e = (int32_t)(ax >> 23) - 127;
  uint32_t m = (ax & 0x7fffffu) | 0x800000u;                    /* 24-bit significand */
  int shift;
  uint32_t base;
  if (e < -14) { shift = 13 + (-14 - e); base = 0; }             /* subnormal half */
  else { shift = 13; base = (uint32_t)(e + 15) << 10; m &= 0x7fffffu; }
  uint32_t q = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  uint32_t r = base + q;
  if (rem > half || (rem == half && (r & 1u))) r++;
  return (uint16_t)(sign | r);
}

void orc_h2f_array(const uint16_t *h, float *f, size_t n) {
  for (size_t i = 0; i < n; i++) f[i] = orc_h2f(h[i]);
}
void orc_f2h_array(const float *f, uint16_t *h, size_t n) {
  for (size_t i = 0; i < n; i++) h[i] = orc_f2h(f[i]);
}

/* ------------------------------------------------------------------------ */
/* Epilogue closed forms (parity unpinned against the reference, see header) */
/* ------------------------------------------------------------------------ */

float orc_gelu(float x) { return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f)); }
float orc_silu(float x) { return x / (1.0f + expf(-x)); }

static float apply_epilogue(float v, int epilogue) {
  if (epilogue == ORC_EPI_GELU) return orc_gelu(v);
  if (epilogue == ORC_EPI_RELU) return v > 0.0f ? v : 0.0f;
  return v;
}

/* ------------------------------------------------------------------------ */
/* GEMM                                                                      */
/* ------------------------------------------------------------------------ */

/* TB/common.h:89-102 (ref_cpumatmul<half,float>): same loop nest, same
 * parallel loop, same accumulation order; leading dimensions added so a
 * sub-matrix can be multiplied in place. */
void orc_gemm_f16(uint32_t M, uint32_t N, uint32_t K,
                  const uint16_t *A, uint32_t lda, const uint16_t *B, uint32_t ldb,
                  uint16_t *C, uint32_t ldc, int epilogue) {
  for (uint32_t i = 0; i < M; i++) {
    #pragma omp parallel for
    for (uint32_t j = 0; j < N; j++) {
      float accum = 0;
      for (uint32_t k = 0; k < K; k++)
        accum += orc_h2f(A[(size_t)i * lda + k]) * orc_h2f(B[(size_t)k * ldb + j]);
      C[(size_t)i * ldc + j] = orc_f2h(apply_epilogue(accum, epilogue));
    }
  }
}

void orc_swiglu_f16(uint32_t M, uint32_t d, const uint16_t *gu, uint32_t ld_gu,
                    uint16_t *h, uint32_t ld_h) {
  for (uint32_t r = 0; r < M; r++)
    for (uint32_t i = 0; i < d; i++) {
      float g = orc_h2f(gu[(size_t)r * ld_gu + i]);
      float u = orc_h2f(gu[(size_t)r * ld_gu + d + i]);
      h[(size_t)r * ld_h + i] = orc_f2h(orc_silu(g) * u);
    }
}

/* The LLaMA feed-forward's first stage with the activation applied to the accumulators, as an epilogue of the
 * GEMM: H[i][j] = silu(sum_k X[i][k] W[k][j]) * (sum_k X[i][k] W[k][d + j]), W = gate | up side by side
 * ([K][2d]).  Both sums are ref_cpumatmul's (TB/common.h:89-102: fp32, k ascending), the product is formed in
 * fp32 and rounded to fp16 once.  This is where the reference puts the activation in its library build
 * (TB/mlp-lib.cu:122-133: LinearCombinationSilu on X W1, then LinearCombinationSwiGLU scaling the accumulator
 * of X V by it); its arithmetic lives in CUTLASS, which is absent, so the closed form x*sigmoid(x)*u stands in. */
void orc_gemm_swiglu_f16(uint32_t M, uint32_t d, uint32_t K,
                         const uint16_t *A, uint32_t lda, const uint16_t *W, uint32_t ldw,
                         uint16_t *H, uint32_t ldh) {
  for (uint32_t i = 0; i < M; i++) {
    #pragma omp parallel for
    for (uint32_t j = 0; j < d; j++) {
      float gate = 0, up = 0;
      for (uint32_t k = 0; k < K; k++) {
        const float a = orc_h2f(A[(size_t)i * lda + k]);
        gate += a * orc_h2f(W[(size_t)k * ldw + j]);
        up += a * orc_h2f(W[(size_t)k * ldw + d + j]);
      }
      H[(size_t)i * ldh + j] = orc_f2h(orc_silu(gate) * up);
    }
  }
}

/* Textbook softmax(mask(Q K^T / sqrt(hd))) V per head, all in fp32.  The S query rows are rows
 * cached .. cached+S-1 of qkv; keys and values are rows 0 .. cached+S-1 (rows below `cached` are the
 * key/value cache of TB/attention.cu:272-276, 289: the projection writes its rows behind `seqlen` cached
 * ones).  Causal: query i sees keys 0 .. cached+i. */
void orc_attention_kv_f16(uint32_t S, uint32_t cached, uint32_t heads, uint32_t hd,
                          const uint16_t *qkv, uint32_t ld_qkv,
                          uint16_t *out, uint32_t ld_out, int causal) {
  uint32_t D = heads * hd;
  float scale = 1.0f / sqrtf((float)hd);
  #pragma omp parallel for collapse(2)
  for (uint32_t h = 0; h < heads; h++)
    for (uint32_t i = 0; i < S; i++) {
      uint32_t total = cached + S;
      float *p = (float *)malloc(sizeof(float) * total);
      float *o = (float *)calloc(hd, sizeof(float));
      uint32_t lim = causal ? cached + i + 1 : total;
      const uint16_t *qrow = qkv + (size_t)(cached + i) * ld_qkv + h * hd;
      float mx = -INFINITY;
      for (uint32_t j = 0; j < lim; j++) {
        float s = 0;
        for (uint32_t c = 0; c < hd; c++)
          s += orc_h2f(qrow[c]) * orc_h2f(qkv[(size_t)j * ld_qkv + D + h * hd + c]);
        p[j] = s * scale;
        if (p[j] > mx) mx = p[j];
      }
      float sum = 0;
      for (uint32_t j = 0; j < lim; j++) { p[j] = expf(p[j] - mx); sum += p[j]; }
      for (uint32_t j = 0; j < lim; j++) {
        float w = p[j] / sum;
        for (uint32_t c = 0; c < hd; c++)
          o[c] += w * orc_h2f(qkv[(size_t)j * ld_qkv + 2 * D + h * hd + c]);
      }
      for (uint32_t c = 0; c < hd; c++) out[(size_t)i * ld_out + h * hd + c] = orc_f2h(o[c]);
      free(p); free(o);
    }
}

void orc_attention_f16(uint32_t S, uint32_t heads, uint32_t hd,
                       const uint16_t *qkv, uint32_t ld_qkv,
                       uint16_t *out, uint32_t ld_out, int causal) {
  orc_attention_kv_f16(S, 0, heads, hd, qkv, ld_qkv, out, ld_out, causal);
}

/* Direct 7-loop NHWC forward convolution, cross-correlation, KRSC filters. */
void orc_conv2d_nhwc_f16(uint32_t N, uint32_t H, uint32_t W, uint32_t C, uint32_t K,
                         uint32_t R, uint32_t S, uint32_t pad, uint32_t stride,
                         const uint16_t *x, const uint16_t *w, uint16_t *y, int epilogue) {
  uint32_t P = (H + 2 * pad - R) / stride + 1;
  uint32_t Q = (W + 2 * pad - S) / stride + 1;
  #pragma omp parallel for collapse(2)
  for (uint32_t n = 0; n < N; n++)
    for (uint32_t p = 0; p < P; p++)
      for (uint32_t q = 0; q < Q; q++)
        for (uint32_t k = 0; k < K; k++) {
          float acc = 0;
          for (uint32_t r = 0; r < R; r++)
            for (uint32_t s = 0; s < S; s++) {
              int64_t h = (int64_t)p * stride + r - pad;
              int64_t ww = (int64_t)q * stride + s - pad;
              if (h < 0 || h >= (int64_t)H || ww < 0 || ww >= (int64_t)W) continue;
              const uint16_t *xp = x + (((size_t)n * H + (size_t)h) * W + (size_t)ww) * C;
              const uint16_t *wp = w + (((size_t)k * R + r) * S + s) * C;
              for (uint32_t c = 0; c < C; c++) acc += orc_h2f(xp[c]) * orc_h2f(wp[c]);
            }
          y[(((size_t)n * P + p) * Q + q) * K + k] = orc_f2h(apply_epilogue(acc, epilogue));
        }
}

/* TB/common.h:104-137 */
int orc_equals_f16(size_t n, const uint16_t *a, const uint16_t *b, float tol) {
  int eq = 1;
  for (size_t i = 0; i < n; i++) {
    float e1 = orc_h2f(a[i]), e2 = orc_h2f(b[i]);
    int ret;
    if (fabsf(e1) < tol && fabsf(e2) < tol) ret = 1;
    else if (fabsf(e1) < tol) ret = 0;
    else if (fabsf(e2) < tol) ret = 0;
    else {
      float m = fabsf(e1) > fabsf(e2) ? fabsf(e1) : fabsf(e2);
      float err = fabsf(fabsf(e1) - fabsf(e2)) / m;
      ret = err <= tol;
    }
    if (!ret) eq = 0;
  }
  return eq;
}

size_t orc_count_mismatch_f16(size_t n, const uint16_t *a, const uint16_t *b,
                              float rel_tol, float abs_tol, float *max_abs_err) {
  size_t bad = 0;
  float mx = 0;
  for (size_t i = 0; i < n; i++) {
    float x = orc_h2f(a[i]), r = orc_h2f(b[i]);
    float d = fabsf(x - r);
    if (!(d <= abs_tol + rel_tol * fabsf(r))) bad++;
    if (d > mx || d != d) mx = d;
  }
  if (max_abs_err) *max_abs_err = mx;
  return bad;
}

int orc_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
