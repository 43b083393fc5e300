// Fused attention stage and the self-attention chain
//   QKV = X Wqkv  ->  O = softmax(mask(Q K^T / sqrt(128))) V per head  ->  Y = O Wo
// run stream-ordered or as three CuSync stages on three streams.  Stands in for
// the reference's attention driver (src/ml-bench/transformer/attention.cu:84-110
// stage wiring, :560-700 baseline, :702-830 overlapped run), which builds the
// same dependency chain out of four CUTLASS GEMMs; here the two inner products
// are one fused kernel that is consumer and producer at once (the role of
// SCuStage / OCuStage, attention.cu:101-104).
#include <hip/hip_runtime.h>

#include <math.h>
#include <string.h>
#include <algorithm>
#include <mutex>

#include "../../include/cusync_amd.h"
#include "rt_internal.h"
#include "attention_kernel.h"
#include "split_choice.h"

namespace {

using cusync::rt::setError;
using namespace cusync::attn;

std::mutex g_attnMutex;
int g_attnResidentPerCU[2] = {-1, -1};      // [0] two stages, [1] four
int g_attnNumCUs = 0;
int g_attnLdsPerCU = 0;

typedef void (*AttnKernel)(AttnParams);
AttnKernel attnKernel(bool deep) { return deep ? attentionKernel<4> : attentionKernel<2>; }
int attnLds(bool deep) { return cusync::attn::ldsBytes(deep ? 4 : 2); }

int residentAttention(bool deep);

// Four stages where the kernel has the device to itself anyway: as a stage of its own between stream-ordered
// launches, and from 2048 key rows on, where the projections around it run 256-row tiles that take a whole CU's
// LDS (measured at 2048 rows x 12 heads: 59 -> 51 us alone; chain under ConsecutiveSync 422 -> 410 us).  Two stages
// where its workgroups are to sit beside those of its producer and consumer (chains up to 1024 rows: with four
// stages every gain of the overlapped chains over the stream-ordered ones was gone) -- as long as the launch has
// no more workgroups than CUs: beyond that the two-stage workgroups end up two to a CU on the CUs that came free
// first, and four stages with a CU each are faster again (1408 rows, 264 workgroups: 291 -> 281 us under
// ConsecutiveSync, 1792 rows: 357 -> 337; 1280 rows, 240 workgroups, stay at two stages: 237 against 246 us).
bool deepPipeline(const cusync_attention_args* a) {
  const bool alone = a->stage.in.kind == CUSYNC_POLICY_NOSYNC && a->stage.out.kind == CUSYNC_POLICY_NOSYNC;
  if (alone || a->seq + a->cached_rows >= 2048) return true;
  if (g_attnNumCUs == 0) residentAttention(false);      // reads the device's CU count
  return g_attnNumCUs > 0 && a->stage.grid.x * a->stage.grid.y * a->stage.grid.z > (uint32_t)g_attnNumCUs;
}

int residentAttention(bool deep) {
  std::lock_guard<std::mutex> lock(g_attnMutex);
  int& perCU = g_attnResidentPerCU[deep ? 1 : 0];
  if (perCU < 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (CUSYNC_HIP(hipGetDevice(&dev)) || CUSYNC_HIP(hipGetDeviceProperties(&prop, dev))) return 0;
    g_attnNumCUs = prop.multiProcessorCount;
    g_attnLdsPerCU = (int)prop.maxSharedMemoryPerMultiProcessor;
    if (CUSYNC_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(attnKernel(deep)),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, std::max(attnLds(deep), g_attnLdsPerCU / 2)))) return 0;
    int n = 0;
    if (CUSYNC_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, attnKernel(deep), kThreads, attnLds(deep)))) return 0;
    perCU = n;
  }
  return perCU * g_attnNumCUs;
}

cusync_policy_desc noSync() {
  cusync_policy_desc p;
  memset(&p, 0, sizeof p);
  p.kind = CUSYNC_POLICY_NOSYNC;
  p.tileM = p.tileN = 1; p.R = p.S = 1;
  return p;
}

}  // namespace

struct cusync_attn_layer {
  cusync_attn_layer_config cfg;
  const void* wqkv;
  const void* wo;
  uint32_t E;                      // heads * head_dim
  int tile1, tile3;
  int split1, split3;              // k-slices of the two projections
  void* ws1;
  void* ws3;                       // their split-K workspaces (null without slices)
  uint32_t kvSplit;                // key/value blocks per attention workgroup, 0 = no split
  void* ws2;                       // workspace of the split attention
  cusync_stage_desc st[3];         // QKV projection, attention, output projection
  hipStream_t stream[3];
  hipEvent_t eStart, eMid1, eMid2, eEnd;
  uint32_t timeoutsSeen;           // sum of the stages' give-up counters when the last run returned
};

extern "C" void cusync_attn_layer_destroy(cusync_attn_layer* L);

// create() failed: gives back what the handle holds so far and keeps the text of the failure
static void discardLayer(cusync_attn_layer* L) {
  const std::string why = cusync_rt_last_error();
  cusync_attn_layer_destroy(L);
  cusync::rt::setError(why);
}

extern "C" {

int cusync_attention_tile_shape(uint32_t* tileM, uint32_t* tileN, uint32_t* blockKV) {
  if (tileM) *tileM = kBQ;
  if (tileN) *tileN = kHD;
  if (blockKV) *blockKV = kBKV;
  return 0;
}

cusync_dim3 cusync_attention_grid(uint32_t seq, uint32_t heads) {
  cusync_dim3 g = {heads, (seq + kBQ - 1) / kBQ, 1};
  return g;
}

cusync_dim3 cusync_attention_grid_split(uint32_t seq, uint32_t heads, uint32_t cached_rows, uint32_t kv_split_blocks) {
  cusync_dim3 g = cusync_attention_grid(seq, heads);
  if (kv_split_blocks) {
    const uint32_t blocks = (cached_rows + seq + kBKV - 1) / kBKV;
    g.z = std::max(1u, (blocks + kv_split_blocks - 1) / kv_split_blocks);
  }
  return g;
}

size_t cusync_attention_workspace_size(const cusync_attention_args* a) {
  if (!a || !a->kv_split_blocks) return 0;
  const cusync_dim3 g = cusync_attention_grid_split(a->seq, a->heads, a->cached_rows, a->kv_split_blocks);
  if (g.z <= 1) return 0;
  const size_t tiles = (size_t)g.x * g.y;
  return tiles * g.z * (64 + 2) * kThreads * sizeof(float) + tiles * sizeof(uint32_t);
}

cusync_error cusync_attention_can_implement(const cusync_attention_args* a) {
  if (!a) return CUSYNC_ERROR_NOT_INITIALIZED;
  if (!a->seq || !a->heads) { setError("attention: empty problem"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (a->head_dim != (uint32_t)kHD) { setError("attention: head width must be 128"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  const uint32_t E = a->heads * kHD;
  if (a->ldqkv < 3 * E || a->ldqkv % 8 || a->ldo < E || a->ldo % 4) { setError("attention: row pitch too small or misaligned"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if ((uint64_t)(a->seq + a->cached_rows) * a->ldqkv * 2 >= 0x80000000ull) { setError("attention: QKV larger than 2 GiB is not addressable by one buffer descriptor"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if ((uintptr_t)a->qkv % 16 || (uintptr_t)a->out % 8 || !a->qkv || !a->out) { setError("attention: misaligned operand"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  const cusync_dim3 g = cusync_attention_grid_split(a->seq, a->heads, a->cached_rows, a->kv_split_blocks);
  const cusync_stage_desc& s = a->stage;
  if (s.grid.x != g.x || s.grid.y != g.y || s.grid.z != g.z) { setError("attention: stage grid does not match cusync_attention_grid / cusync_attention_grid_split"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if ((uint64_t)a->seq * a->ldo * 2 >= 0x80000000ull || cusync_attention_workspace_size(a) >= 0x80000000ull) {
    setError("attention: output or workspace larger than 2 GiB is not addressable by one buffer descriptor");
    return CUSYNC_ERROR_NOT_INITIALIZED;
  }
  if (g.z > 1 && (!a->workspace || (uintptr_t)a->workspace % 16)) { setError("attention: a split key range needs a 16-byte aligned workspace of cusync_attention_workspace_size bytes"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (!s.tileOrder || !s.tileCounter || !s.startCounter || !s.spinTimeouts || !s.xcdTickets) { setError("attention: stage not allocated"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (s.out.kind != CUSYNC_POLICY_NOSYNC && !s.tileStatusWrite) { setError("attention: producer stage without semaphores"); return CUSYNC_ERROR_NOT_INITIALIZED; }
  if (s.in.kind != CUSYNC_POLICY_NOSYNC) {
    if (!s.tileStatusRead) { setError("attention: consumer stage not paired with a producer"); return CUSYNC_ERROR_NOT_INITIALIZED; }
    if (s.in.kind != CUSYNC_POLICY_ROWSYNC && s.in.kind != CUSYNC_POLICY_TILESYNC && s.in.kind != CUSYNC_POLICY_CONSECUTIVESYNC) {
      setError("attention: input policy must be RowSync, TileSync or ConsecutiveSync");
      return CUSYNC_ERROR_NOT_INITIALIZED;
    }
    if (s.in.tileM == 0 || s.in.tileN == 0) { setError("attention: input policy with zero tile extent"); return CUSYNC_ERROR_NOT_INITIALIZED; }
    if (s.in.kind == CUSYNC_POLICY_CONSECUTIVESYNC && (s.in.H / 8 != E || E % s.in.tileN)) {
      setError("attention: ConsecutiveSync must group exactly the Q, K and V column tiles (H/8 == heads*128)");
      return CUSYNC_ERROR_NOT_INITIALIZED;
    }
  }
  if ((s.opts & CUSYNC_OPT_NO_ATOMIC_ADD) && s.out.kind != CUSYNC_POLICY_NOSYNC &&
      cusync::dyn::waitValue(s.out) != cusync::dyn::postValue(s.out)) {
    setError("attention: NoAtomicAdd needs a policy whose wait value equals its post value");
    return CUSYNC_ERROR_NOT_INITIALIZED;
  }
  return CUSYNC_SUCCESS;
}

int cusync_attention_max_resident(void) { return residentAttention(false); }

cusync_error cusync_attention_run(const cusync_attention_args* a, void* stream) {
  cusync_error e = cusync_attention_can_implement(a);
  if (e != CUSYNC_SUCCESS) return e;
  const bool deep = deepPipeline(a);
  const int resident = residentAttention(deep);
  if (resident <= 0) { setError("attention: kernel does not fit on a CU"); return CUSYNC_ERROR_DEVICE; }
  const cusync_stage_desc& s = a->stage;
  uint32_t launched = std::min<uint32_t>(s.grid.x * s.grid.y * s.grid.z, (uint32_t)resident);
  if (a->max_workgroups > 0) launched = std::min<uint32_t>(launched, (uint32_t)a->max_workgroups);

  AttnParams p = {};
  p.stage.d = s;
  p.stage.lineAligned = !cusync::rt::forceAcquire() && s.in.kind != CUSYNC_POLICY_NOSYNC && (uintptr_t)a->qkv % 128 == 0 && (a->ldqkv * 2) % 128 == 0 &&
                        (s.in.kind != CUSYNC_POLICY_TILESYNC || (s.in.tileN * 2) % 128 == 0);
  p.stage.releaseAll = cusync::rt::forceRelease();
  p.S = a->seq; p.heads = a->heads; p.cached = a->cached_rows;
  p.qkv = (const half_t*)a->qkv; p.ldq = a->ldqkv;
  p.out = (half_t*)a->out; p.ldo = a->ldo;
  const float scale = a->scale > 0.0f ? a->scale : 1.0f / sqrtf((float)kHD);
  p.scaleLog2 = scale * 1.4426950408889634f;
  p.causal = a->causal ? 1 : 0;
  p.launched = launched;
  p.stage.prepare(launched);
  p.descending = p.causal;
  cusync::rt::timeline(&p.timeline, &p.timelineCap);
  if (s.grid.z > 1) {
    const size_t tiles = (size_t)s.grid.x * s.grid.y;
    p.chunk = a->kv_split_blocks;
    p.partO = (float*)a->workspace;
    p.partStat = p.partO + tiles * s.grid.z * 64 * kThreads;
    p.arrivals = (uint32_t*)(p.partStat + tiles * s.grid.z * 2 * kThreads);
    p.partBytes = (uint32_t)((char*)p.arrivals - (char*)p.partO);
  }
  // A consumer launch of no more workgroups than CUs asks for half a CU's LDS, so that the dispatcher spreads it one
  // to a CU instead of packing pairs onto the CUs its producer left free (see cusync_gemm_run): 1280 rows, 240
  // workgroups, 264 -> 244 us for the chain under every policy.  Not a launch of up to half as many workgroups as
  // CUs: packed, those are all resident beside the producer early and leave whole CUs to the output projection's
  // workgroups (512 rows, 96 workgroups: 124 us packed, 129 spread).
  int lds = attnLds(deep);
  if (s.in.kind != CUSYNC_POLICY_NOSYNC && !(s.opts & CUSYNC_OPT_AVOID_WAIT_KERNEL) && launched <= (uint32_t)g_attnNumCUs &&
      launched > (uint32_t)g_attnNumCUs / 2 && resident > g_attnNumCUs)
    lds = std::max(lds, g_attnLdsPerCU / 2);
  hipLaunchKernelGGL(attnKernel(deep), dim3(launched), dim3(kThreads), lds, (hipStream_t)stream, p);
  if (CUSYNC_HIP(hipGetLastError())) return CUSYNC_ERROR_DEVICE;
  cusync::rt::noteLaunch(s, launched >= (uint32_t)resident);
  return CUSYNC_SUCCESS;
}

/* ---- the chain ---------------------------------------------------------------- */

cusync_attn_layer* cusync_attn_layer_create(const cusync_attn_layer_config* cfg, const void* wqkv, const void* wo) {
  if (!cfg || !wqkv || !wo) { setError("attn layer: null argument"); return nullptr; }
  if (!cfg->seq || !cfg->hidden || !cfg->heads) { setError("attn layer: empty shape"); return nullptr; }
  if (cfg->head_dim != (uint32_t)kHD) { setError("attn layer: head width must be 128"); return nullptr; }
  cusync_attn_layer* L = new cusync_attn_layer();
  L->cfg = *cfg;
  L->wqkv = wqkv; L->wo = wo;
  L->E = cfg->heads * kHD;
  // Per-row-count choice, from the tuner's measurements (cusync_amd/tile_sizes_db.py, gpt3_attention_mi355x) and
  // sweeps between its row counts.  Widths that are multiples of 192 (4608 = 24 x 192, 12288 = 64 x 192) take the
  // 192-wide direct-to-LDS tiles.  QKV projection (24 column tiles): 64x192x64 in k-slices while the projection
  // streams the weights, up to 320 rows (five row tiles in two slices are 240 workgroups: 56 us against 69 for
  // 128x192); 128x192 with a CU to itself up to 1024 rows, except from 641 to 768 rows, which are three whole row
  // tiles of 256x192 in two slices (105 against 124 us); 256x192 above.  Output projection (64 column tiles):
  // 64x192x64 up to 256 rows, 128x192 alone up to 512, 256x192 up to 1024, and above that 128x192 at two workgroups
  // per CU, whose tiles fill the last round better (1280 rows: 79 -> 69 us, 1536: 80 -> 72, level at 2048).
  // Other widths: tiles that follow the row count up to 128 rows, 128x128 up to 1024 rows, 128x256 above.
  const int small = cfg->seq <= 32 ? CUSYNC_TILE_D32x128x64 : cfg->seq <= 64 ? CUSYNC_TILE_64x128x64 : CUSYNC_TILE_128x128x64;
  const int dflt = cfg->seq <= 128 ? small : cfg->seq <= 1024 ? CUSYNC_TILE_128x128x32 : CUSYNC_TILE_128x256x32;
  const uint32_t S = cfg->seq;
  // (with the 256x192 tile's K loop in assembly, 256x192 in k-slices also leads from 321 to 512 rows and from 769 to
  // 1024: the QKV projection 73 -> 67 us at 384 rows, 131 -> 115 at 896, 137 -> 120 at 1024; from 513 to 640 rows its
  // third row tile is mostly padding and 128x192 stays, 87 against 102 us)
  // (two full row tiles of 128, 193 to 256 rows: 128x192 with the operands fetched 64 columns of K at a time, the QKV
  // projection 55 -> 52 us at 256 rows, 51 -> 49.5 at 224; level below, and at 320 rows its third row tile costs 17 us)
  const int wide1 = S <= 32 ? small : S > 192 && S <= 256 && cfg->hidden % 64 == 0 ? CUSYNC_TILE_D128x192x64
                    : S <= 320 ? CUSYNC_TILE_D64x192x64 : S > 512 && S <= 640 ? CUSYNC_TILE_128x192x32_ALONE
                    : CUSYNC_TILE_256x192x32;
  const int wide3 = S <= 32 ? small : S <= 256 ? CUSYNC_TILE_D64x192x64 : S <= 512 ? CUSYNC_TILE_128x192x32_ALONE
                    : S <= 1024 ? CUSYNC_TILE_256x192x32 : CUSYNC_TILE_128x192x32;
  // (where K is a multiple of 64, the 256x192 tile that fetches both operands 64 columns at a time, K loop in assembly)
  auto inLines = [](int tile, uint32_t K) { return tile == CUSYNC_TILE_256x192x32 && K % 64 == 0 ? (int)CUSYNC_TILE_256x192x64 : tile; };
  L->tile1 = cfg->tile1 >= 0 ? cfg->tile1 : (3 * L->E) % 192 == 0 ? inLines(wide1, cfg->hidden) : dflt;
  L->tile3 = cfg->tile3 >= 0 ? cfg->tile3 : cfg->hidden % 192 == 0 ? inLines(wide3, L->E) : dflt;
  // (above 1024 rows the output projection's five to eight row tiles of 256x384, at most one per CU, beat 128x192 at
  // two workgroups per CU: the chain under RowSync 216 -> 212 us at 1280 rows, 267 -> 255 at 1536, 327 -> 311 at 2048)
  if (cfg->tile3 < 0 && S > 1024 && cfg->hidden % 384 == 0 && L->E % 64 == 0) L->tile3 = CUSYNC_TILE_256x384x32;
  L->ws1 = L->ws3 = L->ws2 = nullptr;
  // Key ranges of 8 blocks (512 rows) or more are cut in two: under a causal mask the last row tiles walk the
  // longest ranges and the launch is as long as its longest workgroup.  Measured alone at 12 heads: 512 rows
  // 26.7 -> 25.3 us, 1024 rows 37.8 -> 30.8 us, 2048 rows 61 -> 50 us; finer cuts lose again (2048 rows in four:
  // 62 us, in eight: 89 us): every cut adds a tile's fixed cost (first blocks, Q fragments, a pass over the
  // partial results) and tickets without work.
  const uint32_t kvBlocks = (cfg->cached_rows + cfg->seq + kBKV - 1) / kBKV;
  L->kvSplit = cfg->kv_split_blocks >= 0 ? (uint32_t)cfg->kv_split_blocks : kvBlocks >= 8 ? (kvBlocks + 1) / 2 : 0u;
  uint32_t tm1 = 0, tn1 = 0;
  if (cusync_gemm_tile_shape(L->tile1, &tm1, &tn1, nullptr) || cusync_gemm_tile_shape(L->tile3, nullptr, nullptr, nullptr)) {
    setError("attn layer: unknown tile id");
    discardLayer(L);
    return nullptr;
  }
  // few rows leave most CUs without a tile: k-slices as in the MLP chain
  uint32_t bk1 = 0, bk3 = 0;
  cusync_gemm_tile_shape(L->tile1, nullptr, nullptr, &bk1);
  cusync_gemm_tile_shape(L->tile3, nullptr, nullptr, &bk3);
  const cusync_dim3 flat1 = cusync_gemm_grid(L->tile1, cfg->seq, 3 * L->E, 1);
  const cusync_dim3 flat3 = cusync_gemm_grid(L->tile3, cfg->seq, cfg->hidden, 1);
  L->split1 = cusync::gemm::pickSplit(0, flat1.x * flat1.y, cfg->hidden, bk1, cusync_gemm_max_resident(L->tile1));
  L->split3 = cusync::gemm::pickSplit(0, flat3.x * flat3.y, L->E, bk3, cusync_gemm_max_resident(L->tile3));
  const cusync_dim3 g1 = cusync_gemm_grid(L->tile1, cfg->seq, 3 * L->E, L->split1);
  const cusync_dim3 g2 = cusync_attention_grid_split(cfg->seq, cfg->heads, cfg->cached_rows, L->kvSplit);
  const cusync_dim3 g3 = cusync_gemm_grid(L->tile3, cfg->seq, cfg->hidden, L->split3);

  cusync_policy_desc sync1 = noSync(), sync2 = noSync();
  int opts = 0;
  switch (cfg->sync) {
    case CUSYNC_SYNC_STREAM:
      break;
    case CUSYNC_SYNC_ROW:       // RowSync<kM> on both edges, attention.cu:84-90
      sync1.kind = CUSYNC_POLICY_ROWSYNC; sync1.order = CUSYNC_ORDER_TRANSPOSE_XY;
      sync1.tileM = tm1; sync1.tileN = 1; sync1.waitValue = g1.x; sync1.postValue = 1;
      sync2 = sync1;
      sync2.tileM = kBQ; sync2.waitValue = g2.x;
      opts = CUSYNC_OPT_REORDER_TILE_LOADS;      // defined for every policy, attention.cu:13
      break;
    case CUSYNC_SYNC_TILE:      // TileSync on both edges, attention.cu:91-97
      sync1.kind = CUSYNC_POLICY_TILESYNC; sync1.order = CUSYNC_ORDER_TRANSPOSE_XY;
      sync1.tileM = tm1; sync1.tileN = tn1; sync1.waitValue = 1; sync1.postValue = 1;
      sync2 = sync1;
      sync2.tileM = kBQ; sync2.tileN = kHD;
      opts = CUSYNC_OPT_NO_ATOMIC_ADD | CUSYNC_OPT_REORDER_TILE_LOADS;
      break;
    case CUSYNC_SYNC_STRIDED:   // ConsecutiveSync into the attention, RowSync out of it, attention.cu:98-110
      if (L->E % tn1) { setError("attn layer: ConsecutiveSync needs heads*128 % tileN == 0"); discardLayer(L); return nullptr; }
      sync1.kind = CUSYNC_POLICY_CONSECUTIVESYNC; sync1.order = CUSYNC_ORDER_TRANSPOSE_XY;
      sync1.tileM = tm1; sync1.tileN = tn1; sync1.H = 8 * L->E;
      sync1.waitValue = L->E / tn1; sync1.postValue = 1;
      sync2.kind = CUSYNC_POLICY_ROWSYNC; sync2.order = CUSYNC_ORDER_TRANSPOSE_XY;
      sync2.tileM = kBQ; sync2.tileN = 1; sync2.waitValue = g2.x; sync2.postValue = 1;
      opts = CUSYNC_OPT_REORDER_TILE_LOADS;
      break;
    default:
      setError("attn layer: unknown sync mode");
      discardLayer(L);
      return nullptr;
  }
  if (cfg->opts >= 0) opts |= cfg->opts;

  const cusync_dim3 grids[3] = {g1, g2, g3};
  const cusync_policy_desc ins[3] = {noSync(), sync1, sync2}, outs[3] = {sync1, sync2, noSync()};
  for (int i = 0; i < 3; i++) {
    memset(&L->st[i], 0, sizeof L->st[i]);
    L->st[i].grid = grids[i]; L->st[i].tileSize = {1, 1, 1}; L->st[i].iter = 1; L->st[i].opts = opts;
    L->st[i].in = ins[i]; L->st[i].out = outs[i];
    if (cusync_stage_create(&L->st[i], CUSYNC_ORDER_TRANSPOSE_XY) != CUSYNC_SUCCESS) { discardLayer(L); return nullptr; }
  }
  if (cfg->sync != CUSYNC_SYNC_STREAM &&
      (cusync_set_producer_consumer_pair(&L->st[0], &L->st[1]) != CUSYNC_SUCCESS ||
       cusync_set_producer_consumer_pair(&L->st[1], &L->st[2]) != CUSYNC_SUCCESS)) {
    setError("attn layer: pairing the stages failed");
    discardLayer(L);
    return nullptr;
  }
  for (int which = 0; which < 2; which++) {
    cusync_gemm_args a;
    memset(&a, 0, sizeof a);
    a.stage = L->st[which == 0 ? 0 : 2];
    a.M = cfg->seq; a.N = which == 0 ? 3 * L->E : cfg->hidden; a.K = which == 0 ? cfg->hidden : L->E;
    a.tile = which == 0 ? L->tile1 : L->tile3;
    a.split_k = which == 0 ? L->split1 : L->split3;
    const size_t bytes = cusync_gemm_workspace_size(&a);
    if (bytes == 0) continue;
    void* ws = nullptr;
    if (CUSYNC_HIP(hipMalloc(&ws, bytes)) || CUSYNC_HIP(hipMemset(ws, 0, bytes))) { discardLayer(L); return nullptr; }
    (which == 0 ? L->ws1 : L->ws3) = ws;
  }
  {
    cusync_attention_args a;
    memset(&a, 0, sizeof a);
    a.seq = cfg->seq; a.heads = cfg->heads; a.cached_rows = cfg->cached_rows; a.kv_split_blocks = L->kvSplit;
    const size_t bytes = cusync_attention_workspace_size(&a);
    if (bytes && (CUSYNC_HIP(hipMalloc(&L->ws2, bytes)) || CUSYNC_HIP(hipMemset(L->ws2, 0, bytes)))) { discardLayer(L); return nullptr; }
  }
  for (int i = 0; i < 3; i++)
    if (CUSYNC_HIP(hipStreamCreateWithFlags(&L->stream[i], hipStreamNonBlocking))) { discardLayer(L); return nullptr; }
  if (CUSYNC_HIP(hipEventCreate(&L->eStart)) || CUSYNC_HIP(hipEventCreate(&L->eMid1)) ||
      CUSYNC_HIP(hipEventCreate(&L->eMid2)) || CUSYNC_HIP(hipEventCreate(&L->eEnd))) { discardLayer(L); return nullptr; }
  return L;
}

// Also the clean-up of a create() that failed half way: the handle is value-initialised, so what has not
// been made yet is null and skipped.
void cusync_attn_layer_destroy(cusync_attn_layer* L) {
  if (!L) return;
  for (int i = 0; i < 3; i++) if (L->stream[i]) (void)hipStreamSynchronize(L->stream[i]);
  for (int i = 0; i < 3; i++) cusync_stage_free(&L->st[i]);
  for (hipEvent_t e : {L->eStart, L->eMid1, L->eMid2, L->eEnd}) if (e) (void)hipEventDestroy(e);
  for (int i = 0; i < 3; i++) if (L->stream[i]) (void)hipStreamDestroy(L->stream[i]);
  if (L->ws1) (void)hipFree(L->ws1);
  if (L->ws3) (void)hipFree(L->ws3);
  if (L->ws2) (void)hipFree(L->ws2);
  delete L;
}

cusync_error cusync_attn_layer_run(cusync_attn_layer* L, const void* x, void* qkv, void* o, void* y, int runs,
                                   double* times_us, double* stage_us) {
  if (!L || !x || !qkv || !o || !y) return CUSYNC_ERROR_NOT_INITIALIZED;
  const bool overlapped = L->cfg.sync != CUSYNC_SYNC_STREAM;
  const uint32_t S = L->cfg.seq, E = L->E, H = L->cfg.hidden;
  for (int r = 0; r < runs; r++) {
    cusync_gemm_args a1, a3;
    memset(&a1, 0, sizeof a1); memset(&a3, 0, sizeof a3);
    a1.stage = L->st[0]; a1.M = S; a1.N = 3 * E; a1.K = H;
    a1.A = x; a1.lda = H; a1.B = L->wqkv; a1.ldb = 3 * E; a1.ldd = 3 * E;
    a1.D = (char*)qkv + (size_t)L->cfg.cached_rows * 3 * E * 2;       // behind the cache rows (attention.cu:289)
    a1.tile = L->tile1; a1.split_k = L->split1; a1.workspace = L->ws1; a1.shared_reduction = 1;
    cusync_attention_args a2;
    memset(&a2, 0, sizeof a2);
    a2.stage = L->st[1]; a2.seq = S; a2.heads = L->cfg.heads; a2.head_dim = kHD;
    a2.qkv = qkv; a2.ldqkv = 3 * E; a2.out = o; a2.ldo = E; a2.scale = 0.0f; a2.causal = L->cfg.causal;
    a2.cached_rows = L->cfg.cached_rows;
    a2.kv_split_blocks = L->kvSplit; a2.workspace = L->ws2;
    a3.stage = L->st[2]; a3.M = S; a3.N = H; a3.K = E;
    a3.A = o; a3.lda = E; a3.B = L->wo; a3.ldb = H; a3.D = y; a3.ldd = H;
    a3.tile = L->tile3; a3.split_k = L->split3; a3.workspace = L->ws3; a3.shared_reduction = 1;

    hipStream_t s0 = L->stream[0], s1 = overlapped ? L->stream[1] : s0, s2 = overlapped ? L->stream[2] : s0;
    cusync_error e;
    if (CUSYNC_HIP(hipEventRecord(L->eStart, s0))) return CUSYNC_ERROR_DEVICE;
    if ((e = cusync_gemm_run(&a1, s0)) != CUSYNC_SUCCESS) return e;
    // overlapped: each consumer's stream is held back until every workgroup of its producer has started: from the
    // host when the producer's launch took every workgroup slot of the device (a wait kernel's wave would keep its
    // last workgroup off the device), by the wait kernel otherwise.  eMid1 / eMid2 only serve the stage timing.
    if (overlapped && (e = cusync_hold_back(&L->st[0], s1)) != CUSYNC_SUCCESS) return e;
    if (CUSYNC_HIP(hipEventRecord(L->eMid1, s1))) return CUSYNC_ERROR_DEVICE;
    if ((e = cusync_attention_run(&a2, s1)) != CUSYNC_SUCCESS) return e;
    if (overlapped) { if ((e = cusync_hold_back(&L->st[1], s2)) != CUSYNC_SUCCESS) return e; }
    else if (CUSYNC_HIP(hipEventRecord(L->eMid2, s0))) return CUSYNC_ERROR_DEVICE;
    if ((e = cusync_gemm_run(&a3, s2)) != CUSYNC_SUCCESS) return e;
    if (CUSYNC_HIP(hipEventRecord(L->eEnd, s2))) return CUSYNC_ERROR_DEVICE;
    if (CUSYNC_HIP(hipEventSynchronize(L->eEnd))) return CUSYNC_ERROR_DEVICE;
    if (overlapped && (CUSYNC_HIP(hipStreamSynchronize(s0)) || CUSYNC_HIP(hipStreamSynchronize(s1)))) return CUSYNC_ERROR_DEVICE;
    float ms = 0;
    if (times_us) {
      if (CUSYNC_HIP(hipEventElapsedTime(&ms, L->eStart, L->eEnd))) return CUSYNC_ERROR_DEVICE;
      times_us[r] = (double)ms * 1000.0;
    }
    if (!overlapped && stage_us) {
      hipEvent_t ev[4] = {L->eStart, L->eMid1, L->eMid2, L->eEnd};
      for (int i = 0; i < 3; i++) {
        if (CUSYNC_HIP(hipEventElapsedTime(&ms, ev[i], ev[i + 1]))) return CUSYNC_ERROR_DEVICE;
        stage_us[3 * r + i] = (double)ms * 1000.0;
      }
    }
    for (int i = 0; i < 3; i++) L->st[i].iter += 1;
  }
  // every run above was synchronised with; a wait that gave up let its kernel go on with unposted data
  const cusync_stage_desc* stages[3] = {&L->st[0], &L->st[1], &L->st[2]};
  return cusync::rt::checkSpinTimeouts(stages, 3, &L->timeoutsSeen, "attn layer");
}

const cusync_stage_desc* cusync_attn_layer_stage(const cusync_attn_layer* L, int which) {
  if (!L || which < 0 || which > 2) return nullptr;
  return &L->st[which];
}

int cusync_attn_layer_tiles(const cusync_attn_layer* L, int* tile1, int* tile3) {
  if (!L) return 1;
  if (tile1) *tile1 = L->tile1;
  if (tile3) *tile3 = L->tile3;
  return 0;
}

}  // extern "C"
