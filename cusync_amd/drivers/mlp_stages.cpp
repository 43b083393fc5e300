// The GPT-3 MLP wired the way the reference's driver wires it (src/ml-bench/transformer/mlp.cu): this file builds the
// two CuStage objects and the two CuSyncGemm launchers itself (:1020-1062), and runs the reference's loop (:645-716)
//
//     gemm_op1.run(true, NULL, producer_stream);
//     prod.invokeWaitKernel(consumer_stream);
//     gemm_op2.run(true, NULL, consumer_stream);
//     ... event wait ... prod.incrementIter(); cons.incrementIter(); and the launchers' copies
//
// on the public C++ headers (include/cusync/cusync.h, gemm.h), without the cusync_mlp_* handle.  Plain host C++.
// Tile shapes are template arguments of the launchers, as ThreadblockShape is in the reference, where a binary is
// built per batch size from tile_sizes_db.py; here one binary holds the pairs of the library's table
// (cusync_mlp_choice) and picks by batch size.
//
//   mlp_stages --batch <rows>[,<rows>...] [--sync rowsync|tilesync|both] [--runs n] [--rounds n] [--check true|false]
//              [--handle true|false] [--tile1 id --tile2 id] [--split-k1 n] [--split-k2 n] [--load dir] [--dump dir]
//
// --load: X, W1 and W2 come from dir/x.bin ([largest batch][12288]), w1.bin and w2.bin (raw fp16) instead of the
// driver's own random numbers; --dump: the launchers' H and Y of every batch size and policy go to
// dir/h_<rows>_<policy>.bin and y_<rows>_<policy>.bin.  Together they let a test hold the outputs against an oracle.
//
// Output per batch size and policy: START-OVERLAPPED: / one {"Total": us} per timed run / END-OVERLAPPED: as the
// reference prints them (mlp.cu:707, 1079-1084), then one summary object
//   {"batch", "sync", "tile1", "tile2", "split_k1", "split_k2", "launcher_us", "handle_us", "runs", "above_1p05"}
// (medians over all timed runs; handle_us: the cusync_mlp_* handle on the same buffers, its rounds of --runs runs
// alternating with the launchers' so that both see the same clocks; above_1p05: launcher runs slower than 1.05 x
// their median).
#include <algorithm>
#include <type_traits>

#include "cusync/cusync.h"
#include "cusync/gemm.h"
#include "driver_common.h"

namespace {

struct MLPParameters {           // mlp.cu:203-330: sizes and device tensors of one run
  int batch, hidden, inner;
  const cusync::half_bits *x, *w1, *w2;
  cusync::half_bits *xw1, *xw12;
  cusync::GemmCoord gemm_size1, gemm_size2;
  float alpha = 1.0f, beta = 0.0f;
};

std::vector<uint16_t> readHalfs(const std::string& path, size_t n) {
  std::vector<uint16_t> v(n);
  FILE* f = fopen(path.c_str(), "rb");
  if (!f || fread(v.data(), 2, n, f) != n) { fprintf(stderr, "cannot read %zu halfs from %s\n", n, path.c_str()); exit(EXIT_FAILURE); }
  fclose(f);
  return v;
}
void writeHalfs(const std::string& path, const std::vector<uint16_t>& v) {
  FILE* f = fopen(path.c_str(), "wb");
  if (!f || fwrite(v.data(), 2, v.size(), f) != v.size()) { fprintf(stderr, "cannot write %s\n", path.c_str()); exit(EXIT_FAILURE); }
  fclose(f);
}

double median(std::vector<double> v) {
  if (v.empty()) return 0;
  std::sort(v.begin(), v.end());
  return v.size() % 2 ? v[v.size() / 2] : 0.5 * (v[v.size() / 2 - 1] + v[v.size() / 2]);
}

#define STATUS_CHECK(call) do { cusync::Status s_ = (call); if (s_ != cusync::Status::kSuccess) { \
  fprintf(stderr, "%s:%d: %s (%s)\n", __FILE__, __LINE__, cusync::cusyncGetStatusString(s_), cusync_rt_last_error()); exit(EXIT_FAILURE); } } while (0)

// runCuSyncGPT3 of the reference (mlp.cu:645-716), its launchers kept alive between calls so that rounds can alternate.
template<typename GemmTy1, typename GemmTy2, typename ProdCuStage, typename ConsCuStage>
struct CuSyncGPT3 {
  GemmTy1 gemm_op1;
  GemmTy2 gemm_op2;
  void *workspace1 = nullptr, *workspace2 = nullptr;
  void *start = nullptr, *end = nullptr;
  ProdCuStage& prod;
  ConsCuStage& cons;

  CuSyncGPT3(int split_k1, int split_k2, MLPParameters& mlpParams, ProdCuStage& prod_, ConsCuStage& cons_) : prod(prod_), cons(cons_) {
    typename GemmTy1::Arguments args1{prod, mlpParams.gemm_size1, {mlpParams.x, mlpParams.hidden}, {mlpParams.w1, mlpParams.inner},
                                      {mlpParams.xw1, mlpParams.inner}, {mlpParams.xw1, mlpParams.inner},
                                      {mlpParams.alpha, mlpParams.beta}, split_k1};
    size_t workspace_size = GemmTy1::get_workspace_size(args1);
    if (workspace_size) RT_CHECK(cusync_rt_malloc(&workspace1, workspace_size));
    STATUS_CHECK(gemm_op1.can_implement(args1));
    STATUS_CHECK(gemm_op1.initialize(args1, workspace1));

    typename GemmTy2::Arguments args2{cons, mlpParams.gemm_size2, {mlpParams.xw1, mlpParams.inner}, {mlpParams.w2, mlpParams.hidden},
                                      {mlpParams.xw12, mlpParams.hidden}, {mlpParams.xw12, mlpParams.hidden},
                                      {mlpParams.alpha, mlpParams.beta}, split_k2};
    workspace_size = GemmTy2::get_workspace_size(args2);
    if (workspace_size) RT_CHECK(cusync_rt_malloc(&workspace2, workspace_size));
    STATUS_CHECK(gemm_op2.can_implement(args2));
    STATUS_CHECK(gemm_op2.initialize(args2, workspace2));
    RT_CHECK(cusync_rt_event_create(&start));
    RT_CHECK(cusync_rt_event_create(&end));
  }

  void run(void* producer_stream, void* consumer_stream, int iters, std::vector<double>* times) {
    for (int r = 0; r < iters; r++) {
      RT_CHECK(cusync_rt_event_record(start, producer_stream));
      STATUS_CHECK(gemm_op1.run(true, NULL, producer_stream));
      prod.invokeWaitKernel(consumer_stream);
      STATUS_CHECK(gemm_op2.run(true, NULL, consumer_stream));
      RT_CHECK(cusync_rt_event_record(end, consumer_stream));
      RT_CHECK(cusync_rt_event_sync(end));
      double us = 0;
      RT_CHECK(cusync_rt_event_elapsed_us(start, end, &us));
      if (times) times->push_back(us);
      prod.incrementIter();
      cons.incrementIter();
      gemm_op2.params_.custage.incrementIter();
      gemm_op1.params_.custage.incrementIter();
    }
  }

  ~CuSyncGPT3() {
    cusync_rt_device_sync();
    if (workspace1) cusync_rt_free(workspace1);
    if (workspace2) cusync_rt_free(workspace2);
    cusync_rt_event_destroy(start);
    cusync_rt_event_destroy(end);
  }
};

struct Request {
  bool row;
  int split_k1, split_k2, runs, rounds, warmup;
  bool withHandle;
};
struct Result { std::vector<double> launcher, handle; };

// The set-up of mlp.cu:1020-1062 for one pair of tile shapes and one policy.
template<int Tile1, int Tile2, bool Row>
Result runPair(MLPParameters& mlpParams, const Request& rq) {
  using ShapeThreadBlock1 = cusync::GemmTileShape<Tile1>;
  using TileOrder = cusync::TransposeXYOrder;
  using Sync = typename std::conditional<Row, cusync::RowSync<ShapeThreadBlock1::kM>,
                                         cusync::TileSync<TileOrder, ShapeThreadBlock1::kM, ShapeThreadBlock1::kN>>::type;
  // mlp.cu:9-16: ReorderTileLoads for every policy, NoAtomicAdd where a semaphore has one poster per run
  constexpr int Opts = Row ? (int)cusync::ReorderTileLoads : (int)cusync::NoAtomicAdd | (int)cusync::ReorderTileLoads;
  using ProdCuStage = cusync::CuStage<TileOrder, cusync::NoSync, Sync, Opts>;
  using ConsCuStage = cusync::CuStage<TileOrder, Sync, cusync::NoSync, Opts>;
  using GemmTy1 = cusync::CuSyncGemm<ProdCuStage, Tile1, CUSYNC_EPILOGUE_GELU>;
  using GemmTy2 = cusync::CuSyncGemm<ConsCuStage, Tile2, CUSYNC_EPILOGUE_NONE>;

  const dim3 gridDim1 = GemmTy1::get_grid_shape(mlpParams.gemm_size1, rq.split_k1);
  const dim3 gridDim2 = GemmTy2::get_grid_shape(mlpParams.gemm_size2, rq.split_k2);
  Sync sync;
  if constexpr (Row) sync = Sync(gridDim1.x);         // RowSync(gridDim1.n()): every column tile of the row posts once

  void *producer_stream = nullptr, *consumer_stream = nullptr;
  RT_CHECK(cusync_rt_stream_create(&producer_stream));
  RT_CHECK(cusync_rt_stream_create(&consumer_stream));

  ProdCuStage prod(gridDim1, {1, 1, 1}, cusync::NoSync(), sync);
  ConsCuStage cons(gridDim2, {1, 1, 1}, sync, cusync::NoSync());
  if (cusync::CuSync::setProducerConsumerPair(prod, cons) != cusync::CuSyncSuccess) { fprintf(stderr, "pairing the stages failed\n"); exit(EXIT_FAILURE); }

  Result out;
  {
    CuSyncGPT3<GemmTy1, GemmTy2, ProdCuStage, ConsCuStage> chain(rq.split_k1, rq.split_k2, mlpParams, prod, cons);
    cusync_mlp* handle = nullptr;
    if (rq.withHandle) {
      cusync_mlp_config c;
      memset(&c, 0, sizeof c);
      c.model = CUSYNC_MLP_GPT3; c.batch = (uint32_t)mlpParams.batch; c.hidden = (uint32_t)mlpParams.hidden; c.inner = (uint32_t)mlpParams.inner;
      c.sync = Row ? CUSYNC_SYNC_ROW : CUSYNC_SYNC_TILE;
      c.tile1 = Tile1; c.tile2 = Tile2; c.opts = -1; c.activation = 1; c.split_k1 = rq.split_k1; c.split_k2 = rq.split_k2;
      handle = cusync_mlp_create(&c, mlpParams.w1, mlpParams.w2);
      if (!handle) { fprintf(stderr, "cusync_mlp_create failed: %s\n", cusync_rt_last_error()); exit(EXIT_FAILURE); }
      DRV_CHECK(cusync_mlp_run(handle, mlpParams.x, mlpParams.xw1, mlpParams.xw12, rq.warmup, nullptr));
    }
    chain.run(producer_stream, consumer_stream, rq.warmup, nullptr);
    std::vector<double> t(rq.runs);
    for (int round = 0; round < rq.rounds; round++) {
      if (handle) {
        DRV_CHECK(cusync_mlp_run(handle, mlpParams.x, mlpParams.xw1, mlpParams.xw12, rq.runs, t.data()));
        out.handle.insert(out.handle.end(), t.begin(), t.end());
      }
      chain.run(producer_stream, consumer_stream, rq.runs, &out.launcher);       // last: what --check reads is the launchers' output
    }
    if (handle) cusync_mlp_destroy(handle);
  }
  uint32_t gaveUp = 0;
  const cusync_stage_desc dc = cons.desc();
  DRV_CHECK(cusync_stage_read_state(&dc, nullptr, nullptr, nullptr, nullptr, nullptr, &gaveUp));
  if (gaveUp) { fprintf(stderr, "%u waits of the consumer gave up\n", gaveUp); exit(EXIT_FAILURE); }
  prod.destroy();
  cons.destroy();
  cusync_rt_stream_destroy(producer_stream);
  cusync_rt_stream_destroy(consumer_stream);
  return out;
}

// The pairs of tile shapes this binary holds: what the library's table takes for the GPT-3 shard from 1 to 2048
// rows and beyond, and the 32-column forms of the large tiles.
#define FOR_EACH_PAIR(X)                                                                                         \
  X(CUSYNC_TILE_D32x128x64, CUSYNC_TILE_D32x128x64) X(CUSYNC_TILE_D64x192x64, CUSYNC_TILE_D64x192x64)           \
  X(CUSYNC_TILE_128x192x32, CUSYNC_TILE_128x192x32) X(CUSYNC_TILE_128x192x32_ALONE, CUSYNC_TILE_128x192x32_ALONE) \
  X(CUSYNC_TILE_256x192x64, CUSYNC_TILE_256x192x64) X(CUSYNC_TILE_256x192x64, CUSYNC_TILE_128x192x32)           \
  X(CUSYNC_TILE_256x192x64, CUSYNC_TILE_256x384x32) X(CUSYNC_TILE_256x192x32, CUSYNC_TILE_256x192x32)           \
  X(CUSYNC_TILE_256x192x32, CUSYNC_TILE_256x384x32) X(CUSYNC_TILE_128x128x64, CUSYNC_TILE_128x128x64)           \
  X(CUSYNC_TILE_D128x192x64, CUSYNC_TILE_D128x192x64)

bool dispatch(int tile1, int tile2, MLPParameters& p, const Request& rq, Result* out) {
#define TRY_PAIR(A, B) \
  if (tile1 == A && tile2 == B) { *out = rq.row ? runPair<A, B, true>(p, rq) : runPair<A, B, false>(p, rq); return true; }
  FOR_EACH_PAIR(TRY_PAIR)
#undef TRY_PAIR
  return false;
}

bool shapesAgree() {          // the compile-time shapes against the library's
  bool ok = true;
#define CHECK_SHAPE(A, B) { uint32_t m = 0, n = 0, k = 0; \
    ok = ok && cusync_gemm_tile_shape(A, &m, &n, &k) == 0 && m == cusync::GemmTileShape<A>::kM && n == cusync::GemmTileShape<A>::kN && k == cusync::GemmTileShape<A>::kK; \
    ok = ok && cusync_gemm_tile_shape(B, &m, &n, &k) == 0 && m == cusync::GemmTileShape<B>::kM && n == cusync::GemmTileShape<B>::kN && k == cusync::GemmTileShape<B>::kK; }
  FOR_EACH_PAIR(CHECK_SHAPE)
#undef CHECK_SHAPE
  return ok;
}

}  // namespace

int main(int argc, char** argv) {
  auto args = drv::parseArgs(argc, argv);
  std::vector<int> batches;
  {
    const std::string list = drv::get(args, "batch", "");
    size_t pos = 0;
    while (pos < list.size()) {
      const size_t comma = std::min(list.find(',', pos), list.size());
      const int b = atoi(list.substr(pos, comma - pos).c_str());
      if (b <= 0) { batches.clear(); break; }
      batches.push_back(b);
      pos = comma + 1;
    }
  }
  const std::string syncName = drv::get(args, "sync", "both");
  if (batches.empty() || (syncName != "rowsync" && syncName != "tilesync" && syncName != "both")) {
    fprintf(stderr, "usage: mlp_stages --batch <int>[,<int>...] [--sync rowsync|tilesync|both] [--runs <int>] [--rounds <int>] "
                    "[--check true|false] [--handle true|false] [--tile1 <id> --tile2 <id>] [--split-k1 <int>] [--split-k2 <int>] [--load <dir>] [--dump <dir>]\n");
    return EXIT_FAILURE;
  }
  if (!shapesAgree()) { fprintf(stderr, "cusync/gemm.h and the library disagree on a tile shape\n"); return EXIT_FAILURE; }
  const bool check = drv::getBool(args, "check", false);
  const int hidden = 12288, inner = 6144;      // GPT-3 175B, 4H/8 columns per GPU (mlp.cu:244-246)
  const int maxBatch = *std::max_element(batches.begin(), batches.end());

  const std::string load = drv::get(args, "load", ""), dump = drv::get(args, "dump", "");
  auto xh = load.empty() ? drv::uniformHalf((size_t)maxBatch * hidden, 1) : readHalfs(load + "/x.bin", (size_t)maxBatch * hidden);
  auto w1h = load.empty() ? drv::normalHalf((size_t)hidden * inner, 2, 0.02f) : readHalfs(load + "/w1.bin", (size_t)hidden * inner);
  auto w2h = load.empty() ? drv::normalHalf((size_t)inner * hidden, 3, 0.02f) : readHalfs(load + "/w2.bin", (size_t)inner * hidden);
  void *x = drv::toDevice(xh), *w1 = drv::toDevice(w1h), *w2 = drv::toDevice(w2h);
  void *h = drv::deviceBuffer((size_t)maxBatch * inner), *y = drv::deviceBuffer((size_t)maxBatch * hidden);

  for (int batch : batches) {
    for (int rowFirst = 1; rowFirst >= 0; rowFirst--) {
      const bool row = rowFirst == 1;
      if ((row && syncName == "tilesync") || (!row && syncName == "rowsync")) continue;
      MLPParameters p;
      p.batch = batch; p.hidden = hidden; p.inner = inner;
      p.x = (const cusync::half_bits*)x; p.w1 = (const cusync::half_bits*)w1; p.w2 = (const cusync::half_bits*)w2;
      p.xw1 = (cusync::half_bits*)h; p.xw12 = (cusync::half_bits*)y;
      p.gemm_size1 = cusync::GemmCoord(batch, inner, hidden);
      p.gemm_size2 = cusync::GemmCoord(batch, hidden, inner);

      cusync_mlp_config c;
      memset(&c, 0, sizeof c);
      c.model = CUSYNC_MLP_GPT3; c.batch = (uint32_t)batch; c.hidden = hidden; c.inner = inner;
      c.sync = row ? CUSYNC_SYNC_ROW : CUSYNC_SYNC_TILE;
      c.tile1 = (int)drv::getInt(args, "tile1", -1); c.tile2 = (int)drv::getInt(args, "tile2", -1); c.opts = -1; c.activation = 1;
      c.split_k1 = (int)drv::getInt(args, "split-k1", 0); c.split_k2 = (int)drv::getInt(args, "split-k2", 0);
      int tile1 = 0, tile2 = 0;
      Request rq;
      rq.row = row;
      if (cusync_mlp_choice(&c, &tile1, &tile2, &rq.split_k1, &rq.split_k2, nullptr) != 0) { fprintf(stderr, "no shapes for %d rows: %s\n", batch, cusync_rt_last_error()); return EXIT_FAILURE; }
      rq.runs = (int)drv::getInt(args, "runs", 20); rq.rounds = (int)drv::getInt(args, "rounds", 1); rq.warmup = 10;
      rq.withHandle = drv::getBool(args, "handle", true);

      RT_CHECK(cusync_rt_memset(h, 0, (size_t)maxBatch * inner * 2));
      RT_CHECK(cusync_rt_memset(y, 0, (size_t)maxBatch * hidden * 2));
      Result res;
      if (!dispatch(tile1, tile2, p, rq, &res)) {
        fprintf(stderr, "tile pair (%d, %d) is not among the launchers compiled into this driver\n", tile1, tile2);
        return EXIT_FAILURE;
      }
      printf("START-OVERLAPPED:\n");
      for (double t : res.launcher) printf("{\"Total\": %lf}\n", t);
      printf("END-OVERLAPPED:\n");
      const double med = median(res.launcher);
      int above = 0;
      for (double t : res.launcher) above += t > 1.05 * med;
      printf("{\"batch\": %d, \"sync\": \"%s\", \"tile1\": %d, \"tile2\": %d, \"split_k1\": %d, \"split_k2\": %d, \"launcher_us\": %.2f, "
             "\"handle_us\": %s, \"runs\": %zu, \"above_1p05\": %d}\n", batch, row ? "rowsync" : "tilesync", tile1, tile2, rq.split_k1, rq.split_k2,
             med, res.handle.empty() ? "null" : std::to_string(median(res.handle)).c_str(), res.launcher.size(), above);
      fflush(stdout);

      if (!dump.empty()) {
        const std::string tag = std::to_string(batch) + (row ? "_rowsync.bin" : "_tilesync.bin");
        writeHalfs(dump + "/h_" + tag, drv::toHost(h, (size_t)batch * inner));
        writeHalfs(dump + "/y_" + tag, drv::toHost(y, (size_t)batch * hidden));
      }
      if (check) {
        // rows 0, batch/2 and batch-1 of both outputs against the host GEMM, GeLU applied as the kernel does
        auto hh = drv::toHost(h, (size_t)batch * inner), yh = drv::toHost(y, (size_t)batch * hidden);
        size_t bad = 0;
        for (long r : {0L, (long)batch / 2, (long)batch - 1}) {
          auto ref1 = drv::gemmRow(&xh[(size_t)r * hidden], w1h, hidden, inner);
          for (size_t j = 0; j < (size_t)inner; j++) {
            const float v = 0.5f * ref1[j] * (1.0f + erff(ref1[j] * 0.70710678f));
            if (!drv::closeEnough(drv::h2f(hh[(size_t)r * inner + j]), v, 1e-2f)) bad++;
          }
          auto ref2 = drv::gemmRow(&hh[(size_t)r * inner], w2h, inner, hidden);
          for (size_t j = 0; j < (size_t)hidden; j++)
            if (!drv::closeEnough(drv::h2f(yh[(size_t)r * hidden + j]), ref2[j], 1e-2f)) bad++;
        }
        printf(bad ? "check: %zu mismatches\n" : "check: passed\n", bad);
        if (bad) return EXIT_FAILURE;
      }
    }
  }
  for (void* p : {x, w1, w2, h, y}) cusync_rt_free(p);
  return 0;
}
