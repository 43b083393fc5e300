// MLP benchmark driver with the command line and output protocol of the reference's
// src/ml-bench/transformer/mlp.cu (:876-1120): stream-ordered baseline, then the CuSync chain.
//
//   mlp --model gpt3|llama --batch <rows> [--check true|false] [--split-k1 n] [--split-k2 n]
//       [--policy baseline|cusync|both] [--sync rowsync|tilesync|stridedsync] [--runs n]
//       [--repack-weights true|false] [--one-launch true|false]
//
// --repack-weights: both chains read padded copies of the weights kept by the handle
// (cusync_mlp_config.repack_weights); --one-launch: the CuSync chain runs both GEMMs in one launch (true), in one
// launch each (false), or, when the option is not given, as the library's table says for the batch size.
//
// Output: "START-BASELINE:", one JSON object per timed run {"Total", "matmul1Time", "matmul2Time"} in
// microseconds, "END-BASELINE:", then the same between START-OVERLAPPED: / END-OVERLAPPED: with {"Total"}
// (mlp.cu:485, 707, 989-993, 1079-1084).  The synchronisation policy, a compile-time macro in the reference
// (ROWSYNC / TILESYNC / STRIDEDSYNC), is the --sync option here.
#include "driver_common.h"

int main(int argc, char** argv) {
  auto args = drv::parseArgs(argc, argv);
  const std::string model = drv::get(args, "model", "");
  const long batch = drv::getInt(args, "batch", 0);
  if ((model != "gpt3" && model != "llama") || batch <= 0) {
    fprintf(stderr, "usage: mlp --model gpt3|llama --batch <int> [--check true|false] [--split-k1 <int>] [--split-k2 <int>] "
                    "[--policy baseline|cusync|both] [--sync rowsync|tilesync|stridedsync] [--runs <int>] "
                    "[--repack-weights true|false] [--one-launch true|false]\n");
    return EXIT_FAILURE;
  }
  const bool check = drv::getBool(args, "check", false);
  const std::string policy = drv::get(args, "policy", "both");
  const std::string syncName = drv::get(args, "sync", model == "llama" ? "stridedsync" : "tilesync");
  const int runs = (int)drv::getInt(args, "runs", 20), warmup = 10;
  const bool llama = model == "llama";
  // GPT-3 175B: H = 12288, 4H/8 columns per GPU; LLaMA 65.2B: H = 8192, d = 2816 = ((8192/3 + 127)/128)*128 (mlp.cu:244-250)
  const uint32_t hidden = llama ? 8192 : 12288, inner = llama ? 2816 : 6144, n1 = llama ? 2 * inner : inner;
  int sync = CUSYNC_SYNC_TILE;
  if (syncName == "rowsync") sync = CUSYNC_SYNC_ROW;
  else if (syncName == "stridedsync") sync = CUSYNC_SYNC_STRIDED;
  else if (syncName != "tilesync") { fprintf(stderr, "unknown --sync %s\n", syncName.c_str()); return EXIT_FAILURE; }
  printf("model=%s batch=%ld check=%d sync=%s\n", model.c_str(), batch, (int)check, syncName.c_str());

  auto xh = drv::uniformHalf((size_t)batch * hidden, 1);
  auto w1h = drv::normalHalf((size_t)hidden * n1, 2, 0.02f);
  auto w2h = drv::normalHalf((size_t)inner * hidden, 3, 0.02f);
  void *x = drv::toDevice(xh), *w1 = drv::toDevice(w1h), *w2 = drv::toDevice(w2h);
  void *h = drv::deviceBuffer((size_t)batch * n1), *y = drv::deviceBuffer((size_t)batch * hidden);

  auto runMode = [&](int mode, const char* tag, bool split) {
    cusync_mlp_config c;
    memset(&c, 0, sizeof c);
    c.model = llama ? CUSYNC_MLP_LLAMA : CUSYNC_MLP_GPT3;
    c.batch = (uint32_t)batch; c.hidden = hidden; c.inner = inner; c.sync = mode;
    c.tile1 = c.tile2 = -1; c.opts = -1;
    c.activation = llama ? 0 : 1;        // the reference's LLaMA chain multiplies the gate half as is (mlp.cu:785-792)
    c.split_k1 = (int)drv::getInt(args, "split-k1", 0); c.split_k2 = (int)drv::getInt(args, "split-k2", 0);
    c.repack_weights = drv::getBool(args, "repack-weights", false) ? 1 : 0;
    c.one_launch = mode == CUSYNC_SYNC_STREAM ? 0 : !args.count("one-launch") ? -1 : drv::getBool(args, "one-launch", false) ? 1 : 0;      // not given: the library picks
    cusync_mlp* m = cusync_mlp_create(&c, w1, w2);
    if (!m) { fprintf(stderr, "cusync_mlp_create failed: %s\n", cusync_rt_last_error()); exit(EXIT_FAILURE); }
    DRV_CHECK(cusync_mlp_run(m, x, h, y, warmup, nullptr));
    std::vector<double> t(runs), g1(runs), g2(runs);
    printf("START-%s:\n", tag);
    DRV_CHECK(cusync_mlp_run_split(m, x, h, y, runs, t.data(), g1.data(), g2.data()));
    for (int i = 0; i < runs; i++) {
      if (split) printf("{\"Total\": %lf, \"matmul1Time\": %lf, \"matmul2Time\": %lf}\n", t[i], g1[i], g2[i]);
      else printf("{\"Total\": %lf}\n", t[i]);
    }
    printf("END-%s:\n", tag);
    cusync_mlp_destroy(m);
    return drv::mean(t);
  };

  double base = 0, over = 0;
  if (policy == "baseline" || policy == "both") base = runMode(CUSYNC_SYNC_STREAM, "BASELINE", true);
  if (policy == "cusync" || policy == "both") over = runMode(sync, "OVERLAPPED", false);
  if (base > 0 && over > 0) printf("baseline %.2f us, %s %.2f us, gain %.2f %%\n", base, syncName.c_str(), over, 100.0 - over / base * 100.0);

  if (check) {
    // rows 0, batch/2 and batch-1 against the host GEMM (linear epilogue only in the reference's check, mlp.cu:333-399;
    // here GeLU is applied as the kernel does)
    auto hh = drv::toHost(h, (size_t)batch * n1), yh = drv::toHost(y, (size_t)batch * hidden);
    size_t bad = 0;
    for (long r : {0L, batch / 2, batch - 1}) {
      auto ref1 = drv::gemmRow(&xh[(size_t)r * hidden], w1h, hidden, n1);
      for (size_t j = 0; j < n1; j++) {
        float v = ref1[j];
        if (!llama) v = 0.5f * v * (1.0f + erff(v * 0.70710678f));
        if (!drv::closeEnough(drv::h2f(hh[(size_t)r * n1 + j]), v, 1e-2f)) bad++;
      }
      // second GEMM on the intermediate the GPU produced (LLaMA: its first `inner` columns)
      std::vector<uint16_t> arow(hh.begin() + (size_t)r * n1, hh.begin() + (size_t)r * n1 + inner);
      auto ref2 = drv::gemmRow(arow.data(), w2h, inner, hidden);
      for (size_t j = 0; j < hidden; j++)
        if (!drv::closeEnough(drv::h2f(yh[(size_t)r * hidden + j]), ref2[j], 1e-2f)) bad++;
    }
    printf(bad ? "check: %zu mismatches\n" : "check: passed\n", bad);
    if (bad) return EXIT_FAILURE;
  }
  for (void* p : {x, w1, w2, h, y}) cusync_rt_free(p);
  return 0;
}
