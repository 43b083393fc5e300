// Self-attention benchmark driver with the command line and output protocol of the reference's
// src/ml-bench/transformer/attention.cu (:874-1075).
//
//   attention --model gpt3|llama --batch <new rows> [--seqlen <cached rows>] [--check true|false]
//             [--sync rowsync|tilesync|stridedsync] [--runs n]
//
// --batch rows are projected to Q|K|V behind --seqlen cached rows (attention.cu:265-276), attend causally to
// all of them, and go through the output projection.  Output: START-BASELINE: / END-BASELINE: {json}
// microseconds, START-OVERLAPPED / END-OVERLAPPED: {json} microseconds (attention.cu:1005-1010, 1066-1069).
// The reference's four GEMM times become three stage times: its matmul2 and matmul3 are one fused kernel here.
#include "driver_common.h"

int main(int argc, char** argv) {
  auto args = drv::parseArgs(argc, argv);
  const std::string model = drv::get(args, "model", "");
  const long batch = drv::getInt(args, "batch", 0), seqlen = drv::getInt(args, "seqlen", 0);
  if ((model != "gpt3" && model != "llama") || batch <= 0 || seqlen < 0) {
    fprintf(stderr, "usage: attention --model gpt3|llama --batch <int> [--seqlen <int>] [--check true|false] "
                    "[--sync rowsync|tilesync|stridedsync] [--runs <int>]\n");
    return EXIT_FAILURE;
  }
  const std::string syncName = drv::get(args, "sync", "tilesync");
  const bool check = drv::getBool(args, "check", false);
  const int runs = (int)drv::getInt(args, "runs", 20), warmup = 10;
  const uint32_t hidden = model == "llama" ? 8192 : 12288, e = hidden / 8, heads = e / 128;   // H/8 columns per GPU
  int sync = CUSYNC_SYNC_TILE;
  if (syncName == "rowsync") sync = CUSYNC_SYNC_ROW;
  else if (syncName == "stridedsync") sync = CUSYNC_SYNC_STRIDED;
  else if (syncName != "tilesync") { fprintf(stderr, "unknown --sync %s\n", syncName.c_str()); return EXIT_FAILURE; }
  printf("model=%s batch=%ld seqlen=%ld check=%d sync=%s\n", model.c_str(), batch, seqlen, (int)check, syncName.c_str());

  auto xh = drv::uniformHalf((size_t)batch * hidden, 1);
  auto wqkvh = drv::normalHalf((size_t)hidden * 3 * e, 2, 0.02f);
  auto woh = drv::normalHalf((size_t)e * hidden, 3, 0.02f);
  auto cacheh = drv::normalHalf((size_t)seqlen * 3 * e, 4, 1.0f);
  cacheh.resize((size_t)(seqlen + batch) * 3 * e, 0);
  void *x = drv::toDevice(xh), *wqkv = drv::toDevice(wqkvh), *wo = drv::toDevice(woh), *qkv = drv::toDevice(cacheh);
  void *o = drv::deviceBuffer((size_t)batch * e), *y = drv::deviceBuffer((size_t)batch * hidden);

  auto runMode = [&](int mode, std::vector<double>* stages) {
    cusync_attn_layer_config c;
    memset(&c, 0, sizeof c);
    c.seq = (uint32_t)batch; c.hidden = hidden; c.heads = heads; c.head_dim = 128; c.sync = mode;
    c.tile1 = c.tile3 = -1; c.opts = -1; c.causal = 1; c.cached_rows = (uint32_t)seqlen; c.kv_split_blocks = -1;
    cusync_attn_layer* l = cusync_attn_layer_create(&c, wqkv, wo);
    if (!l) { fprintf(stderr, "cusync_attn_layer_create failed: %s\n", cusync_rt_last_error()); exit(EXIT_FAILURE); }
    DRV_CHECK(cusync_attn_layer_run(l, x, qkv, o, y, warmup, nullptr, nullptr));
    std::vector<double> t(runs), st(3 * (size_t)runs, 0.0);
    DRV_CHECK(cusync_attn_layer_run(l, x, qkv, o, y, runs, t.data(), st.data()));
    if (stages) {
      stages->assign(3, 0.0);
      for (int r = 0; r < runs; r++) for (int i = 0; i < 3; i++) (*stages)[i] += st[3 * r + i] / runs;
    }
    cusync_attn_layer_destroy(l);
    return drv::mean(t);
  };

  std::vector<double> st;
  printf("START-BASELINE:\n");
  const double base = runMode(CUSYNC_SYNC_STREAM, &st);
  printf("END-BASELINE: {\"Total\": %lf, \"matmul1Time\": %lf, \"attentionTime\": %lf, \"matmul4Time\": %lf} microseconds\n", base, st[0], st[1], st[2]);
  printf("START-OVERLAPPED\n");
  const double over = runMode(sync, nullptr);
  printf("END-OVERLAPPED: {\"Total\": %lf} microseconds\n", over);
  printf("gain %.2f %%\n", 100.0 - over / base * 100.0);

  if (check) {
    // last new row: projection, attention over every visible row, output projection, each on what the GPU produced before it
    auto qkvh = drv::toHost(qkv, (size_t)(seqlen + batch) * 3 * e), oh = drv::toHost(o, (size_t)batch * e), yh = drv::toHost(y, (size_t)batch * hidden);
    const size_t r = batch - 1, row = seqlen + r;
    size_t bad = 0;
    auto ref = drv::gemmRow(&xh[r * hidden], wqkvh, hidden, 3 * e);
    for (size_t j = 0; j < 3 * e; j++) if (!drv::closeEnough(drv::h2f(qkvh[row * 3 * e + j]), ref[j], 1e-2f)) bad++;
    for (uint32_t hd = 0; hd < heads; hd++) {
      std::vector<float> p(row + 1);
      float mx = -INFINITY, sum = 0;
      for (size_t j = 0; j <= row; j++) {
        float s = 0;
        for (int c = 0; c < 128; c++) s += drv::h2f(qkvh[row * 3 * e + hd * 128 + c]) * drv::h2f(qkvh[j * 3 * e + e + hd * 128 + c]);
        p[j] = s / sqrtf(128.0f);
        mx = fmaxf(mx, p[j]);
      }
      for (auto& v : p) { v = expf(v - mx); sum += v; }
      for (int c = 0; c < 128; c++) {
        float acc = 0;
        for (size_t j = 0; j <= row; j++) acc += p[j] / sum * drv::h2f(qkvh[j * 3 * e + 2 * e + hd * 128 + c]);
        if (!drv::closeEnough(drv::h2f(oh[r * e + hd * 128 + c]), acc, 1e-2f)) bad++;
      }
    }
    auto ref3 = drv::gemmRow(&oh[r * e], woh, e, hidden);
    for (size_t j = 0; j < hidden; j++) if (!drv::closeEnough(drv::h2f(yh[r * hidden + j]), ref3[j], 1e-2f)) bad++;
    printf(bad ? "check: %zu mismatches\n" : "check: passed\n", bad);
    if (bad) return EXIT_FAILURE;
  }
  for (void* p : {x, wqkv, wo, qkv, o, y}) cusync_rt_free(p);
  return 0;
}
