// Convolution-chain benchmark driver after the reference's src/ml-bench/volta_conv2d/resnet.cu and vgg.cu
// (options :309-345, output :754-759, 825-827).
//
//   resnet --n 32 --h 56 --w 56 --c 64 [--layers 2] [--iterations 20] [--ref-check] [--sync rowsync|tilesync]
//          [--split_k_slices n]
//
// `layers` 3x3 convolutions with c input and c output channels (2 = the ResNet block, 4 = the VGG block),
// NHWC fp16, ReLU between the layers.  Output: START-BASELINE: / END-BASELINE: {Total, Conv1, ...} micro seconds,
// START-OVERLAP: / END-OVERLAP {Total} micro seconds.
#include "driver_common.h"

int main(int argc, char** argv) {
  auto args = drv::parseArgs(argc, argv);
  if (args.count("help")) {
    printf("resnet --n <int> --h <int> --w <int> --c <int> [--layers <int>] [--iterations <int>] [--ref-check] [--sync rowsync|tilesync] [--split_k_slices <int>]\n");
    return 0;
  }
  const uint32_t n = (uint32_t)drv::getInt(args, "n", 32), h = (uint32_t)drv::getInt(args, "h", 56), w = (uint32_t)drv::getInt(args, "w", 56),
                 c = (uint32_t)drv::getInt(args, "c", 64), layers = (uint32_t)drv::getInt(args, "layers", 2);
  const int runs = (int)drv::getInt(args, "iterations", 20), warmup = 10;
  const bool check = drv::getBool(args, "ref-check", false);
  const int splitK = (int)drv::getInt(args, "split_k_slices", 0);      // 0: the library picks (the reference's default is none)
  const std::string syncName = drv::get(args, "sync", "tilesync");
  const int sync = syncName == "rowsync" ? CUSYNC_SYNC_ROW : CUSYNC_SYNC_TILE;
  if (layers < 1 || layers > 16) { fprintf(stderr, "--layers must be 1..16\n"); return EXIT_FAILURE; }
  printf("n=%u h=%u w=%u c=%u layers=%u sync=%s\n", n, h, w, c, layers, syncName.c_str());

  const size_t pixels = (size_t)n * h * w;
  auto xh = drv::uniformHalf(pixels * c, 1);
  std::vector<std::vector<uint16_t>> wh;
  std::vector<const void*> wd;
  std::vector<void*> yd;
  for (uint32_t i = 0; i < layers; i++) {
    wh.push_back(drv::normalHalf((size_t)c * 9 * c, 2 + i, sqrtf(2.0f / (9.0f * c))));
    wd.push_back(drv::toDevice(wh.back()));
    yd.push_back(drv::deviceBuffer(pixels * c));
  }
  void* x = drv::toDevice(xh);

  auto runMode = [&](int mode, std::vector<double>* perLayer) {
    cusync_conv_chain_config cfg;
    memset(&cfg, 0, sizeof cfg);
    cfg.N = n; cfg.H = h; cfg.W = w; cfg.C = c; cfg.layers = layers; cfg.sync = mode; cfg.tile = -1; cfg.opts = -1; cfg.relu = 1;
    cfg.split_k = splitK;      // --split_k_slices (resnet.cu:329); 0 = the library picks
    cusync_conv_chain* ch = cusync_conv_chain_create(&cfg, wd.data());
    if (!ch) { fprintf(stderr, "cusync_conv_chain_create failed: %s\n", cusync_rt_last_error()); exit(EXIT_FAILURE); }
    DRV_CHECK(cusync_conv_chain_run(ch, x, yd.data(), warmup, nullptr, nullptr));
    std::vector<double> t(runs), per((size_t)runs * layers, 0.0);
    DRV_CHECK(cusync_conv_chain_run(ch, x, yd.data(), runs, t.data(), per.data()));
    if (perLayer) {
      perLayer->assign(layers, 0.0);
      for (int r = 0; r < runs; r++) for (uint32_t i = 0; i < layers; i++) (*perLayer)[i] += per[(size_t)r * layers + i] / runs;
    }
    cusync_conv_chain_destroy(ch);
    return drv::mean(t);
  };

  std::vector<double> per;
  printf("START-BASELINE:\n");
  const double base = runMode(CUSYNC_SYNC_STREAM, &per);
  printf("END-BASELINE: {Total: %lf", base);
  for (uint32_t i = 0; i < layers; i++) printf(", Conv%u: %lf", i + 1, per[i]);
  printf("} micro seconds\n");
  printf("START-OVERLAP:\n");
  const double over = runMode(sync, nullptr);
  printf("END-OVERLAP {Total: %lf} micro seconds\n", over);
  printf("gain %.2f %%\n", 100.0 - over / base * 100.0);

  if (check) {
    // every layer on the input the GPU produced for it, on a sample of output pixels (direct convolution,
    // cross-correlation, pad 1: resnet.cu:678, 704-720; tolerance 1e-2, :724)
    size_t bad = 0;
    std::vector<uint16_t> in = xh;
    for (uint32_t l = 0; l < layers; l++) {
      auto out = drv::toHost(yd[l], pixels * c);
      for (size_t s = 0; s < 64; s++) {
        const size_t pix = s == 0 ? 0 : s == 1 ? pixels - 1 : (s * 2654435761u) % pixels;
        const uint32_t img = (uint32_t)(pix / (h * w)), py = (uint32_t)(pix / w % h), px = (uint32_t)(pix % w);
        for (uint32_t k = 0; k < c; k++) {
          float acc = 0;
          for (int r = 0; r < 3; r++) for (int q = 0; q < 3; q++) {
            const int iy = (int)py + r - 1, ix = (int)px + q - 1;
            if (iy < 0 || iy >= (int)h || ix < 0 || ix >= (int)w) continue;
            const uint16_t* ip = &in[(((size_t)img * h + iy) * w + ix) * c];
            const uint16_t* wp = &wh[l][(((size_t)k * 3 + r) * 3 + q) * c];
            for (uint32_t ch = 0; ch < c; ch++) acc += drv::h2f(ip[ch]) * drv::h2f(wp[ch]);
          }
          if (l + 1 < layers && acc < 0) acc = 0;
          if (!drv::closeEnough(drv::h2f(out[pix * c + k]), acc, 1e-2f)) bad++;
        }
      }
      in.swap(out);
    }
    printf(bad ? "check: %zu mismatches\n" : "check: passed\n", bad);
    if (bad) return EXIT_FAILURE;
  }
  cusync_rt_free(x);
  for (uint32_t i = 0; i < layers; i++) { cusync_rt_free((void*)wd[i]); cusync_rt_free(yd[i]); }
  return 0;
}
