// Shared by the command-line drivers: argument parsing, fp16 conversion, seeded
// inputs, device buffers through the C ABI and a sampled CPU check.  The drivers
// are plain host C++ — everything that touches the GPU goes through
// include/cusync_amd.h, which is the point of them.
#pragma once

#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <map>
#include <random>
#include <string>
#include <vector>

#include "../../include/cusync_amd.h"

#define DRV_CHECK(call) do { cusync_error e_ = (call); if (e_ != CUSYNC_SUCCESS) { \
  fprintf(stderr, "Failed: %s -> %d (%s) at %s:%d\n", #call, (int)e_, cusync_rt_last_error(), __FILE__, __LINE__); exit(EXIT_FAILURE); } } while (0)
#define RT_CHECK(call) do { if ((call) != 0) { \
  fprintf(stderr, "Failed: %s (%s) at %s:%d\n", #call, cusync_rt_last_error(), __FILE__, __LINE__); exit(EXIT_FAILURE); } } while (0)

namespace drv {

// "--name value" and "--name=value"; flags without a value read as "true".
inline std::map<std::string, std::string> parseArgs(int argc, char** argv) {
  std::map<std::string, std::string> m;
  for (int i = 1; i < argc; i++) {
    std::string a = argv[i];
    if (a.rfind("--", 0) != 0) { fprintf(stderr, "unexpected argument %s\n", a.c_str()); exit(EXIT_FAILURE); }
    a = a.substr(2);
    size_t eq = a.find('=');
    if (eq != std::string::npos) m[a.substr(0, eq)] = a.substr(eq + 1);
    else if (i + 1 < argc && strncmp(argv[i + 1], "--", 2) != 0) m[a] = argv[++i];
    else m[a] = "true";
  }
  return m;
}
inline std::string get(const std::map<std::string, std::string>& m, const char* k, const char* dflt) {
  auto it = m.find(k);
  return it == m.end() ? dflt : it->second;
}
inline long getInt(const std::map<std::string, std::string>& m, const char* k, long dflt) {
  auto it = m.find(k);
  return it == m.end() ? dflt : atol(it->second.c_str());
}
inline bool getBool(const std::map<std::string, std::string>& m, const char* k, bool dflt) {
  auto it = m.find(k);
  return it == m.end() ? dflt : (it->second == "true" || it->second == "1");
}

// IEEE binary16 <-> binary32, round to nearest even.
inline uint16_t f2h(float f) {
  uint32_t x; memcpy(&x, &f, 4);
  const uint32_t sign = (x >> 16) & 0x8000u;
  x &= 0x7fffffffu;
  if (x >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (x > 0x7f800000u ? 0x200u : 0));
  if (x >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);                 // overflows to infinity
  if (x < 0x38800000u) {                                                     // subnormal half or zero
    if (x < 0x33000000u) return (uint16_t)sign;
    const int shift = 126 - (int)(x >> 23);                                  // 14..24
    const uint32_t mant = (x & 0x7fffffu) | 0x800000u;
    uint32_t h = mant >> shift;
    const uint32_t rem = mant & ((1u << shift) - 1), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (h & 1))) h++;
    return (uint16_t)(sign | h);
  }
  uint32_t h = ((x - 0x38000000u) >> 13);
  const uint32_t rem = x & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (h & 1))) h++;
  return (uint16_t)(sign | h);
}
inline float h2f(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1f, mant = h & 0x3ffu, x;
  if (exp == 0) {
    if (mant == 0) x = sign;
    else { int e = -1; do { e++; mant <<= 1; } while (!(mant & 0x400u)); x = sign | ((uint32_t)(112 - e) << 23) | ((mant & 0x3ffu) << 13); }
  } else if (exp == 31) x = sign | 0x7f800000u | (mant << 13);
  else x = sign | ((exp + 112) << 23) | (mant << 13);
  float f; memcpy(&f, &x, 4);
  return f;
}

inline std::vector<uint16_t> uniformHalf(size_t n, uint64_t seed) {          // U[-1, 1]
  std::mt19937_64 rng(seed);
  std::uniform_real_distribution<float> d(-1.0f, 1.0f);
  std::vector<uint16_t> v(n);
  for (auto& e : v) e = f2h(d(rng));
  return v;
}
inline std::vector<uint16_t> normalHalf(size_t n, uint64_t seed, float stddev) {
  std::mt19937_64 rng(seed);
  std::normal_distribution<float> d(0.0f, stddev);
  std::vector<uint16_t> v(n);
  for (auto& e : v) e = f2h(d(rng));
  return v;
}

inline void* toDevice(const std::vector<uint16_t>& v) {
  void* p = nullptr;
  RT_CHECK(cusync_rt_malloc(&p, v.size() * 2));
  RT_CHECK(cusync_rt_memcpy_h2d(p, v.data(), v.size() * 2));
  return p;
}
inline void* deviceBuffer(size_t halfs) {
  void* p = nullptr;
  RT_CHECK(cusync_rt_malloc(&p, halfs * 2));
  RT_CHECK(cusync_rt_memset(p, 0, halfs * 2));
  return p;
}
inline std::vector<uint16_t> toHost(const void* p, size_t halfs) {
  std::vector<uint16_t> v(halfs);
  RT_CHECK(cusync_rt_memcpy_d2h(v.data(), p, halfs * 2));
  return v;
}

// The reference's comparison (src/ml-bench/transformer/common.h:104-137): both small -> equal; else relative.
inline bool closeEnough(float got, float want, float tol) {
  if (fabsf(got) < tol && fabsf(want) < tol) return true;
  const float m = fmaxf(fabsf(got), fabsf(want));
  return fabsf(got - want) / m <= tol || fabsf(got - want) <= 1e-3f;
}

// Row `r` of A[*, K] times B[K, N] in fp32 (the reference's host GEMM, common.h:89-102, one row of it).
inline std::vector<float> gemmRow(const uint16_t* a, const std::vector<uint16_t>& b, size_t K, size_t N) {
  std::vector<float> out(N, 0.0f);
  for (size_t k = 0; k < K; k++) {
    const float av = h2f(a[k]);
    const uint16_t* brow = &b[k * N];
    for (size_t j = 0; j < N; j++) out[j] += av * h2f(brow[j]);
  }
  return out;
}

inline double mean(const std::vector<double>& v) {
  double s = 0;
  for (double x : v) s += x;
  return v.empty() ? 0 : s / v.size();
}

}  // namespace drv
