// Shared helpers of the benchmark drivers: device buffers, timing, seeded inputs.
#pragma once

#include <hip/hip_runtime.h>

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "../../include/hq.h"

#define HIP_OK(expr)                                                                     \
  do {                                                                                   \
    hipError_t e_ = (expr);                                                              \
    if (e_ != hipSuccess) {                                                              \
      std::fprintf(stderr, "%s:%d: %s: %s\n", __FILE__, __LINE__, #expr, hipGetErrorString(e_)); \
      std::exit(2);                                                                      \
    }                                                                                    \
  } while (0)

#define HQ_OK_OR_DIE(expr)                                                         \
  do {                                                                             \
    int c_ = (expr);                                                               \
    if (c_ != 0) {                                                                 \
      std::fprintf(stderr, "%s:%d: %s: %s\n", __FILE__, __LINE__, #expr, hq_strerror(c_)); \
      std::exit(2);                                                                \
    }                                                                              \
  } while (0)

template <typename T>
struct DevBuf {
  T* p = nullptr;
  size_t n = 0;
  DevBuf() {}
  explicit DevBuf(size_t count) { alloc(count); }
  DevBuf(const DevBuf&) = delete;
  DevBuf& operator=(const DevBuf&) = delete;
  DevBuf(DevBuf&& o) noexcept : p(o.p), n(o.n) { o.p = nullptr; o.n = 0; }
  ~DevBuf() { if (p) (void)hipFree(p); }
  void alloc(size_t count) {
    n = count;
    HIP_OK(hipMalloc((void**)&p, std::max<size_t>(count, 1) * sizeof(T)));
  }
  void upload(const T* h, size_t count) { HIP_OK(hipMemcpy(p, h, count * sizeof(T), hipMemcpyHostToDevice)); }
  void upload(const std::vector<T>& h) { upload(h.data(), h.size()); }
  void download(T* h, size_t count) const { HIP_OK(hipMemcpy(h, p, count * sizeof(T), hipMemcpyDeviceToHost)); }
  std::vector<T> download() const {
    std::vector<T> h(n);
    download(h.data(), n);
    return h;
  }
};

// Per-call wall-clock samples with min / max / mean / percentile, in milliseconds.
class SampleTimer {
 public:
  void start() { t0_ = std::chrono::steady_clock::now(); }
  double stop() {
    const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0_).count();
    samples_.push_back(ms);
    sorted_ = false;
    return ms;
  }
  double mean() const {
    double s = 0;
    for (double v : samples_) s += v;
    return samples_.empty() ? 0.0 : s / samples_.size();
  }
  double min() { sort(); return samples_.empty() ? 0.0 : samples_.front(); }
  double max() { sort(); return samples_.empty() ? 0.0 : samples_.back(); }
  double percentile(double p) { sort(); return samples_.empty() ? 0.0 : samples_[(size_t)((samples_.size() - 1) * p)]; }

 private:
  void sort() {
    if (!sorted_) { std::sort(samples_.begin(), samples_.end()); sorted_ = true; }
  }
  std::vector<double> samples_;
  bool sorted_ = false;
  std::chrono::steady_clock::time_point t0_;
};

// Microseconds per call of `fn(i)` over `iters` back-to-back calls, timed with HIP
// events on `stream` (the stream the kernels are enqueued on).
template <typename F>
double time_events_us(F fn, int iters, int warmup, hipStream_t stream = nullptr) {
  for (int i = 0; i < warmup; ++i) fn(i);
  HIP_OK(hipStreamSynchronize(stream));
  hipEvent_t a, b;
  HIP_OK(hipEventCreate(&a));
  HIP_OK(hipEventCreate(&b));
  HIP_OK(hipEventRecord(a, stream));
  for (int i = 0; i < iters; ++i) fn(i);
  HIP_OK(hipEventRecord(b, stream));
  HIP_OK(hipEventSynchronize(b));
  float ms = 0;
  HIP_OK(hipEventElapsedTime(&ms, a, b));
  HIP_OK(hipEventDestroy(a));
  HIP_OK(hipEventDestroy(b));
  return (double)ms * 1000.0 / iters;
}

// IEEE binary16 <-> binary32 on the host (round to nearest even).
inline uint16_t f32_to_f16_bits(float f) {
  uint32_t x;
  std::memcpy(&x, &f, 4);
  const uint32_t sign = (x >> 16) & 0x8000u;
  const int32_t exp = (int32_t)((x >> 23) & 0xff) - 127 + 15;
  uint32_t man = x & 0x7fffffu;
  if (((x >> 23) & 0xff) == 0xff) return (uint16_t)(sign | 0x7c00u | (man ? 0x200u : 0));
  if (exp >= 31) return (uint16_t)(sign | 0x7c00u);
  if (exp <= 0) {
    if (exp < -10) return (uint16_t)sign;
    man |= 0x800000u;
    const int shift = 14 - exp;
    uint32_t h = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (h & 1))) ++h;
    return (uint16_t)(sign | h);
  }
  uint32_t h = ((uint32_t)exp << 10) | (man >> 13);
  const uint32_t rem = man & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (h & 1))) ++h;
  return (uint16_t)(sign | h);
}
inline float f16_bits_to_f32(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  const uint32_t exp = (h >> 10) & 31, man = h & 1023u;
  uint32_t x;
  if (exp == 0) {
    if (man == 0) x = sign;
    else {
      int e = -1;
      uint32_t m = man;
      do { ++e; m <<= 1; } while (!(m & 0x400u));
      x = sign | ((uint32_t)(127 - 15 - e) << 23) | ((m & 0x3ffu) << 13);
    }
  } else if (exp == 31) x = sign | 0x7f800000u | (man << 13);
  else x = sign | ((exp - 15 + 127) << 23) | (man << 13);
  float f;
  std::memcpy(&f, &x, 4);
  return f;
}

// Own integer-to-float mappings on std::mt19937 (the distributions of <random> are
// not specified bit for bit across standard libraries).
struct SeededRng {
  std::mt19937 gen;
  explicit SeededRng(uint32_t seed) : gen(seed) {}
  uint32_t u32() { return gen(); }
  double unit() { return (gen() >> 8) * (1.0 / 16777216.0); }  // [0,1)
  double uniform(double lo, double hi) { return lo + (hi - lo) * unit(); }
  double normal() {  // Box-Muller
    const double u1 = 1.0 - unit(), u2 = unit();
    return std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586 * u2);
  }
};

inline void print_device_line() {
  int cus = 0, wave = 0, lds = 0, mclk = 0, bus = 0;
  char name[256];
  HQ_OK_OR_DIE(hq_device_info(&cus, &wave, &lds, &mclk, &bus, name, (int)sizeof(name)));
  std::printf("device: %s, %d CUs, wave%d, %d KB LDS/CU, memory clock %d kHz, bus %d bits\n", name, cus, wave,
              lds / 1024, mclk, bus);
}

constexpr double kHbmPeakGBs = 8000.0;  // MI355X HBM3E, vendor figure
