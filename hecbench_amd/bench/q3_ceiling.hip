// What a single launch over the 16.9 MB weight matrix of the GPTQ 3-bit matvec (K=4096, N=11008) can
// reach on this GPU, measured next to the library's kernel: an empty kernel, plain streaming reads, the
// library kernel's own access pattern with the arithmetic taken out, and what a result store at the end
// of the kernel and a by-value argument structure add.  Weights are rotated over more than 512 MB so that
// every launch reads HBM; every figure is the median of five windows of back-to-back launches, timed with
// HIP events on the launch stream.
//
//   q3_ceiling [launches per window, default 3000]
//
// The access pattern follows hq_q3_matvec's kernel: a workgroup of 8 waves owns 64 columns and all of K;
// a wave's 16-lane quarter streams one 32-row k-group per step as three 128-bit loads.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#include "../../include/hq.h"

typedef uint32_t u4v __attribute__((ext_vector_type(4)));
#define CK(x)                                                                          \
  do {                                                                                 \
    hipError_t e = (x);                                                                \
    if (e != hipSuccess) {                                                             \
      std::printf("%s:%d: %s\n", __FILE__, __LINE__, hipGetErrorString(e));            \
      std::exit(1);                                                                    \
    }                                                                                  \
  } while (0)

__global__ void k_empty() {}

// PER 128-bit loads per thread, strided by the grid (fully coalesced stream)
template <int PER>
__global__ __launch_bounds__(256) void k_stream(const u4v* __restrict__ p, uint32_t* out, size_t n) {
  const size_t t = (size_t)blockIdx.x * 256 + threadIdx.x, T = (size_t)gridDim.x * 256;
  u4v v[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const size_t idx = t + i * T;
    v[i] = idx < n ? __builtin_nontemporal_load(p + idx) : u4v{0, 0, 0, 0};
  }
  uint32_t s = 0;
#pragma unroll
  for (int i = 0; i < PER; ++i) s += v[i].x ^ v[i].y ^ v[i].z ^ v[i].w;
  if (s == 0x12345678) out[t] = s;
}

struct BigArgs {  // a by-value argument structure of the size the library kernel takes
  const uint32_t* w;
  uint32_t* out;
  float* y;
  int N, G, gpw;
  int pad[12];
};

// The matvec kernel's loads without its arithmetic.  STORE: 0 none, 1 plain store of a 64-float result
// row by wave 0, 2 the same as a device-scope (write-through) store.  STRUCT: arguments by value.
template <int WAVES, int STEPS, int STORE, bool STRUCT>
__global__ __launch_bounds__(WAVES * 64) void k_pattern(const uint32_t* __restrict__ w, uint32_t* out, float* y,
                                                       int N, int G, int gpw, BigArgs big) {
  if (STRUCT) { w = big.w; out = big.out; y = big.y; N = big.N; G = big.G; gpw = big.gpw; }
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, c = lane & 15, kb = lane >> 4;
  const int ntiles = N / 64, tile = blockIdx.x % ntiles, split = blockIdx.x / ntiles;
  const int col = tile * 64 + 4 * c;
  u4v v[STEPS][3];
#pragma unroll
  for (int st = 0; st < STEPS; ++st) {
    const int g = min(split * gpw + st * WAVES * 4 + wv * 4 + kb, G - 1);
    const uint32_t* p = w + (size_t)(3 * g) * N + col;
#pragma unroll
    for (int j = 0; j < 3; ++j) v[st][j] = __builtin_nontemporal_load((const u4v*)(p + (size_t)j * N));
  }
  uint32_t s = 0;
#pragma unroll
  for (int st = 0; st < STEPS; ++st)
#pragma unroll
    for (int j = 0; j < 3; ++j) s += v[st][j].x ^ v[st][j].y ^ v[st][j].z ^ v[st][j].w;
  if (s == 0x12345678) out[blockIdx.x * 256 + tid] = s;
  if (STORE && wv == 0) {
    const float val = (float)(s & 1023);
    if (STORE == 1) y[tile * 64 + lane] = val;
    else __hip_atomic_store(&y[tile * 64 + lane], val, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

template <class F>
float window(F f, int iters) {
  hipEvent_t a, b;
  CK(hipEventCreate(&a));
  CK(hipEventCreate(&b));
  for (int i = 0; i < 50; ++i) f(i);
  CK(hipDeviceSynchronize());
  CK(hipEventRecord(a));
  for (int i = 0; i < iters; ++i) f(i);
  CK(hipEventRecord(b));
  CK(hipEventSynchronize(b));
  float ms;
  CK(hipEventElapsedTime(&ms, a, b));
  CK(hipEventDestroy(a));
  CK(hipEventDestroy(b));
  return ms * 1000.f / iters;
}
template <class F>
float median5(F f, int iters) {
  float v[5];
  for (float& x : v) x = window(f, iters);
  std::sort(v, v + 5);
  return v[2];
}

int main(int argc, char** argv) {
  const int K = 4096, N = 11008, G = K / 32, ROWS = 3 * G;
  const int iters = argc > 1 ? std::atoi(argv[1]) : 3000;
  const size_t wbytes = (size_t)ROWS * N * 4, n4 = wbytes / 16;
  const int NB = 34;  // 575 MB of distinct weights
  const double algo = (double)wbytes + 2.0 * N * 4 + K * 4 + N * 4;
  CK(hipSetDevice(0));
  if (hq_init()) { std::printf("hq_init failed\n"); return 1; }
  std::mt19937 rng(1234);
  std::vector<uint32_t> hw(wbytes / 4);
  for (auto& v : hw) v = rng();
  std::vector<uint32_t*> bufs(NB);
  for (int b = 0; b < NB; ++b) {
    CK(hipMalloc(&bufs[b], wbytes));
    for (size_t i = 0; i < 1024; ++i) hw[(i * 7919 + b * 131) % hw.size()] = rng();
    CK(hipMemcpy(bufs[b], hw.data(), wbytes, hipMemcpyHostToDevice));
  }
  std::vector<float> hx(K), hs(N), hz(N);
  std::normal_distribution<float> nd;
  std::uniform_real_distribution<float> ud(0.005f, 0.02f);
  for (auto& v : hx) v = nd(rng);
  for (int i = 0; i < N; ++i) { hs[i] = ud(rng); hz[i] = hs[i] * (3 + (rng() & 1)); }
  float *x, *s, *z, *y;
  CK(hipMalloc(&x, K * 4)); CK(hipMalloc(&s, N * 4)); CK(hipMalloc(&z, N * 4)); CK(hipMalloc(&y, N * 4));
  CK(hipMemcpy(x, hx.data(), K * 4, hipMemcpyHostToDevice));
  CK(hipMemcpy(s, hs.data(), N * 4, hipMemcpyHostToDevice));
  CK(hipMemcpy(z, hz.data(), N * 4, hipMemcpyHostToDevice));
  uint32_t* out;
  CK(hipMalloc(&out, 64 << 20));
  BigArgs big = {};
  big.out = out; big.y = y; big.N = N; big.G = G; big.gpw = 128;

  auto line = [&](const char* what, float us) {
    std::printf("%-86s %6.2f us  %5.0f GB/s  %.3f of 8 TB/s\n", what, us, algo / us / 1e3, algo / us / 1e3 / 8000.0);
    std::fflush(stdout);
  };
  std::printf("K=%d N=%d: %.1f MB of packed weights per launch, %d rotated buffers, %d launches per window\n", K, N,
              wbytes / 1e6, NB, iters);
  std::printf("%-86s %6.2f us\n", "empty kernel, 1 x 64 threads", median5([&](int) { k_empty<<<1, 64>>>(); }, iters));
  std::printf("%-86s %6.2f us\n", "empty kernel, 172 x 512 threads", median5([&](int) { k_empty<<<172, 512>>>(); }, iters));
  { const int blocks = (int)((n4 / 4 + 255) / 256);
    line("streaming read, 4 x 128 bit per thread, 1032 workgroups of 256", median5([&](int i) { k_stream<4><<<blocks, 256>>>((const u4v*)bufs[i % NB], out, n4); }, iters));
    line("  the same from one buffer (served by the caches)", median5([&](int) { k_stream<4><<<blocks, 256>>>((const u4v*)bufs[0], out, n4); }, iters)); }
  { const int blocks = (int)((n4 / 8 + 255) / 256);
    line("streaming read, 8 x 128 bit per thread, 516 workgroups of 256", median5([&](int i) { k_stream<8><<<blocks, 256>>>((const u4v*)bufs[i % NB], out, n4); }, iters)); }
  line("matvec access pattern, loads only: 172 workgroups x 8 waves x 4 steps (the library's)", median5([&](int i) { k_pattern<8, 4, 0, false><<<172, 512>>>(bufs[i % NB], out, y, N, G, 128, big); }, iters));
  line("  the same from one buffer (served by the caches)", median5([&](int) { k_pattern<8, 4, 0, false><<<172, 512>>>(bufs[0], out, y, N, G, 128, big); }, iters));
  line("  + a 44 KB result store at the end (plain)", median5([&](int i) { k_pattern<8, 4, 1, false><<<172, 512>>>(bufs[i % NB], out, y, N, G, 128, big); }, iters));
  line("  + a 44 KB result store at the end (device-scope, write-through)", median5([&](int i) { k_pattern<8, 4, 2, false><<<172, 512>>>(bufs[i % NB], out, y, N, G, 128, big); }, iters));
  line("  + plain store + arguments as a 96-byte structure by value", median5([&](int i) { big.w = bufs[i % NB]; k_pattern<8, 4, 1, true><<<172, 512>>>(nullptr, nullptr, nullptr, 0, 0, 0, big); }, iters));
  line("loads only, K split in two: 344 workgroups x 8 waves x 2 steps", median5([&](int i) { k_pattern<8, 2, 0, false><<<344, 512>>>(bufs[i % NB], out, y, N, G, 64, big); }, iters));
  line("loads only, K split in four: 688 workgroups x 4 waves x 2 steps", median5([&](int i) { k_pattern<4, 2, 0, false><<<688, 256>>>(bufs[i % NB], out, y, N, G, 32, big); }, iters));
  line("loads only, K split in eight: 1376 workgroups x 4 waves x 1 step", median5([&](int i) { k_pattern<4, 1, 0, false><<<1376, 256>>>(bufs[i % NB], out, y, N, G, 16, big); }, iters));
  line("hq_q3_matvec (fp32 x), rotated buffers", median5([&](int i) { hq_q3_matvec(x, HQ_DTYPE_F32, (const int32_t*)bufs[i % NB], s, z, y, K, N, 1, 0, nullptr); }, iters));
  line("hq_q3_matvec (fp32 x), one buffer", median5([&](int) { hq_q3_matvec(x, HQ_DTYPE_F32, (const int32_t*)bufs[0], s, z, y, K, N, 1, 0, nullptr); }, iters));
  return 0;
}
