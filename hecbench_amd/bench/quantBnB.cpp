// quantBnB driver: same command line, inputs, verification and printed lines as the
// HeCBench benchmark (src/quantBnB-hip/main.cu), on top of libhq.
//
//   quantBnB <number of elements> <repeat> [--host-only]
//
// Part 1 is the reference benchmark itself: bitsandbytes dynamic-map 8-bit
// quantisation, device result compared bit for bit with the host function.
// Part 2 runs the blockwise NF4 dequantisation of the same element count
// (blocksize 64, fp16 output) against a host loop, also bit for bit.
// Both host loops are timed as well, on one thread and spread over the host cores with OpenMP (what the
// quantBnB-omp variant of the benchmark does when it runs without a device); --host-only runs nothing
// else, needs no GPU and prints the OpenMP loop's time in the benchmark's own line.
#include <omp.h>
#include "bench_common.h"

namespace {

// The signed dynamic map bitsandbytes builds (7 exponent bits, 256 sorted values);
// the reference ships it as a literal table (src/quantBnB-cuda/code.h).
std::vector<float> dynamic_map() {
  std::vector<float> code;
  for (int i = 0; i < 7; ++i) {
    const int items = (1 << i) + 1;
    std::vector<float> b(items);
    const float start = 0.1f, end = 1.0f;
    const float step = items > 1 ? (end - start) / (float)(items - 1) : 0.f;
    for (int j = 0; j < items; ++j) b[j] = j < items / 2 ? start + step * (float)j : end - step * (float)(items - 1 - j);
    const float sc = (float)std::pow(10.0, -6 + i);
    for (int j = 0; j + 1 < items; ++j) {
      const float mean = (b[j] + b[j + 1]) / 2.0f;
      code.push_back(sc * mean);
      code.push_back(-sc * mean);
    }
  }
  code.push_back(0.f);
  code.push_back(1.f);
  std::sort(code.begin(), code.end());
  return code;
}

// Host statement of the quantiser (src/quantBnB-hip/main.cu:13-66, STOCHASTIC = 0).
uint8_t dquantize_host(const float* code, float x) {
  int pivot = 127, upper_pivot = 255, lower_pivot = 0;
  float lower = -1.0f, upper = 1.0f, val = code[pivot];
  for (int i = 64; i > 0; i >>= 1) {
    if (x > val) { lower_pivot = pivot; lower = val; pivot += i; }
    else { upper_pivot = pivot; upper = val; pivot -= i; }
    val = code[pivot];
  }
  if (upper_pivot == 255) upper = code[upper_pivot];
  if (lower_pivot == 0) lower = code[lower_pivot];
  if (x > val) return (uint8_t)(x > (upper + val) * 0.5f ? upper_pivot : pivot);
  return (uint8_t)(x < (lower + val) * 0.5f ? lower_pivot : pivot);
}

const float kNf4[16] = {-1.0f, -0.6961928009986877f, -0.5250730514526367f, -0.39491748809814453f,
                        -0.28444138169288635f, -0.18477343022823334f, -0.09105003625154495f, 0.0f,
                        0.07958029955625534f, 0.16093020141124725f, 0.24611230194568634f, 0.33791524171829224f,
                        0.44070982933044434f, 0.5626170039176941f, 0.7229568362236023f, 1.0f};

}  // namespace

// Seconds per pass of a host loop over n elements on `threads` threads.
template <class F>
double time_host_loop(F&& body, size_t n, int threads, int passes) {
  const auto t0 = std::chrono::steady_clock::now();
  for (int p = 0; p < passes; ++p) {
#pragma omp parallel for schedule(static) num_threads(threads)
    for (long i = 0; i < (long)n; ++i) body((size_t)i);
  }
  return std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() / passes;
}

int main(int argc, char* argv[]) {
  const bool host_only = argc == 4 && std::string(argv[3]) == "--host-only";
  if (argc != 3 && !host_only) {
    std::printf("Usage: %s <number of elements> <repeat> [--host-only]\n", argv[0]);
    return 1;
  }
  const size_t n = (size_t)std::atol(argv[1]);
  const int repeat = std::atoi(argv[2]);
  const int block_size = 256;
  const int cores = omp_get_max_threads();

  // ---- part 1: kQuantize contract --------------------------------------------------------
  const std::vector<float> code = dynamic_map();
  std::vector<float> A(n);
  std::vector<uint8_t> out(n), ref(n);
  std::mt19937 gen{19937};
  std::normal_distribution<float> d{0.f, 1.f};
  for (size_t i = 0; i < n; ++i) A[i] = d(gen);
  const double host1 = time_host_loop([&](size_t i) { ref[i] = dquantize_host(code.data(), A[i]); }, n, 1, 1);
  const int host_passes = host_only ? (repeat > 0 ? repeat : 1) : 1;
  const double hostN = time_host_loop([&](size_t i) { out[i] = dquantize_host(code.data(), A[i]); }, n, cores, host_passes);
  if (host_only) {
    std::printf("Average execution time of kQuantize kernel with block size %d: %f (us)\n", block_size, hostN * 1e6);
    std::printf("%s\n", out == ref ? "PASS" : "FAIL");
    std::printf("  (host only: OpenMP loop on %d threads; one thread: %f us)\n", cores, host1 * 1e6);
  }
  // NF4 inputs and the host loop of part 2
  const int blocksize = 64;
  SeededRng rng(1234);
  std::vector<uint8_t> packed((n + 1) / 2);
  std::vector<float> absmax((n + blocksize - 1) / blocksize);
  for (auto& b : packed) b = (uint8_t)(rng.u32() >> 24);
  for (auto& a : absmax) a = (float)rng.uniform(0.5, 2.0);
  std::vector<uint16_t> want(n), got(n);
  auto nf4_host = [&](std::vector<uint16_t>& dst) {
    return [&](size_t e) {
      const uint8_t b = packed[e >> 1];
      const unsigned c = (e & 1) ? (b & 15u) : (b >> 4);
      volatile float prod = kNf4[c] * absmax[e / blocksize];  // fp32 product, then one rounding to fp16
      dst[e] = f32_to_f16_bits(prod);
    };
  };
  const double nf4_host1 = time_host_loop(nf4_host(want), n, 1, 1);
  const double nf4_hostN = time_host_loop(nf4_host(got), n, cores, host_passes);
  if (host_only) {
    std::printf("Average execution time of NF4 dequantize kernel with block size %d: %f (us)\n", blocksize, nf4_hostN * 1e6);
    std::printf("%s\n", got == want ? "PASS" : "FAIL");
    std::printf("  (host only: OpenMP loop on %d threads; one thread: %f us)\n", cores, nf4_host1 * 1e6);
    return out == ref && got == want ? 0 : 1;
  }
  HQ_OK_OR_DIE(hq_init());
  DevBuf<float> d_A(n), d_code(256);
  DevBuf<uint8_t> d_out(n);
  d_A.upload(A);
  d_code.upload(code);
  HIP_OK(hipDeviceSynchronize());
  auto start = std::chrono::steady_clock::now();
  for (int i = 0; i < repeat; ++i) HQ_OK_OR_DIE(hq_quantize_dynamic8(d_code.p, d_A.p, d_out.p, (int64_t)n, nullptr));
  HIP_OK(hipDeviceSynchronize());
  auto end = std::chrono::steady_clock::now();
  const double t_ns = std::chrono::duration<double, std::nano>(end - start).count();
  std::printf("Average execution time of kQuantize kernel with block size %d: %f (us)\n", block_size,
              (t_ns * 1e-3) / repeat);
  d_out.download(out.data(), n);
  const bool ok1 = out == ref;
  std::printf("%s\n", ok1 ? "PASS" : "FAIL");
  std::printf("  (%.1f GB/s of 5 B/element traffic; host loop: %.0f us on one thread, %.0f us on %d OpenMP threads)\n",
              5.0 * n / ((t_ns * 1e-3) / repeat) * 1e-3, host1 * 1e6, hostN * 1e6, cores);

  // ---- part 2: blockwise NF4 dequantisation ------------------------------------------------
  // rotate over enough distinct buffers that no call is served from the 256 MB cache
  const size_t per_call = packed.size() + absmax.size() * 4 + n * 2;
  const int nbuf = (int)std::max<size_t>(2, (size_t)(600e6 / (double)per_call) + 1);
  std::vector<DevBuf<uint8_t>> d_packed;
  std::vector<DevBuf<float>> d_absmax;
  std::vector<DevBuf<uint16_t>> d_deq;
  for (int i = 0; i < nbuf; ++i) {
    d_packed.emplace_back(packed.size());
    d_packed.back().upload(packed);
    d_absmax.emplace_back(absmax.size());
    d_absmax.back().upload(absmax);
    d_deq.emplace_back(n);
  }
  const double us = time_events_us([&](int i) {
    const int b = i % nbuf;
    HQ_OK_OR_DIE(hq_dequant_nf4(d_packed[b].p, d_absmax[b].p, d_deq[b].p, (int64_t)n, blocksize, HQ_TABLE_NF4, nullptr));
  }, repeat, 10);
  d_deq[(repeat - 1) % nbuf].download(got.data(), n);
  const bool ok2 = got == want;
  std::printf("Average execution time of NF4 dequantize kernel with block size %d: %f (us)\n", blocksize, us);
  std::printf("%s\n", ok2 ? "PASS" : "FAIL");
  std::printf("  (%.1f GB/s = %.1f%% of %.0f GB/s HBM peak, %zu bytes per call, %d rotated buffers)\n",
              per_call / us * 1e-3, per_call / us * 1e-3 / kHbmPeakGBs * 100, kHbmPeakGBs, per_call, nbuf);
  std::printf("  (host loop: %.0f us on one thread, %.0f us on %d OpenMP threads)\n", nf4_host1 * 1e6, nf4_hostN * 1e6, cores);
  return ok1 && ok2 ? 0 : 1;
}
