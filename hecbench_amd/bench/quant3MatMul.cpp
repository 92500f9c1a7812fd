// quant3MatMul driver: same command line, inputs, verification and printed lines as
// the HeCBench benchmark (src/quant3MatMul-hip/main.cu), on top of libhq.
//
//   quant3MatMul <repeat>                      reference problem (K=49152, N=12288)
//   quant3MatMul <repeat> --config <K> <N>     seeded uniform problem of that shape, with
//                                              rotated weight buffers and a roofline report
#include "bench_common.h"

namespace {

// Reference launch wrappers (src/quant3MatMul-hip/kernels.h:171-217): accumulate into mul.
void vecquant3matmul(float* vec, int* mat, float* mul, float* scales, float* zeros, int height, int width) {
  HQ_OK_OR_DIE(hq_q3_matvec(vec, HQ_DTYPE_F32, mat, scales, zeros, mul, height / 3 * 32, width, 1,
                            HQ_FLAG_ACCUMULATE, nullptr));
}
void vecquant3matmul_faster(uint16_t* vec_f16, int* mat, float* mul, float* scales, float* zeros, int height,
                            int width) {
  HQ_OK_OR_DIE(hq_q3_matvec(vec_f16, HQ_DTYPE_F16, mat, scales, zeros, mul, height / 3 * 32, width, 1,
                            HQ_FLAG_ACCUMULATE, nullptr));
}

int run_reference_problem(int repeat) {
  // OPT-175B FC2 matvec, as in the reference main (main.cu:15-23)
  const int m = 12288 * 4, n = 12288;
  const int mat_height = m / 1024 * 96, mat_width = n;
  const size_t mat_size = (size_t)mat_height * mat_width;

  std::vector<float> h_input(m, 1.f);
  std::vector<uint16_t> h_input_half(m, f32_to_f16_bits(1.f));
  std::vector<int> h_weight(mat_size);
  const unsigned p1 = 0b01001001001001001001001001001001u;  // every 3-bit code is 1
  for (int i = 0; i < mat_height; i += 3)
    for (int j = 0; j < mat_width; ++j) {
      h_weight[(size_t)i * mat_width + j] = (int)p1;
      h_weight[(size_t)(i + 1) * mat_width + j] = (int)(p1 << 1);
      h_weight[(size_t)(i + 2) * mat_width + j] = (int)(p1 << 2);
    }
  std::vector<float> h_scale(n, -1.f), h_bias(n, 0.f), h_output(n);

  DevBuf<float> d_input(m), d_scale(n), d_bias(n), d_output(n);
  DevBuf<uint16_t> d_input_half(m);
  DevBuf<int> d_weight(mat_size);
  d_input.upload(h_input);
  d_input_half.upload(h_input_half);
  d_weight.upload(h_weight);
  d_scale.upload(h_scale);
  d_bias.upload(h_bias);

  auto verify = [&](bool faster) {
    HIP_OK(hipMemset(d_output.p, 0, sizeof(float) * n));
    if (faster) vecquant3matmul_faster(d_input_half.p, d_weight.p, d_output.p, d_scale.p, d_bias.p, mat_height, mat_width);
    else vecquant3matmul(d_input.p, d_weight.p, d_output.p, d_scale.p, d_bias.p, mat_height, mat_width);
    d_output.download(h_output.data(), n);
    bool ok = true;
    for (int i = 0; i < n; ++i)
      if (h_output[i] != -49152.f) { ok = false; break; }
    std::printf("%s\n", ok ? "PASS" : "FAIL");
    return ok;
  };
  bool ok = verify(false);
  ok = verify(true) && ok;

  auto start = std::chrono::steady_clock::now();
  for (int i = 0; i < repeat; ++i) {
    HIP_OK(hipMemsetAsync(d_output.p, 0, sizeof(float) * n, nullptr));
    vecquant3matmul(d_input.p, d_weight.p, d_output.p, d_scale.p, d_bias.p, mat_height, mat_width);
  }
  HIP_OK(hipDeviceSynchronize());
  auto end = std::chrono::steady_clock::now();
  double time = std::chrono::duration<double, std::nano>(end - start).count();
  std::printf("Average execution time of the kernel: %f (us)\n", (time * 1e-3) / repeat);

  start = std::chrono::steady_clock::now();
  for (int i = 0; i < repeat; ++i) {
    HIP_OK(hipMemsetAsync(d_output.p, 0, sizeof(float) * n, nullptr));
    vecquant3matmul_faster(d_input_half.p, d_weight.p, d_output.p, d_scale.p, d_bias.p, mat_height, mat_width);
  }
  HIP_OK(hipDeviceSynchronize());
  end = std::chrono::steady_clock::now();
  time = std::chrono::duration<double, std::nano>(end - start).count();
  std::printf("Average execution time of the faster kernel: %f (us)\n", (time * 1e-3) / repeat);

  // beyond the reference: the same call without the memset (the library overwrites)
  const double bytes = (double)mat_size * 4 + 3.0 * n * 4 + (double)m * 4;
  const double us = time_events_us([&](int) {
    HQ_OK_OR_DIE(hq_q3_matvec(d_input.p, HQ_DTYPE_F32, d_weight.p, d_scale.p, d_bias.p, d_output.p, m, n, 1, 0, nullptr));
  }, repeat, 10);
  std::printf("overwrite mode (no memset): %.3f us per call, %.1f GB/s (%.1f%% of %.0f GB/s)\n", us,
              bytes / us * 1e-3, bytes / us * 1e-3 / kHbmPeakGBs * 100, kHbmPeakGBs);
  return ok ? 0 : 1;
}

// Host check of a sample of columns in double precision (layout of kernels.h:42-86).
double max_rel_err_sample(const std::vector<int>& mat, const std::vector<float>& x, const std::vector<float>& s,
                          const std::vector<float>& z, const std::vector<float>& y, int K, int N) {
  double rms = 0;
  for (int n = 0; n < N; ++n) rms += (double)y[n] * y[n];
  rms = std::sqrt(rms / N);
  double worst = 0;
  for (int n = 0; n < N; n += std::max(1, N / 512)) {
    double acc = 0;
    for (int g = 0; g < K / 32; ++g) {
      uint32_t w[3];
      for (int j = 0; j < 3; ++j) w[j] = (uint32_t)mat[(size_t)(3 * g + j) * N + n];
      for (int i = 0; i < 32; ++i) {
        const int bit = 3 * i, wd = bit >> 5, sh = bit & 31;
        uint32_t q = w[wd] >> sh;
        if (sh > 29) q |= w[wd + 1] << (32 - sh);
        acc += ((double)s[n] * (q & 7u) - (double)z[n]) * x[32 * g + i];
      }
    }
    worst = std::max(worst, std::fabs(acc - y[n]) / std::max(std::fabs(acc), 0.01 * rms));
  }
  return worst;
}

int run_config(int repeat, int K, int N) {
  print_device_line();
  const int rows = 3 * K / 32;
  const size_t mat_size = (size_t)rows * N;
  const size_t mat_bytes = mat_size * 4;
  const int nbuf = (int)std::max<size_t>(2, (size_t)(576e6 / mat_bytes) + 1);  // > 512 MB of distinct weights
  SeededRng rng(1234 + 1);
  std::vector<float> x(K), s(N), z(N);
  for (auto& v : x) v = (float)rng.normal();
  for (int n = 0; n < N; ++n) {
    s[n] = (float)rng.uniform(0.005, 0.02);
    z[n] = s[n] * (float)(3 + (rng.u32() & 1));
  }
  std::vector<int> mat(mat_size);
  std::vector<DevBuf<int>> d_mats;
  for (int b = 0; b < nbuf; ++b) {
    for (auto& v : mat) v = (int)rng.u32();  // uniform words = uniform 3-bit codes
    d_mats.emplace_back(mat_size);
    d_mats.back().upload(mat);
  }
  DevBuf<float> d_x(K), d_s(N), d_z(N), d_y(N);
  d_x.upload(x); d_s.upload(s); d_z.upload(z);
  HQ_OK_OR_DIE(hq_init());
  // correctness on the last buffer (still on the host)
  HQ_OK_OR_DIE(hq_q3_matvec(d_x.p, HQ_DTYPE_F32, d_mats.back().p, d_s.p, d_z.p, d_y.p, K, N, 1, 0, nullptr));
  const std::vector<float> y = d_y.download();
  const double err = max_rel_err_sample(mat, x, s, z, y, K, N);
  std::printf("%s (max relative error %.3e on sampled columns, bound 1e-3)\n", err <= 1e-3 ? "PASS" : "FAIL", err);

  const double bytes = (double)mat_bytes + 3.0 * N * 4 + (double)K * 4;
  const double us = time_events_us([&](int i) {
    HQ_OK_OR_DIE(hq_q3_matvec(d_x.p, HQ_DTYPE_F32, d_mats[i % nbuf].p, d_s.p, d_z.p, d_y.p, K, N, 1, 0, nullptr));
  }, repeat, 50);
  const double hot = time_events_us([&](int) {
    HQ_OK_OR_DIE(hq_q3_matvec(d_x.p, HQ_DTYPE_F32, d_mats[0].p, d_s.p, d_z.p, d_y.p, K, N, 1, 0, nullptr));
  }, repeat, 50);
  std::printf("GPTQ 3-bit matvec K=%d N=%d, %d rotated weight buffers (%.0f MB)\n", K, N, nbuf, nbuf * mat_bytes / 1e6);
  std::printf("Average execution time of the kernel: %f (us)\n", us);
  std::printf("achieved %.1f GB/s = %.1f%% of %.0f GB/s HBM peak (algorithmic bytes %.0f); effective fp16-weight %.1f GB/s\n",
              bytes / us * 1e-3, bytes / us * 1e-3 / kHbmPeakGBs * 100, kHbmPeakGBs, bytes, 2.0 * K * N / us * 1e-3);
  std::printf("hot-cache (one buffer): %f (us)\n", hot);
  return err <= 1e-3 ? 0 : 1;
}

}  // namespace

int main(int argc, char* argv[]) {
  if (argc != 2 && !(argc == 5 && std::strcmp(argv[2], "--config") == 0)) {
    std::printf("Usage: %s <repeat> [--config <K> <N>]\n", argv[0]);
    return 1;
  }
  const int repeat = std::atoi(argv[1]);
  if (argc == 2) return run_reference_problem(repeat);
  return run_config(repeat, std::atoi(argv[3]), std::atoi(argv[4]));
}
