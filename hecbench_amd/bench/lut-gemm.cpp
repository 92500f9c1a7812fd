// lut-gemm driver: same command line, fixtures and printed lines as the HeCBench
// benchmark (src/lut-gemm-hip/main.cu), on top of libhq.
//
//   lut-gemm <test case> <repeat>      case 0: K = 1024, case 1: K = 4096, other: K = 12288
//
// Per fixture (8, 4 and 3 bit planes, group size 128, M = 1, N = 4K): the
// reference's rand()-based inputs, a host double-precision matvec of the
// dequantised weights in place of the reference's BLAS call, "mean Error", then
// per-call latency min / max / avg in milliseconds (call + synchronise).
#include "bench_common.h"

namespace {

// src/lut-gemm-hip/tests.h:11-24
void random_seed() { srand(123); }
bool rand_bool() { return rand() > (RAND_MAX / 2); }
double rand_fp64(double max = 1.0) {
  const double sign[] = {-1.0, 1.0};
  return (double)sign[rand_bool()] * rand() / RAND_MAX * rand() / RAND_MAX * max;
}
float rand_fp32(float max = 1.0) { return (float)(rand_fp64() * max); }

// The weight container of the reference (src/lut-gemm-hip/nQWeight_fp16.h:22-45) as a
// plain struct of device buffers; parsing() converts alpha / q_bias to fp16.
struct nQWeight_fp16 {
  DevBuf<uint32_t> bWeight;  // [kSize/32][nb][mSize]
  DevBuf<uint16_t> alpha;    // [num_groups][nb][mSize]
  DevBuf<uint16_t> q_bias;   // [num_groups][mSize]
  int num_groups = 0, group_size = 0, mSize = 0, kSize = 0, nb = 0;
  bool has_bias = false;
  void parsing(const uint32_t* bW, const float* A, int row, int col, int num_bits, int num_alpha_groups,
               const float* bias) {
    num_groups = num_alpha_groups; nb = num_bits; mSize = col; kSize = row; group_size = kSize / num_groups;
    std::vector<uint16_t> h((size_t)num_groups * mSize * nb);
    for (size_t i = 0; i < h.size(); ++i) h[i] = f32_to_f16_bits(A[i]);
    alpha.alloc(h.size());
    alpha.upload(h);
    has_bias = bias != nullptr;
    if (bias) {
      std::vector<uint16_t> hb((size_t)num_groups * mSize);
      for (size_t i = 0; i < hb.size(); ++i) hb[i] = f32_to_f16_bits(bias[i]);
      q_bias.alloc(hb.size());
      q_bias.upload(hb);
    }
    const size_t words = (size_t)kSize / 32 * nb * mSize;
    bWeight.alloc(words);
    bWeight.upload(bW, words);
  }
};

// matmul(output, input, nqW, m) of src/lut-gemm-hip/kernels.cu:27-31 (no memset needed).
void matmul(void* output, void* input, nQWeight_fp16& w, int /*m*/) {
  HQ_OK_OR_DIE(hq_lut_gemv(w.bWeight.p, w.alpha.p, w.has_bias ? w.q_bias.p : nullptr, input, output, w.kSize, w.mSize,
                           w.nb, w.group_size, nullptr));
}

void run_fixture(int N, int K, int NUM_BITS, int A_GROUP_SIZE, int iter) {
  const int num_groups = K / A_GROUP_SIZE;
  std::vector<uint32_t> bW((size_t)K / 32 * NUM_BITS * N);
  std::vector<float> alpha((size_t)num_groups * NUM_BITS * N), q_bias((size_t)num_groups * N), input(K);
  // makeRandomInput / makeRandomWeight / makeRandomAlpha, src/lut-gemm-hip/main.cu:101-134
  random_seed();
  for (int k = 0; k < K; ++k) input[k] = rand_fp32();
  random_seed();
  for (int n = 0; n < N; ++n)
    for (int b = 0; b < NUM_BITS; ++b)
      for (int k = 0; k < K; k += 32) {
        uint32_t s = 0;
        for (int t = 0; t < 32; ++t)
          if (rand_bool()) s |= 1u << t;
        bW[(size_t)(k / 32) * (NUM_BITS * N) + (size_t)b * N + n] = s;
      }
  random_seed();
  for (int g = 0; g < num_groups; ++g)
    for (int n = 0; n < N; ++n) {
      q_bias[(size_t)g * N + n] = rand_fp32() / (1 << NUM_BITS);
      for (int b = 0; b < NUM_BITS; ++b) alpha[(size_t)g * (NUM_BITS * N) + (size_t)b * N + n] = rand_fp32() / (1 << b);
    }
  // host result in double from the fp16-rounded operands (dequantizeFrom_qW, main.cu:136-146)
  std::vector<uint16_t> x16(K);
  std::vector<double> xd(K), ref(N, 0.0);
  for (int k = 0; k < K; ++k) { x16[k] = f32_to_f16_bits(input[k]); xd[k] = f16_bits_to_f32(x16[k]); }
  for (int g = 0; g < num_groups; ++g) {
    double xsum = 0;
    for (int k = g * A_GROUP_SIZE; k < (g + 1) * A_GROUP_SIZE; ++k) xsum += xd[k];
    for (int n = 0; n < N; ++n) ref[n] += (double)f16_bits_to_f32(f32_to_f16_bits(q_bias[(size_t)g * N + n])) * xsum;
    for (int b = 0; b < NUM_BITS; ++b)
      for (int kw = g * A_GROUP_SIZE / 32; kw < (g + 1) * A_GROUP_SIZE / 32; ++kw)
        for (int n = 0; n < N; ++n) {
          const uint32_t w = bW[(size_t)kw * (NUM_BITS * N) + (size_t)b * N + n];
          double s = 0;
          for (int t = 0; t < 32; ++t) s += (w >> t) & 1u ? xd[kw * 32 + t] : -xd[kw * 32 + t];
          ref[n] += (double)f16_bits_to_f32(f32_to_f16_bits(alpha[(size_t)g * (NUM_BITS * N) + (size_t)b * N + n])) * s;
        }
  }
  nQWeight_fp16 nqW;
  nqW.parsing(bW.data(), alpha.data(), K, N, NUM_BITS, num_groups, q_bias.data());
  DevBuf<uint16_t> d_input(K), d_out(N);
  d_input.upload(x16);
  matmul(d_out.p, d_input.p, nqW, 1);
  HIP_OK(hipDeviceSynchronize());
  const std::vector<uint16_t> out = d_out.download();
  double err = 0;
  for (int n = 0; n < N; ++n) err += std::fabs((double)f16_bits_to_f32(out[n]) - ref[n]);
  std::printf("mean Error: %lf\n", err / N);
  SampleTimer tm;
  matmul(d_out.p, d_input.p, nqW, 1);  // warm-up
  HIP_OK(hipDeviceSynchronize());
  for (int i = 0; i < iter; ++i) {
    tm.start();
    matmul(d_out.p, d_input.p, nqW, 1);
    HIP_OK(hipDeviceSynchronize());
    tm.stop();
  }
  std::printf("latency min : %.5fms, max : %.5fms, avg:%.5f\n", tm.min(), tm.max(), tm.mean());
  const double us = time_events_us([&](int) { matmul(d_out.p, d_input.p, nqW, 1); }, std::max(iter, 20), 5);
  const double bytes = (double)bW.size() * 4 + alpha.size() * 2.0 + q_bias.size() * 2.0 + K * 2.0 + N * 2.0;
  std::printf("  (back-to-back: %.3f us per call, %.1f GB/s of algorithmic bytes, hot cache)\n", us, bytes / us * 1e-3);
}

void test_case(int H, int repeat) {
  std::printf("M = 1, N = %d, K = %d\n", 4 * H, H);
  std::printf("LUT-GEMM [INT8, FP16, FP16]\t");
  run_fixture(4 * H, H, 8, 128, repeat);
  std::printf("LUT-GEMM [INT4, FP16, FP16]\t");
  run_fixture(4 * H, H, 4, 128, repeat);
  std::printf("LUT-GEMM [INT3, FP16, FP16]\t");
  run_fixture(4 * H, H, 3, 128, repeat);
}

}  // namespace

int main(int argc, char* argv[]) {
  if (argc != 3) {
    std::printf("Usage: %s <test case> <repeat>\n", argv[0]);
    std::printf("Case 0: K = 1024\n");
    std::printf("Case 1: K = 4096\n");
    std::printf("Default: K = 12288\n");
    return 1;
  }
  const int option = std::atoi(argv[1]);
  const int repeat = std::atoi(argv[2]);
  HQ_OK_OR_DIE(hq_init());
  if (option == 0) test_case(1024, repeat);
  else if (option == 1) test_case(4096, repeat);
  else test_case(12288, repeat);
  return 0;
}
