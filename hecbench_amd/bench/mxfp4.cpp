// mxfp4: the command line, inputs, printed lines and verification rules of the HeCBench benchmark
// (src/mxfp4-hip/main.cu, src/mxfp4-cuda/verify.h) on top of libhq.
//
//   mxfp4 <number of elements> <repeat>
#include "bench_common.h"

namespace {

uint16_t f32_to_bf16_bits(float f) {  // round to nearest even
  uint32_t b;
  std::memcpy(&b, &f, 4);
  b += 0x7fffu + ((b >> 16) & 1u);
  return (uint16_t)(b >> 16);
}
float bf16_bits_to_f32(uint16_t h) {
  const uint32_t b = (uint32_t)h << 16;
  float f;
  std::memcpy(&f, &b, 4);
  return f;
}

// The acceptance rules of the reference (verify.h:3-88): exact answers for the ties and the
// open intervals between grid points, 1e-3 otherwise.
bool acceptable(float s, float d) {
  if (s == 0.25f) return d == 0.f;
  if (s == 0.75f || s == 1.25f) return d == 1.f;
  if (s == 1.75f || s == 2.5f) return d == 2.f;
  if (s == 3.5f || s == 5.0f) return d == 4.f;
  if (s > 0.5f && s < 0.75f) return d == 0.5f;
  if (s > 0.f && s < 0.25f) return d == 0.f;
  if (s > 0.25f && s < 0.5f) return d == 0.5f;
  if (s > 0.75f && s < 1.f) return d == 1.f;
  if (s < -0.5f && s > -0.75f) return d == -0.5f;
  if (s < 0.f && s > -0.25f) return d == -0.f;
  if (s < -0.25f && s > -0.5f) return d == -0.5f;
  if (s < -0.75f && s > -1.f) return d == -1.f;
  return std::fabs(s - d) <= 1e-3f;
}

void mxfp4_sim(bool bf16, int numel, int niters) {
  std::vector<uint16_t> src(numel), dst(numel);
  const float v[] = {0.0, 0.5, 1.0, 1.5, 2, 3, 4, -0.0, -0.5, -1.0, -1.5, -2, -3, -4, 0.25, 0.75,
                     1.25, 1.75, 2.5, 3.5, 5, 0.1, 0.3, 0.4, 0.6, 0.9, -0.1, -0.3, -0.4, -0.6, -0.9};
  auto enc = [&](float f) { return bf16 ? f32_to_bf16_bits(f) : f32_to_f16_bits(f); };
  auto dec = [&](uint16_t h) { return bf16 ? bf16_bits_to_f32(h) : f16_bits_to_f32(h); };
  srand(123);  // main.cu:187-193: one +-6 per group of 32 fixes the shared scale at 1
  for (int i = 0; i < numel / 32; i++) {
    for (int j = i * 32; j < (i + 1) * 32; j++) src[j] = enc(v[rand() % (sizeof(v) / sizeof(v[0]))]);
    const int r = rand() % 32;
    src[i * 32 + r] = enc(r < 16 ? 6.f : -6.f);
  }
  DevBuf<uint16_t> d_src(numel), d_dst(numel);
  d_src.upload(src);
  const int dtype = bf16 ? HQ_DTYPE_BF16 : HQ_DTYPE_F16;
  HQ_OK_OR_DIE(hq_mxfp4_qdq(d_src.p, d_dst.p, numel, dtype, nullptr));  // warm-up
  HIP_OK(hipDeviceSynchronize());
  auto start = std::chrono::high_resolution_clock::now();
  for (int i = 0; i < niters; i++) HQ_OK_OR_DIE(hq_mxfp4_qdq(d_src.p, d_dst.p, numel, dtype, nullptr));
  HIP_OK(hipDeviceSynchronize());
  auto end = std::chrono::high_resolution_clock::now();
  const double time = std::chrono::duration<double>(end - start).count() / niters;
  const double size = 2.0 * 2.0 * numel / 1.0e9;
  std::printf("size(GB):%.2f, average time(sec):%f, Bandwidth (GB/sec):%f\n", size, time, size / time);
  std::printf("  (%.2f us per call, %.1f%% of 8000 GB/s)\n", time * 1e6, 100.0 * size / time / 8000.0);
  d_dst.download(dst.data(), numel);
  bool ok = true;
  for (int i = 0; i < numel && ok; i++) {
    const float s = dec(src[i]), d = dec(dst[i]);
    if (!acceptable(s, d)) {
      std::printf("%f %f\n", s, d);
      ok = false;
    }
  }
  std::printf("%s\n", ok ? "PASS" : "FAIL");
}

}  // namespace

int main(int argc, char* argv[]) {
  if (argc != 3) {
    std::printf("Usage: %s <number of elements> <repeat>\n", argv[0]);
    return 1;
  }
  const int numel = std::atoi(argv[1]), niters = std::atoi(argv[2]);
  if (numel <= 0 || numel % 64 || niters <= 0) {
    std::printf("Expected qdq_mxfp4 input number of elements to be a multiple of 64, but it is not!");
    return 1;
  }
  HQ_OK_OR_DIE(hq_init());
  mxfp4_sim(false, numel, niters);
  mxfp4_sim(true, numel, niters);
  return 0;
}
