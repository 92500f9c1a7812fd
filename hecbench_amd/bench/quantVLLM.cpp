// quantVLLM driver: same command line, inputs, verification and printed lines as the
// HeCBench benchmark (src/quantVLLM-hip/main.cu), on top of libhq.
//
//   quantVLLM <number of tokens> <hidden size> <repeat>
#include "bench_common.h"

namespace {

// Host statements of the reference checks (src/quantVLLM-cuda/reference.h, utils.h).
int8_t float_to_int8_rn(float x) {
  float dst = std::nearbyint(x);
  dst = dst < -128.f ? -128.f : (127.f < dst ? 127.f : dst);
  return (int8_t)dst;
}
int32_t float_to_int32_rn(float x) {
  const float dst = std::nearbyint(x);
  if (dst >= 2147483648.f) return INT32_MAX;
  if (dst <= -2147483648.f) return INT32_MIN;
  return (int32_t)dst;
}
int8_t int32_to_int8(int32_t x) { return (int8_t)(x < -128 ? -128 : (127 < x ? 127 : x)); }

struct HostRef {
  const std::vector<float>& x;  // inputs widened to fp32 (exact for all three types)
  int64_t tokens;
  int hidden;
  void stat(std::vector<int8_t>& out, float scale, bool has_azp, int32_t azp) const {
    for (size_t i = 0; i < x.size(); ++i)
      out[i] = has_azp ? int32_to_int8(float_to_int32_rn(x[i] / scale) + azp) : float_to_int8_rn(x[i] / scale);
  }
  void dyn(std::vector<int8_t>& out, bool with_azp) const {
    for (int64_t t = 0; t < tokens; ++t) {
      const float* r = x.data() + t * hidden;
      if (!with_azp) {
        float absmax = 0.f;
        for (int i = 0; i < hidden; ++i) absmax = std::max(absmax, std::fabs(r[i]));
        const float tmp = 127.0f / absmax;
        for (int i = 0; i < hidden; ++i) out[t * hidden + i] = float_to_int8_rn(r[i] * tmp);
      } else {
        float mx = std::numeric_limits<float>::min(), mn = std::numeric_limits<float>::max();
        for (int i = 0; i < hidden; ++i) { mx = std::max(mx, r[i]); mn = std::min(mn, r[i]); }
        const float sc = (mx - mn) / 255.0f;
        const int32_t z = (int32_t)std::nearbyint(-128.0f - mn / sc);
        for (int i = 0; i < hidden; ++i) out[t * hidden + i] = int32_to_int8(float_to_int32_rn(r[i] / sc) + z);
      }
    }
  }
};

uint16_t f32_to_bf16_bits(float f) {  // exact for the integer fixture values
  uint32_t u;
  std::memcpy(&u, &f, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
float bf16_bits_to_f32(uint16_t h) {
  const uint32_t u = (uint32_t)h << 16;
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}

void quant(int dtype, int num_tokens, int hidden_size, int repeat) {
  const size_t n = (size_t)num_tokens * hidden_size;
  const int esz = dtype == HQ_DTYPE_F32 ? 4 : 2;
  std::vector<float> xf(n);
  std::vector<uint8_t> raw(n * esz);
  srand(123);
  for (size_t i = 0; i < n; ++i) {
    const float v = (float)(rand() % 1000 - 300);  // main.cu:186-189
    if (dtype == HQ_DTYPE_F32) { std::memcpy(&raw[4 * i], &v, 4); xf[i] = v; }
    else if (dtype == HQ_DTYPE_F16) { const uint16_t h = f32_to_f16_bits(v); std::memcpy(&raw[2 * i], &h, 2); xf[i] = f16_bits_to_f32(h); }
    else { const uint16_t h = f32_to_bf16_bits(v); std::memcpy(&raw[2 * i], &h, 2); xf[i] = bf16_bits_to_f32(h); }
  }
  DevBuf<uint8_t> d_in(raw.size());
  d_in.upload(raw);
  DevBuf<int8_t> d_out(n);
  DevBuf<float> d_scale(num_tokens);
  DevBuf<int32_t> d_azp(num_tokens);
  std::vector<int8_t> h_out(n), h_ref(n);
  const HostRef ref{xf, num_tokens, hidden_size};
  const float scale = 0.1f;
  int error = 0;
  auto timed = [&](const char* name, auto&& call, auto&& check) {
    auto start = std::chrono::steady_clock::now();
    for (int i = 0; i < repeat; ++i) call();
    HIP_OK(hipDeviceSynchronize());
    auto end = std::chrono::steady_clock::now();
    const double t = std::chrono::duration<double, std::nano>(end - start).count();
    std::printf("Average execution time of %s kernel: %f (us)\n", name, (t * 1e-3) / repeat);
    d_out.download(h_out.data(), n);
    check();
    error += std::memcmp(h_out.data(), h_ref.data(), n) != 0;
  };
  timed("static_scaled_int8_quant",
        [&] { HQ_OK_OR_DIE(hq_int8_quant_static(d_in.p, dtype, d_out.p, num_tokens, hidden_size, scale, 0, 0, nullptr)); },
        [&] { ref.stat(h_ref, scale, false, 0); });
  timed("static_scaled_int8_quant_azp",
        [&] { HQ_OK_OR_DIE(hq_int8_quant_static(d_in.p, dtype, d_out.p, num_tokens, hidden_size, scale, 1, 54, nullptr)); },
        [&] { ref.stat(h_ref, scale, true, 54); });
  timed("dynamic_scaled_int8_quant",
        [&] { HQ_OK_OR_DIE(hq_int8_quant_dynamic(d_in.p, dtype, d_out.p, d_scale.p, nullptr, num_tokens, hidden_size, nullptr)); },
        [&] { ref.dyn(h_ref, false); });
  timed("dynamic_scaled_int8_quant_azp",
        [&] { HQ_OK_OR_DIE(hq_int8_quant_dynamic(d_in.p, dtype, d_out.p, d_scale.p, d_azp.p, num_tokens, hidden_size, nullptr)); },
        [&] { ref.dyn(h_ref, true); });
  std::printf("%s\n", error ? "FAIL" : "PASS");
}

}  // namespace

int main(int argc, char* argv[]) {
  if (argc != 4) {
    std::printf("Usage: %s <number of tokens> <hidden size> <repeat>\n", argv[0]);
    return 1;
  }
  const int num_tokens = std::atoi(argv[1]), hidden_size = std::atoi(argv[2]), repeat = std::atoi(argv[3]);
  HQ_OK_OR_DIE(hq_init());
  std::printf("Input type is FP16\n");
  quant(HQ_DTYPE_F16, num_tokens, hidden_size, repeat);
  std::printf("Input type is BF16\n");
  quant(HQ_DTYPE_BF16, num_tokens, hidden_size, repeat);
  std::printf("Input type is FP32\n");
  quant(HQ_DTYPE_F32, num_tokens, hidden_size, repeat);
  return 0;
}
