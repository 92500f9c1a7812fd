// Test infrastructure: the reference host loops of quantVLLM (src/quantVLLM-cuda/reference.h and
// utils.h, HeCBench tree) and its device kernels (src/quantVLLM-hip/main.cu) behind C entry points.
// The reference's device kernels and their launchers (src/quantVLLM-hip/main.cu) come in with it.
#include <cstdint>
#include <limits>
#define main hecbench_quantvllm_hip_main
#include "main.cu"  // pulls in utils.h and reference.h
#undef main

#define EXPORT extern "C" __attribute__((visibility("default")))

template <typename T>
static void run_static(const void* x, int8_t* out, long tokens, int hidden, float scale, int has_azp, int azp) {
  if (has_azp) static_scaled_int8_azp_quant_reference((const T*)x, out, scale, (int32_t)azp, (int64_t)tokens, hidden);
  else static_scaled_int8_quant_reference((const T*)x, out, scale, (int64_t)tokens, hidden);
}
template <typename T>
static void run_dynamic(const void* x, int8_t* out, float* scales, int32_t* azp, long tokens, int hidden) {
  if (azp) dynamic_scaled_int8_azp_quant_reference((const T*)x, out, scales, azp, (int64_t)tokens, hidden);
  else dynamic_scaled_int8_quant_reference((const T*)x, out, scales, (int64_t)tokens, hidden);
}
// dtype: 0 fp32, 1 fp16, 2 bf16
EXPORT void ref_int8_quant_static(const void* x, int dtype, int8_t* out, long tokens, int hidden, float scale,
                                  int has_azp, int azp) {
  if (dtype == 0) run_static<float>(x, out, tokens, hidden, scale, has_azp, azp);
  else if (dtype == 1) run_static<__half>(x, out, tokens, hidden, scale, has_azp, azp);
  else run_static<__hip_bfloat16>(x, out, tokens, hidden, scale, has_azp, azp);
}
EXPORT void ref_int8_quant_dynamic(const void* x, int dtype, int8_t* out, float* scales, int32_t* azp, long tokens,
                                   int hidden) {
  if (dtype == 0) run_dynamic<float>(x, out, scales, azp, tokens, hidden);
  else if (dtype == 1) run_dynamic<__half>(x, out, scales, azp, tokens, hidden);
  else run_dynamic<__hip_bfloat16>(x, out, scales, azp, tokens, hidden);
}

// The device launchers of src/quantVLLM-hip/main.cu:140-168 (default stream; azp == 0 selects the
// kernels without a zero point, as there).
EXPORT void ref_hip_int8_quant_static(const void* x, int dtype, int8_t* out, long tokens, int hidden, float scale,
                                      int azp) {
  if (dtype == 0) static_scaled_int8_quant<float>(out, (const float*)x, hidden, (int)tokens, scale, azp);
  else if (dtype == 1) static_scaled_int8_quant<__half>(out, (const __half*)x, hidden, (int)tokens, scale, azp);
  else static_scaled_int8_quant<__hip_bfloat16>(out, (const __hip_bfloat16*)x, hidden, (int)tokens, scale, azp);
}
EXPORT void ref_hip_int8_quant_dynamic(const void* x, int dtype, int8_t* out, float* scales, int32_t* azp,
                                       long tokens, int hidden) {
  if (dtype == 0) dynamic_scaled_int8_quant<float>(out, (const float*)x, hidden, (int)tokens, scales, azp);
  else if (dtype == 1) dynamic_scaled_int8_quant<__half>(out, (const __half*)x, hidden, (int)tokens, scales, azp);
  else dynamic_scaled_int8_quant<__hip_bfloat16>(out, (const __hip_bfloat16*)x, hidden, (int)tokens, scales, azp);
}
