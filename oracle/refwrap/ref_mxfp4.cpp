// Test infrastructure: the reference mxfp4 quantise-dequantise kernel
// (src/mxfp4-hip/main.cu, HeCBench tree) behind C entry points.
#define main hecbench_mxfp4_main
#include "main.cu"
#undef main

#define EXPORT extern "C" __attribute__((visibility("default")))

// numel a multiple of 64; device pointers; the launch shape of mxfp4(), main.cu:144-160.
EXPORT void ref_mxfp4_qdq(const void* in, void* out, int numel, int is_bf16, void* stream) {
  const int block = numel % 128 == 0 ? 128 : 64;
  if (is_bf16)
    qdq_mxfp4_kernel<__hip_bfloat16, BFLOAT16_EXP_BITS, BFLOAT16_MANTISSA_BITS, BFLOAT16_EXP_BIAS, BFLOAT16_VAL_TO_ADD,
                     BFLOAT16_SIGN_EXPONENT_MASK><<<numel / block, block, 0, (hipStream_t)stream>>>(
        (const __hip_bfloat16*)in, (__hip_bfloat16*)out);
  else
    qdq_mxfp4_kernel<__half, FLOAT16_EXP_BITS, FLOAT16_MANTISSA_BITS, FLOAT16_EXP_BIAS, FLOAT16_VAL_TO_ADD,
                     FLOAT16_SIGN_EXPONENT_MASK><<<numel / block, block, 0, (hipStream_t)stream>>>((const __half*)in,
                                                                                                   (__half*)out);
}
