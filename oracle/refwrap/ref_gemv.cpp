// Test infrastructure: the reference gemv kernels (src/gemv-hip/kernels.h, HeCBench tree)
// behind C entry points, launched the way src/gemv-hip/gemv.cu:10-133 launches them.
#include "kernels.h"

#define EXPORT extern "C" __attribute__((visibility("default")))

// n x n problem, block (bx, by), grid (1, n / by); all pointers are device pointers.
EXPORT void ref_gemv_fp16(void* mat, void* vec, void* res, unsigned n, unsigned bx, unsigned by, void* stream) {
  gemv_fp16<64><<<dim3(1, n / by), dim3(bx, by), 0, (hipStream_t)stream>>>((__half*)mat, (__half*)vec, (__half*)res,
                                                                          n, n / bx);
}
EXPORT void ref_gemv_int8(void* mat, void* vec, void* res, unsigned n, float scale, float zero_point, unsigned bx,
                          unsigned by, void* stream) {
  gemv_quantized_int8<64><<<dim3(1, n / by), dim3(bx, by), 0, (hipStream_t)stream>>>(
      (int8_t*)mat, (__half*)vec, (__half*)res, n, __float2half(scale), __float2half(zero_point), n / bx);
}
EXPORT void ref_gemv_int4(void* mat, void* vec, void* res, unsigned n, float scale, float zero_point, unsigned bx,
                          unsigned by, void* stream) {
  gemv_quantized_int4<64><<<dim3(1, n / by), dim3(bx, by), 0, (hipStream_t)stream>>>(
      (uint4_2*)mat, (__half*)vec, (__half*)res, n, __float2half(scale), __float2half(zero_point), n / bx);
}
