// Test infrastructure: the reference quant3MatMul launchers
// (src/quant3MatMul-hip/kernels.h, HeCBench tree) behind C entry points.
#include "kernels.h"

extern "C" __attribute__((visibility("default"))) void ref_vecquant3matmul_f32(float* vec, int* mat, float* mul, float* scales, float* zeros,
                                        int height, int width) {
  vecquant3matmul<float>(vec, mat, mul, scales, zeros, height, width);
}
extern "C" __attribute__((visibility("default"))) void ref_vecquant3matmul_faster(void* vec_f16, int* mat, float* mul, float* scales,
                                           float* zeros, int height, int width) {
  vecquant3matmul_faster((half*)vec_f16, mat, mul, scales, zeros, height, width);
}
