// Test infrastructure: the reference kQuantize kernel (src/quantBnB-hip/main.cu,
// HeCBench tree) behind a C entry point.
#define main hecbench_quantbnb_hip_main
#include "main.cu"
#undef main

extern "C" __attribute__((visibility("default"))) void ref_kquantize(const float* d_code, const float* d_A, unsigned char* d_out, long n,
                              void* stream) {
  const int block_size = 256;
  dim3 grid((n + block_size - 1) / block_size);
  dim3 block(block_size);
  kQuantize<block_size, block_size><<<grid, block, 0, (hipStream_t)stream>>>(d_code, d_A, d_out, n);
}
extern "C" __attribute__((visibility("default"))) const float* ref_hip_code_table(void) { return code; }
