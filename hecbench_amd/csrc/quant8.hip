// bitsandbytes dynamic-map 8-bit quantisation for gfx950.
//
// Replaces dQuantize<0> / kQuantize<256,256> (src/quantBnB-hip/main.cu:13-130 in
// the HeCBench tree): a 7-step binary search over the sorted 256-entry code
// table followed by a midpoint comparison against the neighbour on the side of x
// (ties keep the pivot).  Bit-exact with the reference for every input.
// A lane converts four consecutive floats (one 128-bit load) into one packed
// 32-bit store; the table is read from LDS.
#include "hq_internal.h"

namespace {

typedef float f4v __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t quantize_one(const float* code, float x) {
  int pivot = 127, upper_pivot = 255, lower_pivot = 0;
  float lower = -1.0f, upper = 1.0f;
  float val = code[pivot];
#pragma unroll
  for (int i = 64; i > 0; i >>= 1) {
    if (x > val) { lower_pivot = pivot; lower = val; pivot += i; }
    else         { upper_pivot = pivot; upper = val; pivot -= i; }
    val = code[pivot];
  }
  if (upper_pivot == 255) upper = code[upper_pivot];
  if (lower_pivot == 0) lower = code[lower_pivot];
  if (x > val) {
    const float midpoint = (upper + val) * 0.5f;
    return x > midpoint ? upper_pivot : pivot;
  }
  const float midpoint = (lower + val) * 0.5f;
  return x < midpoint ? lower_pivot : pivot;
}

__global__ __launch_bounds__(256) void quantize8_kernel(const float* __restrict__ code,
                                                       const float* __restrict__ A,
                                                       uint8_t* __restrict__ out, int64_t n,
                                                       int vec_ok) {
  __shared__ float s_code[256];
  s_code[threadIdx.x] = code[threadIdx.x];
  __syncthreads();
  const int64_t nquads = vec_ok ? n / 4 : 0;
  const int64_t stride = (int64_t)gridDim.x * 256;
  const int64_t t0 = (int64_t)blockIdx.x * 256 + threadIdx.x;
  for (int64_t i = t0; i < nquads; i += stride) {
    const f4v v = __builtin_nontemporal_load(reinterpret_cast<const f4v*>(A) + i);
    const uint32_t q = quantize_one(s_code, v.x) | (quantize_one(s_code, v.y) << 8) |
                       (quantize_one(s_code, v.z) << 16) | (quantize_one(s_code, v.w) << 24);
    __builtin_nontemporal_store(q, reinterpret_cast<uint32_t*>(out) + i);
  }
  for (int64_t e = nquads * 4 + t0; e < n; e += stride) out[e] = (uint8_t)quantize_one(s_code, A[e]);
}

}  // namespace

extern "C" int hq_quantize_dynamic8(const float* code, const float* A, uint8_t* out, int64_t n,
                                    void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (n < 0) return HQ_ERR_BAD_SHAPE;
  if (n == 0) return HQ_OK;
  if (!code || !A || !out) return HQ_ERR_NULL_POINTER;
  if (((uintptr_t)code & 3) || ((uintptr_t)A & 3)) return HQ_ERR_MISALIGNED;
  const HqDevice* dev = nullptr;
  int rc = hq_current_device(&dev);
  if (rc != HQ_OK) return rc;
  const int vec_ok = !((uintptr_t)A & 15) && !((uintptr_t)out & 3);
  int64_t blocks = (n / 4 + 255) / 256;
  const int64_t cap = (int64_t)dev->cus * 16;
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(quantize8_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, code, A, out, n,
                     vec_ok);
  return hq_launch_status();
}
