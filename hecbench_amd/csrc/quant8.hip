// bitsandbytes dynamic-map 8-bit quantisation for gfx950.
//
// Replaces dQuantize<0> / kQuantize<256,256> (src/quantBnB-hip/main.cu:13-130 in
// the HeCBench tree): a 7-step binary search over the sorted 256-entry code
// table followed by a midpoint comparison against the neighbour on the side of x
// (ties keep the pivot).  Bit-exact with the reference for every input.
// A lane converts four consecutive floats (one 128-bit load) into one packed
// 32-bit store; the table is read from LDS in level order.
#include "hq_internal.h"

namespace {

typedef float f4v __attribute__((ext_vector_type(4)));

// The reference search (pivot 127, steps 64..1) walks a perfect binary tree over the table
// entries 0..254 whose leaves are the even indices.  Two facts make it cheap:
//  * stored level by level (node j of level k at (1 << (k-1)) - 1 + j, holding entry
//    ((2j+1) << (8-k)) - 1), the nodes one level touches are contiguous in LDS, so lanes on
//    different nodes hit different banks instead of a few banks 2^(8-k) entries apart;
//  * the bounds the reference tracks on the way down are, at the leaf p, always the
//    neighbours p+1 (the nearest ancestor above; entry 255 when p = 254) and max(p-1, 0)
//    (the nearest ancestor below), so they need not be tracked, only looked up at the end.
// lds: [0..254] level order, [256..511] the table in index order.
__device__ __forceinline__ uint32_t quantize_one(const float* lds, float x) {
  uint32_t j = 0;
  float val = lds[0];
#pragma unroll
  for (int k = 1; k < 8; ++k) {
    j = 2 * j + (x > val ? 1u : 0u);
    val = lds[(1u << k) - 1 + j];
  }
  const uint32_t pivot = 2 * j;  // leaf index = table index
  const bool up = x > val;
  const uint32_t other = up ? pivot + 1 : (pivot == 0 ? 0u : pivot - 1);
  const float bound = lds[256 + other];
  const float midpoint = (bound + val) * 0.5f;
  // ties keep the pivot (strict comparisons, src/quantBnB-hip/main.cu:47-65)
  return (up ? x > midpoint : x < midpoint) ? other : pivot;
}

__global__ __launch_bounds__(256) void quantize8_kernel(const float* __restrict__ code,
                                                       const float* __restrict__ A,
                                                       uint8_t* __restrict__ out, int64_t n,
                                                       int vec_ok) {
  __shared__ float s_code[512];
  {
    const int t = threadIdx.x;  // level-order slot t <- table entry ((2j+1) << (8-k)) - 1
    if (t < 255) {
      const int k = 32 - __builtin_clz((unsigned)t + 1);  // level 1..8
      const int j = t + 1 - (1 << (k - 1));
      s_code[t] = code[((2 * j + 1) << (8 - k)) - 1];
    }
    s_code[256 + t] = code[t];
  }
  __syncthreads();
  const int64_t nquads = vec_ok ? n / 4 : 0;
  const int64_t stride = (int64_t)gridDim.x * 256;
  const int64_t t0 = (int64_t)blockIdx.x * 256 + threadIdx.x;
  // Two quads per trip, searched in lockstep level by level: eight independent LDS reads
  // are in flight per level instead of one dependent chain per element.
  for (int64_t i = t0; i < nquads; i += 2 * stride) {
    const int64_t i1 = i + stride;
    const bool two = i1 < nquads;
    const f4v v0 = __builtin_nontemporal_load(reinterpret_cast<const f4v*>(A) + i);
    const f4v v1 = __builtin_nontemporal_load(reinterpret_cast<const f4v*>(A) + (two ? i1 : i));
    const float x[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
    uint32_t j[8];
    float val[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) { j[e] = 0; val[e] = s_code[0]; }
#pragma unroll
    for (int k = 1; k < 8; ++k) {
#pragma unroll
      for (int e = 0; e < 8; ++e) j[e] = 2 * j[e] + (x[e] > val[e] ? 1u : 0u);
#pragma unroll
      for (int e = 0; e < 8; ++e) val[e] = s_code[(1u << k) - 1 + j[e]];
    }
    uint32_t other[8];
    float bound[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint32_t pivot = 2 * j[e];
      other[e] = x[e] > val[e] ? pivot + 1 : (pivot == 0 ? 0u : pivot - 1);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) bound[e] = s_code[256 + other[e]];
    uint32_t q[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float midpoint = (bound[e] + val[e]) * 0.5f;
      const bool up = x[e] > val[e];
      q[e] = (up ? x[e] > midpoint : x[e] < midpoint) ? other[e] : 2 * j[e];
    }
    __builtin_nontemporal_store(q[0] | (q[1] << 8) | (q[2] << 16) | (q[3] << 24),
                                reinterpret_cast<uint32_t*>(out) + i);
    if (two)
      __builtin_nontemporal_store(q[4] | (q[5] << 8) | (q[6] << 16) | (q[7] << 24),
                                  reinterpret_cast<uint32_t*>(out) + i1);
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
