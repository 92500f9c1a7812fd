// Device-side packers and the 4-bit blockwise quantiser: the inverses of the unpack /
// dequantise steps of the matvec kernels, so that the family round-trips on the GPU.
//
//   hq_q3_pack       codes uint8 [K][N]          -> int32 [3K/32][N]   (layout of
//                                                    src/quant3MatMul-hip/kernels.h:42-86)
//   hq_bcq_pack      signs int8 [K][nb][N]       -> uint32 [K/32][nb][N] (bit packing of
//                                                    src/lut-gemm-hip/main.cu:118-134)
//   hq_quantize_4bit fp32 / fp16 [n]             -> packed nibbles + fp32 absmax per block
//                                                    (inverse of hq_dequant_nf4; no counterpart
//                                                    in the HeCBench tree)
#include "hq_internal.h"

namespace {

__global__ __launch_bounds__(256) void q3_pack_kernel(const uint8_t* __restrict__ codes,
                                                     uint32_t* __restrict__ mat, int G, int N) {
  // thread -> (k-group g, column n); consecutive threads take consecutive columns
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= (int64_t)G * N) return;
  const int g = (int)(t / N), n = (int)(t % N);
  const uint8_t* src = codes + (size_t)(32 * g) * N + n;
  uint64_t lo = 0;   // bits 0..63 of the 96-bit string
  uint32_t hi = 0;   // bits 64..95
#pragma unroll
  for (int i = 0; i < 32; ++i) {
    const uint64_t q = src[(size_t)i * N] & 7u;
    const int bit = 3 * i;
    if (bit < 64) lo |= q << bit;
    if (bit > 61) hi |= (uint32_t)(bit >= 64 ? q << (bit - 64) : q >> (64 - bit));
  }
  uint32_t* dst = mat + (size_t)(3 * g) * N + n;
  dst[0] = (uint32_t)lo;
  dst[N] = (uint32_t)(lo >> 32);
  dst[2 * (size_t)N] = hi;
}

__global__ __launch_bounds__(256) void bcq_pack_kernel(const int8_t* __restrict__ signs,
                                                      uint32_t* __restrict__ bW, int KW, int NB, int N) {
  // thread -> (k-word, plane, column)
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t per_word = (int64_t)NB * N;
  if (t >= (int64_t)KW * per_word) return;
  const int kw = (int)(t / per_word);
  const int64_t rest = t % per_word;  // = b*N + n
  const int8_t* src = signs + (size_t)(32 * kw) * per_word + rest;
  uint32_t w = 0;
#pragma unroll
  for (int i = 0; i < 32; ++i) w |= (src[(size_t)i * per_word] > 0 ? 1u : 0u) << i;
  bW[t] = w;
}

// bitsandbytes code books (same literals as the dequantiser)
__constant__ float c_q_nf4[16] = {
    -1.0f, -0.6961928009986877f, -0.5250730514526367f, -0.39491748809814453f,
    -0.28444138169288635f, -0.18477343022823334f, -0.09105003625154495f, 0.0f,
    0.07958029955625534f, 0.16093020141124725f, 0.24611230194568634f,
    0.33791524171829224f, 0.44070982933044434f, 0.5626170039176941f,
    0.7229568362236023f, 1.0f};

// Nearest NF4 code of a value normalised to [-1, 1]: the number of midpoints between
// adjacent table entries (fp32 (a+b)*0.5) that lie strictly below it, so a value exactly
// on a midpoint takes the lower code.
__device__ __forceinline__ uint32_t nearest_nf4(const float* mid, float v) {
  uint32_t c = 0;
#pragma unroll
  for (int step = 8; step > 0; step >>= 1) c += (v > mid[c + step - 1]) ? step : 0;  // mid[0..14]
  return c;
}

// FP4 (sign bit 3, magnitudes {0, 1/192, 2/3, 1, 1/3, 1/2, 1/6, 1/4}): nearest magnitude,
// ties to the smaller one; codes in increasing magnitude order are 0,1,6,7,4,5,2,3.
__device__ __forceinline__ uint32_t nearest_fp4(float v) {
  const float a = fabsf(v);
  const float mags[8] = {0.0f, 0.005208333333f, 0.16666667f, 0.25f, 0.33333333f, 0.5f, 0.66666667f, 1.0f};
  const uint32_t code_of[8] = {0, 1, 6, 7, 4, 5, 2, 3};
  uint32_t idx = 0;
#pragma unroll
  for (int i = 0; i < 7; ++i) idx += (a > (mags[i] + mags[i + 1]) * 0.5f) ? 1u : 0u;
  return code_of[idx] | (v < 0.f ? 8u : 0u);
}

// One wave per block of `blocksize` elements: absmax by a cross-lane butterfly, then one
// packed byte (two codes) per lane and stride of 64.
template <typename T>
__global__ __launch_bounds__(256) void quantize4_kernel(const T* __restrict__ x, uint8_t* __restrict__ packed,
                                                       float* __restrict__ absmax, int64_t n, int blocksize,
                                                       int table) {
  __shared__ float mid[16];
  if (threadIdx.x < 15) mid[threadIdx.x] = (c_q_nf4[threadIdx.x] + c_q_nf4[threadIdx.x + 1]) * 0.5f;
  __syncthreads();
  const int lane = threadIdx.x & 63;
  const int64_t block = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t e0 = block * blocksize;
  if (e0 >= n) return;  // wave-uniform
  const int64_t e1 = e0 + blocksize < n ? e0 + blocksize : n;
  float amax = 0.f;
  for (int64_t e = e0 + lane; e < e1; e += 64) amax = fmaxf(amax, fabsf((float)x[e]));
#pragma unroll
  for (int m = 32; m > 0; m >>= 1) amax = fmaxf(amax, __shfl_xor(amax, m));
  if (lane == 0) absmax[block] = amax;
  const float inv = amax > 0.f ? 1.0f / amax : 0.f;
  // pairs of elements -> one byte, high nibble first; blocksize is even so pairs never straddle blocks
  for (int64_t p = e0 / 2 + lane; 2 * p < e1; p += 64) {
    const float v0 = (float)x[2 * p] * inv;
    const bool has1 = 2 * p + 1 < n;  // odd n: the last low nibble is padding and stays 0
    const float v1 = has1 ? (float)x[2 * p + 1] * inv : 0.f;
    const uint32_t c0 = table ? nearest_fp4(v0) : nearest_nf4(mid, v0);
    const uint32_t c1 = has1 ? (table ? nearest_fp4(v1) : nearest_nf4(mid, v1)) : 0u;
    packed[p] = (uint8_t)((c0 << 4) | c1);
  }
}

}  // namespace

extern "C" int hq_q3_pack(const uint8_t* codes, int32_t* qweight, int K, int N, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!codes || !qweight) return HQ_ERR_NULL_POINTER;
  if (K <= 0 || N <= 0 || (K & 31)) return HQ_ERR_BAD_SHAPE;
  if ((uintptr_t)qweight & 3) return HQ_ERR_MISALIGNED;
  const HqDevice* dev = nullptr;
  int rc = hq_current_device(&dev);
  if (rc != HQ_OK) return rc;
  const int64_t total = (int64_t)(K / 32) * N;
  if ((total + 255) / 256 > 0x7fffffff) return HQ_ERR_TOO_LARGE;
  hipLaunchKernelGGL(q3_pack_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, codes,
                     reinterpret_cast<uint32_t*>(qweight), K / 32, N);
  return hq_launch_status();
}

extern "C" int hq_bcq_pack(const int8_t* signs, uint32_t* bW, int K, int N, int nbits, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!signs || !bW) return HQ_ERR_NULL_POINTER;
  if (K <= 0 || N <= 0 || (K & 31) || nbits < 1 || nbits > 8) return HQ_ERR_BAD_SHAPE;
  if ((uintptr_t)bW & 3) return HQ_ERR_MISALIGNED;
  const HqDevice* dev = nullptr;
  int rc = hq_current_device(&dev);
  if (rc != HQ_OK) return rc;
  const int64_t total = (int64_t)(K / 32) * nbits * N;
  if ((total + 255) / 256 > 0x7fffffff) return HQ_ERR_TOO_LARGE;
  hipLaunchKernelGGL(bcq_pack_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, signs, bW, K / 32,
                     nbits, N);
  return hq_launch_status();
}

extern "C" int hq_quantize_4bit(const void* x, int x_dtype, uint8_t* packed, float* absmax, int64_t n_elems,
                                int blocksize, int table, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (n_elems < 0 || blocksize <= 0 || (blocksize & 1)) return HQ_ERR_BAD_SHAPE;
  if (x_dtype != HQ_DTYPE_F32 && x_dtype != HQ_DTYPE_F16) return HQ_ERR_BAD_ENUM;
  if (table != HQ_TABLE_NF4 && table != HQ_TABLE_FP4) return HQ_ERR_BAD_ENUM;
  if (n_elems == 0) return HQ_OK;
  if (!x || !packed || !absmax) return HQ_ERR_NULL_POINTER;
  if (((uintptr_t)x & (x_dtype == HQ_DTYPE_F16 ? 1 : 3)) || ((uintptr_t)absmax & 3)) return HQ_ERR_MISALIGNED;
  const HqDevice* dev = nullptr;
  int rc = hq_current_device(&dev);
  if (rc != HQ_OK) return rc;
  const int64_t nblocks = (n_elems + blocksize - 1) / blocksize;
  if ((nblocks + 3) / 4 > 0x7fffffff) return HQ_ERR_TOO_LARGE;
  const dim3 grid((unsigned)((nblocks + 3) / 4));
  if (x_dtype == HQ_DTYPE_F16)
    hipLaunchKernelGGL(quantize4_kernel<_Float16>, grid, dim3(256), 0, stream, (const _Float16*)x, packed, absmax,
                       n_elems, blocksize, table);
  else
    hipLaunchKernelGGL(quantize4_kernel<float>, grid, dim3(256), 0, stream, (const float*)x, packed, absmax, n_elems,
                       blocksize, table);
  return hq_launch_status();
}
