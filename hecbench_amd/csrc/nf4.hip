// Blockwise 4-bit (NF4 / FP4) dequantisation to fp16 for gfx950.
//
//   out[2i]   = fp16_rn(table[packed[i] >> 4] * absmax[(2i)   / blocksize])
//   out[2i+1] = fp16_rn(table[packed[i] & 15] * absmax[(2i+1) / blocksize])
//
// Pure streaming, write-dominated (64 bytes out per 16 bytes in).  A lane owns 16 packed bytes (one 128-bit load, 32 codes) and
// writes 64 contiguous bytes as four 128-bit nontemporal stores.  The 16-entry
// code book sits in LDS: 16 entries occupy 16 distinct banks, so lanes that hit
// the same bank always hit the same address (broadcast) and the lookups are
// conflict-free.  The multiply is a single fp32 operation followed by one
// round-to-nearest-even conversion, which is the bit-exact contract.
#include "hq_internal.h"

namespace {

typedef uint32_t u4v __attribute__((ext_vector_type(4)));
typedef _Float16 h2v __attribute__((ext_vector_type(2)));

// bitsandbytes NF4 code book (fp32 literals of the upstream library).
__constant__ float c_nf4[16] = {
    -1.0f, -0.6961928009986877f, -0.5250730514526367f, -0.39491748809814453f,
    -0.28444138169288635f, -0.18477343022823334f, -0.09105003625154495f, 0.0f,
    0.07958029955625534f, 0.16093020141124725f, 0.24611230194568634f,
    0.33791524171829224f, 0.44070982933044434f, 0.5626170039176941f,
    0.7229568362236023f, 1.0f};
// bitsandbytes FP4 decode tree: bit 3 sign, low bits {0, 1/192, 2/3, 1, 1/3, 1/2, 1/6, 1/4}.
__constant__ float c_fp4[16] = {
    0.0f, 0.005208333333f, 0.66666667f, 1.0f, 0.33333333f, 0.5f, 0.16666667f, 0.25f,
    -0.0f, -0.005208333333f, -0.66666667f, -1.0f, -0.33333333f, -0.5f, -0.16666667f, -0.25f};

// The contract is two roundings: an fp32 product, then fp32 -> fp16.  The empty asm
// pins the fp32 product in a register so that the compiler cannot merge multiply and
// conversion into one mixed-precision instruction, which rounds only once.
__device__ __forceinline__ float mul_rounded_f32(float a, float b) {
  float v = a * b;
  asm volatile("" : "+v"(v));
  return v;
}

__device__ __forceinline__ uint32_t deq_pair(const float* tab, uint32_t byte, float a_hi, float a_lo) {
  // high nibble is the earlier element
  const float v0 = mul_rounded_f32(tab[byte >> 4], a_hi);
  const float v1 = mul_rounded_f32(tab[byte & 15u], a_lo);
  h2v h = {(_Float16)v0, (_Float16)v1};
  return __builtin_bit_cast(uint32_t, h);
}

// Fast path: n_elems % 32 == 0 handled in 32-element lane chunks; blocksize a
// multiple of 32 means one absmax per lane chunk, otherwise (blocksize 2..16 or
// not dividing 32) absmax is looked up per element.
template <bool ONE_ABSMAX>
__global__ __launch_bounds__(256) void dequant4_kernel(const u4v* __restrict__ packed,
                                                      const float* __restrict__ absmax,
                                                      u4v* __restrict__ out, int64_t nchunks,
                                                      int blocksize, int table) {
  __shared__ float tab[16];
  if (threadIdx.x < 16) tab[threadIdx.x] = table ? c_fp4[threadIdx.x] : c_nf4[threadIdx.x];
  __syncthreads();
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nchunks; i += stride) {
    const u4v p = __builtin_nontemporal_load(packed + i);
    const int64_t e0 = i * 32;
    float am = 0.f;
    if (ONE_ABSMAX) am = absmax[e0 / blocksize];
    const uint32_t words[4] = {p.x, p.y, p.z, p.w};
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      uint32_t o[4];
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const uint32_t byte = (words[w] >> (8 * b)) & 255u;
        if (ONE_ABSMAX) {
          o[b] = deq_pair(tab, byte, am, am);
        } else {
          const int64_t e = e0 + (w * 4 + b) * 2;
          o[b] = deq_pair(tab, byte, absmax[e / blocksize], absmax[(e + 1) / blocksize]);
        }
      }
      u4v ov = {o[0], o[1], o[2], o[3]};
      __builtin_nontemporal_store(ov, out + i * 4 + w);
    }
  }
}

// Tail / odd sizes: one element per thread.
__global__ __launch_bounds__(256) void dequant4_tail_kernel(const uint8_t* __restrict__ packed,
                                                           const float* __restrict__ absmax,
                                                           _Float16* __restrict__ out, int64_t e_begin,
                                                           int64_t n, int blocksize, int table) {
  const int64_t e = e_begin + (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= n) return;
  const float* tab = table ? c_fp4 : c_nf4;
  const uint32_t byte = packed[e >> 1];
  const uint32_t code = (e & 1) ? (byte & 15u) : (byte >> 4);
  out[e] = (_Float16)mul_rounded_f32(tab[code], absmax[e / blocksize]);
}

}  // namespace

extern "C" int hq_dequant_nf4(const uint8_t* packed, const float* absmax, void* out_fp16,
                              int64_t n_elems, int blocksize, int table, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (n_elems < 0 || blocksize <= 0 || (blocksize & 1)) return HQ_ERR_BAD_SHAPE;
  if (table != HQ_TABLE_NF4 && table != HQ_TABLE_FP4) return HQ_ERR_BAD_ENUM;
  if (n_elems == 0) return HQ_OK;
  if (!packed || !absmax || !out_fp16) return HQ_ERR_NULL_POINTER;
  if (((uintptr_t)absmax & 3) || ((uintptr_t)out_fp16 & 1)) return HQ_ERR_MISALIGNED;
  const HqDevice* dev = nullptr;
  int rc = hq_current_device(&dev);
  if (rc != HQ_OK) return rc;

  const bool wide = !((uintptr_t)packed & 15) && !((uintptr_t)out_fp16 & 15);
  const int64_t nchunks = wide ? n_elems / 32 : 0;
  if (nchunks > 0) {
    int64_t blocks = (nchunks + 255) / 256;
    const int64_t cap = (int64_t)dev->cus * hq_env_int("HQ_NF4_BLOCKS_PER_CU", 16);
    if (blocks > cap) blocks = cap;
    if (blocksize % 32 == 0)
      hipLaunchKernelGGL(dequant4_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, stream,
                         (const u4v*)packed, absmax, (u4v*)out_fp16, nchunks, blocksize, table);
    else
      hipLaunchKernelGGL(dequant4_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, stream,
                         (const u4v*)packed, absmax, (u4v*)out_fp16, nchunks, blocksize, table);
    rc = hq_launch_status();
    if (rc != HQ_OK) return rc;
  }
  const int64_t e_begin = nchunks * 32;
  if (e_begin < n_elems) {
    const int64_t rest = n_elems - e_begin;
    if ((rest + 255) / 256 > 0x7fffffff) return HQ_ERR_TOO_LARGE;
    hipLaunchKernelGGL(dequant4_tail_kernel, dim3((unsigned)((rest + 255) / 256)), dim3(256), 0, stream,
                       packed, absmax, (_Float16*)out_fp16, e_begin, n_elems, blocksize, table);
    rc = hq_launch_status();
  }
  return rc;
}
