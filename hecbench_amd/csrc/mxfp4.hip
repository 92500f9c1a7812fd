// Microscaling fp4 (e2m1 with a shared power-of-two scale per 32 elements)
// quantise-dequantise of fp16 / bf16 data for gfx950.
//
// Replaces qdq_mxfp4_kernel and its launcher mxfp4() (src/mxfp4-hip/main.cu:19-171 in the
// HeCBench tree).  Per group of 32 consecutive elements: the largest magnitude is rounded
// to a power of two 2^e (the carry happens at a mantissa of 0.75, main.cu:124-126), the
// shared scale is 2^(e-2) clamped to the E8M0 range (main.cu:128-132), and every element
// becomes scale * e2m1(x / scale), where e2m1() rounds to the nearest of 0, .5, 1, 1.5, 2,
// 3, 4, 6 (ties to the even mantissa, saturating at 6, sign kept).  Bit-exact with the
// reference for finite inputs, with two exceptions where the reference's own arithmetic breaks down:
// a group maximum that rounds to zero (the reference divides by a zero scale; this kernel writes signed
// zeros), and a group maximum whose rounding to a power of two leaves the format (fp16 >= 61440, bf16 >=
// 0x7f60: the reference takes log2 of an infinity and writes NaN for the whole group; this kernel uses the
// scale the carry stands for, 2^14 or 2^126, and writes finite values, the maximum itself becoming
// infinity).
//
// HBM-bound: 4 bytes per element.  A lane owns 8 consecutive elements (one 128-bit load, one
// 128-bit nontemporal store), a group is 4 adjacent lanes, and the group maximum takes two
// DPP quad permutes on the integer magnitudes (magnitudes of one format order like their bit
// patterns).  The division and the multiplication by the scale are exact power-of-two
// scalings in fp32, so the only rounding is the one to e2m1.
#include "hq_internal.h"

namespace {

typedef uint32_t u4v __attribute__((ext_vector_type(4)));

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, true);
}

// Nearest e2m1 magnitude of m >= 0.
__device__ __forceinline__ float round_to_e2m1(float m) {
  const float lo = rintf(m * 2.f) * 0.5f;                // steps of 0.5 below 2
  const float mid = rintf(m);                            // steps of 1 in [2, 4)
  const float hi = fminf(rintf(m * 0.5f) * 2.f, 6.f);    // steps of 2 above, saturating
  return m < 2.f ? lo : (m < 4.f ? mid : hi);
}

// Quantise-dequantise of one lane's 8 elements (4 words); `mx` is the lane's largest magnitude on
// entry and is completed over the group's four lanes here.
template <bool BF16>
__device__ __forceinline__ u4v qdq_unit(const u4v raw) {
  constexpr int MANT = BF16 ? 7 : 10;
  constexpr int BIAS = BF16 ? 127 : 15;
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
  uint32_t mx = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) mx = max(mx, max(w[i] & 0x7fffu, (w[i] >> 16) & 0x7fffu));
  mx = max(mx, dpp_u<0xB1>(mx));  // quad_perm [1,0,3,2]
  mx = max(mx, dpp_u<0x4E>(mx));  // quad_perm [2,3,0,1]
  const uint32_t rounded = (mx + (1u << (MANT - 2))) & (0xffffu << MANT) & 0x7fffu;
  const int e = (int)(rounded >> MANT) - BIAS;
  const int scale_exp = max(0, 127 + min(e - 2, 127));  // E8M0 code of the scale
  // 2^(scale_exp - 127) and its reciprocal; code 0 is 2^-127, an fp32 subnormal
  const float scale = scale_exp > 0 ? __uint_as_float((uint32_t)scale_exp << 23) : __uint_as_float(0x00400000u);
  const float inv = scale_exp == 0 ? 1.7014118346046923e38f
                                   : (scale_exp < 254 ? __uint_as_float((uint32_t)(254 - scale_exp) << 23)
                                                      : __uint_as_float(0x00400000u));
  uint32_t o[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    // magnitudes only: the sign bits are copied over at the end (a multiply fused with the
    // conversion would turn -0 into +0)
    float x0, x1;
    if (BF16) {
      x0 = __uint_as_float((w[i] << 16) & 0x7fff0000u);
      x1 = __uint_as_float(w[i] & 0x7fff0000u);
    } else {
      x0 = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[i] & 0x7fffu));
      x1 = (float)__builtin_bit_cast(_Float16, (uint16_t)((w[i] >> 16) & 0x7fffu));
    }
    const float r0 = round_to_e2m1(x0 * inv) * scale, r1 = round_to_e2m1(x1 * inv) * scale;
    uint32_t mag;
    if (rounded == 0) {
      mag = 0;
    } else if (BF16) {
      mag = (__float_as_uint(r0) >> 16) | (__float_as_uint(r1) & 0xffff0000u);  // exact: two mantissa bits
    } else {
      mag = (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)r0) |
            ((uint32_t)__builtin_bit_cast(uint16_t, (_Float16)r1) << 16);
    }
    o[i] = mag | (w[i] & 0x80008000u);
  }
  const u4v res = {o[0], o[1], o[2], o[3]};
  return res;
}

// One 16-byte unit (eight elements) per thread and a plain grid: on this part the wave launcher refills the
// compute units better than a loop that keeps the next trip's loads in flight (4096 x 4096 fp16: 13.6 -> 12.5 us,
// 2^28 elements 180 -> 163 us = 6.6 TB/s), and the results leave as write-through streaming stores (12.5 against
// 13.1 us with nontemporal, 13.8 with plain stores).  units is a multiple of 4, so the four lanes of a group are
// in range or out of range together and the quad permutes never read an idle lane's data.
template <bool BF16>
__global__ __launch_bounds__(256) void mxfp4_qdq_kernel(const u4v* __restrict__ in, u4v* __restrict__ out,
                                                       int64_t units) {
  const int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (u >= units) return;
  const u4v res = qdq_unit<BF16>(__builtin_nontemporal_load(in + u));
  hq_store_stream(reinterpret_cast<hq_u4v*>(out + u), res);
}

}  // namespace

extern "C" int hq_mxfp4_qdq(const void* in, void* out, int64_t n_elems, int dtype, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (dtype != HQ_DTYPE_F16 && dtype != HQ_DTYPE_BF16) return HQ_ERR_BAD_ENUM;
  if (n_elems < 0 || (n_elems & 31)) return HQ_ERR_BAD_SHAPE;
  if (n_elems == 0) return HQ_OK;  // nothing to do, whatever the pointers are
  if (!in || !out) return HQ_ERR_NULL_POINTER;
  if (((uintptr_t)in & 15) || ((uintptr_t)out & 15)) return HQ_ERR_MISALIGNED;
  const HqDevice* dev = nullptr;
  int rc = hq_current_device(&dev);
  if (rc != HQ_OK) return rc;
  const int64_t units = n_elems / 8;
  const int64_t blocks = (units + 255) / 256;
  if (blocks > 0x7fffffffLL) return HQ_ERR_TOO_LARGE;
  if (dtype == HQ_DTYPE_BF16)
    hipLaunchKernelGGL(mxfp4_qdq_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, stream,
                       reinterpret_cast<const u4v*>(in), reinterpret_cast<u4v*>(out), units);
  else
    hipLaunchKernelGGL(mxfp4_qdq_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, stream,
                       reinterpret_cast<const u4v*>(in), reinterpret_cast<u4v*>(out), units);
  return hq_launch_status();
}
