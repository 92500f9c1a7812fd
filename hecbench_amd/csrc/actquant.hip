// Per-token int8 activation quantisation (static / dynamic scale, with or without an
// asymmetric zero point) for gfx950.
//
// Replaces static_scaled_int8_quant / dynamic_scaled_int8_quant and their four kernels
// (src/quantVLLM-hip/main.cu:11-168 in the HeCBench tree; helpers in
// src/quantVLLM-cuda/utils.h).  Bit-exact contract: fp32 IEEE division, round to nearest
// even, saturation, exactly as the reference's host loops (src/quantVLLM-cuda/reference.h).
//
// One workgroup per token.  A lane converts eight consecutive elements per trip (128-bit
// loads for fp16 / bf16, two for fp32) into one packed 64-bit store.  The dynamic variants
// reduce max |x| (or min and max) with cross-lane butterflies and one LDS exchange, and
// keep the row in registers between the two passes when it fits.
#include "hq_internal.h"

namespace {

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(_Float16 v) { return (float)v; }
struct bf16_t { uint16_t bits; };  // bfloat16 = the upper half of an fp32
__device__ __forceinline__ float to_f32(bf16_t v) { return __uint_as_float((uint32_t)v.bits << 16); }

// src/quantVLLM-cuda/utils.h:9-24
__device__ __forceinline__ int float_to_int8_rn(float x) {
  float dst = rintf(x);
  dst = dst < -128.f ? -128.f : (127.f < dst ? 127.f : dst);
  return (int)dst;
}
// src/quantVLLM-cuda/utils.h:26-50
__device__ __forceinline__ int float_to_int32_rn(float x) {
  const float dst = rintf(x);
  if (dst >= 2147483648.f) return 2147483647;
  if (dst <= -2147483648.f) return -2147483647 - 1;
  return (int)dst;
}
// src/quantVLLM-cuda/utils.h:52-61 (saturating add of the zero point happens in int32)
__device__ __forceinline__ int int32_to_int8(int x) { return x < -128 ? -128 : (127 < x ? 127 : x); }

constexpr int kThreads = 256;
constexpr int kVec = 8;       // elements per lane per trip
constexpr int kKeep = 4;      // trips kept in registers by the dynamic kernels (rows up to 8192)

template <typename T>
__device__ __forceinline__ void load8(const T* p, float (&v)[kVec], bool vec_ok, int valid) {
  if (vec_ok && valid == kVec) {
    T tmp[kVec];
    if (sizeof(T) == 2) {
      *reinterpret_cast<uint4*>(tmp) = *reinterpret_cast<const uint4*>(p);
    } else {
      reinterpret_cast<uint4*>(tmp)[0] = reinterpret_cast<const uint4*>(p)[0];
      reinterpret_cast<uint4*>(tmp)[1] = reinterpret_cast<const uint4*>(p)[1];
    }
#pragma unroll
    for (int i = 0; i < kVec; ++i) v[i] = to_f32(tmp[i]);
  } else {
#pragma unroll
    for (int i = 0; i < kVec; ++i) v[i] = i < valid ? to_f32(p[i]) : 0.f;
  }
}

__device__ __forceinline__ void store8(int8_t* p, const int (&q)[kVec], bool vec_ok, int valid) {
  if (vec_ok && valid == kVec) {
    uint2 w;
    w.x = (uint32_t)(q[0] & 255) | ((uint32_t)(q[1] & 255) << 8) | ((uint32_t)(q[2] & 255) << 16) |
          ((uint32_t)(q[3] & 255) << 24);
    w.y = (uint32_t)(q[4] & 255) | ((uint32_t)(q[5] & 255) << 8) | ((uint32_t)(q[6] & 255) << 16) |
          ((uint32_t)(q[7] & 255) << 24);
    *reinterpret_cast<uint2*>(p) = w;
  } else {
#pragma unroll
    for (int i = 0; i < kVec; ++i)
      if (i < valid) p[i] = (int8_t)q[i];
  }
}

// Block-wide reduction of (a: max, b: min) through one LDS exchange.
__device__ __forceinline__ void block_max_min(float& a, float& b, float* lds) {
#pragma unroll
  for (int m = 32; m > 0; m >>= 1) {
    a = fmaxf(a, __shfl_xor(a, m));
    b = fminf(b, __shfl_xor(b, m));
  }
  const int wv = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) { lds[wv] = a; lds[8 + wv] = b; }
  __syncthreads();
#pragma unroll
  for (int w = 0; w < kThreads / 64; ++w) { a = fmaxf(a, lds[w]); b = fminf(b, lds[8 + w]); }
}

template <typename T, bool AZP>
__global__ __launch_bounds__(kThreads) void static_quant_kernel(const T* __restrict__ in, int8_t* __restrict__ out,
                                                               float scale, int azp, int hidden, int vec_ok) {
  const int64_t token = blockIdx.x;
  in += token * hidden;
  out += token * hidden;
  for (int e0 = threadIdx.x * kVec; e0 < hidden; e0 += kThreads * kVec) {
    const int valid = min(kVec, hidden - e0);
    float v[kVec];
    int q[kVec];
    load8(in + e0, v, vec_ok, valid);
#pragma unroll
    for (int i = 0; i < kVec; ++i)
      q[i] = AZP ? int32_to_int8(float_to_int32_rn(v[i] / scale) + azp) : float_to_int8_rn(v[i] / scale);
    store8(out + e0, q, vec_ok, valid);
  }
}

template <typename T, bool AZP>
__global__ __launch_bounds__(kThreads) void dynamic_quant_kernel(const T* __restrict__ in, int8_t* __restrict__ out,
                                                                float* __restrict__ scales, int32_t* __restrict__ azps,
                                                                int hidden, int vec_ok) {
  __shared__ float lds[16];
  const int64_t token = blockIdx.x;
  in += token * hidden;
  out += token * hidden;
  float keep[kKeep][kVec];
  // reference initial values: max starts at FLT_MIN (smallest positive normal), min at FLT_MAX
  // (reference.h:71-72); the symmetric variant starts its absmax at 0 (reference.h:43)
  float mx = AZP ? 1.17549435e-38f : 0.f, mn = 3.40282347e+38f;
  int trip = 0;
  for (int e0 = threadIdx.x * kVec; e0 < hidden; e0 += kThreads * kVec, ++trip) {
    const int valid = min(kVec, hidden - e0);
    float v[kVec];
    load8(in + e0, v, vec_ok, valid);
#pragma unroll
    for (int i = 0; i < kVec; ++i) {
      if (i < valid) {
        if (AZP) { mx = fmaxf(mx, v[i]); mn = fminf(mn, v[i]); }
        else mx = fmaxf(mx, fabsf(v[i]));
      }
      if (trip < kKeep) keep[trip < kKeep ? trip : 0][i] = v[i];
    }
  }
  block_max_min(mx, mn, lds);
  float scale_val, mul = 0.f;
  int azp_val = 0;
  if (AZP) {
    scale_val = (mx - mn) / 255.0f;
    azp_val = (int)rintf(-128.0f - mn / scale_val);
  } else {
    scale_val = mx / 127.0f;
    mul = 127.0f / mx;
  }
  if (threadIdx.x == 0) {
    scales[token] = scale_val;
    if (AZP) azps[token] = azp_val;
  }
  trip = 0;
  for (int e0 = threadIdx.x * kVec; e0 < hidden; e0 += kThreads * kVec, ++trip) {
    const int valid = min(kVec, hidden - e0);
    float v[kVec];
    int q[kVec];
    if (trip < kKeep) {
#pragma unroll
      for (int i = 0; i < kVec; ++i) v[i] = keep[trip < kKeep ? trip : 0][i];
    } else {
      load8(in + e0, v, vec_ok, valid);
    }
#pragma unroll
    for (int i = 0; i < kVec; ++i)
      q[i] = AZP ? int32_to_int8(float_to_int32_rn(v[i] / scale_val) + azp_val) : float_to_int8_rn(v[i] * mul);
    store8(out + e0, q, vec_ok, valid);
  }
}

template <typename T>
int launch_static(const T* in, int8_t* out, int64_t tokens, int hidden, float scale, int has_azp, int azp, int vec_ok,
                  hipStream_t stream) {
  if (has_azp)
    hipLaunchKernelGGL((static_quant_kernel<T, true>), dim3((unsigned)tokens), dim3(kThreads), 0, stream, in, out, scale,
                       azp, hidden, vec_ok);
  else
    hipLaunchKernelGGL((static_quant_kernel<T, false>), dim3((unsigned)tokens), dim3(kThreads), 0, stream, in, out, scale,
                       azp, hidden, vec_ok);
  return hq_launch_status();
}
template <typename T>
int launch_dynamic(const T* in, int8_t* out, float* scales, int32_t* azps, int64_t tokens, int hidden, int vec_ok,
                   hipStream_t stream) {
  if (azps)
    hipLaunchKernelGGL((dynamic_quant_kernel<T, true>), dim3((unsigned)tokens), dim3(kThreads), 0, stream, in, out, scales,
                       azps, hidden, vec_ok);
  else
    hipLaunchKernelGGL((dynamic_quant_kernel<T, false>), dim3((unsigned)tokens), dim3(kThreads), 0, stream, in, out,
                       scales, azps, hidden, vec_ok);
  return hq_launch_status();
}

int check_common(const void* x, int x_dtype, const int8_t* out, int64_t tokens, int hidden, int* vec_ok) {
  if (tokens < 0 || hidden <= 0) return HQ_ERR_BAD_SHAPE;
  if (x_dtype != HQ_DTYPE_F32 && x_dtype != HQ_DTYPE_F16 && x_dtype != HQ_DTYPE_BF16) return HQ_ERR_BAD_ENUM;
  if (tokens == 0) return HQ_OK;
  if (!x || !out) return HQ_ERR_NULL_POINTER;
  if (tokens > 0x7fffffff) return HQ_ERR_TOO_LARGE;
  const int esz = x_dtype == HQ_DTYPE_F32 ? 4 : 2;
  if ((uintptr_t)x & (esz - 1)) return HQ_ERR_MISALIGNED;
  *vec_ok = !((uintptr_t)x & 15) && !((uintptr_t)out & 7) && hidden % kVec == 0;
  return HQ_OK;
}

}  // namespace

extern "C" int hq_int8_quant_static(const void* x, int x_dtype, int8_t* out, int64_t num_tokens, int hidden_size,
                                    float scale, int has_azp, int32_t azp, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  int vec_ok = 0;
  int rc = check_common(x, x_dtype, out, num_tokens, hidden_size, &vec_ok);
  if (rc != HQ_OK || num_tokens == 0) return rc;
  const HqDevice* dev = nullptr;
  rc = hq_current_device(&dev);
  if (rc != HQ_OK) return rc;
  if (x_dtype == HQ_DTYPE_F32)
    return launch_static((const float*)x, out, num_tokens, hidden_size, scale, has_azp, azp, vec_ok, stream);
  if (x_dtype == HQ_DTYPE_F16)
    return launch_static((const _Float16*)x, out, num_tokens, hidden_size, scale, has_azp, azp, vec_ok, stream);
  return launch_static((const bf16_t*)x, out, num_tokens, hidden_size, scale, has_azp, azp, vec_ok, stream);
}

extern "C" int hq_int8_quant_dynamic(const void* x, int x_dtype, int8_t* out, float* scales, int32_t* azp,
                                     int64_t num_tokens, int hidden_size, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  int vec_ok = 0;
  int rc = check_common(x, x_dtype, out, num_tokens, hidden_size, &vec_ok);
  if (rc != HQ_OK || num_tokens == 0) return rc;
  if (!scales) return HQ_ERR_NULL_POINTER;
  if (((uintptr_t)scales & 3) || ((uintptr_t)azp & 3)) return HQ_ERR_MISALIGNED;
  const HqDevice* dev = nullptr;
  rc = hq_current_device(&dev);
  if (rc != HQ_OK) return rc;
  if (x_dtype == HQ_DTYPE_F32)
    return launch_dynamic((const float*)x, out, scales, azp, num_tokens, hidden_size, vec_ok, stream);
  if (x_dtype == HQ_DTYPE_F16)
    return launch_dynamic((const _Float16*)x, out, scales, azp, num_tokens, hidden_size, vec_ok, stream);
  return launch_dynamic((const bf16_t*)x, out, scales, azp, num_tokens, hidden_size, vec_ok, stream);
}
