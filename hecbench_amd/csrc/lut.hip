// LUT-GEMM binary-coded-quantisation matvec for gfx950 (fp16 in / fp16 out).
//
// Replaces matmul() -> nqmv_bias / nqmv -> _nqmv_bias<32> / _nqmv<64>
// (src/lut-gemm-hip/kernels.cu:22-31, mv_fp16.h:28-259 in the HeCBench tree).
//
//   y[n] = sum_k x[k] * ( q_bias[k/G][n] + sum_b alpha[k/G][b][n] * s(k,b,n) )
//
// For every 8-element sub-vector of x the 256 signed sums sum_j (+-x[j]) are
// tabulated once per workgroup in LDS (fp32 entries), and each byte of a packed
// bit-plane word becomes one table lookup.  A workgroup owns a tile of columns
// and a K slice of up to 512*iterations elements: per iteration it tabulates 64
// sub-vectors (64 KB), wave w consumes the 128-element quarter w for all the
// tile's columns, and the four waves' partial sums meet in LDS at the end.
// Everything is accumulated in fp32 and rounded to fp16 once, so unlike the
// reference (fp16 tables, fp16 partial sums, fp16 atomics across 128 K tiles) the
// result does not depend on the order in which workgroups finish.
#include "hq_internal.h"

namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef uint32_t u2v __attribute__((ext_vector_type(2)));

struct LutArgs {
  const uint32_t* bW;
  const _Float16* alpha;
  const _Float16* qbias;  // nullable
  const _Float16* x;
  _Float16* y;
  float* partial;
  unsigned* counters;
  int K, N, nb, G;
  int kslice;  // K elements per workgroup (multiple of 512)
  int nsplit;
};

constexpr int kStepK = 512;        // K elements tabulated per iteration
constexpr int kTables = kStepK / 8;  // 64 tables of 256 fp32 entries

template <int CPL>  // adjacent columns per lane
__global__ __launch_bounds__(256) void lut_gemv_kernel(LutArgs a) {
  extern __shared__ float lds[];
  float* lut = lds;                       // [64][256]
  float* red = lds;                       // reused after the main loop: [4][64*CPL]
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int ntiles = (a.N + 64 * CPL - 1) / (64 * CPL);
  const int tile = blockIdx.x % ntiles, split = blockIdx.x / ntiles;
  const int col = tile * 64 * CPL + lane * CPL;
  const bool col_ok = col < a.N;  // N % CPL == 0 is checked by the host
  const int k_begin = split * a.kslice;
  const int k_end = min(a.K, k_begin + a.kslice);

  float acc[CPL];
#pragma unroll
  for (int c = 0; c < CPL; ++c) acc[c] = 0.f;

  for (int k0 = k_begin; k0 < k_end; k0 += kStepK) {
    __syncthreads();  // previous iteration's lookups are done
    // ---- tabulate: thread -> table t = tid/4, quarter qd = tid%4 (entries 64qd..64qd+63)
    {
      const int t = tid >> 2, qd = tid & 3;
      const int kk = k0 + 8 * t;
      float xv[8];
      if (kk < k_end) {  // K % 32 == 0, so a sub-vector is whole or absent
        const h8 h = *reinterpret_cast<const h8*>(a.x + kk);
#pragma unroll
        for (int j = 0; j < 8; ++j) xv[j] = (float)h[j];
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) xv[j] = 0.f;
      }
      float e[64];
      float base = (qd & 1 ? xv[6] : -xv[6]) + (qd & 2 ? xv[7] : -xv[7]);
#pragma unroll
      for (int j = 0; j < 6; ++j) base -= xv[j];
      e[0] = base;
#pragma unroll
      for (int j = 0; j < 6; ++j)
#pragma unroll
        for (int i = 0; i < (1 << j); ++i) e[(1 << j) + i] = e[i] + 2.f * xv[j];
      float4* dst = reinterpret_cast<float4*>(lut + t * 256 + qd * 64);
#pragma unroll
      for (int i = 0; i < 16; ++i) dst[i] = make_float4(e[4 * i], e[4 * i + 1], e[4 * i + 2], e[4 * i + 3]);
    }
    __syncthreads();
    // ---- consume: wave wv takes k-words 4wv..4wv+3 of this step
    if (col_ok) {
      int g_cur = -1;
      float tsum[8][CPL];
      float al[8][CPL];
      float bias_x = 0.f;  // sum of x over the words of the current group seen by this wave
      auto flush = [&]() {
        if (g_cur < 0) return;
#pragma unroll
        for (int b = 0; b < 8; ++b)
          if (b < a.nb)
#pragma unroll
            for (int c = 0; c < CPL; ++c) acc[c] = fmaf(al[b][c], tsum[b][c], acc[c]);
        if (a.qbias) {
#pragma unroll
          for (int c = 0; c < CPL; ++c)
            acc[c] = fmaf((float)a.qbias[(size_t)g_cur * a.N + col + c], bias_x, acc[c]);
        }
      };
#pragma unroll
      for (int wi = 0; wi < 4; ++wi) {
        const int kw_local = 4 * wv + wi;  // k-word inside the step
        const int k = k0 + 32 * kw_local;
        if (k >= k_end) break;
        const int g = k / a.G;
        if (g != g_cur) {
          flush();
          g_cur = g;
          bias_x = 0.f;
#pragma unroll
          for (int b = 0; b < 8; ++b)
            if (b < a.nb) {
              const _Float16* ap = a.alpha + ((size_t)g * a.nb + b) * a.N + col;
#pragma unroll
              for (int c = 0; c < CPL; ++c) { al[b][c] = (float)ap[c]; tsum[b][c] = 0.f; }
            }
        }
        const float* l0 = lut + (kw_local * 4) * 256;
        bias_x += l0[255] + l0[256 + 255] + l0[512 + 255] + l0[768 + 255];
        const uint32_t* wp = a.bW + ((size_t)(k >> 5) * a.nb) * a.N + col;
#pragma unroll
        for (int b = 0; b < 8; ++b)
          if (b < a.nb) {
            uint32_t w[CPL];
            if (CPL == 2) {
              u2v v = __builtin_nontemporal_load(reinterpret_cast<const u2v*>(wp + (size_t)b * a.N));
              w[0] = v.x; w[CPL - 1] = v.y;
            } else {
#pragma unroll
              for (int c = 0; c < CPL; ++c) w[c] = __builtin_nontemporal_load(wp + (size_t)b * a.N + c);
            }
#pragma unroll
            for (int c = 0; c < CPL; ++c)
              tsum[b][c] += (l0[w[c] & 255u] + l0[256 + ((w[c] >> 8) & 255u)]) +
                            (l0[512 + ((w[c] >> 16) & 255u)] + l0[768 + (w[c] >> 24)]);
          }
      }
      flush();
    }
  }

  // ---- combine the four waves ------------------------------------------------
  __syncthreads();
#pragma unroll
  for (int c = 0; c < CPL; ++c) red[wv * 64 * CPL + lane * CPL + c] = acc[c];
  __syncthreads();
  const int n = tile * 64 * CPL + tid;
  if (tid < 64 * CPL && n < a.N) {
    float v = (red[tid] + red[64 * CPL + tid]) + (red[2 * 64 * CPL + tid] + red[3 * 64 * CPL + tid]);
    if (a.nsplit == 1) a.y[n] = (_Float16)v;
    else  // device-coherent (write-through) store, see the arrival protocol below
      __hip_atomic_store(&a.partial[((size_t)tile * a.nsplit + split) * (64 * CPL) + tid], v, __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
  }
  if (a.nsplit > 1) {
    // Split-K arrival counting with relaxed device-scope atomics only: the barrier
    // waits for this workgroup's write-through partial stores to be acknowledged
    // before the counter is bumped; the last workgroup to arrive adds the partials in
    // split order.  Full release/acquire fences would write back and invalidate the
    // whole L2 of the XCD on every workgroup and cost tens of microseconds per call.
    unsigned* s_last = reinterpret_cast<unsigned*>(lds + kTables * 256);
    __syncthreads();
    if (tid == 0)
      *s_last = (__hip_atomic_fetch_add(&a.counters[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) ==
                 (unsigned)(a.nsplit - 1));
    __syncthreads();
    if (*s_last) {
      if (tid < 64 * CPL && n < a.N) {
        float sum = 0.f;
        for (int s = 0; s < a.nsplit; ++s)
          sum += __hip_atomic_load(&a.partial[((size_t)tile * a.nsplit + s) * (64 * CPL) + tid],
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        a.y[n] = (_Float16)sum;
      }
      if (tid == 0) __hip_atomic_store(&a.counters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

}  // namespace

extern "C" int hq_lut_gemv(const uint32_t* bW, const void* alpha, const void* q_bias, const void* x,
                           void* y, int K, int N, int nbits, int group_size, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!bW || !alpha || !x || !y) return HQ_ERR_NULL_POINTER;
  if (K <= 0 || N <= 0 || nbits < 1 || nbits > 8 || group_size <= 0) return HQ_ERR_BAD_SHAPE;
  if ((K & 31) || (group_size & 31) || (K % group_size)) return HQ_ERR_BAD_SHAPE;
  if (((uintptr_t)bW & 3) || ((uintptr_t)alpha & 1) || ((uintptr_t)q_bias & 1) || ((uintptr_t)x & 15) ||
      ((uintptr_t)y & 1))
    return HQ_ERR_MISALIGNED;
  const HqDevice* dev = nullptr;
  int rc = hq_current_device(&dev);
  if (rc != HQ_OK) return rc;

  const bool pair = (N % 2 == 0) && !((uintptr_t)bW & 7);
  const int cpl = pair ? 2 : 1;
  const int ntiles = (N + 64 * cpl - 1) / (64 * cpl);
  // K slice per workgroup: enough workgroups to cover the CUs about twice.
  int nsplit = hq_env_int("HQ_LUT_KSPLIT", 0);
  const int steps = (K + kStepK - 1) / kStepK;
  if (nsplit <= 0) {
    nsplit = (2 * dev->cus + ntiles - 1) / ntiles;
    if (nsplit < 1) nsplit = 1;
  }
  if (nsplit > steps) nsplit = steps;
  const int steps_per = (steps + nsplit - 1) / nsplit;
  nsplit = (steps + steps_per - 1) / steps_per;

  LutArgs a;
  a.bW = bW; a.alpha = (const _Float16*)alpha; a.qbias = (const _Float16*)q_bias;
  a.x = (const _Float16*)x; a.y = (_Float16*)y; a.partial = nullptr; a.counters = nullptr;
  a.K = K; a.N = N; a.nb = nbits; a.G = group_size; a.kslice = steps_per * kStepK; a.nsplit = nsplit;
  if (nsplit > 1) {
    HqWorkspace ws;
    rc = hq_get_workspace(stream, (size_t)ntiles * nsplit * 64 * cpl, (size_t)ntiles, &ws);
    if (rc != HQ_OK) return rc;
    a.partial = ws.partial;
    a.counters = ws.counters;
  }
  const size_t smem = (size_t)kTables * 256 * sizeof(float) + 16;  // tables + the arrival flag
  static const hipError_t attr2 = hipFuncSetAttribute(reinterpret_cast<const void*>(&lut_gemv_kernel<2>),
                                                      hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
  static const hipError_t attr1 = hipFuncSetAttribute(reinterpret_cast<const void*>(&lut_gemv_kernel<1>),
                                                      hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
  if (attr1 != hipSuccess) return (int)attr1;
  if (attr2 != hipSuccess) return (int)attr2;
  if (pair) hipLaunchKernelGGL(lut_gemv_kernel<2>, dim3(ntiles * nsplit), dim3(256), smem, stream, a);
  else hipLaunchKernelGGL(lut_gemv_kernel<1>, dim3(ntiles * nsplit), dim3(256), smem, stream, a);
  return hq_launch_status();
}
