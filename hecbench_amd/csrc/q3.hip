// GPTQ 3-bit matvec (batch 1) for gfx950.
//
// Replaces VecQuant3MatMulKernel / VecQuant3MatMulKernelFaster and their host
// launchers (src/quant3MatMul-hip/kernels.h:12-217 in the HeCBench tree).
//
//   y[n] = sum_k x[k] * (s[n]*q[k][n] - z[n]) = s[n] * sum_k q[k][n]*x[k] - z[n] * sum_k x[k]
//
// The kernel is HBM-bound only if a weight costs well under two VALU
// instructions (17 MB / 8 TB/s leaves ~1.85 lane-ops per weight on 256 CUs), so
// the integer codes are never converted one by one: each 32-bit window of the
// packed string is ANDed into two subnormal-fp16 fields (see q3_recipe.h) and the
// multiply-accumulate runs on the matrix cores as a 16x16x32 fp16 MFMA whose
// "batch" dimension carries three fixed-point digits (11 bits each, 33 bits below
// the largest |x|) of the fp32 activation vector.  Products and partial sums are
// integers in units of one quantum, so the accumulation is exact; the only
// roundings are the handful of fp32 operations of the epilogue.
//
// Work split: a workgroup owns a 64-column tile and a contiguous range of
// k-groups; a wave's 16-lane quarter `kb` streams one k-group as three
// uint4 loads (4 adjacent columns x 3 packed rows), i.e. 256 contiguous bytes
// per packed row per quarter.  With one workgroup per tile no cross-workgroup
// reduction is needed; with split-K the partial sums go to a workspace and the
// last workgroup to arrive at a tile adds them in a fixed order.
#include "hq_internal.h"
#include "q3_recipe.h"

namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4v __attribute__((ext_vector_type(4)));

__constant__ hq_q3::SlotTable c_slots = hq_q3::make_slot_table();

struct Q3Args {
  const void* x;
  const uint32_t* w;
  const float* scales;
  const float* zeros;
  float* y;
  float* partial;
  unsigned* counters;
  int K, N;
  int gpw;     // k-groups per workgroup
  int nsplit;  // workgroups per column tile
  int x_f16;
  unsigned flags;
};

__device__ __forceinline__ float pow2f(int e) { return __uint_as_float((uint32_t)(e + 127) << 23); }

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int m = 32; m > 0; m >>= 1) v = fmaxf(v, __shfl_xor(v, m));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int m = 32; m > 0; m >>= 1) v += __shfl_xor(v, m);
  return v;
}

// Sixteen two-field registers of one column's k-group.
__device__ __forceinline__ void unpack16(uint32_t w0, uint32_t w1, uint32_t w2, uint32_t (&a)[16]) {
  using namespace hq_q3;
  const uint32_t win[7] = {w0,
                           __builtin_amdgcn_alignbit(w1, w0, 4),
                           __builtin_amdgcn_alignbit(w1, w0, 10),
                           w1,
                           __builtin_amdgcn_alignbit(w2, w1, 9),
                           w2,
                           w2 >> 7};
#pragma unroll
  for (int r = 0; r < 16; ++r) a[r] = win[kRecipe[r].window] & mask_of(r);
}

template <int WAVES, int STEPS>
__global__ __launch_bounds__(WAVES * 64) void q3_matvec_kernel(Q3Args a) {
  constexpr int T = WAVES * 64;
  constexpr int GROUPS_PER_ROUND = WAVES * 4 * STEPS;
  extern __shared__ uint4 smem[];
  // layout: xs[gpw_pad][4 mfma][4 pieces] uint4 | red[WAVES][3][64] float | misc
  const int gpw_pad = (a.gpw + GROUPS_PER_ROUND - 1) / GROUPS_PER_ROUND * GROUPS_PER_ROUND;
  uint4* xs = smem;
  float* red = reinterpret_cast<float*>(smem + (size_t)gpw_pad * 16);
  float* misc = red + WAVES * 3 * 64;  // [0..WAVES) max, [WAVES..2*WAVES) sum

  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int c = lane & 15, kb = lane >> 4;
  const int ntiles = (a.N + 63) >> 6;
  const int tile = blockIdx.x % ntiles, split = blockIdx.x / ntiles;
  const int G = a.K >> 5;
  const int g_begin = split * a.gpw;
  const int g_count = min(a.gpw, G - g_begin);
  const int col = tile * 64 + 4 * c;
  const bool col_ok = col < a.N;
  const int rounds = gpw_pad / GROUPS_PER_ROUND;
  const size_t row_stride = (size_t)a.N;

  uint32_t wreg[STEPS][3][4];
  auto issue = [&](int round) {
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      const int gl = (round * STEPS + s) * (WAVES * 4) + wv * 4 + kb;
      if (col_ok && gl < g_count) {
        const uint32_t* p = a.w + (size_t)(3 * (g_begin + gl)) * row_stride + col;
#pragma unroll
        for (int j = 0; j < 3; ++j) {
          u4v v = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(p + j * row_stride));
          wreg[s][j][0] = v.x; wreg[s][j][1] = v.y; wreg[s][j][2] = v.z; wreg[s][j][3] = v.w;
        }
      } else {
#pragma unroll
        for (int j = 0; j < 3; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q) wreg[s][j][q] = 0u;
      }
    }
  };
  issue(0);  // weights are in flight while the activations are staged

  // ---- stage the activation pieces in operand-slot order -------------------
  for (int i = tid; i < gpw_pad * 16; i += T) xs[i] = make_uint4(0, 0, 0, 0);
  const int k_begin = g_begin * 32, k_count = g_count * 32;
  float amax = 0.f, asum = 0.f;
  for (int k = tid; k < k_count; k += T) {
    float v = a.x_f16 ? (float)reinterpret_cast<const _Float16*>(a.x)[k_begin + k]
                      : reinterpret_cast<const float*>(a.x)[k_begin + k];
    amax = fmaxf(amax, fabsf(v));
    asum += v;
  }
  amax = wave_max(amax);
  asum = wave_sum(asum);
  if (lane == 0) { misc[wv] = amax; misc[WAVES + wv] = asum; }
  __syncthreads();
  float xmax = 0.f, xsum = 0.f;
#pragma unroll
  for (int i = 0; i < WAVES; ++i) { xmax = fmaxf(xmax, misc[i]); xsum += misc[WAVES + i]; }
  // 2^E * max|x| lies in [2^14, 2^15): the hi piece never overflows fp16.
  int E = 14 - ((int)((__float_as_uint(xmax) >> 23) & 255u) - 127);
  E = xmax > 0.f ? max(-100, min(100, E)) : 0;
  const float scaleE = pow2f(E);
  _Float16* xs_h = reinterpret_cast<_Float16*>(xs);
  for (int k = tid; k < k_count; k += T) {
    float xv = a.x_f16 ? (float)reinterpret_cast<const _Float16*>(a.x)[k_begin + k]
                       : reinterpret_cast<const float*>(a.x)[k_begin + k];
    const int gl = k >> 5, ki = k & 31;
    const int slot = c_slots.slot[ki], pos = c_slots.pos[ki];
    // Fixed-point split of u = x*2^E (|u| < 2^15) into three signed 11-bit digits
    // with quanta 2^5, 2^-6, 2^-17.  Every MFMA product is then an integer multiple
    // of one quantum and a wave's partial sums stay below 2^24 quanta, so the matrix
    // core accumulation is exact whatever its internal rounding is.
    const float u = xv * scaleE;
    const float p0 = rintf(u * 0.03125f);
    const float r1 = u - p0 * 32.f;        // exact
    const float p1 = rintf(r1 * 64.f);
    const float r2 = r1 - p1 * 0.015625f;  // exact
    const float p2 = rintf(r2 * 131072.f);
    const float sl = pow2f(4 - pos);       // digit * 2^(4-pos) fits fp16 exactly
    const _Float16 h0 = (_Float16)(p0 * sl), h1 = (_Float16)(p1 * sl), h2 = (_Float16)(p2 * sl);
    _Float16* dst = xs_h + ((size_t)(gl * 4 + (slot >> 3)) * 4) * 8 + (slot & 7);
    dst[0] = h0; dst[8] = h1; dst[16] = h2;
  }
  __syncthreads();

  // ---- main loop ---------------------------------------------------------------
  f4 acc[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) acc[q] = f4{0.f, 0.f, 0.f, 0.f};
  const int piece = c < 3 ? c : 3;
  for (int round = 0; round < rounds; ++round) {
    if (round > 0) issue(round);
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      const int gl_base = (round * STEPS + s) * (WAVES * 4) + wv * 4;
      if (gl_base >= g_count) continue;  // wave-uniform
      const uint4* xb = xs + (size_t)(gl_base + kb) * 16 + piece;
      h8 B[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) B[j] = __builtin_bit_cast(h8, xb[j * 4]);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        uint32_t f[16];
        unpack16(wreg[s][0][q], wreg[s][1][q], wreg[s][2][q], f);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          u4v av = {f[4 * j], f[4 * j + 1], f[4 * j + 2], f[4 * j + 3]};
          acc[q] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, av), B[j], acc[q], 0, 0, 0);
        }
      }
    }
  }

  // ---- combine waves, pieces, scale/zero ------------------------------------------
  // D[row = 4*kb + i][col = c]: row is the weight column (quarter-major), col the piece.
  if (c < 3) {
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[(wv * 3 + c) * 64 + 4 * (4 * kb + i) + q] = acc[q][i];
  }
  __syncthreads();
  const int n = tile * 64 + tid;
  float val = 0.f;
  if (tid < 64 && n < a.N) {
    float c0 = 0.f, c1 = 0.f, c2 = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      c0 += red[(w * 3 + 0) * 64 + tid];
      c1 += red[(w * 3 + 1) * 64 + tid];
      c2 += red[(w * 3 + 2) * 64 + tid];
    }
    const float inv11 = 1.f / 2048.f;
    float S = fmaf(fmaf(c2, inv11, c1), inv11, c0);
    float qx = S * 33554432.f * pow2f(-E);  // 2^20 (operand scale) * 2^5 (digit 0 quantum)
    val = a.scales[n] * qx - a.zeros[n] * xsum;
    if (a.nsplit == 1) {
      a.y[n] = (a.flags & HQ_FLAG_ACCUMULATE) ? a.y[n] + val : val;
    } else {
      a.partial[((size_t)tile * a.nsplit + split) * 64 + tid] = val;
    }
  }
  if (a.nsplit > 1) {
    __shared__ unsigned s_last;
    __threadfence();
    __syncthreads();
    if (tid == 0) {
      unsigned old = atomicAdd(&a.counters[tile], 1u);
      s_last = (old == (unsigned)(a.nsplit - 1));
    }
    __syncthreads();
    if (s_last) {
      __threadfence();
      if (tid < 64 && n < a.N) {
        float sum = 0.f;
        for (int s = 0; s < a.nsplit; ++s)
          sum += __hip_atomic_load(&a.partial[((size_t)tile * a.nsplit + s) * 64 + tid],
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        a.y[n] = (a.flags & HQ_FLAG_ACCUMULATE) ? a.y[n] + sum : sum;
      }
      if (tid == 0) a.counters[tile] = 0u;  // ready for the next call
    }
  }
}

template <int WAVES, int STEPS>
int launch_matvec(const Q3Args& a, int ntiles, hipStream_t stream) {
  constexpr int GPR = WAVES * 4 * STEPS;
  const int gpw_pad = (a.gpw + GPR - 1) / GPR * GPR;
  const size_t smem = (size_t)gpw_pad * 256 + (size_t)WAVES * 3 * 64 * 4 + (size_t)WAVES * 2 * 4;
  static const hipError_t attr =
      hipFuncSetAttribute(reinterpret_cast<const void*>(&q3_matvec_kernel<WAVES, STEPS>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);
  if (attr != hipSuccess) return (int)attr;
  hipLaunchKernelGGL((q3_matvec_kernel<WAVES, STEPS>), dim3(ntiles * a.nsplit), dim3(WAVES * 64), smem,
                     stream, a);
  return hq_launch_status();
}

}  // namespace

int hq_q3_gemm_launch(const void* x, const int32_t* qweight, const float* scales, const float* zeros,
                      float* y, int K, int N, int M, unsigned flags, hipStream_t stream);

extern "C" int hq_q3_matvec(const void* x, int x_dtype, const int32_t* qweight, const float* scales,
                            const float* zeros, float* y, int K, int N, int batch_M, unsigned flags,
                            void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!x || !qweight || !scales || !zeros || !y) return HQ_ERR_NULL_POINTER;
  if (x_dtype != HQ_DTYPE_F32 && x_dtype != HQ_DTYPE_F16) return HQ_ERR_BAD_ENUM;
  if (flags & ~HQ_FLAG_ACCUMULATE) return HQ_ERR_BAD_ENUM;
  if (K <= 0 || N <= 0 || batch_M <= 0 || (K & 31) || (N & 3)) return HQ_ERR_BAD_SHAPE;
  if (((uintptr_t)qweight & 15) || ((uintptr_t)x & (x_dtype == HQ_DTYPE_F16 ? 1 : 3)) ||
      ((uintptr_t)y & 3) || ((uintptr_t)scales & 3) || ((uintptr_t)zeros & 3))
    return HQ_ERR_MISALIGNED;
  const HqDevice* dev = nullptr;
  int rc = hq_current_device(&dev);
  if (rc != HQ_OK) return rc;
  if (batch_M > 1) {
    if (x_dtype != HQ_DTYPE_F16) return HQ_ERR_BAD_ENUM;
    return hq_q3_gemm_launch(x, qweight, scales, zeros, y, K, N, batch_M, flags, stream);
  }

  const int G = K / 32;
  const int ntiles = (N + 63) / 64;
  // Launch shape: WAVES waves per workgroup, each streaming STEPS k-groups per
  // 16-lane quarter per round; split K so that a workgroup runs one round and the
  // grid covers the CU count a few times over.
  int waves = hq_env_int("HQ_Q3_WAVES", 16);
  int steps = hq_env_int("HQ_Q3_STEPS", 2);
  int nsplit = hq_env_int("HQ_Q3_KSPLIT", 0);
  if (waves != 4 && waves != 8 && waves != 16) waves = 16;
  if (steps != 1 && steps != 2 && steps != 4) steps = 2;
  const int gpr = waves * 4 * steps;
  if (nsplit <= 0) nsplit = (G + gpr - 1) / gpr;
  if (nsplit > G) nsplit = G;
  int gpw = (G + nsplit - 1) / nsplit;
  if (gpw > 192) {  // activation pieces of a workgroup must fit its LDS budget
    nsplit = (G + 191) / 192;
    gpw = (G + nsplit - 1) / nsplit;
  }
  nsplit = (G + gpw - 1) / gpw;

  Q3Args a;
  a.x = x; a.w = reinterpret_cast<const uint32_t*>(qweight); a.scales = scales; a.zeros = zeros;
  a.y = y; a.partial = nullptr; a.counters = nullptr; a.K = K; a.N = N; a.gpw = gpw;
  a.nsplit = nsplit; a.x_f16 = (x_dtype == HQ_DTYPE_F16); a.flags = flags;
  if (nsplit > 1) {
    HqWorkspace ws;
    rc = hq_get_workspace(stream, (size_t)ntiles * nsplit * 64, (size_t)ntiles, &ws);
    if (rc != HQ_OK) return rc;
    a.partial = ws.partial;
    a.counters = ws.counters;
  }
#define HQ_Q3_CASE(W, S) \
  if (waves == W && steps == S) return launch_matvec<W, S>(a, ntiles, stream);
  HQ_Q3_CASE(16, 1) HQ_Q3_CASE(16, 2) HQ_Q3_CASE(16, 4)
  HQ_Q3_CASE(8, 1) HQ_Q3_CASE(8, 2) HQ_Q3_CASE(8, 4)
  HQ_Q3_CASE(4, 1) HQ_Q3_CASE(4, 2) HQ_Q3_CASE(4, 4)
#undef HQ_Q3_CASE
  return HQ_ERR_BAD_ENUM;
}
