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
// Work split: a workgroup owns a 64-column tile and WAVES*4*STEPS consecutive
// k-groups; a wave's 16-lane quarter `kb` streams one k-group per step as three
// uint4 loads (4 adjacent columns x 3 packed rows), i.e. 256 contiguous bytes
// per packed row per quarter.  A wave issues all its global loads first, stages
// its own activations in LDS without a workgroup barrier, and meets the other
// waves only in the final reduction.  When one workgroup covers all of K no
// cross-workgroup reduction is needed; otherwise (split-K) the partial sums go to
// a workspace and the last workgroup to arrive at a tile adds them in a fixed
// order, so results do not depend on arrival order.
#include "hq_internal.h"
#include "q3_recipe.h"

namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4v __attribute__((ext_vector_type(4)));
typedef _Float16 h2v __attribute__((ext_vector_type(2)));

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

// Cross-lane reductions without LDS traffic: four DPP butterfly steps inside each
// 16-lane row, then the four row results are read into scalars.
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float lane_f(float v, int l) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), l));
}
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_f<0xB1>(v));   // quad_perm [1,0,3,2]
  v = fmaxf(v, dpp_f<0x4E>(v));   // quad_perm [2,3,0,1]
  v = fmaxf(v, dpp_f<0x141>(v));  // row_half_mirror
  v = fmaxf(v, dpp_f<0x140>(v));  // row_mirror
  return fmaxf(fmaxf(lane_f(v, 0), lane_f(v, 16)), fmaxf(lane_f(v, 32), lane_f(v, 48)));
}
__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_f<0xB1>(v);
  v += dpp_f<0x4E>(v);
  v += dpp_f<0x141>(v);
  v += dpp_f<0x140>(v);
  return (lane_f(v, 0) + lane_f(v, 16)) + (lane_f(v, 32) + lane_f(v, 48));
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

template <int WAVES, int STEPS, bool XF16, bool MULTI>
__global__ __launch_bounds__(WAVES * 64) void q3_matvec_kernel(Q3Args a) {
  // LDS: xs[WAVES][STEPS*4 groups][4 mfma][4 piece slots] uint4 | red[WAVES][3][64] | xsum[WAVES]
  extern __shared__ uint4 smem[];
  uint4* xs = smem;
  float* red = reinterpret_cast<float*>(smem + WAVES * STEPS * 64);
  float* wsum = red + WAVES * 3 * 64;

  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int c = lane & 15, kb = lane >> 4;
  const int tile = blockIdx.x, split = blockIdx.y;
  const int G = a.K >> 5;
  const int g_begin = split * a.gpw;
  const int g_count = min(a.gpw, G - g_begin);
  const size_t row_stride = (size_t)a.N;
  const int n = tile * 64 + tid;

  // ---- loads that do not depend on the round ------------------------------------------------
  float sc_n = 0.f, zr_n = 0.f, y_old = 0.f;
  if (tid < 64) {
    const int nc = min(n, a.N - 1);
    sc_n = a.scales[nc];
    zr_n = a.zeros[nc];
    y_old = ((a.flags & HQ_FLAG_ACCUMULATE) && a.nsplit == 1) ? a.y[nc] : 0.f;
  }
  // activations: lane (c, kb) owns the two codes that unpack16() leaves in register c
  // of k-group kb (element k_lo in the low half, k_hi in the high half)
  const uint64_t tw = c < 8 ? (c < 4 ? hq_q3::packed_entries(0) : hq_q3::packed_entries(1))
                            : (c < 12 ? hq_q3::packed_entries(2) : hq_q3::packed_entries(3));
  const uint32_t te = (uint32_t)(tw >> (16 * (c & 3))) & 0xffffu;
  const int k_lo = te & 31, k_hi = (te >> 5) & 31, p_lo = (te >> 10) & 7, p_hi = (te >> 13) & 7;
  // Scalar base pointers of this workgroup's slice plus 32-bit per-lane byte offsets.
  const char* xbase = reinterpret_cast<const char*>(a.x) + (size_t)g_begin * 32 * (XF16 ? 2 : 4);
  // weights: out-of-range columns read the last valid quad (their results are never
  // stored), out-of-range k-groups read a valid group and get zero activations
  const int tile_cols = min(64, a.N - tile * 64);           // multiple of 4
  const uint32_t col_off = (uint32_t)min(4 * c, tile_cols - 4) * 4u;
  const uint32_t row_bytes = (uint32_t)a.N * 4u;
  const char* wbase = reinterpret_cast<const char*>(a.w) + ((size_t)(3 * g_begin) * row_stride + (size_t)tile * 64) * 4;
  constexpr int GPR = WAVES * 4 * STEPS;  // k-groups per round
  const int rounds = MULTI ? (g_count + GPR - 1) / GPR : 1;  // !MULTI: the host sized gpw <= GPR

  // Every global load of a round is issued up front and none sits under a branch
  // (addresses are clamped instead), so the compiler can count them and the wait for the
  // activations does not wait for the weights.
  auto load_round = [&](int r, float (&xr)[STEPS][2], uint32_t (&wreg)[STEPS][3][4]) {
    uint32_t glc[STEPS];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      glc[s] = (uint32_t)min((r * STEPS + s) * (WAVES * 4) + wv * 4 + kb, g_count - 1);
      if (XF16) {
        xr[s][0] = (float)*reinterpret_cast<const _Float16*>(xbase + (glc[s] * 32u + (uint32_t)k_lo) * 2u);
        xr[s][1] = (float)*reinterpret_cast<const _Float16*>(xbase + (glc[s] * 32u + (uint32_t)k_hi) * 2u);
      } else {
        xr[s][0] = *reinterpret_cast<const float*>(xbase + (glc[s] * 32u + (uint32_t)k_lo) * 4u);
        xr[s][1] = *reinterpret_cast<const float*>(xbase + (glc[s] * 32u + (uint32_t)k_hi) * 4u);
      }
    }
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
#pragma unroll
      for (int j = 0; j < 3; ++j) {
        const uint32_t off = (glc[s] * 3u + (uint32_t)j) * row_bytes + col_off;
        u4v v = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(wbase + off));
        wreg[s][j][0] = v.x; wreg[s][j][1] = v.y; wreg[s][j][2] = v.z; wreg[s][j][3] = v.w;
      }
    }
  };

  uint4* xs_w = xs + wv * (STEPS * 64);
  const int piece = c < 3 ? c : 2;  // columns 3..15 of the MFMA are never read
  float run[4][4];                  // per-digit sums of all rounds, already divided by 2^E
#pragma unroll
  for (int q = 0; q < 4; ++q)
#pragma unroll
    for (int i = 0; i < 4; ++i) run[q][i] = 0.f;
  float asum_total = 0.f;

  float xr[STEPS][2];
  uint32_t wreg[STEPS][3][4];
  load_round(0, xr, wreg);
  for (int r = 0; r < rounds; ++r) {
    float xr_next[STEPS][2];
    uint32_t wreg_next[STEPS][3][4];
    if (MULTI && r + 1 < rounds) load_round(r + 1, xr_next, wreg_next);  // in flight during this round

    // ---- stage this wave's activation digits in operand-slot order (wave-local) ----------
    float amax = 0.f, asum = 0.f;
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      if ((r * STEPS + s) * (WAVES * 4) + wv * 4 + kb >= g_count) { xr[s][0] = 0.f; xr[s][1] = 0.f; }
      amax = fmaxf(amax, fmaxf(fabsf(xr[s][0]), fabsf(xr[s][1])));
      asum += xr[s][0] + xr[s][1];
    }
    const float xmax = wave_max(amax);
    asum_total += wave_sum(asum);
    // 2^E * max|x| lies in [2^14, 2^15): digit 0 never overflows fp16.
    int E = 14 - ((int)((__float_as_uint(xmax) >> 23) & 255u) - 127);
    E = xmax > 0.f ? max(-120, min(120, E)) : 0;
    const float scaleE = pow2f(E);
    // Fixed-point split of v = x * 2^(E + 4 - pos) (|v| < 2^(19-pos)) into three signed
    // 11-bit digits with quanta 2^9, 2^-2, 2^-13, stored as plain fp16 integers.  With the
    // operand value code*2^(pos-24) every digit-0 product is an integer below 2^13 in units
    // of 2^-24, so a round's digit-0 chain (at most 512 slots) is exact in the matrix core
    // whatever its internal rounding is; digits 1 and 2 carry 2^-11 and 2^-22 of the weight.
    const float sE_lo = scaleE * pow2f(4 - p_lo), sE_hi = scaleE * pow2f(4 - p_hi);
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      float d[2][3];
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const float v = xr[s][e] * (e ? sE_hi : sE_lo);
        d[e][0] = rintf(v * 0.001953125f);
        const float r1 = v - d[e][0] * 512.f;   // exact
        d[e][1] = rintf(r1 * 4.f);
        const float r2 = r1 - d[e][1] * 0.25f;  // exact
        d[e][2] = rintf(r2 * 8192.f);
      }
      // register c of MFMA j = c/4 of this k-group: dword c%4 of the 16-byte operand chunk
      uint32_t* dst = reinterpret_cast<uint32_t*>(xs_w + ((s * 4 + kb) * 4 + (c >> 2)) * 4) + (c & 3);
#pragma unroll
      for (int p = 0; p < 3; ++p) {
        const h2v pair = {(_Float16)d[0][p], (_Float16)d[1][p]};
        dst[4 * p] = __builtin_bit_cast(uint32_t, pair);
      }
    }
    // The digits are read back by other lanes of this wave only: order the LDS writes
    // before the reads without a workgroup barrier.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");

    // ---- unpack + MFMA ---------------------------------------------------------------------
    f4 acc[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) acc[q] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      if ((r * STEPS + s) * (WAVES * 4) + wv * 4 >= g_count) continue;  // wave-uniform
      const uint4* xb = xs_w + (size_t)(s * 4 + kb) * 16 + piece;
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
    const float descale = pow2f(-E);
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int i = 0; i < 4; ++i) run[q][i] = fmaf(acc[q][i], descale, run[q][i]);
    // the LDS digits of this round must be consumed before the next round overwrites them
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    if (MULTI && r + 1 < rounds) {
#pragma unroll
      for (int s = 0; s < STEPS; ++s) {
        xr[s][0] = xr_next[s][0]; xr[s][1] = xr_next[s][1];
#pragma unroll
        for (int j = 0; j < 3; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q) wreg[s][j][q] = wreg_next[s][j][q];
      }
    }
  }

  // ---- combine waves, digits, scale/zero --------------------------------------------------
  // D[row = 4*kb + i][col = c]: row is the weight column (quarter-major), col the digit.
  if (c < 3) {
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[(wv * 3 + c) * 64 + 4 * (4 * kb + i) + q] = run[q][i];
  }
  if (lane == 0) wsum[wv] = asum_total;
  __syncthreads();
  float val = 0.f;
  if (tid < 64 && n < a.N) {
    const float inv11 = 1.f / 2048.f;
    float qx = 0.f, xsum = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      const float c0 = red[(w * 3 + 0) * 64 + tid];
      const float c1 = red[(w * 3 + 1) * 64 + tid];
      const float c2 = red[(w * 3 + 2) * 64 + tid];
      qx += fmaf(fmaf(c2, inv11, c1), inv11, c0);
      xsum += wsum[w];
    }
    // 2^24 (operand scale) * 2^9 (digit-0 quantum) * 2^-4 (slot scale)
    val = sc_n * (qx * 536870912.f) - zr_n * xsum;
    if (a.nsplit == 1) {
      a.y[n] = y_old + val;
    } else {
      // Device-coherent (write-through) store: visible to the other XCDs' workgroups
      // without flushing or invalidating this XCD's L2.
      __hip_atomic_store(&a.partial[((size_t)tile * a.nsplit + split) * 64 + tid], val, __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  if (a.nsplit > 1) {
    // Arrival counting with relaxed device-scope atomics only.  The barrier waits for
    // this workgroup's partial-sum stores to be acknowledged (they are write-through,
    // so acknowledged means visible device-wide) before the counter is bumped; the last
    // workgroup to arrive reads every partial with device-coherent loads and adds them
    // in split order, so the result does not depend on the arrival order.  Full
    // release/acquire fences are avoided on purpose: on this multi-XCD part they write
    // back and invalidate the whole L2 and cost tens of microseconds per call.
    __shared__ unsigned s_last;
    __syncthreads();
    if (tid == 0) {
      const unsigned old = __hip_atomic_fetch_add(&a.counters[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      s_last = (old == (unsigned)(a.nsplit - 1));
    }
    __syncthreads();
    if (s_last) {
      if (tid < 64 && n < a.N) {
        float sum = 0.f;
        for (int s = 0; s < a.nsplit; ++s)
          sum += __hip_atomic_load(&a.partial[((size_t)tile * a.nsplit + s) * 64 + tid],
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        a.y[n] = (a.flags & HQ_FLAG_ACCUMULATE) ? a.y[n] + sum : sum;
      }
      if (tid == 0)  // ready for the next call
        __hip_atomic_store(&a.counters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

template <int WAVES, int STEPS, bool XF16, bool MULTI>
int launch_matvec_t(const Q3Args& a, int ntiles, hipStream_t stream) {
  const size_t smem = (size_t)WAVES * STEPS * 1024 + (size_t)WAVES * 3 * 64 * 4 + (size_t)WAVES * 2 * 4;
  static const hipError_t attr =
      hipFuncSetAttribute(reinterpret_cast<const void*>(&q3_matvec_kernel<WAVES, STEPS, XF16, MULTI>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
  if (attr != hipSuccess) return (int)attr;
  hipLaunchKernelGGL((q3_matvec_kernel<WAVES, STEPS, XF16, MULTI>), dim3(ntiles, a.nsplit), dim3(WAVES * 64), smem,
                     stream, a);
  return hq_launch_status();
}
template <int WAVES, int STEPS>
int launch_matvec(const Q3Args& a, int ntiles, hipStream_t stream) {
  const bool multi = a.gpw > WAVES * 4 * STEPS;
  if (a.x_f16)
    return multi ? launch_matvec_t<WAVES, STEPS, true, true>(a, ntiles, stream)
                 : launch_matvec_t<WAVES, STEPS, true, false>(a, ntiles, stream);
  return multi ? launch_matvec_t<WAVES, STEPS, false, true>(a, ntiles, stream)
               : launch_matvec_t<WAVES, STEPS, false, false>(a, ntiles, stream);
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
  if (((uintptr_t)qweight & 15) || ((uintptr_t)x & (x_dtype == HQ_DTYPE_F16 ? 3 : 7)) ||
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
  // Launch shape: a workgroup of WAVES waves covers WAVES*4*STEPS k-groups per round and
  // walks its K range in rounds (the next round's loads are in flight during the current
  // one).  K is split across workgroups only as far as needed to give every CU a
  // workgroup: the split costs a device-scope round trip per workgroup.
  int waves = hq_env_int("HQ_Q3_WAVES", 8);
  int steps = hq_env_int("HQ_Q3_STEPS", 0);
  if (waves != 4 && waves != 8 && waves != 16) waves = 8;
  if (waves == 16) steps = 1;  // register budget of 16-wave workgroups
  if (steps != 1 && steps != 2 && steps != 4 && (steps != 8 || waves != 4)) {
    steps = 4;
    while (steps > 1 && waves * 4 * (steps / 2) >= G) steps /= 2;  // short K: fewer steps
  }
  const int gpr = waves * 4 * steps;  // k-groups one workgroup covers per round
  const int max_split = (G + gpr - 1) / gpr;
  int nsplit = hq_env_int("HQ_Q3_KSPLIT", 0);
  if (nsplit <= 0) nsplit = dev->cus / ntiles;  // only when there are fewer tiles than half the CUs
  if (nsplit > max_split) nsplit = max_split;
  if (nsplit < 1) nsplit = 1;
  int gpw = (G + nsplit - 1) / nsplit;
  gpw = (gpw + gpr - 1) / gpr * gpr;  // whole rounds
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
  HQ_Q3_CASE(16, 1)
  HQ_Q3_CASE(8, 1) HQ_Q3_CASE(8, 2) HQ_Q3_CASE(8, 4)
  HQ_Q3_CASE(4, 1) HQ_Q3_CASE(4, 2) HQ_Q3_CASE(4, 4) HQ_Q3_CASE(4, 8)
#undef HQ_Q3_CASE
  return HQ_ERR_BAD_ENUM;
}
