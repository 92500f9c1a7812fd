// GPTQ 3-bit matvec for two activation rows at once (batch 2) for gfx950.
//
// The batch-1 kernel (q3.hip) leaves seven of the sixteen matrix-core columns unused: its B operand
// carries the eight 4-bit digits of ONE fixed-point activation vector plus a column of ones.  Here the
// sixteen columns carry SEVEN digits of each of TWO rows: |x| in 28-bit fixed point relative to the wave's
// largest magnitude of that row, cut into nibbles, the sign in the fp8 sign bit of every digit byte (so no
// bias has to be taken out and no column of ones is needed).  The packed weights are read once for both
// rows at the matvec's nine VALU instructions per 32 weights, instead of the batched GEMM's twenty plus
// its pre-pass.  Everything else follows q3.hip: a workgroup owns a 64-column tile and all of K, a wave's
// 16-lane quarter streams one k-group per step as three 128-bit loads, every wave stages its own digits
// in LDS behind a wave-local fence, all products and partial sums inside the matrix core are small
// integers (exact), and the waves meet once at the end.  (Three rows of five digits fit as well and were
// built: 25.1 us against the GEMM's 26 at K=8192, N=28672, with 20-bit activations - not worth a second
// accuracy class.)  No counterpart in the reference (its kernels are batch 1:
// src/quant3MatMul-hip/kernels.h:12-217).
#include "hq_internal.h"

namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4v __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));

struct RowsArgs {
  const _Float16* x;  // [rows][K]
  const uint32_t* w;
  const float* scales;
  const float* zeros;
  float* y;           // [rows][N]
  float* partial;     // [tile][split][rows][64] when K is split
  unsigned* counters; // [tile] arrival counters, zero between calls
  int K, N;
  int gpw;            // k-groups per workgroup
  int nsplit;         // workgroups per column tile
  unsigned flags;
};

__device__ __forceinline__ float pow2f(int e) { return __uint_as_float((uint32_t)(e + 127) << 23); }

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

constexpr uint32_t low3_mask(int word) {
  uint32_t m = 0;
  for (int b = 0; b < 32; ++b)
    if ((32 * word + b) % 6 < 3) m |= 1u << b;
  return m;
}

// 4x4 byte transpose: in[j] holds four digits of value j, out[i] digit i of the four values.
__device__ __forceinline__ void transpose4(uint32_t a, uint32_t b, uint32_t c, uint32_t d, uint32_t (&o)[4]) {
  const uint32_t p0 = __builtin_amdgcn_perm(b, a, 0x05010400u);
  const uint32_t p1 = __builtin_amdgcn_perm(b, a, 0x07030602u);
  const uint32_t p2 = __builtin_amdgcn_perm(d, c, 0x05010400u);
  const uint32_t p3 = __builtin_amdgcn_perm(d, c, 0x07030602u);
  o[0] = __builtin_amdgcn_perm(p2, p0, 0x05040100u);
  o[1] = __builtin_amdgcn_perm(p2, p0, 0x07060302u);
  o[2] = __builtin_amdgcn_perm(p3, p1, 0x05040100u);
  o[3] = __builtin_amdgcn_perm(p3, p1, 0x07060302u);
}

constexpr int kDigits = 7;          // 4-bit digits per activation: 28-bit fixed point
constexpr int kRowBytes = 144;      // one B operand row (4 lane quarters x 32 B) plus 16 B: rows start 4 banks apart
constexpr int kStepBytes = 2176;    // fourteen digit rows per step plus room for the step's skew
constexpr int kZeroBytes = 128;     // a wave's row of zeros (4 lane quarters x 32 B) behind its steps
constexpr int kRedStride = 68;      // floats per digit column of a wave's final sums
__device__ __forceinline__ constexpr int step_off(int s) {
  return s * kStepBytes + (s & 1) * 32 + ((s >> 1) & 1) * 128;
}

// MULTI: the workgroup walks its K range in rounds, the next round's loads in flight during the current
// one.  Otherwise its range is one round, it needs half the registers and less than half the LDS of a CU,
// and two workgroups share a CU.
template <int WAVES, int STEPS, int ROWS, bool MULTI>
__global__ __launch_bounds__(WAVES * 64) void q3_rows_kernel(RowsArgs a) {
  // LDS: dig[WAVES][STEPS * kStepBytes + kZeroBytes] (a wave's final sums re-use its area) | part[WAVES][ROWS][64] |
  // wsum[WAVES][ROWS]
  extern __shared__ uint4 smem[];
  constexpr int kWaveBytes = STEPS * kStepBytes + kZeroBytes;
  char* dig = reinterpret_cast<char*>(smem);
  float* part = reinterpret_cast<float*>(dig + WAVES * kWaveBytes);
  float* wsum = part + WAVES * ROWS * 64;
  static_assert(STEPS * kStepBytes >= 14 * kRedStride * 4, "a wave's digit area must hold its final sums");

  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int c = lane & 15, kb = lane >> 4;
  const int tile = blockIdx.x, split = blockIdx.y;
  const int g_begin = split * a.gpw;
  const int G = min(a.gpw, (a.K >> 5) - g_begin);  // k-groups of this workgroup
  const int ncol = tile * 64 + (tid & 63);

  float sc_n = 0.f, zr_n = 0.f, y_old = 0.f;
  if (tid < 64 * ROWS) {
    const int nc = min(ncol, a.N - 1);
    sc_n = a.scales[nc];
    zr_n = a.zeros[nc];
    y_old = ((a.flags & HQ_FLAG_ACCUMULATE) && a.nsplit == 1) ? a.y[(size_t)(tid >> 6) * a.N + nc] : 0.f;
  }
  // staging role: lane converts the eight consecutive activations 8*xq .. 8*xq+7 of k-group xkb of step 4*pass + xs
  const int xs = lane >> 4, xkb = (lane >> 2) & 3, xq = lane & 3;
  constexpr int XP = (STEPS + 3) / 4;
  const int tile_cols = min(64, a.N - tile * 64);  // multiple of 4
  const uint32_t col_off = (uint32_t)min(4 * c, tile_cols - 4) * 4u;
  const uint32_t row_bytes = (uint32_t)a.N * 4u;
  const char* wbase = reinterpret_cast<const char*>(a.w) + (size_t)g_begin * 3 * row_bytes + (size_t)tile * 64 * 4;
  const _Float16* xbase = a.x + (size_t)g_begin * 32;
  constexpr int GPR = WAVES * 4 * STEPS;  // k-groups per round
  const int rounds = MULTI ? (G + GPR - 1) / GPR : 1;  // !MULTI: the host sized gpw <= GPR

  auto load_round = [&](int r, u4v (&xraw)[ROWS][XP], uint32_t (&wreg)[STEPS][3][4]) {
#pragma unroll
    for (int m = 0; m < ROWS; ++m)
#pragma unroll
      for (int p = 0; p < XP; ++p) {
        const int s = min(4 * p + xs, STEPS - 1);
        const uint32_t g = (uint32_t)min((r * STEPS + s) * (WAVES * 4) + wv * 4 + xkb, G - 1);
        xraw[m][p] = *reinterpret_cast<const u4v*>(xbase + (size_t)m * a.K + g * 32u + (uint32_t)xq * 8u);
      }
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      const uint32_t g = (uint32_t)min((r * STEPS + s) * (WAVES * 4) + wv * 4 + kb, G - 1);
#pragma unroll
      for (int j = 0; j < 3; ++j) {
        const size_t off = (size_t)(g * 3u + (uint32_t)j) * row_bytes + col_off;
        const u4v v = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(wbase + off));
        wreg[s][j][0] = v.x; wreg[s][j][1] = v.y; wreg[s][j][2] = v.z; wreg[s][j][3] = v.w;
      }
    }
  };

  char* dig_w = dig + wv * kWaveBytes;
  // MFMA column c reads digit row c of the step while it carries a digit (c < 7 ROWS) and the wave's row of
  // zeros otherwise.
  static_assert(kDigits * ROWS <= 14, "a step holds fourteen digit rows");
  if (lane < kZeroBytes / 4) *reinterpret_cast<uint32_t*>(dig_w + STEPS * kStepBytes + lane * 4) = 0u;
  const bool digit_col = c < kDigits * ROWS;
  const int b_off = digit_col ? c * kRowBytes + kb * 32 : STEPS * kStepBytes + kb * 32;
  const int my_row = min(c / kDigits, ROWS - 1);  // the activation row whose digit this lane's MFMA column carries

  float run[4][4];
#pragma unroll
  for (int q = 0; q < 4; ++q)
#pragma unroll
    for (int i = 0; i < 4; ++i) run[q][i] = 0.f;
  float asum_total[ROWS];
#pragma unroll
  for (int m = 0; m < ROWS; ++m) asum_total[m] = 0.f;
  constexpr uint32_t M0 = low3_mask(0), M1 = low3_mask(1), M2 = low3_mask(2);

  u4v xraw[ROWS][XP];
  uint32_t wreg[STEPS][3][4];
  load_round(0, xraw, wreg);
  for (int r = 0; r < rounds; ++r) {
    u4v xraw_next[ROWS][XP];
    uint32_t wreg_next[STEPS][3][4];
    if (MULTI && r + 1 < rounds) load_round(r + 1, xraw_next, wreg_next);  // in flight during this round

    // ---- stage this wave's digits, one activation row after the other ----------------------------
    float descale_lane = 0.f;
#pragma unroll
    for (int m = 0; m < ROWS; ++m) {
      float xr[XP][8];
      float amax = 0.f, asum = 0.f;
#pragma unroll
      for (int p = 0; p < XP; ++p) {
        const int s = 4 * p + xs;
        const bool live = s < STEPS && (r * STEPS + s) * (WAVES * 4) + wv * 4 + xkb < G;
        const h8 h = __builtin_bit_cast(h8, xraw[m][p]);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          xr[p][j] = live ? (float)h[j] : 0.f;
          amax = fmaxf(amax, fabsf(xr[p][j]));
          asum += xr[p][j];
        }
      }
      const float xmax = wave_max(amax);
      asum_total[m] += wave_sum(asum);
      // 2^E * max|x| lies in [2^27, 2^28): u = rint(|x| * 2^E) stays inside 28 bits (an fp16 maximum times
      // 2^E is a multiple of 2^17), u = sum_d 16^d n_d
      int E = 27 - ((int)((__float_as_uint(xmax) >> 23) & 255u) - 127);
      E = xmax > 0.f ? max(-120, min(120, E)) : 0;
      const float scaleE = pow2f(E);
      if (my_row == m) descale_lane = pow2f(-E);
#pragma unroll
      for (int p = 0; p < XP; ++p) {
        uint32_t ev[8], od[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const uint32_t u = (uint32_t)(int)rintf(fabsf(xr[p][j]) * scaleE);
          const uint32_t sg = (uint32_t)((int)__float_as_uint(xr[p][j]) >> 31) & 0x80808080u;  // fp8 sign bits
          ev[j] = (u & 0x0f0f0f0fu) | sg;         // nibbles 0 2 4 6
          od[j] = ((u >> 4) & 0x0f0f0f0fu) | sg;  // nibbles 1 3 5 (the fourth byte is a signed zero)
        }
        // even / odd elements of the k-group go to neighbouring lane quarters of the fp8 operand (see q3.hip)
        uint32_t de[2][4], dd[2][4];
        transpose4(ev[0], ev[2], ev[4], ev[6], de[0]);
        transpose4(ev[1], ev[3], ev[5], ev[7], de[1]);
        transpose4(od[0], od[2], od[4], od[6], dd[0]);
        transpose4(od[1], od[3], od[5], od[7], dd[1]);
        const int s = 4 * p + xs;
        if (s < STEPS) {
          char* dst = dig_w + step_off(s) + (kDigits * m) * kRowBytes + (xkb & 1) * 64 + (xkb >> 1) * 16 + xq * 4;
#pragma unroll
          for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int i = 0; i < 4; ++i) *reinterpret_cast<uint32_t*>(dst + (2 * i) * kRowBytes + h * 32) = de[h][i];
#pragma unroll
            for (int i = 0; i < 3; ++i) *reinterpret_cast<uint32_t*>(dst + (2 * i + 1) * kRowBytes + h * 32) = dd[h][i];
          }
        }
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");

    // ---- mask + MFMA -----------------------------------------------------------------------
    f4 acc[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) acc[q] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      if ((r * STEPS + s) * (WAVES * 4) + wv * 4 >= G) continue;  // wave-uniform
      const u4v* bp = reinterpret_cast<const u4v*>(dig_w + (digit_col ? step_off(s) + b_off : b_off));
      const u4v b0 = bp[0], b1 = bp[1];
      const v8i B = {(int)b0.x, (int)b0.y, (int)b0.z, (int)b0.w, (int)b1.x, (int)b1.y, (int)b1.z, (int)b1.w};
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const uint32_t w0 = wreg[s][0][q], w1 = wreg[s][1][q], w2 = wreg[s][2][q];
        const v8i A = {(int)(w0 & M0), (int)(w1 & M1), (int)(w2 & M2),
                       (int)(__builtin_amdgcn_alignbit(w1, w0, 3) & M0),
                       (int)(__builtin_amdgcn_alignbit(w2, w1, 3) & M1), (int)((w2 >> 3) & M2), 0, 0};
        // A: fp6 e2m3 (cbsz 2), B: fp8 e4m3 (blgp 0), unit block scales
        acc[q] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A, B, acc[q], 2, 0, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
      }
    }
    // leave the fixed-point scale of the column's activation row
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int i = 0; i < 4; ++i) run[q][i] = fmaf(acc[q][i], descale_lane, run[q][i]);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    if (MULTI && r + 1 < rounds) {
#pragma unroll
      for (int m = 0; m < ROWS; ++m)
#pragma unroll
        for (int p = 0; p < XP; ++p) xraw[m][p] = xraw_next[m][p];
#pragma unroll
      for (int s = 0; s < STEPS; ++s)
#pragma unroll
        for (int j = 0; j < 3; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q) wreg[s][j][q] = wreg_next[s][j][q];
    }
  }

  // ---- combine digits (inside the wave), then waves, scale and zero ------------------------------
  // D[row = 4*kb + i][col = c]: row is the weight column 4*row + q of the tile, col the (row, digit) pair.
  float* red_w = reinterpret_cast<float*>(dig_w);
  if (c < kDigits * ROWS) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const f4 v = {run[0][i], run[1][i], run[2][i], run[3][i]};
      *reinterpret_cast<f4*>(red_w + c * kRedStride + 4 * (4 * kb + i)) = v;
    }
  }
  if (lane == 0) {
#pragma unroll
    for (int m = 0; m < ROWS; ++m) wsum[wv * ROWS + m] = asum_total[m];
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
#pragma unroll
  for (int m = 0; m < ROWS; ++m) {
    const float* rw = red_w + (kDigits * m) * kRedStride + lane;
    float h = rw[(kDigits - 1) * kRedStride];
#pragma unroll
    for (int d = kDigits - 2; d >= 0; --d) h = fmaf(h, 16.f, rw[d * kRedStride]);
    part[(wv * ROWS + m) * 64 + lane] = h;
  }
  __syncthreads();
  if (tid < 64 * ROWS && ncol < a.N) {
    const int m = tid >> 6, col = tid & 63;
    float qx = 0.f, xsum = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      qx += part[(w * ROWS + m) * 64 + col];
      xsum += wsum[w * ROWS + m];
    }
    float val = sc_n * (qx * 4096.f) - zr_n * xsum;  // 2^12: fp6 unit 2^-3 times fp8 unit 2^-9
    val = fmaf(xsum, 0.f, val);  // a NaN or infinity among the activations makes the result NaN
    if (a.nsplit == 1)
      __hip_atomic_store(&a.y[(size_t)m * a.N + ncol], y_old + val, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else
      __hip_atomic_store(&a.partial[(((size_t)tile * a.nsplit + split) * ROWS + m) * 64 + col], val, __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
  }
  if (a.nsplit > 1) {
    // Arrival counting as in q3.hip: write-through partial sums, every wave waits for their acknowledgement,
    // a barrier, one device-scope fetch-add per workgroup, and the last workgroup to arrive adds the partial
    // sums in split order with loads that bypass the non-coherent cache levels.
    __shared__ unsigned s_last;
    const bool strict = (a.flags & HQ_FLAG_STRICT_FENCES) != 0;
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (tid == 0) {
      const unsigned old = strict ? __hip_atomic_fetch_add(&a.counters[tile], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT)
                                  : __hip_atomic_fetch_add(&a.counters[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      s_last = (old == (unsigned)(a.nsplit - 1));
    }
    __syncthreads();
    if (s_last && strict) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    if (s_last) {
      if (tid < 64 * ROWS && ncol < a.N) {
        const int m = tid >> 6, col = tid & 63;
        float sum = 0.f;
        for (int s = 0; s < a.nsplit; ++s)
          sum += __hip_atomic_load(&a.partial[(((size_t)tile * a.nsplit + s) * ROWS + m) * 64 + col], __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
        float* yp = &a.y[(size_t)m * a.N + ncol];
        *yp = (a.flags & HQ_FLAG_ACCUMULATE) ? *yp + sum : sum;
      }
      if (tid == 0)  // ready for the next call
        __hip_atomic_store(&a.counters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

template <int ROWS, bool MULTI>
int launch_rows_t(const RowsArgs& a, hipStream_t stream) {
  constexpr int WAVES = 8, STEPS = 4;
  const size_t smem = (size_t)WAVES * (STEPS * kStepBytes + kZeroBytes) + (size_t)WAVES * ROWS * 64 * 4 +
                      (size_t)WAVES * ROWS * 4 + 16;
  static const hipError_t attr =
      hipFuncSetAttribute(reinterpret_cast<const void*>(&q3_rows_kernel<WAVES, STEPS, ROWS, MULTI>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);
  if (attr != hipSuccess) return (int)attr;
  hipLaunchKernelGGL((q3_rows_kernel<WAVES, STEPS, ROWS, MULTI>), dim3((a.N + 63) / 64, a.nsplit), dim3(WAVES * 64), smem,
                     stream, a);
  return hq_launch_status();
}

}  // namespace

// k-groups one workgroup of the two-row kernel covers per round
int hq_q3_rows_groups_per_round(void) { return 8 * 4 * 4; }

// Two fp16 activation rows; the caller has validated the arguments, sized gpw to whole rounds and, for
// nsplit > 1, provided nsplit * 128 floats of partial sums and one zeroed counter per column tile.
int hq_q3_rows_launch(const void* x, const int32_t* qweight, const float* scales, const float* zeros, float* y,
                      int K, int N, int gpw, int nsplit, float* partial, unsigned* counters, unsigned flags,
                      hipStream_t stream) {
  RowsArgs a;
  a.x = reinterpret_cast<const _Float16*>(x);
  a.w = reinterpret_cast<const uint32_t*>(qweight);
  a.scales = scales; a.zeros = zeros; a.y = y; a.partial = partial; a.counters = counters; a.K = K; a.N = N;
  a.gpw = gpw; a.nsplit = nsplit; a.flags = flags & (HQ_FLAG_ACCUMULATE | HQ_FLAG_STRICT_FENCES);
  return gpw > hq_q3_rows_groups_per_round() ? launch_rows_t<2, true>(a, stream) : launch_rows_t<2, false>(a, stream);
}
