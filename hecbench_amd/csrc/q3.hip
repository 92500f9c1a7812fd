// GPTQ 3-bit matvec (batch 1) for gfx950.
//
// Replaces VecQuant3MatMulKernel / VecQuant3MatMulKernelFaster and their host
// launchers (src/quant3MatMul-hip/kernels.h:12-217 in the HeCBench tree).
//
//   y[n] = sum_k x[k] * (s[n]*q[k][n] - z[n]) = s[n] * sum_k q[k][n]*x[k] - z[n] * sum_k x[k]
//
// The kernel is HBM-bound only if a weight costs well under two VALU
// instructions (17 MB / 8 TB/s leaves ~1.85 lane-ops per weight on 256 CUs), so
// the integer codes are never converted one by one.  The 96-bit string of a
// k-group's 32 codes is, read six bits at a time, a string of 16 fp6 (e2m3)
// numbers whose exponent bits happen to hold the next code: one AND per word
// keeps the even codes as fp6 subnormals code/8, one funnel shift and AND per
// word does the same for the odd codes, and the six registers are the A operand
// of one 16x16x128 f8f6f4 MFMA (nine VALU instructions per 32 weights).  The B
// operand carries the activations as fixed point: x * 2^E rounded to a 31-bit
// integer, biased by 0x88888888 and cut into eight nibbles; a nibble 0..15 in an
// otherwise zero byte is the fp8 (e4m3) number nibble * 2^-9, so no conversion
// is needed, only a byte transpose.  MFMA column d holds nibble d, column 8 a
// constant one (it yields sum_k q[k], which takes the bias out again).  Every
// product and partial sum is a small integer, so the matrix-core accumulation
// is exact; the roundings are those of the fp32 epilogue.
//
// Work split: a workgroup owns a 64-column tile and WAVES*4*STEPS consecutive
// k-groups per round; a wave's 16-lane quarter `kb` streams one k-group per step
// as three uint4 loads (4 adjacent columns x 3 packed rows), i.e. 256 contiguous
// bytes per packed row per quarter.  A wave issues all its global loads first,
// stages its own activation digits in LDS without a workgroup barrier, and meets
// the other waves only in the final reduction.  When one workgroup covers all of
// K no cross-workgroup reduction is needed; otherwise (split-K) the partial sums
// go to a workspace and the last workgroup to arrive at a tile adds them in a
// fixed order, so results do not depend on arrival order.
#include "hq_internal.h"
#include "q3_recipe.h"

namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4v __attribute__((ext_vector_type(4)));
typedef uint32_t u2v __attribute__((ext_vector_type(2)));
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

// Bits of word `word` of the 96-bit string that belong to the low three bits of a 6-bit field.
constexpr uint32_t low3_mask(int word) {
  uint32_t m = 0;
  for (int b = 0; b < 32; ++b)
    if ((32 * word + b) % 6 < 3) m |= 1u << b;
  return m;
}

// Row-wise broadcast of lane 8 of each 16-lane row (DPP row_newbcast:8).
__device__ __forceinline__ float row_bcast8(float v) { return dpp_f<0x158>(v); }

// 4x4 byte transpose: in[j] holds four digits of value j, out[i] digit i of the four values.
__device__ __forceinline__ void transpose4(uint32_t a, uint32_t b, uint32_t c, uint32_t d, uint32_t (&o)[4]) {
  const uint32_t p0 = __builtin_amdgcn_perm(b, a, 0x05010400u);  // a0 b0 a1 b1
  const uint32_t p1 = __builtin_amdgcn_perm(b, a, 0x07030602u);  // a2 b2 a3 b3
  const uint32_t p2 = __builtin_amdgcn_perm(d, c, 0x05010400u);
  const uint32_t p3 = __builtin_amdgcn_perm(d, c, 0x07030602u);
  o[0] = __builtin_amdgcn_perm(p2, p0, 0x05040100u);
  o[1] = __builtin_amdgcn_perm(p2, p0, 0x07060302u);
  o[2] = __builtin_amdgcn_perm(p3, p1, 0x05040100u);
  o[3] = __builtin_amdgcn_perm(p3, p1, 0x07060302u);
}

typedef int v8i __attribute__((ext_vector_type(8)));

// LDS layout of one step's B operand (nine rows: eight digits and the row of ones; four lane quarters, two
// 16-byte halves per quarter and row), chosen so that neither the 128-bit operand reads nor the 32-bit staging
// stores meet in a bank.  Measured on this part: a 128-bit LDS read is served in four passes of 16 lanes - lanes
// 0-3, 12-15 and 20-27, then 4-11, 16-19 and 28-31, then the same of the upper half wave - over 256 bytes of
// banks; 32-bit accesses in two passes of 32 lanes over 128 bytes of banks.  A read pass therefore takes rows
// 0-3 and 8 of one quarter and rows 4-8 of its neighbour: a (quarter, half) block holds its rows as consecutive
// 16-byte pieces (row r at piece r; the row of ones at piece 8 in even quarters, 9 in odd ones), quarters 512
// bytes apart (the same banks), the second half 176 bytes behind the first, steps 1888 bytes apart; the staging
// gives the 32 lanes of a store pass four steps, both halves and one quarter parity (44-, 472- and 944-word
// strides: all eight multiples of four banks).
constexpr int kStepBytes = 1888;
__device__ __forceinline__ constexpr int dig_piece(int row, int quarter, int half) {
  return 16 * row + 512 * quarter + 176 * half;
}
constexpr int kRedStride = 68;    // floats per (wave, digit) row of the final reduction
// Byte offset of step s inside a wave's digit area
__device__ __forceinline__ constexpr int step_off(int s) { return s * kStepBytes; }

// ROUNDS: 0 one round per workgroup, 1 several with a round's loads issued at once one round ahead, 2 several
// with only the first step's loads at the top of a round and step s + 1 of the next round before the
// arithmetic of step s.
template <int WAVES, int STEPS, bool XF16, int ROUNDS, int CPL = 4>
__global__ __launch_bounds__(WAVES * 64) void q3_matvec_kernel(const uint32_t* w_, const void* x_, int K_, int N_, int gpw_,
                                                              int nsplit_, int x_f16_, unsigned flags_,
                                                              const float* scales_, const float* zeros_, float* y_,
                                                              float* partial_, unsigned* counters_) {
  // leading scalars rather than the struct: those are preloaded into scalar registers (the first 14 dwords,
  // i.e. everything the loads and the staging need; y, partial and counters are fetched for the tail)
  Q3Args a;
  a.x = x_; a.w = w_; a.scales = scales_; a.zeros = zeros_; a.y = y_; a.partial = partial_; a.counters = counters_;
  a.K = K_; a.N = N_; a.gpw = gpw_; a.nsplit = nsplit_; a.x_f16 = x_f16_; a.flags = flags_;
  // LDS: dig[WAVES][STEPS * kStepBytes] | red[WAVES][8][kRedStride] | part[WAVES][64] | xsum[WAVES]
  extern __shared__ uint4 smem[];
  char* dig = reinterpret_cast<char*>(smem);
  float* red = reinterpret_cast<float*>(dig + WAVES * STEPS * kStepBytes);
  float* part = red + WAVES * 8 * kRedStride;
  float* wsum = part + WAVES * 64;

  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int c = lane & 15, kb = lane >> 4;
  // A lane owns CPL adjacent columns, a workgroup TW = 16 * CPL.  Narrow tiles (CPL < 4) are dealt out so that
  // the 4 / CPL tiles of a 64-column group (whose packed rows share 128-byte lines) run on one XCD, in
  // neighbouring slots: workgroup b runs on XCD b mod 8.
  constexpr int TW = 16 * CPL, SUB = 4 / CPL;
  const int slot = blockIdx.x >> 3;
  const int tile = CPL == 4 ? (int)blockIdx.x : ((slot / SUB) * 8 + (int)(blockIdx.x & 7)) * SUB + slot % SUB;
  const int split = blockIdx.y;
  if (CPL < 4 && tile * TW >= a.N) return;  // the last group of eight may be short
  const int G = a.K >> 5;
  const int g_begin = split * a.gpw;
  const int g_count = min(a.gpw, G - g_begin);
  const size_t row_stride = (size_t)a.N;
  const int n = tile * TW + tid;

  // ---- loads that do not depend on the round ------------------------------------------------
  float sc_n = 0.f, zr_n = 0.f, y_old = 0.f;
  if (tid < TW) {
    const int nc = min(n, a.N - 1);
    sc_n = a.scales[nc];
    zr_n = a.zeros[nc];
    y_old = ((a.flags & HQ_FLAG_ACCUMULATE) && a.nsplit == 1) ? a.y[nc] : 0.f;
  }
  // Activation staging: lane L converts the eight consecutive activations 8*xq .. 8*xq+7 of
  // k-group xkb of step 4*pass + xs.
  // (lane bit 5, which selects the pass of a 32-bit LDS store, is the k-group's parity)
  const int xs = (lane >> 3) & 3, xkb = ((lane >> 2) & 1) * 2 + (lane >> 5), xq = lane & 3;
  constexpr int XP = (STEPS + 3) / 4;  // staging passes per round
  // Scalar base pointers of this workgroup's slice plus 32-bit per-lane byte offsets.
  const char* xbase = reinterpret_cast<const char*>(a.x) + (size_t)g_begin * 32 * (XF16 ? 2 : 4);
  // weights: out-of-range columns read the last valid quad (their results are never
  // stored), out-of-range k-groups read a valid group and get zero activations
  const int tile_cols = min(TW, a.N - tile * TW);           // multiple of 4
  const uint32_t col_off = (uint32_t)min(CPL * c, tile_cols - CPL) * 4u;
  const uint32_t row_bytes = (uint32_t)a.N * 4u;
  const char* wbase = reinterpret_cast<const char*>(a.w) + ((size_t)(3 * g_begin) * row_stride + (size_t)tile * TW) * 4;
  constexpr int GPR = WAVES * 4 * STEPS;  // k-groups per round
  constexpr bool MULTI = ROUNDS != 0;
  constexpr int kNextEarly = ROUNDS == 2 ? 1 : STEPS;  // steps of the next round loaded at the top of a round
  const int rounds = MULTI ? (g_count + GPR - 1) / GPR : 1;  // !MULTI: the host sized gpw <= GPR

  // No global load sits under a branch (addresses are clamped instead), so the compiler can count
  // them and the wait for the activations does not wait for the weights.  A workgroup with more than one
  // round issues a round's loads at once, one round ahead.  A single-round workgroup issues the
  // activations and the first kEarly steps' weights at entry and the weights of step s + kEarly just before the
  // arithmetic of step s: a compute unit takes about 64 KB of outstanding loads, a wave stalls at a
  // load while that queue is full, and a stalled wave stages nothing (K=4096, N=11008: 5.45 -> 5.38 us; one
  // step early 5.42, three 5.40).
  constexpr int kEarly = MULTI ? STEPS : (STEPS < 2 ? STEPS : 2);
  auto load_steps = [&](int r, uint32_t (&wreg)[STEPS][3][CPL], int s0, int s1) {
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      if (s < s0 || s >= s1) continue;
      const uint32_t g = (uint32_t)min((r * STEPS + s) * (WAVES * 4) + wv * 4 + kb, g_count - 1);
#pragma unroll
      for (int j = 0; j < 3; ++j) {
        const uint32_t off = (g * 3u + (uint32_t)j) * row_bytes + col_off;
        if constexpr (CPL == 4) {
          u4v v = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(wbase + off));
          wreg[s][j][0] = v.x; wreg[s][j][1] = v.y; wreg[s][j][2] = v.z; wreg[s][j][3] = v.w;
        } else if constexpr (CPL == 2) {
          u2v v = __builtin_nontemporal_load(reinterpret_cast<const u2v*>(wbase + off));
          wreg[s][j][0] = v.x; wreg[s][j][1] = v.y;
        } else {
          wreg[s][j][0] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(wbase + off));
        }
      }
    }
  };
  auto load_round = [&](int r, float (&xr)[XP][8], uint32_t (&wreg)[STEPS][3][CPL]) {
#pragma unroll
    for (int p = 0; p < XP; ++p) {
      const int s = min(4 * p + xs, STEPS - 1);
      const uint32_t g = (uint32_t)min((r * STEPS + s) * (WAVES * 4) + wv * 4 + xkb, g_count - 1);
      const uint32_t e = g * 32u + (uint32_t)xq * 8u;
      if (XF16) {
        const u4v raw = *reinterpret_cast<const u4v*>(xbase + e * 2u);
        const h8 h = __builtin_bit_cast(h8, raw);
#pragma unroll
        for (int j = 0; j < 8; ++j) xr[p][j] = (float)h[j];
      } else {
        const f4 lo = *reinterpret_cast<const f4*>(xbase + e * 4u);
        const f4 hi = *reinterpret_cast<const f4*>(xbase + e * 4u + 16u);
#pragma unroll
        for (int j = 0; j < 4; ++j) { xr[p][j] = lo[j]; xr[p][4 + j] = hi[j]; }
      }
    }
    load_steps(r, wreg, 0, (MULTI && r > 0) ? kNextEarly : kEarly);
  };

  char* dig_w = dig + wv * (STEPS * kStepBytes);
  // Row 8 of every step is the constant one (fp8 0x01 = 2^-9, the unit of the digits).
  {
    // lane = (quarter's high bit, step, quarter's low bit, dword): the 32 lanes of a store pass in 32 banks
    const int quarter = (lane >> 5) * 2 + ((lane >> 2) & 1);
#pragma unroll
    for (int s0 = 0; s0 < STEPS; s0 += 4) {
      const int s = s0 + ((lane >> 3) & 3);
      if (s < STEPS) {
        char* ones = dig_w + step_off(s) + dig_piece(8 + (quarter & 1), quarter, 0) + (lane & 3) * 4;
        *reinterpret_cast<uint32_t*>(ones) = 0x01010101u;
        *reinterpret_cast<uint32_t*>(ones + dig_piece(0, 0, 1)) = 0x01010101u;
      }
    }
  }
  float run[CPL][4];  // per-digit sums of all rounds (bias removed, divided by 2^E)
#pragma unroll
  for (int q = 0; q < CPL; ++q)
#pragma unroll
    for (int i = 0; i < 4; ++i) run[q][i] = 0.f;
  float asum_total = 0.f;
  constexpr uint32_t M0 = low3_mask(0), M1 = low3_mask(1), M2 = low3_mask(2);

  float xr[XP][8];
  uint32_t wreg[STEPS][3][CPL];
  load_round(0, xr, wreg);
  if (!MULTI) __builtin_amdgcn_sched_barrier(0);
  for (int r = 0; r < rounds; ++r) {
    float xr_next[XP][8];
    uint32_t wreg_next[STEPS][3][CPL];
    if (MULTI && r + 1 < rounds) load_round(r + 1, xr_next, wreg_next);  // in flight during this round

    // ---- stage this wave's activation digits (wave-local) ---------------------------------
    float amax = 0.f, asum = 0.f;
#pragma unroll
    for (int p = 0; p < XP; ++p) {
      const int s = 4 * p + xs;
      const bool live = s < STEPS && (r * STEPS + s) * (WAVES * 4) + wv * 4 + xkb < g_count;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if (!live) xr[p][j] = 0.f;
        amax = fmaxf(amax, fabsf(xr[p][j]));
        asum += xr[p][j];
      }
    }
    const float xmax = wave_max(amax);
    asum_total += wave_sum(asum);
    // 2^E * max|x| lies in [2^29, 2^30): v = rint(x * 2^E) + 0x88888888 never wraps, and its
    // nibbles n_d satisfy v = sum_d 16^d (n_d - 8).
    int E = 29 - ((int)((__float_as_uint(xmax) >> 23) & 255u) - 127);
    E = xmax > 0.f ? max(-120, min(120, E)) : 0;
    const float scaleE = pow2f(E);
#pragma unroll
    for (int p = 0; p < XP; ++p) {
      uint32_t ev[8], od[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const uint32_t t = (uint32_t)(int)rintf(xr[p][j] * scaleE) + 0x88888888u;
        ev[j] = t & 0x0f0f0f0fu;         // nibbles 0 2 4 6
        od[j] = (t >> 4) & 0x0f0f0f0fu;  // nibbles 1 3 5 7
      }
      // A operand (fp6): lane quarter g holds K indices 32g .. 32g+31 of the MFMA, element k of the
      // group at k/2 (even k) or 16 + k/2 (odd k).  B operand (fp8): lane quarter kb holds K indices
      // 16kb .. 16kb+15 in its first four registers and 64+16kb .. 64+16kb+15 in the last four.
      uint32_t de[2][4], dd[2][4];
      transpose4(ev[0], ev[2], ev[4], ev[6], de[0]);
      transpose4(ev[1], ev[3], ev[5], ev[7], de[1]);
      transpose4(od[0], od[2], od[4], od[6], dd[0]);
      transpose4(od[1], od[3], od[5], od[7], dd[1]);
      const int s = 4 * p + xs;
      if (s < STEPS) {
        // k-group xkb fills half xkb >> 1 of the quarters 2 * (xkb & 1) (even elements) and + 1 (odd elements)
        char* dst = dig_w + step_off(s) + dig_piece(0, 2 * (xkb & 1), xkb >> 1) + xq * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int h = 0; h < 2; ++h) {  // h = 0: even elements, h = 1: odd elements (next lane quarter)
            *reinterpret_cast<uint32_t*>(dst + dig_piece(2 * i, h, 0)) = de[h][i];
            *reinterpret_cast<uint32_t*>(dst + dig_piece(2 * i + 1, h, 0)) = dd[h][i];
          }
      }
    }
    // The digits are read back by other lanes of this wave only: order the LDS writes
    // before the reads without a workgroup barrier.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");

    // ---- mask + MFMA -----------------------------------------------------------------------
    f4 acc[CPL];
#pragma unroll
    for (int q = 0; q < CPL; ++q) acc[q] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      if (!MULTI && s + kEarly < STEPS) {
        load_steps(0, wreg, s + kEarly, s + kEarly + 1);
        __builtin_amdgcn_sched_barrier(0);  // issued here, not where the compiler would like it
      }
      if (ROUNDS == 2 && s + kNextEarly < STEPS && r + 1 < rounds) {
        load_steps(r + 1, wreg_next, s + kNextEarly, s + kNextEarly + 1);
        __builtin_amdgcn_sched_barrier(0);
      }
      if ((r * STEPS + s) * (WAVES * 4) + wv * 4 >= g_count) continue;  // wave-uniform
      // MFMA columns 9..15 are never read: they re-use row 8
      const char* bp = dig_w + step_off(s) + dig_piece(c < 8 ? c : 8 + (kb & 1), kb, 0);
      const u4v b0 = *reinterpret_cast<const u4v*>(bp), b1 = *reinterpret_cast<const u4v*>(bp + dig_piece(0, 0, 1));
      const v8i B = {(int)b0.x, (int)b0.y, (int)b0.z, (int)b0.w, (int)b1.x, (int)b1.y, (int)b1.z, (int)b1.w};
#pragma unroll
      for (int q = 0; q < CPL; ++q) {
        const uint32_t w0 = wreg[s][0][q], w1 = wreg[s][1][q], w2 = wreg[s][2][q];
        const v8i A = {(int)(w0 & M0), (int)(w1 & M1), (int)(w2 & M2),
                       (int)(__builtin_amdgcn_alignbit(w1, w0, 3) & M0),
                       (int)(__builtin_amdgcn_alignbit(w2, w1, 3) & M1), (int)((w2 >> 3) & M2), 0, 0};
        // A: fp6 e2m3 (cbsz 2), B: fp8 e4m3 (blgp 0), unit block scales
        acc[q] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A, B, acc[q], 2, 0, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
      }
    }
    // acc = 2^-12 * sum q*n_d (column d < 8), 2^-12 * sum q (column 8): take the bias out
    // while everything is still an exact integer, then leave the round's fixed-point scale.
    const float descale = pow2f(-E);
#pragma unroll
    for (int q = 0; q < CPL; ++q)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float unbiased = fmaf(row_bcast8(acc[q][i]), -8.f, acc[q][i]);
        run[q][i] = fmaf(unbiased, descale, run[q][i]);
      }
    // the LDS digits of this round must be consumed before the next round overwrites them
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    if (MULTI && r + 1 < rounds) {
#pragma unroll
      for (int p = 0; p < XP; ++p)
#pragma unroll
        for (int j = 0; j < 8; ++j) xr[p][j] = xr_next[p][j];
#pragma unroll
      for (int s = 0; s < STEPS; ++s)
#pragma unroll
        for (int j = 0; j < 3; ++j)
#pragma unroll
          for (int q = 0; q < CPL; ++q) wreg[s][j][q] = wreg_next[s][j][q];
    }
  }

  // ---- combine digits, waves, scale/zero --------------------------------------------------
  // D[row = 4*kb + i][col = c]: row is the weight column CPL*row + q of the tile, col the digit.
  if (c < 8) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float* dst = red + (wv * 8 + c) * kRedStride + CPL * (4 * kb + i);
      if constexpr (CPL == 4) {
        const f4 v = {run[0][i], run[1][i], run[2][i], run[3][i]};
        *reinterpret_cast<f4*>(dst) = v;
      } else {
#pragma unroll
        for (int q = 0; q < CPL; ++q) dst[q] = run[q][i];
      }
    }
  }
  if (lane == 0) wsum[wv] = asum_total;
  // the digit rows written above are read back by this wave only: a wave-local fence, no workgroup barrier
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  {
    const float* rw = red + (wv * 8) * kRedStride + lane;
    float h = rw[7 * kRedStride];
#pragma unroll
    for (int d = 6; d >= 0; --d) h = fmaf(h, 16.f, rw[d * kRedStride]);
    part[wv * 64 + lane] = h;
  }
  __syncthreads();
  float val = 0.f;
  if (tid < TW && n < a.N) {
    float qx = 0.f, xsum = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      qx += part[w * 64 + tid];
      xsum += wsum[w];
    }
    val = sc_n * (qx * 4096.f) - zr_n * xsum;  // 2^12: fp6 unit 2^-3 times fp8 unit 2^-9
    val = fmaf(xsum, 0.f, val);  // a NaN or infinity among the activations makes the result NaN (the
                                 // fixed-point digits cannot carry it)
    if (a.nsplit == 1) {
      // Write-through store: the result is on its way to memory at once instead of waiting in this
      // XCD's L2 for the write-back at the end of the kernel (the last store of a kernel is exposed).
      __hip_atomic_store(&a.y[n], y_old + val, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
      // Device-coherent (write-through) store: visible to the other XCDs' workgroups
      // without flushing or invalidating this XCD's L2.
      __hip_atomic_store(&a.partial[((size_t)tile * a.nsplit + split) * 64 + tid], val, __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  if (a.nsplit > 1) {
    // Arrival counting.  Default protocol, relaxed device-scope atomics only:
    //  (1) the partial sums above are device-scope atomic stores, i.e. write-through stores that are
    //      acknowledged only once they are visible to every XCD;
    //  (2) every wave waits for those acknowledgements (vmcnt 0);
    //  (3) __syncthreads: a workgroup-scope fence plus barrier - the compiler moves no memory access
    //      across it, and after it all of the workgroup's partial sums are visible device-wide;
    //  (4) one device-scope fetch-add per workgroup, performed at the memory side;
    //  (5) the last workgroup to arrive reads every partial with device-scope atomic loads, which
    //      bypass the non-coherent levels, and adds them in split order (deterministic result).
    // What this rests on is the gfx950 cache policy of device-scope atomic accesses (they do not stay
    // in an XCD's L2).  A formal release/acquire pair at device scope writes back and invalidates the
    // whole L2 of the XCD and costs tens of microseconds per call; HQ_FLAG_STRICT_FENCES (set from the
    // HQ_SPLITK_FENCES knob) selects it, for checking that both give the same result.
    __shared__ unsigned s_last;
    const bool strict = (a.flags & HQ_FLAG_STRICT_FENCES) != 0;
    __builtin_amdgcn_s_waitcnt(0);  // (2): a barrier alone does not wait for outstanding stores
    __syncthreads();
    if (tid == 0) {
      const unsigned old = strict ? __hip_atomic_fetch_add(&a.counters[tile], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT)
                                  : __hip_atomic_fetch_add(&a.counters[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      s_last = (old == (unsigned)(a.nsplit - 1));
    }
    __syncthreads();
    if (s_last && strict) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    if (s_last) {
      if (tid < TW && n < a.N) {
        const float sum = hq_sum_partials(&a.partial[(size_t)tile * a.nsplit * 64 + tid], 64, a.nsplit);
        a.y[n] = (a.flags & HQ_FLAG_ACCUMULATE) ? a.y[n] + sum : sum;
      }
      if (tid == 0)  // ready for the next call
        __hip_atomic_store(&a.counters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

template <int WAVES, int STEPS, bool XF16, int ROUNDS, int CPL = 4>
int launch_matvec_t(const Q3Args& a, int ntiles, hipStream_t stream) {
  const size_t smem = (size_t)WAVES * STEPS * kStepBytes + (size_t)WAVES * 8 * kRedStride * 4 + (size_t)WAVES * 64 * 4 +
                      (size_t)WAVES * 4 + 16;
  static const hipError_t attr =
      hipFuncSetAttribute(reinterpret_cast<const void*>(&q3_matvec_kernel<WAVES, STEPS, XF16, ROUNDS, CPL>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
  if (attr != hipSuccess) return (int)attr;
  // narrow tiles: whole groups of eight 64-column tiles (the workgroups beyond N leave at once)
  const int gx = CPL == 4 ? ntiles : ((a.N + 63) / 64 + 7) / 8 * 8 * (4 / CPL);
  hipLaunchKernelGGL((q3_matvec_kernel<WAVES, STEPS, XF16, ROUNDS, CPL>), dim3(gx, a.nsplit), dim3(WAVES * 64), smem,
                     stream, a.w, a.x, a.K, a.N, a.gpw, a.nsplit, a.x_f16, a.flags, a.scales, a.zeros, a.y, a.partial,
                     a.counters);
  return hq_launch_status();
}
template <int WAVES, int STEPS>
int launch_matvec(const Q3Args& a, int ntiles, int cus, int cpl, hipStream_t stream) {
  if constexpr (WAVES == 8 && STEPS == 4) {
    if (cpl == 1)
      return a.x_f16 ? launch_matvec_t<8, 4, true, 0, 1>(a, ntiles, stream) : launch_matvec_t<8, 4, false, 0, 1>(a, ntiles, stream);
    if (cpl == 2)
      return a.x_f16 ? launch_matvec_t<8, 4, true, 0, 2>(a, ntiles, stream) : launch_matvec_t<8, 4, false, 0, 2>(a, ntiles, stream);
  }
  // Several rounds per workgroup: with a workgroup on every compute unit the next round's loads go out a
  // step at a time (K=36864, N=16384 41.0 -> 37.4 us, K=40960, N=8192 25.9 -> 23.6, K=65536, N=4096 22.6 -> 20.7);
  // with compute units to spare a whole round at once keeps more in flight (K=49152, N=12288, 192 tiles: 42.2
  // against 46.9 us).  The default workgroup only: the other shapes are for sweeps.
  const bool multi = a.gpw > WAVES * 4 * STEPS;
  const bool ahead = WAVES == 8 && STEPS == 4 && ntiles * a.nsplit >= cus;
  if (WAVES == 8 && STEPS == 4 && multi && ahead)
    return a.x_f16 ? launch_matvec_t<8, 4, true, 2>(a, ntiles, stream) : launch_matvec_t<8, 4, false, 2>(a, ntiles, stream);
  if (a.x_f16)
    return multi ? launch_matvec_t<WAVES, STEPS, true, 1>(a, ntiles, stream)
                 : launch_matvec_t<WAVES, STEPS, true, 0>(a, ntiles, stream);
  return multi ? launch_matvec_t<WAVES, STEPS, false, 1>(a, ntiles, stream)
               : launch_matvec_t<WAVES, STEPS, false, 0>(a, ntiles, stream);
}

}  // namespace

int hq_q3_gemm_launch(const void* x, const int32_t* qweight, const float* scales, const float* zeros,
                      float* y, int K, int N, int M, unsigned flags, hipStream_t stream, const HqQ3Scratch* fixed);

int hq_q3_block_launch(const void* x, const int32_t* qweight, const float* scales, const float* zeros, float* y,
                       int K, int N, int M, int nsplit, int rpw, int mblocks, float* partial, unsigned* counters,
                       unsigned flags, hipStream_t stream);
int hq_q3_block_groups_per_round(void);
int hq_q3_gemm_need(int cus, int K, int N, size_t* floats, size_t* counters);

namespace {
// Zeroes n words with a kernel (a memset node inside a captured graph is not an option for callers
// that capture the stream).
__global__ __launch_bounds__(256) void fill_zero_kernel(unsigned* p, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0u;
}
}  // namespace

namespace {
// Largest batch the matvec-like kernels take by default, and the most partial-sum rows (tiles x splits x batch)
// the kernel for 2 ... 8 rows may need: what the fixed scratch of the entry point that allocates nothing holds,
// applied to every caller so that both entry points run the same kernel on the same shape.
constexpr size_t kBlockPartialRows = 8192;

// How the kernel for 2 ... 8 rows cuts K: up to eight rounds of 4096 elements, one workgroup per round (as the
// batch-1 kernel); beyond that as many workgroups per column tile as give every compute unit two, each taking
// several rounds one after the other.
void q3_block_split(int cus, int K, int N, int batch_M, int* nsplit, int* rpw) {
  const int gpr = hq_q3_block_groups_per_round();
  const int rounds = (K / 32 + gpr - 1) / gpr;
  const int ntiles = (N + 63) / 64;
  int ns = rounds;
  if (rounds > 8) {
    ns = 2 * cus / ntiles;
    if (ns < 1) ns = 1;
    if (ns > rounds) ns = rounds;
  }
  // no more partial-sum rows than the fixed scratch holds (very wide matrices: fewer, longer ranges of K)
  while (ns > 1 && (size_t)ntiles * ns * batch_M > kBlockPartialRows) --ns;
  *rpw = (rounds + ns - 1) / ns;
  *nsplit = (rounds + *rpw - 1) / *rpw;
}

constexpr int kRowBlockBatchMax = 64;  // rows a batch may have as row blocks of four

// Row blocks (workgroups per column tile, four rows each) of a batch of more than four rows; 1: passes inside
// one workgroup; 0: the four-rows-per-pass kernel does not take this batch at all.
int q3_block_row_blocks(int cus, int K, int N, int batch_M, int nsplit, int rpw) {
  (void)K;
  // Measured (us per call, passes in one workgroup or the GEMM -> row blocks): with a CU for every workgroup,
  // K=4096, N=4096: 5 rows 7.2 -> 5.2, 8 rows 8.4 -> 5.3, 12 rows 11.7 -> 5.3, 16 rows 12.7 -> 5.6; with up to
  // four workgroups per CU, K=4096, N=4096, 32 rows 12.8 -> 8.4; K=4096, N=11008: 8 rows 9.0 -> 8.5, 12 rows
  // 12.3 -> 11.0, 16 rows 14.3 -> 11.4; K=11008, N=4096: 12 rows 15.0 -> 12.8, 16 rows 17.6 -> 13.0; K=4096,
  // N=22016: 7 rows 14.4 -> 11.9, 8 rows 15.2 -> 11.7; K=8192, N=8192: 16 rows 16.5 -> 16.2.  Five and six
  // rows in more workgroups than CUs do not gain (K=4096, N=11008, 5 rows: 7.8 -> 8.4): the second block's one
  // or two rows cost a whole workgroup where a second pass costs two rows of staging.
  const int mode = hq_tune(HQ_TUNE_Q3_ROW_BLOCKS, -1);  // 0: never, 1: wherever possible (tests)
  if (batch_M <= 4) return 1;
  const int mb = (batch_M + 3) / 4;
  const size_t groups = (size_t)((N + 63) / 64) * nsplit;
  const bool possible = mode != 0 && rpw == 1 && nsplit <= 8 && batch_M <= kRowBlockBatchMax &&
                        (nsplit == 1 || groups * mb * 4 <= kBlockPartialRows);
  if (possible) {
    const size_t wgs = groups * mb;
    if (mode == 1 || wgs <= (size_t)cus || (batch_M >= 7 && wgs <= 4 * (size_t)cus)) return mb;
  }
  return batch_M <= 12 ? 1 : 0;
}

int q3_plan(int cus, int K, int N, int batch_M) {
  if (batch_M == 1) return HQ_Q3_PLAN_MATVEC;
  const int limit = hq_tune(HQ_TUNE_Q3_SMALL_BATCH, kRowBlockBatchMax);  // 0: every batch takes the GEMM
  int nsplit, rpw;
  q3_block_split(cus, K, N, batch_M, &nsplit, &rpw);
  if (batch_M > limit) return HQ_Q3_PLAN_GEMM;
  const int mb = q3_block_row_blocks(cus, K, N, batch_M, nsplit, rpw);
  if (mb > 1) return HQ_Q3_PLAN_BLOCK;
  if (mb == 0) return HQ_Q3_PLAN_GEMM;
  // 2 ... 8 rows in one workgroup per tile and K range.  Five to eight rows take
  // two passes per workgroup, which beats the GEMM (7.8-12.4 us against 13-19 us at 4096 x 4096 ... 14336 x
  // 4096, 20.7-24.9 against 24.7 at K=8192, N=22016, 26.5-31.9 against 31.6 at K=28672, N=8192) except where
  // the GEMM's 128-column tiles fill the device without a K split (K=8192, N=28672: 27.8-31.1 against 25.3 us).
  const size_t groups = (size_t)((N + 63) / 64) * nsplit;
  const size_t tiles128 = (size_t)(N + 127) / 128;
  if (batch_M <= 8 && (nsplit == 1 || groups * batch_M <= kBlockPartialRows) &&
      (batch_M <= 4 || (rpw == 1 && 8 * tiles128 < 7 * (size_t)cus)))
    return HQ_Q3_PLAN_BLOCK;
  // 9 ... 12 rows, three passes: where the launch has at most one workgroup per compute unit (it is a matter
  // of latency there, and the GEMM needs three launches)
  if (batch_M <= 12 && rpw == 1 && groups <= (size_t)cus) return HQ_Q3_PLAN_BLOCK;
  return HQ_Q3_PLAN_GEMM;
}

// How the digit kernels divide K: a workgroup covers gpr k-groups per round and walks its K range in rounds
// (the next round's loads are in flight during the current one), or K is split across workgroups whose
// partial sums (rows_out rows of 64 floats per workgroup) the last one to arrive adds up.
// Planning is pure arithmetic (the launch, the workspace reservation and the size query share it);
// q3_split_acquire then takes the scratch, once, when the plan is final.
struct Q3SplitPlan {
  int gpw;          // k-groups per workgroup, whole rounds
  int nsplit;       // workgroups per column tile
  int ntiles;       // column tiles (times row blocks) = arrival counters
  size_t floats;    // partial sums: 0 without a split
  bool too_large;   // the fixed scratch cannot hold this plan
};
struct Q3Limits {  // what a fixed scratch holds; null pointer = the stream's workspace (grows on demand)
  size_t partial_floats, ncounters;
};
Q3SplitPlan q3_split_plan(int cus, int G, int gpr, int ntiles, int rows_out, bool single_round, const Q3Limits* fixed) {
  const int max_split = (G + gpr - 1) / gpr;
  const size_t tile_floats = (size_t)ntiles * rows_out * 64;
  int nsplit = single_round ? max_split : hq_tune(HQ_TUNE_Q3_KSPLIT, 0);
  if (nsplit <= 0) {
    // One workgroup per round of K.  Single-round workgroups need half the registers, so two share a CU and
    // one's reduction tail runs under the other's loads, and the workgroups spread evenly over the CUs
    // whatever the tile count (batch 1 at K=8192: N=22016, 344 tiles, 20.4 -> 15.1 us; N=28672, 448 tiles,
    // 21.4 -> 18.6 us; K=28672, N=8192 21.7 -> 19.6 us).  A plain grid of short workgroups also streams faster
    // than workgroups that walk K (K=49152, N=12288, 192 tiles: 40.2 against 43.0 us; K=40960, N=22016,
    // 344 tiles: 57.4 against 70.7; K=36864, N=20480: 49.3 against 62.6), except beyond eight rounds where the
    // unsplit workgroups would fill the CUs evenly anyway and the exchange is all a split adds (K=36864,
    // N=16384, 256 tiles: 37.8 unsplit, 39.4 split).
    const int per_cu = (ntiles + cus - 1) / cus;
    const bool even = (size_t)ntiles * 20 >= (size_t)per_cu * cus * 19;
    nsplit = (max_split <= 8 || !even) ? max_split : 1;
    if (fixed && nsplit > 1 && (tile_floats * nsplit > fixed->partial_floats || (size_t)ntiles > fixed->ncounters))
      nsplit = cus / ntiles;  // the fixed scratch is too small for the full split
  }
  if (nsplit > max_split) nsplit = max_split;
  if (nsplit < 1) nsplit = 1;
  Q3SplitPlan p;
  p.gpw = (G + nsplit - 1) / nsplit;
  p.gpw = (p.gpw + gpr - 1) / gpr * gpr;  // whole rounds
  p.nsplit = (G + p.gpw - 1) / p.gpw;
  p.ntiles = ntiles;
  p.floats = p.nsplit > 1 ? tile_floats * p.nsplit : 0;
  p.too_large = p.nsplit > 1 && fixed && (p.floats > fixed->partial_floats || (size_t)ntiles > fixed->ncounters);
  return p;
}

struct Q3Split {
  float* partial;
  unsigned* counters;
};
int q3_split_acquire(const Q3SplitPlan& p, const HqQ3Scratch* fixed, hipStream_t stream, Q3Split* out) {
  out->partial = nullptr;
  out->counters = nullptr;
  if (p.nsplit <= 1) return HQ_OK;
  if (fixed) {
    // fixed scratch shared by every call on this device: the counters start from zero by a fill kernel
    // on the same stream (they also reset themselves, but an earlier call may have been cut short)
    if (p.too_large) return HQ_ERR_TOO_LARGE;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((p.ntiles + 255) / 256), dim3(256), 0, stream, fixed->counters, p.ntiles);
    const int rc = hq_launch_status();
    if (rc != HQ_OK) return rc;
    out->partial = fixed->partial;
    out->counters = fixed->counters;
    return HQ_OK;
  }
  HqWorkspace ws;
  const int rc = hq_get_workspace(stream, p.floats, (size_t)p.ntiles, &ws);
  if (rc != HQ_OK) return rc;
  out->partial = ws.partial;
  out->counters = ws.counters;
  return HQ_OK;
}

// Launch shape of the batch-1 kernel (pure arithmetic).
struct Q3MatvecPlan {
  int waves, steps, cpl, ntiles;
  Q3SplitPlan split;
};
Q3MatvecPlan q3_matvec_shape(int cus, int K, int N, const Q3Limits* fixed) {
  const int G = K / 32;
  Q3MatvecPlan m;
  m.ntiles = (N + 63) / 64;
  // A workgroup of WAVES waves covers WAVES*4*STEPS k-groups per round and walks its K range in rounds
  // (the next round's loads are in flight during the current one), or K is split across workgroups whose
  // partial sums the last one to arrive adds up.
  m.waves = hq_tune(HQ_TUNE_Q3_WAVES, 8);
  m.steps = hq_tune(HQ_TUNE_Q3_STEPS, 0);
  if (m.waves != 4 && m.waves != 8 && m.waves != 16) m.waves = 8;
  if (m.waves == 16) m.steps = 1;  // register budget of 16-wave workgroups
  if (m.steps != 1 && m.steps != 2 && m.steps != 4 && (m.steps != 8 || m.waves != 4)) {
    m.steps = 4;
    while (m.steps > 1 && m.waves * 4 * (m.steps / 2) >= G) m.steps /= 2;  // short K: fewer steps
  }
  const int gpr = m.waves * 4 * m.steps;  // k-groups one workgroup covers per round
  // Few column tiles (the default workgroup, one round of K per workgroup): narrower tiles, 32 or 16 columns,
  // as long as every workgroup still has a CU of its own - the idle CUs' load queues join in.
  // HQ_Q3_TILE: 4, 2 or 1 columns per lane, unset: by the launch size.
  m.cpl = 4;
  {
    const int rounds = (G + gpr - 1) / gpr;
    const int want = hq_tune(HQ_TUNE_Q3_TILE, -1);
    if (m.waves == 8 && m.steps == 4 && rounds <= 8 && hq_tune(HQ_TUNE_Q3_KSPLIT, -1) < 0) {
      if (want == 1 || want == 2) m.cpl = want;
      else if (want < 0) m.cpl = 4 * m.ntiles * rounds <= cus ? 1 : (2 * m.ntiles * rounds <= cus ? 2 : 4);
    }
    if (m.cpl < 4) m.ntiles = (N + 16 * m.cpl - 1) / (16 * m.cpl);
  }
  m.split = q3_split_plan(cus, G, gpr, m.ntiles, 1, false, fixed);
  if (m.cpl < 4 && (m.split.gpw > gpr || m.split.too_large)) {  // narrow tiles are for single-round workgroups only
    m.cpl = 4;
    m.ntiles = (N + 63) / 64;
    m.split = q3_split_plan(cus, G, gpr, m.ntiles, 1, false, fixed);
  }
  return m;
}

// Split of the kernel for batches 2 ... 64 (pure arithmetic): row blocks or passes.
struct Q3BlockPlan {
  int nsplit, rpw, mblocks;
  Q3SplitPlan split;
};
Q3BlockPlan q3_block_shape(int cus, int K, int N, int batch_M, const Q3Limits* fixed) {
  Q3BlockPlan b;
  q3_block_split(cus, K, N, batch_M, &b.nsplit, &b.rpw);
  b.mblocks = q3_block_row_blocks(cus, K, N, batch_M, b.nsplit, b.rpw);
  if (b.mblocks < 1) b.mblocks = 1;
  if (b.mblocks > 1)
    b.split = q3_split_plan(cus, K / 32, hq_q3_block_groups_per_round(), (N + 63) / 64 * b.mblocks, 4, true, fixed);
  else
    b.split = q3_split_plan(cus, K / 32, b.rpw * hq_q3_block_groups_per_round(), (N + 63) / 64, batch_M, true, fixed);
  return b;
}
}  // namespace

extern "C" int hq_q3_matvec_plan(int K, int N, int batch_M) {
  if (K <= 0 || N <= 0 || batch_M <= 0 || (K & 31) || (N & 3)) return HQ_ERR_BAD_SHAPE;
  const HqDevice* dev = nullptr;
  const int rc = hq_current_device(&dev);
  return rc != HQ_OK ? rc : q3_plan(dev->cus, K, N, batch_M);
}

// Workspace one hq_q3_matvec call takes from its stream on a device of `cus` compute units: the same plan
// functions as the launch (host arithmetic only, no device is touched).
int hq_q3_workspace_need_impl(int cus, int K, int N, int batch_M, size_t* floats, size_t* counters) {
  if (K <= 0 || N <= 0 || batch_M <= 0 || (K & 31) || (N & 3) || cus <= 0) return HQ_ERR_BAD_SHAPE;
  *floats = 0;
  *counters = 0;
  if (batch_M == 1) {
    const Q3MatvecPlan m = q3_matvec_shape(cus, K, N, nullptr);
    *floats = m.split.floats;
    *counters = m.split.nsplit > 1 ? (size_t)m.split.ntiles : 0;
    return HQ_OK;
  }
  if (q3_plan(cus, K, N, batch_M) == HQ_Q3_PLAN_BLOCK) {
    const Q3BlockPlan b = q3_block_shape(cus, K, N, batch_M, nullptr);
    *floats = b.split.floats;
    *counters = b.split.nsplit > 1 ? (size_t)b.split.ntiles : 0;
    return HQ_OK;
  }
  return hq_q3_gemm_need(cus, K, N, floats, counters);
}

extern "C" int hq_q3_workspace_need(int compute_units, int K, int N, int batch_M, int64_t* floats, int64_t* counters) {
  if (!floats || !counters) return HQ_ERR_NULL_POINTER;
  size_t f = 0, c = 0;
  const int rc = hq_q3_workspace_need_impl(compute_units, K, N, batch_M, &f, &c);
  *floats = (int64_t)f;
  *counters = (int64_t)c;
  return rc;
}

extern "C" int hq_q3_matvec(const void* x, int x_dtype, const int32_t* qweight, const float* scales,
                            const float* zeros, float* y, int K, int N, int batch_M, unsigned flags,
                            void* stream) {
  return hq_q3_matvec_impl(x, x_dtype, qweight, scales, zeros, y, K, N, batch_M, flags, (hipStream_t)stream, nullptr);
}

int hq_q3_matvec_impl(const void* x, int x_dtype, const int32_t* qweight, const float* scales, const float* zeros,
                      float* y, int K, int N, int batch_M, unsigned flags, hipStream_t stream,
                      const HqQ3Scratch* fixed) {
  if (!x || !qweight || !scales || !zeros || !y) return HQ_ERR_NULL_POINTER;
  if (x_dtype != HQ_DTYPE_F32 && x_dtype != HQ_DTYPE_F16) return HQ_ERR_BAD_ENUM;
  if (flags & ~HQ_FLAG_ACCUMULATE) return HQ_ERR_BAD_ENUM;
  if (hq_tune(HQ_TUNE_SPLITK_FENCES, 0)) flags |= HQ_FLAG_STRICT_FENCES;
  if (K <= 0 || N <= 0 || batch_M <= 0 || (K & 31) || (N & 3)) return HQ_ERR_BAD_SHAPE;
  if (((uintptr_t)qweight & 15) || ((uintptr_t)x & 15) ||  // activations are read with 128-bit loads
      ((uintptr_t)y & 3) || ((uintptr_t)scales & 3) || ((uintptr_t)zeros & 3))
    return HQ_ERR_MISALIGNED;
  // batches share one alignment contract whichever kernel the plan picks: the GEMM reads scale / zero and
  // writes y four columns at a time
  if (batch_M > 1 && (((uintptr_t)scales & 15) || ((uintptr_t)zeros & 15) || ((uintptr_t)y & 15))) return HQ_ERR_MISALIGNED;
  const HqDevice* dev = nullptr;
  int rc = hq_current_device(&dev);
  if (rc != HQ_OK) return rc;
  Q3Limits lim_s, *lim = nullptr;
  if (fixed) {
    lim_s.partial_floats = fixed->partial_floats;
    lim_s.ncounters = fixed->ncounters;
    lim = &lim_s;
  }
  Q3Split sp;
  if (batch_M > 1) {
    if (x_dtype != HQ_DTYPE_F16) return HQ_ERR_BAD_ENUM;
    // Small batches ride on the matvec's digit kernels (one pass over the weights, one launch); everything
    // else takes the batched GEMM.
    if (q3_plan(dev->cus, K, N, batch_M) == HQ_Q3_PLAN_BLOCK) {
      const Q3BlockPlan b = q3_block_shape(dev->cus, K, N, batch_M, lim);
      if (b.split.nsplit != b.nsplit) return HQ_ERR_BAD_SHAPE;
      rc = q3_split_acquire(b.split, fixed, stream, &sp);
      if (rc != HQ_OK) return rc;
      return hq_q3_block_launch(x, qweight, scales, zeros, y, K, N, batch_M, b.nsplit, b.rpw, b.mblocks, sp.partial,
                                sp.counters, flags, stream);
    }
    return hq_q3_gemm_launch(x, qweight, scales, zeros, y, K, N, batch_M, flags, stream, fixed);
  }

  const Q3MatvecPlan m = q3_matvec_shape(dev->cus, K, N, lim);
  rc = q3_split_acquire(m.split, fixed, stream, &sp);
  if (rc != HQ_OK) return rc;
  const int waves = m.waves, steps = m.steps, cpl = m.cpl, ntiles = m.ntiles;

  Q3Args a;
  a.x = x; a.w = reinterpret_cast<const uint32_t*>(qweight); a.scales = scales; a.zeros = zeros;
  a.y = y; a.partial = sp.partial; a.counters = sp.counters; a.K = K; a.N = N; a.gpw = m.split.gpw;
  a.nsplit = m.split.nsplit; a.x_f16 = (x_dtype == HQ_DTYPE_F16); a.flags = flags;
#define HQ_Q3_CASE(W, S) \
  if (waves == W && steps == S) return launch_matvec<W, S>(a, ntiles, dev->cus, cpl, stream);
  HQ_Q3_CASE(16, 1)
  HQ_Q3_CASE(8, 1) HQ_Q3_CASE(8, 2) HQ_Q3_CASE(8, 4)
  HQ_Q3_CASE(4, 1) HQ_Q3_CASE(4, 2) HQ_Q3_CASE(4, 4) HQ_Q3_CASE(4, 8)
#undef HQ_Q3_CASE
  return HQ_ERR_BAD_ENUM;
}
