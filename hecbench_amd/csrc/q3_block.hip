// GPTQ 3-bit product for batches of 2 ... 64 activation rows on the matvec's matrix-core kernel, gfx950: four
// rows per pass over the weights; up to twelve rows as passes of one workgroup, up to 64 as row blocks of four
// rows in workgroups of their own (q3_block_rows_kernel below).
//
// q3.hip (batch 1) carries the activations as fixed point relative to the largest magnitude a wave sees in a
// round, eight 4-bit digits per activation, so one matrix-core pass over the weights serves one row (a
// two-row kernel with seven sign-magnitude digits was the first small-batch kernel; this one took its place
// when it ran a batch of 2 as fast or faster on every shape).  Here every k-group (32 consecutive activations of a row) has its own
// power of two, applied by the matrix core itself: the fp8 operand of v_mfma_scale_f32_16x16x128_f8f6f4 takes
// one E8M0 scale per 32 elements of K and column.  And a digit is not a nibble but a small fp8 (e4m3) number:
// with v = the activation times the power of two that puts the k-group's largest magnitude into [1/8, 1/4),
//   b1 = fp8(v), b2 = fp8(16 (v - b1)), b3 = fp8(16 (16 (v - b1) - b2)), b4 likewise,
// every term takes the next four significant bits of what is left, but never below the fp8 format's
// subnormal step 2^-9: in units of that step the terms are integers up to 127 with four significant bits.
// (All of it in packed fp16, two activations per instruction: v_cvt_scalef32_pk_fp8_f16 divides by the scale
// 2^-E / 16^t while it converts, v_cvt_scalef32_pk_f16_fp8 multiplies by it on the way back, and what is left of
// an fp16 number after its rounded leading part is an fp16 number again, exactly.)
// Products with the 3-bit codes and their sums over the 128 elements of an MFMA stay below 2^17 in those
// units, so the matrix core adds them exactly, as it does the nibbles of q3.hip.  Four terms reach 19 bits
// below the k-group's largest magnitude (an fp16 activation within 2^8 of it enters exactly, one 2^12 below
// it keeps seven bits); the 16^-t of term t rides on the same E8M0 scale, so a row's result is the plain sum
// of its four columns and the sixteen operand columns carry FOUR rows.  (Three terms that follow the
// activation's own exponent all the way - exact fp16 in fifteen columns for five rows - were built as well:
// the matrix core does not add products that far apart exactly, 5e-5 of the output RMS was lost.)
// Five to eight rows take two passes over the weights held in registers: terms of four rows staged in LDS,
// sixteen MFMAs per wave, the pass's sums folded into four registers, next four rows; nine to twelve rows
// take three passes where the launch is small (see q3_block_kernel_many below).
// Everything else follows q3.hip: a workgroup owns a 64-column tile and one round of K (8 waves x 4 steps x
// 4 k-groups = 4096 elements), a wave's 16-lane quarter streams one k-group per step as three 128-bit loads,
// every wave stages its own operand behind a wave-local fence, the waves meet once at the end, and K beyond
// one round is split across workgroups whose partial sums the last one to arrive adds up in split order.
// The weights are read once for all rows at nine VALU instructions per 32 weights and pass, in one launch,
// where the batched GEMM (q3_gemm.hip) needs a pre-pass, twenty per 32 weights, and a third launch when it
// splits K.  No counterpart in the reference (its kernels are batch 1: src/quant3MatMul-hip/kernels.h:12-217).
#include "hq_internal.h"

namespace {

typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4v __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef _Float16 h2v __attribute__((ext_vector_type(2)));
typedef short s2v __attribute__((ext_vector_type(2)));
__device__ __forceinline__ h2v as_h2(uint32_t v) { return __builtin_bit_cast(h2v, v); }

struct BlockArgs {
  const _Float16* x;  // [M][K]
  const uint32_t* w;
  const float* scales;
  const float* zeros;
  float* y;           // [M][N]
  float* partial;     // [tile][split][M][64] when K is split
  unsigned* counters; // [tile] arrival counters, zero between calls
  int K, N, M;
  int nsplit;         // workgroups per column tile
  int rpw;            // rounds of K per workgroup
  unsigned flags;
  int prow;            // rows of partial sums a (virtual) column tile has per split
};

template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float quad_max(float v) {
  v = fmaxf(v, dpp_f<0xB1>(v));  // quad_perm [1,0,3,2]
  return fmaxf(v, dpp_f<0x4E>(v));  // quad_perm [2,3,0,1]
}
__device__ __forceinline__ float quad_sum(float v) {
  v += dpp_f<0xB1>(v);
  return v + dpp_f<0x4E>(v);
}

constexpr uint32_t low3_mask(int word) {
  uint32_t m = 0;
  for (int b = 0; b < 32; ++b)
    if ((32 * word + b) % 6 < 3) m |= 1u << b;
  return m;
}

constexpr int kWaves = 8, kSteps = 4;
constexpr int kGroupsPerRound = kWaves * 4 * kSteps;  // k-groups of one workgroup
constexpr int kTerms = 4;                     // fp8 terms per activation
constexpr int kPassRows = 4;                  // rows of activations per pass: sixteen operand columns
// LDS layout of a step's sixteen operand rows (the bank rules are those measured for q3.hip: a 128-bit read is
// served in passes of 16 lanes - rows 0-3 and 12-15 of one lane quarter with rows 4-11 of its neighbour - over
// 256 bytes of banks, a 32-bit store in passes of 32 lanes over 128 bytes): a (quarter, half) block holds its
// sixteen rows as consecutive 16-byte pieces, i.e. one whole bank period; neighbouring quarters lie 256 bytes
// apart, quarter pairs 512, the second halves 1040 bytes behind the first, steps 2080 bytes apart, and the
// lanes of a store pass share a quarter parity.  No read and no store meets another in a bank.
constexpr int kStepBytes = 2080;
__device__ __forceinline__ constexpr int dig_piece(int row, int quarter, int half) {
  return 16 * row + 256 * (quarter & 1) + 512 * (quarter >> 1) + 1040 * half;
}
constexpr int kScaleOff = kSteps * kStepBytes;  // behind the last step
constexpr int kWaveBytes = (kScaleOff + 64 + 127) / 128 * 128;  // + scales[4 rows][4 quarters][4 steps], one byte each
constexpr int kMaxRows = 3 * kPassRows;
constexpr int kWsumStride = 16;
__device__ __forceinline__ constexpr int step_off(int s) { return s * kStepBytes; }

// PASSES = ceil(M / 4).  A pass leaves four registers per lane (its sixteen sums spread over the four lanes
// of a row's columns); a wave's final sums re-use its operand area.  Two workgroups share a compute unit
// (at most 128 registers, 76 KB of LDS): one's staging and reduction run under the other's loads.
// MULTI: the workgroup takes several rounds of K (K beyond eight rounds; one pass only).
// (Staging both passes' operands, in areas of their own, before the first MFMA - possible where a launch has
// at most one workgroup per compute unit - changes nothing: a pass costs its ~450 VALU instructions per wave
// wherever they stand.)
template <int PASSES, bool MULTI>
__device__ __forceinline__ void q3_block_body(const BlockArgs& a, const int tile, const int vtile) {
  // LDS: dig[kWaves][kAreaBytes] | wsum[kWaves][kWsumStride]
  extern __shared__ uint4 smem[];
  constexpr int kAreaBytes = kWaveBytes;
  char* dig = reinterpret_cast<char*>(smem);
  float* wsum = reinterpret_cast<float*>(dig + kWaves * kAreaBytes);
  static_assert(kSteps * kStepBytes >= kMaxRows * 64 * 4, "a wave's digit area must hold its final sums");

  const int tid = threadIdx.x, lane = tid & 63;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 15, kb = lane >> 4;
  const int split = blockIdx.y;
  const int g_begin = split * a.rpw * kGroupsPerRound;
  const int g_count = min(a.rpw * kGroupsPerRound, (a.K >> 5) - g_begin);  // k-groups of this workgroup
  const int M = a.M;

  // staging role: lane converts the eight consecutive activations 8*xq .. 8*xq+7 of k-group xkb of step xs
  // (lane bit 5, which selects the pass of a 32-bit LDS store, is the k-group's parity)
  const int xs = (lane >> 3) & 3, xkb = ((lane >> 2) & 1) * 2 + (lane >> 5), xq = lane & 3;
  const int tile_cols = min(64, a.N - tile * 64);  // multiple of 4
  const uint32_t col_off = (uint32_t)min(4 * c, tile_cols - 4) * 4u;
  const uint32_t row_bytes = (uint32_t)a.N * 4u;
  char* dig_w0 = dig + wv * kAreaBytes;
  float* red_w = reinterpret_cast<float*>(dig_w0);
  // MFMA column c carries term c % 4 of row c / 4 of the pass
  const int crow = c >> 2, cterm = c & 3;
  f4 keep[PASSES];
  float rowsum[PASSES];  // sum of the activations of row crow of the pass over this wave's k-groups
#pragma unroll
  for (int p = 0; p < PASSES; ++p) {
    keep[p] = f4{0.f, 0.f, 0.f, 0.f};
    rowsum[p] = 0.f;
  }
  // The sums of the activations (for the zero term) come from the matrix core as well: one more MFMA per step
  // with a weight operand of all 1/8 (fp6 000001) adds up every operand column, i.e. every term of every row,
  // with the same scales - the sum of exactly the activations the products see.
  const v8i eighths = {0x41041041, 0x10410410, 0x04104104, 0x41041041, 0x10410410, 0x04104104, 0, 0};
  constexpr uint32_t M0 = low3_mask(0), M1 = low3_mask(1), M2 = low3_mask(2);

  // A workgroup's rounds run one after the other, nothing of the next round in flight during this one: two
  // workgroups share the compute unit and one's loads run under the other's arithmetic.
  for (int g0 = 0; g0 < (MULTI ? g_count : 1); g0 += kGroupsPerRound) {
  const int G = min(kGroupsPerRound, g_count - g0);  // k-groups of this round
  const char* wbase = reinterpret_cast<const char*>(a.w) + (size_t)(g_begin + g0) * 3 * row_bytes + (size_t)tile * 64 * 4;
  const _Float16* xbase = a.x + (size_t)(g_begin + g0) * 32;

  // ---- the loads of the workgroup's round: the activation rows first (L2 hits: a compute unit returns its
  // loads in issue order, so the rows are there, and can be staged, while the weights still stream in from HBM)
  const int xg = xs * (kWaves * 4) + wv * 4 + xkb;  // the k-group this lane stages
  const bool live = xg < G;
  u4v xraw[PASSES][kPassRows];
#pragma unroll
  for (int p = 0; p < PASSES; ++p)
#pragma unroll
    for (int m = 0; m < kPassRows; ++m) {
      const int mg = min(kPassRows * p + m, M - 1);  // rows beyond the batch repeat the last one and are not used
      xraw[p][m] = *reinterpret_cast<const u4v*>(xbase + (size_t)mg * a.K + (uint32_t)min(xg, G - 1) * 32u + (uint32_t)xq * 8u);
    }
  __builtin_amdgcn_sched_barrier(0);  // keeps the compiler from moving activation loads behind weight loads
  uint32_t wreg[kSteps][3][4];
  auto load_step = [&](int s) {
    const uint32_t g = (uint32_t)min(s * (kWaves * 4) + wv * 4 + kb, G - 1);
#pragma unroll
    for (int j = 0; j < 3; ++j) {
      const size_t off = (size_t)(g * 3u + (uint32_t)j) * row_bytes + col_off;
      const u4v v = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(wbase + off));
      wreg[s][j][0] = v.x; wreg[s][j][1] = v.y; wreg[s][j][2] = v.z; wreg[s][j][3] = v.w;
    }
  };
  // The weight loads of one step go out at once, the other steps' between the rows of the first pass's staging:
  // a wave stalls at a load while the compute unit's queue of outstanding loads is full, and a stalled wave
  // stages nothing; nor do the later waves' activations, queued behind all twelve weight loads of the earlier
  // waves, come back soon.  K=4096, N=11008, batch 4: all steps up front 7.1 us, two 6.7, one 6.2, none 6.5
  // (and 8.0 us where the compiler was free to move the activation loads behind the weight loads).
  constexpr int kEarly = 1;
#pragma unroll
  for (int s = 0; s < kEarly; ++s) load_step(s);
  __builtin_amdgcn_sched_barrier(0);

  // ---- stage the fp8 terms and scales of rows 4p .. 4p+3 ---------------------------------------------
  auto stage = [&](int p) {
    char* dig_w = dig_w0;
    unsigned char* sc_tab = reinterpret_cast<unsigned char*>(dig_w + kScaleOff);
#pragma unroll
    for (int m = 0; m < kPassRows; ++m) {
      if (p == 0 && m > 0) {
        constexpr int per = (kSteps - kEarly + 2) / 3;  // the remaining steps' loads go between the rows of the first pass
#pragma unroll
        for (int s = kEarly + (m - 1) * per; s < kEarly + m * per && s < kSteps; ++s) load_step(s);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (kPassRows * p + m >= M) continue;  // uniform; the operand columns of a missing row feed result columns nobody reads
      // The lane's eight activations stay fp16, in pairs (0, 2), (4, 6), (1, 3), (5, 7): even / odd elements of the
      // k-group go to neighbouring lane quarters of the fp8 operand (see q3.hip), and the conversions below take
      // and give pairs.
      const u4v raw = xraw[p][m];
      const uint32_t w0 = live ? raw.x : 0u, w1 = live ? raw.y : 0u, w2 = live ? raw.z : 0u, w3 = live ? raw.w : 0u;
      h2v pr[4] = {as_h2(__builtin_amdgcn_perm(w1, w0, 0x05040100u)), as_h2(__builtin_amdgcn_perm(w3, w2, 0x05040100u)),
                   as_h2(__builtin_amdgcn_perm(w1, w0, 0x07060302u)), as_h2(__builtin_amdgcn_perm(w3, w2, 0x07060302u))};
      h2v mx = {(_Float16)0.f, (_Float16)0.f};
#pragma unroll
      for (int i = 0; i < 4; ++i) mx = __builtin_elementwise_max(mx, __builtin_elementwise_abs(pr[i]));
      const float amax = fmaxf((float)mx[0], (float)mx[1]);
      const float gmax = quad_max(amax);  // the k-group's largest magnitude (its four lanes)
      // 2^E * max|x| lies in [2^-3, 2^-2): 64 ... 127 subnormal steps of the fp8 format.  fp16 magnitudes: E in -18 ... 21.
      int E = -3 - ((int)((__float_as_uint(gmax) >> 23) & 255u) - 127);
      E = gmax > 0.f ? max(-18, min(21, E)) : 0;
      // k-group xkb fills half xkb >> 1 of the quarters 2 * (xkb & 1) (even elements) and + 1 (odd elements)
      char* dst = dig_w + step_off(xs) + dig_piece(kTerms * m, 2 * (xkb & 1), xkb >> 1) + xq * 4;
      // Term t is fp8(what is left * 2^E * 16^t): the conversion divides by the scale 2^-E / 16^t itself, and the
      // conversion back multiplies by it, so what is left, x - b1 - b2 - ..., stays an fp16 number in the
      // activation's own units (exactly: every term is the rounded leading part of it).
      uint32_t sbits = (uint32_t)(127 - E) << 23;
#pragma unroll
      for (int t = 0; t < kTerms; ++t) {
        const float scale = __uint_as_float(sbits);
        s2v be = {0, 0}, bo = {0, 0};
        be = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(be, pr[0], scale, false);
        be = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(be, pr[1], scale, true);
        bo = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(bo, pr[2], scale, false);
        bo = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(bo, pr[3], scale, true);
        const uint32_t ue = __builtin_bit_cast(uint32_t, be), uo = __builtin_bit_cast(uint32_t, bo);
        *reinterpret_cast<uint32_t*>(dst + dig_piece(t, 0, 0)) = ue;
        *reinterpret_cast<uint32_t*>(dst + dig_piece(t, 1, 0)) = uo;
        if (t + 1 < kTerms) {
          pr[0] -= __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(ue, scale, false);
          pr[1] -= __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(ue, scale, true);
          pr[2] -= __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(uo, scale, false);
          pr[3] -= __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(uo, scale, true);
          sbits -= 4u << 23;
        }
      }
      // E8M0 scale of term 0: 2^-E for the k-group's power of two, 2^3 for the unit of the fp6 operand (code / 8)
      if (xq == 0) sc_tab[(m * 4 + xkb) * 4 + xs] = (unsigned char)(127 + 3 - E);
    }
  };
  // ---- mask + MFMA -------------------------------------------------------------------------
  auto multiply = [&](int p) {
    char* dig_w = dig_w0;
    unsigned char* sc_tab = reinterpret_cast<unsigned char*>(dig_w + kScaleOff);
    // The matrix-core operand of the weights (six registers per sixteen MFMAs) is rebuilt in every pass: kept
    // across passes it would double the registers the weights take.  The empty statement hides from the compiler
    // that the weights are the same as in the last pass.
    if (p > 0) {
#pragma unroll
      for (int s = 0; s < kSteps; ++s)
#pragma unroll
        for (int j = 0; j < 3; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q) asm volatile("" : "+v"(wreg[s][j][q]));
    }
    // the scales of the column's row for this lane quarter's k-group in the four steps, times 16^-term
    const uint32_t sc4 = *reinterpret_cast<const uint32_t*>(sc_tab + (crow * 4 + kb) * 4) - (uint32_t)cterm * 0x04040404u;
    f4 acc[4], colsum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int q = 0; q < 4; ++q) acc[q] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < kSteps; ++s) {
      if (s * (kWaves * 4) + wv * 4 >= G) continue;  // wave-uniform
      const char* bp = dig_w + step_off(s) + dig_piece(c, kb, 0);
      const u4v b0 = *reinterpret_cast<const u4v*>(bp), b1 = *reinterpret_cast<const u4v*>(bp + dig_piece(0, 0, 1));
      const v8i B = {(int)b0.x, (int)b0.y, (int)b0.z, (int)b0.w, (int)b1.x, (int)b1.y, (int)b1.z, (int)b1.w};
      const int scale_b = (int)(sc4 >> (8 * s));  // byte 0: this step's scale
      colsum = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(eighths, B, colsum, 2, 0, 0, 0x7f7f7f7f, 0, scale_b);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const uint32_t w0 = wreg[s][0][q], w1 = wreg[s][1][q], w2 = wreg[s][2][q];
        const v8i A = {(int)(w0 & M0), (int)(w1 & M1), (int)(w2 & M2),
                       (int)(__builtin_amdgcn_alignbit(w1, w0, 3) & M0),
                       (int)(__builtin_amdgcn_alignbit(w2, w1, 3) & M1), (int)((w2 >> 3) & M2), 0, 0};
        // A: fp6 e2m3 (cbsz 2), unit scale; B: fp8 e4m3 (blgp 0), scale per lane = per column and k-group
        acc[q] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A, B, acc[q], 2, 0, 0, 0x7f7f7f7f, 0, scale_b);
      }
    }
    // D[row = 4*kb + i][col = c]: row is the weight column 4*row + q of the tile; a row of activations is the
    // sum of its four columns (four neighbouring lanes).  Lane c keeps the sums of i = c & 3.
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float v0 = quad_sum(acc[q][0]), v1 = quad_sum(acc[q][1]), v2 = quad_sum(acc[q][2]), v3 = quad_sum(acc[q][3]);
      float v = (c & 2) ? ((c & 1) ? v3 : v2) : ((c & 1) ? v1 : v0);
      asm volatile("" : "+v"(v));  // selected here, not where it is stored (four candidates alive until then)
      keep[p][q] += v;
    }
    rowsum[p] += quad_sum(colsum[0]);  // every result row holds the column sums
  };
#pragma unroll
  for (int p = 0; p < PASSES; ++p) {
    stage(p);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    multiply(p);
    // the next pass rewrites, and the sums below overwrite, the operand and scales this pass's lanes have just read
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
  }
  }  // rounds
#pragma unroll
  for (int p = 0; p < PASSES; ++p) {
    *reinterpret_cast<f4*>(red_w + (kPassRows * p + crow) * 64 + 4 * (4 * kb + cterm)) = keep[p];
    if (kb == 0 && cterm == 0) wsum[wv * kWsumStride + kPassRows * p + crow] = rowsum[p];
  }
  __syncthreads();

  // ---- combine the waves, scale and zero --------------------------------------------------------------
  const int col = tid & 63;
  const int ncol = tile * 64 + col;
  const int nc = min(ncol, a.N - 1);
  const float sc_n = a.scales[nc], zr_n = a.zeros[nc];
  for (int m = tid >> 6; m < M; m += kWaves) {
    float qx = 0.f, xsum = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const float* rw = reinterpret_cast<const float*>(dig + w * kAreaBytes);
      qx += rw[m * 64 + col];
      xsum += wsum[w * kWsumStride + m];
    }
    float val = sc_n * qx - zr_n * xsum;
    val = fmaf(xsum, 0.f, val);  // a NaN or infinity among the activations makes the result NaN
    if (ncol < a.N) {
      if (a.nsplit == 1) {
        float* yp = &a.y[(size_t)m * a.N + ncol];
        const float y_old = (a.flags & HQ_FLAG_ACCUMULATE) ? *yp : 0.f;
        __hip_atomic_store(yp, y_old + val, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      } else {
        __hip_atomic_store(&a.partial[(((size_t)vtile * a.nsplit + split) * a.prow + m) * 64 + col], val, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
      }
    }
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
      const unsigned old = strict ? __hip_atomic_fetch_add(&a.counters[vtile], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT)
                                  : __hip_atomic_fetch_add(&a.counters[vtile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      s_last = (old == (unsigned)(a.nsplit - 1));
    }
    __syncthreads();
    if (s_last && strict) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    if (s_last) {
      if (ncol < a.N) {
        for (int m = tid >> 6; m < M; m += kWaves) {
          const float sum = hq_sum_partials(&a.partial[((size_t)vtile * a.nsplit * a.prow + m) * 64 + col],
                                            (size_t)a.prow * 64, a.nsplit);
          float* yp = &a.y[(size_t)m * a.N + ncol];
          *yp = (a.flags & HQ_FLAG_ACCUMULATE) ? *yp + sum : sum;
        }
      }
      if (tid == 0)  // ready for the next call
        __hip_atomic_store(&a.counters[vtile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

// One and two passes: at most 128 registers, so that two workgroups share a compute unit.
template <int PASSES, bool MULTI>
__global__ __launch_bounds__(kWaves * 64) __attribute__((amdgpu_waves_per_eu(4, 4))) void q3_block_kernel(
                   const uint32_t* w_, const _Float16* x_, int K_, int N_, int M_, int nsplit_, int rpw_, unsigned flags_,
                   const float* scales_, const float* zeros_, float* y_, float* partial_, unsigned* counters_) {
  // leading scalars, not the struct: the first 14 dwords of the arguments arrive preloaded in scalar registers
  BlockArgs a;
  a.x = x_; a.w = w_; a.scales = scales_; a.zeros = zeros_; a.y = y_; a.partial = partial_; a.counters = counters_;
  a.K = K_; a.N = N_; a.M = M_; a.nsplit = nsplit_; a.rpw = rpw_; a.flags = flags_; a.prow = M_;
  q3_block_body<PASSES, MULTI>(a, blockIdx.x, blockIdx.x);
}
// More than four rows as several workgroups per column tile, each with up to four rows of its own (one pass):
// the rows need no exchange, a launch that leaves compute units idle has room for the workgroups, and the
// workgroups of a tile run on one XCD, close in time (workgroup b runs on XCD b mod 8: slot b / 8 of an XCD
// is row block slot % mblocks of tile (slot / mblocks) * 8 + b mod 8), so the tile's weights come out of
// that XCD's L2 for all but the first of them.
__global__ __launch_bounds__(kWaves * 64) __attribute__((amdgpu_waves_per_eu(4, 4))) void q3_block_rows_kernel(
                   const uint32_t* w_, const _Float16* x_, int K_, int N_, int M_, int nsplit_, int mblocks_, unsigned flags_,
                   const float* scales_, const float* zeros_, float* y_, float* partial_, unsigned* counters_) {
  const int slot = blockIdx.x >> 3;
  const int tile = (slot / mblocks_) * 8 + (blockIdx.x & 7), mb = slot % mblocks_;
  if (tile * 64 >= N_) return;  // the last group of eight tiles may be short
  BlockArgs a;
  a.x = x_ + (size_t)mb * kPassRows * K_;
  a.y = y_ + (size_t)mb * kPassRows * N_;
  a.w = w_; a.scales = scales_; a.zeros = zeros_; a.partial = partial_; a.counters = counters_;
  a.K = K_; a.N = N_; a.M = min(kPassRows, M_ - mb * kPassRows); a.nsplit = nsplit_; a.rpw = 1; a.flags = flags_; a.prow = kPassRows;
  q3_block_body<1, false>(a, tile, tile * mblocks_ + mb);
}
// Three passes (9 ... 12 rows) take 127 registers and more time than two workgroups per compute unit leave
// room for; they run where the launch has at most one workgroup per compute unit and is a matter of latency
// (K=4096, N=11008: 11.2-12.7 us against the batched GEMM's 14.7; four passes: 16.1 against 14.9 at 16 rows).
template <int PASSES>
__global__ __launch_bounds__(kWaves * 64) void q3_block_kernel_many(
                   const uint32_t* w_, const _Float16* x_, int K_, int N_, int M_, int nsplit_, int rpw_, unsigned flags_,
                   const float* scales_, const float* zeros_, float* y_, float* partial_, unsigned* counters_) {
  // leading scalars, not the struct: the first 14 dwords of the arguments arrive preloaded in scalar registers
  BlockArgs a;
  a.x = x_; a.w = w_; a.scales = scales_; a.zeros = zeros_; a.y = y_; a.partial = partial_; a.counters = counters_;
  a.K = K_; a.N = N_; a.M = M_; a.nsplit = nsplit_; a.rpw = rpw_; a.flags = flags_; a.prow = M_;
  q3_block_body<PASSES, false>(a, blockIdx.x, blockIdx.x);
}

template <auto KERNEL>
int launch_block(const BlockArgs& a, hipStream_t stream) {
  const size_t smem = (size_t)kWaves * kWaveBytes + (size_t)kWaves * kWsumStride * 4 + 16;
  static const hipError_t attr =
      hipFuncSetAttribute(reinterpret_cast<const void*>(KERNEL), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
  if (attr != hipSuccess) return (int)attr;
  hipLaunchKernelGGL(KERNEL, dim3((a.N + 63) / 64, a.nsplit), dim3(kWaves * 64), smem, stream, a.w, a.x, a.K, a.N, a.M,
                     a.nsplit, a.rpw, a.flags, a.scales, a.zeros, a.y, a.partial, a.counters);
  return hq_launch_status();
}

}  // namespace

// k-groups one workgroup covers (its one round)
int hq_q3_block_groups_per_round(void) { return kGroupsPerRound; }

// 2 ... 12 fp16 activation rows; the caller has validated the arguments, cut K into nsplit ranges of rpw rounds
// of 4096 elements and, for nsplit > 1, provided nsplit * M * 64 floats of partial sums per column tile and
// one zeroed counter per column tile.
int hq_q3_block_launch(const void* x, const int32_t* qweight, const float* scales, const float* zeros, float* y,
                       int K, int N, int M, int nsplit, int rpw, int mblocks, float* partial, unsigned* counters,
                       unsigned flags, hipStream_t stream) {
  const int rounds = (K / 32 + kGroupsPerRound - 1) / kGroupsPerRound;
  if (M < 1 || (M > kMaxRows && mblocks <= 1) || rpw < 1 || nsplit != (rounds + rpw - 1) / rpw) return HQ_ERR_BAD_SHAPE;
  BlockArgs a;
  a.x = reinterpret_cast<const _Float16*>(x);
  a.w = reinterpret_cast<const uint32_t*>(qweight);
  a.scales = scales; a.zeros = zeros; a.y = y; a.partial = partial; a.counters = counters; a.K = K; a.N = N; a.M = M;
  a.nsplit = nsplit; a.rpw = rpw; a.flags = flags & (HQ_FLAG_ACCUMULATE | HQ_FLAG_STRICT_FENCES); a.prow = M;
  if (mblocks > 1) {
    if (rpw != 1 || mblocks != (M + kPassRows - 1) / kPassRows) return HQ_ERR_BAD_SHAPE;
    const size_t smem = (size_t)kWaves * kWaveBytes + (size_t)kWaves * kWsumStride * 4 + 16;
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&q3_block_rows_kernel),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (attr != hipSuccess) return (int)attr;
    const int groups8 = ((N + 63) / 64 + 7) / 8;
    hipLaunchKernelGGL(q3_block_rows_kernel, dim3(groups8 * mblocks * 8, nsplit), dim3(kWaves * 64), smem, stream, a.w, a.x,
                       a.K, a.N, a.M, a.nsplit, mblocks, a.flags, a.scales, a.zeros, a.y, a.partial, a.counters);
    return hq_launch_status();
  }
  if (rpw > 1) return M <= kPassRows ? launch_block<&q3_block_kernel<1, true>>(a, stream) : HQ_ERR_BAD_SHAPE;
  if (M <= kPassRows) return launch_block<&q3_block_kernel<1, false>>(a, stream);
  if (M <= 2 * kPassRows) return launch_block<&q3_block_kernel<2, false>>(a, stream);
  return launch_block<&q3_block_kernel_many<3>>(a, stream);
}
