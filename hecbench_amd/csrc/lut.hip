// LUT-GEMM binary-coded-quantisation matvec for gfx950 (fp16 in / fp16 out).
//
// Replaces matmul() -> nqmv_bias / nqmv -> _nqmv_bias<32> / _nqmv<64>
// (src/lut-gemm-hip/kernels.cu:22-31, mv_fp16.h:28-259 in the HeCBench tree).
//
//   y[n] = sum_k x[k] * ( q_bias[k/G][n] + sum_b alpha[k/G][b][n] * s(k,b,n) )
//
// Shapes with N % 64 == 0 and a group size that is a multiple of 128, 64 or 32 run on the matrix cores
// (bcq_planes_kernel and bcq_mfma_grouped_kernel below: the packed bits themselves are the operands, no
// tables).
// Every other shape runs the table kernel: for every 8-element sub-vector of x the 256
// signed sums sum_j (+-x[j]) are tabulated once per workgroup in LDS (fp32 entries), and
// each byte of a packed bit-plane word becomes one table lookup.  A workgroup owns a tile of columns
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
  int strict;  // formal release/acquire in the split-K arrival (HQ_SPLITK_FENCES)
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
    // Split-K arrival counting with relaxed device-scope atomics only (the protocol and what it rests
    // on are spelled out at the same place in q3.hip): write-through partial stores, wait for their
    // acknowledgement, workgroup fence + barrier, one device-scope fetch-add, and the last workgroup
    // to arrive adds the partials in split order.  a.strict selects formal release/acquire instead.
    unsigned* s_last = reinterpret_cast<unsigned*>(lds + kTables * 256);
    __builtin_amdgcn_s_waitcnt(0);  // the stores above are acknowledged (a barrier alone does not wait for them)
    __syncthreads();
    if (tid == 0) {
      const unsigned old = a.strict ? __hip_atomic_fetch_add(&a.counters[tile], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT)
                                    : __hip_atomic_fetch_add(&a.counters[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      *s_last = (old == (unsigned)(a.nsplit - 1));
    }
    __syncthreads();
    if (*s_last && a.strict) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    if (*s_last) {
      if (tid < 64 * CPL && n < a.N) {
        const float sum = hq_sum_partials(&a.partial[(size_t)tile * a.nsplit * (64 * CPL) + tid], 64 * CPL, a.nsplit);
        a.y[n] = (_Float16)sum;
      }
      if (tid == 0) __hip_atomic_store(&a.counters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}


// ======================================================================================
// Matrix-core paths (group size a multiple of 128: bcq_planes_kernel; 64 or 32: bcq_mfma_grouped_kernel).
//
// sum_k s*x = 2*(sum_k bit*x - (sum_k x)/2).  An fp4 (e2m1) nibble with only its lowest bit set
// is the number 0.5, so `(word >> p) & 0x11111111` (p = 0..3) turns a packed 32-bit word into
// the four operand registers (32 fp4 values) of one 16x16x128 f8f6f4 MFMA: seven VALU
// instructions per 32 weights, no table, no LDS lookup.  The activations of a round are
// scaled to 16-bit fixed point and cut into four nibbles; a nibble 0..15 in an otherwise zero
// byte is the fp8 (e4m3) number nibble * 2^-9, so the digits need no conversion, only a byte
// transpose.  Every product is an integer and the matrix-core sums are exact; alpha is applied to
// the sums in fp32 and everything is rounded to fp16 once.
typedef _Float16 h2v __attribute__((ext_vector_type(2)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4v __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));

// A operand: element 8p + i of a lane quarter is bit 4i + p of its word.
__device__ __forceinline__ v8i unpack_bits_fp4(uint32_t w) {
  const v8i a = {(int)(w & 0x11111111u), (int)((w >> 1) & 0x11111111u), (int)((w >> 2) & 0x11111111u),
                 (int)((w >> 3) & 0x11111111u), 0, 0, 0, 0};
  return a;
}

__device__ __forceinline__ f4 mfma_fp4_fp8(v8i a, v8i b, f4 c) {
  // A fp4 e2m1 (cbsz 4), B fp8 e4m3 (blgp 0), both block scales 2^0 (E8M0 code 127)
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, 4, 0, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
}

template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float lane_f(float v, int l) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), l));
}
// Maximum over the 64 lanes: four DPP butterfly steps per 16-lane row, then the row results.
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

struct Half16 {  // sixteen fp16 values as two 128-bit loads
  h8 lo, hi;
  __device__ __forceinline__ float get(int i) const { return (float)(i < 8 ? lo[i] : hi[i - 8]); }
};
// The same 128-bit loads for rows that start at any element (N not a multiple of 8 or 4): the types carry
// the element's own alignment, the hardware reads unaligned global addresses.
typedef _Float16 h8_any __attribute__((ext_vector_type(8), aligned(2)));
typedef uint32_t u4v_any __attribute__((ext_vector_type(4), aligned(4)));
template <bool RAGGED>
__device__ __forceinline__ Half16 load_half16(const _Float16* p) {
  Half16 h;
  if (RAGGED) {
    h.lo = reinterpret_cast<const h8_any*>(p)[0];
    h.hi = reinterpret_cast<const h8_any*>(p)[1];
  } else {
    h.lo = reinterpret_cast<const h8*>(p)[0];
    h.hi = reinterpret_cast<const h8*>(p)[1];
  }
  return h;
}
template <bool RAGGED>
__device__ __forceinline__ u4v load_words(const uint32_t* p) {
  if (RAGGED) return *reinterpret_cast<const u4v_any*>(p);
  return __builtin_nontemporal_load(reinterpret_cast<const u4v*>(p));
}

// ---- group size a multiple of 128: up to three bit planes per MFMA ---------------------------------
// A matvec has one activation vector, so of the sixteen rows of the activation operand only the four
// digits would be used.  The bit planes fill the rest:
//  - the weights are the SECOND operand: lane quarter kb of MFMA m of a quad (128 elements of K) streams
//    block j = 4m + kb of the quad's 4*P (k-word, plane) blocks, k-word j / P and plane j % P (P <= 3 planes
//    per set; consecutive rows of bW, since the planes of a k-word are adjacent): P MFMAs cover the quad
//    for P planes and 16 columns, four adjacent columns per lane and 128-bit load;
//  - the digits are the FIRST operand: row 4b + d holds digit d at the K positions of the blocks of plane b
//    and zeros elsewhere.  Result row 4b + d, column n is then plane b's sum of digit d for weight column
//    n over the whole quad, accumulated across the P MFMAs inside the matrix core: lane (n, kb) holds the
//    four digits of plane kb in its four result registers, combines them in registers and applies
//    alpha[plane kb][n] ONCE per quad, set and column block.  Lane quarter 3 of the first set carries the
//    q_bias term the same way (its rows are zero; +sum(x)/2 is added to its sum where the others get -sum(x)/2);
//  - the digits are sign-magnitude: |x| in 16-bit fixed point cut into four nibbles, the sign in the fp8
//    sign bit of every digit byte, so no bias has to be taken out and no bit counts are needed;
//  - one more MFMA per quad, all-ones weights against the plain digits, gives sum(x) of the quad.
// Per 128 x 64 x 3-plane quad a lane spends 84 instructions on operands and about 30 on everything else,
// and loads 8 bytes of alpha.  (A kernel with one plane per MFMA - digits as MFMA columns, alpha applied
// per MFMA, 96 bytes of alpha per lane and quad - measured 9.57 us at K=4096, N=16384, 3 planes, this one
// 8.24 us; its loads alone take 6.9 us.)
typedef _Float16 h4v __attribute__((ext_vector_type(4)));
typedef _Float16 h4v_any __attribute__((ext_vector_type(4), aligned(2)));

__device__ __forceinline__ f4 mfma_fp8_fp4(v8i a, v8i b, f4 c) {
  // A fp8 e4m3 (cbsz 0), B fp4 e2m1 (blgp 4), both block scales 2^0
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, 0, 4, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
}

// LDS layout of a quad's digits: 32 operand bytes per (k-word, digit) as two 16-byte pieces, and a piece of
// zeros.  Placed by the bank rules measured on this part (a 128-bit read is served in passes of 16 lanes - lanes
// 0-3, 12-15, 20-27 / 4-11, 16-19, 28-31 of each half wave - over 256 bytes of banks; narrower stores in passes
// of 32 lanes over 128 bytes): k-words 80 bytes apart, digits 16, the second pieces 336 bytes behind the first,
// the zeros at byte 144, quads 704 bytes apart.  Neither an operand read (one, two or three planes per set) nor
// a staging store meets another in a bank (with rows of 32 bytes, 128 bytes per k-word, the stores of the four
// k-words fell into one bank and a quarter of the LDS cycles were conflicts).
constexpr int kDigQuad = 704;
constexpr int kDigZero = 144;
__device__ __forceinline__ constexpr int dig_piece(int kword, int digit, int half) {
  return 80 * kword + 16 * digit + 336 * half;
}
constexpr int planes_of_set(int nb, int s) { return nb - 3 * s < 3 ? nb - 3 * s : 3; }

template <int NB, int QUADS, int WAVES, bool BIAS, bool RAGGED, bool ONE_ROUND>
__global__ __launch_bounds__(WAVES * 64) void bcq_planes_kernel(
    const uint32_t* bW_, const _Float16* x_, const _Float16* alpha_, const _Float16* qbias_, int K_, int N_, int nb_,
    int G_, int kslice_, int nsplit_, int strict_, _Float16* y_, float* partial_, unsigned* counters_) {
  // leading scalars, not the struct: the first 14 dwords of the arguments (all that the loads need) arrive
  // preloaded in scalar registers
  LutArgs a;
  a.bW = bW_; a.alpha = alpha_; a.qbias = qbias_; a.x = x_; a.y = y_; a.partial = partial_; a.counters = counters_;
  a.K = K_; a.N = N_; a.nb = nb_; a.G = G_; a.kslice = kslice_; a.nsplit = nsplit_; a.strict = strict_;
  constexpr int SETS = (NB + 2) / 3;
  extern __shared__ float lds[];
  char* xs = reinterpret_cast<char*>(lds);                                   // [waves][QUADS][kDigQuad]
  float* red = reinterpret_cast<float*>(xs + WAVES * QUADS * kDigQuad);      // [waves][4 quarters][64]
  float* poison_w = red + WAVES * 4 * 64;                                    // [waves]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: addresses of a round stay scalar
  const int c = lane & 15, kb = lane >> 4;
  const int tile = blockIdx.x;
  // K split: workgroup (tile, split) takes the quads of its slice; nquads is where the slice ends
  const int q_begin = blockIdx.y * (a.kslice >> 7);
  const int nquads = min(a.K >> 7, q_begin + (a.kslice >> 7));
  const size_t n0 = RAGGED ? (size_t)min(tile * 64, a.N - 64) : (size_t)tile * 64;
  const uint32_t col_off = 4u * c;  // the lane's four columns: weights, alpha and results
  char* xs_w = xs + wv * (QUADS * kDigQuad);
  // Staging role of a lane: 16 lanes per quad; lane (st, sm) owns the eight consecutive activations
  // 8*sm .. 8*sm+7 of quad st (one 128-bit load).  Element e of the fp4 operand block of a k-word is bit
  // 4*(e & 7) + (e >> 3) of the word, so activation 8*(sm & 3) + i of k-word sm >> 2 is element
  // 8*(i & 3) + 2*(sm & 3) + (i >> 2): activations i and i + 4 are neighbours in a digit row.
  const int st = lane >> 4, sm = lane & 15;
  const int stage_off = dig_piece(sm >> 2, 0, 0) + 2 * (sm & 3);

  // what a lane multiplies its combined digits with, per set: alpha of plane 3s + kb, the bias (quarter 3
  // of set 0) or nothing (then its sums are zero)
  const _Float16* cbase[SETS];
  size_t cstride[SETS];  // elements per group
  float half_sign[SETS];
#pragma unroll
  for (int s = 0; s < SETS; ++s) {
    const int P = planes_of_set(NB, s);
    const bool is_bias = BIAS && s == 0 && kb == 3;
    const bool has_plane = kb < P;
    cbase[s] = (is_bias ? a.qbias : a.alpha + (size_t)(3 * s + min(kb, P - 1)) * a.N) + n0 + col_off;
    cstride[s] = is_bias ? (size_t)a.N : (size_t)NB * a.N;
    half_sign[s] = is_bias ? 0.5f : (has_plane ? -0.5f : 0.f);
  }

  // byte offsets of the lane's weight rows inside a quad's 4*NB rows: block j = 4m + kb of set s is k-word
  // j / P, plane 3s + j % P (a quad's rows stay below 4 GB: the host checks N)
  uint32_t wbyte[NB];
#pragma unroll
  for (int s = 0; s < SETS; ++s) {
    const int P = planes_of_set(NB, s);
#pragma unroll
    for (int m = 0; m < 3; ++m) {
      if (m >= P) continue;
      const int j = 4 * m + kb;
      wbyte[3 * s + m] = (uint32_t)(((size_t)((j / P) * NB + 3 * s + j % P) * a.N + n0 + col_off) * 4);
    }
  }

  float tot[4] = {0.f, 0.f, 0.f, 0.f};
  float poison = 0.f;  // becomes NaN when an activation is NaN or infinite (the digits cannot carry that)

  // One round of a wave: QUADS quads.  All loads are unconditional, with clamped addresses.
  struct Round {
    u4v xh;  // eight fp16 activations
    u4v wq[QUADS][NB];
    h4v cf[QUADS][SETS];
  };
  auto load_x = [&](int q0, Round& r) {
    const int quad = min(q0 + min(st, QUADS - 1), nquads - 1);
    r.xh = *reinterpret_cast<const u4v*>(a.x + (size_t)quad * 128 + 8 * sm);
  };
  auto load_quad = [&](int q0, int t, Round& r) {
    const int quad = min(q0 + t, nquads - 1);
    const char* qb = reinterpret_cast<const char*>(a.bW + ((size_t)(4 * quad) * NB) * a.N);  // scalar
#pragma unroll
    for (int i = 0; i < NB; ++i) r.wq[t][i] = load_words<RAGGED>(reinterpret_cast<const uint32_t*>(qb + wbyte[i]));
    const int g = (quad * 128) / a.G;
#pragma unroll
    for (int s = 0; s < SETS; ++s) {
      const _Float16* cp = cbase[s] + (size_t)g * cstride[s];
      if (RAGGED) r.cf[t][s] = *reinterpret_cast<const h4v_any*>(cp);
      else r.cf[t][s] = *reinterpret_cast<const h4v*>(cp);
    }
  };
  // Load schedule: the activations and the first quad go out at kernel entry, before anything else is set
  // up, and every further quad just before the arithmetic of the quad ahead of it (the last quad of a round
  // is followed by the activations and the first quad of the next round, into the other of two register
  // sets; the loop over rounds is unrolled by two, the sets swap without copies).  A compute unit takes
  // about 64 KB of outstanding loads and a wave stalls at a load while that queue is full; with all of a
  // round's loads issued at once (4 NB + 5 KB per wave) the first four waves fill the queue, the other four
  // get their loads in, and their data back, late and do all their arithmetic after the stream has ended.
  // One quad ahead keeps 8 waves x (NB + 1) loads in flight, every wave's arithmetic runs under the stream:
  // 8.17 -> 6.89 us at K=4096, N=16384, three planes (two quads ahead 7.34, all quads right after the digits
  // are staged 7.70, nothing before that 7.56-8.6).
  Round ra, rb;
  int q0 = q_begin + wv * QUADS;
  load_x(q0, ra);
  load_quad(q0, 0, ra);
  __builtin_amdgcn_sched_barrier(0);

  // Digit operand reads.  The fp8 operand of lane quarter kb holds MFMA K indices 16kb .. 16kb+15 in its
  // first 16 bytes and 64+16kb .. 64+16kb+15 in its last 16: halves h = 0, 1 lie in block 2h + (kb >> 1),
  // elements 16*(kb & 1) .. +15 of it.  Row c = 4b + d takes digit d there if the block's plane is b.
  int doff[SETS][3][2];
#pragma unroll
  for (int s = 0; s < SETS; ++s) {
    const int P = planes_of_set(NB, s);
#pragma unroll
    for (int m = 0; m < 3; ++m)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int jj = 4 * m + 2 * h + (kb >> 1);
        const int b = jj % P, kw = jj / P;
        doff[s][m][h] = (m < P && (c >> 2) == b) ? dig_piece(kw, c & 3, kb & 1) : kDigZero;
      }
  }
  // plain operand (every row r holds digit r & 3 of all four k-words): one MFMA with all-ones weights
  // gives the digit sums of the quad in every lane
  const int poff0 = dig_piece(kb >> 1, c & 3, kb & 1), poff1 = dig_piece((kb >> 1) + 2, c & 3, kb & 1);
  v8i ones;
#pragma unroll
  for (int r = 0; r < 8; ++r) ones[r] = r < 4 ? 0x11111111 : 0;
  if (lane < 4 * QUADS) *reinterpret_cast<uint32_t*>(xs_w + (lane >> 2) * kDigQuad + kDigZero + (lane & 3) * 4) = 0u;

  constexpr int STRIDE = WAVES * QUADS;
  auto compute_round = [&](int q0, Round& r, Round& next) {
    // ---- scale to 16-bit fixed point magnitudes, cut into nibbles, sign into every byte, stage ----
    float xv[8];
    float amax = 0.f;
    const bool live = st < QUADS && q0 + st < nquads;
    {
      const h8 h = __builtin_bit_cast(h8, r.xh);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        xv[j] = live ? (float)h[j] : 0.f;
        poison = fmaf(xv[j], 0.f, poison);
        amax = fmaxf(amax, fabsf(xv[j]));
      }
    }
    const float xmax = wave_max(amax);
    // 2^E * max|x| lies in [2^14, 2^15): u = rint(|x| * 2^E) <= 2^15 stays inside 16 bits
    int E = 14 - ((int)((__float_as_uint(xmax) >> 23) & 255u) - 127);
    E = xmax > 0.f ? max(-120, min(120, E)) : 0;
    const float scaleE = __uint_as_float((uint32_t)(E + 127) << 23);
    {
      uint32_t ev[8], od[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const uint32_t u = (uint32_t)(int)rintf(fabsf(xv[j]) * scaleE);
        const uint32_t sg = (uint32_t)((int)__float_as_uint(xv[j]) >> 31) & 0x8080u;
        ev[j] = (u & 0x0f0fu) | sg;         // nibbles 0 (byte 0) and 2 (byte 1)
        od[j] = ((u >> 4) & 0x0f0fu) | sg;  // nibbles 1 and 3
      }
      if (st < QUADS) {
        char* dst = xs_w + st * kDigQuad + stage_off;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          // digits of activations i and i + 4 side by side: bytes (d0, d0', d2, d2') and (d1, d1', d3, d3')
          const uint32_t pe = __builtin_amdgcn_perm(ev[i + 4], ev[i], 0x05010400u);
          const uint32_t po = __builtin_amdgcn_perm(od[i + 4], od[i], 0x05010400u);
          const int at = dig_piece(0, 0, i >> 1) + 8 * (i & 1);  // byte 8 * i of the row's 32
          *reinterpret_cast<uint16_t*>(dst + dig_piece(0, 0, 0) + at) = (uint16_t)pe;
          *reinterpret_cast<uint16_t*>(dst + dig_piece(0, 1, 0) + at) = (uint16_t)po;
          *reinterpret_cast<uint16_t*>(dst + dig_piece(0, 2, 0) + at) = (uint16_t)(pe >> 16);
          *reinterpret_cast<uint16_t*>(dst + dig_piece(0, 3, 0) + at) = (uint16_t)(po >> 16);
        }
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    // ---- MFMAs ------------------------------------------------------------------------------------
    float run[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int t = 0; t < QUADS; ++t) {
      if (q0 + t >= nquads) break;  // wave-uniform
      if (t + 1 < QUADS) {
        load_quad(q0, t + 1, r);
      } else if (!ONE_ROUND && q0 + STRIDE < nquads) {  // wave-uniform
        load_x(q0 + STRIDE, next);
        load_quad(q0 + STRIDE, 0, next);
      }
      __builtin_amdgcn_sched_barrier(0);  // issued here, not where the compiler would like it
      const char* dq = xs_w + t * kDigQuad;
      auto operand = [&](int o0, int o1) {
        const u4v lo = *reinterpret_cast<const u4v*>(dq + o0), hi = *reinterpret_cast<const u4v*>(dq + o1);
        const v8i A = {(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
        return A;
      };
      // digit sums of the quad (register i: digit i), in units of 2^-10, identical in all lanes
      const f4 dsum = mfma_fp8_fp4(operand(poff0, poff1), ones, f4{0.f, 0.f, 0.f, 0.f});
      const float xsum = fmaf(fmaf(fmaf(dsum[3], 16.f, dsum[2]), 16.f, dsum[1]), 16.f, dsum[0]);  // sum of the quad's x
#pragma unroll
      for (int s = 0; s < SETS; ++s) {
        const int P = planes_of_set(NB, s);
        const float h0 = half_sign[s] * xsum;  // sum s*x = 2 sum bit*x - sum x; +sum x / 2 for the bias quarter
        f4 acc[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) acc[q] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int m = 0; m < 3; ++m) {
          if (m >= P) continue;
          const v8i A = operand(doff[s][m][0], doff[s][m][1]);
          const u4v wv4 = r.wq[t][3 * s + m];
          const uint32_t words[4] = {wv4.x, wv4.y, wv4.z, wv4.w};
#pragma unroll
          for (int q = 0; q < 4; ++q) acc[q] = mfma_fp8_fp4(A, unpack_bits_fp4(words[q]), acc[q]);
        }
        // registers 0..3 are the digits of the lane's plane for weight column 4c + q
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float h = fmaf(fmaf(fmaf(acc[q][3], 16.f, acc[q][2]), 16.f, acc[q][1]), 16.f, acc[q][0] + h0);
          run[q] = fmaf((float)r.cf[t][s][q], h, run[q]);
        }
      }
    }
    const float descale = __uint_as_float((uint32_t)(127 - E) << 23);
#pragma unroll
    for (int q = 0; q < 4; ++q) tot[q] = fmaf(run[q], descale, tot[q]);
    // the digits of this round are consumed before the next round overwrites them
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
  };
  if (ONE_ROUND) {
    if (q0 < nquads) compute_round(q0, ra, rb);
  } else {
    while (q0 < nquads) {
      compute_round(q0, ra, rb);
      q0 += STRIDE;
      if (q0 >= nquads) break;
      compute_round(q0, rb, ra);
      q0 += STRIDE;
    }
  }
  // ---- combine lane quarters (planes, bias) and waves --------------------------------------------------
  {
    const float wp = wave_sum(poison);
    if (lane == 0) poison_w[wv] = wp;
  }
  *reinterpret_cast<f4*>(red + (wv * 4 + kb) * 64 + 4 * c) = f4{tot[0], tot[1], tot[2], tot[3]};
  __syncthreads();
  const int n = (int)n0 + tid;
  if (tid < 64 && n < a.N) {
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      const float* rw = red + (w * 4) * 64 + tid;
      v += (rw[0] + rw[64]) + (rw[128] + rw[192]);
      v += poison_w[w];
    }
    // operand units 2^-10, and the sums hold half of sum s*x
    if (a.nsplit == 1) a.y[n] = (_Float16)(v * 2048.f);
    else __hip_atomic_store(&a.partial[((size_t)tile * a.nsplit + blockIdx.y) * 64 + tid], v, __ATOMIC_RELAXED,
                            __HIP_MEMORY_SCOPE_AGENT);
  }
  if (a.nsplit > 1) {
    // Arrival counting as in the table kernel above and in q3.hip: write-through partial sums, every wave waits
    // for their acknowledgement, a barrier, one device-scope fetch-add per workgroup, and the last workgroup
    // to arrive adds the partial sums in split order with loads that bypass the non-coherent cache levels.
    // (the flag lives in the dynamic LDS block: a static variable would move that block off its 16-byte
    // alignment, and every 128-bit operand read with it)
    unsigned* s_last = reinterpret_cast<unsigned*>(poison_w + WAVES);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (tid == 0) {
      const unsigned old = a.strict ? __hip_atomic_fetch_add(&a.counters[tile], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT)
                                    : __hip_atomic_fetch_add(&a.counters[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      *s_last = (old == (unsigned)(a.nsplit - 1));
    }
    __syncthreads();
    const bool last = *s_last != 0;
    if (last && a.strict) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    if (last) {
      if (tid < 64 && n < a.N) {
        const float sum = hq_sum_partials(&a.partial[(size_t)tile * a.nsplit * 64 + tid], 64, a.nsplit);
        a.y[n] = (_Float16)(sum * 2048.f);
      }
      if (tid == 0)  // ready for the next call
        __hip_atomic_store(&a.counters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

// ---- group sizes 64 and 32 --------------------------------------------------------------------------
// Here the weights are the first operand (lane quarter kb streams k-word 4*quad + kb of one plane, one MFMA
// sums a quad of one bit plane for 16 columns) and the digits the second: the activations are biased by
// 0x8888 before they are cut into nibbles, MFMA column d carries nibble d, and a column of ones counts the
// set bits, which takes the bias out at the very end.
// A 128-element quad spans GS = 2 or 4 alpha / bias groups, so one sum per quad is not enough.  The
// B operand gets a row per (group, digit): row 4g + d holds digit d at the K positions of group g and zeros
// elsewhere (GS * 4 <= 16 MFMA columns), and a second operand holds a row of ones per group for the bit
// counts; both are zeroed once, their constant parts written once, and only the digit bytes are rewritten
// per round.  Every MFMA column then carries one group's sum, is scaled by that group's alpha (lane column
// c takes the alpha of group c / 4), and the groups are added when the digits are combined at the end.
// One B operand row is 4 lane quarters x 32 B, rows 128 B apart.  Rows 0, 2, 4 (and 1, 3) then share LDS banks
// and the bank-conflict counter shows it; rows 144 B apart (an odd multiple of 16 B, no two rows on the same
// banks) were built and measured slower, so the operand reads are not what bounds the kernel.
constexpr int kLutRow = 128;
constexpr int kGroupedQuadBytes = 20 * kLutRow;  // sixteen digit rows and up to four rows of ones
constexpr int kGroupedRedBytes = 20 * 64 * 4;  // a wave's final sums: twenty columns of 64 outputs

template <int NB, int GS, int QUADS, int WAVES, bool BIAS, bool RAGGED>
__global__ __launch_bounds__(WAVES * 64) void bcq_mfma_grouped_kernel(
    const uint32_t* bW_, const _Float16* x_, const _Float16* alpha_, const _Float16* qbias_, int K_, int N_, int nb_,
    int G_, int kslice_, int nsplit_, int strict_, _Float16* y_, float* partial_, unsigned* counters_) {
  // leading scalars, not the struct: the first 14 dwords of the arguments (all that the loads need) arrive
  // preloaded in scalar registers
  LutArgs a;
  a.bW = bW_; a.alpha = alpha_; a.qbias = qbias_; a.x = x_; a.y = y_; a.partial = partial_; a.counters = counters_;
  a.K = K_; a.N = N_; a.nb = nb_; a.G = G_; a.kslice = kslice_; a.nsplit = nsplit_; a.strict = strict_;
  constexpr int kWaveBytes = QUADS * kGroupedQuadBytes > kGroupedRedBytes ? QUADS * kGroupedQuadBytes : kGroupedRedBytes;
  extern __shared__ float lds[];
  char* xs = reinterpret_cast<char*>(lds);  // [waves][kWaveBytes]: operands in the loop, the final sums after it
  float* poison_w = reinterpret_cast<float*>(xs + WAVES * kWaveBytes);  // [waves]
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int c = lane & 15, kb = lane >> 4;
  const int tile = blockIdx.x;
  const int nquads = a.K >> 7;
  const size_t n0 = RAGGED ? (size_t)min(tile * 64, a.N - 64) : (size_t)tile * 64;
  const uint32_t col_off = 4u * c;
  const uint32_t acol = 16u * kb;
  const int cg = min(c >> 2, GS - 1);  // the group whose sums this lane's MFMA column carries
  char* xs_w = xs + wv * kWaveBytes;
  // staging role of a lane, as in bcq_mfma_kernel; its four activations lie in group sg of the quad
  const int st = lane >> 5, sa = (lane >> 3) & 3, sp = (lane >> 1) & 3, sh = lane & 1;
  const int e0 = 8 * sp + 4 * sh;
  const int s_quarter = 2 * (sa & 1) + (e0 >> 4), s_byte = 16 * (sa >> 1) + (e0 & 15);
  const int sg = (sa * GS) >> 2;
  constexpr int SP = (QUADS + 1) / 2;

  v8i ones;
#pragma unroll
  for (int r = 0; r < 8; ++r) ones[r] = r < 4 ? 0x11111111 : 0;
  // zero both operands of every quad, then the rows of ones: dword w of a row sits in lane quarter w / 8
  // at bytes 4 (w % 8), which are MFMA K indices 64 (byte / 16) + 16 quarter + byte % 16
  {
    const u4v zero = {0u, 0u, 0u, 0u};
    for (int i = lane; i < QUADS * kGroupedQuadBytes / 16; i += 64) reinterpret_cast<u4v*>(xs_w)[i] = zero;
    if (lane < 32) {
      const int k0 = 64 * ((lane & 7) >> 2) + 16 * (lane >> 3);
      const int grp = (k0 * GS) >> 7;
#pragma unroll
      for (int t = 0; t < QUADS; ++t)
        *reinterpret_cast<uint32_t*>(xs_w + t * kGroupedQuadBytes + (16 + grp) * kLutRow + lane * 4) = 0x01010101u;
    }
  }

  float tot[4][4], totp[4][4];  // digit columns and bit counts, alpha applied
#pragma unroll
  for (int q = 0; q < 4; ++q)
#pragma unroll
    for (int i = 0; i < 4; ++i) tot[q][i] = totp[q][i] = 0.f;
  float poison = 0.f;

  for (int q0 = wv * QUADS; q0 < nquads; q0 += WAVES * QUADS) {
    float xv[SP][4];
    u4v wq[QUADS][NB];
#pragma unroll
    for (int sp_ = 0; sp_ < SP; ++sp_) {
      const int quad = min(q0 + min(2 * sp_ + st, QUADS - 1), nquads - 1);
      const _Float16* xp = a.x + (size_t)quad * 128 + 32 * sa + 16 * sh + sp;
#pragma unroll
      for (int j = 0; j < 4; ++j) xv[sp_][j] = (float)xp[4 * j];
    }
    // The activations and the first quad's loads go out here, every further quad's just before the
    // arithmetic of the quad ahead of it (see bcq_planes_kernel: a wave stalls at a load while the compute
    // unit's queue of outstanding loads is full, and with a round's loads issued at once the later waves
    // get their data, and do their arithmetic, after the stream has ended).
    Half16 al[QUADS][NB], bi[QUADS];
    auto load_quad = [&](int t) {
      const int quad = min(q0 + t, nquads - 1);
      const uint32_t* wp = a.bW + ((size_t)(4 * quad + kb) * NB) * a.N + n0 + col_off;
#pragma unroll
      for (int b = 0; b < NB; ++b) wq[t][b] = load_words<RAGGED>(wp + (size_t)b * a.N);
      const int g = quad * GS + cg;
#pragma unroll
      for (int b = 0; b < NB; ++b) al[t][b] = load_half16<RAGGED>(a.alpha + ((size_t)g * NB + b) * a.N + n0 + acol);
      if (BIAS) bi[t] = load_half16<RAGGED>(a.qbias + (size_t)g * a.N + n0 + acol);
    };
    load_quad(0);
    __builtin_amdgcn_sched_barrier(0);
    float amax = 0.f;
#pragma unroll
    for (int sp_ = 0; sp_ < SP; ++sp_) {
      const int t = 2 * sp_ + st;
      const bool live = t < QUADS && q0 + t < nquads;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (!live) xv[sp_][j] = 0.f;
        poison = fmaf(xv[sp_][j], 0.f, poison);
        amax = fmaxf(amax, fabsf(xv[sp_][j]));
      }
    }
    const float xmax = wave_max(amax);
    int E = 13 - ((int)((__float_as_uint(xmax) >> 23) & 255u) - 127);
    E = xmax > 0.f ? max(-120, min(120, E)) : 0;
    const float scaleE = __uint_as_float((uint32_t)(E + 127) << 23);
#pragma unroll
    for (int sp_ = 0; sp_ < SP; ++sp_) {
      uint32_t ev[4], od[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t u = (uint32_t)((int)rintf(xv[sp_][j] * scaleE) + 0x8888);
        ev[j] = u & 0x0f0fu;
        od[j] = (u >> 4) & 0x0f0fu;
      }
      const uint32_t pe = __builtin_amdgcn_perm(ev[1], ev[0], 0x05010400u);
      const uint32_t qe = __builtin_amdgcn_perm(ev[3], ev[2], 0x05010400u);
      const uint32_t po = __builtin_amdgcn_perm(od[1], od[0], 0x05010400u);
      const uint32_t qo = __builtin_amdgcn_perm(od[3], od[2], 0x05010400u);
      const uint32_t dg[4] = {__builtin_amdgcn_perm(qe, pe, 0x05040100u), __builtin_amdgcn_perm(qo, po, 0x05040100u),
                              __builtin_amdgcn_perm(qe, pe, 0x07060302u), __builtin_amdgcn_perm(qo, po, 0x07060302u)};
      const int t = 2 * sp_ + st;
      if (t < QUADS) {
        char* dst = xs_w + t * kGroupedQuadBytes + (4 * sg) * kLutRow + s_quarter * 32 + s_byte;
#pragma unroll
        for (int d = 0; d < 4; ++d) *reinterpret_cast<uint32_t*>(dst + d * kLutRow) = dg[d];
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    float run[4][4], runp[4][4];
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int i = 0; i < 4; ++i) run[q][i] = runp[q][i] = 0.f;
#pragma unroll
    for (int t = 0; t < QUADS; ++t) {
      if (q0 + t >= nquads) break;  // wave-uniform
      if (t + 1 < QUADS) {
        load_quad(t + 1);
        __builtin_amdgcn_sched_barrier(0);  // issued here, not where the compiler would like it
      }
      // digit rows: MFMA column c reads row c (rows past 4 GS stay zero and are never used);
      // rows of ones: column c reads its group's
      const u4v* bp = reinterpret_cast<const u4v*>(xs_w + t * kGroupedQuadBytes + c * kLutRow + kb * 32);
      const u4v* pp = reinterpret_cast<const u4v*>(xs_w + t * kGroupedQuadBytes + (16 + cg) * kLutRow + kb * 32);
      const u4v b0 = bp[0], b1 = bp[1], p0 = pp[0], p1 = pp[1];
      const v8i B = {(int)b0.x, (int)b0.y, (int)b0.z, (int)b0.w, (int)b1.x, (int)b1.y, (int)b1.z, (int)b1.w};
      const v8i P = {(int)p0.x, (int)p0.y, (int)p0.z, (int)p0.w, (int)p1.x, (int)p1.y, (int)p1.z, (int)p1.w};
      const f4 dsum = mfma_fp4_fp8(ones, B, f4{0.f, 0.f, 0.f, 0.f});
      const f4 psum = mfma_fp4_fp8(ones, P, f4{0.f, 0.f, 0.f, 0.f});
      const f4 init = {-0.5f * dsum[0], -0.5f * dsum[1], -0.5f * dsum[2], -0.5f * dsum[3]};
      const f4 initp = {-0.5f * psum[0], -0.5f * psum[1], -0.5f * psum[2], -0.5f * psum[3]};
      if (BIAS) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            run[q][i] = fmaf(bi[t].get(4 * i + q), 0.5f * dsum[i], run[q][i]);
            runp[q][i] = fmaf(bi[t].get(4 * i + q), 0.5f * psum[i], runp[q][i]);
          }
      }
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        const uint32_t words[4] = {wq[t][b].x, wq[t][b].y, wq[t][b].z, wq[t][b].w};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const v8i A = unpack_bits_fp4(words[q]);
          const f4 acc = mfma_fp4_fp8(A, B, init);
          const f4 accp = mfma_fp4_fp8(A, P, initp);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float al_n = al[t][b].get(4 * i + q);
            run[q][i] = fmaf(al_n, acc[i], run[q][i]);
            runp[q][i] = fmaf(al_n, accp[i], runp[q][i]);
          }
        }
      }
    }
    const float descale = __uint_as_float((uint32_t)(127 - E) << 23);
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        tot[q][i] = fmaf(run[q][i], descale, tot[q][i]);
        totp[q][i] = fmaf(runp[q][i], descale, totp[q][i]);
      }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
  }
  // ---- combine digits, groups and waves: the wave's operand area now takes its sums -----------------
  {
    const float wp = wave_sum(poison);
    if (lane == 0) poison_w[wv] = wp;
  }
  float* red_w = reinterpret_cast<float*>(xs_w);  // [20][64]: rows 4g + d digits, rows 16 + g bit counts
  if (c < 4 * GS) {
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int i = 0; i < 4; ++i) red_w[c * 64 + 16 * kb + 4 * i + q] = tot[q][i];
  }
  if (c < 4 * GS && (c & 3) == 0) {
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int i = 0; i < 4; ++i) red_w[(16 + (c >> 2)) * 64 + 16 * kb + 4 * i + q] = totp[q][i];
  }
  __syncthreads();
  const int n = (int)n0 + tid;
  if (tid < 64 && n < a.N) {
    float v = 0.f;
    for (int w = 0; w < WAVES; ++w) {
      const float* rw = reinterpret_cast<const float*>(xs + w * kWaveBytes) + tid;
#pragma unroll
      for (int g = 0; g < GS; ++g) {
        const float* rg = rw + 4 * g * 64;
        v += (((rg[192] * 16.f + rg[128]) * 16.f + rg[64]) * 16.f + rg[0]) - 34952.f * rw[(16 + g) * 64];
      }
      v += poison_w[w];
    }
    a.y[n] = (_Float16)(v * 2048.f);
  }
}

template <int NB, int GS, int QUADS>
int launch_bcq_grouped(const LutArgs& a, bool ragged, hipStream_t stream) {
  constexpr int WAVES = 8;
  constexpr int kWaveBytes = QUADS * kGroupedQuadBytes > kGroupedRedBytes ? QUADS * kGroupedQuadBytes : kGroupedRedBytes;
  const size_t smem = (size_t)WAVES * kWaveBytes + (size_t)WAVES * 4;
  const dim3 grid((a.N + 63) / 64), block(WAVES * 64);
#define HQ_LUT_GO(BIAS, RAG) \
  hipLaunchKernelGGL((bcq_mfma_grouped_kernel<NB, GS, QUADS, WAVES, BIAS, RAG>), grid, block, smem, stream, a.bW, a.x, a.alpha, a.qbias, a.K, a.N, a.nb, a.G, a.kslice, a.nsplit, a.strict, a.y, a.partial, a.counters)
  if (a.qbias) { if (ragged) HQ_LUT_GO(true, true); else HQ_LUT_GO(true, false); }
  else { if (ragged) HQ_LUT_GO(false, true); else HQ_LUT_GO(false, false); }
#undef HQ_LUT_GO
  return hq_launch_status();
}
template <int GS>
int launch_bcq_grouped_nb(const LutArgs& a, bool ragged, hipStream_t stream) {
  switch (a.nb) {  // quads per wave per round, bounded by the register budget
    case 1: return launch_bcq_grouped<1, GS, 2>(a, ragged, stream);
    case 2: return launch_bcq_grouped<2, GS, 2>(a, ragged, stream);
    case 3: return launch_bcq_grouped<3, GS, 2>(a, ragged, stream);
    case 4: return launch_bcq_grouped<4, GS, 2>(a, ragged, stream);
    case 5: return launch_bcq_grouped<5, GS, 1>(a, ragged, stream);
    case 6: return launch_bcq_grouped<6, GS, 1>(a, ragged, stream);
    case 7: return launch_bcq_grouped<7, GS, 1>(a, ragged, stream);
    default: return launch_bcq_grouped<8, GS, 1>(a, ragged, stream);
  }
}

// Eight waves per workgroup (two per SIMD, up to 256 VGPRs each); QUADS is bounded by the two register
// sets of a round's loads.
template <int NB, int QUADS>
int launch_bcq_planes(LutArgs a, bool ragged, int cus, hipStream_t stream) {
  constexpr int WAVES = 8;
  // K split: with fewer column tiles than compute units, whole rounds (128 QUADS WAVES elements of K) go to
  // workgroups of their own, as many as there are compute units to take them (K=11008, N=4096, three planes:
  // 64 tiles x 3 rounds)
  const int ntiles = (a.N + 63) / 64;
  const int nquads = a.K >> 7;
  const int rounds = (nquads + WAVES * QUADS - 1) / (WAVES * QUADS);
  int nsplit = cus / ntiles;
  if (nsplit > rounds) nsplit = rounds;
  if (nsplit < 1) nsplit = 1;
  const int rpw = (rounds + nsplit - 1) / nsplit;
  nsplit = (rounds + rpw - 1) / rpw;
  a.kslice = rpw * WAVES * QUADS * 128;
  a.nsplit = nsplit;
  a.strict = hq_tune(HQ_TUNE_SPLITK_FENCES, 0);
  if (nsplit > 1) {
    HqWorkspace ws;
    const int rc = hq_get_workspace(stream, (size_t)ntiles * nsplit * 64, (size_t)ntiles, &ws);
    if (rc != HQ_OK) return rc;
    a.partial = ws.partial;
    a.counters = ws.counters;
  }
  const dim3 grid(ntiles, nsplit), block(WAVES * 64);
  const size_t smem = (size_t)WAVES * QUADS * kDigQuad + (size_t)WAVES * 4 * 64 * 4 + (size_t)WAVES * 4 + 16;
  const bool one_round = rpw == 1;
#define HQ_LUT_GO(BIAS, RAG)                                                                                        \
  do {                                                                                                              \
    if (one_round) hipLaunchKernelGGL((bcq_planes_kernel<NB, QUADS, WAVES, BIAS, RAG, true>), grid, block, smem, stream, \
                                       a.bW, a.x, a.alpha, a.qbias, a.K, a.N, a.nb, a.G, a.kslice, a.nsplit, a.strict, a.y, a.partial, a.counters); \
    else hipLaunchKernelGGL((bcq_planes_kernel<NB, QUADS, WAVES, BIAS, RAG, false>), grid, block, smem, stream, \
                            a.bW, a.x, a.alpha, a.qbias, a.K, a.N, a.nb, a.G, a.kslice, a.nsplit, a.strict, a.y, a.partial, a.counters); \
  } while (0)
  if (a.qbias) { if (ragged) HQ_LUT_GO(true, true); else HQ_LUT_GO(true, false); }
  else { if (ragged) HQ_LUT_GO(false, true); else HQ_LUT_GO(false, false); }
#undef HQ_LUT_GO
  return hq_launch_status();
}

// Which kernel a call takes (HQ_LUT_PLAN_* in hq.h).
int lut_plan(const void* bW, const void* alpha, const void* q_bias, int K, int N, int group_size) {
  if (hq_tune(HQ_TUNE_LUT_PATH, 1) != 1) return HQ_LUT_PLAN_TABLE;
  if (K % 128 != 0 || N < 64 || N >= (1 << 25)) return HQ_LUT_PLAN_TABLE;  // 32-bit byte offsets inside 32 rows
  const bool aligned = N % 64 == 0 && !((uintptr_t)bW & 15) && !((uintptr_t)alpha & 15) && !((uintptr_t)q_bias & 15);
  int plan;
  if (group_size == 64 || group_size == 32) plan = HQ_LUT_PLAN_MFMA_GROUPED;
  else if (group_size % 128 == 0) plan = HQ_LUT_PLAN_MFMA;
  else return HQ_LUT_PLAN_TABLE;
  return aligned ? plan : (plan | HQ_LUT_PLAN_RAGGED);
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

  const int plan = lut_plan(bW, alpha, q_bias, K, N, group_size);
  if (plan != HQ_LUT_PLAN_TABLE) {
    const bool ragged = (plan & HQ_LUT_PLAN_RAGGED) != 0;
    LutArgs a;
    a.bW = bW; a.alpha = (const _Float16*)alpha; a.qbias = (const _Float16*)q_bias;
    a.x = (const _Float16*)x; a.y = (_Float16*)y; a.partial = nullptr; a.counters = nullptr;
    a.K = K; a.N = N; a.nb = nbits; a.G = group_size; a.kslice = K; a.nsplit = 1; a.strict = 0;
    if ((plan & ~HQ_LUT_PLAN_RAGGED) == HQ_LUT_PLAN_MFMA_GROUPED)
      return group_size == 64 ? launch_bcq_grouped_nb<2>(a, ragged, stream) : launch_bcq_grouped_nb<4>(a, ragged, stream);
    switch (nbits) {  // quads per wave per round, bounded by the register budget
      case 1: return launch_bcq_planes<1, 4>(a, ragged, dev->cus, stream);
      case 2: return launch_bcq_planes<2, 4>(a, ragged, dev->cus, stream);
      case 3: return launch_bcq_planes<3, 4>(a, ragged, dev->cus, stream);
      case 4: return launch_bcq_planes<4, 2>(a, ragged, dev->cus, stream);
      case 5: return launch_bcq_planes<5, 2>(a, ragged, dev->cus, stream);
      case 6: return launch_bcq_planes<6, 2>(a, ragged, dev->cus, stream);
      case 7: return launch_bcq_planes<7, 1>(a, ragged, dev->cus, stream);
      default: return launch_bcq_planes<8, 1>(a, ragged, dev->cus, stream);
    }
  }
  const bool pair = (N % 2 == 0) && !((uintptr_t)bW & 7);
  const int cpl = pair ? 2 : 1;
  const int ntiles = (N + 64 * cpl - 1) / (64 * cpl);
  // K slice per workgroup: enough workgroups to cover the CUs about twice.
  int nsplit = hq_tune(HQ_TUNE_LUT_KSPLIT, 0);
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
  a.K = K; a.N = N; a.nb = nbits; a.G = group_size; a.kslice = steps_per * kStepK; a.nsplit = nsplit; a.strict = hq_tune(HQ_TUNE_SPLITK_FENCES, 0);
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

extern "C" int hq_lut_gemv_plan(const uint32_t* bW, const void* alpha, const void* q_bias, int K, int N, int nbits,
                                int group_size) {
  if (K <= 0 || N <= 0 || nbits < 1 || nbits > 8 || group_size <= 0) return HQ_ERR_BAD_SHAPE;
  if ((K & 31) || (group_size & 31) || (K % group_size)) return HQ_ERR_BAD_SHAPE;
  return lut_plan(bW, alpha, q_bias, K, N, group_size);
}
