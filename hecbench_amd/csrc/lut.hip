// LUT-GEMM binary-coded-quantisation matvec for gfx950 (fp16 in / fp16 out).
//
// Replaces matmul() -> nqmv_bias / nqmv -> _nqmv_bias<32> / _nqmv<64>
// (src/lut-gemm-hip/kernels.cu:22-31, mv_fp16.h:28-259 in the HeCBench tree).
//
//   y[n] = sum_k x[k] * ( q_bias[k/G][n] + sum_b alpha[k/G][b][n] * s(k,b,n) )
//
// Two kernels.  Shapes with group size % 128 == 0 and N % 64 == 0 run on the matrix cores
// (bcq_mfma_kernel below: the packed bits themselves are the fp8 operands, no tables).
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


// ======================================================================================
// Matrix-core path (group size a multiple of 128, N a multiple of 64).
//
// sum_k s*x = 2*(sum_k bit*x - (sum_k x)/2).  An fp8 (e4m3) byte whose exponent field is
// zero is the subnormal mantissa*2^-9, so a single weight bit left in place at bit p
// (p <= 2) of an otherwise zero byte IS the fp8 number 2^(p-9): eight ANDs and two shifts
// turn a packed 32-bit word into the eight operand registers (32 fp8 values) of one
// 16x16x128 fp8 MFMA; the factor 2^p is folded into the activation of that slot.  No table,
// no LDS lookup, no bank conflicts.  The activations of a round (256 of them per wave) are
// scaled to 16-bit fixed point and split into four signed 4-bit digits carried by MFMA
// columns 0..3, so every product is an integer and the matrix-core sums are exact.  Lane
// quarter kb streams k-word 4*quad + kb, so one MFMA sums a whole 128-element quad of one
// bit plane for 16 columns (four adjacent columns per lane and 128-bit load); alpha is
// applied to that sum in fp32, per digit, and the digits are combined once at the end.
typedef _Float16 h2v __attribute__((ext_vector_type(2)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4v __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));

// operand register r of a word holds bit r of each of its four bytes, at mantissa bit p(r)
__device__ __forceinline__ constexpr int bit_pos(int r) { return r < 6 ? r % 3 : r - 6; }
__device__ __forceinline__ constexpr uint32_t bit_mask(int r) { return 0x01010101u << bit_pos(r); }

__device__ __forceinline__ v8i unpack_bits_fp8(uint32_t w) {
  const uint32_t w3 = w >> 3, w6 = w >> 6;
  v8i a;
#pragma unroll
  for (int r = 0; r < 8; ++r) a[r] = (int)((r < 3 ? w : (r < 6 ? w3 : w6)) & bit_mask(r));
  return a;
}

__device__ __forceinline__ f4 mfma_fp8(v8i a, v8i b, f4 c) {
  // fp8 x fp8, both block scales 2^0 (E8M0 code 127)
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, 0, 0, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
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

struct Half16 {  // sixteen fp16 values as two 128-bit loads
  u4v lo, hi;
  __device__ __forceinline__ float get(int i) const {
    const uint32_t w[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    const uint32_t d = w[i >> 1];
    return (float)__builtin_bit_cast(_Float16, (uint16_t)((i & 1) ? (d >> 16) : (d & 0xffffu)));
  }
};
__device__ __forceinline__ Half16 load_half16(const _Float16* p) {
  Half16 h;
  h.lo = reinterpret_cast<const u4v*>(p)[0];
  h.hi = reinterpret_cast<const u4v*>(p)[1];
  return h;
}

// NB bit planes, QUADS 128-element quads per wave per round, WAVES waves per workgroup.
template <int NB, int QUADS, int WAVES, bool BIAS>
__global__ __launch_bounds__(WAVES * 64) void bcq_mfma_kernel(LutArgs a) {
  extern __shared__ float lds[];
  uint32_t* xs = reinterpret_cast<uint32_t*>(lds);  // [waves][QUADS][4 kb][4 digits][8 regs] dwords
  float* red = lds + WAVES * QUADS * 128;           // [waves][4 digits][64]
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int c = lane & 15, kb = lane >> 4;
  const int tile = blockIdx.x;
  const int nquads = a.K >> 7;
  const size_t n0 = (size_t)tile * 64;
  const uint32_t col_off = 4u * c;   // first of the lane's 4 columns (N % 64 == 0: no partial tiles)
  const uint32_t acol = 16u * kb;    // first of the 16 columns this lane applies alpha to
  // staging role of lane (c, kb): elements k_lo = (c&7) + 16*(c>>3) and k_lo + 8 of k-word kb,
  // i.e. operand register r = c&7, bytes 2*(c>>3) and 2*(c>>3)+1
  const int r_slot = c & 7, k_lo = r_slot + 16 * (c >> 3);
  const float slot_scale = __uint_as_float((uint32_t)(127 + 2 - bit_pos(r_slot)) << 23);  // 2^(2-p)
  uint32_t* xs_w = xs + wv * (QUADS * 128);
  const int digit = c & 3;  // MFMA column -> digit (columns 4..15 repeat them and are never read)

  v8i ones;  // every slot's bit set: one MFMA with it sums the digits of a quad
#pragma unroll
  for (int r = 0; r < 8; ++r) ones[r] = (int)bit_mask(r);

  float tot[4][4];
#pragma unroll
  for (int q = 0; q < 4; ++q)
#pragma unroll
    for (int i = 0; i < 4; ++i) tot[q][i] = 0.f;

  for (int q0 = wv * QUADS; q0 < nquads; q0 += WAVES * QUADS) {
    // ---- loads of this round (unconditional, clamped): activations, then packed words -------
    float xlo[QUADS], xhi[QUADS];
    u4v wq[QUADS][NB];
#pragma unroll
    for (int t = 0; t < QUADS; ++t) {
      const int quad = min(q0 + t, nquads - 1);
      const _Float16* xp = a.x + (size_t)quad * 128 + 32 * kb + k_lo;
      xlo[t] = (float)xp[0];
      xhi[t] = (float)xp[8];
    }
#pragma unroll
    for (int t = 0; t < QUADS; ++t) {
      const int quad = min(q0 + t, nquads - 1);
      const uint32_t* wp = a.bW + ((size_t)(4 * quad + kb) * NB) * a.N + n0 + col_off;
#pragma unroll
      for (int b = 0; b < NB; ++b)
        wq[t][b] = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(wp + (size_t)b * a.N));
    }
    // ---- scale to 16-bit fixed point, split into four signed 4-bit digits, stage (wave-local)
    float amax = 0.f;
#pragma unroll
    for (int t = 0; t < QUADS; ++t) {
      if (q0 + t >= nquads) { xlo[t] = 0.f; xhi[t] = 0.f; }
      amax = fmaxf(amax, fmaxf(fabsf(xlo[t]), fabsf(xhi[t])));
    }
    const float xmax = wave_max(amax);
    // 2^E * max|x| lies in [2^14, 2^15)
    int E = 14 - ((int)((__float_as_uint(xmax) >> 23) & 255u) - 127);
    E = xmax > 0.f ? max(-120, min(120, E)) : 0;
    const float scaleE = __uint_as_float((uint32_t)(E + 127) << 23);
#pragma unroll
    for (int t = 0; t < QUADS; ++t) {
      float d[2][4];
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const float X = rintf((e ? xhi[t] : xlo[t]) * scaleE);
        d[e][0] = rintf(X * (1.f / 4096.f));
        const float r1 = X - d[e][0] * 4096.f;
        d[e][1] = rintf(r1 * (1.f / 256.f));
        const float r2 = r1 - d[e][1] * 256.f;
        d[e][2] = rintf(r2 * (1.f / 16.f));
        d[e][3] = r2 - d[e][2] * 16.f;
      }
      uint16_t* dst = reinterpret_cast<uint16_t*>(xs_w + ((t * 4 + kb) * 4) * 8 + r_slot) + (c >> 3);
#pragma unroll
      for (int dg = 0; dg < 4; ++dg) {
        // digit * 2^(2-p) is exact in fp8 (|digit| <= 8)
        const int pk = __builtin_amdgcn_cvt_pk_fp8_f32(d[0][dg] * slot_scale, d[1][dg] * slot_scale, 0, false);
        dst[dg * 16] = (uint16_t)pk;  // next digit: 8 registers = 16 halves further
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    // ---- MFMAs ------------------------------------------------------------------------------------
    float run[4][4];
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int i = 0; i < 4; ++i) run[q][i] = 0.f;
#pragma unroll
    for (int t = 0; t < QUADS; ++t) {
      if (q0 + t >= nquads) break;  // wave-uniform
      const int quad = q0 + t;
      const int g = (quad * 128) / a.G;
      Half16 al[NB];
#pragma unroll
      for (int b = 0; b < NB; ++b) al[b] = load_half16(a.alpha + ((size_t)g * NB + b) * a.N + n0 + acol);
      const u4v* bp = reinterpret_cast<const u4v*>(xs_w + ((t * 4 + kb) * 4 + digit) * 8);
      const u4v b0 = bp[0], b1 = bp[1];
      const v8i B = {(int)b0.x, (int)b0.y, (int)b0.z, (int)b0.w, (int)b1.x, (int)b1.y, (int)b1.z, (int)b1.w};
      // digit sum of the quad (in operand units 2^-7), identical in all four result rows
      const f4 dsum = mfma_fp8(ones, B, f4{0.f, 0.f, 0.f, 0.f});
      const f4 init = {-0.5f * dsum[0], -0.5f * dsum[1], -0.5f * dsum[2], -0.5f * dsum[3]};
      if (BIAS) {
        const Half16 bi = load_half16(a.qbias + (size_t)g * a.N + n0 + acol);
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int q = 0; q < 4; ++q) run[q][i] = fmaf(bi.get(4 * i + q), 0.5f * dsum[i], run[q][i]);
      }
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        const uint32_t words[4] = {wq[t][b].x, wq[t][b].y, wq[t][b].z, wq[t][b].w};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          // one MFMA = this digit's sum over the quad of bit*x, minus half the digit sum
          const f4 acc = mfma_fp8(unpack_bits_fp8(words[q]), B, init);
          // rows 4*kb + i of the tile's 16-column block q: column 16*kb + 4*i + q
#pragma unroll
          for (int i = 0; i < 4; ++i) run[q][i] = fmaf(al[b].get(4 * i + q), acc[i], run[q][i]);
        }
      }
    }
    const float descale = __uint_as_float((uint32_t)(127 - E) << 23);
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int i = 0; i < 4; ++i) tot[q][i] = fmaf(run[q][i], descale, tot[q][i]);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
  }
  // ---- combine digits and waves -------------------------------------------------------------------
  if (c < 4) {
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[(wv * 4 + c) * 64 + 16 * kb + 4 * i + q] = tot[q][i];
  }
  __syncthreads();
  const int n = tile * 64 + tid;
  if (tid < 64 && n < a.N) {
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      const float* rw = red + (w * 4) * 64 + tid;
      v += ((rw[0] * 16.f + rw[64]) * 16.f + rw[128]) * 16.f + rw[192];
    }
    // operand units 2^-7, and the sums hold half of sum s*x
    a.y[n] = (_Float16)(v * 256.f);
  }
}

// Eight waves per workgroup (two per SIMD, up to 256 VGPRs each): sixteen-wave variants
// spill and measured slower.
template <int NB, int QUADS>
int launch_bcq_mfma(const LutArgs& a, hipStream_t stream) {
  constexpr int WAVES = 8;
  const size_t smem = (size_t)WAVES * QUADS * 512 + (size_t)WAVES * 4 * 64 * 4;
  const int ntiles = a.N / 64;
  if (a.qbias)
    hipLaunchKernelGGL((bcq_mfma_kernel<NB, QUADS, WAVES, true>), dim3(ntiles), dim3(WAVES * 64), smem, stream, a);
  else
    hipLaunchKernelGGL((bcq_mfma_kernel<NB, QUADS, WAVES, false>), dim3(ntiles), dim3(WAVES * 64), smem, stream, a);
  return hq_launch_status();
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

  if (group_size % 128 == 0 && N % 64 == 0 && !((uintptr_t)bW & 15) && !((uintptr_t)alpha & 15) &&
      !((uintptr_t)q_bias & 15) && hq_env_int("HQ_LUT_PATH", 1) == 1) {
    LutArgs a;
    a.bW = bW; a.alpha = (const _Float16*)alpha; a.qbias = (const _Float16*)q_bias;
    a.x = (const _Float16*)x; a.y = (_Float16*)y; a.partial = nullptr; a.counters = nullptr;
    a.K = K; a.N = N; a.nb = nbits; a.G = group_size; a.kslice = K; a.nsplit = 1;
    switch (nbits) {  // quads per wave per round, bounded by the register budget
      case 1: return launch_bcq_mfma<1, 2>(a, stream);
      case 2: return launch_bcq_mfma<2, 2>(a, stream);
      case 3: return launch_bcq_mfma<3, 2>(a, stream);
      case 4: return launch_bcq_mfma<4, 2>(a, stream);
      case 5: return launch_bcq_mfma<5, 2>(a, stream);
      case 6: return launch_bcq_mfma<6, 2>(a, stream);
      case 7: return launch_bcq_mfma<7, 1>(a, stream);
      default: return launch_bcq_mfma<8, 1>(a, stream);
    }
  }
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
