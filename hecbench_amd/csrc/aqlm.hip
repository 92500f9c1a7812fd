// AQLM 1x16 code-book matvec for gfx950 (fp16 in / fp16 out).
//
// Replaces Code1x16MatVec / code1x16_matvec (src/quantAQLM-hip/main.cu:29-139
// in the HeCBench tree).
//
//   y[m] = fp16_rn( scale[m] * sum_g dot8(codebook[cb(m)][u16(codes[m][g])], x[8g..8g+7]) )
//
// One wave owns ROWS consecutive output rows.  Lane l always works on the same
// 64 activations (codes 8l..8l+7 of a 512-code chunk), so the activations live
// in registers for every row of the wave and LDS is not needed.  A row chunk is
// one 128-bit code load per lane (1 KB contiguous per wave); each code gathers a
// 16-byte code-book entry (the 1 MB code book stays L2-resident) and feeds four
// fp16 dot2 instructions with fp32 accumulation.  Lanes are combined with a
// cross-lane butterfly, the scale is applied in fp32 and the result is rounded
// to fp16 once.
#include "hq_internal.h"

namespace {

typedef _Float16 h2v __attribute__((ext_vector_type(2)));
typedef uint32_t u4v __attribute__((ext_vector_type(4)));

struct AqlmArgs {
  const u4v* codes;      // [M][K/64] as 16-byte units
  const u4v* codebooks;  // 16-byte entries
  const _Float16* scales;  // nullable
  const u4v* x;          // [K/8]
  _Float16* y;
  int M, K;
  int cb_sizes[4];
  int cb_stride;  // in 16-byte units
};

__device__ __forceinline__ h2v as_h2(uint32_t v) { return __builtin_bit_cast(h2v, v); }

__device__ __forceinline__ float dot8(u4v e, u4v xv, float acc) {
  // components are copied to scalars first: bit-casting a vector element in place
  // makes the compiler read element 0 for every component
  const uint32_t e0 = e.x, e1 = e.y, e2 = e.z, e3 = e.w;
  const uint32_t x0 = xv.x, x1 = xv.y, x2 = xv.z, x3 = xv.w;
  acc = __builtin_amdgcn_fdot2(as_h2(e0), as_h2(x0), acc, false);
  acc = __builtin_amdgcn_fdot2(as_h2(e1), as_h2(x1), acc, false);
  acc = __builtin_amdgcn_fdot2(as_h2(e2), as_h2(x2), acc, false);
  acc = __builtin_amdgcn_fdot2(as_h2(e3), as_h2(x3), acc, false);
  return acc;
}

template <int ROWS>
__global__ __launch_bounds__(256) void aqlm_matvec_kernel(const u4v* codes_, const u4v* codebooks_, const u4v* x_, int M_, int K_, int cb_stride_,
                                                         int cb0_, int cb1_, int cb2_, int cb3_,
                                                         const _Float16* scales_, _Float16* y_) {
  // leading scalars, not the struct: the first 14 dwords of the arguments arrive preloaded in scalar registers
  AqlmArgs a;
  a.codes = codes_; a.codebooks = codebooks_; a.scales = scales_; a.x = x_; a.y = y_;
  a.M = M_; a.K = K_; a.cb_stride = cb_stride_;
  a.cb_sizes[0] = cb0_; a.cb_sizes[1] = cb1_; a.cb_sizes[2] = cb2_; a.cb_sizes[3] = cb3_;
  const int lane = threadIdx.x & 63;
  // Workgroups b, b + 8, b + 16, ... run on the same XCD; inside every 64 of them the row blocks are dealt
  // out so that the eight workgroups whose results share a 128-byte line of y are on one XCD (its L2 then
  // writes the line back whole instead of eight XCDs writing 16 bytes of it each).
  const int b = blockIdx.x;
  const int blk = b < (int)(gridDim.x & ~63u) ? ((b & ~63) | ((b & 7) << 3) | ((b >> 3) & 7)) : b;
  const int wave = (blk * 256 + threadIdx.x) >> 6;
  const int row0 = wave * ROWS;
  if (row0 >= a.M) return;  // wave-uniform
  const int units_per_row = a.K >> 6;         // 16-byte code units (8 codes) per row; K % 64 == 0
  const u4v* cb[ROWS];
  float acc[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const int m = min(row0 + r, a.M - 1);
    const u4v* p = a.codebooks;
    for (int j = 0; j < 4 && m >= a.cb_sizes[j]; ++j) p += a.cb_stride;
    cb[r] = p;
    acc[r] = 0.f;
  }
  for (int u0 = 0; u0 < units_per_row; u0 += 64) {
    const int u = u0 + lane;
    if (u < units_per_row) {
      u4v xv[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) xv[i] = a.x[(size_t)u * 8 + i];
      u4v cw[ROWS];
#pragma unroll
      for (int r = 0; r < ROWS; ++r) {
        const int m = min(row0 + r, a.M - 1);
        cw[r] = __builtin_nontemporal_load(a.codes + (size_t)m * units_per_row + u);
      }
#pragma unroll
      for (int r = 0; r < ROWS; ++r) {
        const uint32_t w[4] = {cw[r].x, cw[r].y, cw[r].z, cw[r].w};
        u4v e[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const uint32_t code = (w[i >> 1] >> (16 * (i & 1))) & 0xffffu;  // read as unsigned
          e[i] = cb[r][code];
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[r] = dot8(e[i], xv[i], acc[r]);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    float v = acc[r];
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) v += __shfl_xor(v, m);
    if (lane == 0 && row0 + r < a.M) {
      if (a.scales) v *= (float)a.scales[row0 + r];
      a.y[row0 + r] = (_Float16)v;
    }
  }
}

}  // namespace

extern "C" int hq_aqlm_matvec(const int16_t* codes, const void* codebooks, const void* scales,
                              const void* x, void* y, int M, int K, const int cb_a_sizes[4],
                              int cb_stride_int4, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!codes || !codebooks || !x || !y || !cb_a_sizes) return HQ_ERR_NULL_POINTER;
  if (M <= 0 || K <= 0 || (K & 63) || cb_stride_int4 < 0) return HQ_ERR_BAD_SHAPE;
  if (((uintptr_t)codes & 15) || ((uintptr_t)codebooks & 15) || ((uintptr_t)x & 15) ||
      ((uintptr_t)y & 1) || ((uintptr_t)scales & 1))
    return HQ_ERR_MISALIGNED;
  const HqDevice* dev = nullptr;
  int rc = hq_current_device(&dev);
  if (rc != HQ_OK) return rc;

  AqlmArgs a;
  a.codes = (const u4v*)codes; a.codebooks = (const u4v*)codebooks; a.scales = (const _Float16*)scales;
  a.x = (const u4v*)x; a.y = (_Float16*)y; a.M = M; a.K = K; a.cb_stride = cb_stride_int4;
  for (int j = 0; j < 4; ++j) a.cb_sizes[j] = cb_a_sizes[j];
  // Rows per wave: keep at least ~8 waves per CU in flight (mirrors the CU-count
  // based sizing of the reference launcher, src/quantAQLM-hip/main.cu:108-121).
  int rows = hq_tune(HQ_TUNE_AQLM_ROWS, 0);
  if (rows != 1 && rows != 2 && rows != 4) {
    const long waves_wanted = (long)dev->cus * 8;
    rows = (M >= 4 * waves_wanted) ? 4 : (M >= 2 * waves_wanted ? 2 : 1);
  }
  const int nwaves = (M + rows - 1) / rows;
  const int blocks = (nwaves + 3) / 4;
  if (rows == 4) hipLaunchKernelGGL(aqlm_matvec_kernel<4>, dim3(blocks), dim3(256), 0, stream, a.codes, a.codebooks, a.x, a.M, a.K, a.cb_stride, a.cb_sizes[0], a.cb_sizes[1], a.cb_sizes[2], a.cb_sizes[3], a.scales, a.y);
  else if (rows == 2) hipLaunchKernelGGL(aqlm_matvec_kernel<2>, dim3(blocks), dim3(256), 0, stream, a.codes, a.codebooks, a.x, a.M, a.K, a.cb_stride, a.cb_sizes[0], a.cb_sizes[1], a.cb_sizes[2], a.cb_sizes[3], a.scales, a.y);
  else hipLaunchKernelGGL(aqlm_matvec_kernel<1>, dim3(blocks), dim3(256), 0, stream, a.codes, a.codebooks, a.x, a.M, a.K, a.cb_stride, a.cb_sizes[0], a.cb_sizes[1], a.cb_sizes[2], a.cb_sizes[3], a.scales, a.y);
  return hq_launch_status();
}
