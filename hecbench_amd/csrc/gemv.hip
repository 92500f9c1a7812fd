// Dense and weight-quantised matrix-vector products for gfx950 (fp16 vector, fp16 result):
//
//   fp16 : res[r] = f16( sum_j mat[r][j] * vec[j] )
//   int8 : res[r] = f16( scale * sum_j (mat[r][j] - zp) * vec[j] ),  mat int8
//   int4 : res[r] = f16( scale * sum_j (nib[r][j] - zp) * vec[j] ),  two codes per byte, code j in the
//          low nibble of byte j/2 for even j and in the high nibble for odd j
//
// Replaces gemv_fp16 / gemv_quantized_int8 / gemv_quantized_int4 and their launchers
// (src/gemv-hip/kernels.h:66-311, src/gemv-hip/gemv.cu:10-133 in the HeCBench tree).  Like
// the reference, scale and zero point are rounded to fp16 before use and sums are kept in
// fp32; unlike it, the zero point is taken out once per row ( sum (q - zp) v = sum q v -
// zp sum v ), which leaves a sign-extending conversion and one fused multiply-add per int8 weight and
// 9 instructions per 8 int4 weights.
//
// A wave owns R consecutive rows and walks the columns in steps of 64 lanes x 16 bytes of
// matrix per row (1 KB contiguous per wave and row); the matching piece of the vector is
// loaded once and used for the R rows.  A 4-bit code left in place in the low bits of
// a 16-bit half is the fp16 subnormal code * 2^-24, so `word >> 4i & 0x000f000f` is a pair
// of operands for a two-term fp16 dot product with fp32 accumulation (exact products).
// Lanes are combined with DPP butterflies; one rounding to fp16 at the end.
#include "hq_internal.h"

namespace {

typedef _Float16 h2v __attribute__((ext_vector_type(2)));
typedef uint32_t u4v __attribute__((ext_vector_type(4)));

__device__ __forceinline__ h2v as_h2(uint32_t v) { return __builtin_bit_cast(h2v, v); }

template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float lane_f(float v, int l) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), l));
}
__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_f<0xB1>(v);   // quad_perm [1,0,3,2]
  v += dpp_f<0x4E>(v);   // quad_perm [2,3,0,1]
  v += dpp_f<0x141>(v);  // row_half_mirror
  v += dpp_f<0x140>(v);  // row_mirror
  return (lane_f(v, 0) + lane_f(v, 16)) + (lane_f(v, 32) + lane_f(v, 48));
}

enum { kF16 = 0, kI8 = 1, kI4 = 2 };

struct GemvArgs {
  const char* mat;
  const u4v* vec;  // fp16, 16-byte units
  _Float16* res;
  int rows, n;
  float scale, zp;  // already rounded to fp16 precision
};

template <int MODE> struct Geom;
template <> struct Geom<kF16> { static constexpr int kPerUnit = 8, kVecUnits = 1; };   // weights per 16-byte unit
template <> struct Geom<kI8> { static constexpr int kPerUnit = 16, kVecUnits = 2; };
template <> struct Geom<kI4> { static constexpr int kPerUnit = 32, kVecUnits = 4; };

// Sum of the sixteen-byte vector piece (eight halves) in fp32.
__device__ __forceinline__ float sum8(u4v v, float acc) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
  const h2v one = {(_Float16)1.f, (_Float16)1.f};
#pragma unroll
  for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_fdot2(as_h2(w[i]), one, acc, false);
  return acc;
}

// One step of a wave: R matrix units m[r] (16 bytes per lane and row) against the matching pieces v[] of the
// vector.  SUM: also add the pieces' elements to vsum (needed once per wave, not once per row group).
template <int MODE, int R, bool SUM>
__device__ __forceinline__ void gemv_step(const u4v (&m)[R], const u4v (&v)[Geom<MODE>::kVecUnits], float (&acc)[R],
                                          float (&acc16)[R], float& vsum) {
  using G = Geom<MODE>;
  uint32_t vw[4 * G::kVecUnits];
#pragma unroll
  for (int i = 0; i < G::kVecUnits; ++i) { vw[4 * i] = v[i].x; vw[4 * i + 1] = v[i].y; vw[4 * i + 2] = v[i].z; vw[4 * i + 3] = v[i].w; }

  if (MODE == kF16) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const uint32_t mw[4] = {m[r].x, m[r].y, m[r].z, m[r].w};
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[r] = __builtin_amdgcn_fdot2(as_h2(mw[i]), as_h2(vw[i]), acc[r], false);
    }
  } else if (MODE == kI8) {
    if (SUM) {
#pragma unroll
      for (int i = 0; i < 2; ++i) vsum = sum8(v[i], vsum);
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const uint32_t mw[4] = {m[r].x, m[r].y, m[r].z, m[r].w};
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        // bytes 0..3 of word d are columns 4d..4d+3: vector halves vw[2d].lo, .hi, vw[2d+1].lo, .hi
        const h2v x01 = as_h2(vw[2 * d]), x23 = as_h2(vw[2 * d + 1]);
        acc[r] = fmaf((float)x01[0], (float)(int8_t)(mw[d] & 0xffu), acc[r]);
        acc[r] = fmaf((float)x01[1], (float)(int8_t)((mw[d] >> 8) & 0xffu), acc[r]);
        acc[r] = fmaf((float)x23[0], (float)(int8_t)((mw[d] >> 16) & 0xffu), acc[r]);
        acc[r] = fmaf((float)x23[1], (float)(int8_t)(mw[d] >> 24), acc[r]);
      }
    }
  } else {
    if (SUM) {
#pragma unroll
      for (int i = 0; i < 4; ++i) vsum = sum8(v[i], vsum);
    }
    // word d holds columns 8d..8d+7 in nibbles 0..7; `(w >> 4i) & 0x000f000f` pairs columns
    // i and i+4, so the vector halves are paired the same way once for all rows
    uint32_t pv[4][4];
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      pv[d][0] = __builtin_amdgcn_perm(vw[4 * d + 2], vw[4 * d], 0x05040100u);      // v0 v4
      pv[d][1] = __builtin_amdgcn_perm(vw[4 * d + 2], vw[4 * d], 0x07060302u);      // v1 v5
      pv[d][2] = __builtin_amdgcn_perm(vw[4 * d + 3], vw[4 * d + 1], 0x05040100u);  // v2 v6
      pv[d][3] = __builtin_amdgcn_perm(vw[4 * d + 3], vw[4 * d + 1], 0x07060302u);  // v3 v7
    }
    // nibbles 1 and 3 are masked where they stand, four bits up, which makes them 16 times too large:
    // they go to a second sum that is divided by 16 at the end (5 instead of 7 shift / mask
    // instructions per word)
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const uint32_t mw[4] = {m[r].x, m[r].y, m[r].z, m[r].w};
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const uint32_t up = mw[d] >> 8;
        acc[r] = __builtin_amdgcn_fdot2(as_h2(mw[d] & 0x000f000fu), as_h2(pv[d][0]), acc[r], false);
        acc16[r] = __builtin_amdgcn_fdot2(as_h2(mw[d] & 0x00f000f0u), as_h2(pv[d][1]), acc16[r], false);
        acc[r] = __builtin_amdgcn_fdot2(as_h2(up & 0x000f000fu), as_h2(pv[d][2]), acc[r], false);
        acc16[r] = __builtin_amdgcn_fdot2(as_h2(up & 0x00f000f0u), as_h2(pv[d][3]), acc16[r], false);
      }
    }
  }
}

// Lane sums, zero point and scale, one rounding to fp16: rows row0 .. row0 + R - 1 of a wave.
template <int MODE, int R>
__device__ __forceinline__ void gemv_finish(const GemvArgs& a, int row0, const float (&acc)[R], const float (&acc16)[R],
                                            float vs) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    float s = wave_sum(MODE == kI4 ? fmaf(acc16[r], 0.0625f, acc[r]) : acc[r]);
    if (MODE == kI8) s = a.scale * (s - a.zp * vs);
    if (MODE == kI4) s = a.scale * (s * 16777216.f - a.zp * vs);  // codes were fp16 subnormals code * 2^-24
    if (lane == 0 && row0 + r < a.rows) a.res[row0 + r] = (_Float16)s;
  }
}

template <int MODE, int R>
__global__ __launch_bounds__(256) void gemv_kernel(const char* mat_, const u4v* vec_, _Float16* res_, int rows_, int n_, float scale_,
                                                  float zp_) {
  // leading scalars, not the struct: the arguments arrive preloaded in scalar registers
  GemvArgs a;
  a.mat = mat_; a.vec = vec_; a.res = res_; a.rows = rows_; a.n = n_; a.scale = scale_; a.zp = zp_;
  using G = Geom<MODE>;
  const int lane = threadIdx.x & 63;
  const int wave = (blockIdx.x * 256 + threadIdx.x) >> 6;
  const int row0 = wave * R;
  if (row0 >= a.rows) return;  // wave-uniform
  const int units = a.n / G::kPerUnit;  // 16-byte units per matrix row
  const size_t row_bytes = (size_t)units * 16;
  const u4v* rowp[R];
#pragma unroll
  for (int r = 0; r < R; ++r)
    rowp[r] = reinterpret_cast<const u4v*>(a.mat + (size_t)min(row0 + r, a.rows - 1) * row_bytes);

  float acc[R], acc16[R], vsum = 0.f;
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = acc16[r] = 0.f;

  for (int u = lane; u < units; u += 64) {
    u4v m[R];
#pragma unroll
    for (int r = 0; r < R; ++r) m[r] = __builtin_nontemporal_load(rowp[r] + u);
    u4v v[G::kVecUnits];
#pragma unroll
    for (int i = 0; i < G::kVecUnits; ++i) v[i] = a.vec[(size_t)u * G::kVecUnits + i];
    gemv_step<MODE, R, true>(m, v, acc, acc16, vsum);
  }

  gemv_finish<MODE, R>(a, row0, acc, acc16, MODE == kF16 ? 0.f : wave_sum(vsum));
}

// Rows cut across the waves of a workgroup.  On this part a stream moves fastest when every wave issues a
// few loads and ends - the wave launcher refills the compute units better than any loop (a plain read of 537 MB
// runs at 7.0 TB/s with one 128-bit load per thread and at 5.6 TB/s as a grid-stride loop) - so for long rows a
// workgroup of SPLIT waves shares R rows, every wave takes every SPLIT-th two-step piece of the columns,
// and the waves' sums meet in LDS in wave order (deterministic).
template <int MODE, int R, int SPLIT>
__global__ __launch_bounds__(SPLIT * 64) void gemv_split_kernel(const char* mat_, const u4v* vec_, _Float16* res_, int rows_,
                                                                int n_, float scale_, float zp_) {
  GemvArgs a;
  a.mat = mat_; a.vec = vec_; a.res = res_; a.rows = rows_; a.n = n_; a.scale = scale_; a.zp = zp_;
  using G = Geom<MODE>;
  __shared__ float part[SPLIT][R + 1];
  const int lane = threadIdx.x & 63;
  const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int row0 = blockIdx.x * R;
  const int units = a.n / G::kPerUnit;  // 16-byte units per matrix row
  const size_t row_bytes = (size_t)units * 16;
  const u4v* rowp[R];
#pragma unroll
  for (int r = 0; r < R; ++r)
    rowp[r] = reinterpret_cast<const u4v*>(a.mat + (size_t)min(row0 + r, a.rows - 1) * row_bytes);
  float acc[R], acc16[R], vsum = 0.f;
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = acc16[r] = 0.f;
  // pieces of two steps (2 KB per row) dealt to the waves in turn: neighbouring waves start 2 KB apart
  // whatever the row length (waves 4 KB apart measured 97 against 76 us at 16384 x 16384)
  for (int u0 = wv * 128; u0 < units; u0 += SPLIT * 128) {
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      const int u = u0 + st * 64 + lane;
      if (u < units) {
        u4v m[R];
#pragma unroll
        for (int r = 0; r < R; ++r) m[r] = __builtin_nontemporal_load(rowp[r] + u);
        u4v v[G::kVecUnits];
#pragma unroll
        for (int i = 0; i < G::kVecUnits; ++i) v[i] = a.vec[(size_t)u * G::kVecUnits + i];
        gemv_step<MODE, R, true>(m, v, acc, acc16, vsum);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const float s = wave_sum(MODE == kI4 ? fmaf(acc16[r], 0.0625f, acc[r]) : acc[r]);
    if (lane == 0) part[wv][r] = s;
  }
  if (MODE != kF16) {
    const float vs = wave_sum(vsum);
    if (lane == 0) part[wv][R] = vs;
  }
  __syncthreads();
  if (threadIdx.x < R && row0 + (int)threadIdx.x < a.rows) {
    const int r = threadIdx.x;
    float s = 0.f, vs = 0.f;
#pragma unroll
    for (int w = 0; w < SPLIT; ++w) {
      s += part[w][r];
      if (MODE != kF16) vs += part[w][R];
    }
    if (MODE == kI8) s = a.scale * (s - a.zp * vs);
    if (MODE == kI4) s = a.scale * (s * 16777216.f - a.zp * vs);  // codes were fp16 subnormals code * 2^-24
    a.res[row0 + r] = (_Float16)s;
  }
}

// The vector in LDS, the workgroups persistent.  A CU returns its loads in issue order and holds about
// 64 KB of them, whichever cache serves them: every piece of the vector a wave loads next to its matrix
// rows (as many bytes as the rows themselves for int8 with two rows per wave and int4 with four) takes a
// place in that queue from the matrix.  Here a workgroup of sixteen waves copies the vector into LDS once
// (piece i of matrix unit u at [i][u], so that a wave's reads of one piece are contiguous) and then walks
// over groups of R rows, one group per wave and trip, with nothing but the matrix in the load queue.
// Units between the pieces of the vector in LDS: the row length rounded up to 8 / kVecUnits past a multiple of
// eight units.  The copy writes piece i of unit u from consecutive lanes (u = t / kVecUnits, i = t % kVecUnits);
// a 128-bit LDS store is served eight lanes at a time over 128 bytes of banks, and with the pieces a multiple
// of 128 bytes apart the pieces of one unit met in a bank.
template <int MODE>
__host__ __device__ constexpr int gemv_lds_stride(int units) {
  return (units + 7) / 8 * 8 + 8 / Geom<MODE>::kVecUnits % 8;
}

template <int MODE, int R>
__global__ __launch_bounds__(1024) void gemv_lds_kernel(const char* mat_, const u4v* vec_, _Float16* res_, int rows_, int n_, float scale_,
                                                       float zp_, int groups) {
  // leading scalars, not the struct: the arguments arrive preloaded in scalar registers
  GemvArgs a;
  a.mat = mat_; a.vec = vec_; a.res = res_; a.rows = rows_; a.n = n_; a.scale = scale_; a.zp = zp_;
  using G = Geom<MODE>;
  extern __shared__ u4v vl[];
  const int lane = threadIdx.x & 63;
  const int units = a.n / G::kPerUnit;  // 16-byte units per matrix row
  const int vstride = gemv_lds_stride<MODE>(units);
  const size_t row_bytes = (size_t)units * 16;
  const int waves = gridDim.x * 16;
  int grp = blockIdx.x * 16 + (threadIdx.x >> 6);

  auto rows_of = [&](int g, const u4v* (&rowp)[R]) {
#pragma unroll
    for (int r = 0; r < R; ++r)
      rowp[r] = reinterpret_cast<const u4v*>(a.mat + (size_t)min(g * R + r, a.rows - 1) * row_bytes);
  };
  // the first matrix units are on their way while the vector is copied
  const u4v* rowp[R];
  u4v m[R];
  rows_of(min(grp, groups - 1), rowp);
#pragma unroll
  for (int r = 0; r < R; ++r) m[r] = __builtin_nontemporal_load(rowp[r] + min(lane, units - 1));
  for (int t = threadIdx.x; t < units * G::kVecUnits; t += 1024) {
    const int u = t / G::kVecUnits, i = t % G::kVecUnits;
    vl[i * vstride + u] = a.vec[t];
  }
  __syncthreads();

  float vs = 0.f;
  bool first = true;
  for (; grp < groups; grp += waves) {
    float acc[R], acc16[R], vsum = 0.f;
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = acc16[r] = 0.f;
    for (int u = lane; u < units; u += 64) {
      u4v cur[R], v[G::kVecUnits];
#pragma unroll
      for (int r = 0; r < R; ++r) cur[r] = m[r];
      // the next step's units (the next group's first ones at the end of a row) before this step's arithmetic
      if (u + 64 >= units) rows_of(min(grp + waves, groups - 1), rowp);
      const int un = u + 64 < units ? u + 64 : min(lane, units - 1);
#pragma unroll
      for (int r = 0; r < R; ++r) m[r] = __builtin_nontemporal_load(rowp[r] + un);
#pragma unroll
      for (int i = 0; i < G::kVecUnits; ++i) v[i] = vl[i * vstride + u];
      if (first) gemv_step<MODE, R, true>(cur, v, acc, acc16, vsum);
      else gemv_step<MODE, R, false>(cur, v, acc, acc16, vsum);
    }
    if (first && MODE != kF16) vs = wave_sum(vsum);
    first = false;
    gemv_finish<MODE, R>(a, grp * R, acc, acc16, vs);
  }
}

constexpr size_t kMaxVectorLds = 128 * 1024;  // bytes of the vector the LDS kernel takes (n <= 65536)

template <int MODE, int R>
int launch_gemv_lds(const GemvArgs& a, int cus, hipStream_t stream) {
  const size_t smem = (size_t)gemv_lds_stride<MODE>(a.n / Geom<MODE>::kPerUnit) * Geom<MODE>::kVecUnits * 16;
  static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemv_lds_kernel<MODE, R>),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxVectorLds + 1024);
  if (attr != hipSuccess) return (int)attr;
  const int groups = (a.rows + R - 1) / R;
  const int wgs = (groups + 15) / 16;
  hipLaunchKernelGGL((gemv_lds_kernel<MODE, R>), dim3(wgs < cus ? wgs : cus), dim3(1024), smem, stream, a.mat, a.vec, a.res, a.rows, a.n, a.scale, a.zp, groups);
  return hq_launch_status();
}

template <int MODE>
int launch_gemv(const void* mat, const void* vec, void* res, int rows, int n, float scale, float zp,
                hipStream_t stream) {
  if (!mat || !vec || !res) return HQ_ERR_NULL_POINTER;
  if (rows <= 0 || n <= 0 || (n % Geom<MODE>::kPerUnit)) return HQ_ERR_BAD_SHAPE;
  if (((uintptr_t)mat & 15) || ((uintptr_t)vec & 15) || ((uintptr_t)res & 1)) return HQ_ERR_MISALIGNED;
  const HqDevice* dev = nullptr;
  int rc = hq_current_device(&dev);
  if (rc != HQ_OK) return rc;
  GemvArgs a;
  a.mat = reinterpret_cast<const char*>(mat);
  a.vec = reinterpret_cast<const u4v*>(vec);
  a.res = reinterpret_cast<_Float16*>(res);
  a.rows = rows; a.n = n;
  a.scale = (float)(_Float16)scale;  // the reference rounds both to fp16 (src/gemv-hip/gemv.cu:18-19)
  a.zp = (float)(_Float16)zp;
  // several rows per wave (the vector piece is loaded and prepared once for them) once there are
  // enough rows to fill the chip with such waves
  // (int4 reads four times as many bytes of the vector per byte of the matrix as fp16: rows per wave pay
  // there even when they leave only eight waves per compute unit - 8192 x 28672: 33.1 us with one row per
  // wave, 25.0 with two, 20.6 with four; fp16 at 4096 x 16384: 23.7 us with one row, 28.0 with two)
  // The LDS kernel pays where a wave loads as many bytes of the vector as of the matrix and walks over several
  // row groups: int4 with four rows per wave (32768 x 8192 29.0 -> 24.2 us, 28672 x 8192 25.7 -> 22.5,
  // 16384 x 28672 41.7 -> 38.8, 16384 x 16384 25.8 -> 25.5); fp16 and int8 gain on some shapes and lose on
  // others (fp16 16384 x 16384 88.7 -> 83.0 us but 28672 x 8192 70.6 -> 79.0), fewer rows lose throughout.
  // HQ_GEMV_LDS: 0 never, 1 wherever the vector fits, unset: the rule above.
  // Rows cut across the waves of a workgroup: fp16 rows of 8192 elements or more, two steps of two rows per
  // wave (16384 x 16384: 88.7 -> 75.7 us = 7.1 TB/s; 28672 x 8192 70.5 -> 64.3; 8192 x 28672 73.8 -> 66.8;
  // 4096 x 16384 23.0 -> 21.0).  Other step counts per wave are worse, some much (four steps, i.e. waves that
  // start 4 KB apart: 97.5 us at 16384 x 16384), and int8 / int4 rows gain little or lose: they keep whole
  // rows per wave.  HQ_GEMV_SPLIT: 0 never, 4 / 8 / 16 that many waves per pair of rows, unset: this rule.
  {
    int split = hq_tune(HQ_TUNE_GEMV_SPLIT, -1);
    const int units = n / Geom<MODE>::kPerUnit;
    if (split < 0)  // (a forced choice between the two whole-row kernels below stands)
      split = (MODE == kF16 && units >= 1024 && hq_tune(HQ_TUNE_GEMV_LDS, -1) < 0) ? (units >= 2048 ? 16 : 8) : 0;
    const int groups = (rows + 1) / 2;
#define HQ_GEMV_SPLIT_CASE(S) \
    if (split == S) { \
      hipLaunchKernelGGL((gemv_split_kernel<MODE, 2, S>), dim3(groups), dim3(S * 64), 0, stream, a.mat, a.vec, a.res, a.rows, a.n, a.scale, a.zp); \
      return hq_launch_status(); \
    }
    HQ_GEMV_SPLIT_CASE(4) HQ_GEMV_SPLIT_CASE(8) HQ_GEMV_SPLIT_CASE(16)
#undef HQ_GEMV_SPLIT_CASE
  }
  const int lds = hq_tune(HQ_TUNE_GEMV_LDS, -1);
  const int full = dev->cus * 16;  // waves of a full launch of the LDS kernel
  if ((size_t)n * 2 <= kMaxVectorLds && (lds == 1 || (lds < 0 && MODE == kI4 && rows >= full * 4))) {
    if (rows >= full * 4) return launch_gemv_lds<MODE, 4>(a, dev->cus, stream);
    if (rows >= full * 2) return launch_gemv_lds<MODE, 2>(a, dev->cus, stream);
    return launch_gemv_lds<MODE, 1>(a, dev->cus, stream);
  }
  constexpr int RMAX = MODE == kI4 ? 4 : 2;
  constexpr int kMinWaves = MODE == kI4 ? 8 : 16;  // per compute unit
  if (rows >= dev->cus * kMinWaves * RMAX) {
    const int waves = (rows + RMAX - 1) / RMAX;
    hipLaunchKernelGGL((gemv_kernel<MODE, RMAX>), dim3((waves + 3) / 4), dim3(256), 0, stream, a.mat, a.vec, a.res, a.rows, a.n, a.scale, a.zp);
  } else if (RMAX > 2 && rows >= dev->cus * kMinWaves * 2) {
    const int waves = (rows + 1) / 2;
    hipLaunchKernelGGL((gemv_kernel<MODE, 2>), dim3((waves + 3) / 4), dim3(256), 0, stream, a.mat, a.vec, a.res, a.rows, a.n, a.scale, a.zp);
  } else {
    hipLaunchKernelGGL((gemv_kernel<MODE, 1>), dim3((rows + 3) / 4), dim3(256), 0, stream, a.mat, a.vec, a.res, a.rows, a.n, a.scale, a.zp);
  }
  return hq_launch_status();
}

}  // namespace

extern "C" int hq_gemv_fp16(const void* mat, const void* vec, void* res, int rows, int n, void* stream) {
  return launch_gemv<kF16>(mat, vec, res, rows, n, 1.f, 0.f, (hipStream_t)stream);
}
extern "C" int hq_gemv_int8(const int8_t* mat, const void* vec, void* res, int rows, int n, float scale,
                            float zero_point, void* stream) {
  return launch_gemv<kI8>(mat, vec, res, rows, n, scale, zero_point, (hipStream_t)stream);
}
extern "C" int hq_gemv_int4(const uint8_t* mat, const void* vec, void* res, int rows, int n, float scale,
                            float zero_point, void* stream) {
  return launch_gemv<kI4>(mat, vec, res, rows, n, scale, zero_point, (hipStream_t)stream);
}
