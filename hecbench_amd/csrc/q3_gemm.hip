// Batched GPTQ 3-bit GEMM for gfx950 (fp16 activations, fp32 output):
//
//   out[m][n] = sum_k A[m][k] * (s[n]*q[k][n] - z[n])
//             = s[n] * sum_k A[m][k]*q[k][n]  -  z[n] * sum_k A[m][k]
//
// The reference benchmark has only the batch-1 matvec
// (src/quant3MatMul-hip/kernels.h in the HeCBench tree); this is the same
// arithmetic applied to up to 64 activation rows per pass on the matrix cores.
//
// As in the matvec, the packed codes are never converted: an AND turns a 32-bit
// window of the packed string into two subnormal-fp16 MFMA operands
// (q3_recipe.h).  The factor 2^pos of each operand slot is folded into the
// activations by a small pre-pass that also reorders them into operand-slot order
// ([k-group][mfma j][row][8 halves]), scales every row by a power of two so that
// the fold stays inside the fp16 normal range, and computes the row sums for the
// zero term.
// The main kernel streams the weights once: a workgroup (4 waves, one per SIMD) owns 128
// output columns and all of K and walks K in steps of 8 k-groups; each wave owns two
// k-groups of a step, loads their activation slices (from L2) and packed rows (from
// HBM) straight into registers three steps ahead, and multiplies 2 k-groups x 128
// columns x 64 rows per step with 32x32x16 fp16 MFMAs (fp32 accumulate).  There is
// no LDS traffic and no barrier in the loop.  The four waves' accumulators are
// summed through LDS at the end and scale/zero are applied once per output.
#include <mutex>

#include "hq_internal.h"
#include "q3_recipe.h"

namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef float f4v __attribute__((ext_vector_type(4)));
typedef float f2v __attribute__((ext_vector_type(2)));
typedef uint32_t u4v __attribute__((ext_vector_type(4)));

constexpr int kWaves = 4;       // one per SIMD, up to 512 registers each
constexpr int kStepGroups = 8;  // k-groups a workgroup consumes per step (two per wave)
constexpr int kDeep = 3;        // steps of operands in flight ahead of the one being multiplied
constexpr int kBufs = kDeep + 1;
constexpr int kChunk = kStepGroups * kBufs;  // the pre-pass pads K to a multiple of this many k-groups
constexpr int kTileN = 128;     // output columns per workgroup
constexpr int kMaxSplitGroups = 256;  // workgroups of a K-split launch (tiles times splits)


// ---- pre-pass: activations -> operand-slot order, scaled by P[m] * 2^-pos; row sums ------------
// Ap[((g*4 + j)*Mpad + m)*8 + e] = A[m][32g + k] * P[m] * 2^-pos(k) with slot(k) = 8j + e; rows >= M and
// groups >= G hold zeros.  One block per row: it finds the row's largest magnitude and sum, picks the
// power of two P[m] that puts the largest magnitude in [2^14, 2^15), and re-orders its row.  The 2^-pos
// of an operand slot (pos <= 7) then leaves every entry within 2^21 of its row's largest an fp16 normal
// number, i.e. exactly the input's mantissa; the main kernel's epilogue divides by P[m] again.  (Without
// P[m] the slot factor alone pushed activations below 2^-7 into the fp16 subnormals.)
__global__ __launch_bounds__(256) void q3_gemm_prep(const _Float16* __restrict__ A, _Float16* __restrict__ Ap,
                                                   float* __restrict__ rowsum, float* __restrict__ rowinv,
                                                   int M, int K, int Mpad, int Gpad) {
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int G = K >> 5;
  // Eight consecutive rows share the 128-byte lines of Ap; workgroups b, b + 8, b + 16, ... run on the same
  // XCD, so the rows of a line go to workgroups of one XCD and its L2 writes whole lines back instead of
  // eight XCDs writing an eighth of every line each.
  // (64 workgroups whatever Mpad; those beyond Mpad have nothing to do).
  const int m = (blockIdx.x & 7) * 8 + (blockIdx.x >> 3);
  if (m >= Mpad) return;
  __shared__ float s_sum[4], s_max[4];
  float sum = 0.f, amax = 0.f;
  if (m < M) {
    const u4v* src = reinterpret_cast<const u4v*>(A + (size_t)m * K);
    const int n16 = K >> 3;
    for (int i0 = 0; i0 < n16; i0 += 4 * 256) {
      u4v raw[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int i = i0 + u * 256 + (int)threadIdx.x;
        raw[u] = src[min(i, n16 - 1)];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int i = i0 + u * 256 + (int)threadIdx.x;
        const _Float16* in = reinterpret_cast<const _Float16*>(&raw[u]);
        float s8 = 0.f, m8 = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          s8 += (float)in[e];
          m8 = fmaxf(m8, fabsf((float)in[e]));
        }
        sum += i < n16 ? s8 : 0.f;
        amax = i < n16 ? fmaxf(amax, m8) : amax;
      }
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    sum += __shfl_xor(sum, off);
    amax = fmaxf(amax, __shfl_xor(amax, off));
  }
  if (lane == 0) { s_sum[wv] = sum; s_max[wv] = amax; }
  __syncthreads();
  amax = fmaxf(fmaxf(s_max[0], s_max[1]), fmaxf(s_max[2], s_max[3]));
  // P = 2^(14 - floor(log2 amax)); an all-zero or non-finite row keeps P = 1 (fp16 magnitudes span 2^-24 .. 2^16)
  const int ex = (int)((__float_as_uint(amax) >> 23) & 255u) - 127;
  const int pe = (amax > 0.f && ex < 128) ? 14 - ex : 0;
  if (threadIdx.x == 0) {
    rowsum[m] = (s_sum[0] + s_sum[1]) + (s_sum[2] + s_sum[3]);
    rowinv[m] = __uint_as_float((uint32_t)(127 - pe) << 23);
  }
  // second pass over the row (it is in the caches now): thread = k-group
  for (int g = threadIdx.x; g < Gpad; g += 256) {
    _Float16 out[32];
#pragma unroll
    for (int i = 0; i < 32; ++i) out[i] = (_Float16)0.f;
    if (m < M && g < G) {
      const u4v* src = reinterpret_cast<const u4v*>(A + (size_t)m * K + 32 * g);
      u4v raw[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) raw[i] = src[i];
      const _Float16* in = reinterpret_cast<const _Float16*>(raw);
#pragma unroll
      for (int k = 0; k < 32; ++k)
        out[hq_q3::slot_of(k)] =
            (_Float16)((float)in[k] * __uint_as_float((uint32_t)(127 + pe - hq_q3::pos_of(k)) << 23));
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      u4v* dst = reinterpret_cast<u4v*>(Ap + ((size_t)(g * 4 + j) * Mpad + m) * 8);
      *dst = *reinterpret_cast<const u4v*>(out + 8 * j);
    }
  }
}

// Sixteen two-field registers of one column's k-group (see q3_recipe.h).
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

struct GemmArgs {
  const uint32_t* w;
  const u4v* Ap;        // [Gpad][4][Mpad] 16-byte operand chunks
  const float* rowsum;  // [Mpad]
  const float* rowinv;  // [Mpad] 1 / P[m]
  const float* scales;
  const float* zeros;
  float* out;           // [M][N]
  float* partial;       // K split: [tile][split][Mpad][128] raw sums of a workgroup
  int M, K, N, Gpad;
  int nsplit, spp;      // workgroups per column tile, steps per workgroup (a multiple of kBufs)
  unsigned flags;
};

// ---- main kernel -----------------------------------------------------------------------------------
// One wave per SIMD with up to 512 registers (the accumulators of 64 rows x 128 columns take 128 of them,
// in the accumulation registers), kDeep steps of operands in flight.  The buffers rotate by unrolling,
// never by copying: a register move out of a buffer whose load is still in flight would wait for it.
// (Two waves per SIMD with one step in flight measured 38.4 us at M=64, K=8192, N=28672 against 36.2; the
// depth itself, 2 to 5 steps, changes little: what a workgroup moves through its CU's L1 - all of the
// re-ordered activations, 1 MB, next to 0.4 MB of weights - bounds the loop, not the latency.)
template <int MB>  // 32-row blocks of activations
__global__ __launch_bounds__(kWaves * 64) void q3_gemm_kernel(const uint32_t* w_, const u4v* Ap_, int M_, int K_, int N_,
                                                             int Gpad_, int nsplit_, int spp_, unsigned flags_,
                                                             const float* scales_, const float* zeros_,
                                                             const float* rowsum_, const float* rowinv_, float* out_,
                                                             float* partial_) {
  // leading scalars, not the struct: the first 14 dwords of the arguments arrive preloaded in scalar registers
  GemmArgs a;
  a.w = w_; a.Ap = Ap_; a.rowsum = rowsum_; a.rowinv = rowinv_; a.scales = scales_; a.zeros = zeros_; a.out = out_;
  a.partial = partial_; a.M = M_; a.K = K_; a.N = N_; a.Gpad = Gpad_; a.nsplit = nsplit_; a.spp = spp_; a.flags = flags_;
  constexpr int Mpad = 32 * MB;
  extern __shared__ u4v lds[];  // used by the final reduction only
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int nl = lane & 31, kb = lane >> 5;
  const int G = a.K >> 5;
  // K split: workgroup (tile, split) takes steps t_begin .. t_begin + nsteps - 1 (both multiples of kBufs:
  // Gpad is a multiple of 32 k-groups) and leaves its raw sums to hq_q3_gemm_reduce
  const int t_begin = blockIdx.y * a.spp;
  const int nsteps = min(a.spp, a.Gpad / kStepGroups - t_begin);
  const int col0 = blockIdx.x * kTileN;
  const int col = min(col0 + 4 * nl, a.N - 4);
  const size_t row_stride = (size_t)a.N;
  const int n_out = col0 + 4 * nl;
  f4v sc = {0.f, 0.f, 0.f, 0.f}, zr = {0.f, 0.f, 0.f, 0.f};
  if (n_out < a.N) {
    sc = *reinterpret_cast<const f4v*>(a.scales + n_out);
    zr = *reinterpret_cast<const f4v*>(a.zeros + n_out);
  }
  // final reduction: a wave finishes rows 8*wv .. 8*wv+7 of every 32-row block, half wave kb four of them
  float rs[MB][4], ri[MB][4];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      rs[mb][j] = a.rowsum[mb * 32 + 8 * wv + 4 * kb + j];
      ri[mb][j] = a.rowinv[mb * 32 + 8 * wv + 4 * kb + j] * 16777216.f;  // 2^24: the unit of the code operands
    }

  f16v acc[MB][4];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mb][q][i] = 0.f;

  const u4v* ap_lane = a.Ap + (size_t)((2 * wv + kb) * 4) * Mpad + nl;
  auto load_step = [&](int tl, u4v (&A)[4][MB], uint32_t (&wr)[3][4]) {
    const int t = t_begin + tl;
    const int g = min(t * kStepGroups + 2 * wv + kb, G - 1);  // padded groups: any valid weights, zero activations
#pragma unroll
    for (int j = 0; j < 3; ++j) {
      const u4v v = __builtin_nontemporal_load(
          reinterpret_cast<const u4v*>(a.w + (size_t)(3 * g + j) * row_stride + col));
      wr[j][0] = v.x; wr[j][1] = v.y; wr[j][2] = v.z; wr[j][3] = v.w;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) A[j][mb] = ap_lane[(size_t)t * (kStepGroups * 4 * Mpad) + j * Mpad + mb * 32];
  };
  auto compute = [&](const u4v (&A)[4][MB], const uint32_t (&wr)[3][4]) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      uint32_t f[16];
      unpack16(wr[0][q], wr[1][q], wr[2][q], f);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const u4v bv = {f[4 * j], f[4 * j + 1], f[4 * j + 2], f[4 * j + 3]};
        const h8 B = __builtin_bit_cast(h8, bv);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
          acc[mb][q] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h8, A[j][mb]), B, acc[mb][q], 0, 0, 0);
      }
    }
  };

  u4v Ab[kBufs][4][MB];
  uint32_t wb[kBufs][3][4];
#pragma unroll
  for (int b = 0; b < kDeep; ++b) load_step(min(b, nsteps - 1), Ab[b], wb[b]);
  for (int t0 = 0; t0 < nsteps; t0 += kBufs) {
#pragma unroll
    for (int b = 0; b < kBufs; ++b) {
      // step t0 + b is multiplied from buffer b while step t0 + b + kDeep goes into the buffer freed one
      // step ago (the last trips re-read the last step instead of branching)
      load_step(min(t0 + b + kDeep, nsteps - 1), Ab[(b + kDeep) % kBufs], wb[(b + kDeep) % kBufs]);
      __builtin_amdgcn_sched_barrier(0);
      compute(Ab[b], wb[b]);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  __syncthreads();

  float* red = reinterpret_cast<float*>(lds);
  constexpr int REGION = 32 * kTileN;
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    if (mb) __syncthreads();
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int r = (i >> 2) * 8 + kb * 4 + (i & 3);
      const f4v v = {acc[mb][0][i], acc[mb][1][i], acc[mb][2][i], acc[mb][3][i]};
      *reinterpret_cast<f4v*>(red + (size_t)wv * REGION + r * kTileN + 4 * nl) = v;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int r = 8 * wv + 4 * kb + j;
      const int m = mb * 32 + r;
      f4v v = *reinterpret_cast<const f4v*>(red + r * kTileN + 4 * nl);
#pragma unroll
      for (int w = 1; w < kWaves; ++w)
        v += *reinterpret_cast<const f4v*>(red + (size_t)w * REGION + r * kTileN + 4 * nl);
      if (a.nsplit > 1) {
        f4v* dst = reinterpret_cast<f4v*>(a.partial + (((size_t)blockIdx.x * a.nsplit + blockIdx.y) * Mpad + m) * kTileN) + nl;
        __builtin_nontemporal_store(v, dst);
      } else if (m < a.M && n_out < a.N) {
        f4v o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = sc[e] * (v[e] * ri[mb][j]) - zr[e] * rs[mb][j];
        f4v* dst = reinterpret_cast<f4v*>(a.out + (size_t)m * a.N + n_out);
        if (a.flags & HQ_FLAG_ACCUMULATE) { const f4v old = *dst; o += old; }
        *dst = o;
      }
    }
  }
}

// K split: sums the workgroups' raw sums of a tile in split order and applies scale, zero and the row's power
// of two.  A thread owns four adjacent columns of one row.
__global__ __launch_bounds__(256) void q3_gemm_reduce(GemmArgs a, int Mpad) {
  const int tile = blockIdx.x;
  const int nl = threadIdx.x & 31;
  const int n_out = tile * kTileN + 4 * nl;
  if (n_out >= a.N) return;
  const f4v sc = *reinterpret_cast<const f4v*>(a.scales + n_out);
  const f4v zr = *reinterpret_cast<const f4v*>(a.zeros + n_out);
  for (int m = blockIdx.y * 8 + (threadIdx.x >> 5); m < a.M; m += gridDim.y * 8) {
    const float* p = a.partial + (((size_t)tile * a.nsplit) * Mpad + m) * kTileN + 4 * nl;
    f4v v = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < a.nsplit; s0 += 8) {  // eight loads in flight, added in split order
      f4v t[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int s = s0 + j < a.nsplit ? s0 + j : a.nsplit - 1;
        t[j] = __builtin_nontemporal_load(reinterpret_cast<const f4v*>(p + (size_t)s * Mpad * kTileN));
      }
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (s0 + j < a.nsplit) v += t[j];
    }
    const float ri = a.rowinv[m] * 16777216.f, rs = a.rowsum[m];
    f4v o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = sc[e] * (v[e] * ri) - zr[e] * rs;
    f4v* dst = reinterpret_cast<f4v*>(a.out + (size_t)m * a.N + n_out);
    if (a.flags & HQ_FLAG_ACCUMULATE) { const f4v old = *dst; o += old; }
    *dst = o;
  }
}

template <int MB>
int launch_gemm(const GemmArgs& a, hipStream_t stream) {
  const size_t smem = (size_t)kWaves * 32 * kTileN * 4;
  static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&q3_gemm_kernel<MB>),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
  if (attr != hipSuccess) return (int)attr;
  const int ntiles = (a.N + kTileN - 1) / kTileN;
  hipLaunchKernelGGL((q3_gemm_kernel<MB>), dim3(ntiles, a.nsplit), dim3(kWaves * 64), smem, stream, a.w, a.Ap, a.M, a.K,
                     a.N, a.Gpad, a.nsplit, a.spp, a.flags, a.scales, a.zeros, a.rowsum, a.rowinv, a.out, a.partial);
  int rc = hq_launch_status();
  if (rc != HQ_OK || a.nsplit == 1) return rc;
  hipLaunchKernelGGL(q3_gemm_reduce, dim3(ntiles, (a.M + 7) / 8 < 8 ? (a.M + 7) / 8 : 8), dim3(256), 0, stream, a, 32 * MB);
  return hq_launch_status();
}

}  // namespace

// Launch plan of the batched GEMM (host arithmetic only; the launch, the workspace reservation and the size
// query share it).  K split: column tiles alone leave most CUs idle when N is small (N = 4096: 32 tiles), so K
// is cut into as many ranges as give every CU a workgroup (at most kMaxSplitGroups of them, which is what the
// fixed scratch of the entry point that allocates nothing holds), each range a multiple of kBufs steps; the
// workgroups leave raw sums in the workspace and a second kernel adds them in split order (deterministic).
namespace {
struct GemmPlan {
  int Gpad, nsplit, spp;
  size_t ap_halves, partial_floats;
};
GemmPlan gemm_plan(int cus, int K, int N) {
  GemmPlan p;
  const int G = K / 32;
  p.Gpad = (G + kChunk - 1) / kChunk * kChunk;
  p.ap_halves = (size_t)p.Gpad * 4 * 64 * 8;
  const int ntiles = (N + kTileN - 1) / kTileN;
  const int nsteps = p.Gpad / kStepGroups;
  p.nsplit = (cus < kMaxSplitGroups ? cus : kMaxSplitGroups) / ntiles;
  if (p.nsplit > nsteps / kBufs) p.nsplit = nsteps / kBufs;
  if (p.nsplit < 1) p.nsplit = 1;
  p.spp = (nsteps + p.nsplit - 1) / p.nsplit;
  p.spp = (p.spp + kBufs - 1) / kBufs * kBufs;
  p.nsplit = (nsteps + p.spp - 1) / p.spp;
  p.partial_floats = p.nsplit > 1 ? (size_t)ntiles * p.nsplit * 64 * kTileN : 0;
  return p;
}
}  // namespace

int hq_q3_gemm_need(int cus, int K, int N, size_t* floats, size_t* counters) {
  const GemmPlan p = gemm_plan(cus, K, N);
  *floats = p.ap_halves / 2 + 128 + p.partial_floats;
  *counters = 1;
  return HQ_OK;
}

int hq_q3_gemm_launch(const void* x, const int32_t* qweight, const float* scales, const float* zeros, float* y,
                      int K, int N, int M, unsigned flags, hipStream_t stream, const HqQ3Scratch* fixed) {
  if (((uintptr_t)x & 15) || (K & 7)) return HQ_ERR_MISALIGNED;
  if (((uintptr_t)scales & 15) || ((uintptr_t)zeros & 15) || ((uintptr_t)y & 15)) return HQ_ERR_MISALIGNED;
  const HqDevice* dev = nullptr;
  int rc = hq_current_device(&dev);
  if (rc != HQ_OK) return rc;
  const GemmPlan plan = gemm_plan(dev->cus, K, N);
  const int Gpad = plan.Gpad, nsplit = plan.nsplit, spp = plan.spp;
  const size_t ap_halves = plan.ap_halves, partial_floats = plan.partial_floats;
  _Float16* Ap;
  float *rowsum, *rowinv, *partial = nullptr;
  if (fixed) {
    if (ap_halves / 2 > fixed->partial_floats || partial_floats > fixed->sums_floats) return HQ_ERR_TOO_LARGE;
    Ap = reinterpret_cast<_Float16*>(fixed->partial);
    rowsum = fixed->rows;
    rowinv = fixed->rows + 64;
    partial = fixed->sums;
  } else {
    HqWorkspace ws;
    rc = hq_get_workspace(stream, ap_halves / 2 + 128 + partial_floats, 1, &ws);
    if (rc != HQ_OK) return rc;
    Ap = reinterpret_cast<_Float16*>(ws.partial);
    rowsum = ws.partial + ap_halves / 2;
    rowinv = rowsum + 64;
    partial = rowsum + 128;
  }
  // up to 64 rows per pass over the weights
  for (int m0 = 0; m0 < M; m0 += 64) {
    const int Mb = M - m0 < 64 ? M - m0 : 64;
    const int MB = Mb > 32 ? 2 : 1;
    const int Mpad = 32 * MB;
    const _Float16* A = reinterpret_cast<const _Float16*>(x) + (size_t)m0 * K;
    hipLaunchKernelGGL(q3_gemm_prep, dim3(64), dim3(256), 0, stream, A, Ap, rowsum, rowinv, Mb, K, Mpad, Gpad);
    rc = hq_launch_status();
    if (rc != HQ_OK) return rc;
    GemmArgs a;
    a.w = reinterpret_cast<const uint32_t*>(qweight);
    a.Ap = reinterpret_cast<const u4v*>(Ap);
    a.rowsum = rowsum;
    a.rowinv = rowinv;
    a.scales = scales;
    a.zeros = zeros;
    a.out = y + (size_t)m0 * N;
    a.M = Mb; a.K = K; a.N = N; a.Gpad = Gpad; a.flags = flags;
    a.partial = partial; a.nsplit = nsplit; a.spp = spp;
    rc = MB == 2 ? launch_gemm<2>(a, stream) : launch_gemm<1>(a, stream);
    if (rc != HQ_OK) return rc;
  }
  return HQ_OK;
}

// ---- the entry point that allocates nothing ----------------------------------------------------
// Its scratch (split-K partial sums and arrival counters of the matvec, re-ordered activations, row
// sums, row scales and K-split sums of the batched GEMM) lives in a fixed device array instead of the stream's
// workspace.  Every GPU holds its own copy of the array at its own address, resolved once per device.
namespace {
constexpr size_t kScratchPartialBytes = (size_t)2 << 20;  // 2 MiB: K <= 16384 batched, 8192 partial rows of 64 floats
constexpr size_t kScratchRowBytes = 1024;                 // 128 floats used
constexpr size_t kScratchCounterBytes = 64 * 1024 - kScratchRowBytes;
constexpr size_t kScratchSumBytes = (size_t)kMaxSplitGroups * 64 * kTileN * sizeof(float);  // 8 MiB: the GEMM's K split
constexpr size_t kScratchBytes = kScratchPartialBytes + kScratchRowBytes + kScratchCounterBytes + kScratchSumBytes;
}  // namespace
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[kMaxDevices];  // device address of `scratch` on each device, null until resolved

int scratch_of_current_device(void** out) {
  int dev = 0;
  HQ_HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return HQ_ERR_UNSUPPORTED_DEVICE;
  std::lock_guard<std::mutex> lk(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    HQ_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return (int)hipErrorInvalidSymbol;
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return HQ_OK;
}
}  // namespace

int hq_noalloc_setup(void) {
  void* p = nullptr;
  return scratch_of_current_device(&p);
}

extern "C" int hq_q3_matvec_noalloc(const void* x, int x_dtype, const int32_t* qweight, const float* scales,
                                    const float* zeros, float* y, int K, int N, int batch_M, unsigned flags,
                                    void* stream) {
  void* base = nullptr;
  int rc = scratch_of_current_device(&base);
  if (rc != HQ_OK) return rc;
  unsigned char* b = static_cast<unsigned char*>(base);
  HqQ3Scratch s;
  s.partial = reinterpret_cast<float*>(b);
  s.partial_floats = kScratchPartialBytes / sizeof(float);
  s.rows = reinterpret_cast<float*>(b + kScratchPartialBytes);
  s.counters = reinterpret_cast<unsigned*>(b + kScratchPartialBytes + kScratchRowBytes);
  s.ncounters = kScratchCounterBytes / sizeof(unsigned);
  s.sums = reinterpret_cast<float*>(b + kScratchPartialBytes + kScratchRowBytes + kScratchCounterBytes);
  s.sums_floats = kScratchSumBytes / sizeof(float);
  return hq_q3_matvec_impl(x, x_dtype, qweight, scales, zeros, y, K, N, batch_M, flags, (hipStream_t)stream, &s);
}
