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
// ([k-group][mfma j][row][8 halves]) and computes the row sums for the zero term.
// The main kernel streams the weights once: a workgroup (8 waves) owns 128 output
// columns and all of K, walks K in chunks of 16 k-groups whose activation slices
// are double-buffered in LDS, and each wave multiplies 2 k-groups x 128 columns x
// 64 rows per chunk with 32x32x16 fp16 MFMAs (fp32 accumulate).  The eight waves'
// accumulators are summed through LDS at the end and scale/zero are applied once
// per output.
#include "hq_internal.h"
#include "q3_recipe.h"

namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef float f4v __attribute__((ext_vector_type(4)));
typedef float f2v __attribute__((ext_vector_type(2)));
typedef uint32_t u4v __attribute__((ext_vector_type(4)));

constexpr int kChunk = 16;   // k-groups per LDS chunk
constexpr int kWaves = 8;
constexpr int kTileN = 128;  // output columns per workgroup


// ---- pre-pass: activations -> operand-slot order, scaled by 2^-pos; row sums ----------------
// grid (Mpad), block 256.  Ap[((g*4 + j)*Mpad + m)*8 + e] = A[m][32g + k] * 2^-pos(k) with
// slot(k) = 8j + e; rows >= M and groups >= G hold zeros.
__global__ __launch_bounds__(256) void q3_gemm_prep(const _Float16* __restrict__ A, _Float16* __restrict__ Ap,
                                                   float* __restrict__ rowsum, int M, int K, int Mpad,
                                                   int Gpad) {
  const int m = blockIdx.x, tid = threadIdx.x;
  const int G = K >> 5;
  __shared__ float part[256];
  float sum = 0.f;
  for (int g = tid; g < Gpad; g += 256) {
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
      for (int k = 0; k < 32; ++k) {
        const float v = (float)in[k];
        sum += v;
        // exact power-of-two scaling (subnormal results lose bits below 2^-24 only)
        out[hq_q3::slot_of(k)] = (_Float16)(v * __uint_as_float((uint32_t)(127 - hq_q3::pos_of(k)) << 23));
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      u4v* dst = reinterpret_cast<u4v*>(Ap + ((size_t)(g * 4 + j) * Mpad + m) * 8);
      *dst = *reinterpret_cast<const u4v*>(out + 8 * j);
    }
  }
  part[tid] = sum;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) {
    if (tid < s) part[tid] += part[tid + s];
    __syncthreads();
  }
  if (tid == 0) rowsum[m] = part[0];
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
  const float* scales;
  const float* zeros;
  float* out;           // [M][N]
  int M, K, N, Gpad;
  unsigned flags;
};

template <int MB>  // 32-row blocks of activations
__global__ __launch_bounds__(kWaves * 64) void q3_gemm_kernel(GemmArgs a) {
  constexpr int Mpad = 32 * MB;
  constexpr int CHUNK_U4 = kChunk * 4 * Mpad;  // 16-byte units of one activation chunk
  constexpr int T = kWaves * 64;
  constexpr int COPY = CHUNK_U4 / T;           // 16-byte units each thread copies per chunk
  extern __shared__ u4v lds[];                 // 2 * CHUNK_U4 (double buffer); reused by the reduction

  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int nl = lane & 31, kb = lane >> 5;
  const int G = a.K >> 5;
  const int nchunks = a.Gpad / kChunk;
  const int col0 = blockIdx.x * kTileN;
  const int col = min(col0 + 4 * nl, a.N - 4);  // out-of-range columns re-read valid data, never stored
  const size_t row_stride = (size_t)a.N;

  f16v acc[MB][4];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mb][q][i] = 0.f;

  u4v stage[COPY];
  uint32_t wreg[3][4];
  auto load_chunk = [&](int ch) {
    const u4v* src = a.Ap + (size_t)ch * CHUNK_U4;
#pragma unroll
    for (int i = 0; i < COPY; ++i) stage[i] = src[tid + i * T];
    // this wave's two k-groups of the chunk: group index 2*wv + kb
    const int g = min(ch * kChunk + 2 * wv + kb, G - 1);  // padded groups: any valid weights, zero activations
    const uint32_t* p = a.w + (size_t)(3 * g) * row_stride + col;
#pragma unroll
    for (int j = 0; j < 3; ++j) {
      const u4v v = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(p + j * row_stride));
      wreg[j][0] = v.x; wreg[j][1] = v.y; wreg[j][2] = v.z; wreg[j][3] = v.w;
    }
  };
  auto store_chunk = [&](int buf) {
    u4v* dst = lds + buf * CHUNK_U4;
#pragma unroll
    for (int i = 0; i < COPY; ++i) dst[tid + i * T] = stage[i];
  };

  load_chunk(0);
  store_chunk(0);
  uint32_t wcur[3][4];
#pragma unroll
  for (int j = 0; j < 3; ++j)
#pragma unroll
    for (int q = 0; q < 4; ++q) wcur[j][q] = wreg[j][q];
  __syncthreads();

  for (int ch = 0; ch < nchunks; ++ch) {
    const bool more = ch + 1 < nchunks;
    if (more) load_chunk(ch + 1);  // global loads in flight during the MFMAs
    const u4v* abuf = lds + (ch & 1) * CHUNK_U4 + (size_t)((2 * wv + kb) * 4) * Mpad + nl;
    h8 A[4][MB];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) A[j][mb] = __builtin_bit_cast(h8, abuf[j * Mpad + mb * 32]);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      uint32_t f[16];
      unpack16(wcur[0][q], wcur[1][q], wcur[2][q], f);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const u4v bv = {f[4 * j], f[4 * j + 1], f[4 * j + 2], f[4 * j + 3]};
        const h8 B = __builtin_bit_cast(h8, bv);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
          acc[mb][q] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A[j][mb], B, acc[mb][q], 0, 0, 0);
      }
    }
    if (more) {
      store_chunk((ch + 1) & 1);
#pragma unroll
      for (int j = 0; j < 3; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) wcur[j][q] = wreg[j][q];
    }
    __syncthreads();
  }

  // ---- sum the eight waves' accumulators through LDS ------------------------------------------
  // D[row][col = nl]: register i of a lane holds row (i/4)*8 + kb*4 + i%4 of its 32-row block;
  // the four accumulators q of a lane are four adjacent output columns 4*nl + q.
  float* red = reinterpret_cast<float*>(lds);  // regions of [Mpad][128] floats
  constexpr int REGION = Mpad * kTileN;
  auto put = [&](int region) {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int m = mb * 32 + (i >> 2) * 8 + kb * 4 + (i & 3);
        f4v v = {acc[mb][0][i], acc[mb][1][i], acc[mb][2][i], acc[mb][3][i]};
        *reinterpret_cast<f4v*>(red + (size_t)region * REGION + m * kTileN + 4 * nl) = v;
      }
  };
  if (wv >= 4) put(wv - 4);
  __syncthreads();
  if (wv < 4) {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int m = mb * 32 + (i >> 2) * 8 + kb * 4 + (i & 3);
        const f4v v = *reinterpret_cast<const f4v*>(red + (size_t)wv * REGION + m * kTileN + 4 * nl);
        acc[mb][0][i] += v.x; acc[mb][1][i] += v.y; acc[mb][2][i] += v.z; acc[mb][3][i] += v.w;
      }
  }
  __syncthreads();
  if (wv < 4) put(wv);
  __syncthreads();
  // every wave finishes Mpad/8 rows: lane -> two adjacent columns
  const int n = col0 + 2 * lane;
  if (n < a.N) {  // N % 4 == 0 and n even: n + 1 < N as well
    const f2v sc = *reinterpret_cast<const f2v*>(a.scales + n);
    const f2v zr = *reinterpret_cast<const f2v*>(a.zeros + n);
#pragma unroll
    for (int r = 0; r < Mpad / kWaves; ++r) {
      const int m = wv * (Mpad / kWaves) + r;
      if (m >= a.M) break;
      f2v s = {0.f, 0.f};
#pragma unroll
      for (int region = 0; region < 4; ++region) {
        const f2v v = *reinterpret_cast<const f2v*>(red + (size_t)region * REGION + m * kTileN + 2 * lane);
        s.x += v.x; s.y += v.y;
      }
      const float rs = a.rowsum[m];
      f2v o = {sc.x * (s.x * 16777216.f) - zr.x * rs, sc.y * (s.y * 16777216.f) - zr.y * rs};
      f2v* dst = reinterpret_cast<f2v*>(a.out + (size_t)m * a.N + n);
      if (a.flags & HQ_FLAG_ACCUMULATE) { const f2v old = *dst; o.x += old.x; o.y += old.y; }
      *dst = o;
    }
  }
}

template <int MB>
int launch_gemm(const GemmArgs& a, hipStream_t stream) {
  constexpr int Mpad = 32 * MB;
  const size_t smem = (size_t)2 * kChunk * 4 * Mpad * 16;
  static_assert((size_t)4 * Mpad * kTileN * 4 <= (size_t)2 * kChunk * 4 * Mpad * 16, "reduction regions fit the chunk buffers");
  static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&q3_gemm_kernel<MB>),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
  if (attr != hipSuccess) return (int)attr;
  hipLaunchKernelGGL((q3_gemm_kernel<MB>), dim3((a.N + kTileN - 1) / kTileN), dim3(kWaves * 64), smem, stream, a);
  return hq_launch_status();
}

}  // namespace

int hq_q3_gemm_launch(const void* x, const int32_t* qweight, const float* scales, const float* zeros, float* y,
                      int K, int N, int M, unsigned flags, hipStream_t stream) {
  if (((uintptr_t)x & 15) || (K & 7)) return HQ_ERR_MISALIGNED;
  if (((uintptr_t)scales & 7) || ((uintptr_t)zeros & 7) || ((uintptr_t)y & 7)) return HQ_ERR_MISALIGNED;
  const int G = K / 32;
  const int Gpad = (G + kChunk - 1) / kChunk * kChunk;
  const size_t ap_halves = (size_t)Gpad * 4 * 64 * 8;
  HqWorkspace ws;
  int rc = hq_get_workspace(stream, ap_halves / 2 + 64, 1, &ws);
  if (rc != HQ_OK) return rc;
  _Float16* Ap = reinterpret_cast<_Float16*>(ws.partial);
  float* rowsum = ws.partial + ap_halves / 2;
  // up to 64 rows per pass over the weights
  for (int m0 = 0; m0 < M; m0 += 64) {
    const int Mb = M - m0 < 64 ? M - m0 : 64;
    const int MB = Mb > 32 ? 2 : 1;
    const int Mpad = 32 * MB;
    const _Float16* A = reinterpret_cast<const _Float16*>(x) + (size_t)m0 * K;
    hipLaunchKernelGGL(q3_gemm_prep, dim3(Mpad), dim3(256), 0, stream, A, Ap, rowsum, Mb, K, Mpad, Gpad);
    rc = hq_launch_status();
    if (rc != HQ_OK) return rc;
    GemmArgs a;
    a.w = reinterpret_cast<const uint32_t*>(qweight);
    a.Ap = reinterpret_cast<const u4v*>(Ap);
    a.rowsum = rowsum;
    a.scales = scales;
    a.zeros = zeros;
    a.out = y + (size_t)m0 * N;
    a.M = Mb; a.K = K; a.N = N; a.Gpad = Gpad; a.flags = flags;
    rc = MB == 2 ? launch_gemm<2>(a, stream) : launch_gemm<1>(a, stream);
    if (rc != HQ_OK) return rc;
  }
  return HQ_OK;
}
