// Blockwise 4-bit (NF4 / FP4) dequantisation to fp16 for gfx950.
//
//   out[2i]   = fp16_rn(table[packed[i] >> 4] * absmax[(2i)   / blocksize])
//   out[2i+1] = fp16_rn(table[packed[i] & 15] * absmax[(2i+1) / blocksize])
//
// Pure streaming, write-dominated (64 bytes out per 16 bytes in).  The 16-entry
// code book sits in LDS: 16 entries occupy 16 distinct banks, so lanes that hit
// the same bank always hit the same address (broadcast) and the lookups are
// conflict-free.  The multiply is a single fp32 operation followed by one
// round-to-nearest-even conversion, which is the bit-exact contract.
#include "hq_internal.h"

namespace {

typedef uint32_t u4v __attribute__((ext_vector_type(4)));
typedef _Float16 h2v __attribute__((ext_vector_type(2)));

// bitsandbytes NF4 code book (fp32 literals of the upstream library).
__constant__ float c_nf4[16] = {
    -1.0f, -0.6961928009986877f, -0.5250730514526367f, -0.39491748809814453f,
    -0.28444138169288635f, -0.18477343022823334f, -0.09105003625154495f, 0.0f,
    0.07958029955625534f, 0.16093020141124725f, 0.24611230194568634f,
    0.33791524171829224f, 0.44070982933044434f, 0.5626170039176941f,
    0.7229568362236023f, 1.0f};
// bitsandbytes FP4 decode tree: bit 3 sign, low bits {0, 1/192, 2/3, 1, 1/3, 1/2, 1/6, 1/4}.
__constant__ float c_fp4[16] = {
    0.0f, 0.005208333333f, 0.66666667f, 1.0f, 0.33333333f, 0.5f, 0.16666667f, 0.25f,
    -0.0f, -0.005208333333f, -0.66666667f, -1.0f, -0.33333333f, -0.5f, -0.16666667f, -0.25f};

// The contract is two roundings: an fp32 product, then fp32 -> fp16.  The empty asm
// pins the fp32 product in a register so that the compiler cannot merge multiply and
// conversion into one mixed-precision instruction, which rounds only once.
__device__ __forceinline__ float mul_rounded_f32(float a, float b) {
  float v = a * b;
  asm volatile("" : "+v"(v));
  return v;
}

// Streaming 128-bit store, write-through and non-temporal ("sc1 nt"): the line goes straight to memory
// and is not kept in the L2.  Measured on MI355X for a 33.5 MB write stream: 5.80 us against 6.46 us
// with nt alone and 7.04 us with plain stores; with the 9.4 MB of reads next to it 7.23 against 7.32 us.
__device__ __forceinline__ void store_stream(u4v* p, u4v v) { hq_store_stream(reinterpret_cast<hq_u4v*>(p), v); }

// The fp32 product as an instruction of its own (one rounding), so that the conversion to fp16 that follows
// is a second rounding: written as inline assembly, the compiler can neither fuse the two nor needs a copy.
__device__ __forceinline__ float mul_f32_own(float a, float b) {
  float r;
  asm("v_mul_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}

__device__ __forceinline__ uint32_t deq_pair(const float* tab, uint32_t byte, float a_hi, float a_lo) {
  // high nibble is the earlier element
  const float v0 = mul_rounded_f32(tab[byte >> 4], a_hi);
  const float v1 = mul_rounded_f32(tab[byte & 15u], a_lo);
  h2v h = {(_Float16)v0, (_Float16)v1};
  return __builtin_bit_cast(uint32_t, h);
}

// Main path.  A lane turns one packed 32-bit word (8 codes) into one 128-bit store,
// so every load instruction of a wave reads 256 contiguous bytes and every store
// instruction writes 1 KB of contiguous, fully covered cache lines (a lane that
// writes its own 64 contiguous bytes instead leaves every line partially written per
// instruction and runs 3-4x slower).  A workgroup covers 256*U consecutive words and
// issues its U loads before the first store.  NT bit 0: nontemporal loads, bit 1:
// nontemporal stores.
//   MODE 0: blocksize == 1 << shift and blocksize % 8 == 0 (one absmax per word)
//   MODE 1: blocksize % 8 == 0, not a power of two (one absmax per word, division)
//   MODE 2: any even blocksize (absmax looked up per element)
template <int U, int MODE, int NT>
__global__ __launch_bounds__(256) void dequant4_kernel(const uint32_t* __restrict__ packed,
                                                      const float* __restrict__ absmax,
                                                      u4v* __restrict__ out, int64_t nwords,
                                                      int blocksize, int shift, int table) {
  __shared__ float tab[16];
  if (threadIdx.x < 16) tab[threadIdx.x] = table ? c_fp4[threadIdx.x] : c_nf4[threadIdx.x];
  const int64_t base = (int64_t)blockIdx.x * (256 * U) + threadIdx.x;
  uint32_t w[U];
  float am[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int64_t i = base + u * 256;
    w[u] = 0u;
    am[u] = 0.f;
    if (i < nwords) {
      w[u] = (NT & 1) ? __builtin_nontemporal_load(packed + i) : packed[i];
      if (MODE == 0) am[u] = absmax[(i * 8) >> shift];
      if (MODE == 1) am[u] = absmax[(i * 8) / blocksize];
    }
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int64_t i = base + u * 256;
    if (i >= nwords) continue;
    uint32_t o[4];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const uint32_t byte = (w[u] >> (8 * b)) & 255u;
      if (MODE == 2) {
        const int64_t e = i * 8 + 2 * b;
        o[b] = deq_pair(tab, byte, absmax[e / blocksize], absmax[(e + 1) / blocksize]);
      } else {
        o[b] = deq_pair(tab, byte, am[u], am[u]);
      }
    }
    u4v ov = {o[0], o[1], o[2], o[3]};
    if (NT & 2) store_stream(out + i, ov);
    else out[i] = ov;
  }
}

// Persistent variant of the main path (MODE 0 only, fewer than 2^31 words): a workgroup walks chunks of 256*U
// words with the next chunk's loads in flight while the current chunk is converted and stored, so the read and
// the write streams overlap in time.  Index arithmetic is 32-bit; the table offsets of a word's eight codes
// come from two masked copies of the word (low and high nibble of every byte, times four).
template <int U>
__global__ __launch_bounds__(256) void dequant4_pipelined_kernel(const uint32_t* __restrict__ packed,
                                                                const float* __restrict__ absmax,
                                                                u4v* __restrict__ out, uint32_t nwords, int shift,
                                                                int table) {
  __shared__ float tab[16];
  if (threadIdx.x < 16) tab[threadIdx.x] = table ? c_fp4[threadIdx.x] : c_nf4[threadIdx.x];
  constexpr uint32_t chunk_words = 256 * U;
  const uint32_t nchunks = (nwords + chunk_words - 1) / chunk_words;
  const int wshift = shift - 3;  // words per block = blocksize / 8
  uint32_t w[U], wn[U];
  float am[U], amn[U];
  auto load = [&](uint32_t chunk, uint32_t (&ww)[U], float (&aa)[U]) {
    const uint32_t base = chunk * chunk_words + threadIdx.x;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t i = min(base + u * 256, nwords - 1);  // clamped: a duplicate is loaded, never stored
      ww[u] = packed[i];
      aa[u] = absmax[i >> wshift];
    }
  };
  uint32_t chunk = blockIdx.x;
  if (chunk < nchunks) load(chunk, w, am);
  __syncthreads();
  const char* tb = reinterpret_cast<const char*>(tab);
  for (; chunk < nchunks; chunk += gridDim.x) {
    const uint32_t next = chunk + gridDim.x;
    if (next < nchunks) load(next, wn, amn);
    const uint32_t base = chunk * chunk_words + threadIdx.x;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t i = base + u * 256;
      const uint32_t lo4 = (w[u] << 2) & 0x3c3c3c3cu;  // low nibble of every byte, times 4: the later element
      const uint32_t hi4 = (w[u] >> 2) & 0x3c3c3c3cu;  // high nibble of every byte, times 4: the earlier element
      uint32_t o[4];
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const float t0 = *reinterpret_cast<const float*>(tb + ((hi4 >> (8 * b)) & 255u));
        const float t1 = *reinterpret_cast<const float*>(tb + ((lo4 >> (8 * b)) & 255u));
        const h2v h = {(_Float16)mul_f32_own(t0, am[u]), (_Float16)mul_f32_own(t1, am[u])};
        o[b] = __builtin_bit_cast(uint32_t, h);
      }
      const u4v ov = {o[0], o[1], o[2], o[3]};
      if (i < nwords) store_stream(out + i, ov);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) { w[u] = wn[u]; am[u] = amn[u]; }
  }
}

// Tail / odd sizes: one element per thread.
__global__ __launch_bounds__(256) void dequant4_tail_kernel(const uint8_t* __restrict__ packed,
                                                           const float* __restrict__ absmax,
                                                           _Float16* __restrict__ out, int64_t e_begin,
                                                           int64_t n, int blocksize, int table) {
  const int64_t e = e_begin + (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= n) return;
  const float* tab = table ? c_fp4 : c_nf4;
  const uint32_t byte = packed[e >> 1];
  const uint32_t code = (e & 1) ? (byte & 15u) : (byte >> 4);
  out[e] = (_Float16)mul_rounded_f32(tab[code], absmax[e / blocksize]);
}

}  // namespace

extern "C" int hq_dequant_nf4(const uint8_t* packed, const float* absmax, void* out_fp16,
                              int64_t n_elems, int blocksize, int table, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (n_elems < 0 || blocksize <= 0 || (blocksize & 1)) return HQ_ERR_BAD_SHAPE;
  if (table != HQ_TABLE_NF4 && table != HQ_TABLE_FP4) return HQ_ERR_BAD_ENUM;
  if (n_elems == 0) return HQ_OK;
  if (!packed || !absmax || !out_fp16) return HQ_ERR_NULL_POINTER;
  if (((uintptr_t)absmax & 3) || ((uintptr_t)out_fp16 & 1)) return HQ_ERR_MISALIGNED;
  const HqDevice* dev = nullptr;
  int rc = hq_current_device(&dev);
  if (rc != HQ_OK) return rc;

  const bool wide = !((uintptr_t)packed & 3) && !((uintptr_t)out_fp16 & 15);
  const int64_t nwords = wide ? n_elems / 8 : 0;
  if (nwords > 0) {
    const bool pow2 = (blocksize & (blocksize - 1)) == 0;
    int shift = 0;
    while ((1 << shift) < blocksize) ++shift;
    const uint32_t* pw = reinterpret_cast<const uint32_t*>(packed);
    const int mode = (blocksize % 8 == 0) ? (pow2 ? 0 : 1) : 2;
    // Measured on MI355X (4096x4096, blocksize 64): plain loads + nontemporal stores is the
    // fastest combination (7.8 us; plain stores 10-12 us), flat in U from 1 to 8.
    constexpr int U = 8, NT = 2;
    const int64_t blocks = (nwords + 256 * U - 1) / (256 * U);
    if (blocks > 0x7fffffff) return HQ_ERR_TOO_LARGE;
#define HQ_NF4_LAUNCH(MM)                                                                                    \
  if (mode == MM)                                                                                            \
    hipLaunchKernelGGL((dequant4_kernel<U, MM, NT>), dim3((unsigned)blocks), dim3(256), 0, stream, pw, absmax, \
                       (u4v*)out_fp16, nwords, blocksize, shift, table);
    // Pipelined variant, up to eight workgroups per CU, fewer for larger inputs (us per call, one-shot grid /
    // 2 / 4 / 8 workgroups per CU): 2^19 elements 5.17 / 4.11 / 4.13 / 4.11, 2^21 5.23 / 3.97 / 3.94 / 3.96,
    // 2^23 5.87 / 4.86 / 4.74 / 4.70, 2^24 (4096 x 4096) 7.78 / 7.44 / 7.10 / 7.20, 2^25 14.4 / 13.2 / 13.1 / 13.3,
    // 2^26 26.8 / 24.7 / 25.3 / 25.3, 2^27 51.5 / 47.3 / 49.8 / -; from 2^28 elements on the one-shot grid is the
    // faster one (121.0 against 122.6 with four and 168 with two; 484 against 507 us at 2^30).
    int pipe = hq_tune(HQ_TUNE_NF4_PIPE, -1);
    if (pipe < 0) pipe = nwords >= (1 << 25) ? 0 : (nwords <= (1 << 20) ? 8 : (nwords <= (1 << 22) ? 4 : 2));
    if (mode == 0 && pipe > 0 && shift >= 3 && nwords < ((int64_t)1 << 31)) {
      constexpr int PU = 4;
      const int64_t nch = (nwords + 256 * PU - 1) / (256 * PU);
      const int64_t grid = std::min<int64_t>((int64_t)dev->cus * pipe, nch);
      hipLaunchKernelGGL((dequant4_pipelined_kernel<PU>), dim3((unsigned)grid), dim3(256), 0, stream, pw, absmax,
                         (u4v*)out_fp16, (uint32_t)nwords, shift, table);
    } else {
    HQ_NF4_LAUNCH(0) HQ_NF4_LAUNCH(1) HQ_NF4_LAUNCH(2)
    }
#undef HQ_NF4_LAUNCH
    rc = hq_launch_status();
    if (rc != HQ_OK) return rc;
  }
  const int64_t e_begin = nwords * 8;
  if (e_begin < n_elems) {
    const int64_t rest = n_elems - e_begin;
    if ((rest + 255) / 256 > 0x7fffffff) return HQ_ERR_TOO_LARGE;
    hipLaunchKernelGGL(dequant4_tail_kernel, dim3((unsigned)((rest + 255) / 256)), dim3(256), 0, stream,
                       packed, absmax, (_Float16*)out_fp16, e_begin, n_elems, blocksize, table);
    rc = hq_launch_status();
  }
  return rc;
}
