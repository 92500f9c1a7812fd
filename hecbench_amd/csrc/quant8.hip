// bitsandbytes dynamic-map 8-bit quantisation for gfx950.
//
// Replaces dQuantize<0> / kQuantize<256,256> (src/quantBnB-hip/main.cu:13-130 in
// the HeCBench tree): a 7-step binary search over the sorted 256-entry code
// table followed by a midpoint comparison against the neighbour on the side of x
// (ties keep the pivot).  Bit-exact with the reference for every input.
// A lane converts four consecutive floats (one 128-bit load) into one packed 32-bit store.  A sorted
// table (the normal case, checked in the kernel) is served by a bucket table of thresholds built in LDS
// by every workgroup: one LDS read and about ten vector instructions per element instead of nine reads
// and over forty; any other table by the descent itself, read from LDS in level order.
#include "hq_internal.h"

namespace {

typedef float f4v __attribute__((ext_vector_type(4)));

// The reference search (pivot 127, steps 64..1) walks a perfect binary tree over the table
// entries 0..254 whose leaves are the even indices.  Two facts make it cheap:
//  * stored level by level (node j of level k at (1 << (k-1)) - 1 + j, holding entry
//    ((2j+1) << (8-k)) - 1), the nodes one level touches are contiguous in LDS, so lanes on
//    different nodes hit different banks instead of a few banks 2^(8-k) entries apart;
//  * the bounds the reference tracks on the way down are, at the leaf p, always the
//    neighbours p+1 (the nearest ancestor above; entry 255 when p = 254) and max(p-1, 0)
//    (the nearest ancestor below), so they need not be tracked, only looked up at the end.
// lds: [0..254] level order, [256..511] the table in index order.
__device__ __forceinline__ uint32_t quantize_one(const float* lds, float x) {
  uint32_t j = 0;
  float val = lds[0];
#pragma unroll
  for (int k = 1; k < 8; ++k) {
    j = 2 * j + (x > val ? 1u : 0u);
    val = lds[(1u << k) - 1 + j];
  }
  const uint32_t pivot = 2 * j;  // leaf index = table index
  const bool up = x > val;
  const uint32_t other = up ? pivot + 1 : (pivot == 0 ? 0u : pivot - 1);
  const float bound = lds[256 + other];
  const float midpoint = (bound + val) * 0.5f;
  // ties keep the pivot (strict comparisons, src/quantBnB-hip/main.cu:47-65)
  return (up ? x > midpoint : x < midpoint) ? other : pivot;
}

// ---- fast path for a sorted table ---------------------------------------------------------------
// With the table in increasing order the reference's result is a step function of x: it is the number
// of thresholds T_i = (c_i + c_i+1) / 2, i = 0..254, that x has passed, where an even i is passed by
// x > T_i and an odd i by x >= T_i (ties keep the pivot, and pivots are the even entries).  That holds
// whenever c_i < T_i < c_i+1; a gap where rounding or equal entries break it is "degenerate".
// Inputs are binned by a monotone key (the exponent and six mantissa bits of |x| + off: 64 buckets per
// binade down to off = M / 4096, linear below, one overflow bucket beyond the largest magnitude M; the
// sign picks one of two slots).  A bucket's entry holds the number of thresholds in lower buckets and
// the one threshold inside it (an odd i as the float just below T_i, so that every test is x > t;
// +inf if there is none), so a lookup is one 8-byte LDS read, one compare and one add.  Buckets with
// two or more thresholds, or touching a degenerate gap, carry a NaN pattern instead of a count: one
// unordered compare of that word with x finds them and the NaN inputs, and those lanes take the tree
// descent instead.

constexpr int kKeyShift = 17;       // six mantissa bits
constexpr int kMaxBuckets = 13 * 64 + 66;  // per sign: 12 binades from off to M, the linear one, a partial top, overflow
constexpr uint32_t kSlow = 0x7fc00000u;

struct FastTables {
  uint2 entry[2 * kMaxBuckets];  // slot 2 * idx (x >= +0) or 2 * idx + 1 (sign bit set): {threshold, count}
  uint32_t inside[(2 * kMaxBuckets + 255) / 256 * 256];  // thresholds per bucket, in value order
  float tval[256];               // the thresholds as "x > t" tests
  uint32_t wave_total[4];
};

__device__ __forceinline__ uint32_t bucket_slot(float x, float off, uint32_t base, uint32_t cnt) {
  const float y2 = fabsf(x) + off;  // >= off; a NaN lands in the overflow bucket
  const uint32_t idx = min((__float_as_uint(y2) - base) >> kKeyShift, cnt);
  return 2 * idx + (__float_as_uint(x) >> 31);
}
// buckets in the order of the values they hold: negative overflow first, positive overflow last
__device__ __forceinline__ uint32_t slot_order(uint32_t slot, uint32_t cnt) {
  const uint32_t idx = slot >> 1;
  return (slot & 1u) ? cnt - idx : cnt + 1 + idx;
}
__device__ __forceinline__ uint32_t order_slot(uint32_t pos, uint32_t cnt) {
  return pos <= cnt ? 2 * (cnt - pos) + 1 : 2 * (pos - cnt - 1);
}

// a, b: table entries t and t + 1 of thread t (t < 255).  All 256 threads.  Thresholds are counted into
// their buckets, a scan over the buckets in value order gives every bucket the number of thresholds
// before it, which is also the index of the first threshold inside it.
__device__ __forceinline__ void build_fast_tables(FastTables& ft, float a, float b, float off, uint32_t base,
                                                  uint32_t cnt) {
  const int t = threadIdx.x;
  const uint32_t nb = 2 * cnt + 2;             // buckets, both signs and overflows
  constexpr uint32_t kPer = (2 * kMaxBuckets + 255) / 256;  // buckets per thread
  bool degenerate = false;
  uint32_t mine = 0;
#pragma unroll
  for (uint32_t k = 0; k < kPer; ++k) ft.inside[t * kPer + k] = 0;
  if (t < 255) {
    float T = (b + a) * 0.5f;
    degenerate = !(a < T && T < b);
    float tv;
    if (t & 1) {  // x >= T: as x > the float just below T; a zero T must let -0 pass, so it goes to the negative side
      if (T == 0.f) T = -0.f;
      const uint32_t u = __float_as_uint(T);
      tv = T == 0.f ? __uint_as_float(0x80000001u) : __uint_as_float(T > 0.f ? u - 1 : u + 1);
    } else {      // x > T: a zero T must not let +0 pass from a higher bucket, so it goes to the positive side
      T = T + 0.f;
      tv = T;
    }
    mine = slot_order(bucket_slot(T, off, base, cnt), cnt);
    ft.tval[t] = tv;
  }
  __syncthreads();
  if (t < 255) atomicAdd(&ft.inside[mine], 1u);
  __syncthreads();
  uint32_t c[kPer], sum = 0;
#pragma unroll
  for (uint32_t k = 0; k < kPer; ++k) { c[k] = ft.inside[t * kPer + k]; sum += c[k]; }
  uint32_t incl = sum;  // inclusive scan over the wave, then over the four waves
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const uint32_t up = __shfl_up(incl, d);
    if ((t & 63) >= d) incl += up;
  }
  if ((t & 63) == 63) ft.wave_total[t >> 6] = incl;
  __syncthreads();
  uint32_t before = incl - sum;
  for (int w = 0; w < (t >> 6); ++w) before += ft.wave_total[w];
#pragma unroll
  for (uint32_t k = 0; k < kPer; ++k) {
    const uint32_t pos = t * kPer + k;
    if (pos < nb) {
      uint2 e;
      e.x = c[k] ? __float_as_uint(ft.tval[min(before, 254u)]) : 0x7f800000u;  // +inf: x > t never holds
      e.y = c[k] <= 1 ? before : kSlow;
      ft.entry[order_slot(pos, cnt)] = e;
    }
    before += c[k];
  }
  __syncthreads();
  if (degenerate) {  // every input between and on the two entries is in one of their buckets
    ft.entry[bucket_slot(a, off, base, cnt)].y = kSlow;
    ft.entry[bucket_slot(b, off, base, cnt)].y = kSlow;
    if (a == 0.f || b == 0.f) ft.entry[0].y = ft.entry[1].y = kSlow;  // both zeros' buckets
  }
  __syncthreads();
}

constexpr int kQuads = 4;  // 16-byte loads per thread and trip

__global__ __launch_bounds__(256) void quantize8_kernel(const float* __restrict__ code,
                                                       const float* __restrict__ A,
                                                       uint8_t* __restrict__ out, int64_t n,
                                                       int vec_ok, int allow_fast) {
  __shared__ float s_code[512];
  __shared__ __align__(16) FastTables ft;
  const int t = threadIdx.x;
  const float ct = code[t], cn = code[min(t + 1, 255)];
  const float M = fmaxf(fabsf(code[0]), fabsf(code[255]));
  {
    if (t < 255) {  // level-order slot t <- table entry ((2j+1) << (8-k)) - 1
      const int k = 32 - __builtin_clz((unsigned)t + 1);  // level 1..8
      const int j = t + 1 - (1 << (k - 1));
      s_code[t] = code[((2 * j + 1) << (8 - k)) - 1];
    }
    s_code[256 + t] = ct;
  }
  // the fast path wants a sorted table of finite, moderate values (midpoints cannot overflow) with a
  // usable magnitude
  const float off = M * (1.f / 4096.f);
  const uint32_t base = __float_as_uint(off) & ~((1u << kKeyShift) - 1);
  const uint32_t cnt = ((__float_as_uint(M + off) - base) >> kKeyShift) + 1;  // index of the overflow bucket
  const bool fast = __syncthreads_and((ct <= cn) && fabsf(ct) <= 1e30f) && M >= 1e-30f && allow_fast &&
                    cnt < (uint32_t)kMaxBuckets;
  const int64_t nquads = vec_ok ? n / 4 : 0;
  const int64_t stride = (int64_t)gridDim.x * 256;
  const int64_t t0 = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (fast) {
    // the first trip's loads are in flight while the tables are built, and each later trip's while the
    // one before is converted
    f4v v[kQuads], vn[kQuads];
    auto load = [&](int64_t i, f4v (&dst)[kQuads]) {
#pragma unroll
      for (int k = 0; k < kQuads; ++k) {
        const int64_t ik = i + k * stride;
        dst[k] = __builtin_nontemporal_load(reinterpret_cast<const f4v*>(A) + (ik < nquads ? ik : i));
      }
    };
    if (t0 < nquads) load(t0, v);
    build_fast_tables(ft, ct, cn, off, base, cnt);
    for (int64_t i = t0; i < nquads; i += kQuads * stride) {
      const int64_t inext = i + kQuads * stride;
      if (inext < nquads) load(inext, vn);
      uint32_t q[4 * kQuads];
      bool slow = false;
#pragma unroll
      for (int k = 0; k < kQuads; ++k) {
        const float x[4] = {v[k].x, v[k].y, v[k].z, v[k].w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const uint2 en = ft.entry[bucket_slot(x[e], off, base, cnt)];
          q[4 * k + e] = en.y + (x[e] > __uint_as_float(en.x) ? 1u : 0u);
          slow |= !(__uint_as_float(en.y) <= x[e] || __uint_as_float(en.y) > x[e]);  // unordered: flagged bucket or NaN input
        }
      }
      if (__builtin_amdgcn_ballot_w64(slow)) {
#pragma unroll
        for (int k = 0; k < kQuads; ++k) {
          const float x[4] = {v[k].x, v[k].y, v[k].z, v[k].w};
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (q[4 * k + e] > 255u || x[e] != x[e]) q[4 * k + e] = quantize_one(s_code, x[e]);
        }
      }
#pragma unroll
      for (int k = 0; k < kQuads; ++k) {
        const int64_t ik = i + k * stride;
        if (ik < nquads)
          __builtin_nontemporal_store(q[4 * k] | (q[4 * k + 1] << 8) | (q[4 * k + 2] << 16) | (q[4 * k + 3] << 24),
                                      reinterpret_cast<uint32_t*>(out) + ik);
      }
#pragma unroll
      for (int k = 0; k < kQuads; ++k) v[k] = vn[k];
    }
  } else {
  __syncthreads();
  // Two quads per trip, searched in lockstep level by level: eight independent LDS reads
  // are in flight per level instead of one dependent chain per element.
  for (int64_t i = t0; i < nquads; i += 2 * stride) {
    const int64_t i1 = i + stride;
    const bool two = i1 < nquads;
    const f4v v0 = __builtin_nontemporal_load(reinterpret_cast<const f4v*>(A) + i);
    const f4v v1 = __builtin_nontemporal_load(reinterpret_cast<const f4v*>(A) + (two ? i1 : i));
    const float x[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
    uint32_t j[8];
    float val[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) { j[e] = 0; val[e] = s_code[0]; }
#pragma unroll
    for (int k = 1; k < 8; ++k) {
#pragma unroll
      for (int e = 0; e < 8; ++e) j[e] = 2 * j[e] + (x[e] > val[e] ? 1u : 0u);
#pragma unroll
      for (int e = 0; e < 8; ++e) val[e] = s_code[(1u << k) - 1 + j[e]];
    }
    uint32_t other[8];
    float bound[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint32_t pivot = 2 * j[e];
      other[e] = x[e] > val[e] ? pivot + 1 : (pivot == 0 ? 0u : pivot - 1);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) bound[e] = s_code[256 + other[e]];
    uint32_t q[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float midpoint = (bound[e] + val[e]) * 0.5f;
      const bool up = x[e] > val[e];
      q[e] = (up ? x[e] > midpoint : x[e] < midpoint) ? other[e] : 2 * j[e];
    }
    __builtin_nontemporal_store(q[0] | (q[1] << 8) | (q[2] << 16) | (q[3] << 24),
                                reinterpret_cast<uint32_t*>(out) + i);
    if (two)
      __builtin_nontemporal_store(q[4] | (q[5] << 8) | (q[6] << 16) | (q[7] << 24),
                                  reinterpret_cast<uint32_t*>(out) + i1);
  }
  }
  for (int64_t e = nquads * 4 + t0; e < n; e += stride) out[e] = (uint8_t)quantize_one(s_code, A[e]);
}

}  // namespace

extern "C" int hq_quantize_dynamic8(const float* code, const float* A, uint8_t* out, int64_t n,
                                    void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (n < 0) return HQ_ERR_BAD_SHAPE;
  if (n == 0) return HQ_OK;
  if (!code || !A || !out) return HQ_ERR_NULL_POINTER;
  if (((uintptr_t)code & 3) || ((uintptr_t)A & 3)) return HQ_ERR_MISALIGNED;
  const HqDevice* dev = nullptr;
  int rc = hq_current_device(&dev);
  if (rc != HQ_OK) return rc;
  const int vec_ok = !((uintptr_t)A & 15) && !((uintptr_t)out & 3);
  int64_t blocks = (n / 4 + 256 * kQuads - 1) / (256 * kQuads);  // one trip of the fast path each, or grid-stride
  // workgroups per CU of the persistent fast path: five up to 2^24 elements (16.5 us; two 17.8, eight 19.2),
  // two from 2^25 on (2^25: 30.5 against 31.4 us with five, 2^26: 55.4 against 59.7, 2^27: 108.6 against 123.2)
  const int64_t cap = (int64_t)dev->cus * hq_tune(HQ_TUNE_Q8_WGS, n >= ((int64_t)1 << 25) ? 2 : 5);
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(quantize8_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, code, A, out, n,
                     vec_ok, hq_tune(HQ_TUNE_Q8_FAST, 1));
  return hq_launch_status();
}
