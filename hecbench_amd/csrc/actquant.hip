// Per-token int8 activation quantisation (static / dynamic scale, with or without an
// asymmetric zero point) for gfx950.
//
// Replaces static_scaled_int8_quant / dynamic_scaled_int8_quant and their four kernels
// (src/quantVLLM-hip/main.cu:11-168 in the HeCBench tree; helpers in
// src/quantVLLM-cuda/utils.h).  Bit-exact contract: fp32 IEEE division, round to nearest
// even, saturation, exactly as the reference's host loops (src/quantVLLM-cuda/reference.h).
//
// HBM-bound: 3 bytes per fp16 / bf16 element, 5 per fp32 element.  The tensor is cut into units of
// eight consecutive elements on a grid anchored at element 0 of the tensor, not of the row, so that a
// unit is one aligned 128-bit load (two for fp32) and one 64-bit store whatever the hidden size is
// (the reference's run size is 5137); a unit that straddles a row boundary is masked.
//   static : no row structure at all, a flat grid-stride loop over the units.
//   dynamic: a wave per row up to 1536 elements, a workgroup per row beyond; the row stays in registers
//            between the max / min pass and the quantise pass (one read of x, up to 10240 elements);
//            one launch slot per row, many workgroups per CU.
// The division by a scale shared by many elements is done as a multiplication by its reciprocal
// wherever that provably rounds to the same integer (the product is further from a tie than its error
// bound, or saturates either way); the other lanes divide.
#include "hq_internal.h"

namespace {

typedef uint32_t u4v __attribute__((ext_vector_type(4)));
typedef uint32_t u2v __attribute__((ext_vector_type(2)));

struct bf16_t { uint16_t bits; };  // bfloat16 = the upper half of an fp32

// src/quantVLLM-cuda/utils.h:9-24
// The saturation is done on the converted integer (the hardware conversion saturates at the int32 range
// and turns a NaN into 0, as the conversion of the clamped float did): one integer median instead of
// two compares and two selects per element.
__device__ __forceinline__ int float_to_int8_rn(float x) {
  const float dst = rintf(x);
  int r;
  asm("v_cvt_i32_f32 %0, %1" : "=v"(r) : "v"(dst));
  return min(max(r, -128), 127);
}
// src/quantVLLM-cuda/utils.h:26-50: round to nearest even, saturating at the int32 range.  The
// hardware conversion saturates by itself (and turns a NaN into 0); it is written as an instruction
// because the C conversion of an out-of-range value is undefined.
__device__ __forceinline__ int float_to_int32_rn(float x) {
  const float dst = rintf(x);
  int r;
  asm("v_cvt_i32_f32 %0, %1" : "=v"(r) : "v"(dst));
  return r;
}
// src/quantVLLM-cuda/utils.h:52-61 (saturating add of the zero point happens in int32)
__device__ __forceinline__ int int32_to_int8(int x) { return x < -128 ? -128 : (127 < x ? 127 : x); }

constexpr int kVec = 8;  // elements per unit

// One unit of raw data: 16 bytes of fp16 / bf16 or 32 bytes of fp32.
template <typename T> struct Raw { u4v w[sizeof(T) == 4 ? 2 : 1]; };

template <typename T>
__device__ __forceinline__ Raw<T> load_unit(const T* __restrict__ base, int64_t unit) {
  Raw<T> r;
  const u4v* p = reinterpret_cast<const u4v*>(base + unit * kVec);
#pragma unroll
  for (int i = 0; i < (int)(sizeof(T) == 4 ? 2 : 1); ++i) r.w[i] = __builtin_nontemporal_load(p + i);
  return r;
}
// A unit that reaches past the end of the tensor: element by element, zeros beyond.
template <typename T>
__device__ __forceinline__ Raw<T> load_unit_tail(const T* __restrict__ base, int64_t unit, int64_t total) {
  Raw<T> r;
  T tmp[kVec];
#pragma unroll
  for (int i = 0; i < kVec; ++i) {
    const int64_t e = unit * kVec + i;
    tmp[i] = e < total ? base[e] : T{};
  }
  __builtin_memcpy(&r, tmp, sizeof(r));
  return r;
}
__device__ __forceinline__ void unpack(const Raw<float>& r, float (&v)[kVec]) {
#pragma unroll
  for (int i = 0; i < kVec; ++i) v[i] = __uint_as_float(r.w[i >> 2][i & 3]);
}
__device__ __forceinline__ void unpack(const Raw<_Float16>& r, float (&v)[kVec]) {
#pragma unroll
  for (int i = 0; i < kVec; ++i)
    v[i] = (float)__builtin_bit_cast(_Float16, (uint16_t)(r.w[0][i >> 1] >> (16 * (i & 1))));
}
__device__ __forceinline__ void unpack(const Raw<bf16_t>& r, float (&v)[kVec]) {
#pragma unroll
  for (int i = 0; i < kVec; ++i)
    v[i] = __uint_as_float((i & 1) ? (r.w[0][i >> 1] & 0xffff0000u) : (r.w[0][i >> 1] << 16));
}

// y[i] = element i * m.  An fp16 element is converted and multiplied by one mixed-precision instruction
// (the added +0 only turns a product of -0 into +0, which rounds to the same integer).
template <typename T>
__device__ __forceinline__ void products(const Raw<T>& r, float m, float (&y)[kVec]) {
  float v[kVec];
  unpack(r, v);
#pragma unroll
  for (int i = 0; i < kVec; ++i) y[i] = v[i] * m;
}
__device__ __forceinline__ void products(const Raw<_Float16>& r, float m, float (&y)[kVec]) {
#pragma unroll
  for (int i = 0; i < kVec / 2; ++i) {
    asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel_hi:[1,0,0]" : "=v"(y[2 * i]) : "v"(r.w[0][i]), "v"(m));
    asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(y[2 * i + 1]) : "v"(r.w[0][i]), "v"(m));
  }
}

// Running maximum and minimum of whole units.  fp16 units are scanned as packed halves (the maximum of
// magnitudes on the bits with the signs cleared), everything else as converted floats.
typedef _Float16 h2v __attribute__((ext_vector_type(2)));
template <typename T, bool AZP>
struct UnitScan {
  __device__ __forceinline__ void add(const Raw<T>& r, float& mx, float& mn) {
    float v[kVec];
    unpack(r, v);
#pragma unroll
    for (int i = 0; i < kVec; ++i) {
      if (AZP) { mx = fmaxf(mx, v[i]); mn = fminf(mn, v[i]); }
      else mx = fmaxf(mx, fabsf(v[i]));
    }
  }
  __device__ __forceinline__ void fold(float&, float&) {}
};
template <bool AZP>
struct UnitScan<_Float16, AZP> {
  h2v hi, lo;
  __device__ __forceinline__ UnitScan() {
    const _Float16 inf = (_Float16)__builtin_inff();
    hi = AZP ? h2v{-inf, -inf} : h2v{(_Float16)0.f, (_Float16)0.f};
    lo = h2v{inf, inf};
  }
  __device__ __forceinline__ void add(const Raw<_Float16>& r, float&, float&) {
#pragma unroll
    for (int i = 0; i < kVec / 2; ++i) {
      const h2v x = __builtin_bit_cast(h2v, AZP ? r.w[0][i] : (r.w[0][i] & 0x7fff7fffu));
      hi = __builtin_elementwise_max(hi, x);
      if (AZP) lo = __builtin_elementwise_min(lo, x);
    }
  }
  __device__ __forceinline__ void fold(float& mx, float& mn) {
    mx = fmaxf(mx, fmaxf((float)hi.x, (float)hi.y));
    if (AZP) mn = fminf(mn, fminf((float)lo.x, (float)lo.y));
  }
};

// Makes the compiler forget what it knows about a unit's bits, so that the values converted for the
// first pass are not kept alive (at twice the registers of the raw data) for the second.
template <typename T>
__device__ __forceinline__ void forget(Raw<T>& r) {
#pragma unroll
  for (int i = 0; i < (int)(sizeof(T) == 4 ? 2 : 1); ++i)
    asm volatile("" : "+v"(r.w[i]));
}

// The low bytes of four integers as one word, a first: byte selects instead of masks and shifts.
__device__ __forceinline__ uint32_t pack4(int a, int b, int c, int d) {
  const uint32_t lo = __builtin_amdgcn_perm((uint32_t)b, (uint32_t)a, 0x0c0c0400u);
  const uint32_t hi = __builtin_amdgcn_perm((uint32_t)d, (uint32_t)c, 0x04000c0cu);
  return lo | hi;
}

// Stores elements [lo, hi) of a unit's eight results; all eight as one 64-bit store.  STREAM: as a
// write-through nontemporal store, which the one-pass static kernels gain from (14.2 -> 13.5 us at 4096 x 5137
// fp16) and the two-pass dynamic kernels lose by (18.5 -> 22.9 us).
template <bool STREAM>
__device__ __forceinline__ void store_unit(int8_t* __restrict__ out, int64_t unit, const int (&q)[kVec], int lo, int hi,
                                           bool aligned) {
  int8_t* p = out + unit * kVec;
  if (lo == 0 && hi == kVec && aligned) {
    u2v w;
    w.x = pack4(q[0], q[1], q[2], q[3]);
    w.y = pack4(q[4], q[5], q[6], q[7]);
    if (STREAM) hq_store_stream(reinterpret_cast<hq_u2v*>(p), w);
    else __builtin_nontemporal_store(w, reinterpret_cast<u2v*>(p));
  } else if (aligned) {
    // a unit shared with the neighbouring row: the fewest naturally aligned pieces that cover [lo, hi)
    // (a store instruction costs the same whatever it carries, and the other lanes wait for it)
    uint32_t w[2];
    w[0] = pack4(q[0], q[1], q[2], q[3]);
    w[1] = pack4(q[4], q[5], q[6], q[7]);
#pragma unroll
    for (int d = 0; d < 2; ++d) {
      const bool whole = lo <= 4 * d && hi >= 4 * d + 4;
      if (whole) reinterpret_cast<uint32_t*>(p)[d] = w[d];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int b = 4 * d + 2 * h;
        const bool half = !whole && lo <= b && hi >= b + 2;
        if (half) reinterpret_cast<uint16_t*>(p)[2 * d + h] = (uint16_t)(w[d] >> (16 * h));
        if (!whole && !half) {
          if (lo <= b && hi > b) p[b] = (int8_t)q[b];
          if (lo <= b + 1 && hi > b + 1) p[b + 1] = (int8_t)q[b + 1];
        }
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < kVec; ++i)
      if (i >= lo && i < hi) p[i] = (int8_t)q[i];
  }
}

// Division by a scale that many elements share.  y = v * (1 / s) differs from the rounded quotient q by
// less than 1.5 * 2^-23 |q| (2^-24 relative each for the reciprocal, the product and the quotient itself),
// so both round to the same integer unless y is within that of a tie; the checks below allow twice as
// much, 3 * 2^-23 |y|, which also covers their own rounding.  Where the result saturates the quotient
// need not be known at all.  The reciprocal must be a normal number for that bound.
struct Divisor {
  float s, r;
  bool usable;
  __device__ __forceinline__ explicit Divisor(float scale) : s(scale), r(1.0f / scale) {
    const float a = fabsf(scale);
    usable = a >= 0x1p-100f && a <= 0x1p100f;
  }
};

// float_to_int8_rn(v / s) or, with AZP, int32_to_int8(float_to_int32_rn(v / s) + azp), for eight values.
template <bool AZP, typename T>
__device__ __forceinline__ void quantise8(const Raw<T>& raw, const Divisor& d, int azp, int (&q)[kVec]) {
  float y[kVec];
  products(raw, d.r, y);
  auto divide = [&]() {
    float v[kVec];
    unpack(raw, v);
#pragma unroll
    for (int i = 0; i < kVec; ++i) y[i] = v[i] / d.s;
  };
  if (!AZP) {
    // Without a zero point only |y| < 129 can end anywhere but at a bound, and there 3 * 2^-23 |y| is less
    // than 2^-15: one constant margin for all eight, taken on the largest distance of a product from its
    // nearest integer.  The subtraction is exact and must stay one (contracted into a multiply-add it
    // would return the rounding error of products beyond 2^23 and send those to the division).  A NaN
    // distance - an infinite or NaN input - drops out of the maximum: such a product converts to the same
    // bound, or to 0, as the quotient.
#pragma clang fp contract(off)
    float worst = 0.f;
#pragma unroll
    for (int i = 0; i < kVec; ++i) worst = fmaxf(worst, fabsf(y[i] - rintf(y[i])));
    const bool exact = !d.usable || !(worst <= 0.5f - 0x1p-15f);
    if (__builtin_amdgcn_ballot_w64(exact)) divide();
#pragma unroll
    for (int i = 0; i < kVec; ++i) q[i] = float_to_int8_rn(y[i]);
    return;
  }
  // With a zero point any quotient may matter: the margin is relative (a subnormal product has no
  // relative bound and no tie near it either); it reaches 0.5, i.e. sends the unit to the division, from
  // |y| = 2^20.4 on.  One comparison for the largest of the eight; a NaN drops out as above.
  float worst = 0.f;
  {
#pragma clang fp contract(off)
#pragma unroll
    for (int i = 0; i < kVec; ++i) {
      const float dist = fabsf(y[i] - rintf(y[i]));  // distance to the nearest integer
      worst = fmaxf(worst, fmaf(fabsf(y[i]), 0x1.8p-22f, dist));
    }
  }
  const bool exact = !d.usable || !(worst < 0.5f - 0x1p-24f);
  if (__builtin_amdgcn_ballot_w64(exact)) divide();
#pragma unroll
  for (int i = 0; i < kVec; ++i) q[i] = int32_to_int8(float_to_int32_rn(y[i]) + azp);
}

// ---- static scale: elementwise over the whole tensor ---------------------------------------------
constexpr int kStaticUnroll = 2;

template <typename T, bool AZP>
__global__ __launch_bounds__(256) void static_quant_kernel(const T* __restrict__ in, int8_t* __restrict__ out,
                                                          float scale, int azp, int64_t total, int aligned) {
  const Divisor d(scale);
  const int64_t units = (total + kVec - 1) / kVec;
  const int64_t full = aligned ? total / kVec : 0;  // units loaded whole: inside the tensor, pointers aligned
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t u0 = (int64_t)blockIdx.x * 256 + threadIdx.x; u0 < units; u0 += stride * kStaticUnroll) {
    Raw<T> raw[kStaticUnroll];
#pragma unroll
    for (int k = 0; k < kStaticUnroll; ++k) {
      const int64_t u = u0 + k * stride;
      if (u < full) raw[k] = load_unit(in, u);
      else if (u < units) raw[k] = load_unit_tail(in, u, total);
      else raw[k] = Raw<T>{};
    }
#pragma unroll
    for (int k = 0; k < kStaticUnroll; ++k) {
      const int64_t u = u0 + k * stride;
      int q[kVec];
      quantise8<AZP>(raw[k], d, azp, q);
      if (u < units) store_unit<true>(out, u, q, 0, (int)min((int64_t)kVec, total - u * kVec), aligned);
    }
  }
}

// ---- dynamic scale: LANES threads per row --------------------------------------------------------
// Maximum of a and minimum of b over the LANES threads of a row.
// (Neither is a NaN: the scans drop them.)  Within a wave: lane exchanges inside rows of 16 lanes on the
// data path of the instruction (DPP), then the four rows through scalar registers; six rounds of
// shuffles through the LDS crossbar took about three times as long.
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float lane_f(float v, int l) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), l));
}
template <bool MAX>
__device__ __forceinline__ float wave_extreme(float v) {
  auto pick = [](float x, float y) { return MAX ? fmaxf(x, y) : fminf(x, y); };
  v = pick(v, dpp_f<0xB1>(v));   // quad_perm [1,0,3,2]
  v = pick(v, dpp_f<0x4E>(v));   // quad_perm [2,3,0,1]
  v = pick(v, dpp_f<0x141>(v));  // row_half_mirror
  v = pick(v, dpp_f<0x140>(v));  // row_mirror
  return pick(pick(lane_f(v, 0), lane_f(v, 16)), pick(lane_f(v, 32), lane_f(v, 48)));
}
template <int LANES>
__device__ __forceinline__ void row_max_min(float& a, float& b, float* lds) {
  a = wave_extreme<true>(a);
  b = wave_extreme<false>(b);
  if (LANES > 64) {  // the row spans the workgroup
    const int wv = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) { lds[wv] = a; lds[4 + wv] = b; }
    __syncthreads();
#pragma unroll
    for (int w = 0; w < LANES / 64; ++w) { a = fmaxf(a, lds[w]); b = fminf(b, lds[4 + w]); }
  }
}

// LANES threads per row (a wave, or the workgroup), so 256 / LANES rows per workgroup and one workgroup
// for every 256 / LANES rows: nothing loops over rows.  KEEP units per thread stay in registers between
// the max / min pass and the quantise pass; a longer row streams the rest twice.  (Workgroups that walked
// over several rows, the next rows' loads in flight during the reduction, the quantisation and the stores,
// needed twice the registers for half the waves per CU and measured 18.8 us where this takes 14.0, 4096
// rows of 5137 fp16: the hardware overlaps one row's stores with another's loads by itself when enough
// workgroups fit a CU.)
// VEC: both pointers are aligned and the tensor is a whole number of units, so every unit is loaded whole.
template <typename T, bool AZP, int LANES, int KEEP, bool VEC>
__global__ __launch_bounds__(256) void dynamic_quant_kernel(const T* __restrict__ in, int8_t* __restrict__ out,
                                                           float* __restrict__ scales, int32_t* __restrict__ azps,
                                                           int64_t tokens, int hidden) {
  constexpr bool aligned = VEC;
  __shared__ float lds[8];
  const int lane = threadIdx.x % LANES;
  const int64_t total = tokens * hidden;
  // uniform over the wave (LANES == 64) or the workgroup
  const int64_t token = LANES == 64 ? (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6) : blockIdx.x;
  if (token >= tokens) return;
  // The row's units, and the multiple of 64 at or before its first: lanes are laid over the units from
  // there, so that a wave's loads and stores cover whole 128-byte lines of the output (256 of the
  // input) except at the row's ends.  Everything per row is uniform: base pointers at that multiple of
  // 64, and 32-bit unit numbers j relative to it (valid in [first, end)).
  const int64_t g0 = token * hidden;
  const int64_t u_first = g0 / kVec;
  const int64_t ubase = u_first & ~(int64_t)63;
  const int first = (int)(u_first - ubase);
  const int end = (int)((g0 + hidden + kVec - 1) / kVec - ubase);
  const int head = (int)(g0 - u_first * kVec);  // elements of the first unit that belong to the row before
  const T* row_in = in + ubase * kVec;
  int8_t* row_out = out + ubase * kVec;
  auto fetch = [&](int j) { return VEC ? load_unit(row_in, j) : load_unit_tail(in, ubase + j, total); };

  Raw<T> keep[KEEP];
#pragma unroll
  for (int k = 0; k < KEEP; ++k) {
    const int j = lane + k * LANES;
    // whole units are loaded without a branch, so that the loads stay one straight run the waits can
    // count; a unit outside the row repeats the row's first or last
    if (VEC) keep[k] = load_unit(row_in, min(max(j, first), end - 1));
    else if (j >= first && j < end) keep[k] = fetch(j);
  }

  // reference initial values: max starts at FLT_MIN (smallest positive normal), min at FLT_MAX
  // (reference.h:71-72); the symmetric variant starts its absmax at 0 (reference.h:43)
  float mx = AZP ? 1.17549435e-38f : 0.f;
  float mn = 3.40282347e+38f;
  UnitScan<T, AZP> whole;
  auto scan = [&](const Raw<T>& raw, int j) {
    const int rel = (j - first) * kVec - head;  // row position of the unit's element 0
    const int lo = max(-rel, 0), hi = min(hidden - rel, kVec);
    if (lo == 0 && hi == kVec) {  // all but the row's first and last unit
      whole.add(raw, mx, mn);
    } else {
      float v[kVec];
      unpack(raw, v);
#pragma unroll
      for (int i = 0; i < kVec; ++i)
        if (i >= lo && i < hi) {
          if (AZP) { mx = fmaxf(mx, v[i]); mn = fminf(mn, v[i]); }
          else mx = fmaxf(mx, fabsf(v[i]));
        }
    }
  };
#pragma unroll
  for (int k = 0; k < KEEP; ++k) {
    const int j = lane + k * LANES;
    if (j >= first && j < end) scan(keep[k], j);
  }
  for (int j = lane + KEEP * LANES; j < end; j += LANES) scan(fetch(j), j);
  whole.fold(mx, mn);
  row_max_min<LANES>(mx, mn, lds);

  float scale_val, mul = 0.f;
  int azp_val = 0;
  if (AZP) {
    scale_val = (mx - mn) / 255.0f;
    azp_val = (int)rintf(-128.0f - mn / scale_val);
  } else {
    scale_val = mx / 127.0f;
    mul = 127.0f / mx;
  }
  if (lane == 0) {
    scales[token] = scale_val;
    if (AZP) azps[token] = azp_val;
  }
  const Divisor d(scale_val);
  auto emit = [&](Raw<T> raw, int j) {
    int q[kVec];
    forget(raw);
    if (AZP) {
      quantise8<true>(raw, d, azp_val, q);
    } else {
      float y[kVec];
      products(raw, mul, y);
#pragma unroll
      for (int i = 0; i < kVec; ++i) q[i] = float_to_int8_rn(y[i]);
    }
    const int rel = (j - first) * kVec - head;
    store_unit<false>(row_out, j, q, max(-rel, 0), min(hidden - rel, kVec), aligned);
  };
#pragma unroll
  for (int k = 0; k < KEEP; ++k) {
    const int j = lane + k * LANES;
    if (j >= first && j < end) emit(keep[k], j);
  }
  for (int j = lane + KEEP * LANES; j < end; j += LANES) emit(fetch(j), j);
}

// The 128-bit loads and 64-bit stores need both base pointers on their grid; other pointers are served
// element by element.
__host__ inline int pointers_aligned(const void* in, const void* out) {
  return !((uintptr_t)in & 15) && !((uintptr_t)out & 7);
}

template <typename T>
int launch_static(const T* in, int8_t* out, int64_t tokens, int hidden, float scale, int has_azp, int azp,
                  const HqDevice* dev, hipStream_t stream) {
  const int aligned = pointers_aligned(in, out);
  const int64_t total = tokens * hidden;
  const int64_t units = (total + kVec - 1) / kVec;
  int64_t blocks = (units + 256 * kStaticUnroll - 1) / (256 * kStaticUnroll);
  // six workgroups per CU, grid-stride beyond that (us per call at 32 / 6 per CU, fp16: 4096 x 5137 13.8 / 12.8,
  // 4096 x 4096 11.3 / 10.7, 8192 x 5120 24.3 / 23.3, 16384 x 8192 72.4 / 71.6; four and eight per CU, and grids
  // sized so that every workgroup makes the same number of trips, measured in between)
  const int64_t cap = (int64_t)dev->cus * 6;
  if (blocks > cap) blocks = cap;
  if (has_azp)
    hipLaunchKernelGGL((static_quant_kernel<T, true>), dim3((unsigned)blocks), dim3(256), 0, stream, in, out, scale, azp,
                       total, aligned);
  else
    hipLaunchKernelGGL((static_quant_kernel<T, false>), dim3((unsigned)blocks), dim3(256), 0, stream, in, out, scale, azp,
                       total, aligned);
  return hq_launch_status();
}

template <typename T, bool AZP, bool VEC>
void launch_dynamic_vec(const T* in, int8_t* out, float* scales, int32_t* azps, int64_t tokens, int hidden,
                        const HqDevice* dev, hipStream_t stream) {
  // short rows get a wave each, the others the workgroup; the units a thread must keep pick the kernel
  const bool wave_rows = hidden <= 64 * kVec * 3;
  const int lanes = wave_rows ? 64 : 256;
  const int span = (hidden + kVec - 1) / kVec + 1 + 63;  // units from the 64-unit boundary before a ragged row to its end
  const int need = (span + lanes - 1) / lanes;
  const int64_t groups = wave_rows ? (tokens + 3) / 4 : tokens;
  const dim3 grid((unsigned)groups), block(256);
#define HQ_ROWS(LANES, KEEP)                                                                                    \
  hipLaunchKernelGGL((dynamic_quant_kernel<T, AZP, LANES, KEEP, VEC>), grid, block, 0, stream, in, out, scales, \
                     azps, tokens, hidden)
  if (wave_rows) {
    if (need <= 2) HQ_ROWS(64, 2);
    else if (need <= 3) HQ_ROWS(64, 3);
    else HQ_ROWS(64, 5);
  } else {
    if (need <= 2) HQ_ROWS(256, 2);
    else if (need <= 3) HQ_ROWS(256, 3);
    else HQ_ROWS(256, 5);
  }
#undef HQ_ROWS
}

template <typename T, bool AZP>
void launch_dynamic_azp(const T* in, int8_t* out, float* scales, int32_t* azps, int64_t tokens, int hidden,
                        const HqDevice* dev, hipStream_t stream) {
  if (pointers_aligned(in, out) && (tokens * hidden) % kVec == 0)
    launch_dynamic_vec<T, AZP, true>(in, out, scales, azps, tokens, hidden, dev, stream);
  else
    launch_dynamic_vec<T, AZP, false>(in, out, scales, azps, tokens, hidden, dev, stream);
}

template <typename T>
int launch_dynamic(const T* in, int8_t* out, float* scales, int32_t* azps, int64_t tokens, int hidden,
                   const HqDevice* dev, hipStream_t stream) {
  if (azps) launch_dynamic_azp<T, true>(in, out, scales, azps, tokens, hidden, dev, stream);
  else launch_dynamic_azp<T, false>(in, out, scales, azps, tokens, hidden, dev, stream);
  return hq_launch_status();
}

int check_common(const void* x, int x_dtype, const int8_t* out, int64_t tokens, int hidden) {
  if (tokens < 0 || hidden <= 0) return HQ_ERR_BAD_SHAPE;
  if (x_dtype != HQ_DTYPE_F32 && x_dtype != HQ_DTYPE_F16 && x_dtype != HQ_DTYPE_BF16) return HQ_ERR_BAD_ENUM;
  if (tokens == 0) return HQ_OK;
  if (!x || !out) return HQ_ERR_NULL_POINTER;
  if (tokens > 0x7fffffff) return HQ_ERR_TOO_LARGE;
  const int esz = x_dtype == HQ_DTYPE_F32 ? 4 : 2;
  if ((uintptr_t)x & (esz - 1)) return HQ_ERR_MISALIGNED;
  return HQ_OK;
}

}  // namespace

extern "C" int hq_int8_quant_static(const void* x, int x_dtype, int8_t* out, int64_t num_tokens, int hidden_size,
                                    float scale, int has_azp, int32_t azp, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  int rc = check_common(x, x_dtype, out, num_tokens, hidden_size);
  if (rc != HQ_OK || num_tokens == 0) return rc;
  const HqDevice* dev = nullptr;
  rc = hq_current_device(&dev);
  if (rc != HQ_OK) return rc;
  if (x_dtype == HQ_DTYPE_F32)
    return launch_static((const float*)x, out, num_tokens, hidden_size, scale, has_azp, azp, dev, stream);
  if (x_dtype == HQ_DTYPE_F16)
    return launch_static((const _Float16*)x, out, num_tokens, hidden_size, scale, has_azp, azp, dev, stream);
  return launch_static((const bf16_t*)x, out, num_tokens, hidden_size, scale, has_azp, azp, dev, stream);
}

extern "C" int hq_int8_quant_dynamic(const void* x, int x_dtype, int8_t* out, float* scales, int32_t* azp,
                                     int64_t num_tokens, int hidden_size, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  int rc = check_common(x, x_dtype, out, num_tokens, hidden_size);
  if (rc != HQ_OK || num_tokens == 0) return rc;
  if (!scales) return HQ_ERR_NULL_POINTER;
  if (((uintptr_t)scales & 3) || ((uintptr_t)azp & 3)) return HQ_ERR_MISALIGNED;
  const HqDevice* dev = nullptr;
  rc = hq_current_device(&dev);
  if (rc != HQ_OK) return rc;
  if (x_dtype == HQ_DTYPE_F32)
    return launch_dynamic((const float*)x, out, scales, azp, num_tokens, hidden_size, dev, stream);
  if (x_dtype == HQ_DTYPE_F16)
    return launch_dynamic((const _Float16*)x, out, scales, azp, num_tokens, hidden_size, dev, stream);
  return launch_dynamic((const bf16_t*)x, out, scales, azp, num_tokens, hidden_size, dev, stream);
}
