// Internal helpers shared by the libhq translation units (not part of the ABI).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/hq.h"

// internal flag bit of the split-K kernels: formal release/acquire fences in the arrival protocol
#define HQ_FLAG_STRICT_FENCES 0x80000000u

#define HQ_HIP_TRY(expr)                      \
  do {                                        \
    hipError_t hq_e_ = (expr);                \
    if (hq_e_ != hipSuccess) return (int)hq_e_; \
  } while (0)

// Returns the launch status of the kernel just enqueued as an hq return code.
static inline int hq_launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? HQ_OK : (int)e;
}

struct HqDevice {
  int ordinal;
  int cus;         // compute units reported by hipGetDeviceProperties
  int lds_per_cu;  // bytes
  bool ok;         // gfx950
};

// Device facts for the current device (cached per ordinal).  Returns an hq code.
int hq_current_device(const HqDevice** out);

struct HqWorkspace {
  float* partial;      // split-K partial sums
  unsigned* counters;  // arrival counters, zero between calls (self-resetting)
  size_t partial_floats;
  size_t ncounters;
};

// Workspace of (current device, stream) holding at least the requested sizes.
// Allocated on first use, grown geometrically on demand, freed by hq_shutdown().
int hq_get_workspace(hipStream_t stream, size_t need_floats, size_t need_counters,
                     HqWorkspace* out);

// Caller-provided scratch of the GPTQ 3-bit paths (the entry point that allocates nothing passes its
// fixed device array here; a null pointer means "use the stream's workspace").
struct HqQ3Scratch {
  float* partial;          // split-K partial sums, also the batched GEMM's re-ordered activations
  size_t partial_floats;
  float* rows;             // 128 floats: row sums and row scales of the batched GEMM
  unsigned* counters;      // split-K arrival counters (cleared by the call that uses them)
  size_t ncounters;
  float* sums;             // raw sums of the batched GEMM's K split
  size_t sums_floats;
};
int hq_q3_matvec_impl(const void* x, int x_dtype, const int32_t* qweight, const float* scales, const float* zeros,
                      float* y, int K, int N, int batch_M, unsigned flags, hipStream_t stream,
                      const HqQ3Scratch* fixed);
// Resolves the current device's copy of the fixed scratch array (once per device).
int hq_noalloc_setup(void);

// Launch-shape overrides for tests and sweeps (hq_set_tunable, or the environment variable of the
// same name, which is read once per process).  hq_tune returns dflt while a knob is unset; it costs
// one relaxed atomic load.
enum HqTunable {
  HQ_TUNE_Q3_WAVES, HQ_TUNE_Q3_STEPS, HQ_TUNE_Q3_KSPLIT, HQ_TUNE_Q3_TILE, HQ_TUNE_Q3_SMALL_BATCH, HQ_TUNE_Q3_ROW_BLOCKS, HQ_TUNE_LUT_PATH, HQ_TUNE_LUT_KSPLIT,
  HQ_TUNE_NF4_PIPE, HQ_TUNE_AQLM_ROWS, HQ_TUNE_Q8_WGS, HQ_TUNE_Q8_FAST, HQ_TUNE_GEMV_LDS, HQ_TUNE_GEMV_SPLIT, HQ_TUNE_SPLITK_FENCES, HQ_TUNE_COUNT
};
int hq_tune(HqTunable id, int dflt);

// Sum of the nsplit partial sums p[s * stride] of a K split, added in split order (the result does not depend
// on which workgroup arrived last).  The loads are device-scope atomic loads, which bypass the non-coherent
// cache levels; eight of them are in flight at a time - one after the other each costs a trip to memory, and
// the last workgroup of a tile is the last thing a kernel does.
__device__ __forceinline__ float hq_sum_partials(const float* p, size_t stride, int nsplit) {
  float sum = 0.f;
  for (int s0 = 0; s0 < nsplit; s0 += 8) {
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int s = s0 + j < nsplit ? s0 + j : nsplit - 1;
      v[j] = __hip_atomic_load(p + (size_t)s * stride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) sum += s0 + j < nsplit ? v[j] : 0.f;
  }
  return sum;
}

// Streaming stores: write-through (sc1) and nontemporal (nt), i.e. the data is on its way to memory at once
// and is not kept in the L2.  For a 33.5 MB write stream on MI355X: 5.80 us against 6.46 us with nt alone
// and 7.04 us with plain stores.  The compiler cannot see that the assembly is a store, so the wait states it
// would put between a store of more than 64 bits and the next write to the data registers are part of the
// assembly.
typedef uint32_t hq_u2v __attribute__((ext_vector_type(2)));
typedef uint32_t hq_u4v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void hq_store_stream(hq_u4v* p, hq_u4v v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void hq_store_stream(hq_u2v* p, hq_u2v v) {
  asm volatile("global_store_dwordx2 %0, %1, off sc1 nt" ::"v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void hq_store_stream(uint32_t* p, uint32_t v) {
  asm volatile("global_store_dword %0, %1, off sc1 nt" ::"v"(p), "v"(v) : "memory");
}
