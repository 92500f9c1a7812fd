// Internal helpers shared by the libhq translation units (not part of the ABI).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/hq.h"

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
// Allocated on first use and grown on demand; never freed while the process runs.
int hq_get_workspace(hipStream_t stream, size_t need_floats, size_t need_counters,
                     HqWorkspace* out);

// Integer tuning knob from the environment (used by the benchmark drivers to
// sweep launch shapes); returns dflt when unset or unparsable.
int hq_env_int(const char* name, int dflt);
