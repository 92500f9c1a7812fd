// Library-wide state of libhq: device facts, per-stream workspaces, error text.
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <utility>

#include "hq_internal.h"

namespace {
std::mutex g_mu;
std::map<int, HqDevice> g_devices;
std::map<std::pair<int, hipStream_t>, HqWorkspace> g_workspaces;
}  // namespace

int hq_env_int(const char* name, int dflt) {
  const char* v = std::getenv(name);
  if (!v || !*v) return dflt;
  char* end = nullptr;
  long r = std::strtol(v, &end, 10);
  return (end && *end == '\0') ? (int)r : dflt;
}

int hq_current_device(const HqDevice** out) {
  int dev = 0;
  HQ_HIP_TRY(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lk(g_mu);
  auto it = g_devices.find(dev);
  if (it == g_devices.end()) {
    hipDeviceProp_t p;
    HQ_HIP_TRY(hipGetDeviceProperties(&p, dev));
    HqDevice d;
    d.ordinal = dev;
    d.cus = p.multiProcessorCount;
    d.lds_per_cu = (int)p.maxSharedMemoryPerMultiProcessor;
    d.ok = std::strncmp(p.gcnArchName, "gfx950", 6) == 0 && p.warpSize == 64;
    it = g_devices.emplace(dev, d).first;
  }
  if (!it->second.ok) return HQ_ERR_UNSUPPORTED_DEVICE;
  *out = &it->second;
  return HQ_OK;
}

int hq_get_workspace(hipStream_t stream, size_t need_floats, size_t need_counters,
                     HqWorkspace* out) {
  int dev = 0;
  HQ_HIP_TRY(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lk(g_mu);
  HqWorkspace& ws = g_workspaces[std::make_pair(dev, stream)];
  if (ws.partial_floats < need_floats) {
    size_t n = need_floats < (1u << 20) ? (1u << 20) : need_floats;
    float* p = nullptr;
    HQ_HIP_TRY(hipMalloc((void**)&p, n * sizeof(float)));
    // The previous buffer may still be read by kernels in flight: keep it.
    ws.partial = p;
    ws.partial_floats = n;
  }
  if (ws.ncounters < need_counters) {
    size_t n = need_counters < (1u << 14) ? (1u << 14) : need_counters;
    unsigned* c = nullptr;
    HQ_HIP_TRY(hipMalloc((void**)&c, n * sizeof(unsigned)));
    HQ_HIP_TRY(hipMemset(c, 0, n * sizeof(unsigned)));
    ws.counters = c;
    ws.ncounters = n;
  }
  *out = ws;
  return HQ_OK;
}

extern "C" int hq_abi_version(void) { return 1; }

extern "C" const char* hq_strerror(int code) {
  switch (code) {
    case HQ_OK: return "ok";
    case HQ_ERR_NULL_POINTER: return "hq: null pointer argument";
    case HQ_ERR_BAD_SHAPE: return "hq: shape argument out of range or not a multiple of the required tile";
    case HQ_ERR_BAD_ENUM: return "hq: unknown dtype / table / flag value";
    case HQ_ERR_MISALIGNED: return "hq: pointer not aligned as required";
    case HQ_ERR_UNSUPPORTED_DEVICE: return "hq: current device is not a gfx950 (MI355X) GPU";
    case HQ_ERR_TOO_LARGE: return "hq: problem exceeds the library's limits";
    default: break;
  }
  if (code > 0) return hipGetErrorString((hipError_t)code);
  return "hq: unknown error code";
}

extern "C" int hq_init(void) {
  const HqDevice* d = nullptr;
  int rc = hq_current_device(&d);
  if (rc != HQ_OK) return rc;
  HqWorkspace ws;
  return hq_get_workspace(nullptr, 1, 1, &ws);
}

extern "C" int hq_device_info(int* compute_units, int* wavefront_size, int* lds_bytes_per_cu,
                              int* memory_clock_khz, int* memory_bus_bits, char* name,
                              int name_len) {
  int dev = 0;
  HQ_HIP_TRY(hipGetDevice(&dev));
  hipDeviceProp_t p;
  HQ_HIP_TRY(hipGetDeviceProperties(&p, dev));
  if (compute_units) *compute_units = p.multiProcessorCount;
  if (wavefront_size) *wavefront_size = p.warpSize;
  if (lds_bytes_per_cu) *lds_bytes_per_cu = (int)p.maxSharedMemoryPerMultiProcessor;
  if (memory_clock_khz) *memory_clock_khz = p.memoryClockRate;
  if (memory_bus_bits) *memory_bus_bits = p.memoryBusWidth;
  if (name && name_len > 0) {
    std::snprintf(name, (size_t)name_len, "%s (%s)", p.name, p.gcnArchName);
  }
  return HQ_OK;
}
