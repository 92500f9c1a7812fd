// Library-wide state of libhq: device facts, per-stream workspaces, error text.
#include <atomic>
#include <climits>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <utility>
#include <vector>

#include "hq_internal.h"

namespace {
std::mutex g_mu;
std::map<int, HqDevice> g_devices;
std::map<std::pair<int, hipStream_t>, HqWorkspace> g_workspaces;
std::vector<std::pair<int, void*>> g_retired;  // outgrown buffers, freed by hq_shutdown()
}  // namespace

// ---- launch-shape overrides ------------------------------------------------------------------
// Every knob is an int that is "unset" by default.  The environment variable of the same name is
// read ONCE (first use), hq_set_tunable() changes a knob at run time; a launch path reads a knob
// with one relaxed atomic load, never the environment.
namespace {
const char* const kTunableNames[HQ_TUNE_COUNT] = {
    "HQ_Q3_WAVES", "HQ_Q3_STEPS", "HQ_Q3_KSPLIT", "HQ_Q3_TILE", "HQ_Q3_SMALL_BATCH", "HQ_Q3_ROW_BLOCKS", "HQ_LUT_PATH", "HQ_LUT_KSPLIT", "HQ_NF4_PIPE",
    "HQ_AQLM_ROWS", "HQ_Q8_WGS", "HQ_Q8_FAST", "HQ_GEMV_LDS", "HQ_GEMV_SPLIT", "HQ_SPLITK_FENCES"};
constexpr int kUnset = INT_MIN;
std::atomic<int> g_tunables[HQ_TUNE_COUNT];
std::once_flag g_tunables_once;

void seed_tunables_from_env() {
  for (int i = 0; i < HQ_TUNE_COUNT; ++i) {
    int v = kUnset;
    const char* e = std::getenv(kTunableNames[i]);
    if (e && *e) {
      char* end = nullptr;
      const long r = std::strtol(e, &end, 10);
      if (end && *end == '\0') v = (int)r;
    }
    g_tunables[i].store(v, std::memory_order_relaxed);
  }
}
}  // namespace

int hq_tune(HqTunable id, int dflt) {
  std::call_once(g_tunables_once, seed_tunables_from_env);
  const int v = g_tunables[id].load(std::memory_order_relaxed);
  return v == kUnset ? dflt : v;
}

extern "C" int hq_set_tunable(const char* name, int value, int clear) {
  if (!name) return HQ_ERR_NULL_POINTER;
  std::call_once(g_tunables_once, seed_tunables_from_env);
  for (int i = 0; i < HQ_TUNE_COUNT; ++i)
    if (std::strcmp(name, kTunableNames[i]) == 0) {
      g_tunables[i].store(clear ? kUnset : value, std::memory_order_relaxed);
      return HQ_OK;
    }
  return HQ_ERR_BAD_ENUM;
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
    // grow geometrically: a stream that sees larger and larger problems allocates O(log) times
    size_t n = ws.partial_floats ? ws.partial_floats * 2 : (size_t)1 << 20;
    while (n < need_floats) n *= 2;
    float* p = nullptr;
    HQ_HIP_TRY(hipMalloc((void**)&p, n * sizeof(float)));
    // kernels in flight may still read the previous buffer: it is kept until hq_shutdown()
    if (ws.partial) g_retired.push_back(std::make_pair(dev, (void*)ws.partial));
    ws.partial = p;
    ws.partial_floats = n;
  }
  if (ws.ncounters < need_counters) {
    size_t n = ws.ncounters ? ws.ncounters * 2 : (size_t)1 << 14;
    while (n < need_counters) n *= 2;
    unsigned* c = nullptr;
    HQ_HIP_TRY(hipMalloc((void**)&c, n * sizeof(unsigned)));
    HQ_HIP_TRY(hipMemset(c, 0, n * sizeof(unsigned)));
    if (ws.counters) g_retired.push_back(std::make_pair(dev, (void*)ws.counters));
    ws.counters = c;
    ws.ncounters = n;
  }
  *out = ws;
  return HQ_OK;
}

// Upper bound of what any hq_q3_matvec call with K <= max_K, N <= max_N (any batch) and any hq_lut_gemv call
// of those sizes takes from its stream's workspace on a device of `cus` compute units, with the default launch
// policy.  Host arithmetic only.  (tests/test_workspace_cpu.py checks it against the per-call need over a
// sweep of shapes.)
static void reserve_bound(int cus, int max_K, int max_N, size_t* floats, size_t* counters) {
  // batched GEMM: re-ordered activations of 64 rows (128 bytes per input feature, K padded to 1024), the row
  // sums and scales, and - whenever some N <= max_N leaves compute units without a 128-column tile and K has
  // two or more ranges of four steps, i.e. always but for very short K - the raw sums of its K split, at most
  // 256 blocks of 64 x 128
  const size_t kpad = ((size_t)max_K + 1023) / 1024 * 1024;
  const size_t gemm_floats = kpad * 32 + 128 + (kpad >= 2048 ? (size_t)256 * 64 * 128 : 0);
  // split-K matvecs: a partial row of 64 floats per column tile and split - one split per 4096 elements of K
  // (a shorter K than max_K splits no further); narrow tiles (16 or 32 columns) only while tiles x splits stay
  // within the compute units.  The LUT kernels: two workgroups per compute unit, 128 floats each.
  const size_t tiles = ((size_t)max_N + 63) / 64;
  const size_t rounds = ((size_t)max_K + 4095) / 4096;
  const size_t full_split = tiles * rounds;
  const size_t per_cu = tiles + 2 * (size_t)cus;
  size_t split_floats = (full_split > per_cu ? full_split : per_cu) * 64 * 2;
  // batches 2 ... 64 on the matvec-like kernel: one partial row per tile, range of K and activation row, at most
  // 8192 of them whatever the shape
  if ((size_t)8192 * 64 > split_floats) split_floats = (size_t)8192 * 64;
  *floats = gemm_floats > split_floats ? gemm_floats : split_floats;
  // arrival counters: one per column tile, narrow tiles four per 64 columns, row blocks sixteen per tile
  *counters = tiles > 1 ? tiles * 16 : 16;
}

extern "C" int hq_reserve_need(int compute_units, int max_K, int max_N, int64_t* floats, int64_t* counters) {
  if (!floats || !counters) return HQ_ERR_NULL_POINTER;
  if (max_K < 0 || max_N < 0 || compute_units <= 0) return HQ_ERR_BAD_SHAPE;
  size_t f = 0, c = 0;
  reserve_bound(compute_units, max_K, max_N, &f, &c);
  *floats = (int64_t)f;
  *counters = (int64_t)c;
  return HQ_OK;
}

extern "C" int hq_reserve_workspace(void* stream, int max_K, int max_N) {
  if (max_K < 0 || max_N < 0) return HQ_ERR_BAD_SHAPE;
  const HqDevice* d = nullptr;
  int rc = hq_current_device(&d);
  if (rc != HQ_OK) return rc;
  size_t floats = 0, counters = 0;
  reserve_bound(d->cus, max_K, max_N, &floats, &counters);
  HqWorkspace ws;
  return hq_get_workspace((hipStream_t)stream, floats, counters, &ws);
}

extern "C" int hq_shutdown(void) {
  HQ_HIP_TRY(hipDeviceSynchronize());
  std::lock_guard<std::mutex> lk(g_mu);
  int cur = 0;
  HQ_HIP_TRY(hipGetDevice(&cur));
  int rc = HQ_OK;
  auto release = [&](int dev, void* p) {
    if (!p) return;
    hipError_t e = hipSetDevice(dev);
    if (e == hipSuccess) e = hipDeviceSynchronize();
    if (e == hipSuccess) e = hipFree(p);
    if (e != hipSuccess && rc == HQ_OK) rc = (int)e;
  };
  for (auto& kv : g_workspaces) {
    release(kv.first.first, kv.second.partial);
    release(kv.first.first, kv.second.counters);
  }
  for (auto& r : g_retired) release(r.first, r.second);
  g_workspaces.clear();
  g_retired.clear();
  (void)hipSetDevice(cur);
  return rc;
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
  rc = hq_get_workspace(nullptr, 1, 1, &ws);
  if (rc != HQ_OK) return rc;
  return hq_noalloc_setup();  // this device's address of the fixed scratch of hq_q3_matvec_noalloc
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
