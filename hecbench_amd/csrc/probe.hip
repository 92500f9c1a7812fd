// Memory-system probes: what this device delivers to the simplest possible kernels, so that a benchmark
// line can set a kernel's rate beside a rate measured on the same box instead of a data-sheet figure only.
//   hq_probe_stream: a plain streaming read (mode 0) or copy (mode 1) of `bytes` bytes;
//   hq_probe_gather16: independent 16-byte reads at pseudo-random entries of a table (the access
//                      pattern of a code-book lookup), the rate of which is bounded by cache requests per
//                      second, not by bytes.
//   hq_probe_lds: LDS reads or writes of 32, 64 or 128 bits per lane at byte offsets the caller gives per
//                 lane, so that the hardware's bank-conflict counter can be read against patterns whose
//                 conflicts are known (and the operand layouts of the library's kernels checked with it).
// There is no counterpart in the HeCBench tree; the benchmark drivers call them for their report.
#include "hq_internal.h"

namespace {
typedef uint32_t u4v __attribute__((ext_vector_type(4)));

// units = 16-byte pieces, ONE per thread: on this part the plain grid - a workgroup's worth of loads per
// workgroup, 131072 workgroups for 512 MiB - streams faster than any grid-stride loop (512 MiB read: 6.98 TB/s
// against 5.6 TB/s with sixteen workgroups per compute unit and four loads in flight per thread, 6.76 TB/s with
// one trip of four loads per thread; copy 6.5 against 4.7 TB/s): the wave launcher is the better load scheduler.
template <bool COPY>
__global__ __launch_bounds__(256) void probe_stream_kernel(const u4v* __restrict__ src, u4v* __restrict__ dst,
                                                          long units, u4v* __restrict__ sink) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= units) return;
  const u4v v = __builtin_nontemporal_load(src + i);
  if (COPY) __builtin_nontemporal_store(v, dst + i);
  // keeps the load alive; the condition is false for any realistic data
  else if ((v.x & v.y & v.z & v.w) == 0xffffffffu && v.x + v.y == 12345u) *sink = v;
}

// every lane performs `per_lane` independent 16-byte reads, eight in flight at a time
__global__ __launch_bounds__(256) void probe_gather_kernel(const u4v* __restrict__ table, uint32_t mask, int per_lane,
                                                          u4v* __restrict__ sink) {
  uint32_t s = (blockIdx.x * 256u + threadIdx.x) * 2654435761u + 12345u;
  u4v acc = {0u, 0u, 0u, 0u};
  for (int i = 0; i < per_lane; i += 8) {
    u4v v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      s ^= s << 13; s ^= s >> 17; s ^= s << 5;  // xorshift32
      v[u] = table[s & mask];
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) acc ^= v[u];
  }
  if ((acc.x & acc.y & acc.z & acc.w) == 0xffffffffu && acc.x + acc.y == 12345u) *sink = acc;
}

// Every lane repeats one LDS access of WIDTH bits at its own byte offset (taken from a table of 64 offsets,
// the same for every wave) inside its wave's 8 KB.
template <int WIDTH, bool WRITE>
__global__ __launch_bounds__(256) void probe_lds_kernel(const uint32_t* __restrict__ offsets, int repeats,
                                                       u4v* __restrict__ sink) {
  __shared__ u4v buf[2048 + 256];  // 32 KB and a margin for the widest access at the last offset
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  for (int i = tid; i < 2048 + 256; i += 256) buf[i] = u4v{(uint32_t)i, 1u, 2u, 3u};
  __syncthreads();
  const uint32_t base = (uint32_t)(uintptr_t)buf + (uint32_t)wv * 8192u + (offsets[lane] & 8191u & ~(uint32_t)(WIDTH / 8 - 1));
  u4v acc = {0u, 0u, 0u, 0u};
  for (int r = 0; r < repeats; ++r) {
    const uint32_t p = base;
    if (WRITE) {
      const u4v v = {acc.x + (uint32_t)r, 1u, 2u, 3u};
      if (WIDTH == 32) asm volatile("ds_write_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" ::"v"(p), "v"(v.x) : "memory");
      else if (WIDTH == 64) asm volatile("ds_write_b64 %0, %1\n\ts_waitcnt lgkmcnt(0)" ::"v"(p), "v"(((uint64_t)v.y << 32) | v.x) : "memory");
      else asm volatile("ds_write_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" ::"v"(p), "v"(v) : "memory");
    } else if (WIDTH == 32) {
      uint32_t v;
      asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(p) : "memory");
      acc.x ^= v;
    } else if (WIDTH == 64) {
      uint64_t v;
      asm volatile("ds_read_b64 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(p) : "memory");
      acc.x ^= (uint32_t)v; acc.y ^= (uint32_t)(v >> 32);
    } else {
      u4v v;
      asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(p) : "memory");
      acc ^= v;
    }
  }
  if ((acc.x & acc.y & acc.z & acc.w) == 0xffffffffu && acc.x + acc.y == 12345u) *sink = acc;
}
}  // namespace

extern "C" int hq_probe_stream(int mode, const void* src, void* dst, int64_t bytes, void* stream) {
  if (!src || !dst) return HQ_ERR_NULL_POINTER;
  if (mode != 0 && mode != 1) return HQ_ERR_BAD_ENUM;
  if (bytes < 16 || (bytes & 15)) return HQ_ERR_BAD_SHAPE;
  if (((uintptr_t)src & 15) || ((uintptr_t)dst & 15)) return HQ_ERR_MISALIGNED;
  const HqDevice* dev = nullptr;
  const int rc = hq_current_device(&dev);
  if (rc != HQ_OK) return rc;
  const long units = bytes / 16;
  const long wgs = (units + 255) / 256;
  if (wgs > 0x7fffffffL) return HQ_ERR_TOO_LARGE;
  if (mode == 1)
    hipLaunchKernelGGL(probe_stream_kernel<true>, dim3((unsigned)wgs), dim3(256), 0, (hipStream_t)stream,
                       (const u4v*)src, (u4v*)dst, units, (u4v*)dst);
  else  // mode 0 writes nothing (dst is only the never-taken sink)
    hipLaunchKernelGGL(probe_stream_kernel<false>, dim3((unsigned)wgs), dim3(256), 0, (hipStream_t)stream,
                       (const u4v*)src, (u4v*)dst, units, (u4v*)dst);
  return hq_launch_status();
}

extern "C" int hq_probe_gather16(const void* table, int64_t table_bytes, int64_t gathers, void* sink16, void* stream) {
  if (!table || !sink16) return HQ_ERR_NULL_POINTER;
  if (table_bytes < 16 || (table_bytes & (table_bytes - 1)) || table_bytes > ((int64_t)1 << 32)) return HQ_ERR_BAD_SHAPE;
  if (gathers <= 0) return HQ_ERR_BAD_SHAPE;
  if (((uintptr_t)table & 15) || ((uintptr_t)sink16 & 15)) return HQ_ERR_MISALIGNED;
  const HqDevice* dev = nullptr;
  const int rc = hq_current_device(&dev);
  if (rc != HQ_OK) return rc;
  // eight workgroups per compute unit; the number of reads is rounded up to a whole trip of every lane
  const long lanes = (long)dev->cus * 8 * 256;
  long per_lane = (gathers + lanes - 1) / lanes;
  per_lane = (per_lane + 7) / 8 * 8;
  if (per_lane > (1 << 24)) return HQ_ERR_TOO_LARGE;
  hipLaunchKernelGGL(probe_gather_kernel, dim3((unsigned)(dev->cus * 8)), dim3(256), 0, (hipStream_t)stream,
                     (const u4v*)table, (uint32_t)(table_bytes / 16 - 1), (int)per_lane, (u4v*)sink16);
  return hq_launch_status();
}

extern "C" int64_t hq_probe_gather16_count(int64_t gathers) {
  const HqDevice* dev = nullptr;
  if (gathers <= 0 || hq_current_device(&dev) != HQ_OK) return -1;
  const long lanes = (long)dev->cus * 8 * 256;
  long per_lane = (gathers + lanes - 1) / lanes;
  per_lane = (per_lane + 7) / 8 * 8;
  return per_lane * lanes;
}

extern "C" int hq_probe_lds(const uint32_t* offsets64, int width_bits, int write, int repeats, void* sink16,
                            void* stream) {
  if (!offsets64 || !sink16) return HQ_ERR_NULL_POINTER;
  if (width_bits != 32 && width_bits != 64 && width_bits != 128) return HQ_ERR_BAD_ENUM;
  if (repeats <= 0 || repeats > (1 << 20)) return HQ_ERR_BAD_SHAPE;
  if (((uintptr_t)sink16 & 15) || ((uintptr_t)offsets64 & 3)) return HQ_ERR_MISALIGNED;
  const HqDevice* dev = nullptr;
  const int rc = hq_current_device(&dev);
  if (rc != HQ_OK) return rc;
  const dim3 grid((unsigned)dev->cus), block(256);
#define HQ_PROBE_LDS(W, WR) \
  hipLaunchKernelGGL((probe_lds_kernel<W, WR>), grid, block, 0, (hipStream_t)stream, offsets64, repeats, (u4v*)sink16)
  if (write) {
    if (width_bits == 32) HQ_PROBE_LDS(32, true); else if (width_bits == 64) HQ_PROBE_LDS(64, true); else HQ_PROBE_LDS(128, true);
  } else {
    if (width_bits == 32) HQ_PROBE_LDS(32, false); else if (width_bits == 64) HQ_PROBE_LDS(64, false); else HQ_PROBE_LDS(128, false);
  }
#undef HQ_PROBE_LDS
  return hq_launch_status();
}
