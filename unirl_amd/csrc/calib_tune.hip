// Measurement build only (python -m unirl_amd.build --tune): yardstick kernels for the benchmark
// (a plain copy that calibrates hardware byte counters, the launch floor of a streaming shape,
// a bare grid-wide reduction finished three ways) and the host side of the device timeline.
// None of this is part of libunirl_hip.so; the entry points are declared in unirl_tune.h.

#include <string>
#include <vector>

#include "common_hip.h"
#include "unirl_internal.h"
#include "unirl_tune.h"

namespace unirl {

// Plain streaming copy, the yardstick for hardware byte counters: it moves exactly `n_vec`*16
// bytes in and out.
__global__ __launch_bounds__(256) void calib_copy_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst,
                                                         size_t n_vec) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_vec; i += stride)
    stream_store16(dst + i, stream_load16(src + i));
}

// Launch-floor yardstick: reads `n_read` and writes `n_write` 16-byte vectors with no arithmetic
// and no dependence between the two streams, four vectors in flight per lane like the fused
// kernels.  `sink` only keeps the loads alive.
__global__ __launch_bounds__(256) void calib_stream_kernel(const u32x4* __restrict__ src, size_t n_read,
                                                           u32x4* __restrict__ dst, size_t n_write,
                                                           unsigned int* sink) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  const size_t n = n_read > n_write ? n_read : n_write;
  u32x4 acc = {0u, 0u, 0u, 0u};
  const u32x4 fill = {0x3f800000u, 0x3f800000u, 0x3f800000u, 0x3f800000u};
  for (size_t i0 = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i0 < n; i0 += 4 * stride) {
    u32x4 v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const size_t i = i0 + k * stride;
      v[k] = (i < n_read) ? stream_load16(src + i) : acc;
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const size_t i = i0 + k * stride;
      acc ^= v[k];
      if (i < n_write) stream_store16(dst + i, fill);
    }
  }
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) sink[0] = acc.x;  // practically never taken
}

// The dependent second launch of a two-launch reduction, reduced to its minimum: one wavefront, one store.
__global__ __launch_bounds__(64) void calib_tail_kernel(unsigned int* sink) {
  if (threadIdx.x == 0) sink[1] = 1u;
}

// ---------------------------------------------------------------------------
// Measurement aid: a grid-wide sum of `n_vec` 16-byte vectors of floats, finished three ways.
// It answers one question: what does finishing a reduction cost after the streaming part?
//   mode 0  the streaming kernel alone (one fp64 partial per workgroup stored, nothing finished)
//   mode 1  plus a second launch whose one workgroup adds the partials (what the library does)
//   mode 2  one launch: every workgroup publishes its partial as two 8-byte units
//           {32 payload bits, 32-bit call tag} with relaxed device-scope atomic stores, and the
//           last workgroup polls the units with device-scope atomic loads until all carry this
//           call's tag (bounded by a one-second clock budget), then adds them in index order and
//           advances the tag kept in the scratch buffer's first word.  No fence, no ticket, no
//           ordering between locations: each unit validates itself.
// ---------------------------------------------------------------------------
constexpr int kCalibThreads = 256;

__device__ __forceinline__ double calib_stream_sum(const u32x4* __restrict__ src, size_t n_vec, double* lds) {
  const size_t stride = (size_t)gridDim.x * kCalibThreads;
  float acc = 0.0f;
  for (size_t i0 = (size_t)blockIdx.x * kCalibThreads + threadIdx.x; i0 < n_vec; i0 += 4 * stride) {
    u32x4 v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const size_t i = i0 + k * stride;
      v[k] = (i < n_vec) ? stream_load16(src + i) : u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int k = 0; k < 4; ++k)
      acc += (__uint_as_float(v[k].x) + __uint_as_float(v[k].y)) + (__uint_as_float(v[k].z) + __uint_as_float(v[k].w));
  }
  return block_sum<double>((double)acc, lds);
}

__global__ __launch_bounds__(kCalibThreads) void calib_reduce_kernel(const u32x4* __restrict__ src, size_t n_vec,
                                                                    double* __restrict__ partials) {
  __shared__ double lds[kCalibThreads / kWave];
  const double part = calib_stream_sum(src, n_vec, lds);
  if (threadIdx.x == 0) partials[blockIdx.x] = part;
}

__global__ __launch_bounds__(kCalibThreads) void calib_reduce_finalize_kernel(const double* __restrict__ partials,
                                                                             unsigned int nblk, double* out) {
  __shared__ double lds[kCalibThreads / kWave];
  double x = 0.0;
  for (unsigned int j = threadIdx.x; j < nblk; j += kCalibThreads) x += partials[j];
  const double tot = block_sum<double>(x, lds);
  if (threadIdx.x == 0) out[0] = tot;
}

__global__ __launch_bounds__(kCalibThreads) void calib_reduce_polled_kernel(const u32x4* __restrict__ src, size_t n_vec,
                                                                           unsigned long long* ws, double* out) {
  __shared__ double lds[kCalibThreads / kWave];
  const unsigned int tag = (unsigned int)ws[0] + 1u;  // ws[0]: advanced by the previous call's last workgroup
  unsigned long long* units = ws + 2;
  const double part = calib_stream_sum(src, n_vec, lds);
  if (threadIdx.x < 2) {
    const unsigned long long bits = (unsigned long long)__double_as_longlong(part);
    const unsigned int half = (unsigned int)(threadIdx.x == 0 ? bits : bits >> 32);
    __hip_atomic_store(units + 2 * (size_t)blockIdx.x + threadIdx.x, ((unsigned long long)tag << 32) | half,
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  if (blockIdx.x != gridDim.x - 1) return;
  // The last workgroup in dispatch order finishes: every other workgroup is already running (or
  // done) when it starts, and none of them ever waits, so the poll below ends; the clock budget
  // makes sure it ends even if that reasoning were wrong (the result is then NaN).
  const long long t_start = wall_clock64();
  double x = 0.0;
  bool timed_out = false;
  for (unsigned int j = threadIdx.x; j < gridDim.x; j += kCalibThreads) {
    unsigned long long lo, hi;
    for (;;) {
      lo = __hip_atomic_load(units + 2 * (size_t)j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      hi = __hip_atomic_load(units + 2 * (size_t)j + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if ((unsigned int)(lo >> 32) == tag && (unsigned int)(hi >> 32) == tag) break;
      if (wall_clock64() - t_start > 100000000LL) {  // one second of the 100 MHz clock
        timed_out = true;
        break;
      }
    }
    if (timed_out) break;
    x += __longlong_as_double((long long)(((hi & 0xffffffffull) << 32) | (lo & 0xffffffffull)));
  }
  if (timed_out) x = __longlong_as_double(0x7ff8000000000000LL);
  // per-thread sums over j = t, t+256, ... then the workgroup: a fixed order
  const double tot = block_sum<double>(x, lds);
  if (threadIdx.x == 0) {
    out[0] = tot;
    __hip_atomic_store(ws, (unsigned long long)tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

}  // namespace unirl

using namespace unirl;

// The host side of the device timeline.
namespace unirl {
namespace {
struct TraceEntry { std::string name; unsigned int nblocks; size_t offset; };
unsigned long long* g_trace_buf = nullptr;
size_t g_trace_cap = 0, g_trace_cur = 0;  // in 8-byte words
std::vector<TraceEntry> g_trace_log;
}  // namespace
unsigned long long* trace_next(const char* name, unsigned int nblocks) {
  const size_t need = (size_t)nblocks * 4;
  if (!g_trace_buf || g_trace_cur + need > g_trace_cap) return nullptr;
  unsigned long long* p = g_trace_buf + g_trace_cur;
  g_trace_log.push_back({name, nblocks, g_trace_cur});
  g_trace_cur += need;
  return p;
}
}  // namespace unirl
extern "C" int unirl_trace_begin(void* buf, size_t bytes) {
  unirl::g_trace_buf = reinterpret_cast<unsigned long long*>(buf);
  unirl::g_trace_cap = bytes / 8;
  unirl::g_trace_cur = 0;
  unirl::g_trace_log.clear();
  return 0;
}
extern "C" int unirl_trace_count(void) { return (int)unirl::g_trace_log.size(); }
extern "C" const char* unirl_trace_entry(int i, unsigned int* nblocks, size_t* offset_words) {
  const auto& e = unirl::g_trace_log[(size_t)i];
  *nblocks = e.nblocks;
  *offset_words = e.offset;
  return e.name.c_str();
}

extern "C" int unirl_calib_copy(const void* src, void* dst, size_t bytes, void* stream) {
  if (!src || !dst) return UNIRL_E_NULL;
  if (bytes % 16 != 0) return UNIRL_E_SHAPE;
  if (!aligned_to(src, 16) || !aligned_to(dst, 16)) return UNIRL_E_ALIGN;
  if (bytes == 0) return UNIRL_OK;
  hipLaunchKernelGGL(calib_copy_kernel, dim3(8192), dim3(256), 0, (hipStream_t)stream,
                     reinterpret_cast<const u32x4*>(src), reinterpret_cast<u32x4*>(dst), bytes / 16);
  return (int)hipGetLastError();
}

extern "C" int unirl_calib_stream(const void* src, size_t read_bytes, void* dst, size_t write_bytes,
                                  int tail_launch, void* sink, void* stream) {
  if (!sink) return UNIRL_E_NULL;
  if ((read_bytes && !src) || (write_bytes && !dst)) return UNIRL_E_NULL;
  if (read_bytes % 16 != 0 || write_bytes % 16 != 0) return UNIRL_E_SHAPE;
  if (!aligned_to(src, 16) || !aligned_to(dst, 16) || !aligned_to(sink, 4)) return UNIRL_E_ALIGN;
  const size_t n_read = read_bytes / 16, n_write = write_bytes / 16;
  const size_t n = n_read > n_write ? n_read : n_write;
  hipStream_t st = (hipStream_t)stream;
  if (n > 0) {
    size_t blocks = (n + 256 * 4 - 1) / (256 * 4);
    if (blocks > 8192) blocks = 8192;
    hipLaunchKernelGGL(calib_stream_kernel, dim3((unsigned int)blocks), dim3(256), 0, st,
                       reinterpret_cast<const u32x4*>(src), n_read, reinterpret_cast<u32x4*>(dst), n_write,
                       reinterpret_cast<unsigned int*>(sink));
    const int rc = (int)hipGetLastError();
    if (rc != 0) return rc;
  }
  if (tail_launch) {
    hipLaunchKernelGGL(calib_tail_kernel, dim3(1), dim3(64), 0, st, reinterpret_cast<unsigned int*>(sink));
    return (int)hipGetLastError();
  }
  return UNIRL_OK;
}

extern "C" int unirl_calib_reduce(const void* src, size_t read_bytes, int mode, unsigned int n_workgroups,
                                  void* scratch, size_t scratch_bytes, double* out, void* stream) {
  if (!src || !scratch || !out) return UNIRL_E_NULL;
  if (mode < 0 || mode > 2) return UNIRL_E_DTYPE;
  if (read_bytes == 0 || read_bytes % 16 != 0 || n_workgroups < 1 || n_workgroups > 65535) return UNIRL_E_SHAPE;
  if (!aligned_to(src, 16) || !aligned_to(scratch, 16) || !aligned_to(out, 8)) return UNIRL_E_ALIGN;
  if (scratch_bytes < 16 + (size_t)n_workgroups * 16) return UNIRL_E_WORKSPACE;
  hipStream_t st = (hipStream_t)stream;
  const u32x4* s = reinterpret_cast<const u32x4*>(src);
  if (mode == 2) {
    hipLaunchKernelGGL(calib_reduce_polled_kernel, dim3(n_workgroups), dim3(kCalibThreads), 0, st, s, read_bytes / 16,
                       reinterpret_cast<unsigned long long*>(scratch), out);
    return (int)hipGetLastError();
  }
  double* partials = reinterpret_cast<double*>(scratch) + 2;
  hipLaunchKernelGGL(calib_reduce_kernel, dim3(n_workgroups), dim3(kCalibThreads), 0, st, s, read_bytes / 16, partials);
  int rc = (int)hipGetLastError();
  if (rc != 0 || mode == 0) return rc;
  hipLaunchKernelGGL(calib_reduce_finalize_kernel, dim3(1), dim3(kCalibThreads), 0, st, partials, n_workgroups, out);
  return (int)hipGetLastError();
}
