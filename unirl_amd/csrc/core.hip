// Library-level entry points: ABI version, status strings, workspace set-up.

#include "common.cuh"
#include "unirl_internal.h"

namespace unirl {

__global__ __launch_bounds__(256) void fill_zero_kernel(uint32_t* p, size_t n_words) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_words; i += stride) p[i] = 0u;
}

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

}  // namespace unirl

using namespace unirl;

extern "C" int unirl_abi_version(void) { return UNIRL_ABI_VERSION; }

extern "C" const char* unirl_status_string(int status) {
  switch (status) {
    case UNIRL_OK: return "ok";
    case UNIRL_E_NULL: return "a required pointer is NULL";
    case UNIRL_E_SHAPE: return "negative or inconsistent extent";
    case UNIRL_E_DTYPE: return "unknown dtype, kind or mode";
    case UNIRL_E_WORKSPACE: return "workspace missing or smaller than unirl_workspace_bytes()";
    case UNIRL_E_ALIGN: return "pointer not aligned to its element size";
    case UNIRL_E_LIMIT: return "extent beyond a documented limit";
  }
  if (status > 0) return hipGetErrorString((hipError_t)status);
  return "unknown status";
}

extern "C" size_t unirl_workspace_bytes(void) { return kWorkspaceBytes; }

extern "C" int unirl_workspace_init(void* workspace, size_t workspace_bytes, void* stream) {
  if (!workspace) return UNIRL_E_NULL;
  if (workspace_bytes < kWorkspaceBytes) return UNIRL_E_WORKSPACE;
  if (!aligned_to(workspace, 16)) return UNIRL_E_ALIGN;
  // Nothing in the library depends on the contents; the fill only gives a fresh allocation defined
  // values.  A fill kernel rather than a memset node, so the call is safe to capture in a graph.
  hipLaunchKernelGGL(fill_zero_kernel, dim3(256), dim3(256), 0, (hipStream_t)stream,
                     reinterpret_cast<uint32_t*>(workspace), workspace_bytes / 4);
  return (int)hipGetLastError();
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
