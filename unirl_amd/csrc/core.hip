// Library-level entry points: ABI version, status strings, workspace set-up.

#include "common_hip.h"
#include "unirl_internal.h"

namespace unirl {

__global__ __launch_bounds__(256) void fill_zero_kernel(uint32_t* p, size_t n_words) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_words; i += stride) p[i] = 0u;
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
