// Host-side declarations shared by the translation units of libunirl_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>
#include <type_traits>

#include "../../include/unirl_hip.h"

namespace unirl {

// Workspace: fp64 per-workgroup partials, written by a streaming kernel and read
// by its finalize kernel.  No state survives a call.
constexpr int64_t kMaxPartialBlocks = 2048;       // workgroups per reduced row
constexpr int64_t kPartialCapacity = 512 * 1024;  // doubles
constexpr size_t kWorkspaceBytes = (size_t)kPartialCapacity * sizeof(double);

inline double* ws_partials(void* ws) { return reinterpret_cast<double*>(ws); }

// Launch-shape knobs for measurement sweeps.  The shipped library is built without UNIRL_TUNE:
// every knob is then its compile-time default and the process environment is never read.  A
// build with -DUNIRL_TUNE (used for sweeps only) reads them from the environment at each call.
#ifdef UNIRL_TUNE
inline int64_t tune_int(const char* name, int64_t dflt) {
  const char* s = getenv(name);
  if (!s || !*s) return dflt;
  char* end = nullptr;
  const long long v = strtoll(s, &end, 10);
  return (end && *end == '\0' && v > 0) ? (int64_t)v : dflt;
}
#else
constexpr int64_t tune_int(const char*, int64_t dflt) { return dflt; }
#endif

// Device-side timeline for measurement builds (-DUNIRL_TRACE): every workgroup of a traced
// kernel stores four 100 MHz clock readings (start, two marks, end) into a buffer the host
// registered with unirl_trace_begin(); trace_next() hands each launch its own slice and logs the
// kernel's name.  In the shipped library all of this compiles to nothing.
#ifdef UNIRL_TRACE
unsigned long long* trace_next(const char* name, unsigned int nblocks);
#define UNIRL_TRACE_FIELD unsigned long long* trace;
#define UNIRL_TRACE_SET(A, name, nblocks) (A).trace = unirl::trace_next(name, nblocks)
#else
#define UNIRL_TRACE_FIELD
#define UNIRL_TRACE_SET(A, name, nblocks) ((void)0)
#endif

inline size_t dtype_size(int dt) { return dt == UNIRL_F32 ? 4 : 2; }
inline bool dtype_ok(int dt) { return dt == UNIRL_F32 || dt == UNIRL_BF16 || dt == UNIRL_F16; }
// NULL counts as aligned: optional pointers are checked only when present.
inline bool aligned_to(const void* p, size_t a) { return p == nullptr || (reinterpret_cast<uintptr_t>(p) % a) == 0; }
inline const void* offset_ptr(const void* p, int64_t elems, size_t elem_size) {
  return p ? (const void*)(reinterpret_cast<const char*>(p) + elems * (int64_t)elem_size) : nullptr;
}
inline float* offset_f32(float* p, int64_t elems) { return p ? p + elems : nullptr; }
inline const float* offset_f32(const float* p, int64_t elems) { return p ? p + elems : nullptr; }

}  // namespace unirl
