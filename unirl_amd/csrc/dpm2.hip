// One step of the deterministic DPM-Solver-2 sampler of unirl/sde/kernels.py:360-471
// (_convert_model_output, the DDIM / first-order / second-order updates of _dpm_step).
//
// The reference computes the step's scalar coefficients from the sigma schedule as 0-dim
// tensors (float64 for the two DPM updates) and then runs six to twelve element-wise fp32 ops;
// here the host passes the coefficients already rounded to fp32 -- the value torch multiplies
// the fp32 tensors by -- and one kernel does the element-wise part in the reference's order of
// operations (no contraction: every product and sum rounds on its own):
//   x0   = sample - sigma * model_output                               :366-367
//   DDIM : eps = (sample - (1-s) * x0) / s;  prev = (1-t) * x0 + sqrt(t^2) * eps      :449-453
//   1st  : prev = (sigma_t/sigma_s) * sample - (alpha_t (e^-h - 1)) * x0              :391
//   2nd  : D1 = (1/r0) * (x0 - x0_prev);  prev = c1 * sample - c2 * x0 - (0.5 c2) * D1   :416-425
// x0 is the solver's state (the next step's x0_prev) and is written next to prev.
//
// HBM traffic: model_output and sample read once (+ x0_prev for the second order), x0 and prev
// written once: 16 (20) bytes per element for fp32 inputs.

#include "common_hip.h"
#include "unirl_internal.h"

namespace unirl {

constexpr int kDpmThreads = 256;

struct DpmArgs {
  const void* v;
  const void* x;
  const float* x0_prev;
  unirl_dpm2_coeffs c;
  int64_t n;
  float* x0_out;
  float* prev_out;
};

template <int BRANCH>
__device__ __forceinline__ void dpm_elem(const unirl_dpm2_coeffs& c, float v, float x, float m1, float& x0,
                                         float& prev) {
  x0 = x - c.sigma * v;
  if (BRANCH == UNIRL_DPM2_DDIM) {
    const float eps = (x - c.one_minus_s * x0) / c.s;
    prev = c.one_minus_t * x0 + c.sqrt_t2 * eps;
  } else if (BRANCH == UNIRL_DPM2_FIRST) {
    prev = c.c1 * x - c.c2 * x0;
  } else {
    const float d1 = c.inv_r0 * (x0 - m1);
    prev = (c.c1 * x - c.c2 * x0) - c.half_c2 * d1;
  }
}

template <typename TV, typename TX, int VEC, int BRANCH>
__global__ __launch_bounds__(kDpmThreads) void dpm2_step_kernel(DpmArgs A) {
  const TV* __restrict__ vp = reinterpret_cast<const TV*>(A.v);
  const TX* __restrict__ xp = reinterpret_cast<const TX*>(A.x);
  const int64_t nvec = A.n / VEC;
  const int64_t stride = (int64_t)gridDim.x * kDpmThreads;
  for (int64_t i = (int64_t)blockIdx.x * kDpmThreads + threadIdx.x; i < nvec; i += stride) {
    float v[VEC], x[VEC], m1[VEC], x0[VEC], prev[VEC];
    Vec<TV, VEC>::load(vp + i * VEC, v);
    Vec<TX, VEC>::load(xp + i * VEC, x);
    if (BRANCH == UNIRL_DPM2_SECOND) Vec<float, VEC>::load(A.x0_prev + i * VEC, m1);
#pragma unroll
    for (int k = 0; k < VEC; ++k)
      dpm_elem<BRANCH>(A.c, v[k], x[k], BRANCH == UNIRL_DPM2_SECOND ? m1[k] : 0.0f, x0[k], prev[k]);
    Vec<float, VEC>::store(A.x0_out + i * VEC, x0);
    Vec<float, VEC>::store(A.prev_out + i * VEC, prev);
  }
  // the last n % VEC elements, one lane each
  const int64_t t = nvec * VEC + (int64_t)blockIdx.x * kDpmThreads + threadIdx.x;
  if (t < A.n) {
    float x0, prev;
    dpm_elem<BRANCH>(A.c, Elem<TV>::load(vp + t), Elem<TX>::load(xp + t),
                     BRANCH == UNIRL_DPM2_SECOND ? A.x0_prev[t] : 0.0f, x0, prev);
    A.x0_out[t] = x0;
    A.prev_out[t] = prev;
  }
}

template <typename TV, typename TX, int VEC>
static int launch_dpm_branch(const DpmArgs& A, int branch, dim3 grid, hipStream_t st) {
  dim3 block(kDpmThreads);
  if (branch == UNIRL_DPM2_DDIM)
    hipLaunchKernelGGL((dpm2_step_kernel<TV, TX, VEC, UNIRL_DPM2_DDIM>), grid, block, 0, st, A);
  else if (branch == UNIRL_DPM2_FIRST)
    hipLaunchKernelGGL((dpm2_step_kernel<TV, TX, VEC, UNIRL_DPM2_FIRST>), grid, block, 0, st, A);
  else
    hipLaunchKernelGGL((dpm2_step_kernel<TV, TX, VEC, UNIRL_DPM2_SECOND>), grid, block, 0, st, A);
  return (int)hipGetLastError();
}

template <typename TV, typename TX>
static int launch_dpm(const DpmArgs& A, int branch, hipStream_t st) {
  // four elements per lane when every pointer allows 16-byte fp32 (8-byte 16-bit) accesses
  bool vec4 = aligned_to(A.v, 4 * sizeof(TV)) && aligned_to(A.x, 4 * sizeof(TX)) && aligned_to(A.x0_prev, 16) &&
              aligned_to(A.x0_out, 16) && aligned_to(A.prev_out, 16);
  const int64_t per = vec4 ? 4 : 1;
  int64_t nblk = (A.n / per + kDpmThreads - 1) / kDpmThreads;
  if (nblk > 8192) nblk = 8192;
  if (nblk < 1) nblk = 1;
  dim3 grid((unsigned int)nblk);
  return vec4 ? launch_dpm_branch<TV, TX, 4>(A, branch, grid, st) : launch_dpm_branch<TV, TX, 1>(A, branch, grid, st);
}

template <typename TV>
static int launch_dpm_x(const DpmArgs& A, int dtype_x, int branch, hipStream_t st) {
  switch (dtype_x) {
    case UNIRL_F32: return launch_dpm<TV, float>(A, branch, st);
    case UNIRL_BF16: return launch_dpm<TV, bf16_t>(A, branch, st);
    case UNIRL_F16: return launch_dpm<TV, f16_t>(A, branch, st);
  }
  return UNIRL_E_DTYPE;
}

}  // namespace unirl

using namespace unirl;

extern "C" int unirl_dpm2_step(const void* model_output, int dtype_v, const void* sample, int dtype_x,
                               const float* x0_prev, int branch, const unirl_dpm2_coeffs* coeffs, int64_t n,
                               float* x0_out, float* prev_out, void* stream) {
  if (!dtype_ok(dtype_v) || !dtype_ok(dtype_x)) return UNIRL_E_DTYPE;
  if (branch != UNIRL_DPM2_DDIM && branch != UNIRL_DPM2_FIRST && branch != UNIRL_DPM2_SECOND) return UNIRL_E_DTYPE;
  if (n < 0) return UNIRL_E_SHAPE;
  if (!coeffs) return UNIRL_E_NULL;
  if (n == 0) return UNIRL_OK;
  if (!model_output || !sample || !x0_out || !prev_out) return UNIRL_E_NULL;
  if (branch == UNIRL_DPM2_SECOND && !x0_prev) return UNIRL_E_NULL;
  if (!aligned_to(model_output, dtype_size(dtype_v)) || !aligned_to(sample, dtype_size(dtype_x)) ||
      !aligned_to(x0_prev, 4) || !aligned_to(x0_out, 4) || !aligned_to(prev_out, 4))
    return UNIRL_E_ALIGN;
  DpmArgs A = {};
  A.v = model_output;
  A.x = sample;
  A.x0_prev = (branch == UNIRL_DPM2_SECOND) ? x0_prev : nullptr;
  A.c = *coeffs;
  A.n = n;
  A.x0_out = x0_out;
  A.prev_out = prev_out;
  hipStream_t st = (hipStream_t)stream;
  switch (dtype_v) {
    case UNIRL_F32: return launch_dpm_x<float>(A, dtype_x, branch, st);
    case UNIRL_BF16: return launch_dpm_x<bf16_t>(A, dtype_x, branch, st);
    case UNIRL_F16: return launch_dpm_x<f16_t>(A, dtype_x, branch, st);
  }
  return UNIRL_E_DTYPE;
}
