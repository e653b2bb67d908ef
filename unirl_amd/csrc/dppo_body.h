// Device code shared by the Flow-DPPO kernels of kl.hip and sde.hip: the Gaussian KL's element
// arithmetic and the KL-ADV masked loss over the [B,S'] log-probs.
#pragma once

#include "common_hip.h"

namespace unirl {

// (p - q)^2 with torch's type promotion for means of dtype T: the subtraction and the square are
// rounded to T (unirl/algorithms/flowdppo.py:51 on 16-bit means; the divide by 2 sigma^2 is fp32).
template <typename T>
__device__ __forceinline__ float kl_sq(float p, float q) {
  const float d = Elem<T>::round_trip(p - q);
  return Elem<T>::round_trip(d * d);
}

constexpr int64_t kDppoWaveMax = 4096;

// ---------------------------------------------------------------------------
// KL-ADV masked loss over the [B,S'] log-probs (unirl/algorithms/flowdppo.py:86-137):
// ratio, masks, where(keep, -A*r, 0) and the twelve logged metrics, one workgroup.
// ---------------------------------------------------------------------------
struct DppoArgs {
  const float* nw;
  const float* od;
  const float* adv;
  const float* kl;
  int64_t n;
  float threshold;
  float* loss_elem;
  float* metrics;
  float* grad_new;  // NULL, or receives grad_scale * loss_elem (the gradient of grad_scale * n * mean)
  float grad_scale;
};

// Five fp64 sums per lane; the four counters are wave-wide from the start (a comparison is a lane
// mask and counting it is one scalar instruction, where a sum over lanes is six shifts and adds).
enum { D_SR = 0, D_SR2, D_LD2, D_KL, D_LOSS, D_SUMS };
enum { C_NKL = 0, C_POS, C_NEG, C_RM, C_VALS };

struct DppoAcc {
  double acc[D_SUMS];
  unsigned long long cnt[C_VALS] = {0ull, 0ull, 0ull, 0ull};  // wave-uniform
  float rmin = INFINITY, rmax = -INFINITY, klmax = -INFINITY;
  __device__ __forceinline__ DppoAcc() {
#pragma unroll
    for (int v = 0; v < D_SUMS; ++v) acc[v] = 0.0;
  }
};

// Element i of the [B,S'] problem: ratio, the two removal masks, the kept loss (and its gradient).
// The whole wavefront calls together; `valid` is false for a lane past the end.
__device__ __forceinline__ void dppo_elem_of(const DppoArgs& A, int64_t i, bool valid, float nw, float od, float a,
                                             float kl, DppoAcc& s) {
  const float ld = nw - od;
  const float r = expf(ld);
  const bool low_kl = kl < A.threshold;
  const bool pos = !low_kl && (r > 1.0f) && (a > 0.0f);
  const bool neg = !low_kl && (r < 1.0f) && (a < 0.0f);
  const bool rm = pos || neg;
  const float loss = rm ? 0.0f : (-a) * r;
  s.cnt[C_NKL] += (unsigned long long)__builtin_popcountll(__builtin_amdgcn_ballot_w64(valid && !low_kl));
  s.cnt[C_POS] += (unsigned long long)__builtin_popcountll(__builtin_amdgcn_ballot_w64(valid && pos));
  s.cnt[C_NEG] += (unsigned long long)__builtin_popcountll(__builtin_amdgcn_ballot_w64(valid && neg));
  s.cnt[C_RM] += (unsigned long long)__builtin_popcountll(__builtin_amdgcn_ballot_w64(valid && rm));
  if (!valid) return;
  A.loss_elem[i] = loss;
  if (A.grad_new) A.grad_new[i] = A.grad_scale * loss;  // d(-a*exp(new-old))/dnew = the loss itself
  s.acc[D_SR] += (double)r;
  s.acc[D_SR2] += (double)r * (double)r;
  s.acc[D_LD2] += (double)(0.5f * (ld * ld));
  s.acc[D_KL] += (double)kl;
  s.acc[D_LOSS] += (double)loss;
  s.rmin = fminf(s.rmin, r);
  s.rmax = fmaxf(s.rmax, r);
  s.klmax = fmaxf(s.klmax, kl);
}

// The twelve metrics from the totals; one thread.
__device__ __forceinline__ void dppo_metrics(const DppoArgs& A, const double (&tot)[D_SUMS],
                                             const unsigned long long (&cnt)[C_VALS], float rmin, float rmax,
                                             float klmax) {
  const double N = (double)A.n;
  // One reciprocal for every mean (x * (1/N) and x / N agree to an ulp of fp64, far below fp32): the
  // hardware's fp32 estimate and two Newton steps in fp64 (the error squares twice from 2^-23).
  const double r0 = (double)__builtin_amdgcn_rcpf((float)N);
  const double r1 = fma(fma(-N, r0, 1.0), r0, r0);
  const double inv_n = fma(fma(-N, r1, 1.0), r1, r1);
  // the variance's numerator cancels and is formed in fp64; quotient and root are fp32 operations
  float sd = 0.0f;
  if (A.n > 1) {
    const double num = tot[D_SR2] - tot[D_SR] * tot[D_SR] * inv_n;
    sd = sqrtf(fmaxf((float)num, 0.0f) / (float)(N - 1.0));
    if (num != num) sd = quiet_nan();  // fmaxf would drop it
  }
  float* M = A.metrics;
  M[0] = (float)(tot[D_SR] * inv_n);
  M[1] = sd;
  // min()/max() of the reference return NaN when any element is NaN; ratios and KL values are
  // >= 0, so their sums are NaN exactly then
  const bool r_nan = tot[D_SR] != tot[D_SR], kl_nan = tot[D_KL] != tot[D_KL];
  M[2] = r_nan ? quiet_nan() : rmin;
  M[3] = r_nan ? quiet_nan() : rmax;
  M[4] = (float)(tot[D_LD2] * inv_n);
  M[5] = (float)(tot[D_KL] * inv_n);
  M[6] = kl_nan ? quiet_nan() : klmax;
  M[7] = (float)((double)cnt[C_NKL] * inv_n);
  M[8] = (float)((double)cnt[C_POS] * inv_n);
  M[9] = (float)((double)cnt[C_NEG] * inv_n);
  M[10] = (float)((double)cnt[C_RM] * inv_n);
  M[11] = (float)((N - (double)cnt[C_RM]) * inv_n);
  M[12] = (float)(tot[D_LOSS] * inv_n);
  M[13] = M[14] = M[15] = 0.0f;
}

// The whole [B,S'] problem on one wavefront (it is a few dozen elements): no barriers, the
// reductions are DPP only.  `kl` points at global or LDS memory.  Every lane must call.
// `first`: the lane's first element (new, old, advantage), already loaded by the caller, or null.
__device__ __forceinline__ void dppo_on_one_wave(const DppoArgs& A, const float* kl, const float* first = nullptr) {
  const int lane = threadIdx.x & (kWave - 1);
  DppoAcc s;
  // wave-uniform trip count: every lane runs every pass (the counters are taken across the wavefront)
  for (int64_t base = 0; base < A.n; base += kWave) {
    const int64_t i = base + lane;
    const bool valid = i < A.n;
    float nw = 0.0f, od = 0.0f, a = 0.0f, k = 0.0f;
    if (valid) {
      k = kl[i];
      if (first && base == 0) {
        nw = first[0];
        od = first[1];
        a = first[2];
      } else {
        nw = A.nw[i];
        od = A.od[i];
        a = A.adv[i];
      }
    }
    dppo_elem_of(A, i, valid, nw, od, a, k, s);
  }
  double tot[D_SUMS];
#pragma unroll
  for (int v = 0; v < D_SUMS; ++v) tot[v] = wave_sum(s.acc[v]);
  const float rmin = wave_min(s.rmin), rmax = wave_max(s.rmax), klmax = wave_max(s.klmax);
  if (lane == 0) dppo_metrics(A, tot, s.cnt, rmin, rmax, klmax);
}

}  // namespace unirl
