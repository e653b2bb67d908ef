// Flow-matching SDE transition + per-sample Gaussian log-prob, fused.
//
// Arithmetic follows unirl/sde/kernels.py of the reference op for op in fp32:
//   FlowSDEStrategy.step            :207-236
//   DanceSDEStrategy.step           :304-333
//   CPSSDEStrategy.step             :255-279
//   compute_log_prob                :193-205 / :247-253 / :290-302
//   SDEStrategy._finalize_logp      :154-177 (dtype round trip, mean over D)
// The scalar coefficients (one set per sample) are evaluated in the kernel with
// the same fp32 operation order torch uses on the [1,1,..] sigma tensors, so
// prev_sample and prev_sample_mean come out bit-identical to eager torch on the
// CPU.  The log-prob accumulates sum((prev-mean)^2) per lane in fp32 over a few
// elements, then in fp64 across lanes / wavefronts / workgroups in a fixed
// order.
//
// HBM traffic per element (fp32, sampling): read v, x, noise; write prev, mean
// = 20 bytes; replay with the mean kept: read v, x, prev; write mean = 16.

#include "common_hip.h"
#include "dppo_body.h"
#include "unirl_internal.h"

namespace unirl {

constexpr int kSdeThreads = 256;
constexpr float kHalfLog2Pi = 0.9189385332046727f;  // 0.5*log(2*pi) as torch casts it to f32

struct SdeCoef {
  // flow / dance: mean = x*a + (v*b)*dt ; prev = mean + s_noise*n
  // cps         : mean = (x - sigma*v)*om_sn + (x + v*om_s)*c2 ; prev = mean + s_noise*n
  float a, b, dt, s_noise;
  float sigma, om_s, om_sn, c2;
  float den;   // 2*std_var^2   (flow / dance log-prob denominator)
  float logs;  // log(std_var)
};

struct SdeScalars {
  float eta;      // (float)eta
  float eta2;     // (float)(eta*eta)            -- dance: python computes eta**2 in double
  float sin_eta;  // (float)sin(eta*pi/2)        -- cps
};

// Correctly rounded f32 divide / sqrt through f64 (53 >= 2*24+2 bits, so the
// double rounding is innocuous); independent of how the compiler lowers the
// f32 forms.
__device__ __forceinline__ float div_rn(float a, float b) { return (float)((double)a / (double)b); }
__device__ __forceinline__ float sqrt_rn(float a) { return (float)sqrt((double)a); }

__device__ __forceinline__ SdeCoef sde_coef(int kind, float s, float sn, float smax, SdeScalars sc) {
  SdeCoef c;
  c.sigma = s;
  c.om_s = 1.0f - s;
  c.om_sn = 1.0f - sn;
  c.dt = sn - s;
  c.a = 1.0f;
  c.b = 1.0f;
  c.c2 = 0.0f;
  if (kind == UNIRL_SDE_FLOW) {
    const float den0 = 1.0f - ((s == 1.0f) ? smax : s);
    const float std_dev = sqrt_rn(div_rn(s, den0)) * sc.eta;
    const float std2 = std_dev * std_dev;
    c.a = 1.0f + div_rn(std2, 2.0f * s) * c.dt;
    c.b = 1.0f + div_rn(std2 * (1.0f - s), 2.0f * s);
    c.s_noise = std_dev * sqrt_rn(-c.dt);
  } else if (kind == UNIRL_SDE_DANCE) {
    // eta**2 / (2*sigma) is float.__truediv__(tensor) = tensor.reciprocal() * scalar
    c.a = 1.0f + (div_rn(1.0f, 2.0f * s) * sc.eta2) * c.dt;
    c.b = 1.0f + div_rn((1.0f - s) * sc.eta2, 2.0f * s);
    c.s_noise = sqrt_rn(-c.dt) * sc.eta;
  } else {  // CPS
    const float std_dev = sn * sc.sin_eta;
    c.c2 = sqrt_rn(sn * sn - std_dev * std_dev);
    c.s_noise = std_dev;
  }
  const float sv = c.s_noise;
  c.den = 2.0f * (sv * sv);
  c.logs = (float)log((double)sv);  // correctly rounded f32 log
  return c;
}

// One element of the transition.  Returns prev - mean (the log-prob residual).
template <typename TX, bool SAMPLING>
__device__ __forceinline__ float sde_elem(int kind, const SdeCoef& c, float v, float x, float third,
                                          float& mean, float& prev) {
  if (kind == UNIRL_SDE_CPS) {
    const float po = x - c.sigma * v;
    const float ne = x + v * c.om_s;
    mean = po * c.om_sn + ne * c.c2;
  } else {
    mean = x * c.a + (v * c.b) * c.dt;
  }
  if (SAMPLING) {
    prev = mean + c.s_noise * third;
  } else {
    prev = third;
  }
  prev = Elem<TX>::round_trip(prev);
  return prev - mean;
}

// Final per-sample log-prob from sum((prev-mean)^2) over D elements.
__device__ __forceinline__ float sde_finish_logp(int kind, const SdeCoef& c, double q, double D, int logp_sum) {
  double lp;
  if (kind == UNIRL_SDE_CPS) {
    lp = -(q / D);
  } else {
    lp = -(q / D) / (double)c.den - (double)c.logs - (double)kHalfLog2Pi;
  }
  if (logp_sum) lp *= D;
  return (float)lp;
}

struct SdeStepArgs {
  const void* v;
  const void* x;
  const void* third;  // noise (f32) when sampling, prev_sample (TX) when replaying; may be null when sampling
  const float* sigma;
  const float* sigma_next;
  const float* sigma_max_ptr;
  float sigma_max_val;
  int sigma_stride;
  SdeScalars sc;
  int kind;
  int want_logp;
  int logp_sum;
  int64_t D;
  int64_t stride_v, stride_x, stride_third;  // elements between consecutive samples
  void* prev_out;
  void* mean_out;
  int prev_dtype, mean_dtype;                // unirl_dtype of the two outputs
  int64_t stride_prev, stride_mean;
  float* logp_out;
  int64_t stride_logp;
  double* partials;        // [rows][gridDim.x]
  float* coef_out;         // [rows][2]: the row's log-prob denominator and log(std), left for the finalize / finish kernel
  // sampling only: noise drawn in the kernel (third == nullptr), optionally stored
  int rng;
  RngKey rng_key;
  int64_t rng_row0;        // index of the launch's first sample within the call
  float* noise_out;
  int64_t stride_noise_out;
  // fused Flow-DPPO replay only: the old policy's means [rows, D] (dense, the latents' dtype), whose
  // Gaussian-KL numerator against this pass's means is summed beside the log-prob residual
  const void* kl_old;
  double* partials_kl;     // [rows][gridDim.x]
  unsigned int nblk;       // host only: grid.x
  int items;               // host only: vectors in flight per lane
  UNIRL_TRACE_FIELD
};

// Rows of a batched replay.  A launch of the step kernels covers `rows` independent transitions
// (grid.y); in the plain step a row is a sample.  In a replay of S recorded steps per sample, row
// = b * S + j is step j of sample b: the velocity sits at v + b*stride_v + j*v_step, the latent
// the step starts from and the stored next latent at their slots of the sample's trajectory
// stack (element offsets off_x[j], off_t[j] from the sample's base), sigma at index j, and the
// outputs are dense in the row index.
struct SdeRowMap {
  int S;
  int64_t v_step;
  int64_t off_x[UNIRL_MAX_ROLLOUT_STEPS];
  int64_t off_t[UNIRL_MAX_ROLLOUT_STEPS];
};

// Store VEC floats as `dtype` (wave-uniform switch) at element index `idx` of `base`.
template <int VEC>
__device__ __forceinline__ void sde_store_as(void* base, int dtype, int64_t idx, const float (&o)[VEC]) {
  if (dtype == UNIRL_F32)
    Vec<float, VEC>::store(reinterpret_cast<float*>(base) + idx, o);
  else if (dtype == UNIRL_BF16)
    Vec<bf16_t, VEC>::store(reinterpret_cast<bf16_t*>(base) + idx, o);
  else
    Vec<f16_t, VEC>::store(reinterpret_cast<f16_t*>(base) + idx, o);
}

// KL (replay rows only): also read the old policy's mean of every element and accumulate
// (round(mean) - old)^2 in the means' dtype beside the log-prob residual -- the numerator of
// _gaussian_kl_div (unirl/algorithms/flowdppo.py:51) on the means the reference would have stored
// (`.to(trajectory_dtype)`, unirl/models/sd3/diffusion.py:496) -- so that the Flow-DPPO loss needs
// no second pass over the means.  Both partials go to the workspace whatever the grid.
// RNG (sampling only): the noise is drawn in the kernel (A.rng_key) instead of read through `third`.
template <typename TV, typename TX, int VEC, int ITEMS, bool SAMPLING, bool ROWS, bool KL = false, bool RNG = false>
__device__ __forceinline__ void sde_step_body(const SdeStepArgs& A, const SdeRowMap* M) {
  static_assert(!RNG || (SAMPLING && !ROWS && !KL), "noise is drawn for the plain sampling step only");
  __shared__ double lds[(KL ? 2 : 1) * (kSdeThreads / kWave)];
  using T3 = typename std::conditional<SAMPLING, float, TX>::type;
  UNIRL_TRACE_T0();

  const int64_t row = blockIdx.y;
  const int64_t D = A.D;
  const int kind = A.kind;

  // plain step: the row is the sample; replay rows: (sample, step)
  int64_t b = row, off_v = 0, off_x = 0, off_t = 0, sig_idx = row * A.sigma_stride;
  if (ROWS) {
    b = row / M->S;
    const int j = (int)(row - b * M->S);
    off_v = j * M->v_step;
    off_x = M->off_x[j];
    off_t = M->off_t[j];
    sig_idx = j;
  }
  const TV* __restrict__ vp = reinterpret_cast<const TV*>(A.v) + b * A.stride_v + off_v;
  const TX* __restrict__ xp = reinterpret_cast<const TX*>(A.x) + b * A.stride_x + off_x;
  const T3* __restrict__ tp = A.third ? reinterpret_cast<const T3*>(A.third) + b * A.stride_third + off_t : nullptr;
  const TX* __restrict__ qp = KL ? reinterpret_cast<const TX*>(A.kl_old) + row * A.D : nullptr;
  void* const po = A.prev_out;
  void* const mo = A.mean_out;
  const int64_t po0 = row * A.stride_prev, mo0 = row * A.stride_mean;
  const int pdt = A.prev_dtype, mdt = A.mean_dtype;

  const int64_t nvec = D / VEC;  // VEC == 1 or D % VEC == 0 (checked on the host)
  const int64_t stride = (int64_t)gridDim.x * kSdeThreads;
  float acc = 0.0f, acc_kl = 0.0f;

  float v[ITEMS][VEC], x[ITEMS][VEC], t[ITEMS][VEC], q[KL ? ITEMS : 1][VEC];
  auto load_pass = [&](int64_t i0) {
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      const int64_t i = i0 + it * stride;
      if (i < nvec) {
        Vec<TV, VEC>::load(vp + i * VEC, v[it]);
        Vec<TX, VEC>::load(xp + i * VEC, x[it]);
        if (KL) Vec<TX, VEC>::load(qp + i * VEC, q[KL ? it : 0]);
        if (tp) {
          Vec<T3, VEC>::load(tp + i * VEC, t[it]);
        } else if (!RNG) {
#pragma unroll
          for (int k = 0; k < VEC; ++k) t[it][k] = 0.0f;
        }
      }
    }
    if (RNG) {
      // the noise of the pass is worked out while its loads are in flight
#pragma unroll
      for (int it = 0; it < ITEMS; ++it) {
        const int64_t i = i0 + it * stride;
        if (i < nvec) {
          rng_normals<VEC>(A.rng_key, (uint64_t)((A.rng_row0 + row) * D + i * VEC), 0u, t[it]);
          if (A.noise_out) Vec<float, VEC>::store(A.noise_out + row * A.stride_noise_out + i * VEC, t[it]);
        }
      }
    }
  };

  // The first pass of loads goes out before the coefficients are worked out: the sigma loads and
  // the fp64 divide / sqrt / log behind the coefficients take about as long as a trip to memory,
  // and at small sizes (one pass per lane) the two would otherwise run back to back.
  int64_t i0 = (int64_t)blockIdx.x * kSdeThreads + threadIdx.x;
  load_pass(i0);
  const float s = A.sigma[sig_idx];
  const float sn = A.sigma_next[sig_idx];
  const float smax = A.sigma_max_ptr ? *A.sigma_max_ptr : A.sigma_max_val;
  const SdeCoef c = sde_coef(kind, s, sn, smax, A.sc);

  while (i0 < nvec) {
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      const int64_t i = i0 + it * stride;
      if (i < nvec) {
        float mean[VEC], prev[VEC];
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
          const float d = sde_elem<TX, SAMPLING>(kind, c, v[it][k], x[it][k], t[it][k], mean[k], prev[k]);
          acc = fmaf(d, d, acc);
          if (KL) acc_kl += kl_sq<TX>(Elem<TX>::round_trip(mean[k]), q[KL ? it : 0][k]);
        }
        if (po) sde_store_as<VEC>(po, pdt, po0 + i * VEC, prev);
        if (mo) sde_store_as<VEC>(mo, mdt, mo0 + i * VEC, mean);
      }
    }
    i0 += stride * ITEMS;
    if (i0 < nvec) load_pass(i0);
  }

  UNIRL_TRACE_MARK1();
  if (!A.want_logp) {  // uniform across the grid
    UNIRL_TRACE_END(A.trace);
    return;
  }

  if (KL) {
    // both sums through one barrier: wavefront totals side by side, added in wavefront order
    const double w_lp = wave_sum((double)acc), w_kl = wave_sum((double)acc_kl);
    constexpr int kWaves = kSdeThreads / kWave;
    const int wid = threadIdx.x / kWave;
    if ((threadIdx.x & (kWave - 1)) == 0) {
      lds[wid] = w_lp;
      lds[kWaves + wid] = w_kl;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      double p_lp = lds[0], p_kl = lds[kWaves];
#pragma unroll
      for (int w = 1; w < kWaves; ++w) {
        p_lp += lds[w];
        p_kl += lds[kWaves + w];
      }
      A.partials[row * gridDim.x + blockIdx.x] = p_lp;     // both summed by flowdppo_replay_finish_kernel
      A.partials_kl[row * gridDim.x + blockIdx.x] = p_kl;
      if (blockIdx.x == 0) {  // the coefficients are worked out here anyway: the finish kernel only reads them
        A.coef_out[2 * row] = c.den;
        A.coef_out[2 * row + 1] = c.logs;
      }
    }
    UNIRL_TRACE_END(A.trace);
    return;
  }
  const double part = block_sum<double>((double)acc, lds);
  if (threadIdx.x != 0) return;
  if (gridDim.x == 1) {
    A.logp_out[row * A.stride_logp] = sde_finish_logp(kind, c, part, (double)D, A.logp_sum);
  } else {
    A.partials[row * gridDim.x + blockIdx.x] = part;  // summed by sde_step_finalize_kernel
    if (blockIdx.x == 0) {  // worked out here anyway, behind the first pass of loads: the finalize only reads them
      A.coef_out[2 * row] = c.den;
      A.coef_out[2 * row + 1] = c.logs;
    }
  }
  UNIRL_TRACE_END(A.trace);
}

template <typename TV, typename TX, int VEC, int ITEMS, bool SAMPLING, bool RNG = false>
__global__ __launch_bounds__(kSdeThreads) void sde_step_kernel(SdeStepArgs A) {
  sde_step_body<TV, TX, VEC, ITEMS, SAMPLING, false, false, RNG>(A, nullptr);
}

// The replay of S recorded steps per sample as one launch over the (sample, step) rows.
template <typename TV, typename TX, int VEC, int ITEMS>
__global__ __launch_bounds__(kSdeThreads) void sde_replay_kernel(SdeStepArgs A, SdeRowMap M) {
  sde_step_body<TV, TX, VEC, ITEMS, false, true>(A, &M);
}

// The same replay with the Flow-DPPO KL numerator against the old means accumulated in the pass.
template <typename TV, typename TX, int VEC, int ITEMS>
__global__ __launch_bounds__(kSdeThreads) void sde_replay_kl_kernel(SdeStepArgs A, SdeRowMap M) {
  sde_step_body<TV, TX, VEC, ITEMS, false, true, true>(A, &M);
}

// Finish of the fused Flow-DPPO replay step: one workgroup, arranged so that nothing is evaluated
// twice -- on a single compute unit the fp64 divide / sqrt / log behind the coefficients and the
// per-row divisions are what a replicated finish would spend its time on:
//   1. every wavefront takes rows in turn and adds the row's log-prob and KL partials (fixed order;
//      with one partial per lane the loads of four rows are in flight at once), leaving the two
//      sums in LDS;
//   2. the rows' coefficients (log-prob denominator, log std) are not worked out again: the streaming
//      kernel, which needs them anyway, has left them in the workspace;
//   3. after one barrier the first wavefront finishes the rows, lane = row (log-prob as
//      sde_step_finalize_kernel, KL as gaussian_kl_finalize_kernel), and runs the [B,S'] KL-ADV
//      problem on them (unirl/algorithms/flowdppo.py:86-137): masks, loss, the twelve metrics, the
//      gradient with respect to the new log-probs.
// R <= kReplayKlMaxRows.
struct ReplayKlFinish {
  const float* sigma_t;  // the KL's noise scale: row r uses sigma_t[r % n_sigma_t]
  int64_t n_sigma_t;
  float threshold;
  float* kl_out;
  uint8_t* mask_out;
};
constexpr int kReplayFinishThreads = 1024;
constexpr int64_t kReplayKlMaxRows = 2048;

__global__ __launch_bounds__(kReplayFinishThreads) void flowdppo_replay_finish_kernel(SdeStepArgs A, DppoArgs P,
                                                                                     ReplayKlFinish F, unsigned int nblk) {
  __shared__ double lds_q[2][kReplayKlMaxRows];  // per row: the two sums of partials
  __shared__ float lds_lp[kReplayKlMaxRows];
  __shared__ float lds_kl[kReplayKlMaxRows];
  UNIRL_TRACE_T0();
  const int wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  const int64_t R = P.n;
  constexpr int kWaves = kReplayFinishThreads / kWave;
  // the first wavefront's share of the [B,S'] problem and of the KL scales is loaded now, with the partials
  float first_od = 0.0f, first_adv = 0.0f, first_st = 1.0f, first_den = 1.0f, first_logs = 0.0f;
  if (wave == 0 && lane < R) {
    first_od = P.od[lane];
    first_adv = P.adv[lane];
    first_st = F.sigma_t[lane % F.n_sigma_t];
    first_den = A.coef_out[2 * lane];
    first_logs = A.coef_out[2 * lane + 1];
  }

  auto store_row = [&](int64_t row, double q_lp, double q_kl) {
    q_lp = wave_sum(q_lp);
    q_kl = wave_sum(q_kl);
    if (lane == 0) {
      lds_q[0][row] = q_lp;
      lds_q[1][row] = q_kl;
    }
  };
  if (nblk <= kWave) {
    // One partial per lane and row: a wavefront keeps the loads of four of its rows in flight at once
    // (every trip to memory that waits for the one before costs about a microsecond here).  A row
    // past the end repeats the last row's loads and is dropped.
    constexpr int kRows = 4;
    const unsigned int jl = (unsigned int)lane < nblk ? lane : nblk - 1;
    for (int64_t base = wave; base < R; base += kWaves * kRows) {
      double y_lp[kRows], y_kl[kRows];
#pragma unroll
      for (int r = 0; r < kRows; ++r) {
        const int64_t row = base + r * kWaves;
        const int64_t rc = row < R ? row : R - 1;
        y_lp[r] = A.partials[rc * nblk + jl];
        y_kl[r] = A.partials_kl[rc * nblk + jl];
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int r = 0; r < kRows; ++r) {
        const int64_t row = base + r * kWaves;
        if (row < R) {  // wave-uniform
          const bool ok = (unsigned int)lane < nblk;
          store_row(row, ok ? y_lp[r] : 0.0, ok ? y_kl[r] : 0.0);
        }
      }
    }
  } else {
    // many partials per row means few rows (rows * nblk is capped by the launch): one row at a time
    for (int64_t row = wave; row < R; row += kWaves) {
      double q_lp, q_kl;
      lane_ordered_sum2(A.partials + row * nblk, A.partials_kl + row * nblk, nblk, q_lp, q_kl);
      store_row(row, q_lp, q_kl);
    }
  }
  UNIRL_TRACE_MARK1();
  __syncthreads();
  if (wave != 0) return;
  // lane = row: the log-prob and the KL of 64 rows per pass, then the loss on them
  for (int64_t row = lane; row < R; row += kWave) {
    const bool head = (row == lane);  // the lane's first row: its operands were loaded at kernel entry
    SdeCoef c;
    c.den = head ? first_den : A.coef_out[2 * row];
    c.logs = head ? first_logs : A.coef_out[2 * row + 1];
    const float lp = sde_finish_logp(A.kind, c, lds_q[0][row], (double)A.D, A.logp_sum);
    const float st = head ? first_st : F.sigma_t[row % F.n_sigma_t];
    const float den = 2.0f * (st * st);
    const float kl = (float)((lds_q[1][row] / (double)den) / (double)A.D);
    A.logp_out[row * A.stride_logp] = lp;
    F.kl_out[row] = kl;
    if (F.mask_out) F.mask_out[row] = (kl < F.threshold) ? 1 : 0;
    lds_lp[row] = lp;
    lds_kl[row] = kl;
  }
  UNIRL_TRACE_MARK2();
  DppoArgs Q = P;
  Q.nw = lds_lp;  // the new log-probs never leave the workgroup before the loss has used them
  float first[3] = {0.0f, first_od, first_adv};
  if (lane < R) first[0] = lds_lp[lane];
  dppo_on_one_wave(Q, lds_kl, first);
  UNIRL_TRACE_END(A.trace);
}

// One wavefront per row: adds the workgroup partials in index order and finishes the log-prob.
// The row's coefficients (log-prob denominator, log std) come from the workspace, where the
// streaming kernel has left them: worked out here they would follow the sigma loads -- a trip to
// memory, then an fp64 divide, square root and logarithm with nothing to overlap them.
// kBatch: partial loads a lane has in flight, chosen by the host from nblk (1, 2, 4 or 8 cover 64,
// 128, 256 and more partials per row: surplus loads of a short row cost more than they hide).
template <int kBatch>
__global__ __launch_bounds__(kSdeThreads) void sde_step_finalize_kernel(SdeStepArgs A, int64_t B, unsigned int nblk) {
  UNIRL_TRACE_T0();
  const int64_t b = (int64_t)blockIdx.x * (kSdeThreads / kWave) + threadIdx.x / kWave;
  if (b >= B) return;
  const int lane = threadIdx.x & (kWave - 1);
  const double* __restrict__ pp = A.partials + b * nblk;
  double y[kBatch];  // lane l adds partials l, l + 64, ... in that order
#pragma unroll
  for (int k = 0; k < kBatch; ++k) {
    const unsigned int j = lane + k * kWave;
    y[k] = pp[j < nblk ? j : nblk - 1];  // past the end: a harmless repeat, discarded below
  }
  SdeCoef c;
  c.den = A.coef_out[2 * b];
  c.logs = A.coef_out[2 * b + 1];
  __builtin_amdgcn_sched_barrier(0);  // all of the above in flight before the first value is used
  double q = 0.0;
#pragma unroll
  for (int k = 0; k < kBatch; ++k) q += (lane + k * kWave < (int)nblk) ? y[k] : 0.0;
  if (nblk > kBatch * kWave) q += lane_ordered_sum(pp, nblk, kBatch * kWave);
  q = wave_sum(q);
  UNIRL_TRACE_MARK1();
  if (lane != 0) return;
  A.logp_out[b * A.stride_logp] = sde_finish_logp(A.kind, c, q, (double)A.D, A.logp_sum);
  UNIRL_TRACE_END(A.trace);
}

// ---------------------------------------------------------------------------
// Backward.  With r = prev - mean (prev detached) and, for flow / dance,
//   logp_b = mean_D( -r^2/den ) + const      => dlogp/dmean = 2 r / (den * D)
//   mean   = x*a + v*(b*dt)                  => dmean/dv = b*dt, dmean/dx = a
// cps: dlogp/dmean = 2 r / D ; dmean/dv = -sigma*om_sn + om_s*c2 ; dmean/dx = om_sn + c2.
// In sampling mode prev = mean + s*n also carries g_prev, and prev is detached
// inside the log-prob, so r contributes no second path.
// ---------------------------------------------------------------------------
struct SdeBwdArgs {
  const void* v;
  const void* x;
  const void* third;
  const float* sigma;
  const float* sigma_next;
  const float* sigma_max_ptr;
  float sigma_max_val;
  int sigma_stride;
  SdeScalars sc;
  int kind;
  int logp_sum;
  int64_t D;
  const float* g_logp;
  const float* g_mean;
  const float* g_prev;
  void* grad_v;
  void* grad_x;
  int dtype_gv, dtype_gx;  // unirl_dtype of the two outputs
  int64_t stride_v, stride_x;  // replay rows only: elements between consecutive samples
};

template <typename TV, typename TX, int VEC, bool SAMPLING, bool ROWS>
__device__ __forceinline__ void sde_step_bwd_body(const SdeBwdArgs& A, const SdeRowMap* M) {
  using T3 = typename std::conditional<SAMPLING, float, TX>::type;
  const int64_t b = blockIdx.y;  // the row: a sample, or (sample, step) of a batched replay
  const int64_t D = A.D;
  // plain: dense [B, D] operands; replay rows: velocity / latents addressed through the row map
  // (the velocity's gradient takes the velocity's layout), the incoming mean gradient dense in
  // the row index
  int64_t base_v = b * D, base_x = b * D, base_t = b * D, sig_idx = b * A.sigma_stride;
  if (ROWS) {
    const int64_t smp = b / M->S;
    const int j = (int)(b - smp * M->S);
    base_v = smp * A.stride_v + j * M->v_step;
    base_x = smp * A.stride_x + M->off_x[j];
    base_t = smp * A.stride_x + M->off_t[j];
    sig_idx = j;
  }
  const float s = A.sigma[sig_idx];
  const float sn = A.sigma_next[sig_idx];
  const float smax = A.sigma_max_ptr ? *A.sigma_max_ptr : A.sigma_max_val;
  const int kind = A.kind;
  const SdeCoef c = sde_coef(kind, s, sn, smax, A.sc);

  const TV* __restrict__ vp = reinterpret_cast<const TV*>(A.v) + base_v;
  const TX* __restrict__ xp = reinterpret_cast<const TX*>(A.x) + base_x;
  const T3* __restrict__ tp = A.third ? reinterpret_cast<const T3*>(A.third) + base_t : nullptr;
  const float* __restrict__ gm = A.g_mean ? A.g_mean + b * D : nullptr;
  const float* __restrict__ gp = A.g_prev ? A.g_prev + b * D : nullptr;
  void* const gv = A.grad_v;
  void* const gx = A.grad_x;
  const int dgv = A.dtype_gv, dgx = A.dtype_gx;

  float dmean_dv, dmean_dx, k_lp;
  const float glp = A.g_logp ? A.g_logp[b] : 0.0f;
  const float scale = A.logp_sum ? 1.0f : 1.0f / (float)D;
  if (kind == UNIRL_SDE_CPS) {
    dmean_dv = c.om_s * c.c2 - c.sigma * c.om_sn;
    dmean_dx = c.om_sn + c.c2;
    k_lp = 2.0f * glp * scale;
  } else {
    dmean_dv = c.b * c.dt;
    dmean_dx = c.a;
    k_lp = 2.0f * glp * scale / c.den;
  }

  const int64_t nvec = D / VEC;
  const int64_t stride = (int64_t)gridDim.x * kSdeThreads;
  for (int64_t i = (int64_t)blockIdx.x * kSdeThreads + threadIdx.x; i < nvec; i += stride) {
    float v[VEC], x[VEC], t[VEC], g1[VEC], g2[VEC], ov[VEC], ox[VEC];
    Vec<TV, VEC>::load(vp + i * VEC, v);
    Vec<TX, VEC>::load(xp + i * VEC, x);
    if (tp) {
      Vec<T3, VEC>::load(tp + i * VEC, t);
    } else {
#pragma unroll
      for (int k = 0; k < VEC; ++k) t[k] = 0.0f;
    }
#pragma unroll
    for (int k = 0; k < VEC; ++k) g1[k] = g2[k] = 0.0f;
    if (gm) Vec<float, VEC>::load(gm + i * VEC, g1);
    if (gp) Vec<float, VEC>::load(gp + i * VEC, g2);
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
      float mean, prev;
      const float r = sde_elem<TX, SAMPLING>(kind, c, v[k], x[k], t[k], mean, prev);
      float g = k_lp * r + g1[k];
      if (SAMPLING) g += g2[k];
      ov[k] = g * dmean_dv;
      ox[k] = g * dmean_dx;
    }
    if (gv) sde_store_as<VEC>(gv, dgv, (ROWS ? base_v : b * D) + i * VEC, ov);
    if (gx) sde_store_as<VEC>(gx, dgx, b * D + i * VEC, ox);
  }
}

template <typename TV, typename TX, int VEC, bool SAMPLING>
__global__ __launch_bounds__(kSdeThreads) void sde_step_bwd_kernel(SdeBwdArgs A) {
  sde_step_bwd_body<TV, TX, VEC, SAMPLING, false>(A, nullptr);
}

// Backward of the batched replay with respect to the velocities (the latents are stored data).
template <typename TV, typename TX, int VEC>
__global__ __launch_bounds__(kSdeThreads) void sde_replay_bwd_kernel(SdeBwdArgs A, SdeRowMap M) {
  sde_step_bwd_body<TV, TX, VEC, false, true>(A, &M);
}

// ---------------------------------------------------------------------------
// S chained transitions, latent in registers.
// ---------------------------------------------------------------------------
struct SdeRolloutArgs {
  const void* x0;
  const void* v[UNIRL_MAX_ROLLOUT_STEPS];
  const float* n[UNIRL_MAX_ROLLOUT_STEPS];
  SdeScalars sc[UNIRL_MAX_ROLLOUT_STEPS];
  unsigned char want_logp[UNIRL_MAX_ROLLOUT_STEPS];
  const float* sigmas;
  const float* sigma_max_ptr;
  float sigma_max_val;
  int S;
  int kind;
  int logp_sum;
  int64_t D;
  int64_t BD;
  float* x_out;
  float* traj_out;
  float* logp_out;         // [B][S]
  double* partials;        // [B][S][gridDim.x]
  unsigned int nblk;       // host only: grid.x
  int items;               // host only: vectors per lane (one pass covers a sample)
};

// What the drawing variant of the rollout kernel needs beside SdeRolloutArgs.
struct SdeRolloutRng {
  RngKey key;
  int64_t row0;                                  // index of the launch's first sample within the call
  unsigned char draw[UNIRL_MAX_ROLLOUT_STEPS];   // the step's noise is drawn in the kernel
  float* n_out[UNIRL_MAX_ROLLOUT_STEPS];         // where a step's drawn noise is stored, or null
};

template <typename TV, typename TX, int VEC, int ITEMS, bool RNG>
__device__ __forceinline__ void sde_rollout_body(const SdeRolloutArgs& A, const SdeRolloutRng* G) {
  constexpr int NW = kSdeThreads / kWave;
  __shared__ double lds_q[UNIRL_MAX_ROLLOUT_STEPS][NW];
  __shared__ SdeCoef lds_c[UNIRL_MAX_ROLLOUT_STEPS];

  const int64_t b = blockIdx.y;
  const int64_t D = A.D;
  const int S = A.S;
  const int kind = A.kind;
  const float smax = A.sigma_max_ptr ? *A.sigma_max_ptr : A.sigma_max_val;
  const int lane = threadIdx.x & (kWave - 1);
  const int wid = threadIdx.x / kWave;

  const int64_t nvec = D / VEC;
  const int64_t stride = (int64_t)gridDim.x * kSdeThreads;
  const int64_t i_first = (int64_t)blockIdx.x * kSdeThreads + threadIdx.x;
  // host guarantees gridDim.x * kSdeThreads * ITEMS >= nvec: one pass covers the sample.

  float x[ITEMS][VEC];
  const TX* __restrict__ xp = reinterpret_cast<const TX*>(A.x0) + b * D;
#pragma unroll
  for (int it = 0; it < ITEMS; ++it) {
    const int64_t i = i_first + it * stride;
    if (i < nvec) Vec<TX, VEC>::load(xp + i * VEC, x[it]);
  }

  // Each step's coefficients cost an fp64 divide / sqrt / log chain (about a microsecond of one
  // wavefront).  Lane k of the first wavefront works out step k once, while the x0 loads are in
  // flight, and every wavefront reads them from LDS afterwards.
  if ((int)threadIdx.x < S)
    lds_c[threadIdx.x] = sde_coef(kind, A.sigmas[threadIdx.x], A.sigmas[threadIdx.x + 1], smax, A.sc[threadIdx.x]);
  __syncthreads();

  for (int k = 0; k < S; ++k) {
    const SdeCoef c = lds_c[k];
    const TV* __restrict__ vp = reinterpret_cast<const TV*>(A.v[k]) + b * D;
    const float* __restrict__ np = A.n[k] ? A.n[k] + b * D : nullptr;
    float* __restrict__ tj = A.traj_out ? A.traj_out + (int64_t)k * A.BD + b * D : nullptr;
    float v[ITEMS][VEC], n[ITEMS][VEC];
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      const int64_t i = i_first + it * stride;
      if (i < nvec) {
        Vec<TV, VEC>::load(vp + i * VEC, v[it]);
        if (np) {
          Vec<float, VEC>::load(np + i * VEC, n[it]);
        } else if (!RNG || !G->draw[k]) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) n[it][e] = 0.0f;
        }
      }
    }
    if (RNG && G->draw[k]) {  // wave-uniform: the step's noise, worked out while its velocity loads are in flight
      float* __restrict__ no = G->n_out[k] ? G->n_out[k] + b * D : nullptr;
#pragma unroll
      for (int it = 0; it < ITEMS; ++it) {
        const int64_t i = i_first + it * stride;
        if (i < nvec) {
          rng_normals<VEC>(G->key, (uint64_t)((G->row0 + b) * D + i * VEC), (uint32_t)k, n[it]);
          if (no) Vec<float, VEC>::store(no + i * VEC, n[it]);
        }
      }
    }
    float acc = 0.0f;
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      const int64_t i = i_first + it * stride;
      if (i < nvec) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          float mean, prev;
          const float d = sde_elem<TX, true>(kind, c, v[it][e], x[it][e], n[it][e], mean, prev);
          acc = fmaf(d, d, acc);
          x[it][e] = prev;
        }
        if (tj) Vec<float, VEC>::store(tj + i * VEC, x[it]);
      }
    }
    const double w = wave_sum((double)acc);
    if (lane == 0) lds_q[k][wid] = w;
  }

  float* __restrict__ xo = A.x_out + b * D;
#pragma unroll
  for (int it = 0; it < ITEMS; ++it) {
    const int64_t i = i_first + it * stride;
    if (i < nvec) Vec<float, VEC>::store(xo + i * VEC, x[it]);
  }

  __syncthreads();
  const unsigned int nblk = gridDim.x;
  // workgroup totals per step, summed in wave order
  if ((int)threadIdx.x < S) {
    double q = 0.0;
#pragma unroll
    for (int w = 0; w < NW; ++w) q += lds_q[threadIdx.x][w];
    if (nblk == 1) {
      if (A.want_logp[threadIdx.x]) {
        const SdeCoef c = lds_c[threadIdx.x];
        A.logp_out[b * S + threadIdx.x] = sde_finish_logp(kind, c, q, (double)D, A.logp_sum);
      } else {
        A.logp_out[b * S + threadIdx.x] = __uint_as_float(0x7fc00000u);
      }
    } else {
      A.partials[((int64_t)b * S + threadIdx.x) * nblk + blockIdx.x] = q;  // summed by sde_rollout_finalize_kernel
    }
  }
}

template <typename TV, typename TX, int VEC, int ITEMS>
__global__ __launch_bounds__(kSdeThreads) void sde_rollout_kernel(SdeRolloutArgs A) {
  sde_rollout_body<TV, TX, VEC, ITEMS, false>(A, nullptr);
}
// The same with the noise of some (or all) steps drawn in the kernel.
template <typename TV, typename TX, int VEC, int ITEMS>
__global__ __launch_bounds__(kSdeThreads) void sde_rollout_rng_kernel(SdeRolloutArgs A, SdeRolloutRng G) {
  sde_rollout_body<TV, TX, VEC, ITEMS, true>(A, &G);
}

// One wavefront per (sample, step).  The step's sigma pair is requested first and the partials right
// behind it, so that the coefficients (an fp64 divide, square root and logarithm) are worked out
// while the partials are still on their way, instead of a second trip to memory after the sum.
__global__ __launch_bounds__(kSdeThreads) void sde_rollout_finalize_kernel(SdeRolloutArgs A, int64_t B,
                                                                           unsigned int nblk) {
  const int64_t row = (int64_t)blockIdx.x * (kSdeThreads / kWave) + threadIdx.x / kWave;  // b * S + k
  if (row >= B * A.S) return;
  const int lane = threadIdx.x & (kWave - 1);
  const int k = (int)(row % A.S);
  const bool want = A.want_logp[k] != 0;  // wave-uniform
  float s = 0.5f, sn = 0.25f, smax = A.sigma_max_val;
  if (want) {
    s = A.sigmas[k];
    sn = A.sigmas[k + 1];
    if (A.sigma_max_ptr) smax = *A.sigma_max_ptr;
  }
  constexpr int kBatch = 2;
  const double* __restrict__ pp = A.partials + row * nblk;
  double y[kBatch];  // lane l adds partials l, l + 64, ... in that order
#pragma unroll
  for (int j = 0; j < kBatch; ++j) {
    const unsigned int i = lane + j * kWave;
    y[j] = pp[i < nblk ? i : nblk - 1];  // past the end: a harmless repeat, discarded below
  }
  __builtin_amdgcn_sched_barrier(0);  // everything above in flight before the first value is used
  const SdeCoef c = sde_coef(A.kind, s, sn, smax, A.sc[k]);
  double q = 0.0;
#pragma unroll
  for (int j = 0; j < kBatch; ++j) q += (lane + j * kWave < (int)nblk) ? y[j] : 0.0;
  if (nblk > kBatch * kWave) q += lane_ordered_sum(pp, nblk, kBatch * kWave);
  q = wave_sum(q);
  if (lane != 0) return;
  A.logp_out[row] = want ? sde_finish_logp(A.kind, c, q, (double)A.D, A.logp_sum) : __uint_as_float(0x7fc00000u);
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------
static SdeScalars make_scalars(double eta) {
  SdeScalars sc;
  sc.eta = (float)eta;
  sc.eta2 = (float)(eta * eta);
  sc.sin_eta = (float)sin(eta * 3.141592653589793 / 2.0);
  return sc;
}

// Workgroups per sample: enough that each lane keeps ITEMS vectors in flight
// in one pass, capped so a launch stays a few waves of workgroups over the chip.
static unsigned int sde_blocks_per_sample(int64_t nvec, int items, int64_t B, int64_t default_cap = 4096) {
  const int64_t per_pass = (int64_t)kSdeThreads * items;
  int64_t nblk = (nvec + per_pass - 1) / per_pass;
  const int64_t cap = tune_int("UNIRL_SDE_MAX_BLOCKS", default_cap);
  int64_t max_per_sample = cap / (B > 0 ? B : 1);
  if (max_per_sample < 1) max_per_sample = 1;
  if (nblk > max_per_sample) nblk = max_per_sample;
  if (nblk > kMaxPartialBlocks) nblk = kMaxPartialBlocks;
  if (nblk < 1) nblk = 1;
  return (unsigned int)nblk;
}

// Samples per launch so that the partials fit the workspace (and grid.y its limit).
static int64_t sde_samples_per_launch(int64_t B, int64_t partials_per_sample) {
  // one more slot per row: its two fp32 coefficients, stored behind the launch's partials
  int64_t nb = kPartialCapacity / ((partials_per_sample > 0 ? partials_per_sample : 1) + 1);
  if (nb > 32768) nb = 32768;
  if (nb > B) nb = B;
  return nb < 1 ? 1 : nb;
}

// Finalize launch of a step / replay call: one wavefront per row, the in-flight batch picked from nblk.
static int launch_step_finalize(const SdeStepArgs& A, int64_t rows, unsigned int nblk, hipStream_t st) {
  const int per_block = kSdeThreads / kWave;
  const dim3 grid((unsigned int)((rows + per_block - 1) / per_block)), block(kSdeThreads);
  if (nblk <= kWave)
    hipLaunchKernelGGL(sde_step_finalize_kernel<1>, grid, block, 0, st, A, rows, nblk);
  else if (nblk <= 2 * kWave)
    hipLaunchKernelGGL(sde_step_finalize_kernel<2>, grid, block, 0, st, A, rows, nblk);
  else if (nblk <= 4 * kWave)
    hipLaunchKernelGGL(sde_step_finalize_kernel<4>, grid, block, 0, st, A, rows, nblk);
  else
    hipLaunchKernelGGL(sde_step_finalize_kernel<8>, grid, block, 0, st, A, rows, nblk);
  return (int)hipGetLastError();
}

template <typename TV, typename TX, bool SAMPLING, bool RNG = false>
static int launch_step(const SdeStepArgs& A, int64_t B, int vec, hipStream_t st) {
  const int items = A.items;
  dim3 grid(A.nblk, (unsigned int)B), block(kSdeThreads);
  if (vec == 8) {
    // sixteen-byte accesses on the 16-bit operands; only built where there is one
    if constexpr (sizeof(TV) == 2 || sizeof(TX) == 2)
      hipLaunchKernelGGL((sde_step_kernel<TV, TX, 8, 2, SAMPLING, RNG>), grid, block, 0, st, A);
    else
      return UNIRL_E_DTYPE;
  } else if (vec == 4) {
    if (items >= 4 || RNG)  // the drawing variant is built for four vectors per lane only
      hipLaunchKernelGGL((sde_step_kernel<TV, TX, 4, 4, SAMPLING, RNG>), grid, block, 0, st, A);
    else if (items >= 2)
      hipLaunchKernelGGL((sde_step_kernel<TV, TX, 4, 2, SAMPLING, false>), grid, block, 0, st, A);
    else
      hipLaunchKernelGGL((sde_step_kernel<TV, TX, 4, 1, SAMPLING, false>), grid, block, 0, st, A);
  } else {
    hipLaunchKernelGGL((sde_step_kernel<TV, TX, 1, 2, SAMPLING, RNG>), grid, block, 0, st, A);
  }
  return (int)hipGetLastError();
}

template <typename TV, typename TX>
static int launch_step_mode(const SdeStepArgs& A, int64_t B, int vec, bool sampling, hipStream_t st) {
  if (sampling && A.rng) return launch_step<TV, TX, true, true>(A, B, vec, st);
  return sampling ? launch_step<TV, TX, true>(A, B, vec, st) : launch_step<TV, TX, false>(A, B, vec, st);
}

template <typename TV>
static int launch_step_x(const SdeStepArgs& A, int dtype_x, int64_t B, int vec, bool sampling, hipStream_t st) {
  switch (dtype_x) {
    case UNIRL_F32: return launch_step_mode<TV, float>(A, B, vec, sampling, st);
    case UNIRL_BF16: return launch_step_mode<TV, bf16_t>(A, B, vec, sampling, st);
    case UNIRL_F16: return launch_step_mode<TV, f16_t>(A, B, vec, sampling, st);
  }
  return UNIRL_E_DTYPE;
}

template <typename TV, typename TX, bool SAMPLING>
static int launch_bwd(const SdeBwdArgs& A, int64_t B, int vec, hipStream_t st) {
  const int64_t nvec = A.D / vec;
  const unsigned int nblk = sde_blocks_per_sample(nvec, 1, B);
  dim3 grid(nblk, (unsigned int)B), block(kSdeThreads);
  if (vec == 8) {
    if constexpr (sizeof(TV) == 2 || sizeof(TX) == 2)
      hipLaunchKernelGGL((sde_step_bwd_kernel<TV, TX, 8, SAMPLING>), grid, block, 0, st, A);
    else
      return UNIRL_E_DTYPE;
  } else if (vec == 4) {
    hipLaunchKernelGGL((sde_step_bwd_kernel<TV, TX, 4, SAMPLING>), grid, block, 0, st, A);
  } else {
    hipLaunchKernelGGL((sde_step_bwd_kernel<TV, TX, 1, SAMPLING>), grid, block, 0, st, A);
  }
  return (int)hipGetLastError();
}

template <typename TV>
static int launch_bwd_x(const SdeBwdArgs& A, int dtype_x, int64_t B, int vec, bool sampling, hipStream_t st) {
  switch (dtype_x) {
    case UNIRL_F32:
      return sampling ? launch_bwd<TV, float, true>(A, B, vec, st) : launch_bwd<TV, float, false>(A, B, vec, st);
    case UNIRL_BF16:
      return sampling ? launch_bwd<TV, bf16_t, true>(A, B, vec, st) : launch_bwd<TV, bf16_t, false>(A, B, vec, st);
    case UNIRL_F16:
      return sampling ? launch_bwd<TV, f16_t, true>(A, B, vec, st) : launch_bwd<TV, f16_t, false>(A, B, vec, st);
  }
  return UNIRL_E_DTYPE;
}

template <typename TV, typename TX>
static int launch_replay(const SdeStepArgs& A, const SdeRowMap& M, int64_t rows, int vec, hipStream_t st) {
  dim3 grid(A.nblk, (unsigned int)rows), block(kSdeThreads);
  if (vec == 8) {
    if constexpr (sizeof(TV) == 2 || sizeof(TX) == 2)
      hipLaunchKernelGGL((sde_replay_kernel<TV, TX, 8, 2>), grid, block, 0, st, A, M);
    else
      return UNIRL_E_DTYPE;
  } else if (vec == 4) {
    hipLaunchKernelGGL((sde_replay_kernel<TV, TX, 4, 4>), grid, block, 0, st, A, M);
  } else {
    hipLaunchKernelGGL((sde_replay_kernel<TV, TX, 1, 2>), grid, block, 0, st, A, M);
  }
  return (int)hipGetLastError();
}

template <typename TV>
static int launch_replay_x(const SdeStepArgs& A, const SdeRowMap& M, int dtype_x, int64_t rows, int vec, hipStream_t st) {
  switch (dtype_x) {
    case UNIRL_F32: return launch_replay<TV, float>(A, M, rows, vec, st);
    case UNIRL_BF16: return launch_replay<TV, bf16_t>(A, M, rows, vec, st);
    case UNIRL_F16: return launch_replay<TV, f16_t>(A, M, rows, vec, st);
  }
  return UNIRL_E_DTYPE;
}

template <typename TV, typename TX>
static int launch_replay_kl(const SdeStepArgs& A, const SdeRowMap& M, int64_t rows, int vec, hipStream_t st) {
  dim3 grid(A.nblk, (unsigned int)rows), block(kSdeThreads);
  if (vec == 8) {
    if constexpr (sizeof(TV) == 2 || sizeof(TX) == 2)
      hipLaunchKernelGGL((sde_replay_kl_kernel<TV, TX, 8, 2>), grid, block, 0, st, A, M);
    else
      return UNIRL_E_DTYPE;
  } else if (vec == 4) {
    hipLaunchKernelGGL((sde_replay_kl_kernel<TV, TX, 4, 4>), grid, block, 0, st, A, M);
  } else {
    hipLaunchKernelGGL((sde_replay_kl_kernel<TV, TX, 1, 2>), grid, block, 0, st, A, M);
  }
  return (int)hipGetLastError();
}

template <typename TV>
static int launch_replay_kl_x(const SdeStepArgs& A, const SdeRowMap& M, int dtype_x, int64_t rows, int vec,
                              hipStream_t st) {
  switch (dtype_x) {
    case UNIRL_F32: return launch_replay_kl<TV, float>(A, M, rows, vec, st);
    case UNIRL_BF16: return launch_replay_kl<TV, bf16_t>(A, M, rows, vec, st);
    case UNIRL_F16: return launch_replay_kl<TV, f16_t>(A, M, rows, vec, st);
  }
  return UNIRL_E_DTYPE;
}

template <typename TV, typename TX>
static int launch_replay_bwd(const SdeBwdArgs& A, const SdeRowMap& M, int64_t rows, int vec, hipStream_t st) {
  const unsigned int nblk = sde_blocks_per_sample(A.D / vec, 1, rows);
  dim3 grid(nblk, (unsigned int)rows), block(kSdeThreads);
  if (vec == 8) {
    if constexpr (sizeof(TV) == 2 || sizeof(TX) == 2)
      hipLaunchKernelGGL((sde_replay_bwd_kernel<TV, TX, 8>), grid, block, 0, st, A, M);
    else
      return UNIRL_E_DTYPE;
  } else if (vec == 4) {
    hipLaunchKernelGGL((sde_replay_bwd_kernel<TV, TX, 4>), grid, block, 0, st, A, M);
  } else {
    hipLaunchKernelGGL((sde_replay_bwd_kernel<TV, TX, 1>), grid, block, 0, st, A, M);
  }
  return (int)hipGetLastError();
}

template <typename TV>
static int launch_replay_bwd_x(const SdeBwdArgs& A, const SdeRowMap& M, int dtype_x, int64_t rows, int vec,
                               hipStream_t st) {
  switch (dtype_x) {
    case UNIRL_F32: return launch_replay_bwd<TV, float>(A, M, rows, vec, st);
    case UNIRL_BF16: return launch_replay_bwd<TV, bf16_t>(A, M, rows, vec, st);
    case UNIRL_F16: return launch_replay_bwd<TV, f16_t>(A, M, rows, vec, st);
  }
  return UNIRL_E_DTYPE;
}

// Argument checks and the row map shared by the replay's forward and backward entry points.
struct ReplayPlan {
  int64_t stride_v, v_step, stride_x, slot_stride;
  int vec;
  SdeRowMap M;
};

static int plan_replay(const unirl_sde_replay_desc* d, const void* extra_f32_a, const void* extra_b, size_t extra_b_size,
                       ReplayPlan& P) {
  if (!d) return UNIRL_E_NULL;
  const int dtype_v = d->noise_pred.dtype, dtype_x = d->latents.dtype;
  const int64_t B = d->B, S = d->S, D = d->D, K = d->K;
  if (!dtype_ok(dtype_v) || !dtype_ok(dtype_x)) return UNIRL_E_DTYPE;
  if (d->kind < UNIRL_SDE_FLOW || d->kind > UNIRL_SDE_CPS) return UNIRL_E_DTYPE;
  if (d->mean_out && !dtype_ok(d->mean_dtype)) return UNIRL_E_DTYPE;
  if (B < 0 || S < 1 || D <= 0 || K < 1) return UNIRL_E_SHAPE;
  if (S > UNIRL_MAX_ROLLOUT_STEPS) return UNIRL_E_LIMIT;
  if (B * S > 32768) return UNIRL_E_LIMIT;  // one row per grid.y index
  if (!d->slot_sample || !d->slot_prev) return UNIRL_E_NULL;
  P.v_step = d->noise_pred_step_stride ? d->noise_pred_step_stride : D;
  P.stride_v = d->noise_pred.sample_stride ? d->noise_pred.sample_stride : S * D;
  P.slot_stride = d->latents_slot_stride ? d->latents_slot_stride : D;
  P.stride_x = d->latents.sample_stride ? d->latents.sample_stride : K * P.slot_stride;
  if (P.v_step < D || P.stride_v < 0 || P.slot_stride < D || P.stride_x < 0) return UNIRL_E_SHAPE;
  const size_t sv = dtype_size(dtype_v), sx = dtype_size(dtype_x);
  const size_t smo = d->mean_out ? dtype_size(d->mean_dtype) : 4;
  if (!aligned_to(d->noise_pred.ptr, sv) || !aligned_to(d->latents.ptr, sx) || !aligned_to(d->mean_out, smo) ||
      !aligned_to(d->logp_out, 4) || !aligned_to(extra_f32_a, 4) || !aligned_to(extra_b, extra_b_size))
    return UNIRL_E_ALIGN;
  P.M.S = (int)S;
  P.M.v_step = P.v_step;
  for (int64_t j = 0; j < S; ++j) {
    const int64_t a = d->slot_sample[j], b = d->slot_prev[j];
    if (a < 0 || a >= K || b < 0 || b >= K) return UNIRL_E_SHAPE;
    P.M.off_x[j] = a * P.slot_stride;
    P.M.off_t[j] = b * P.slot_stride;
  }
  // vectors of four (or eight, when the 16-bit tensors carry at least as many bytes as the fp32
  // ones: same rule as the single step) need every row base on the vector's boundary
  int vec = 4;
  if (D % 4 != 0 || P.v_step % 4 || P.stride_v % 4 || P.slot_stride % 4 || P.stride_x % 4 ||
      !aligned_to(d->noise_pred.ptr, 4 * sv) || !aligned_to(d->latents.ptr, 4 * sx) ||
      !aligned_to(d->mean_out, 4 * smo) || !aligned_to(extra_f32_a, 16) || !aligned_to(extra_b, 4 * extra_b_size))
    vec = 1;
  if (vec == 4 && (sv == 2 || sx == 2) && D % 8 == 0) {
    size_t narrow = 0, wide = 0;
    bool ok = true;
    auto visit = [&](const void* p, size_t es, bool strides_ok) {
      if (!p) return;
      (es == 2 ? narrow : wide) += es;
      ok = ok && aligned_to(p, 16) && (es == 4 || strides_ok);
    };
    visit(d->noise_pred.ptr, sv, P.v_step % 8 == 0 && P.stride_v % 8 == 0);
    visit(d->latents.ptr, sx, P.slot_stride % 8 == 0 && P.stride_x % 8 == 0);
    visit(d->latents.ptr, sx, true);  // read twice: the step's input and the stored next latent
    visit(d->mean_out, smo, true);
    visit(extra_f32_a, 4, true);
    visit(extra_b, extra_b_size, P.v_step % 8 == 0 && P.stride_v % 8 == 0);
    if (ok && narrow >= wide) vec = 8;
  }
  P.vec = vec;
  return UNIRL_OK;
}

template <typename TV, typename TX>
static int launch_rollout(const SdeRolloutArgs& A, const SdeRolloutRng* G, int64_t B, int vec, hipStream_t st) {
  dim3 grid(A.nblk, (unsigned int)B), block(kSdeThreads);
  const int items = A.items;
#define UNIRL_LAUNCH_ROLLOUT(VEC, ITEMS)                                                                   \
  do {                                                                                                     \
    if (G) hipLaunchKernelGGL((sde_rollout_rng_kernel<TV, TX, VEC, ITEMS>), grid, block, 0, st, A, *G);    \
    else hipLaunchKernelGGL((sde_rollout_kernel<TV, TX, VEC, ITEMS>), grid, block, 0, st, A);              \
  } while (0)
  if (vec == 4) {
    if (items >= 4) UNIRL_LAUNCH_ROLLOUT(4, 4);
    else if (items == 2) UNIRL_LAUNCH_ROLLOUT(4, 2);
    else UNIRL_LAUNCH_ROLLOUT(4, 1);
  } else {
    if (items >= 4) UNIRL_LAUNCH_ROLLOUT(1, 4);
    else if (items == 2) UNIRL_LAUNCH_ROLLOUT(1, 2);
    else UNIRL_LAUNCH_ROLLOUT(1, 1);
  }
#undef UNIRL_LAUNCH_ROLLOUT
  return (int)hipGetLastError();
}

template <typename TV>
static int launch_rollout_x(const SdeRolloutArgs& A, const SdeRolloutRng* G, int dtype_x, int64_t B, int vec,
                            hipStream_t st) {
  switch (dtype_x) {
    case UNIRL_F32: return launch_rollout<TV, float>(A, G, B, vec, st);
    case UNIRL_BF16: return launch_rollout<TV, bf16_t>(A, G, B, vec, st);
    case UNIRL_F16: return launch_rollout<TV, f16_t>(A, G, B, vec, st);
  }
  return UNIRL_E_DTYPE;
}

}  // namespace unirl

using namespace unirl;

extern "C" int unirl_sde_step_logp_ex(const unirl_sde_step_desc* d, void* workspace, size_t workspace_bytes,
                                      void* stream) {
  if (!d) return UNIRL_E_NULL;
  const int dtype_v = d->noise_pred.dtype, dtype_x = d->sample.dtype;
  const int64_t B = d->B, D = d->D;
  if (!dtype_ok(dtype_v) || !dtype_ok(dtype_x)) return UNIRL_E_DTYPE;
  if (d->kind < UNIRL_SDE_FLOW || d->kind > UNIRL_SDE_CPS) return UNIRL_E_DTYPE;
  if ((d->prev_out && !dtype_ok(d->prev_dtype)) || (d->mean_out && !dtype_ok(d->mean_dtype))) return UNIRL_E_DTYPE;
  if (B < 0 || D <= 0 || (d->sigma_stride != 0 && d->sigma_stride != 1)) return UNIRL_E_SHAPE;
  // sample strides: 0 means densely packed; inputs may overlap or repeat (any stride >= 0 is
  // readable), outputs must not alias across samples
  const int64_t stride_v = d->noise_pred.sample_stride ? d->noise_pred.sample_stride : D;
  const int64_t stride_x = d->sample.sample_stride ? d->sample.sample_stride : D;
  const int64_t stride_p = d->prev_sample.sample_stride ? d->prev_sample.sample_stride : D;
  const int64_t stride_n = d->noise_stride ? d->noise_stride : D;
  const int64_t stride_po = d->prev_stride ? d->prev_stride : D;
  const int64_t stride_mo = d->mean_stride ? d->mean_stride : D;
  const int64_t stride_lp = d->logp_stride ? d->logp_stride : 1;
  if (stride_v < 0 || stride_x < 0 || stride_p < 0 || stride_n < 0 || stride_po < D || stride_mo < D || stride_lp < 1)
    return UNIRL_E_SHAPE;
  if (B == 0) return UNIRL_OK;
  const void* noise_pred = d->noise_pred.ptr;
  const void* sample = d->sample.ptr;
  const void* prev_sample = d->prev_sample.ptr;
  if (!noise_pred || !sample || !d->sigma || !d->sigma_next) return UNIRL_E_NULL;
  const bool sampling = (prev_sample == nullptr);
  if (!sampling && d->prev_sample.dtype != dtype_x) return UNIRL_E_DTYPE;
  const bool want_logp = (d->logp_out != nullptr) && !(d->eta < 1e-7);
  if (want_logp && (!workspace || workspace_bytes < kWorkspaceBytes)) return UNIRL_E_WORKSPACE;
  // noise drawn in the kernel: sampling, no noise tensor given, a stochastic step
  const bool draw = sampling && d->rng.enabled && !d->noise && !(d->eta < 1e-7);
  const int64_t stride_no = d->noise_out_stride ? d->noise_out_stride : D;
  if (draw && d->noise_out && stride_no < D) return UNIRL_E_SHAPE;
  const size_t sv = dtype_size(dtype_v), sx = dtype_size(dtype_x);
  const size_t spo = d->prev_out ? dtype_size(d->prev_dtype) : 4, smo = d->mean_out ? dtype_size(d->mean_dtype) : 4;
  if (!aligned_to(noise_pred, sv) || !aligned_to(sample, sx) || !aligned_to(prev_sample, sx) ||
      !aligned_to(d->noise, 4) || !aligned_to(d->prev_out, spo) || !aligned_to(d->mean_out, smo) ||
      !aligned_to(d->logp_out, 4) || (draw && !aligned_to(d->noise_out, 4)))
    return UNIRL_E_ALIGN;

  // 4-element vectors need every per-sample base to keep the vector alignment.
  int vec = 4;
  if (D % 4 != 0 || !aligned_to(noise_pred, 4 * sv) || !aligned_to(sample, 4 * sx) ||
      !aligned_to(prev_sample, 4 * sx) || !aligned_to(d->noise, 16) || !aligned_to(d->prev_out, 4 * spo) ||
      !aligned_to(d->mean_out, 4 * smo) || stride_v % 4 || stride_x % 4 || (!sampling && stride_p % 4) ||
      (sampling && d->noise && stride_n % 4) || (d->prev_out && stride_po % 4) || (d->mean_out && stride_mo % 4) ||
      (draw && d->noise_out && (stride_no % 4 || !aligned_to(d->noise_out, 16))))
    vec = 1;

  // 16-bit operands: eight elements per lane make their accesses sixteen bytes too, while an
  // fp32 operand then takes two accesses that each cover only half of every cache line, which
  // costs more than it gains once fp32 traffic dominates (sampling with fp32 noise and outputs:
  // 55 -> 61 us at [8, 2M]; replay of bf16 tensors: 45 -> 38 us).  So: eight when the 16-bit
  // tensors carry at least as many bytes as the fp32 ones, and every base and sample stride of a
  // 16-bit tensor sits on a 16-byte boundary.
  if (vec == 4 && (sv == 2 || sx == 2) && tune_int("UNIRL_SDE_VEC8", 1) == 1) {
    size_t narrow = 0, wide = 0;
    bool ok = (D % 8 == 0);
    auto visit = [&](const void* p, size_t es, int64_t stride) {
      if (!p) return;
      (es == 2 ? narrow : wide) += es;
      ok = ok && aligned_to(p, 16) && (es == 4 || stride % 8 == 0);
    };
    visit(noise_pred, sv, stride_v);
    visit(sample, sx, stride_x);
    if (sampling) visit(d->noise, 4, stride_n); else visit(prev_sample, sx, stride_p);
    if (draw) visit(d->noise_out, 4, stride_no);
    visit(d->prev_out, spo, stride_po);
    visit(d->mean_out, smo, stride_mo);
    if (ok && narrow >= wide) vec = 8;
  }
  const int items = (vec == 8) ? 2 : (vec == 4) ? (int)tune_int("UNIRL_SDE_ITEMS", 4) : 2;
  const unsigned int nblk = sde_blocks_per_sample(D / vec, items, B);
  const int64_t per_launch = sde_samples_per_launch(B, nblk);
  hipStream_t st = (hipStream_t)stream;

  for (int64_t b0 = 0; b0 < B; b0 += per_launch) {
    const int64_t nb = (B - b0 < per_launch) ? (B - b0) : per_launch;
    SdeStepArgs A = {};
    A.v = offset_ptr(noise_pred, b0 * stride_v, sv);
    A.x = offset_ptr(sample, b0 * stride_x, sx);
    A.third = sampling ? (const void*)offset_f32(d->noise, b0 * stride_n) : offset_ptr(prev_sample, b0 * stride_p, sx);
    A.stride_v = stride_v;
    A.stride_x = stride_x;
    A.stride_third = sampling ? stride_n : stride_p;
    A.sigma = d->sigma + b0 * d->sigma_stride;
    A.sigma_next = d->sigma_next + b0 * d->sigma_stride;
    A.sigma_max_ptr = d->sigma_max_ptr;
    A.sigma_max_val = d->sigma_max_val;
    A.sigma_stride = d->sigma_stride;
    A.sc = make_scalars(d->eta);
    A.kind = d->kind;
    A.want_logp = want_logp ? 1 : 0;
    A.logp_sum = d->logp_sum;
    A.D = D;
    A.prev_out = const_cast<void*>(offset_ptr(d->prev_out, b0 * stride_po, spo));
    A.mean_out = const_cast<void*>(offset_ptr(d->mean_out, b0 * stride_mo, smo));
    A.prev_dtype = d->prev_dtype;
    A.mean_dtype = d->mean_dtype;
    A.stride_prev = stride_po;
    A.stride_mean = stride_mo;
    A.logp_out = offset_f32(d->logp_out, b0 * stride_lp);
    A.stride_logp = stride_lp;
    A.partials = ws_partials(workspace);
    A.coef_out = reinterpret_cast<float*>(A.partials + nb * (int64_t)nblk);
    A.nblk = nblk;
    A.items = items;
    if (draw) {
      A.rng = 1;
      A.rng_key = RngKey{(uint32_t)d->rng.seed, (uint32_t)(d->rng.seed >> 32), (uint32_t)d->rng.offset,
                         (uint32_t)(d->rng.offset >> 32)};
      A.rng_row0 = b0;
      A.noise_out = offset_f32(d->noise_out, b0 * stride_no);
      A.stride_noise_out = stride_no;
    }
    UNIRL_TRACE_SET(A, "sde_step", nblk * (unsigned int)nb);
    int rc = UNIRL_E_DTYPE;
    switch (dtype_v) {
      case UNIRL_F32: rc = launch_step_x<float>(A, dtype_x, nb, vec, sampling, st); break;
      case UNIRL_BF16: rc = launch_step_x<bf16_t>(A, dtype_x, nb, vec, sampling, st); break;
      case UNIRL_F16: rc = launch_step_x<f16_t>(A, dtype_x, nb, vec, sampling, st); break;
    }
    if (rc != 0) return rc;
    if (want_logp && nblk > 1) {
      UNIRL_TRACE_SET(A, "sde_finalize", (unsigned int)((nb + kSdeThreads / kWave - 1) / (kSdeThreads / kWave)));
      rc = launch_step_finalize(A, nb, nblk, st);
      if (rc != 0) return rc;
    }
  }
  return UNIRL_OK;
}

extern "C" int unirl_sde_replay_logp(const unirl_sde_replay_desc* d, void* workspace, size_t workspace_bytes,
                                     void* stream) {
  ReplayPlan P;
  int rc = plan_replay(d, nullptr, nullptr, 4, P);
  if (rc != 0) return rc;
  const int64_t B = d->B, S = d->S, D = d->D;
  if (B == 0) return UNIRL_OK;
  if (!d->noise_pred.ptr || !d->latents.ptr || !d->sigma || !d->sigma_next) return UNIRL_E_NULL;
  const bool want_logp = (d->logp_out != nullptr) && !(d->eta < 1e-7);
  if (want_logp && (!workspace || workspace_bytes < kWorkspaceBytes)) return UNIRL_E_WORKSPACE;
  const int vec = P.vec;
  const int items = (vec == 8) ? 2 : (vec == 4) ? 4 : 2;
  const int64_t rows_all = B * S;
  // a replay is tens of rows of megabytes each: a quarter of the single step's workgroup cap
  // (measured: 16.4 -> 15.3 us at the SD3 shape, 46.7 -> 44.8 us at the WAN shape)
  const unsigned int nblk = sde_blocks_per_sample(D / vec, items, rows_all, 1024);
  // whole samples per launch, so that a launch's rows stay (sample, step) pairs
  int64_t per_launch = sde_samples_per_launch(rows_all, nblk) / S;
  if (per_launch < 1) return UNIRL_E_LIMIT;
  const size_t sv = dtype_size(d->noise_pred.dtype), sx = dtype_size(d->latents.dtype);
  const size_t smo = d->mean_out ? dtype_size(d->mean_dtype) : 4;
  hipStream_t st = (hipStream_t)stream;
  for (int64_t b0 = 0; b0 < B; b0 += per_launch) {
    const int64_t nb = (B - b0 < per_launch) ? (B - b0) : per_launch;
    SdeStepArgs A = {};
    A.v = offset_ptr(d->noise_pred.ptr, b0 * P.stride_v, sv);
    A.x = offset_ptr(d->latents.ptr, b0 * P.stride_x, sx);
    A.third = A.x;  // the stored next latent lives in the same stack
    A.stride_v = P.stride_v;
    A.stride_x = P.stride_x;
    A.stride_third = P.stride_x;
    A.sigma = d->sigma;
    A.sigma_next = d->sigma_next;
    A.sigma_max_ptr = d->sigma_max_ptr;
    A.sigma_max_val = d->sigma_max_val;
    A.sigma_stride = 0;
    A.sc = make_scalars(d->eta);
    A.kind = d->kind;
    A.want_logp = want_logp ? 1 : 0;
    A.logp_sum = d->logp_sum;
    A.D = D;
    A.prev_out = nullptr;
    A.mean_out = const_cast<void*>(offset_ptr(d->mean_out, b0 * S * D, smo));
    A.prev_dtype = UNIRL_F32;
    A.mean_dtype = d->mean_dtype;
    A.stride_prev = D;
    A.stride_mean = D;
    A.logp_out = offset_f32(d->logp_out, b0 * S);
    A.stride_logp = 1;
    A.partials = ws_partials(workspace);
    A.coef_out = reinterpret_cast<float*>(A.partials + nb * S * (int64_t)nblk);
    A.nblk = nblk;
    A.items = items;
    UNIRL_TRACE_SET(A, "sde_replay", nblk * (unsigned int)(nb * S));
    rc = UNIRL_E_DTYPE;
    switch (d->noise_pred.dtype) {
      case UNIRL_F32: rc = launch_replay_x<float>(A, P.M, d->latents.dtype, nb * S, vec, st); break;
      case UNIRL_BF16: rc = launch_replay_x<bf16_t>(A, P.M, d->latents.dtype, nb * S, vec, st); break;
      case UNIRL_F16: rc = launch_replay_x<f16_t>(A, P.M, d->latents.dtype, nb * S, vec, st); break;
    }
    if (rc != 0) return rc;
    if (want_logp && nblk > 1) {
      UNIRL_TRACE_SET(A, "sde_finalize", (unsigned int)((nb * S + kSdeThreads / kWave - 1) / (kSdeThreads / kWave)));
      rc = launch_step_finalize(A, nb * S, nblk, st);
      if (rc != 0) return rc;
    }
  }
  return UNIRL_OK;
}

extern "C" int unirl_flowdppo_replay_step(const unirl_sde_replay_desc* d, const void* old_means, const float* sigma_t,
                                          int64_t n_sigma_t, const float* old_logp, const float* advantages,
                                          float threshold, float loss_scale, float* kl_out, uint8_t* mask_out,
                                          float* loss_elem, float* grad_logp, float* metrics, void* workspace,
                                          size_t workspace_bytes, void* stream) {
  if (!d) return UNIRL_E_NULL;
  ReplayPlan P;
  const size_t sx = dtype_ok(d->latents.dtype) ? dtype_size(d->latents.dtype) : 4;
  int rc = plan_replay(d, nullptr, old_means, sx, P);
  if (rc != 0) return rc;
  const int64_t B = d->B, S = d->S, D = d->D, R = B * S;
  if (R <= 0 || n_sigma_t <= 0) return UNIRL_E_SHAPE;
  if (d->eta < 1e-7) return UNIRL_E_SHAPE;  // a deterministic step has no log-prob to build a ratio from
  if (R > kReplayKlMaxRows) return UNIRL_E_LIMIT;
  if (!d->noise_pred.ptr || !d->latents.ptr || !d->sigma || !d->sigma_next || !d->logp_out || !old_means || !sigma_t ||
      !old_logp || !advantages || !kl_out || !loss_elem || !metrics)
    return UNIRL_E_NULL;
  if (!aligned_to(sigma_t, 4) || !aligned_to(old_logp, 4) || !aligned_to(advantages, 4) || !aligned_to(kl_out, 4) ||
      !aligned_to(loss_elem, 4) || !aligned_to(grad_logp, 4) || !aligned_to(metrics, 4))
    return UNIRL_E_ALIGN;
  if (!workspace || workspace_bytes < kWorkspaceBytes) return UNIRL_E_WORKSPACE;
  const int vec = P.vec;
  const int items = (vec == 8) ? 2 : (vec == 4) ? 4 : 2;
  // Workgroups: at most 768 in all -- with its fourth operand in flight the kernel holds 136 - 157 vector
  // registers, three wavefronts per SIMD, so 3 x 256 workgroups are resident at once and a 769th would
  // wait for a whole workgroup's lifetime (896 at the WAN shape: 50 us per call, 728: 43 us) -- at most
  // 64 per row (the finish kernel then has one partial per lane and keeps several rows in flight),
  // and the fewest that keep the number of passes, so that every pass of a lane is a full one.
  unsigned int nblk = sde_blocks_per_sample(D / vec, items, R, 768);
  if (nblk > (unsigned int)kWave) nblk = kWave;
  {
    const int64_t per_lane = (int64_t)kSdeThreads * items, nvec = D / vec;
    const int64_t passes = (nvec + nblk * per_lane - 1) / (nblk * per_lane);
    const int64_t even = (nvec + passes * per_lane - 1) / (passes * per_lane);
    if (even >= 1 && even < (int64_t)nblk) nblk = (unsigned int)even;
  }
  if ((2 * (int64_t)nblk + 1) * R > kPartialCapacity) return UNIRL_E_LIMIT;
  hipStream_t st = (hipStream_t)stream;
  SdeStepArgs A = {};
  A.v = d->noise_pred.ptr;
  A.x = d->latents.ptr;
  A.third = A.x;  // the stored next latent lives in the same stack
  A.stride_v = P.stride_v;
  A.stride_x = P.stride_x;
  A.stride_third = P.stride_x;
  A.sigma = d->sigma;
  A.sigma_next = d->sigma_next;
  A.sigma_max_ptr = d->sigma_max_ptr;
  A.sigma_max_val = d->sigma_max_val;
  A.sigma_stride = 0;
  A.sc = make_scalars(d->eta);
  A.kind = d->kind;
  A.want_logp = 1;
  A.logp_sum = d->logp_sum;
  A.D = D;
  A.prev_out = nullptr;
  A.mean_out = d->mean_out;  // only on request: the loss itself never needs the means in memory
  A.prev_dtype = UNIRL_F32;
  A.mean_dtype = d->mean_dtype;
  A.stride_prev = D;
  A.stride_mean = D;
  A.logp_out = d->logp_out;
  A.stride_logp = 1;
  A.partials = ws_partials(workspace);
  A.partials_kl = ws_partials(workspace) + (int64_t)nblk * R;
  A.coef_out = reinterpret_cast<float*>(ws_partials(workspace) + 2 * (int64_t)nblk * R);
  A.kl_old = old_means;
  A.nblk = nblk;
  A.items = items;
  UNIRL_TRACE_SET(A, "sde_replay_kl", nblk * (unsigned int)R);
  rc = UNIRL_E_DTYPE;
  switch (d->noise_pred.dtype) {
    case UNIRL_F32: rc = launch_replay_kl_x<float>(A, P.M, d->latents.dtype, R, vec, st); break;
    case UNIRL_BF16: rc = launch_replay_kl_x<bf16_t>(A, P.M, d->latents.dtype, R, vec, st); break;
    case UNIRL_F16: rc = launch_replay_kl_x<f16_t>(A, P.M, d->latents.dtype, R, vec, st); break;
  }
  if (rc != 0) return rc;
  DppoArgs Q;
  Q.nw = nullptr;  // taken from the finish kernel's LDS
  Q.od = old_logp;
  Q.adv = advantages;
  Q.kl = nullptr;
  Q.n = R;
  Q.threshold = threshold;
  Q.loss_elem = loss_elem;
  Q.metrics = metrics;
  Q.grad_new = grad_logp;
  Q.grad_scale = loss_scale / (float)R;
  ReplayKlFinish F;
  F.sigma_t = sigma_t;
  F.n_sigma_t = n_sigma_t;
  F.threshold = threshold;
  F.kl_out = kl_out;
  F.mask_out = mask_out;
  UNIRL_TRACE_SET(A, "flowdppo_replay_finish", 1);
  hipLaunchKernelGGL(flowdppo_replay_finish_kernel, dim3(1), dim3(kReplayFinishThreads), 0, st, A, Q, F, nblk);
  return (int)hipGetLastError();
}

extern "C" int unirl_sde_replay_logp_bwd(const unirl_sde_replay_desc* d, const float* g_logp, const float* g_mean,
                                         void* grad_v, int dtype_gv, void* stream) {
  if (grad_v && !dtype_ok(dtype_gv)) return UNIRL_E_DTYPE;
  ReplayPlan P;
  int rc = plan_replay(d, g_mean, grad_v, grad_v ? dtype_size(dtype_gv) : 4, P);
  if (rc != 0) return rc;
  if (d->B == 0 || !grad_v) return UNIRL_OK;
  if (!d->noise_pred.ptr || !d->latents.ptr || !d->sigma || !d->sigma_next) return UNIRL_E_NULL;
  if (!aligned_to(g_logp, 4)) return UNIRL_E_ALIGN;
  SdeBwdArgs A = {};
  A.v = d->noise_pred.ptr;
  A.x = d->latents.ptr;
  A.third = d->latents.ptr;
  A.sigma = d->sigma;
  A.sigma_next = d->sigma_next;
  A.sigma_max_ptr = d->sigma_max_ptr;
  A.sigma_max_val = d->sigma_max_val;
  A.sigma_stride = 0;
  A.sc = make_scalars(d->eta);
  A.kind = d->kind;
  A.logp_sum = d->logp_sum;
  A.D = d->D;
  A.g_logp = (d->eta < 1e-7) ? nullptr : g_logp;
  A.g_mean = g_mean;
  A.g_prev = nullptr;
  A.grad_v = grad_v;
  A.grad_x = nullptr;
  A.dtype_gv = dtype_gv;
  A.dtype_gx = UNIRL_F32;
  A.stride_v = P.stride_v;
  A.stride_x = P.stride_x;
  hipStream_t st = (hipStream_t)stream;
  switch (d->noise_pred.dtype) {
    case UNIRL_F32: return launch_replay_bwd_x<float>(A, P.M, d->latents.dtype, d->B * d->S, P.vec, st);
    case UNIRL_BF16: return launch_replay_bwd_x<bf16_t>(A, P.M, d->latents.dtype, d->B * d->S, P.vec, st);
    case UNIRL_F16: return launch_replay_bwd_x<f16_t>(A, P.M, d->latents.dtype, d->B * d->S, P.vec, st);
  }
  return UNIRL_E_DTYPE;
}

extern "C" int unirl_sde_step_logp(const void* noise_pred, int dtype_v, const void* sample, int dtype_x,
                                   const void* prev_sample, const float* noise, const float* sigma,
                                   const float* sigma_next, int sigma_stride, const float* sigma_max_ptr,
                                   float sigma_max_val, double eta, int kind, int64_t B, int64_t D,
                                   float* prev_out, float* mean_out, float* logp_out, int logp_sum,
                                   void* workspace, size_t workspace_bytes, void* stream) {
  unirl_sde_step_desc d = {};
  d.noise_pred = {noise_pred, dtype_v, 0};
  d.sample = {sample, dtype_x, 0};
  d.prev_sample = {prev_sample, dtype_x, 0};
  d.noise = noise;
  d.sigma = sigma;
  d.sigma_next = sigma_next;
  d.sigma_stride = sigma_stride;
  d.sigma_max_ptr = sigma_max_ptr;
  d.sigma_max_val = sigma_max_val;
  d.eta = eta;
  d.kind = kind;
  d.B = B;
  d.D = D;
  d.prev_out = prev_out;
  d.prev_dtype = UNIRL_F32;
  d.mean_out = mean_out;
  d.mean_dtype = UNIRL_F32;
  d.logp_out = logp_out;
  d.logp_sum = logp_sum;
  return unirl_sde_step_logp_ex(&d, workspace, workspace_bytes, stream);
}

extern "C" int unirl_sde_step_logp_bwd(const void* noise_pred, int dtype_v, const void* sample, int dtype_x,
                                       const void* prev_sample, const float* noise, const float* sigma,
                                       const float* sigma_next, int sigma_stride, const float* sigma_max_ptr,
                                       float sigma_max_val, double eta, int kind, int64_t B, int64_t D,
                                       const float* g_logp, const float* g_mean, const float* g_prev,
                                       int logp_sum, void* grad_v, int dtype_gv, void* grad_x, int dtype_gx,
                                       void* stream) {
  if (!dtype_ok(dtype_v) || !dtype_ok(dtype_x)) return UNIRL_E_DTYPE;
  if ((grad_v && !dtype_ok(dtype_gv)) || (grad_x && !dtype_ok(dtype_gx))) return UNIRL_E_DTYPE;
  if (kind < UNIRL_SDE_FLOW || kind > UNIRL_SDE_CPS) return UNIRL_E_DTYPE;
  if (B < 0 || D <= 0 || (sigma_stride != 0 && sigma_stride != 1)) return UNIRL_E_SHAPE;
  if (B == 0) return UNIRL_OK;
  if (!noise_pred || !sample || !sigma || !sigma_next) return UNIRL_E_NULL;
  if (!grad_v && !grad_x) return UNIRL_OK;
  const bool sampling = (prev_sample == nullptr);
  const size_t sv = dtype_size(dtype_v), sx = dtype_size(dtype_x);
  const size_t sgv = grad_v ? dtype_size(dtype_gv) : 4, sgx = grad_x ? dtype_size(dtype_gx) : 4;
  if (!aligned_to(noise_pred, sv) || !aligned_to(sample, sx) || !aligned_to(prev_sample, sx) ||
      !aligned_to(noise, 4) || !aligned_to(g_mean, 4) || !aligned_to(g_prev, 4) || !aligned_to(grad_v, sgv) ||
      !aligned_to(grad_x, sgx))
    return UNIRL_E_ALIGN;
  int vec = 4;
  if (D % 4 != 0 || !aligned_to(noise_pred, 4 * sv) || !aligned_to(sample, 4 * sx) ||
      !aligned_to(prev_sample, 4 * sx) || !aligned_to(noise, 16) || !aligned_to(g_mean, 16) ||
      !aligned_to(g_prev, 16) || !aligned_to(grad_v, 4 * sgv) || !aligned_to(grad_x, 4 * sgx))
    vec = 1;
  // eight elements per lane when the 16-bit tensors carry at least as many bytes as the fp32
  // ones (same rule and reason as in the forward step)
  if (vec == 4 && (sv == 2 || sx == 2) && D % 8 == 0 && tune_int("UNIRL_SDE_VEC8", 1) == 1) {
    size_t narrow = 0, wide = 0;
    bool ok = true;
    auto visit = [&](const void* p, size_t es) {
      if (!p) return;
      (es == 2 ? narrow : wide) += es;
      ok = ok && aligned_to(p, 16);
    };
    visit(noise_pred, sv);
    visit(sample, sx);
    if (sampling) visit(noise, 4); else visit(prev_sample, sx);
    visit(g_mean, 4);
    if (sampling) visit(g_prev, 4);
    visit(grad_v, sgv);
    visit(grad_x, sgx);
    if (ok && narrow >= wide) vec = 8;
  }
  hipStream_t st = (hipStream_t)stream;
  const int64_t per_launch = 32768;  // grid.y limit is 65535
  for (int64_t b0 = 0; b0 < B; b0 += per_launch) {
    const int64_t nb = (B - b0 < per_launch) ? (B - b0) : per_launch;
    const int64_t off = b0 * D;
    SdeBwdArgs A;
    A.v = offset_ptr(noise_pred, off, sv);
    A.x = offset_ptr(sample, off, sx);
    A.third = sampling ? (const void*)offset_f32(noise, off) : offset_ptr(prev_sample, off, sx);
    A.sigma = sigma + b0 * sigma_stride;
    A.sigma_next = sigma_next + b0 * sigma_stride;
    A.sigma_max_ptr = sigma_max_ptr;
    A.sigma_max_val = sigma_max_val;
    A.sigma_stride = sigma_stride;
    A.sc = make_scalars(eta);
    A.kind = kind;
    A.logp_sum = logp_sum;
    A.D = D;
    A.g_logp = (eta < 1e-7) ? nullptr : offset_f32(g_logp, b0);
    A.g_mean = offset_f32(g_mean, off);
    A.g_prev = offset_f32(g_prev, off);
    A.grad_v = const_cast<void*>(offset_ptr(grad_v, off, sgv));
    A.grad_x = const_cast<void*>(offset_ptr(grad_x, off, sgx));
    A.dtype_gv = dtype_gv;
    A.dtype_gx = dtype_gx;
    int rc = UNIRL_E_DTYPE;
    switch (dtype_v) {
      case UNIRL_F32: rc = launch_bwd_x<float>(A, dtype_x, nb, vec, sampling, st); break;
      case UNIRL_BF16: rc = launch_bwd_x<bf16_t>(A, dtype_x, nb, vec, sampling, st); break;
      case UNIRL_F16: rc = launch_bwd_x<f16_t>(A, dtype_x, nb, vec, sampling, st); break;
    }
    if (rc != 0) return rc;
  }
  return UNIRL_OK;
}

extern "C" int unirl_sde_rollout_logp(const void* x0, int dtype_x, const void* const* v_steps, int dtype_v,
                                      const float* const* noise_steps, const unirl_rng* rng,
                                      float* const* noise_out_steps, const float* sigmas, const double* etas,
                                      int S, const float* sigma_max_ptr, float sigma_max_val, int kind, int64_t B,
                                      int64_t D, float* x_out, float* traj_out, float* logp_out, int logp_sum,
                                      void* workspace, size_t workspace_bytes, void* stream) {
  if (!dtype_ok(dtype_v) || !dtype_ok(dtype_x)) return UNIRL_E_DTYPE;
  if (kind < UNIRL_SDE_FLOW || kind > UNIRL_SDE_CPS) return UNIRL_E_DTYPE;
  if (B < 0 || D <= 0 || S < 1) return UNIRL_E_SHAPE;
  if (S > UNIRL_MAX_ROLLOUT_STEPS) return UNIRL_E_LIMIT;
  if (B == 0) return UNIRL_OK;
  const bool has_rng = rng && rng->enabled;
  if (!x0 || !x_out || !logp_out || !v_steps || (!noise_steps && !has_rng) || !sigmas || !etas) return UNIRL_E_NULL;
  if (!workspace || workspace_bytes < kWorkspaceBytes) return UNIRL_E_WORKSPACE;
  const size_t sv = dtype_size(dtype_v), sx = dtype_size(dtype_x);
  if (!aligned_to(x0, sx) || !aligned_to(x_out, 4) || !aligned_to(traj_out, 4)) return UNIRL_E_ALIGN;

  int vec = 4;
  if (D % 4 != 0 || !aligned_to(x0, 4 * sx) || !aligned_to(x_out, 16) || !aligned_to(traj_out, 16)) vec = 1;
  for (int k = 0; k < S; ++k) {
    if (!v_steps[k]) return UNIRL_E_NULL;
    const float* nz = noise_steps ? noise_steps[k] : nullptr;
    const float* no = (has_rng && noise_out_steps) ? noise_out_steps[k] : nullptr;
    if (!aligned_to(v_steps[k], sv) || !aligned_to(nz, 4) || !aligned_to(no, 4)) return UNIRL_E_ALIGN;
    if (!aligned_to(v_steps[k], 4 * sv) || !aligned_to(nz, 16) || !aligned_to(no, 16)) vec = 1;
  }

  // One pass must cover a sample (the latent lives in registers): pick the
  // vectors per lane, the workgroup count follows.
  const int64_t nvec = D / vec;
  int items = (int)tune_int("UNIRL_ROLLOUT_ITEMS", 4);
  if (items != 1 && items != 2 && items != 4) items = 1;
  int64_t nblk = (nvec + (int64_t)kSdeThreads * items - 1) / ((int64_t)kSdeThreads * items);
  while (nblk * S > kPartialCapacity && items < 4) {
    items *= 2;
    nblk = (nvec + (int64_t)kSdeThreads * items - 1) / ((int64_t)kSdeThreads * items);
  }
  if (nblk * S > kPartialCapacity) return UNIRL_E_LIMIT;
  const int64_t per_launch = sde_samples_per_launch(B, nblk * S);
  hipStream_t st = (hipStream_t)stream;

  for (int64_t b0 = 0; b0 < B; b0 += per_launch) {
    const int64_t nb = (B - b0 < per_launch) ? (B - b0) : per_launch;
    const int64_t off = b0 * D;
    SdeRolloutArgs A = {};
    SdeRolloutRng G = {};
    bool any_draw = false;
    for (int k = 0; k < S; ++k) {
      A.v[k] = offset_ptr(v_steps[k], off, sv);
      A.n[k] = offset_f32(noise_steps ? noise_steps[k] : nullptr, off);
      A.sc[k] = make_scalars(etas[k]);
      A.want_logp[k] = !(etas[k] < 1e-7);
      // a stochastic step without a noise tensor draws its noise when a generator is given
      G.draw[k] = (has_rng && !A.n[k] && A.want_logp[k]) ? 1 : 0;
      G.n_out[k] = (G.draw[k] && noise_out_steps) ? offset_f32(noise_out_steps[k], off) : nullptr;
      any_draw = any_draw || G.draw[k];
    }
    if (has_rng) {
      G.key = RngKey{(uint32_t)rng->seed, (uint32_t)(rng->seed >> 32), (uint32_t)rng->offset,
                     (uint32_t)(rng->offset >> 32)};
      G.row0 = b0;
    }
    A.x0 = offset_ptr(x0, off, sx);
    A.sigmas = sigmas;
    A.sigma_max_ptr = sigma_max_ptr;
    A.sigma_max_val = sigma_max_val;
    A.S = S;
    A.kind = kind;
    A.logp_sum = logp_sum;
    A.D = D;
    A.BD = B * D;
    A.x_out = offset_f32(x_out, off);
    A.traj_out = offset_f32(traj_out, off);
    A.logp_out = offset_f32(logp_out, b0 * S);
    A.partials = ws_partials(workspace);
    A.nblk = (unsigned int)nblk;
    A.items = items;
    int rc = UNIRL_E_DTYPE;
    switch (dtype_v) {
      case UNIRL_F32: rc = launch_rollout_x<float>(A, any_draw ? &G : nullptr, dtype_x, nb, vec, st); break;
      case UNIRL_BF16: rc = launch_rollout_x<bf16_t>(A, any_draw ? &G : nullptr, dtype_x, nb, vec, st); break;
      case UNIRL_F16: rc = launch_rollout_x<f16_t>(A, any_draw ? &G : nullptr, dtype_x, nb, vec, st); break;
    }
    if (rc != 0) return rc;
    if (nblk > 1) {
      const int per_block = kSdeThreads / kWave;
      hipLaunchKernelGGL(sde_rollout_finalize_kernel, dim3((unsigned int)((nb * S + per_block - 1) / per_block)),
                         dim3(kSdeThreads), 0, st, A, nb, (unsigned int)nblk);
      rc = (int)hipGetLastError();
      if (rc != 0) return rc;
    }
  }
  return UNIRL_OK;
}
