// Token-level ratio losses (GRPO clipped ratio, DRPO quadratic regulariser)
// with the aggregation and every logged metric reduced in the same pass.
//
// Per-token arithmetic follows the reference in fp32, op for op:
//   _grpo_clip_loss               unirl/algorithms/base.py:133-156
//   _drpo_loss                    unirl/algorithms/drpo.py:131-158
//   rollout_replay_logp_absdiff   unirl/algorithms/base.py:98-103
// Advantage expansion (grpo.py:187-198) is a lookup of the token's sequence;
// the three aggregation modes (grpo.py:148-155, drpo.py:323-330) are weighted
// global sums:  token-mean = sum/N,  seq-mean-token-sum-norm = sum/(n_seq*h),
// seq-mean-token-mean = sum_tok(loss/len_seq)/n_seq.
// The ratio's mean and unbiased std come from the shifted moments sum(r-1) and
// sum((r-1)^2): r-1 is exact in fp32 for r in [0.5, 2], so the variance of ~1e6
// ratios near 1 keeps full accuracy.  Sums run fp32 per lane over at most a few
// dozen tokens and fp64 from there up, in a fixed order.
//
// HBM traffic: 8 bytes read per valid token (+4 with a mask, +4 with per-token
// advantages), +4 written when loss_per_elem is requested.

#include "common.cuh"
#include "unirl_internal.h"

namespace unirl {

constexpr int kRlThreads = 256;
constexpr int kRlVals = 16;  // partial values per workgroup

enum { LAYOUT_FLAT = 0, LAYOUT_PADDED = 1, LAYOUT_PACKED = 2 };

// slots of the per-workgroup partial vector
enum {
  P_SR = 0, P_SR2, P_LOSS, P_KL, P_PEN, P_ABS, P_CNT, P_CHI, P_CLO, P_CANY, P_RMIN, P_RMAX, P_AMAX
};

struct RatioConsts {
  int kind;
  int agg_mode;
  int mu_weighted;
  int adv_per_token;
  float clamp_lo, clamp_hi;  // (float)(1 - clip_low), (float)(1 + clip_high)
  float eps_lo, eps_hi;      // (float)clip_low, (float)clip_high
  float drpo_eps;            // (float)epsilon
  float drpo_two_eps;        // (float)(2.0 * epsilon)
  float inv_two_eps;         // 1 / drpo_two_eps, correctly rounded
  float horizon;
};

struct RatioArgs {
  const float* nw;
  const float* od;
  const float* adv;
  const int64_t* seq;  // padded: lengths[n_seq]; packed: cu_seqlens[n_seq+1]; flat: null
  const float* mask;
  int64_t n_seq, seq_stride, n_tok;
  int layout;
  RatioConsts C;
  float* loss_elem;
  float* metrics;
  double* partials;
  // backward only
  const float* g_scale;
  const float* g_elem;
  const float* n_valid;  // device scalar: valid-token count from the forward
  int aggregate;
  float* grad_new;
};

// exp(x) for fp32 within ~1.5 ulp in eight instructions: 2^(x*log2(e)) on the hardware exp2,
// with the rounding error of the product (carried in a second float) applied as a first-order
// correction.  +inf above ln(FLT_MAX), 0 below the denormal range, NaN for NaN.
__device__ __forceinline__ float exp_f32(float x) {
  constexpr float kL2eHi = 1.44269502162933349609375f;  // log2(e) rounded to fp32
  constexpr float kL2eLo = 1.925963033500011e-8f;       // log2(e) - kL2eHi
  const float t = x * kL2eHi;
  float lo = fmaf(x, kL2eHi, -t);
  lo = fmaf(x, kL2eLo, lo);
  const float e = __builtin_amdgcn_exp2f(t);
  float r = fmaf(e, lo * 0.693147182f, e);
  r = (x > 88.72283172607422f) ? INFINITY : r;  // e is +inf from here on and inf*lo + inf could be NaN
  r = (x < -104.0f) ? 0.0f : r;                 // t and lo overflow for x = -inf
  return r;
}

// x / c for a loop-invariant c with inv_c = 1/c: quotient estimate, exact remainder, one
// correction -- the core of the IEEE division sequence without its range scaling (c is a
// user constant of ordinary magnitude).  Correctly rounded away from overflow and underflow.
__device__ __forceinline__ float div_by_const(float x, float c, float inv_c) {
  const float q = x * inv_c;
  const float rem = fmaf(-q, c, x);
  const float q1 = fmaf(rem, inv_c, q);
  return (q1 == q1) ? q1 : q;  // inf/NaN operands: keep the plain product's result
}

// 1 / x for x > 0 from the hardware reciprocal and one Newton step (within 1 ulp).
__device__ __forceinline__ float recip_pos(float x) {
  const float r0 = __builtin_amdgcn_rcpf(x);
  const float e = fmaf(-x, r0, 1.0f);
  const float r1 = fmaf(e, r0, r0);
  return (r1 == r1) ? r1 : r0;  // x = inf or denormal: the step yields NaN, the estimate is exact enough
}

struct TokVals {
  float r, d0, ld, loss, pen, kterm, dloss;
  bool hi, lo;
};

// Everything about one token, backward factor included (the forward kernels use the leaner
// accumulate_token below, which repeats the same arithmetic).
template <int KIND>
__device__ __forceinline__ TokVals ratio_token(float nw, float od, float A, const RatioConsts& C) {
  TokVals o;
  o.d0 = nw - od;
  if (KIND == UNIRL_LOSS_GRPO) {
    o.ld = o.d0;
    o.r = exp_f32(o.ld);
    const float nA = -A;
    const float u = nA * o.r;
    const float rc = nan_clamp(o.r, C.clamp_lo, C.clamp_hi);
    const float c = nA * rc;
    o.loss = nan_max(u, c);
    o.hi = (o.r - 1.0f) > C.eps_hi;
    o.lo = (1.0f - o.r) > C.eps_lo;
    o.kterm = 0.5f * (o.ld * o.ld);
    o.pen = 0.0f;
    const bool inside = (o.r >= C.clamp_lo) && (o.r <= C.clamp_hi);
    const float dc = inside ? c : 0.0f;
    o.dloss = (u > c) ? u : ((u < c) ? dc : 0.5f * (u + dc));
  } else {
    o.ld = nan_clamp(o.d0, -20.0f, 20.0f);
    o.r = exp_f32(o.ld);
    const float mu = exp_f32(od);
    const float rd = o.r - 1.0f;
    const float w = C.mu_weighted ? mu : 1.0f;
    o.pen = ((fabsf(A) * w) * (rd * rd)) / C.drpo_two_eps;
    o.loss = (-A) * o.r + o.pen;
    float aeps = C.drpo_eps;
    if (C.mu_weighted) aeps = (mu > 0.0f) ? (1.0f / mu) * C.drpo_eps : INFINITY;
    o.hi = o.r > (1.0f + aeps);
    o.lo = o.r < (1.0f - aeps);
    o.kterm = rd - o.ld;
    const bool clamped = (o.d0 < -20.0f) || (o.d0 > 20.0f);
    o.dloss = clamped ? 0.0f : ((-A) + (fabsf(A) * w) * rd / C.drpo_eps) * o.r;
  }
  return o;
}

// min for the ratio minimum, max for the two maxima, sum for everything else
__device__ __forceinline__ double combine(int v, double x, double y) {
  return (v == P_RMIN) ? fmin(x, y) : ((v == P_RMAX || v == P_AMAX) ? fmax(x, y) : x + y);
}

// Per-lane accumulators.  The six sums are fp32 and are flushed into fp64 totals after every
// pass (at most ITEMS*VEC tokens), so their rounding does not grow with the input.  The extrema
// are kept as bit patterns: ratios and |new-old| are >= 0 (or NaN), where unsigned integer order
// is float order, so each update is one integer min / max.
struct Acc {
  float s1 = 0.0f, s2 = 0.0f;  // sums of (r-1) and (r-1)^2
  float loss = 0.0f;
  float kl = 0.0f;             // GRPO: sum of ld^2 (halved at the end); DRPO: sum of (r-1) - ld
  float pen = 0.0f, ab = 0.0f;
  double t_s1 = 0.0, t_s2 = 0.0, t_loss = 0.0, t_kl = 0.0, t_pen = 0.0, t_ab = 0.0;
  unsigned int rmin = 0x7f800000u, rmax = 0u, amax = 0u;
  unsigned int cnt = 0, chi = 0, clo = 0, cany = 0;

  __device__ __forceinline__ void flush() {
    t_s1 += (double)s1;
    t_s2 += (double)s2;
    t_loss += (double)loss;
    t_kl += (double)kl;
    t_pen += (double)pen;
    t_ab += (double)ab;
    s1 = s2 = loss = kl = pen = ab = 0.0f;
  }
};

// One token into the accumulators; returns its loss.  `lw` = loss_mask * aggregation weight.
// The arithmetic is the reference's, op for op; two rewrites are exact:
//   maximum(u, c) = (c > u) ? c : u   -- u is NaN whenever c is (c = -A*clamp(r), u = -A*r), so
//                                        NaN reaches the result as in torch.maximum;
//   1 - r = -(r - 1)                  -- rounding is symmetric, so the lower clip test reuses r-1.
template <int KIND>
__device__ __forceinline__ float accumulate_token(float nw, float od, float A, float lw, const RatioConsts& C,
                                                  Acc& acc) {
  const float d0 = nw - od;
  float r, loss;
  bool hi, lo;
  if (KIND == UNIRL_LOSS_GRPO) {
    r = exp_f32(d0);
    const float nA = -A;
    const float u = nA * r;
    const float c = nA * fminf(fmaxf(r, C.clamp_lo), C.clamp_hi);
    loss = (c > u) ? c : u;
    const float d = r - 1.0f;
    hi = d > C.eps_hi;
    lo = -d > C.eps_lo;
    acc.s1 += d;
    acc.s2 = fmaf(d, d, acc.s2);
    acc.kl = fmaf(d0, d0, acc.kl);
  } else {
    const float ld = (d0 != d0) ? d0 : fminf(fmaxf(d0, -20.0f), 20.0f);  // torch.clamp keeps NaN
    r = exp_f32(ld);
    const float mu = exp_f32(od);
    const float d = r - 1.0f;
    const float w = C.mu_weighted ? mu : 1.0f;
    const float pen = div_by_const((fabsf(A) * w) * (d * d), C.drpo_two_eps, C.inv_two_eps);
    loss = (-A) * r + pen;
    float aeps = C.drpo_eps;
    if (C.mu_weighted) aeps = (mu > 0.0f) ? recip_pos(mu) * C.drpo_eps : INFINITY;
    hi = r > (1.0f + aeps);
    lo = r < (1.0f - aeps);
    acc.s1 += d;
    acc.s2 = fmaf(d, d, acc.s2);
    acc.kl += d - ld;
    acc.pen += pen;
  }
  acc.loss += loss * lw;
  const float a0 = fabsf(d0);
  acc.ab += a0;
  const unsigned int rb = __float_as_uint(r), ab = __float_as_uint(a0);
  acc.rmin = rb < acc.rmin ? rb : acc.rmin;
  acc.rmax = rb > acc.rmax ? rb : acc.rmax;
  acc.amax = ab > acc.amax ? ab : acc.amax;
  acc.chi += hi ? 1u : 0u;
  acc.clo += lo ? 1u : 0u;
  acc.cany += (hi || lo) ? 1u : 0u;
  return loss;
}

// sequence lookup for the packed layout: largest s with cu[s] <= tok
__device__ __forceinline__ int64_t find_seq(const int64_t* cu, int64_t n_seq, int64_t tok) {
  int64_t lo = 0, hi = n_seq;  // invariant: cu[lo] <= tok < cu[hi]
  while (hi - lo > 1) {
    const int64_t mid = (lo + hi) >> 1;
    if (cu[mid] <= tok) lo = mid; else hi = mid;
  }
  return lo;
}

// Weight of a token of a sequence of `len` tokens inside the aggregated loss,
// up to the global factor applied at the end.
__device__ __forceinline__ float seq_weight(const RatioConsts& C, int64_t len) {
  return (C.agg_mode == UNIRL_AGG_SEQ_MEAN_TOKEN_MEAN) ? 1.0f / (float)len : 1.0f;
}

// Per-lane context of the sequence a token belongs to.
struct SeqCtx {
  float adv = 0.0f;      // advantage of the current sequence (per-sequence advantages)
  float w = 1.0f;        // aggregation weight of its tokens
  int64_t cur_end = -1;  // packed layout: first token index past the current sequence
};

// One loaded vector of VEC tokens starting at row-relative index t0; tokens at or past `count`
// are padding.  mk[] holds 1 when there is no loss mask.  Accumulates into acc and leaves the
// per-token loss in out[].  Whole vectors outside the packed layout take a path without
// per-token bounds or sequence checks.
template <int KIND, int VEC, bool PACKED>
__device__ __forceinline__ void ratio_vec_fwd(const RatioArgs& A, const RatioConsts& C, int64_t t0, int64_t count,
                                              const float (&nw)[VEC], const float (&od)[VEC],
                                              const float (&ad)[VEC], const float (&mk)[VEC], SeqCtx& sq,
                                              Acc& acc, float (&out)[VEC]) {
  if (!PACKED && t0 + VEC <= count) {
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
      const float a = C.adv_per_token ? ad[k] : sq.adv;
      out[k] = accumulate_token<KIND>(nw[k], od[k], a, mk[k] * sq.w, C, acc);
    }
    acc.cnt += VEC;
    return;
  }
#pragma unroll
  for (int k = 0; k < VEC; ++k) {
    const int64_t t = t0 + k;
    out[k] = 0.0f;
    if (t < count) {
      if (PACKED && t >= sq.cur_end) {
        const int64_t s = find_seq(A.seq, A.n_seq, t);
        sq.cur_end = A.seq[s + 1];
        sq.w = seq_weight(C, sq.cur_end - A.seq[s]);
        if (!C.adv_per_token) sq.adv = A.adv[s];
      }
      const float a = C.adv_per_token ? ad[k] : sq.adv;
      out[k] = accumulate_token<KIND>(nw[k], od[k], a, mk[k] * sq.w, C, acc);
      acc.cnt += 1u;
    }
  }
}

// Workgroup partial vector -> A.partials[workgroup].  Every thread must call.
__device__ __forceinline__ void store_block_partials(const RatioArgs& A, Acc& acc, double (*lds_v)[kRlVals]) {
  constexpr int NW = kRlThreads / kWave;
  acc.flush();
  double vals[kRlVals];
  vals[P_SR] = wave_sum(acc.t_s1);
  vals[P_SR2] = wave_sum(acc.t_s2);
  // a lane's total of these four is a handful of fp32 terms: rounding it to fp32 loses nothing the
  // 1e-5 budget can see, and an fp32 DPP tree costs half the moves of an fp64 one
  vals[P_LOSS] = (double)wave_sum((float)acc.t_loss);
  vals[P_KL] = (double)wave_sum((float)acc.t_kl);
  vals[P_PEN] = (double)wave_sum((float)acc.t_pen);
  vals[P_ABS] = (double)wave_sum((float)acc.t_ab);
  vals[P_CNT] = (double)wave_sum(acc.cnt);
  vals[P_CHI] = (double)wave_sum(acc.chi);
  vals[P_CLO] = (double)wave_sum(acc.clo);
  vals[P_CANY] = (double)wave_sum(acc.cany);
  // NaN patterns drop out of the float min / max here; the finalize kernel restores NaN from the sums
  vals[P_RMIN] = (double)wave_min(__uint_as_float(acc.rmin));
  vals[P_RMAX] = (double)wave_max(acc.cnt ? __uint_as_float(acc.rmax) : -INFINITY);
  vals[P_AMAX] = (double)wave_max(acc.cnt ? __uint_as_float(acc.amax) : -INFINITY);
  vals[13] = vals[14] = vals[15] = 0.0;
  const int lane = threadIdx.x & (kWave - 1);
  const int wid = threadIdx.x / kWave;
  if (lane == 0) {
#pragma unroll
    for (int v = 0; v < kRlVals; ++v) lds_v[wid][v] = vals[v];
  }
  __syncthreads();
  const unsigned int blk = blockIdx.y * gridDim.x + blockIdx.x;
  if (threadIdx.x < kRlVals) {
    const int v = threadIdx.x;
    double x = lds_v[0][v];
    for (int w = 1; w < NW; ++w) x = combine(v, x, lds_v[w][v]);
    A.partials[(int64_t)blk * kRlVals + v] = x;  // reduced by ratio_loss_finalize_kernel
  }
}

template <int VEC>
__device__ __forceinline__ void fill_ones(float (&m)[VEC]) {
#pragma unroll
  for (int k = 0; k < VEC; ++k) m[k] = 1.0f;
}

template <int KIND, int VEC, bool PACKED>
__global__ __launch_bounds__(kRlThreads) void ratio_loss_fwd_kernel(RatioArgs A) {
  constexpr int NW = kRlThreads / kWave;
  constexpr int ITEMS = 2;  // vectors in flight per lane
  __shared__ double lds_v[NW][kRlVals];
  const RatioConsts C = A.C;

  Acc acc;
  SeqCtx sq;
  const bool padded = (A.layout == LAYOUT_PADDED);
  const int64_t n_rows = padded ? A.n_seq : 1;
  const int64_t stride = (int64_t)gridDim.x * kRlThreads;
  const int64_t first = (int64_t)blockIdx.x * kRlThreads + threadIdx.x;

  for (int64_t r = blockIdx.y; r < n_rows; r += gridDim.y) {
    // tokens [base, base+count) are valid; whole vectors may be loaded up to base+row_end
    int64_t base = 0, count = A.n_tok, row_end = A.n_tok;
    if (padded) {
      int64_t len = A.seq[r];
      len = len < 0 ? 0 : (len > A.seq_stride ? A.seq_stride : len);
      base = r * A.seq_stride;
      count = len;
      row_end = A.seq_stride;
      if (!C.adv_per_token) sq.adv = A.adv[r];
      sq.w = (len > 0) ? seq_weight(C, len) : 1.0f;
    }
    const int64_t nvec = (count + VEC - 1) / VEC;  // vectors holding a valid token
    const int64_t nvec_full = row_end / VEC;       // vectors that can be loaded whole
    const int64_t nload = nvec < nvec_full ? nvec : nvec_full;

    for (int64_t i0 = first; i0 < nload; i0 += stride * ITEMS) {
      float nw[ITEMS][VEC], od[ITEMS][VEC], ad[ITEMS][VEC], mk[ITEMS][VEC];
#pragma unroll
      for (int it = 0; it < ITEMS; ++it) {
        const int64_t i = i0 + it * stride;
        fill_ones(mk[it]);
        if (i < nload) {
          Vec<float, VEC>::load(A.nw + base + i * VEC, nw[it]);
          Vec<float, VEC>::load(A.od + base + i * VEC, od[it]);
          if (C.adv_per_token) Vec<float, VEC>::load(A.adv + base + i * VEC, ad[it]);
          if (A.mask) Vec<float, VEC>::load(A.mask + base + i * VEC, mk[it]);
        }
      }
#pragma unroll
      for (int it = 0; it < ITEMS; ++it) {
        const int64_t i = i0 + it * stride;
        if (i < nload) {
          float out[VEC];
          ratio_vec_fwd<KIND, VEC, PACKED>(A, C, i * VEC, count, nw[it], od[it], ad[it], mk[it], sq, acc, out);
          if (A.loss_elem) Vec<float, VEC>::store(A.loss_elem + base + i * VEC, out);
        }
      }
      acc.flush();
    }
    // a row whose length is not a multiple of VEC ends in one vector that cannot be loaded whole
    if (nvec > nvec_full && first == nvec_full % stride) {
      const int64_t t0 = nvec_full * VEC;
      float nw[VEC], od[VEC], ad[VEC], mk[VEC], out[VEC];
#pragma unroll
      for (int k = 0; k < VEC; ++k) {
        const bool ok = (t0 + k) < count;
        nw[k] = ok ? A.nw[base + t0 + k] : 0.0f;
        od[k] = ok ? A.od[base + t0 + k] : 0.0f;
        ad[k] = (ok && C.adv_per_token) ? A.adv[base + t0 + k] : 0.0f;
        mk[k] = (ok && A.mask) ? A.mask[base + t0 + k] : 1.0f;
      }
      ratio_vec_fwd<KIND, VEC, PACKED>(A, C, t0, count, nw, od, ad, mk, sq, acc, out);
      if (A.loss_elem) {
#pragma unroll
        for (int k = 0; k < VEC; ++k)
          if (t0 + k < row_end) A.loss_elem[base + t0 + k] = out[k];
      }
      acc.flush();
    }
    // padded layout: zero the loss of the slots past the sequence end
    if (A.loss_elem && padded) {
      for (int64_t t = nvec * VEC + first; t < row_end; t += stride) A.loss_elem[base + t] = 0.0f;
    }
  }
  store_block_partials(A, acc, lds_v);
}

// One workgroup: fixed-order reduction of every workgroup's partial vector, then the metrics.
__global__ __launch_bounds__(kRlThreads) void ratio_loss_finalize_kernel(RatioArgs A, unsigned int nblk) {
  __shared__ double lds_fin[kRlThreads];
  const RatioConsts C = A.C;
  {
    // thread = (value v, slice j0): 16 slices walk the workgroups' vectors, kBatch loads in flight each
    const int v = threadIdx.x % kRlVals;
    const int j0 = threadIdx.x / kRlVals;  // 0..15
    constexpr int kSlices = kRlThreads / kRlVals;
    constexpr int kBatch = 32;  // 512 workgroups: every partial of a thread in flight at once
    double x = (v == P_RMIN) ? (double)INFINITY : ((v == P_RMAX || v == P_AMAX) ? -(double)INFINITY : 0.0);
    const double ident = x;
    for (unsigned int j = j0; j < nblk; j += kSlices * kBatch) {
      double y[kBatch];
#pragma unroll
      for (int b = 0; b < kBatch; ++b) {
        const unsigned int jj = j + b * kSlices;
        y[b] = (jj < nblk) ? A.partials[(int64_t)jj * kRlVals + v] : ident;
      }
      // one kind of operation per lane, chosen once per batch (three short divergent runs) rather
      // than a three-way select per element
      if (v < P_RMIN) {
#pragma unroll
        for (int b = 0; b < kBatch; ++b) x += y[b];
      } else if (v == P_RMIN) {
#pragma unroll
        for (int b = 0; b < kBatch; ++b) x = fmin(x, y[b]);
      } else {
#pragma unroll
        for (int b = 0; b < kBatch; ++b) x = fmax(x, y[b]);
      }
    }
    lds_fin[threadIdx.x] = x;
  }
  __syncthreads();
  if (threadIdx.x < kRlVals) {
    const int v = threadIdx.x;
    double x = lds_fin[v];
    if (v < P_RMIN) {
      for (int j = 1; j < kRlThreads / kRlVals; ++j) x += lds_fin[j * kRlVals + v];
    } else if (v == P_RMIN) {
      for (int j = 1; j < kRlThreads / kRlVals; ++j) x = fmin(x, lds_fin[j * kRlVals + v]);
    } else {
      for (int j = 1; j < kRlThreads / kRlVals; ++j) x = fmax(x, lds_fin[j * kRlVals + v]);
    }
    lds_fin[v] = x;
  }
  __syncthreads();
  if (threadIdx.x != 0) return;
  const double N = lds_fin[P_CNT];
  const double sr = lds_fin[P_SR], sr2 = lds_fin[P_SR2];
  // One fp64 reciprocal serves every mean (this thread runs alone; an fp64 divide per metric was a
  // third of the kernel).  x * (1/N) and x / N differ by at most an ulp of fp64, far below the
  // fp32 result's rounding.
  const double inv_n = 1.0 / N;
  double loss = lds_fin[P_LOSS];
  if (C.agg_mode == UNIRL_AGG_TOKEN_MEAN)
    loss = loss * inv_n;
  else if (C.agg_mode == UNIRL_AGG_SEQ_MEAN_TOKEN_SUM)
    loss = loss / ((double)A.n_seq * (double)C.horizon);
  else
    loss = loss / (double)A.n_seq;
  // sr, sr2: sums of (r-1) and (r-1)^2
  double var = 0.0;
  if (N > 1.0) {
    var = (sr2 - sr * sr * inv_n) / (N - 1.0);
    if (var < 0.0) var = 0.0;
  }
  float* M = A.metrics;
  M[UNIRL_M_LOSS] = (float)loss;
  M[UNIRL_M_RATIO_MEAN] = (float)(1.0 + sr * inv_n);
  M[UNIRL_M_RATIO_STD] = (float)sqrt(var);
  // min()/max() of the reference return NaN when any ratio is NaN; the ratios are >= 0, so their
  // sum is NaN exactly then (likewise the absolute differences below)
  M[UNIRL_M_RATIO_MIN] = (sr != sr) ? quiet_nan() : (float)lds_fin[P_RMIN];
  M[UNIRL_M_RATIO_MAX] = (sr != sr) ? quiet_nan() : (float)lds_fin[P_RMAX];
  M[UNIRL_M_CLIP_FRACTION] = (float)(lds_fin[P_CANY] * inv_n);
  M[UNIRL_M_CLIPFRAC_HI] = (float)(lds_fin[P_CHI] * inv_n);
  M[UNIRL_M_CLIPFRAC_LO] = (float)(lds_fin[P_CLO] * inv_n);
  // GRPO accumulates ld^2; mean(0.5*ld^2) = 0.5*sum/N exactly (halving commutes with rounding)
  M[UNIRL_M_APPROX_KL] = (float)((C.kind == UNIRL_LOSS_GRPO ? 0.5 : 1.0) * lds_fin[P_KL] * inv_n);
  M[UNIRL_M_PENALTY_MEAN] = (float)(lds_fin[P_PEN] * inv_n);
  M[UNIRL_M_ABSDIFF_MEAN] = (float)(lds_fin[P_ABS] * inv_n);
  M[UNIRL_M_ABSDIFF_MAX] = (lds_fin[P_ABS] != lds_fin[P_ABS]) ? quiet_nan() : (float)lds_fin[P_AMAX];
  M[UNIRL_M_NUM_TOKENS] = (float)N;
  M[13] = M[14] = M[15] = 0.0f;
}

template <int KIND, int VEC>
__global__ __launch_bounds__(kRlThreads) void ratio_loss_bwd_kernel(RatioArgs A) {
  const RatioConsts C = A.C;
  // global factor of the aggregation (1 when the caller reduces loss_per_elem itself)
  float gfac = A.g_scale ? *A.g_scale : 1.0f;
  if (A.aggregate) {
    if (C.agg_mode == UNIRL_AGG_TOKEN_MEAN)
      gfac = gfac / *A.n_valid;
    else if (C.agg_mode == UNIRL_AGG_SEQ_MEAN_TOKEN_SUM)
      gfac = (gfac / (float)A.n_seq) / C.horizon;
    else
      gfac = gfac / (float)A.n_seq;
  }
  const bool padded = (A.layout == LAYOUT_PADDED);
  const int64_t n_rows = padded ? A.n_seq : 1;
  const int64_t stride = (int64_t)gridDim.x * kRlThreads;
  int64_t cur_end = -1;
  float row_adv = 0.0f, row_w = 1.0f;

  for (int64_t r = blockIdx.y; r < n_rows; r += gridDim.y) {
    int64_t base = 0, count = A.n_tok, row_end = A.n_tok;
    if (padded) {
      int64_t len = A.seq[r];
      len = len < 0 ? 0 : (len > A.seq_stride ? A.seq_stride : len);
      base = r * A.seq_stride;
      count = len;
      row_end = A.seq_stride;
      if (!C.adv_per_token) row_adv = A.adv[r];
      row_w = (len > 0) ? seq_weight(C, len) : 1.0f;
    }
    const int64_t nvec = (row_end + VEC - 1) / VEC;  // every slot of the row is written
    const int64_t nvec_full = row_end / VEC;
    for (int64_t i = (int64_t)blockIdx.x * kRlThreads + threadIdx.x; i < nvec; i += stride) {
      float nw[VEC], od[VEC], ad[VEC], mk[VEC], ge[VEC], out[VEC];
      const int64_t t0 = i * VEC;
      const bool whole = (i < nvec_full);
      if (t0 < count) {
        if (VEC == 1 || whole) {
          Vec<float, VEC>::load(A.nw + base + t0, nw);
          Vec<float, VEC>::load(A.od + base + t0, od);
          if (C.adv_per_token) Vec<float, VEC>::load(A.adv + base + t0, ad);
          if (A.mask) Vec<float, VEC>::load(A.mask + base + t0, mk);
          if (A.g_elem) Vec<float, VEC>::load(A.g_elem + base + t0, ge);
        } else {
#pragma unroll
          for (int k = 0; k < VEC; ++k) {
            const bool ok = (t0 + k) < count;
            nw[k] = ok ? A.nw[base + t0 + k] : 0.0f;
            od[k] = ok ? A.od[base + t0 + k] : 0.0f;
            if (C.adv_per_token) ad[k] = ok ? A.adv[base + t0 + k] : 0.0f;
            if (A.mask) mk[k] = ok ? A.mask[base + t0 + k] : 0.0f;
            if (A.g_elem) ge[k] = ok ? A.g_elem[base + t0 + k] : 0.0f;
          }
        }
      }
#pragma unroll
      for (int k = 0; k < VEC; ++k) {
        const int64_t t = t0 + k;
        out[k] = 0.0f;
        if (t < count) {
          if (A.layout == LAYOUT_PACKED && t >= cur_end) {
            const int64_t sq = find_seq(A.seq, A.n_seq, t);
            cur_end = A.seq[sq + 1];
            row_w = seq_weight(C, cur_end - A.seq[sq]);
            if (!C.adv_per_token) row_adv = A.adv[sq];
          }
          const float a = C.adv_per_token ? ad[k] : row_adv;
          const TokVals v = ratio_token<KIND>(nw[k], od[k], a, C);
          float g = gfac;
          if (A.aggregate) {
            g *= row_w;
            if (A.mask) g *= mk[k];
          }
          if (A.g_elem) g *= ge[k];
          out[k] = g * v.dloss;
        }
      }
      if (VEC == 1 || whole) {
        Vec<float, VEC>::store(A.grad_new + base + t0, out);
      } else {
#pragma unroll
        for (int k = 0; k < VEC; ++k)
          if (t0 + k < row_end) A.grad_new[base + t0 + k] = out[k];
      }
    }
  }
}

static int fill_consts(const unirl_ratio_loss_params* p, RatioConsts& C) {
  if (p->kind != UNIRL_LOSS_GRPO && p->kind != UNIRL_LOSS_DRPO) return UNIRL_E_DTYPE;
  if (p->agg_mode < UNIRL_AGG_TOKEN_MEAN || p->agg_mode > UNIRL_AGG_SEQ_MEAN_TOKEN_MEAN) return UNIRL_E_DTYPE;
  C.kind = p->kind;
  C.agg_mode = p->agg_mode;
  C.mu_weighted = p->mu_weighted;
  C.adv_per_token = p->adv_per_token;
  C.clamp_lo = (float)(1.0 - p->clip_low);
  C.clamp_hi = (float)(1.0 + p->clip_high);
  C.eps_lo = (float)p->clip_low;
  C.eps_hi = (float)p->clip_high;
  C.drpo_eps = (float)p->drpo_epsilon;
  C.drpo_two_eps = (float)(2.0 * p->drpo_epsilon);
  C.inv_two_eps = (float)(1.0 / (double)C.drpo_two_eps);
  C.horizon = (float)p->horizon;
  return UNIRL_OK;
}

struct RatioShape {
  int vec;
  dim3 grid;
};

static int plan(const RatioArgs& A, bool bwd, RatioShape& S) {
  const bool padded = (A.layout == LAYOUT_PADDED);
  int vec = 4;
  const void* ptrs[] = {A.nw, A.od, A.mask, A.loss_elem, A.g_elem, A.grad_new, A.C.adv_per_token ? A.adv : nullptr};
  for (const void* q : ptrs)
    if (!aligned_to(q, 16)) vec = 1;
  if (padded && A.seq_stride % 4 != 0) vec = 1;
  const int64_t row_tok = padded ? A.seq_stride : A.n_tok;
  const int64_t nvec = (row_tok + vec - 1) / vec;
  // forward: one partial vector per workgroup is read back by a single finalize workgroup, whose
  // time grows with their number (about 1 us per 128); 512 suits inputs of a few MB, 1024 large ones
  const int64_t cap = bwd ? 16384 : tune_int("UNIRL_RATIO_MAX_BLOCKS", A.n_tok >= (16 << 20) ? 1024 : 512);
  int64_t rows = padded ? A.n_seq : 1;
  if (rows > cap) rows = cap;
  if (rows < 1) rows = 1;
  int64_t nbx = (nvec + kRlThreads - 1) / kRlThreads;
  int64_t max_x = cap / rows;
  if (max_x < 1) max_x = 1;
  if (nbx > max_x) nbx = max_x;
  if (nbx < 1) nbx = 1;
  S.vec = vec;
  S.grid = dim3((unsigned int)nbx, (unsigned int)rows);
  return UNIRL_OK;
}

}  // namespace unirl

using namespace unirl;

static int check_common(const float* new_logp, const float* old_logp, const float* advantages,
                        const int64_t* lengths, int64_t n_seq, int64_t seq_stride, int64_t n_tok,
                        const unirl_ratio_loss_params* params, RatioArgs& A) {
  if (!params) return UNIRL_E_NULL;
  const int rc = fill_consts(params, A.C);
  if (rc != 0) return rc;
  if (n_seq < 0 || seq_stride < 0 || n_tok < 0) return UNIRL_E_SHAPE;
  if (!new_logp || !old_logp || !advantages) return UNIRL_E_NULL;
  if (!aligned_to(new_logp, 4) || !aligned_to(old_logp, 4) || !aligned_to(advantages, 4) || !aligned_to(lengths, 8))
    return UNIRL_E_ALIGN;
  if (!lengths) {
    A.layout = LAYOUT_FLAT;
    if (!A.C.adv_per_token) return UNIRL_E_NULL;  // per-sequence advantages need the sequence lengths
    if (A.C.agg_mode != UNIRL_AGG_TOKEN_MEAN) return UNIRL_E_NULL;
  } else if (seq_stride > 0) {
    A.layout = LAYOUT_PADDED;
    if (n_seq * seq_stride != n_tok) return UNIRL_E_SHAPE;
  } else {
    A.layout = LAYOUT_PACKED;
  }
  A.nw = new_logp;
  A.od = old_logp;
  A.adv = advantages;
  A.seq = lengths;
  A.n_seq = n_seq;
  A.seq_stride = seq_stride;
  A.n_tok = n_tok;
  return UNIRL_OK;
}

extern "C" int unirl_ratio_loss_fwd(const float* new_logp, const float* old_logp, const float* advantages,
                                    const int64_t* lengths, const float* loss_mask, int64_t n_seq,
                                    int64_t seq_stride, int64_t n_tok, const unirl_ratio_loss_params* params,
                                    float* loss_per_elem, float* metrics, void* workspace, size_t workspace_bytes,
                                    void* stream) {
  RatioArgs A = {};
  const int rc = check_common(new_logp, old_logp, advantages, lengths, n_seq, seq_stride, n_tok, params, A);
  if (rc != 0) return rc;
  if (!metrics) return UNIRL_E_NULL;
  if (!workspace || workspace_bytes < kWorkspaceBytes) return UNIRL_E_WORKSPACE;
  A.mask = loss_mask;
  A.loss_elem = loss_per_elem;
  A.metrics = metrics;
  A.partials = ws_partials(workspace);
  RatioShape S;
  plan(A, false, S);
  if ((int64_t)S.grid.x * S.grid.y * kRlVals > kPartialCapacity) return UNIRL_E_LIMIT;
  hipStream_t st = (hipStream_t)stream;
  dim3 block(kRlThreads);
  const bool packed = (A.layout == LAYOUT_PACKED);
#define UNIRL_LAUNCH_FWD(KIND, VEC)                                                                      \
  do {                                                                                                   \
    if (packed)                                                                                          \
      hipLaunchKernelGGL((ratio_loss_fwd_kernel<KIND, VEC, true>), S.grid, block, 0, st, A);             \
    else                                                                                                 \
      hipLaunchKernelGGL((ratio_loss_fwd_kernel<KIND, VEC, false>), S.grid, block, 0, st, A);            \
  } while (0)
  if (A.C.kind == UNIRL_LOSS_GRPO) {
    if (S.vec == 4) UNIRL_LAUNCH_FWD(UNIRL_LOSS_GRPO, 4); else UNIRL_LAUNCH_FWD(UNIRL_LOSS_GRPO, 1);
  } else {
    if (S.vec == 4) UNIRL_LAUNCH_FWD(UNIRL_LOSS_DRPO, 4); else UNIRL_LAUNCH_FWD(UNIRL_LOSS_DRPO, 1);
  }
#undef UNIRL_LAUNCH_FWD
  const int launch_rc = (int)hipGetLastError();
  if (launch_rc != 0) return launch_rc;
  hipLaunchKernelGGL(ratio_loss_finalize_kernel, dim3(1), block, 0, st, A, S.grid.x * S.grid.y);
  return (int)hipGetLastError();
}

extern "C" int unirl_ratio_loss_bwd(const float* new_logp, const float* old_logp, const float* advantages,
                                    const int64_t* lengths, const float* loss_mask, int64_t n_seq,
                                    int64_t seq_stride, int64_t n_tok, const unirl_ratio_loss_params* params,
                                    const float* g_scale, const float* g_elem, int aggregate,
                                    const float* n_valid, float* grad_new, void* stream) {
  RatioArgs A = {};
  const int rc = check_common(new_logp, old_logp, advantages, lengths, n_seq, seq_stride, n_tok, params, A);
  if (rc != 0) return rc;
  if (!grad_new) return UNIRL_E_NULL;
  if (aggregate && A.C.agg_mode == UNIRL_AGG_TOKEN_MEAN && !n_valid) return UNIRL_E_NULL;
  if (n_tok == 0) return UNIRL_OK;
  A.mask = loss_mask;
  A.g_scale = g_scale;
  A.g_elem = g_elem;
  A.n_valid = n_valid;
  A.aggregate = aggregate;
  A.grad_new = grad_new;
  RatioShape S;
  plan(A, true, S);
  hipStream_t st = (hipStream_t)stream;
  dim3 block(kRlThreads);
  if (A.C.kind == UNIRL_LOSS_GRPO) {
    if (S.vec == 4)
      hipLaunchKernelGGL((ratio_loss_bwd_kernel<UNIRL_LOSS_GRPO, 4>), S.grid, block, 0, st, A);
    else
      hipLaunchKernelGGL((ratio_loss_bwd_kernel<UNIRL_LOSS_GRPO, 1>), S.grid, block, 0, st, A);
  } else {
    if (S.vec == 4)
      hipLaunchKernelGGL((ratio_loss_bwd_kernel<UNIRL_LOSS_DRPO, 4>), S.grid, block, 0, st, A);
    else
      hipLaunchKernelGGL((ratio_loss_bwd_kernel<UNIRL_LOSS_DRPO, 1>), S.grid, block, 0, st, A);
  }
  return (int)hipGetLastError();
}
