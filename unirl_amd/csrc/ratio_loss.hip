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
// Sums of the ratio and its square run in fp64 per lane (the unbiased std of
// ~1e6 values near 1 needs it); the other sums run fp32 per lane over a handful
// of tokens and fp64 from the wavefront up, in a fixed order.
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

struct TokVals {
  float r, d0, ld, loss, pen, kterm, dloss;
  bool hi, lo;
};

template <int KIND>
__device__ __forceinline__ TokVals ratio_token(float nw, float od, float A, const RatioConsts& C) {
  TokVals o;
  o.d0 = nw - od;
  if (KIND == UNIRL_LOSS_GRPO) {
    o.ld = o.d0;
    o.r = expf(o.ld);
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
    o.r = expf(o.ld);
    const float mu = expf(od);
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

struct Acc {
  double sr = 0.0, sr2 = 0.0;
  float loss = 0.0f, kl = 0.0f, pen = 0.0f, ab = 0.0f;
  float rmin = INFINITY, rmax = -INFINITY, amax = -INFINITY;
  unsigned int cnt = 0, chi = 0, clo = 0, cany = 0;
};

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
// are padding.  Accumulates into acc and leaves the per-token loss in out[].
template <int KIND, int VEC>
__device__ __forceinline__ void ratio_vec_fwd(const RatioArgs& A, const RatioConsts& C, int64_t t0, int64_t count,
                                              const float (&nw)[VEC], const float (&od)[VEC],
                                              const float (&ad)[VEC], const float (&mk)[VEC], SeqCtx& sq,
                                              Acc& acc, float (&out)[VEC]) {
#pragma unroll
  for (int k = 0; k < VEC; ++k) {
    const int64_t t = t0 + k;
    out[k] = 0.0f;
    if (t < count) {
      if (A.layout == LAYOUT_PACKED && t >= sq.cur_end) {
        const int64_t s = find_seq(A.seq, A.n_seq, t);
        sq.cur_end = A.seq[s + 1];
        sq.w = seq_weight(C, sq.cur_end - A.seq[s]);
        if (!C.adv_per_token) sq.adv = A.adv[s];
      }
      const float a = C.adv_per_token ? ad[k] : sq.adv;
      const TokVals v = ratio_token<KIND>(nw[k], od[k], a, C);
      out[k] = v.loss;
      float lm = v.loss;
      if (A.mask) lm = lm * mk[k];
      acc.sr += (double)v.r;
      acc.sr2 = fma((double)v.r, (double)v.r, acc.sr2);
      acc.loss += lm * sq.w;
      acc.kl += v.kterm;
      acc.pen += v.pen;
      const float ad0 = fabsf(v.d0);
      acc.ab += ad0;
      acc.rmin = fminf(acc.rmin, v.r);
      acc.rmax = fmaxf(acc.rmax, v.r);
      acc.amax = fmaxf(acc.amax, ad0);
      acc.cnt += 1u;
      acc.chi += v.hi ? 1u : 0u;
      acc.clo += v.lo ? 1u : 0u;
      acc.cany += (v.hi || v.lo) ? 1u : 0u;
    }
  }
}

template <int KIND, int VEC>
__global__ __launch_bounds__(kRlThreads) void ratio_loss_fwd_kernel(RatioArgs A) {
  constexpr int NW = kRlThreads / kWave;
  constexpr int ITEMS = (VEC == 4) ? 4 : 2;  // vectors in flight per lane
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
          ratio_vec_fwd<KIND, VEC>(A, C, i * VEC, count, nw[it], od[it], ad[it], mk[it], sq, acc, out);
          if (A.loss_elem) Vec<float, VEC>::store(A.loss_elem + base + i * VEC, out);
        }
      }
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
        mk[k] = (ok && A.mask) ? A.mask[base + t0 + k] : 0.0f;
      }
      ratio_vec_fwd<KIND, VEC>(A, C, t0, count, nw, od, ad, mk, sq, acc, out);
      if (A.loss_elem) {
#pragma unroll
        for (int k = 0; k < VEC; ++k)
          if (t0 + k < row_end) A.loss_elem[base + t0 + k] = out[k];
      }
    }
    // padded layout: zero the loss of the slots past the sequence end
    if (A.loss_elem && padded) {
      for (int64_t t = nvec * VEC + first; t < row_end; t += stride) A.loss_elem[base + t] = 0.0f;
    }
  }

  // ---- workgroup partials -------------------------------------------------
  double vals[kRlVals];
  vals[P_SR] = wave_sum(acc.sr);
  vals[P_SR2] = wave_sum(acc.sr2);
  // 64 lanes x a handful of tokens: an fp32 shuffle tree keeps full accuracy at half the shuffles
  vals[P_LOSS] = (double)wave_sum(acc.loss);
  vals[P_KL] = (double)wave_sum(acc.kl);
  vals[P_PEN] = (double)wave_sum(acc.pen);
  vals[P_ABS] = (double)wave_sum(acc.ab);
  vals[P_CNT] = (double)wave_sum(acc.cnt);
  vals[P_CHI] = (double)wave_sum(acc.chi);
  vals[P_CLO] = (double)wave_sum(acc.clo);
  vals[P_CANY] = (double)wave_sum(acc.cany);
  vals[P_RMIN] = (double)wave_min(acc.rmin);
  vals[P_RMAX] = (double)wave_max(acc.rmax);
  vals[P_AMAX] = (double)wave_max(acc.amax);
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

// One workgroup: fixed-order reduction of every workgroup's partial vector, then the metrics.
__global__ __launch_bounds__(kRlThreads) void ratio_loss_finalize_kernel(RatioArgs A, unsigned int nblk) {
  __shared__ double lds_fin[kRlThreads];
  const RatioConsts C = A.C;
  {
    // thread = (value v, slice j0): 16 slices walk the workgroups' vectors, eight loads in flight each
    const int v = threadIdx.x % kRlVals;
    const int j0 = threadIdx.x / kRlVals;  // 0..15
    constexpr int kSlices = kRlThreads / kRlVals;
    constexpr int kBatch = 8;
    double x = (v == P_RMIN) ? (double)INFINITY : ((v == P_RMAX || v == P_AMAX) ? -(double)INFINITY : 0.0);
    const double ident = x;
    for (unsigned int j = j0; j < nblk; j += kSlices * kBatch) {
      double y[kBatch];
#pragma unroll
      for (int b = 0; b < kBatch; ++b) {
        const unsigned int jj = j + b * kSlices;
        y[b] = (jj < nblk) ? A.partials[(int64_t)jj * kRlVals + v] : ident;
      }
#pragma unroll
      for (int b = 0; b < kBatch; ++b) x = combine(v, x, y[b]);
    }
    lds_fin[threadIdx.x] = x;
  }
  __syncthreads();
  if (threadIdx.x < kRlVals) {
    const int v = threadIdx.x;
    double x = lds_fin[v];
    for (int j = 1; j < kRlThreads / kRlVals; ++j) x = combine(v, x, lds_fin[j * kRlVals + v]);
    lds_fin[v] = x;
  }
  __syncthreads();
  if (threadIdx.x != 0) return;
  const double N = lds_fin[P_CNT];
  const double sr = lds_fin[P_SR], sr2 = lds_fin[P_SR2];
  double loss = lds_fin[P_LOSS];
  if (C.agg_mode == UNIRL_AGG_TOKEN_MEAN)
    loss = loss / N;
  else if (C.agg_mode == UNIRL_AGG_SEQ_MEAN_TOKEN_SUM)
    loss = (loss / (double)A.n_seq) / (double)C.horizon;
  else
    loss = loss / (double)A.n_seq;
  double var = 0.0;
  if (N > 1.0) {
    var = (sr2 - sr * sr / N) / (N - 1.0);
    if (var < 0.0) var = 0.0;
  }
  float* M = A.metrics;
  M[UNIRL_M_LOSS] = (float)loss;
  M[UNIRL_M_RATIO_MEAN] = (float)(sr / N);
  M[UNIRL_M_RATIO_STD] = (float)sqrt(var);
  // min()/max() of the reference return NaN when any ratio is NaN; the ratios are >= 0, so their
  // sum is NaN exactly then (likewise the absolute differences below)
  M[UNIRL_M_RATIO_MIN] = (sr != sr) ? quiet_nan() : (float)lds_fin[P_RMIN];
  M[UNIRL_M_RATIO_MAX] = (sr != sr) ? quiet_nan() : (float)lds_fin[P_RMAX];
  M[UNIRL_M_CLIP_FRACTION] = (float)lds_fin[P_CANY] / (float)N;
  M[UNIRL_M_CLIPFRAC_HI] = (float)lds_fin[P_CHI] / (float)N;
  M[UNIRL_M_CLIPFRAC_LO] = (float)lds_fin[P_CLO] / (float)N;
  M[UNIRL_M_APPROX_KL] = (float)(lds_fin[P_KL] / N);
  M[UNIRL_M_PENALTY_MEAN] = (float)(lds_fin[P_PEN] / N);
  M[UNIRL_M_ABSDIFF_MEAN] = (float)(lds_fin[P_ABS] / N);
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
  const int64_t cap = bwd ? 16384 : tune_int("UNIRL_RATIO_MAX_BLOCKS", 512);
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
  if (A.C.kind == UNIRL_LOSS_GRPO) {
    if (S.vec == 4)
      hipLaunchKernelGGL((ratio_loss_fwd_kernel<UNIRL_LOSS_GRPO, 4>), S.grid, block, 0, st, A);
    else
      hipLaunchKernelGGL((ratio_loss_fwd_kernel<UNIRL_LOSS_GRPO, 1>), S.grid, block, 0, st, A);
  } else {
    if (S.vec == 4)
      hipLaunchKernelGGL((ratio_loss_fwd_kernel<UNIRL_LOSS_DRPO, 4>), S.grid, block, 0, st, A);
    else
      hipLaunchKernelGGL((ratio_loss_fwd_kernel<UNIRL_LOSS_DRPO, 1>), S.grid, block, 0, st, A);
  }
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
