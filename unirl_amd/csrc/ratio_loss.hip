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
// Kernels: ratio_loss_fwd_kernel (padded [n_seq, stride] + lengths, and flat),
// ratio_loss_packed_kernel ([n_tok] + cu_seqlens), each optionally writing the
// gradient of the aggregated loss in the same pass (the one-pass training step),
// ratio_loss_finalize_kernel (workgroup partials -> the 16 metrics) and
// ratio_loss_bwd_kernel (stand-alone backward).
//
// HBM traffic: 8 bytes read per valid token (+4 with a mask, +4 with per-token
// advantages), +4 written per slot when loss_per_elem or grad_new is requested.

#include "common_hip.h"
#include "unirl_internal.h"

namespace unirl {

constexpr int kRlThreads = 256;
constexpr int kRlVals = 16;  // slots of the workgroup reduction (13 in use)

enum { LAYOUT_FLAT = 0, LAYOUT_PADDED = 1, LAYOUT_PACKED = 2 };

// Slots of the workgroup reduction: six fp64 sums, four token counters, three fp32 maxima (the
// ratio minimum travels negated).  The reductions handle four consecutive slots per wavefront,
// so this order gives every wavefront one type and one operation.  6, 7 and 15 are unused.
enum {
  P_SR = 0, P_SR2, P_LOSS, P_KL, P_PEN, P_ABS,
  P_CNT = 8, P_CHI, P_CLO, P_CANY,
  P_NRMIN = 12, P_RMAX = 13, P_AMAX = 14
};
constexpr int kNumSums = 6, kFirstCnt = 8, kNumCnt = 4, kFirstMax = 12, kNumMax = 3;
constexpr int kRlParts = 16;  // threads that share one slot in the reductions below
static_assert(kRlParts * 16 == 256, "reductions assume 256 threads = 16 slots x 16 parts");

// What a workgroup hands to the finalize kernel: 76 bytes in five 16-byte chunks -- sums 0-1,
// 2-3, 4-5, the four counters (they fit 32 bits: a workgroup sees far fewer than 2^32 tokens),
// the three extrema (fp32 values).  The chunks are stored chunk-major, so that each finalize
// wavefront reads one contiguous array, and inside a chunk array the workgroups are ordered by
// (j mod 8, j / 8): consecutive workgroups run on different XCDs (dispatch deals them out in
// turn), each behind its own L2, and a 128-byte line written piecewise from eight L2s costs the
// reader far more than one written from a single L2 -- this order makes every line of the arrays
// the work of one XCD.  (Only speed depends on that dispatch order, never a result.)
constexpr int kRlChunks = 5;
constexpr unsigned int kXcds = 8;
__host__ __device__ __forceinline__ unsigned int partial_per_xcd(unsigned int nblk) { return (nblk + kXcds - 1) / kXcds; }
__device__ __forceinline__ char* partial_slot(char* base, unsigned int nblk, unsigned int blk, int v) {
  int chunk, off;
  if (v < kNumSums) {
    chunk = v >> 1;
    off = (v & 1) * 8;
  } else if (v < kFirstMax) {
    chunk = 3;
    off = (v - kFirstCnt) * 4;
  } else {
    chunk = 4;
    off = (v - kFirstMax) * 4;
  }
  const unsigned int per = partial_per_xcd(nblk);
  return base + ((size_t)chunk * (per * kXcds) + (blk % kXcds) * per + blk / kXcds) * 16 + off;
}

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
  float inv_eps;             // 1 / drpo_eps, correctly rounded
  float horizon;
  // DRPO, token-adaptive boundary: with epsilon >= 1 a token with mu <= 1 and r <= fast_hi =
  // fl(1 + epsilon) can be on neither side of its trust region (see drpo_flags_provably_clear)
  int fast_ok;
  float fast_hi;
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
  char* partials;  // kRlChunks * n_workgroups 16-byte units, see partial_slot
  // backward only
  const float* g_scale;
  const float* g_elem;
  const float* n_valid;  // device scalar: valid-token count from the forward
  int aggregate;
  float* grad_new;
  // fused forward + backward only
  float loss_scale;      // gradient arriving at the aggregated loss
  int64_t n_valid_host;  // token-mean denominator when the host knows it, else < 0
  int64_t per_wave;      // packed kernel: vectors in a wavefront's run (a multiple of 64)
  double inv_seq_scale;  // sequence-mean modes: 1 / n_seq or 1 / (n_seq * horizon), the loss's factor
  UNIRL_TRACE_FIELD
#ifdef UNIRL_TUNE
  int synth_len;  // timing experiment: row lengths from a hash of the row instead of the load
#endif
};

// exp(x) for fp32 within ~1.5 ulp: 2^(x*log2(e)) on the hardware exp2, with the rounding error
// of the product (carried in a second float) applied as a first-order correction.
// exp_f32_core is valid for |x| < 88.7 and NaN (callers that clamp x use it directly);
// exp_f32 falls back to the bare 2^t outside that range, which is exactly +inf above
// ln(FLT_MAX), 0 for -inf, and a denormal within 1e-5 relative in between.
__device__ __forceinline__ float exp_f32_core(float x, float& e_out) {
  constexpr float kL2eHi = 1.44269502162933349609375f;  // log2(e) rounded to fp32
  constexpr float kL2eLo = 1.925963033500011e-8f;       // log2(e) - kL2eHi
  const float t = x * kL2eHi;
  float lo = fmaf(x, kL2eHi, -t);
  lo = fmaf(x, kL2eLo, lo);
  const float e = __builtin_amdgcn_exp2f(t);
  e_out = e;
  return fmaf(e, lo * 0.693147182f, e);
}
__device__ __forceinline__ float exp_f32(float x) {
  float e;
  const float r = exp_f32_core(x, e);
  return (fabsf(x) < 88.72283172607422f) ? r : e;  // inf * lo and inf - inf would give NaN out there
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

// Per-lane accumulators.  The six sums are fp32 and are flushed into fp64 totals after every
// pass (at most ITEMS*VEC tokens), so their rounding does not grow with the input.  The ratio
// extrema are kept as bit patterns: ratios are >= 0 (or NaN), where unsigned integer order is
// float order, so each update is one integer min / max.
struct Acc {
  float s1 = 0.0f, s2 = 0.0f;  // sums of (r-1) and (r-1)^2
  float loss = 0.0f;
  float kl = 0.0f;             // GRPO: sum of ld^2 (halved at the end); DRPO: sum of (r-1) - ld
  float pen = 0.0f, ab = 0.0f;
  double t_s1 = 0.0, t_s2 = 0.0, t_loss = 0.0, t_kl = 0.0, t_pen = 0.0, t_ab = 0.0;
  unsigned int rmin = 0x7f800000u, rmax = 0u;
  float amax = 0.0f;
  unsigned int cnt = 0;
  unsigned int chi = 0, clo = 0, cany = 0;  // clip counts of the guarded path (see WaveCounts)

  // `w`: aggregation weight shared by every token of the pass (1 when the tokens carry their own)
  __device__ __forceinline__ void flush(double w) {
    t_s1 += (double)s1;
    t_s2 += (double)s2;
    t_loss = fma((double)loss, w, t_loss);  // the product is exact in fp64
    t_kl += (double)kl;
    t_pen += (double)pen;
    t_ab += (double)ab;
    s1 = s2 = loss = kl = pen = ab = 0.0f;
  }
};

// Clip counters of one wavefront.  A comparison result is a lane mask, so counting it is one
// scalar population count: the counters cost the vector unit nothing beyond the compare.  Only
// for code the whole wavefront runs together (a pass over 64 whole vectors); lanes that sit
// behind a lane-dependent branch count in Acc instead.
struct WaveCounts {
  unsigned int hi = 0, lo = 0, any = 0;
  __device__ __forceinline__ void add(bool h, bool l) {
    const unsigned long long mh = __builtin_amdgcn_ballot_w64(h), ml = __builtin_amdgcn_ballot_w64(l);
    hi += (unsigned int)__builtin_popcountll(mh);
    lo += (unsigned int)__builtin_popcountll(ml);
    any += (unsigned int)__builtin_popcountll(mh | ml);
  }
};

// One token into the accumulators; returns its loss and its two clip flags.  `lw` multiplies the
// loss inside the sum (loss mask, and the aggregation weight where it changes inside a pass).
// The arithmetic is the reference's, op for op; two rewrites are exact:
//   maximum(u, c) = (c > u) ? c : u   -- u is NaN whenever c is (c = -A*clamp(r), u = -A*r), so
//                                        NaN reaches the result as in torch.maximum;
//   1 - r = -(r - 1)                  -- rounding is symmetric, so the lower clip test reuses r-1.
// With GRAD the derivative of the token's loss with respect to new_logp is left in `dl` (the
// expressions of ratio_token, which the stand-alone backward kernel uses).
// DRPO's two boundary flags of one token: ratio beyond 1 +- epsilon_t with epsilon_t = epsilon / mu
// (torch evaluates scalar / tensor as reciprocal(tensor) * scalar; infinity where mu == 0).
__device__ __forceinline__ void drpo_flags(float r, float mu, const RatioConsts& C, bool& hi, bool& lo) {
  float aeps = C.drpo_eps;
  if (C.mu_weighted) aeps = (mu > 0.0f) ? recip_pos(mu) * C.drpo_eps : INFINITY;
  hi = r > (1.0f + aeps);
  lo = r < (1.0f - aeps);
}
// True when both flags are false without evaluating them (C.fast_ok: mu-weighted, epsilon >= 1).
// mu <= 1 gives fl(1/mu) >= 1, so epsilon_t = fl(fl(1/mu) * epsilon) >= epsilon and, rounding
// being monotone, fl(1 + epsilon_t) >= fl(1 + epsilon) = fast_hi >= r: not above.  And
// fl(1 - epsilon_t) <= fl(1 - epsilon) <= 0 < r (r = exp of a clamped value): not below.  A NaN in
// mu or r fails the comparisons and sends the token to drpo_flags.
__device__ __forceinline__ bool drpo_flags_provably_clear(float r, float mu, const RatioConsts& C) {
  return (mu <= 1.0f) && (r <= C.fast_hi);
}

// FLAGS = false (DRPO only): the boundary flags are left to the caller, who gets r and mu.
template <int KIND, bool GRAD, bool FLAGS = true>
__device__ __forceinline__ float accumulate_token(float nw, float od, float A, float lw, const RatioConsts& C,
                                                  Acc& acc, bool& hi, bool& lo, float& dl, float& r_out,
                                                  float& mu_out) {
  const float d0 = nw - od;
  float r, loss;
  dl = 0.0f;
  mu_out = 0.0f;
  if (KIND == UNIRL_LOSS_GRPO) {
    r = exp_f32(d0);
    const float nA = -A;
    const float u = nA * r;
    // clamp as a median of three (fill_consts keeps clamp_lo <= clamp_hi); like fmin(fmax()) it
    // drops a NaN ratio, which the select below then restores from u
    const float c = nA * __builtin_amdgcn_fmed3f(r, C.clamp_lo, C.clamp_hi);
    loss = (c > u) ? c : u;
    const float d = r - 1.0f;
    hi = d > C.eps_hi;
    lo = -d > C.eps_lo;
    acc.s1 += d;
    acc.s2 = fmaf(d, d, acc.s2);
    acc.kl = fmaf(d0, d0, acc.kl);
    if (GRAD) {
      const bool inside = (r >= C.clamp_lo) && (r <= C.clamp_hi);
      const float dc = inside ? c : 0.0f;
      dl = (u > c) ? u : ((u < c) ? dc : 0.5f * (u + dc));
    }
  } else {
    const float ld = (d0 != d0) ? d0 : fminf(fmaxf(d0, -20.0f), 20.0f);  // torch.clamp keeps NaN
    float e;
    r = exp_f32_core(ld, e);  // |ld| <= 20
    const float mu = exp_f32(od);
    const float d = r - 1.0f;
    const float w = C.mu_weighted ? mu : 1.0f;
    const float pen = div_by_const((fabsf(A) * w) * (d * d), C.drpo_two_eps, C.inv_two_eps);
    loss = (-A) * r + pen;
    if (FLAGS) drpo_flags(r, mu, C, hi, lo);
    else hi = lo = false;
    mu_out = mu;
    acc.s1 += d;
    acc.s2 = fmaf(d, d, acc.s2);
    acc.kl += d - ld;
    acc.pen += pen;
    if (GRAD) {
      const bool clamped = (d0 < -20.0f) || (d0 > 20.0f);
      dl = clamped ? 0.0f : ((-A) + div_by_const((fabsf(A) * w) * d, C.drpo_eps, C.inv_eps)) * r;
    }
  }
  acc.loss += loss * lw;
  const float a0 = fabsf(d0);
  acc.ab += a0;
  acc.amax = fmaxf(acc.amax, a0);  // a NaN drops out here; the finalize kernel restores it from the sum
  const unsigned int rb = __float_as_uint(r);
  acc.rmin = rb < acc.rmin ? rb : acc.rmin;
  acc.rmax = rb > acc.rmax ? rb : acc.rmax;
  r_out = r;
  return loss;
}
template <int KIND, bool GRAD>
__device__ __forceinline__ float accumulate_token(float nw, float od, float A, float lw, const RatioConsts& C,
                                                  Acc& acc, bool& hi, bool& lo, float& dl) {
  float r, mu;
  return accumulate_token<KIND, GRAD, true>(nw, od, A, lw, C, acc, hi, lo, dl, r, mu);
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
// are padding.  mk[] holds 1 when there is no loss mask.  Accumulates into acc, leaves the
// per-token loss in out[] and the clip flags in hi[] / lo[] (false for padding).  Whole vectors
// outside the packed layout take a path without per-token bounds or sequence checks.  Outside
// the packed layout the aggregation weight is the same for the whole pass and is applied by
// Acc::flush; in the packed layout it rides on every token.
template <int KIND, int VEC, bool PACKED, bool GRAD>
__device__ __forceinline__ void ratio_vec_fwd(const RatioArgs& A, const RatioConsts& C, int64_t t0, int64_t count,
                                              const float (&nw)[VEC], const float (&od)[VEC],
                                              const float (&ad)[VEC], const float (&mk)[VEC], bool adv_tok,
                                              float gfac, SeqCtx& sq, Acc& acc, float (&out)[VEC],
                                              float (&gr)[VEC]) {
  if (!PACKED && t0 + VEC <= count) {
    const float grow = gfac * sq.w;
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
      const float a = adv_tok ? ad[k] : sq.adv;
      bool hi, lo;
      float dl;
      out[k] = accumulate_token<KIND, GRAD>(nw[k], od[k], a, mk[k], C, acc, hi, lo, dl);
      gr[k] = (grow * mk[k]) * dl;
      acc.chi += hi ? 1u : 0u;
      acc.clo += lo ? 1u : 0u;
      acc.cany += (hi || lo) ? 1u : 0u;
    }
    acc.cnt += VEC;
    return;
  }
#pragma unroll
  for (int k = 0; k < VEC; ++k) {
    const int64_t t = t0 + k;
    out[k] = 0.0f;
    gr[k] = 0.0f;
    if (t < count) {
      if (PACKED && t >= sq.cur_end) {
        const int64_t s = find_seq(A.seq, A.n_seq, t);
        sq.cur_end = A.seq[s + 1];
        sq.w = seq_weight(C, sq.cur_end - A.seq[s]);
        if (!adv_tok) sq.adv = A.adv[s];
      }
      const float a = adv_tok ? ad[k] : sq.adv;
      bool hi, lo;
      float dl;
      out[k] = accumulate_token<KIND, GRAD>(nw[k], od[k], a, PACKED ? mk[k] * sq.w : mk[k], C, acc, hi, lo, dl);
      gr[k] = ((gfac * sq.w) * mk[k]) * dl;
      acc.chi += hi ? 1u : 0u;
      acc.clo += lo ? 1u : 0u;
      acc.cany += (hi || lo) ? 1u : 0u;
      acc.cnt += 1u;
    }
  }
}

// The same for a vector that is whole and valid in all 64 lanes (outside the packed layout): no
// bounds checks, and the clip flags are counted per wavefront.
// WTOK: the aggregation weight rides on every token (packed layout) instead of on the flush.
template <int KIND, int VEC, bool GRAD, bool WTOK = false>
__device__ __forceinline__ void ratio_vec_wave(const RatioConsts& C, const float (&nw)[VEC],
                                               const float (&od)[VEC], const float (&ad)[VEC],
                                               const float (&mk)[VEC], bool adv_tok, float gfac, const SeqCtx& sq,
                                               Acc& acc, WaveCounts& wc, float (&out)[VEC], float (&gr)[VEC]) {
  const float grow = gfac * sq.w;
  if (KIND == UNIRL_LOSS_DRPO && C.fast_ok) {
    // The boundary flags cost a reciprocal and two comparisons per token and are almost never set:
    // evaluate them only when some token of the wavefront's vector is not provably clear of both.
    float r[VEC], mu[VEC];
    bool slow = false;
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
      const float a = adv_tok ? ad[k] : sq.adv;
      bool hi, lo;
      float dl;
      out[k] = accumulate_token<KIND, GRAD, false>(nw[k], od[k], a, WTOK ? mk[k] * sq.w : mk[k], C, acc, hi, lo, dl,
                                                   r[k], mu[k]);
      gr[k] = (grow * mk[k]) * dl;
      slow = slow || !drpo_flags_provably_clear(r[k], mu[k], C);
    }
    if (__builtin_amdgcn_ballot_w64(slow) != 0ull) {
#pragma unroll
      for (int k = 0; k < VEC; ++k) {
        bool hi, lo;
        drpo_flags(r[k], mu[k], C, hi, lo);
        wc.add(hi, lo);
      }
    }
    acc.cnt += VEC;
    return;
  }
#pragma unroll
  for (int k = 0; k < VEC; ++k) {
    const float a = adv_tok ? ad[k] : sq.adv;
    bool hi, lo;
    float dl;
    out[k] = accumulate_token<KIND, GRAD>(nw[k], od[k], a, WTOK ? mk[k] * sq.w : mk[k], C, acc, hi, lo, dl);
    gr[k] = (grow * mk[k]) * dl;
    wc.add(hi, lo);
  }
  acc.cnt += VEC;
}

__device__ __forceinline__ bool slot_used(int v) {
  return v < kNumSums || (v >= kFirstCnt && v < kFirstCnt + kNumCnt) || (v >= kFirstMax && v < kFirstMax + kNumMax);
}

// LDS of the workgroup reduction, each value in its own type: [slot][thread].
struct RlLds {
  double sums[kNumSums][kRlThreads];
  unsigned int cnts[kNumCnt][kRlThreads];
  float exts[kNumMax][kRlThreads];
};

// Workgroup partial vector -> A.partials[workgroup].  Every thread must call.
// Through LDS rather than thirteen wavefront reductions: every thread stores its values as
// [slot][thread] (consecutive lanes, consecutive words), then thread (slot, part) = (tid / 16,
// tid % 16) combines the sixteen entries part, part + 16, ... of its slot and four row shifts
// finish each 16-lane row.  Fixed order, one barrier.
__device__ __forceinline__ void store_block_partials(const RatioArgs& A, Acc& acc, const WaveCounts& wc, RlLds& lds) {
  const int t = threadIdx.x;
  const bool lead = (t & (kWave - 1)) == 0;  // carries the wavefront's own counters
  lds.sums[P_SR][t] = acc.t_s1;
  lds.sums[P_SR2][t] = acc.t_s2;
  lds.sums[P_LOSS][t] = acc.t_loss;
  lds.sums[P_KL][t] = acc.t_kl;
  lds.sums[P_PEN][t] = acc.t_pen;
  lds.sums[P_ABS][t] = acc.t_ab;
  lds.cnts[P_CNT - kFirstCnt][t] = acc.cnt;
  lds.cnts[P_CHI - kFirstCnt][t] = acc.chi + (lead ? wc.hi : 0u);
  lds.cnts[P_CLO - kFirstCnt][t] = acc.clo + (lead ? wc.lo : 0u);
  lds.cnts[P_CANY - kFirstCnt][t] = acc.cany + (lead ? wc.any : 0u);
  // NaN ratios drop out of the maxima below; the finalize kernel restores NaN from the sums
  lds.exts[P_NRMIN - kFirstMax][t] = -__uint_as_float(acc.rmin);
  lds.exts[P_RMAX - kFirstMax][t] = acc.cnt ? __uint_as_float(acc.rmax) : -INFINITY;
  lds.exts[P_AMAX - kFirstMax][t] = acc.cnt ? acc.amax : -INFINITY;
  __syncthreads();
  constexpr int kPer = kRlThreads / kRlParts;
  const int v = t / kRlParts, part = t % kRlParts;
  const unsigned int blk = blockIdx.y * gridDim.x + blockIdx.x, nblk = gridDim.x * gridDim.y;
  char* out = partial_slot(A.partials, nblk, blk, v);  // reduced by ratio_loss_finalize_kernel
  // The chunk arrays hold 8 * ceil(nblk / 8) positions; when nblk is not a multiple of 8 the last
  // position of the XCDs nblk % 8 ... 7 belongs to no workgroup: workgroup 0 stores the identity there.
  if (blk == 0 && (nblk % kXcds) != 0 && t < kRlChunks * (int)kXcds) {
    const unsigned int chunk = t / kXcds, x = t % kXcds, per = partial_per_xcd(nblk);
    if (x >= nblk % kXcds) {
      const unsigned int w = (chunk == 4) ? 0xff800000u : 0u;  // -inf for the maxima, 0 for sums and counters
      const u32x4 ident = {w, w, w, w};
      reinterpret_cast<u32x4*>(A.partials)[(size_t)chunk * (per * kXcds) + x * per + per - 1] = ident;
    }
  }
  if (v < kNumSums) {
    double y[kPer];
#pragma unroll
    for (int j = 0; j < kPer; ++j) y[j] = lds.sums[v][j * kRlParts + part];
    double x = y[0];
#pragma unroll
    for (int j = 1; j < kPer; ++j) x += y[j];
    x = row_sum_last(x);
    if (part == kRlParts - 1) *reinterpret_cast<double*>(out) = x;
  } else if (v >= kFirstCnt && v < kFirstCnt + kNumCnt) {
    unsigned int x = 0;
#pragma unroll
    for (int j = 0; j < kPer; ++j) x += lds.cnts[v - kFirstCnt][j * kRlParts + part];
    x = row_sum_last(x);
    if (part == kRlParts - 1) *reinterpret_cast<unsigned int*>(out) = x;
  } else if (v >= kFirstMax && v < kFirstMax + kNumMax) {
    float y[kPer];
#pragma unroll
    for (int j = 0; j < kPer; ++j) y[j] = lds.exts[v - kFirstMax][j * kRlParts + part];
    float x = y[0];
#pragma unroll
    for (int j = 1; j < kPer; ++j) x = fmaxf(x, y[j]);
    x = row_max_last(x);
    if (part == kRlParts - 1) *reinterpret_cast<float*>(out) = x;
  }
}

template <int VEC>
__device__ __forceinline__ void fill_ones(float (&m)[VEC]) {
#pragma unroll
  for (int k = 0; k < VEC; ++k) m[k] = 1.0f;
}

// FLAGS >= 0 fixes at compile time whether a loss mask (bit 0) and per-token advantages (bit 1)
// are read, which keeps the loads of a pass straight-line code (all of them in flight before the
// first use); FLAGS < 0 reads both switches at run time.
// With GRAD the kernel also writes grad_new = loss_scale * w_tok * dloss/dnew (the aggregation
// weights of ratio_loss_bwd_kernel with aggregate set), so a training step reads new / old once.
// ITEMS: vectors in flight per lane and pass.  Two on large inputs (four cost registers: 10 %
// slower for DRPO on 8 M tokens); four when that covers every row in a single pass, because a
// second pass cannot start before the first has come back and at a few MB a trip to memory is
// most of the kernel (9.2 -> 8.7 us on 1.1 M tokens in 256 ragged rows).
template <int KIND, int VEC, bool PACKED, int FLAGS, bool GRAD, int ITEMS = 2>
__global__ __launch_bounds__(kRlThreads) void ratio_loss_fwd_kernel(RatioArgs A) {
  __shared__ RlLds lds_v;
  UNIRL_TRACE_T0();
  const RatioConsts C = A.C;
  const bool has_mask = (FLAGS < 0) ? (A.mask != nullptr) : ((FLAGS & 1) != 0);
  const bool adv_tok = (FLAGS < 0) ? (C.adv_per_token != 0) : ((FLAGS & 2) != 0);

  // global factor of the gradient; the token-mean denominator is the number of valid tokens,
  // which is the sum of the (clamped) lengths when the host did not pass it.  That sum is only
  // needed once the first data has arrived: its loads go out here, and the sum itself (a
  // workgroup reduction) is taken by every wavefront after it has issued its first pass of
  // loads -- or after the row loop, for a wavefront without a pass.  Every wavefront of the
  // workgroup takes it exactly once, so the barriers inside pair up.
  float gfac = 0.0f;
  bool sum_pending = false;
  int64_t len_first = 0;
  if (GRAD) {
    if (C.agg_mode == UNIRL_AGG_TOKEN_MEAN) {
      if (A.n_valid_host < 0) {
        sum_pending = true;
        if ((int64_t)threadIdx.x < A.n_seq) len_first = A.seq[threadIdx.x];
      } else {
        gfac = A.loss_scale / (float)(double)A.n_valid_host;
      }
    } else if (C.agg_mode == UNIRL_AGG_SEQ_MEAN_TOKEN_SUM) {
      gfac = (A.loss_scale / (float)A.n_seq) / C.horizon;
    } else {
      gfac = A.loss_scale / (float)A.n_seq;
    }
  }
  auto finish_token_count = [&]() {
    auto clamped = [&](int64_t len) { return len < 0 ? 0 : (len > A.seq_stride ? A.seq_stride : len); };
    double s = (double)clamped(len_first);  // exact: lengths are far below 2^53
    for (int64_t i = (int64_t)threadIdx.x + kRlThreads; i < A.n_seq; i += kRlThreads) s += (double)clamped(A.seq[i]);
    const double nv = block_sum(s, &lds_v.sums[0][0]);
    __syncthreads();  // lds_v is reused at the end
    gfac = A.loss_scale / (float)nv;
    sum_pending = false;
  };

  Acc acc;
  WaveCounts wc;
  SeqCtx sq;
  const bool padded = (A.layout == LAYOUT_PADDED);
  const int64_t n_rows = padded ? A.n_seq : 1;
  const int64_t stride = (int64_t)gridDim.x * kRlThreads;
  // The pass loop runs on a wave-uniform index (every lane makes the same trips; lanes past the
  // end idle inside a pass), which keeps the wave together where the clip flags are counted.
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave_first =
      (int64_t)blockIdx.x * kRlThreads + (__builtin_amdgcn_readfirstlane((int)threadIdx.x) & ~(kWave - 1));
  const int64_t first = wave_first + lane;

  for (int64_t r = blockIdx.y; r < n_rows; r += gridDim.y) {
    // tokens [base, base+count) are valid; whole vectors may be loaded up to base+row_end
    int64_t base = 0, count = A.n_tok, row_end = A.n_tok;
    if (padded) {
      int64_t len;
#ifdef UNIRL_TUNE
      // measurement build only: what the kernel would cost if a row's length needed no trip to
      // memory (the results are those of other lengths; a timing experiment)
      if (A.synth_len) len = 512 + (int64_t)(((unsigned int)r * 2654435761u) >> 8) % (A.seq_stride - 511);
      else
#endif
      len = A.seq[r];
      len = len < 0 ? 0 : (len > A.seq_stride ? A.seq_stride : len);
      base = r * A.seq_stride;
      count = len;
      row_end = A.seq_stride;
      if (!adv_tok) sq.adv = A.adv[r];
      sq.w = (len > 0) ? seq_weight(C, len) : 1.0f;
    }
    const double pass_w = PACKED ? 1.0 : (double)sq.w;
    const int64_t nvec = (count + VEC - 1) / VEC;  // vectors holding a valid token
    const int64_t nvec_full = row_end / VEC;       // vectors that can be loaded whole
    const int64_t nload = nvec < nvec_full ? nvec : nvec_full;

    // INVARIANT: finish_token_count() holds the only workgroup barriers before store_block_partials,
    // and every wavefront takes it exactly once -- inside this loop (its first pass) or after the row
    // loop.  The wavefronts therefore reach those barriers at different program points, which pairs up
    // only because s_barrier counts arrivals and this loop's bounds are wave-uniform.  No other barrier
    // may be placed inside the row loop, and no loop bound here may become lane-dependent.
    for (int64_t w0 = wave_first; w0 < nload; w0 += stride * ITEMS) {
      float nw[ITEMS][VEC], od[ITEMS][VEC], ad[ITEMS][VEC], mk[ITEMS][VEC];
      // Every item loads: past the end the index falls back to the row's last loadable vector
      // (in flight for another lane anyway) and the values go unused, so no load waits behind a
      // branch and all of a pass are in flight together.
#pragma unroll
      for (int it = 0; it < ITEMS; ++it) {
        const int64_t i = w0 + lane + it * stride;
        const int64_t ic = (i < nload) ? i : nload - 1;
        Vec<float, VEC>::load(A.nw + base + ic * VEC, nw[it]);
        Vec<float, VEC>::load(A.od + base + ic * VEC, od[it]);
        if (adv_tok) Vec<float, VEC>::load(A.adv + base + ic * VEC, ad[it]);
        if (has_mask) Vec<float, VEC>::load(A.mask + base + ic * VEC, mk[it]);
        else fill_ones(mk[it]);
      }
      if (GRAD && sum_pending) finish_token_count();
#pragma unroll
      for (int it = 0; it < ITEMS; ++it) {
        const int64_t wv = w0 + it * stride;  // the wavefront's first vector of this item
        const int64_t i = wv + lane;
        float out[VEC], gr[VEC];
        if (!PACKED && (wv + kWave) * VEC <= count) {
          ratio_vec_wave<KIND, VEC, GRAD>(C, nw[it], od[it], ad[it], mk[it], adv_tok, gfac, sq, acc, wc, out, gr);
          if (A.loss_elem) Vec<float, VEC>::store(A.loss_elem + base + i * VEC, out);
          if (GRAD) Vec<float, VEC>::store(A.grad_new + base + i * VEC, gr);
        } else if (i < nload) {
          ratio_vec_fwd<KIND, VEC, PACKED, GRAD>(A, C, i * VEC, count, nw[it], od[it], ad[it], mk[it], adv_tok, gfac,
                                                 sq, acc, out, gr);
          if (A.loss_elem) Vec<float, VEC>::store(A.loss_elem + base + i * VEC, out);
          if (GRAD) Vec<float, VEC>::store(A.grad_new + base + i * VEC, gr);
        }
      }
      acc.flush(pass_w);
    }
    // a row whose length is not a multiple of VEC ends in one vector that cannot be loaded whole;
    // one lane of the grid takes it token by token
    if (nvec > nvec_full && first == nvec_full % stride) {  // (flat layout only: no pending sum there)
      const int64_t t0 = nvec_full * VEC;
      float nw[VEC], od[VEC], ad[VEC], mk[VEC], out[VEC], gr[VEC];
#pragma unroll
      for (int k = 0; k < VEC; ++k) {
        const bool ok = (t0 + k) < count;
        nw[k] = ok ? A.nw[base + t0 + k] : 0.0f;
        od[k] = ok ? A.od[base + t0 + k] : 0.0f;
        ad[k] = (ok && adv_tok) ? A.adv[base + t0 + k] : 0.0f;
        mk[k] = (ok && has_mask) ? A.mask[base + t0 + k] : 1.0f;
      }
      ratio_vec_fwd<KIND, VEC, PACKED, GRAD>(A, C, t0, count, nw, od, ad, mk, adv_tok, gfac, sq, acc, out, gr);
#pragma unroll
      for (int k = 0; k < VEC; ++k) {
        if (t0 + k < row_end) {
          if (A.loss_elem) A.loss_elem[base + t0 + k] = out[k];
          if (GRAD) A.grad_new[base + t0 + k] = gr[k];
        }
      }
      acc.flush(pass_w);
    }
    // padded layout: zero the loss (and the gradient) of the slots past the sequence end
    if ((A.loss_elem || GRAD) && padded) {
      // whole vectors first (about half of a ragged batch is padding), then the row's last slots
      float zero[VEC];
#pragma unroll
      for (int k = 0; k < VEC; ++k) zero[k] = 0.0f;
      for (int64_t i = nvec + first; i < nvec_full; i += stride) {
        if (A.loss_elem) Vec<float, VEC>::store(A.loss_elem + base + i * VEC, zero);
        if (GRAD) Vec<float, VEC>::store(A.grad_new + base + i * VEC, zero);
      }
      const int64_t t_tail = (nvec > nvec_full ? nvec : nvec_full) * VEC;
      for (int64_t t = t_tail + first; t < row_end; t += stride) {
        if (A.loss_elem) A.loss_elem[base + t] = 0.0f;
        if (GRAD) A.grad_new[base + t] = 0.0f;
      }
    }
  }
  if (GRAD && sum_pending) finish_token_count();
  UNIRL_TRACE_MARK1();
  store_block_partials(A, acc, wc, lds_v);
  UNIRL_TRACE_END(A.trace);
}

// Largest s in [lo, n_seq) with cu(s) <= tok, found by the whole wavefront: every round 64 lanes
// probe the bracket at equal steps and a ballot picks the step, so n_seq <= 4096 takes two
// dependent loads where a bisection takes twelve.  Requires cu(lo) <= tok; wave-uniform result.
template <typename CU>
__device__ __forceinline__ int64_t wave_find_seq(const CU& cu, int64_t n_seq, int64_t tok, int64_t lo) {
  const int lane = threadIdx.x & (kWave - 1);
  int64_t hi = n_seq;
  while (hi - lo > 1) {
    const int64_t step = (hi - lo + kWave - 1) / kWave;
    const int64_t probe = lo + lane * step;
    const bool ok = probe < hi && cu(probe) <= tok;  // true on a prefix of the lanes (cu is sorted)
    int k = __builtin_popcountll(__builtin_amdgcn_ballot_w64(ok)) - 1;
    k = k < 0 ? 0 : k;
    const int64_t nlo = lo + k * step;
    const int64_t nhi = nlo + step;
    lo = nlo;
    hi = nhi < hi ? nhi : hi;
  }
  return lo;
}

// Packed layout ([n_tok] tokens, cu_seqlens), 16-byte vectors.  Every wavefront owns one
// contiguous run of vectors -- the valid tokens are balanced exactly, whatever the sequence
// lengths -- and walks it in spans of 64 vectors while it tracks the sequence under its span
// in scalar registers.  A span inside one sequence (all but one or two per sequence) runs the
// wave-uniform path of the padded kernel with a scalar advantage and weight; a span that holds
// one sequence boundary picks the advantage and the weight per token from the two sequences;
// only a span with several boundaries (sequences shorter than 256 tokens) walks lane by lane.
// The sequence lookups read cu_seqlens from memory (a 64-way search: two dependent loads up to
// 4096 sequences; afterwards the next sequence is one load away).  Copies of the table in LDS,
// or in the wavefront's registers with ballot searches, were measured and are no faster: the
// workgroup barrier, or the chain of lane reads, costs what the loads cost.
template <int KIND, int FLAGS, bool GRAD, int ITEMS>
__global__ __launch_bounds__(kRlThreads) void ratio_loss_packed_kernel(RatioArgs A) {
  constexpr int VEC = 4;
  __shared__ RlLds lds_v;
  UNIRL_TRACE_T0();
  const RatioConsts C = A.C;
  const bool has_mask = (FLAGS & 1) != 0;
  const bool adv_tok = (FLAGS & 2) != 0;

  float gfac = 0.0f;
  if (GRAD) {
    // the gradient arriving at the loss: a host scalar (one-pass step) or a device scalar (backward)
    const float ls = A.g_scale ? *A.g_scale : A.loss_scale;
    if (C.agg_mode == UNIRL_AGG_TOKEN_MEAN)
      gfac = ls / (float)A.n_tok;
    else if (C.agg_mode == UNIRL_AGG_SEQ_MEAN_TOKEN_SUM)
      gfac = (ls / (float)A.n_seq) / C.horizon;
    else
      gfac = ls / (float)A.n_seq;
  }

  Acc acc;
  WaveCounts wc;
  SeqCtx sq;  // per-lane state of the token-by-token tail
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave_id =
      (int64_t)blockIdx.x * (kRlThreads / kWave) + __builtin_amdgcn_readfirstlane((int)threadIdx.x) / kWave;
  const int64_t count = A.n_tok;
  const int64_t nvec_full = count / VEC;
  // The wavefront's run: A.per_wave vectors, an equal share rounded up to whole spans (the host
  // launches just the wavefronts that have one).  Dealing the spans to the wavefronts in turn
  // instead, as the padded kernel does, needs a sequence search per span: 10 % slower.
  const int64_t per_wave = A.per_wave;
  const int64_t v0 = wave_id * per_wave < nvec_full ? wave_id * per_wave : nvec_full;
  const int64_t v1 = (v0 + per_wave < nvec_full) ? v0 + per_wave : nvec_full;

  int64_t cur = 0, cur_end = -1;  // sequence under the current span; cur_end < 0: none yet
  SeqCtx u;                       // its advantage and weight (wave-uniform)

  float nw[ITEMS][VEC], od[ITEMS][VEC], ad[ITEMS][VEC], mk[ITEMS][VEC];
  // every lane loads every item: past the run's end the index falls back to its last vector
  auto load_pass = [&](int64_t w0) {
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      const int64_t i = w0 + it * kWave + lane;
      const int64_t ic = (i < v1) ? i : v1 - 1;
      Vec<float, VEC>::load(A.nw + ic * VEC, nw[it]);
      Vec<float, VEC>::load(A.od + ic * VEC, od[it]);
      if (adv_tok) Vec<float, VEC>::load(A.adv + ic * VEC, ad[it]);
      if (has_mask) Vec<float, VEC>::load(A.mask + ic * VEC, mk[it]);
      else fill_ones(mk[it]);
    }
  };
  if (v0 < v1) load_pass(v0);  // in flight while the first sequence is looked up

  const int64_t n_seq = A.n_seq;
  auto cu = [&](int64_t j) -> int64_t { return A.seq[j]; };
  auto seq_adv = [&](int64_t j) -> float { return A.adv[j]; };

  for (int64_t w0 = v0; w0 < v1; w0 += kWave * ITEMS) {
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      const int64_t s0 = w0 + it * kWave;  // first vector of the span (wave-uniform)
      if (s0 < v1) {
        const int64_t tok0 = s0 * VEC;
        if (tok0 >= cur_end) {
          // usually the next sequence; a full search only at the start and past very short ones
          bool found = false;
          if (cur_end >= 0 && cur + 2 <= n_seq) {
            const int64_t e2 = cu(cur + 2);
            if (tok0 < e2) {
              u.w = seq_weight(C, e2 - cur_end);
              cur += 1;
              cur_end = e2;
              found = true;
            }
          }
          if (!found) {
            cur = wave_find_seq(cu, n_seq, tok0, cur_end < 0 ? 0 : cur);
            const int64_t beg = cu(cur);
            cur_end = cu(cur + 1);
            u.w = seq_weight(C, cur_end - beg);
          }
          if (!adv_tok) u.adv = seq_adv(cur);
        }
        const int64_t i = s0 + lane;
        float out[VEC], gr[VEC];
        const bool whole = (s0 + kWave <= v1);  // all 64 lanes hold a vector of the run
        const int64_t span_end = (s0 + kWave) * VEC;
        // end of the next sequence, when the span runs past the current one
        const int64_t next_end = (whole && span_end > cur_end && cur + 2 <= n_seq) ? cu(cur + 2) : -1;
        if (whole && span_end <= cur_end) {
          ratio_vec_wave<KIND, VEC, GRAD, true>(C, nw[it], od[it], ad[it], mk[it], adv_tok, gfac, u, acc, wc, out, gr);
          if (A.loss_elem) Vec<float, VEC>::store(A.loss_elem + i * VEC, out);
          if (GRAD) Vec<float, VEC>::store(A.grad_new + i * VEC, gr);
        } else if (whole && span_end <= next_end) {
          // exactly one sequence ends inside the span: still the wave-uniform path, with the
          // advantage and the weight picked per token from the two sequences
          SeqCtx nx;
          nx.w = seq_weight(C, next_end - cur_end);
          if (!adv_tok) nx.adv = seq_adv(cur + 1);
          float ad2[VEC], mk2[VEC];
#pragma unroll
          for (int k = 0; k < VEC; ++k) {
            const bool second = (i * VEC + k) >= cur_end;
            ad2[k] = adv_tok ? ad[it][k] : (second ? nx.adv : u.adv);
            mk2[k] = mk[it][k] * (second ? nx.w : u.w);
          }
          SeqCtx one;  // weight 1: it is inside mk2
          ratio_vec_wave<KIND, VEC, GRAD, false>(C, nw[it], od[it], ad2, mk2, true, gfac, one, acc, wc, out, gr);
          cur += 1;
          cur_end = next_end;
          u = nx;
          if (A.loss_elem) Vec<float, VEC>::store(A.loss_elem + i * VEC, out);
          if (GRAD) Vec<float, VEC>::store(A.grad_new + i * VEC, gr);
        } else if (i < v1) {
          // a sequence ends inside the span: every lane walks on from the span's first sequence
          int64_t ls = cur, lend = cur_end;
          float lw = u.w, ladv = u.adv;
#pragma unroll
          for (int k = 0; k < VEC; ++k) {
            const int64_t t = i * VEC + k;
            while (t >= lend && ls + 1 < n_seq) {
              ++ls;
              const int64_t e = cu(ls + 1);
              lw = seq_weight(C, e - lend);
              lend = e;
              if (!adv_tok) ladv = seq_adv(ls);
            }
            bool hi, lo;
            float dl;
            out[k] = accumulate_token<KIND, GRAD>(nw[it][k], od[it][k], adv_tok ? ad[it][k] : ladv, mk[it][k] * lw, C,
                                                  acc, hi, lo, dl);
            gr[k] = ((gfac * lw) * mk[it][k]) * dl;
            acc.chi += hi ? 1u : 0u;
            acc.clo += lo ? 1u : 0u;
            acc.cany += (hi || lo) ? 1u : 0u;
          }
          acc.cnt += VEC;
          if (A.loss_elem) Vec<float, VEC>::store(A.loss_elem + i * VEC, out);
          if (GRAD) Vec<float, VEC>::store(A.grad_new + i * VEC, gr);
        }
      }
    }
    if (w0 + kWave * ITEMS < v1) load_pass(w0 + kWave * ITEMS);
    acc.flush(1.0);
  }
  // the last count % VEC tokens cannot be loaded as a vector; one lane takes them
  if (nvec_full * VEC < count && blockIdx.x == 0 && threadIdx.x == 0) {
    const int64_t t0 = nvec_full * VEC;
    float nw[VEC], od[VEC], ad[VEC], mk[VEC], out[VEC], gr[VEC];
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
      const bool ok = (t0 + k) < count;
      nw[k] = ok ? A.nw[t0 + k] : 0.0f;
      od[k] = ok ? A.od[t0 + k] : 0.0f;
      ad[k] = (ok && adv_tok) ? A.adv[t0 + k] : 0.0f;
      mk[k] = (ok && has_mask) ? A.mask[t0 + k] : 1.0f;
    }
    ratio_vec_fwd<KIND, VEC, true, GRAD>(A, C, t0, count, nw, od, ad, mk, adv_tok, gfac, sq, acc, out, gr);
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
      if (t0 + k < count) {
        if (A.loss_elem) A.loss_elem[t0 + k] = out[k];
        if (GRAD) A.grad_new[t0 + k] = gr[k];
      }
    }
    acc.flush(1.0);
  }
  UNIRL_TRACE_MARK1();
  if (A.partials) store_block_partials(A, acc, wc, lds_v);  // absent when only the gradient is wanted
  UNIRL_TRACE_END(A.trace);
}

// One workgroup of six wavefronts.  Wavefronts 0-2 read the three chunks of sums, wavefronts 3 and
// 4 the counter chunk (two counters each: no wavefront reduces more than two 64-bit values),
// wavefront 5 the extrema; lane l takes the vectors l, l + 64, ... of its chunk, every load of a
// lane in flight at once; the lane adds its values pairwise (a tree of fixed shape), one wavefront
// reduction per value then leaves the thirteen totals in LDS and sixteen lanes turn them into the
// metrics.  Fixed order throughout.
// kBatch: loads a lane has in flight per trip, chosen by the host to cover the positions in one trip
// where it can (4, 8 or 16 for up to 256, 512 or more positions): a surplus load costs as much as
// a useful one.
constexpr int kFinThreads = 6 * kWave;
template <int kBatch>
__global__ __launch_bounds__(kFinThreads) void ratio_loss_finalize_kernel(RatioArgs A, unsigned int nblk) {
  __shared__ double lds_tot[kRlVals];
  UNIRL_TRACE_T0();
  const RatioConsts C = A.C;
  const int t = threadIdx.x;
  {
    const int lane = t & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(t) / kWave;  // wave-uniform
    const int chunk = wave < 4 ? wave : wave - 1;                // wavefronts 3 and 4 share the counters
    const unsigned int per = partial_per_xcd(nblk), npos = per * kXcds;
    const u32x4* src = reinterpret_cast<const u32x4*>(A.partials) + (size_t)chunk * npos;
    const unsigned int idw = (chunk == 4) ? 0xff800000u : 0u;  // -inf for the maxima, 0 for the sums
    const u32x4 ident = {idw, idw, idw, idw};
    double a0 = 0.0, a1 = 0.0;
    float m0 = -INFINITY, m1 = -INFINITY, m2 = -INFINITY;
    for (unsigned int j0 = 0; j0 < npos; j0 += kWave * kBatch) {
      u32x4 y[kBatch];
#pragma unroll
      for (int b = 0; b < kBatch; ++b) {
        // Every position below npos holds a workgroup's chunk or the identity (store_block_partials).
        // A lane past the end loads the last position and discards it: a load behind a condition
        // would make the compiler wait for each one before issuing the next.
        const unsigned int pos = j0 + b * kWave + lane;
        y[b] = src[pos < npos ? pos : npos - 1];
      }
      __builtin_amdgcn_sched_barrier(0);  // every load issued before the first value is touched
#pragma unroll
      for (int b = 0; b < kBatch; ++b)
        if (j0 + b * kWave + lane >= npos) y[b] = ident;
      double u[kBatch], w[kBatch];
      auto add_pairwise = [&]() {
#pragma unroll
        for (int width = kBatch / 2; width >= 1; width /= 2) {
#pragma unroll
          for (int b = 0; b < width; ++b) {
            u[b] += u[b + width];
            w[b] += w[b + width];
          }
        }
        a0 += u[0];
        a1 += w[0];
      };
      // one straight-line block per kind of wavefront (the kind is wave-uniform)
      if (chunk < 3) {
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
          u[b] = __longlong_as_double((long long)(((unsigned long long)y[b].y << 32) | y[b].x));
          w[b] = __longlong_as_double((long long)(((unsigned long long)y[b].w << 32) | y[b].z));
        }
        add_pairwise();
      } else if (wave == 3) {  // counters are exact in fp64
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
          u[b] = (double)y[b].x;
          w[b] = (double)y[b].y;
        }
        add_pairwise();
      } else if (wave == 4) {
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
          u[b] = (double)y[b].z;
          w[b] = (double)y[b].w;
        }
        add_pairwise();
      } else {
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
          m0 = fmaxf(m0, __uint_as_float(y[b].x));
          m1 = fmaxf(m1, __uint_as_float(y[b].y));
          m2 = fmaxf(m2, __uint_as_float(y[b].z));
        }
      }
    }
    UNIRL_TRACE_MARK1();
    if (chunk < 4) {
      a0 = wave_sum(a0);
      a1 = wave_sum(a1);
      if (lane == 0) {
        const int slot = chunk < 3 ? 2 * chunk : kFirstCnt + 2 * (wave - 3);
        lds_tot[slot] = a0;
        lds_tot[slot + 1] = a1;
      }
    } else {
      m0 = wave_max(m0);
      m1 = wave_max(m1);
      m2 = wave_max(m2);
      if (lane == 0) {
        lds_tot[kFirstMax] = (double)m0;
        lds_tot[kFirstMax + 1] = (double)m1;
        lds_tot[kFirstMax + 2] = (double)m2;
        lds_tot[6] = lds_tot[7] = lds_tot[15] = 0.0;
      }
    }
  }
  __syncthreads();
  UNIRL_TRACE_MARK2();
  if (t >= kRlVals) return;
  // Lane v turns slot v into its metric; the lanes run the same straight-line code.
  const int v = t;
  const double N = lds_tot[P_CNT], sr = lds_tot[P_SR], sr2 = lds_tot[P_SR2], sab = lds_tot[P_ABS];
  const double x = lds_tot[v];
  // One reciprocal serves every mean.  N is a whole number below 2^32: the hardware's fp32
  // reciprocal refined by two Newton steps in fp64 is within an ulp of fp64's 1/N (the error
  // squares twice from 2^-23), far below the fp32 result's rounding, at a third of the division's
  // instructions.  N = 0 gives inf * 0 = NaN in the step; the estimate (inf) is kept, as 1.0 / 0.
  const double r0 = (double)__builtin_amdgcn_rcpf((float)N);
  const double r1 = fma(fma(-N, r0, 1.0), r0, r0);
  const double r2 = fma(fma(-N, r1, 1.0), r1, r1);
  const double inv_n = (r2 == r2) ? r2 : r0;
  double loss_scale = inv_n;
  if (C.agg_mode != UNIRL_AGG_TOKEN_MEAN) loss_scale = (double)A.inv_seq_scale;
  // sr, sr2: sums of (r-1) and (r-1)^2.  The numerator cancels, so it is formed in fp64; the
  // quotient and the root are fp32 operations on an fp32 result.
  float sd = 0.0f;
  if (N > 1.0) {
    const double num = sr2 - sr * sr * inv_n;
    sd = sqrtf(fmaxf((float)num, 0.0f) / (float)(N - 1.0));
    if (num != num) sd = quiet_nan();  // fmaxf would drop it
  }
  double y = x * inv_n;  // the means: penalty, |new-old|, the three clip fractions
  if (v == P_SR) y = 1.0 + y;
  // GRPO accumulates ld^2; mean(0.5*ld^2) = 0.5*sum/N exactly (halving commutes with rounding)
  if (v == P_KL && C.kind == UNIRL_LOSS_GRPO) y = 0.5 * y;
  if (v == P_LOSS) y = x * loss_scale;
  if (v == P_SR2) y = (double)sd;
  if (v == P_CNT) y = x;
  // min()/max() of the reference return NaN when any ratio is NaN; the ratios are >= 0, so their
  // sum is NaN exactly then (likewise the absolute differences)
  if (v == P_NRMIN) y = (sr != sr) ? (double)quiet_nan() : -x;
  if (v == P_RMAX) y = (sr != sr) ? (double)quiet_nan() : x;
  if (v == P_AMAX) y = (sab != sab) ? (double)quiet_nan() : x;
  if (!slot_used(v)) y = 0.0;
  // metric index of each slot, four bits per slot
  constexpr unsigned long long kMetricOf =
      ((unsigned long long)UNIRL_M_RATIO_MEAN << (4 * P_SR)) | ((unsigned long long)UNIRL_M_RATIO_STD << (4 * P_SR2)) |
      ((unsigned long long)UNIRL_M_LOSS << (4 * P_LOSS)) | ((unsigned long long)UNIRL_M_APPROX_KL << (4 * P_KL)) |
      ((unsigned long long)UNIRL_M_PENALTY_MEAN << (4 * P_PEN)) |
      ((unsigned long long)UNIRL_M_ABSDIFF_MEAN << (4 * P_ABS)) |
      ((unsigned long long)UNIRL_M_NUM_TOKENS << (4 * P_CNT)) | ((unsigned long long)UNIRL_M_CLIPFRAC_HI << (4 * P_CHI)) |
      ((unsigned long long)UNIRL_M_CLIPFRAC_LO << (4 * P_CLO)) |
      ((unsigned long long)UNIRL_M_CLIP_FRACTION << (4 * P_CANY)) | (13ull << (4 * 6)) | (14ull << (4 * 7)) |
      ((unsigned long long)UNIRL_M_RATIO_MIN << (4 * P_NRMIN)) | ((unsigned long long)UNIRL_M_RATIO_MAX << (4 * P_RMAX)) |
      ((unsigned long long)UNIRL_M_ABSDIFF_MAX << (4 * P_AMAX)) | (15ull << (4 * 15));
  A.metrics[(kMetricOf >> (4 * v)) & 15u] = (float)y;
  UNIRL_TRACE_END(A.trace);
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
  // torch.clamp(min > max) returns max everywhere; a collapsed interval gives the kernel's
  // median-of-three the same result
  if (C.clamp_lo > C.clamp_hi) C.clamp_lo = C.clamp_hi;
  C.eps_lo = (float)p->clip_low;
  C.eps_hi = (float)p->clip_high;
  C.drpo_eps = (float)p->drpo_epsilon;
  C.drpo_two_eps = (float)(2.0 * p->drpo_epsilon);
  C.inv_two_eps = (float)(1.0 / (double)C.drpo_two_eps);
  C.inv_eps = (float)(1.0 / (double)C.drpo_eps);
  C.horizon = (float)p->horizon;
  C.fast_ok = (p->kind == UNIRL_LOSS_DRPO && p->mu_weighted && C.drpo_eps >= 1.0f) ? 1 : 0;
  C.fast_hi = 1.0f + C.drpo_eps;  // fp32, as the kernel would form it
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
  // forward: one partial vector per workgroup is read back by a single finalize workgroup, which
  // one compute unit's memory pipeline feeds (about 1 us per 512 vectors); 512 workgroups suit
  // inputs of a few MB, 1024 large ones
  const int64_t cap = bwd ? 16384 : tune_int("UNIRL_RATIO_MAX_BLOCKS", A.n_tok >= (8 << 20) ? 1024 : 512);
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
    if (n_tok > 0 && n_seq < 1) return UNIRL_E_SHAPE;  // cu_seqlens holds n_seq + 1 >= 2 entries
  }
  A.nw = new_logp;
  A.od = old_logp;
  A.adv = advantages;
  A.seq = lengths;
  A.n_seq = n_seq;
  A.seq_stride = seq_stride;
  A.n_tok = n_tok;
  A.inv_seq_scale = (A.C.agg_mode == UNIRL_AGG_SEQ_MEAN_TOKEN_SUM) ? 1.0 / ((double)n_seq * (double)A.C.horizon)
                                                                   : 1.0 / (double)n_seq;
#ifdef UNIRL_TUNE
  A.synth_len = (int)tune_int("UNIRL_RATIO_SYNTH_LEN", 0);
#endif
  return UNIRL_OK;
}

// Forward kernel (+ gradient when A.grad_new is set) and its finalize launch.
static int launch_forward(RatioArgs& A, hipStream_t st) {
  RatioShape S;
  plan(A, false, S);
  if (((size_t)S.grid.x * S.grid.y + kXcds) * kRlChunks * 16 > kWorkspaceBytes) return UNIRL_E_LIMIT;
  dim3 block(kRlThreads);
  const bool packed = (A.layout == LAYOUT_PACKED);
  const bool grad = (A.grad_new != nullptr);
  // 16-byte vectors: mask / per-token-advantage switches compiled in; scalar tokens: read at run time
  const int flags = (A.mask ? 1 : 0) | (A.C.adv_per_token ? 2 : 0);
  // packed layout: every wavefront takes one contiguous run of vectors, an equal share rounded up
  // to whole spans of 64; only the workgroups whose wavefronts have a run are launched, and a run
  // of up to four spans goes out as a single pass of loads
  bool one_pass = false;
  // padded / flat layout: four vectors per lane when one pass of four then covers a whole row
  const int64_t row_vec = ((A.layout == LAYOUT_PADDED ? A.seq_stride : A.n_tok) + 3) / 4;
  const bool four_items = !packed && S.vec == 4 && row_vec > (int64_t)S.grid.x * kRlThreads * 2 &&
                          row_vec <= (int64_t)S.grid.x * kRlThreads * 4 && tune_int("UNIRL_RATIO_ITEMS4", 1) == 1;
  if (packed && S.vec == 4) {
    const int64_t waves_per_wg = kRlThreads / kWave;
    const int64_t n_waves = (int64_t)S.grid.x * waves_per_wg;
    const int64_t nvec = A.n_tok / 4;
    A.per_wave = ((nvec + n_waves - 1) / n_waves + kWave - 1) / kWave * kWave;
    if (A.per_wave < kWave) A.per_wave = kWave;
    const int64_t active = (nvec + A.per_wave - 1) / A.per_wave;
    int64_t nwg = (active + waves_per_wg - 1) / waves_per_wg;
    if (nwg < 1) nwg = 1;
    S.grid.x = (unsigned int)nwg;
    one_pass = A.per_wave / kWave <= 4;
  }
#define UNIRL_LAUNCH_FWD5(KIND, VEC, PACKED, FLAGS, ITEMS)                                                     \
  do {                                                                                                         \
    if (grad)                                                                                                  \
      hipLaunchKernelGGL((ratio_loss_fwd_kernel<KIND, VEC, PACKED, FLAGS, true, ITEMS>), S.grid, block, 0, st, A);  \
    else                                                                                                       \
      hipLaunchKernelGGL((ratio_loss_fwd_kernel<KIND, VEC, PACKED, FLAGS, false, ITEMS>), S.grid, block, 0, st, A); \
  } while (0)
#define UNIRL_LAUNCH_FWD4(KIND, VEC, PACKED, FLAGS)                                                            \
  do {                                                                                                         \
    if (VEC == 4 && !PACKED && four_items) UNIRL_LAUNCH_FWD5(KIND, VEC, PACKED, FLAGS, 4);                     \
    else UNIRL_LAUNCH_FWD5(KIND, VEC, PACKED, FLAGS, 2);                                                       \
  } while (0)
#define UNIRL_LAUNCH_PACKED2(KIND, FLAGS, ITEMS)                                                               \
  do {                                                                                                         \
    if (grad)                                                                                                  \
      hipLaunchKernelGGL((ratio_loss_packed_kernel<KIND, FLAGS, true, ITEMS>), S.grid, block, 0, st, A);       \
    else                                                                                                       \
      hipLaunchKernelGGL((ratio_loss_packed_kernel<KIND, FLAGS, false, ITEMS>), S.grid, block, 0, st, A);      \
  } while (0)
#define UNIRL_LAUNCH_PACKED(KIND, FLAGS)                                                                       \
  do {                                                                                                         \
    if (one_pass) UNIRL_LAUNCH_PACKED2(KIND, FLAGS, 4); else UNIRL_LAUNCH_PACKED2(KIND, FLAGS, 2);             \
  } while (0)
#define UNIRL_LAUNCH_FWD3(KIND, VEC, FLAGS)                                                                    \
  do {                                                                                                         \
    if (packed) UNIRL_LAUNCH_FWD4(KIND, VEC, true, FLAGS); else UNIRL_LAUNCH_FWD4(KIND, VEC, false, FLAGS);    \
  } while (0)
#define UNIRL_LAUNCH_FWD(KIND)                                                                                 \
  do {                                                                                                         \
    if (S.vec != 4) UNIRL_LAUNCH_FWD3(KIND, 1, -1);                                                            \
    else if (packed && flags == 0) UNIRL_LAUNCH_PACKED(KIND, 0);                                               \
    else if (packed && flags == 1) UNIRL_LAUNCH_PACKED(KIND, 1);                                               \
    else if (packed && flags == 2) UNIRL_LAUNCH_PACKED(KIND, 2);                                               \
    else if (packed) UNIRL_LAUNCH_PACKED(KIND, 3);                                                             \
    else if (flags == 0) UNIRL_LAUNCH_FWD4(KIND, 4, false, 0);                                                 \
    else if (flags == 1) UNIRL_LAUNCH_FWD4(KIND, 4, false, 1);                                                 \
    else if (flags == 2) UNIRL_LAUNCH_FWD4(KIND, 4, false, 2);                                                 \
    else UNIRL_LAUNCH_FWD4(KIND, 4, false, 3);                                                                 \
  } while (0)
  UNIRL_TRACE_SET(A, packed ? "ratio_packed" : "ratio_fwd", S.grid.x * S.grid.y);
  if (A.C.kind == UNIRL_LOSS_GRPO) UNIRL_LAUNCH_FWD(UNIRL_LOSS_GRPO); else UNIRL_LAUNCH_FWD(UNIRL_LOSS_DRPO);
#undef UNIRL_LAUNCH_FWD5
#undef UNIRL_LAUNCH_FWD4
#undef UNIRL_LAUNCH_PACKED
#undef UNIRL_LAUNCH_PACKED2
#undef UNIRL_LAUNCH_FWD3
#undef UNIRL_LAUNCH_FWD
  const int launch_rc = (int)hipGetLastError();
  if (launch_rc != 0 || !A.metrics) return launch_rc;
  const unsigned int nblk = S.grid.x * S.grid.y;
  UNIRL_TRACE_SET(A, "ratio_finalize", 1);
  const unsigned int npos = partial_per_xcd(nblk) * kXcds;
  if (npos <= 4 * kWave)
    hipLaunchKernelGGL(ratio_loss_finalize_kernel<4>, dim3(1), dim3(kFinThreads), 0, st, A, nblk);
  else if (npos <= 8 * kWave)
    hipLaunchKernelGGL(ratio_loss_finalize_kernel<8>, dim3(1), dim3(kFinThreads), 0, st, A, nblk);
  else
    hipLaunchKernelGGL(ratio_loss_finalize_kernel<16>, dim3(1), dim3(kFinThreads), 0, st, A, nblk);
  return (int)hipGetLastError();
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
  if (!aligned_to(workspace, 16)) return UNIRL_E_ALIGN;
  A.mask = loss_mask;
  A.loss_elem = loss_per_elem;
  A.metrics = metrics;
  A.partials = reinterpret_cast<char*>(workspace);
  return launch_forward(A, (hipStream_t)stream);
}

extern "C" int unirl_ratio_loss_fwd_bwd(const float* new_logp, const float* old_logp, const float* advantages,
                                        const int64_t* lengths, const float* loss_mask, int64_t n_seq,
                                        int64_t seq_stride, int64_t n_tok, const unirl_ratio_loss_params* params,
                                        float loss_scale, int64_t n_valid, float* grad_new, float* metrics,
                                        void* workspace, size_t workspace_bytes, void* stream) {
  RatioArgs A = {};
  const int rc = check_common(new_logp, old_logp, advantages, lengths, n_seq, seq_stride, n_tok, params, A);
  if (rc != 0) return rc;
  if (!metrics || !grad_new) return UNIRL_E_NULL;
  if (!aligned_to(grad_new, 4)) return UNIRL_E_ALIGN;
  if (!workspace || workspace_bytes < kWorkspaceBytes) return UNIRL_E_WORKSPACE;
  if (!aligned_to(workspace, 16)) return UNIRL_E_ALIGN;
  A.mask = loss_mask;
  A.metrics = metrics;
  A.partials = reinterpret_cast<char*>(workspace);
  A.grad_new = grad_new;
  A.loss_scale = loss_scale;
  // the token-mean denominator counts every valid token (masked ones too): all tokens outside
  // the padded layout; in the padded layout the caller's count, or the kernel sums the lengths
  A.n_valid_host = (A.layout == LAYOUT_PADDED) ? n_valid : n_tok;
  return launch_forward(A, (hipStream_t)stream);
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
  // packed layout, gradient of the aggregated loss: the packed forward kernel with its gradient
  // output and nothing else stored -- it follows the sequences span by span, where the kernel
  // below looks each token's sequence up (37 -> 25 us on 8.8 M tokens)
  if (A.layout == LAYOUT_PACKED && S.vec == 4 && aggregate && !g_elem) {
    A.loss_scale = 1.0f;  // stands in for a NULL g_scale
    A.partials = nullptr;
    A.metrics = nullptr;
    return launch_forward(A, st);
  }
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
