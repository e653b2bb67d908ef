// Token log-prob + entropy over the vocabulary: one streaming pass per row.
//
// Replaces, per row of logits x (with lf = x.float()/T):
//   logp = lf[id] - logsumexp(lf)     unirl/models/qwen3/ar.py:82-85 (also
//                                      qwen3/ar.py:144-174, qwen_vl/ar.py:334-335,
//                                      hunyuan_image3/ar.py:509-510)
//   H    = logsumexp(lf) - sum softmax(lf)*lf      (no counterpart in the
//          reference; equals torch.distributions.Categorical(logits=lf).entropy(),
//          which clamps -inf logits to the lowest finite value)
//
// One workgroup owns one row and streams it with non-temporal 16-byte loads.
// Each lane keeps online sums relative to a reference r = fl(m*c) shared by its
// wavefront, m the largest logit the wavefront has seen and c = log2(e)/T:
//     a_i = fma(x_i, c, -r)        one FMA; exact single rounding
//     e_i = 2^a_i                  one v_exp_f32
//     s  += e_i ,  t += e_i * a_i  (t <= ~0: every term has the same sign)
// m is wave-uniform: per chunk of UNROLL vectors every lane compares its own
// maximum with m and the wavefront branches on the compare's lane mask, so
// raising the reference (a DPP max-reduction, then the rescale) is a uniform,
// rarely taken branch (about ln(#chunks) times per row; per-lane references
// would make some lane take it in almost every chunk) and the common path pays
// one compare per chunk for it; inside that branch the elements equal to the new maximum are
// counted apart (cnt) so that sum = cnt*2^r0 + s keeps full relative accuracy
// when one logit dominates (sum = 1 + tiny), r0 = fma(m, c, -r) being the exact
// residual of the rounded reference.  With sum and t:
//     logsumexp = ln2*(r + log2 sum),  H = ln sum - ln2 * t/sum,
//     logp = ln2*a_id - ln sum.
// Lanes of a wavefront share the reference, so their sums just add; wavefronts
// merge through LDS; the last few operations run in fp64 on one lane.
//
// The fast path spends no instruction on -inf / NaN logits; a row whose sums
// come out non-finite is simply done again with clamping (SAFE = true).
//
// HBM traffic: V*sizeof(T) bytes read per row + 8 bytes of id + 4..12 bytes out.

#include <float.h>

#include "common_hip.h"
#include "unirl_internal.h"

namespace unirl {

constexpr int kTokThreads = 256;
constexpr float kLog2e = 1.4426950408889634f;
constexpr double kLn2 = 0.6931471805599453;

// Reference shared by the 64 lanes of a wavefront (wave-uniform, lives in scalar registers).
struct TokRef {
  float m;  // largest logit the wavefront has seen (-inf: none yet)
  float r;  // fl(m * c)
};
// Per-lane sums relative to the wavefront's reference.
struct TokAcc {
  float cnt;  // elements equal to m, counted when m was last raised
  float s;    // sum of 2^(x*c - r) over all other elements
  float t;    // sum of 2^a * a over them, a = x*c - r
};
// A whole state (one lane's, one wavefront's or one row's).
struct TokState {
  float m, r, cnt, s, t;
};

__device__ __forceinline__ float tok_exp2(float a) { return __builtin_amdgcn_exp2f(a); }

// Re-express sums relative to a higher maximum M.  (m, r) -> (M, fl(M*c)).
__device__ __forceinline__ void tok_raise(float& m, float& r, TokAcc& acc, float M, float c) {
  if (m == M) return;
  const float R = M * c;
  if (m != -INFINITY) {
    // the former maxima become ordinary terms: each is 2^r0 with a = r0
    const float r0 = fmaf(m, c, -r);
    const float e0 = acc.cnt * tok_exp2(r0);
    const float s_all = acc.s + e0;
    const float t_all = fmaf(e0, r0, acc.t);
    const float delta = r - R;  // < 0: every a shifts by delta, every e scales by 2^delta
    const float f = tok_exp2(delta);
    acc.s = f * s_all;
    acc.t = f * fmaf(delta, s_all, t_all);
  }  // else nothing has been summed yet: s and t are 0, or s carries the NaN mark of tok_update
  acc.cnt = 0.0f;
  m = M;
  r = R;
}

// One chunk of N elements per lane.  `active` is false for lanes past the end of the row.
template <int N, bool SAFE>
__device__ __forceinline__ void tok_update(TokRef& ref, TokAcc& acc, const float (&x)[N], bool active, float c) {
  float cm = x[0];
#pragma unroll
  for (int k = 1; k < N; ++k) cm = fmaxf(cm, x[k]);
  // "does any lane hold a new maximum" is one compare (its lane mask is tested on the scalar
  // unit); the DPP max-reduction runs only when it does
  if (__builtin_expect(__builtin_amdgcn_ballot_w64(active && cm > ref.m) != 0, 0)) {
    // Wave-uniform and rare (about ln(chunks) times per row): move to the new maximum, then
    // split this chunk's exact maxima from the rest.
    const float wm = wave_max(active ? cm : -INFINITY);
    tok_raise(ref.m, ref.r, acc, wm, c);
    if (active) {
#pragma unroll
      for (int k = 0; k < N; ++k) {
        if (x[k] == ref.m) {
          acc.cnt += 1.0f;
        } else {
          float a = fmaf(x[k], c, -ref.r);
          if (SAFE) a = (a < -FLT_MAX) ? -FLT_MAX : a;
          const float e = tok_exp2(a);
          acc.s += e;
          acc.t = fmaf(e, a, acc.t);
        }
      }
    }
  } else if (ref.m != -INFINITY) {
    if (SAFE && ref.m == INFINITY) {
      // a +inf logit has been met: every other term is 0 against it, a further +inf is one more
      // maximum (inf - inf above would make it a NaN), and only a NaN still matters
      if (active) {
#pragma unroll
        for (int k = 0; k < N; ++k) {
          if (x[k] == INFINITY) acc.cnt += 1.0f;
          else if (x[k] != x[k]) acc.s = x[k];
        }
      }
    } else if (active) {
#pragma unroll
      for (int k = 0; k < N; ++k) {
        float a = fmaf(x[k], c, -ref.r);
        if (SAFE) a = (a < -FLT_MAX) ? -FLT_MAX : a;  // -inf logit: e = 0 and e*a = 0; NaN stays NaN
        const float e = tok_exp2(a);
        acc.s += e;
        acc.t = fmaf(e, a, acc.t);
      }
    }
  } else if (active) {
    // The wavefront has met nothing but -inf and NaN so far, and so nothing is summed: a NaN has
    // to be remembered by hand (the maximum above dropped it).  Rare: the start of a masked row.
#pragma unroll
    for (int k = 0; k < N; ++k)
      if (x[k] != x[k]) acc.s = x[k];
  }
}

__device__ __forceinline__ void tok_merge(TokState& a, TokState b, float c) {
  const float M = fmaxf(a.m, b.m);
  TokAcc aa{a.cnt, a.s, a.t}, bb{b.cnt, b.s, b.t};
  tok_raise(a.m, a.r, aa, M, c);
  tok_raise(b.m, b.r, bb, M, c);
  a.cnt = aa.cnt + bb.cnt;
  a.s = aa.s + bb.s;
  a.t = aa.t + bb.t;
}

// 16 bytes of logits -> floats

template <typename T>
struct Stream16;
template <>
struct Stream16<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void unpack(u32x4 v, float* o) {
    o[0] = __uint_as_float(v.x);
    o[1] = __uint_as_float(v.y);
    o[2] = __uint_as_float(v.z);
    o[3] = __uint_as_float(v.w);
  }
};
template <>
struct Stream16<bf16_t> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void unpack(u32x4 v, float* o) {
    o[0] = __uint_as_float(v.x << 16);
    o[1] = __uint_as_float(v.x & 0xffff0000u);
    o[2] = __uint_as_float(v.y << 16);
    o[3] = __uint_as_float(v.y & 0xffff0000u);
    o[4] = __uint_as_float(v.z << 16);
    o[5] = __uint_as_float(v.z & 0xffff0000u);
    o[6] = __uint_as_float(v.w << 16);
    o[7] = __uint_as_float(v.w & 0xffff0000u);
  }
};
template <>
struct Stream16<f16_t> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void unpack(u32x4 v, float* o) {
    o[0] = f16_bits_to_f32(v.x & 0xffffu);
    o[1] = f16_bits_to_f32(v.x >> 16);
    o[2] = f16_bits_to_f32(v.y & 0xffffu);
    o[3] = f16_bits_to_f32(v.y >> 16);
    o[4] = f16_bits_to_f32(v.z & 0xffffu);
    o[5] = f16_bits_to_f32(v.z >> 16);
    o[6] = f16_bits_to_f32(v.w & 0xffffu);
    o[7] = f16_bits_to_f32(v.w >> 16);
  }
};

// Inverse of Stream16<T>::unpack: N floats -> one 16-byte vector of T (round to nearest even).
template <typename T>
struct Pack16;
template <>
struct Pack16<float> {
  static __device__ __forceinline__ u32x4 pack(const float* o) {
    u32x4 v;
    v.x = __float_as_uint(o[0]);
    v.y = __float_as_uint(o[1]);
    v.z = __float_as_uint(o[2]);
    v.w = __float_as_uint(o[3]);
    return v;
  }
};
template <>
struct Pack16<bf16_t> {
  static __device__ __forceinline__ u32x4 pack(const float* o) {
    u32x4 v;
    v.x = f32x2_to_bf16x2_bits(o[0], o[1]);
    v.y = f32x2_to_bf16x2_bits(o[2], o[3]);
    v.z = f32x2_to_bf16x2_bits(o[4], o[5]);
    v.w = f32x2_to_bf16x2_bits(o[6], o[7]);
    return v;
  }
};
template <>
struct Pack16<f16_t> {
  static __device__ __forceinline__ u32x4 pack(const float* o) {
    u32x4 v;
    v.x = f32_to_f16_bits(o[0]) | (f32_to_f16_bits(o[1]) << 16);
    v.y = f32_to_f16_bits(o[2]) | (f32_to_f16_bits(o[3]) << 16);
    v.z = f32_to_f16_bits(o[4]) | (f32_to_f16_bits(o[5]) << 16);
    v.w = f32_to_f16_bits(o[6]) | (f32_to_f16_bits(o[7]) << 16);
    return v;
  }
};

struct TokArgs {
  const void* logits;
  const int64_t* ids;
  int64_t rows, V, row_stride;
  float c;      // log2(e)/T
  float inv_t;  // 1/T
  float* logp;
  float* ent;
  float* lse;
};

// One pass over the row; returns the workgroup's merged state in thread 0.
template <typename T, int UNROLL, int TPB, bool SAFE>
__device__ __forceinline__ TokState tok_scan_row(const T* __restrict__ p, int64_t V, float c, float (*lds)[5]) {
  constexpr int VEC = Stream16<T>::N;
  constexpr int NW = TPB / kWave;
  constexpr int CHUNK = UNROLL * VEC;

  // peel to a 16-byte boundary
  int64_t head = (int64_t)(((16u - (unsigned)(reinterpret_cast<uintptr_t>(p) & 15u)) & 15u) / sizeof(T));
  if (head > V) head = V;
  const int64_t nvec = (V - head) / VEC;
  const int64_t tail0 = head + nvec * VEC;

  TokRef ref{-INFINITY, -INFINITY};
  TokAcc acc{0.0f, 0.0f, 0.0f};
  if (head > 0) {  // workgroup-uniform
    const bool on = (int64_t)threadIdx.x < head;
    const float x[1] = {on ? Elem<T>::load(p + threadIdx.x) : 0.0f};
    tok_update<1, SAFE>(ref, acc, x, on, c);
  }
  if (tail0 < V) {
    const bool on = tail0 + (int64_t)threadIdx.x < V;
    const float x[1] = {on ? Elem<T>::load(p + tail0 + threadIdx.x) : 0.0f};
    tok_update<1, SAFE>(ref, acc, x, on, c);
  }

  const T* __restrict__ pv = p + head;
  const int64_t per_iter = (int64_t)TPB * UNROLL;
  const int64_t n_full = nvec / per_iter;
  // Unguarded body: UNROLL vectors per lane, the lanes of a wavefront on consecutive 16-byte
  // words.  The next chunk's loads are issued before the current chunk is consumed.
  if (n_full > 0) {
    const T* __restrict__ q = pv + (int64_t)threadIdx.x * VEC;
    u32x4 cur[UNROLL], nxt[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) cur[u] = stream_load16(q + (int64_t)u * TPB * VEC);
    for (int64_t it = 1; it < n_full; ++it) {  // every pass but the last prefetches unconditionally
      q += per_iter * VEC;
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) nxt[u] = stream_load16(q + (int64_t)u * TPB * VEC);
      float x[CHUNK];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) Stream16<T>::unpack(cur[u], x + u * VEC);
      tok_update<CHUNK, SAFE>(ref, acc, x, true, c);
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) cur[u] = nxt[u];
    }
    float x[CHUNK];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) Stream16<T>::unpack(cur[u], x + u * VEC);
    tok_update<CHUNK, SAFE>(ref, acc, x, true, c);
  }
  // remainder: fewer than UNROLL vectors per lane; trip count is workgroup-uniform
  for (int64_t i0 = n_full * per_iter; i0 < nvec; i0 += TPB) {
    const int64_t i = i0 + threadIdx.x;
    const bool on = i < nvec;
    float x[VEC];
    if (on) {
      Stream16<T>::unpack(stream_load16(pv + i * VEC), x);
    } else {
#pragma unroll
      for (int k = 0; k < VEC; ++k) x[k] = 0.0f;
    }
    tok_update<VEC, SAFE>(ref, acc, x, on, c);
  }

  // lanes -> wavefront: the lanes share (m, r), so the sums simply add
  TokState st{ref.m, ref.r, wave_sum(acc.cnt), wave_sum(acc.s), wave_sum(acc.t)};
  const int lane = threadIdx.x & (kWave - 1);
  const int wid = threadIdx.x / kWave;
  __syncthreads();  // lds may still be read from a previous scan of this row
  if (lane == 0) {
    lds[wid][0] = st.m;
    lds[wid][1] = st.r;
    lds[wid][2] = st.cnt;
    lds[wid][3] = st.s;
    lds[wid][4] = st.t;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
#pragma unroll
    for (int w = 1; w < NW; ++w) tok_merge(st, TokState{lds[w][0], lds[w][1], lds[w][2], lds[w][3], lds[w][4]}, c);
  }
  return st;
}

template <typename T, int UNROLL, int TPB>
__global__ __launch_bounds__(TPB) void token_logp_entropy_kernel(TokArgs A) {
  __shared__ float lds[TPB / kWave][5];
  __shared__ int redo;

  const int64_t row = blockIdx.x;
  const T* __restrict__ p = reinterpret_cast<const T*>(A.logits) + row * A.row_stride;
  const int64_t V = A.V;
  const float c = A.c;

  // The target id and its logit are fetched before the scan (two dependent trips to memory that
  // would otherwise sit in the row's tail, after the last vector has been consumed).
  int64_t id = -1;
  float x_id = 0.0f;
  if (threadIdx.x == 0 && A.logp) {
    id = A.ids[row];
    if (id >= 0 && id < V) x_id = Elem<T>::load(p + id);
  }

  TokState st = tok_scan_row<T, UNROLL, TPB, false>(p, V, c, lds);
  if (threadIdx.x == 0) redo = !(fabsf(st.s) <= FLT_MAX) || !(fabsf(st.t) <= FLT_MAX);  // inf or NaN
  __syncthreads();
  if (redo) st = tok_scan_row<T, 1, TPB, true>(p, V, c, lds);  // -inf (or NaN) logits in this row
  if (threadIdx.x != 0) return;

  if (st.m == INFINITY) {
    // a +inf logit: logsumexp is +inf, so a finite logit has log-prob -inf and the +inf logit
    // itself inf - inf = NaN; softmax is 0/NaN, so the entropy is NaN.  A NaN anywhere in the row
    // (st.s is NaN then) makes everything NaN.
    const bool has_nan = st.s != st.s;
    if (A.lse) A.lse[row] = has_nan ? quiet_nan() : INFINITY;
    if (A.ent) A.ent[row] = quiet_nan();
    if (A.logp) {
      float out = quiet_nan();
      if (!has_nan && id >= 0 && id < V && x_id < INFINITY) out = -INFINITY;  // x_id: false for +inf and NaN
      A.logp[row] = out;
    }
    return;
  }
  if (st.m == -INFINITY) {
    // every logit is -inf: logsumexp is -inf (torch.logsumexp), the log-prob -inf - (-inf) = NaN
    // and the softmax 0/0, so the entropy is NaN too
    if (A.lse) A.lse[row] = -INFINITY;
    if (A.ent) A.ent[row] = quiet_nan();
    if (A.logp) A.logp[row] = quiet_nan();
    return;
  }
  // sum = cnt*2^r0 + s relative to the reference r;  ln sum = r0 ln2 + ln cnt + log1p(s 2^-r0 / cnt)
  const double r0 = (double)fmaf(st.m, c, -st.r);
  const double cnt = (double)st.cnt;
  const double e0 = cnt * exp2(r0);
  const double sum = e0 + (double)st.s;
  const double ln_sum = r0 * kLn2 + log(cnt) + log1p((double)st.s * exp2(-r0) / cnt);
  const double t_all = (double)st.t + e0 * r0;
  if (A.lse) A.lse[row] = (float)(kLn2 * (double)st.r + ln_sum);
  if (A.ent) {
    const double h = ln_sum - kLn2 * t_all / sum;
    A.ent[row] = (float)(h < 0.0 ? 0.0 : h);  // rounding may leave -1e-21 when one logit holds all the mass; NaN stays
  }
  if (A.logp) {
    float out = __uint_as_float(0x7fc00000u);
    if (id >= 0 && id < V) {
      const double a_id = (double)x_id * (double)c - (double)st.r;
      out = (float)(kLn2 * a_id - ln_sum);
    }
    A.logp[row] = out;
  }
}

// grad[r, j] = g[r]/T * (1[j == id] - softmax(lf)[r, j]), written in the logits dtype.
struct TokBwdArgs {
  const void* logits;
  const int64_t* ids;
  int64_t rows, V, row_stride, grad_row_stride;
  float c;
  float inv_t;
  const float* lse;
  const float* g;
  void* grad;
};

__device__ __forceinline__ float tok_bwd_elem(float x, float c, float lse2, float gs, float one) {
  return gs * (one - tok_exp2(fmaf(x, c, -lse2)));
}

// One workgroup per row.  The row is read and its gradient written once, as 16-byte streaming
// vectors when the logits row and the gradient row share their offset from a 16-byte boundary
// (always, for contiguous tensors whose V*sizeof(T) is a multiple of 16), else element-wise.
template <typename T, int UNROLL>
__global__ __launch_bounds__(kTokThreads) void token_logp_bwd_kernel(TokBwdArgs A) {
  constexpr int VEC = Stream16<T>::N;
  const int64_t row = blockIdx.x;
  // No __restrict__ on the logits and the gradient: the caller may pass one buffer for both (the
  // gradient then overwrites the logits it was computed from, element for element).
  const T* p = reinterpret_cast<const T*>(A.logits) + row * A.row_stride;
  T* gp = reinterpret_cast<T*>(A.grad) + row * A.grad_row_stride;
  const float c = A.c;
  const int64_t id = A.ids[row];
  const int64_t V = A.V;
  const int tid = threadIdx.x;
  // A target outside [0, V) has no log-prob (the forward returns NaN for it): its row gets a zero
  // gradient rather than -g*softmax.  lse = +inf makes every softmax term exactly 0.
  const bool id_ok = id >= 0 && id < V;
  const float lse2 = id_ok ? A.lse[row] * kLog2e : INFINITY;
  const float gs = id_ok ? A.g[row] * A.inv_t : 0.0f;

  const unsigned mis_p = (unsigned)(reinterpret_cast<uintptr_t>(p) & 15u);
  const unsigned mis_g = (unsigned)(reinterpret_cast<uintptr_t>(gp) & 15u);
  if (mis_p != mis_g) {  // row-uniform
    for (int64_t j = tid; j < V; j += kTokThreads)
      Elem<T>::store(gp + j, tok_bwd_elem(Elem<T>::load(p + j), c, lse2, gs, (j == id) ? 1.0f : 0.0f));
    return;
  }
  int64_t head = (int64_t)(((16u - mis_p) & 15u) / sizeof(T));
  if (head > V) head = V;
  const int64_t nvec = (V - head) / VEC;
  const int64_t tail0 = head + nvec * VEC;
  if (tid < head) Elem<T>::store(gp + tid, tok_bwd_elem(Elem<T>::load(p + tid), c, lse2, gs, (tid == id) ? 1.0f : 0.0f));
  if (tail0 + tid < V) {
    const int64_t j = tail0 + tid;
    Elem<T>::store(gp + j, tok_bwd_elem(Elem<T>::load(p + j), c, lse2, gs, (j == id) ? 1.0f : 0.0f));
  }

  const T* pv = p + head;
  T* gv = gp + head;
  const int64_t idv = id - head;  // position of the gathered column in the vector region
  const int64_t per_iter = (int64_t)kTokThreads * UNROLL;
  const int64_t n_full = nvec / per_iter;
  for (int64_t it = 0; it < n_full; ++it) {
    const int64_t v0 = it * per_iter + tid;
    u32x4 raw[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) raw[u] = stream_load16(pv + (v0 + (int64_t)u * kTokThreads) * VEC);
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int64_t e0 = (v0 + (int64_t)u * kTokThreads) * VEC;
      float x[VEC];
      Stream16<T>::unpack(raw[u], x);
#pragma unroll
      for (int k = 0; k < VEC; ++k) x[k] = tok_bwd_elem(x[k], c, lse2, gs, 0.0f);
      if ((uint64_t)(idv - e0) < (uint64_t)VEC) {  // this vector holds the gathered column
        float y[VEC];
        Stream16<T>::unpack(raw[u], y);
#pragma unroll
        for (int k = 0; k < VEC; ++k)
          if (idv - e0 == k) x[k] = tok_bwd_elem(y[k], c, lse2, gs, 1.0f);
      }
      stream_store16(gv + e0, Pack16<T>::pack(x));
    }
  }
  for (int64_t v = n_full * per_iter + tid; v < nvec; v += kTokThreads) {
    const int64_t e0 = v * VEC;
    const u32x4 raw = stream_load16(pv + e0);
    float x[VEC], y[VEC];
    Stream16<T>::unpack(raw, y);
#pragma unroll
    for (int k = 0; k < VEC; ++k) x[k] = tok_bwd_elem(y[k], c, lse2, gs, (idv - e0 == k) ? 1.0f : 0.0f);
    stream_store16(gv + e0, Pack16<T>::pack(x));
  }
}

template <typename T, int TPB>
static int launch_tok_tpb(const TokArgs& A, hipStream_t st, int unroll) {
  dim3 grid((unsigned int)A.rows), block(TPB);
  if (unroll >= 8)
    hipLaunchKernelGGL((token_logp_entropy_kernel<T, 8, TPB>), grid, block, 0, st, A);
  else if (unroll >= 4)
    hipLaunchKernelGGL((token_logp_entropy_kernel<T, 4, TPB>), grid, block, 0, st, A);
  else if (unroll >= 2)
    hipLaunchKernelGGL((token_logp_entropy_kernel<T, 2, TPB>), grid, block, 0, st, A);
  else
    hipLaunchKernelGGL((token_logp_entropy_kernel<T, 1, TPB>), grid, block, 0, st, A);
  return (int)hipGetLastError();
}

template <typename T>
static int launch_tok(const TokArgs& A, hipStream_t st) {
  const int unroll = (int)tune_int("UNIRL_TOK_UNROLL", 4);
  const int tpb = (int)tune_int("UNIRL_TOK_THREADS", 256);
  if (tpb >= 1024) return launch_tok_tpb<T, 1024>(A, st, unroll);
  if (tpb >= 512) return launch_tok_tpb<T, 512>(A, st, unroll);
  return launch_tok_tpb<T, 256>(A, st, unroll);
}

}  // namespace unirl

using namespace unirl;

extern "C" int unirl_token_logp_entropy(const void* logits, int dtype, int64_t rows, int64_t V, int64_t row_stride,
                                        const int64_t* ids, float temperature, float* logp_out, float* ent_out,
                                        float* lse_out, void* stream) {
  if (!dtype_ok(dtype)) return UNIRL_E_DTYPE;
  if (rows < 0 || V <= 0 || row_stride < V) return UNIRL_E_SHAPE;
  if (rows == 0) return UNIRL_OK;
  if (!logits || (logp_out && !ids)) return UNIRL_E_NULL;
  if (!aligned_to(logits, dtype_size(dtype)) || !aligned_to(ids, 8)) return UNIRL_E_ALIGN;
  if (rows > 0x7fffffffLL) return UNIRL_E_LIMIT;
  const float T = (temperature > 0.0f) ? temperature : 1.0f;
  TokArgs A;
  A.logits = logits;
  A.ids = ids;
  A.rows = rows;
  A.V = V;
  A.row_stride = row_stride;
  A.c = (float)(1.4426950408889634 / (double)T);
  A.inv_t = (float)(1.0 / (double)T);
  A.logp = logp_out;
  A.ent = ent_out;
  A.lse = lse_out;
  hipStream_t st = (hipStream_t)stream;
  switch (dtype) {
    case UNIRL_F32: return launch_tok<float>(A, st);
    case UNIRL_BF16: return launch_tok<bf16_t>(A, st);
    case UNIRL_F16: return launch_tok<f16_t>(A, st);
  }
  return UNIRL_E_DTYPE;
}

extern "C" int unirl_token_logp_bwd(const void* logits, int dtype, int64_t rows, int64_t V, int64_t row_stride,
                                    const int64_t* ids, float temperature, const float* lse, const float* g_logp,
                                    void* grad_logits, int64_t grad_row_stride, void* stream) {
  if (!dtype_ok(dtype)) return UNIRL_E_DTYPE;
  if (rows < 0 || V <= 0 || row_stride < V || grad_row_stride < V) return UNIRL_E_SHAPE;
  if (rows == 0) return UNIRL_OK;
  if (!logits || !ids || !lse || !g_logp || !grad_logits) return UNIRL_E_NULL;
  if (!aligned_to(logits, dtype_size(dtype)) || !aligned_to(grad_logits, dtype_size(dtype)) || !aligned_to(ids, 8))
    return UNIRL_E_ALIGN;
  const float T = (temperature > 0.0f) ? temperature : 1.0f;
  hipStream_t st = (hipStream_t)stream;
  const int64_t per_launch = 32768;
  for (int64_t r0 = 0; r0 < rows; r0 += per_launch) {
    const int64_t nr = (rows - r0 < per_launch) ? (rows - r0) : per_launch;
    TokBwdArgs A;
    A.logits = offset_ptr(logits, r0 * row_stride, dtype_size(dtype));
    A.ids = ids + r0;
    A.rows = nr;
    A.V = V;
    A.row_stride = row_stride;
    A.grad_row_stride = grad_row_stride;
    A.c = (float)(1.4426950408889634 / (double)T);
    A.inv_t = (float)(1.0 / (double)T);
    A.lse = lse + r0;
    A.g = g_logp + r0;
    A.grad = const_cast<void*>(offset_ptr(grad_logits, r0 * grad_row_stride, dtype_size(dtype)));
    dim3 grid((unsigned int)nr), block(kTokThreads);
    switch (dtype) {
      case UNIRL_F32: hipLaunchKernelGGL((token_logp_bwd_kernel<float, 4>), grid, block, 0, st, A); break;
      case UNIRL_BF16: hipLaunchKernelGGL((token_logp_bwd_kernel<bf16_t, 4>), grid, block, 0, st, A); break;
      case UNIRL_F16: hipLaunchKernelGGL((token_logp_bwd_kernel<f16_t, 4>), grid, block, 0, st, A); break;
    }
    const int rc = (int)hipGetLastError();
    if (rc != 0) return rc;
  }
  return UNIRL_OK;
}
