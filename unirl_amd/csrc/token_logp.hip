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
// One workgroup owns one row.  Every lane keeps an online (max, sum e, sum e*x)
// triple over 16-byte vectors, rescaling only when a vector raises the running
// maximum; lanes merge by wavefront shuffles, wavefronts through LDS.  The
// exponent is evaluated in base 2 with the temperature folded into one
// constant: e = 2^(-(m - x)*c), c = log2(e)/T, and the entropy sum is kept as
// sum e*(m - x) >= 0, so a row dominated by one logit loses no digits.
//
// HBM traffic: V*sizeof(T) bytes read per row + 8 bytes of id + 4..12 bytes out.

#include <float.h>

#include "common.cuh"
#include "unirl_internal.h"

namespace unirl {

constexpr int kTokThreads = 256;
constexpr float kLog2e = 1.4426950408889634f;

struct TokState {
  float m;    // running maximum of the raw logits seen by this lane
  float cnt;  // how many elements equalled m when m was last raised (their e is exactly 1)
  float s;    // sum of e over every other element, e = 2^(-(m - x) * c) = exp((x - m)/T)
  float t;    // sum e*(m - x) (every term >= 0: no cancellation for peaked rows)
};
// sum exp((x-m)/T) = cnt + s.  Keeping the exact ones apart from the small terms keeps
// ln(sum) accurate when one logit dominates (sum = 1 + tiny).

// Move a state to a higher maximum M: every e scales by f = 2^(-(M-m)c), (m - x)
// grows by (M - m), and the former maxima join the ordinary terms.
__device__ __forceinline__ void tok_raise(TokState& a, float M, float c) {
  if (a.m == M) return;
  if (a.m == -INFINITY) {  // nothing accumulated yet
    a.s = 0.0f;
    a.t = 0.0f;
  } else {
    const float dm = M - a.m;
    const float f = __builtin_amdgcn_exp2f(-(dm * c));
    const float all = a.s + a.cnt;
    a.t = f * fmaf(dm, all, a.t);
    a.s = f * all;
  }
  a.cnt = 0.0f;
  a.m = M;
}

template <int N>
__device__ __forceinline__ void tok_update(TokState& st, float (&x)[N], float c) {
  float vm = x[0];
#pragma unroll
  for (int k = 1; k < N; ++k) vm = fmaxf(vm, x[k]);
  if (vm > st.m) {
    // rare: this vector holds the lane's new maximum; split its exact maxima from the rest
    tok_raise(st, vm, c);
#pragma unroll
    for (int k = 0; k < N; ++k) {
      const float d = fminf(st.m - x[k], FLT_MAX);
      if (d == 0.0f) {
        st.cnt += 1.0f;
      } else {
        const float e = __builtin_amdgcn_exp2f(-(d * c));
        st.s += e;
        st.t = fmaf(e, d, st.t);
      }
    }
    return;
  }
  if (st.m == -INFINITY) return;  // nothing finite seen yet: every term is 0
#pragma unroll
  for (int k = 0; k < N; ++k) {
    const float d = fminf(st.m - x[k], FLT_MAX);  // x = -inf contributes 0 to both sums
    const float e = __builtin_amdgcn_exp2f(-(d * c));
    st.s += e;
    st.t = fmaf(e, d, st.t);
  }
}

__device__ __forceinline__ void tok_merge(TokState& a, float m2, float c2, float s2, float t2, float c) {
  TokState b{m2, c2, s2, t2};
  const float M = fmaxf(a.m, b.m);
  tok_raise(a, M, c);
  tok_raise(b, M, c);
  a.cnt += b.cnt;
  a.s += b.s;
  a.t += b.t;
}

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

template <typename T, int UNROLL>
__global__ __launch_bounds__(kTokThreads) void token_logp_entropy_kernel(TokArgs A) {
  constexpr int VEC = 16 / sizeof(T);
  constexpr int NW = kTokThreads / kWave;
  __shared__ float lm[NW], lc[NW], ls[NW], lt[NW];

  const int64_t row = blockIdx.x;
  const T* __restrict__ p = reinterpret_cast<const T*>(A.logits) + row * A.row_stride;
  const int64_t V = A.V;
  const float c = A.c;

  // peel to a 16-byte boundary
  int64_t head = (int64_t)(((16u - (unsigned)(reinterpret_cast<uintptr_t>(p) & 15u)) & 15u) / sizeof(T));
  if (head > V) head = V;
  const int64_t nvec = (V - head) / VEC;
  const int64_t tail0 = head + nvec * VEC;

  TokState st{-INFINITY, 0.0f, 0.0f, 0.0f};
  if ((int64_t)threadIdx.x < head) {
    float x[1] = {Elem<T>::load(p + threadIdx.x)};
    tok_update<1>(st, x, c);
  }
  if (tail0 + (int64_t)threadIdx.x < V) {
    float x[1] = {Elem<T>::load(p + tail0 + threadIdx.x)};
    tok_update<1>(st, x, c);
  }

  const T* __restrict__ pv = p + head;
  for (int64_t i0 = threadIdx.x; i0 < nvec; i0 += (int64_t)kTokThreads * UNROLL) {
    float x[UNROLL][VEC];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int64_t i = i0 + (int64_t)u * kTokThreads;
      if (i < nvec) Vec<T, VEC>::load(pv + i * VEC, x[u]);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int64_t i = i0 + (int64_t)u * kTokThreads;
      if (i < nvec) tok_update<VEC>(st, x[u], c);
    }
  }

  // lanes -> wavefront
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) {
    const float m2 = __shfl_xor(st.m, o, kWave);
    const float c2 = __shfl_xor(st.cnt, o, kWave);
    const float s2 = __shfl_xor(st.s, o, kWave);
    const float t2 = __shfl_xor(st.t, o, kWave);
    tok_merge(st, m2, c2, s2, t2, c);
  }
  const int lane = threadIdx.x & (kWave - 1);
  const int wid = threadIdx.x / kWave;
  if (lane == 0) {
    lm[wid] = st.m;
    lc[wid] = st.cnt;
    ls[wid] = st.s;
    lt[wid] = st.t;
  }
  __syncthreads();
  if (threadIdx.x != 0) return;
#pragma unroll
  for (int w = 1; w < NW; ++w) tok_merge(st, lm[w], lc[w], ls[w], lt[w], c);

  // with lf = x/T:  logsumexp = m/T + ln s ;  H = ln s + (t/s)/T ;  logp = -(m - x_id)/T - ln s
  // ln(cnt + s); cnt >= 1 whenever the row holds a finite logit
  const double ln_s = log((double)st.cnt) + log1p((double)st.s / (double)st.cnt);
  const double sum = (double)st.cnt + (double)st.s;
  const double inv_t = (double)A.inv_t;
  if (A.lse) A.lse[row] = (float)((double)st.m * inv_t + ln_s);
  if (A.ent) A.ent[row] = (float)(ln_s + ((double)st.t / sum) * inv_t);
  if (A.logp) {
    const int64_t id = A.ids[row];
    float out = __uint_as_float(0x7fc00000u);
    if (id >= 0 && id < V) out = (float)(-(((double)st.m - (double)Elem<T>::load(p + id)) * inv_t) - ln_s);
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

template <typename T>
__global__ __launch_bounds__(kTokThreads) void token_logp_bwd_kernel(TokBwdArgs A) {
  const int64_t row = blockIdx.y;
  const T* __restrict__ p = reinterpret_cast<const T*>(A.logits) + row * A.row_stride;
  T* __restrict__ gp = reinterpret_cast<T*>(A.grad) + row * A.grad_row_stride;
  const float lse2 = A.lse[row] * kLog2e;
  const float gs = A.g[row] * A.inv_t;
  const int64_t id = A.ids[row];
  const int64_t stride = (int64_t)gridDim.x * kTokThreads;
  for (int64_t j = (int64_t)blockIdx.x * kTokThreads + threadIdx.x; j < A.V; j += stride) {
    const float x = Elem<T>::load(p + j);
    const float prob = __builtin_amdgcn_exp2f(fmaf(x, A.c, -lse2));
    const float one = (j == id) ? 1.0f : 0.0f;
    Elem<T>::store(gp + j, gs * (one - prob));
  }
}

template <typename T>
static int launch_tok(const TokArgs& A, hipStream_t st) {
  const int unroll = (int)tune_int("UNIRL_TOK_UNROLL", 4);
  dim3 grid((unsigned int)A.rows), block(kTokThreads);
  if (unroll >= 8)
    hipLaunchKernelGGL((token_logp_entropy_kernel<T, 8>), grid, block, 0, st, A);
  else if (unroll >= 4)
    hipLaunchKernelGGL((token_logp_entropy_kernel<T, 4>), grid, block, 0, st, A);
  else if (unroll >= 2)
    hipLaunchKernelGGL((token_logp_entropy_kernel<T, 2>), grid, block, 0, st, A);
  else
    hipLaunchKernelGGL((token_logp_entropy_kernel<T, 1>), grid, block, 0, st, A);
  return (int)hipGetLastError();
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
    int64_t nbx = (V + kTokThreads * 4 - 1) / (kTokThreads * 4);
    if (nbx > 1024) nbx = 1024;
    dim3 grid((unsigned int)nbx, (unsigned int)nr), block(kTokThreads);
    switch (dtype) {
      case UNIRL_F32: hipLaunchKernelGGL((token_logp_bwd_kernel<float>), grid, block, 0, st, A); break;
      case UNIRL_BF16: hipLaunchKernelGGL((token_logp_bwd_kernel<bf16_t>), grid, block, 0, st, A); break;
      case UNIRL_F16: hipLaunchKernelGGL((token_logp_bwd_kernel<f16_t>), grid, block, 0, st, A); break;
    }
    const int rc = (int)hipGetLastError();
    if (rc != 0) return rc;
  }
  return UNIRL_OK;
}
