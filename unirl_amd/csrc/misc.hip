// Small kernels around the hot path: group-normalised advantages and the
// step gather.

#include "common_hip.h"
#include "unirl_internal.h"

namespace unirl {

// ---------------------------------------------------------------------------
// Group advantages: unirl/types/rollout_resp.py:277-283 (global scope) and
// :314-333 (group scope).  One workgroup; statistics in fp64, rounded to f32 at
// the points where the reference holds f32 tensors (mean, var/std), then the
// same f32 operations: `+ eps`, `.sqrt()`, `(r - mean) / std`.
// ---------------------------------------------------------------------------
constexpr int kAdvThreads = 256;

struct AdvArgs {
  const float* r;
  int64_t n_groups, branch;
  int normalize, scope_global, use_global_std;
  float eps;
  float* out;
};

__global__ __launch_bounds__(kAdvThreads) void group_advantages_kernel(AdvArgs A) {
  __shared__ double lds[kAdvThreads / kWave];
  const int64_t n = A.n_groups * A.branch;
  float g_mean = 0.0f, g_std = 1.0f;
  if (A.scope_global || (A.normalize && A.use_global_std)) {
    double s = 0.0;
    for (int64_t i = threadIdx.x; i < n; i += kAdvThreads) s += (double)A.r[i];
    s = block_sum<double>(s, lds);
    const double mean = s / (double)n;
    double q = 0.0;
    for (int64_t i = threadIdx.x; i < n; i += kAdvThreads) {
      const double d = (double)A.r[i] - mean;
      q += d * d;
    }
    q = block_sum<double>(q, lds);
    g_mean = (float)mean;
    const float std_unbiased = (float)sqrt(q / (double)(n - 1));  // n == 1 -> NaN, as torch.std
    g_std = std_unbiased + A.eps;
  }
  if (A.scope_global) {
    for (int64_t i = threadIdx.x; i < n; i += kAdvThreads) {
      const float c = A.r[i] - g_mean;
      A.out[i] = A.normalize ? c / g_std : c;
    }
    return;
  }
  // one lane per group; groups are short (the branching factor of a prompt)
  for (int64_t g = threadIdx.x; g < A.n_groups; g += kAdvThreads) {
    const float* rg = A.r + g * A.branch;
    double s = 0.0;
    for (int64_t j = 0; j < A.branch; ++j) s += (double)rg[j];
    const double mean = s / (double)A.branch;
    const float mean_f = (float)mean;
    float std_f = 1.0f;
    if (A.normalize) {
      if (A.use_global_std) {
        std_f = g_std;
      } else {
        double q = 0.0;
        for (int64_t j = 0; j < A.branch; ++j) {
          const double d = (double)rg[j] - mean;
          q += d * d;
        }
        const float var_pop = (float)(q / (double)A.branch);
        std_f = sqrtf(var_pop + A.eps);
      }
    }
    for (int64_t j = 0; j < A.branch; ++j) {
      const float c = rg[j] - mean_f;
      A.out[g * A.branch + j] = A.normalize ? c / std_f : c;
    }
  }
}

// ---------------------------------------------------------------------------
// out[b, j, :] = src[b, pos[j], :]   (unirl/algorithms/base.py:70,80)
// ---------------------------------------------------------------------------
constexpr int kGatherThreads = 256;

template <typename W>
__global__ __launch_bounds__(kGatherThreads) void gather_steps_kernel(const W* __restrict__ src, int64_t S,
                                                                      int64_t inner, const int64_t* __restrict__ pos,
                                                                      int64_t n_pos, W* __restrict__ out) {
  const int64_t bj = blockIdx.y;  // b * n_pos + j
  const int64_t b = bj / n_pos, j = bj % n_pos;
  const int64_t p = pos[j];
  if (p < 0 || p >= S) return;  // validated on the host; never read out of bounds
  const W* s = src + (b * S + p) * inner;
  W* o = out + bj * inner;
  const int64_t stride = (int64_t)gridDim.x * kGatherThreads;
  for (int64_t i = (int64_t)blockIdx.x * kGatherThreads + threadIdx.x; i < inner; i += stride) o[i] = s[i];
}

// ---------------------------------------------------------------------------
// out[t] = vals[seq(t)] for packed tokens: the per-token expansion of per-sample
// advantages (unirl/algorithms/grpo.py:187-198) without a host loop.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(kGatherThreads) void expand_per_seq_kernel(const float* __restrict__ vals,
                                                                        const int64_t* __restrict__ cu, int64_t n_seq,
                                                                        int64_t n_tok, float* __restrict__ out) {
  const int64_t stride = (int64_t)gridDim.x * kGatherThreads;
  int64_t end = -1;
  float v = 0.0f;
  for (int64_t t = (int64_t)blockIdx.x * kGatherThreads + threadIdx.x; t < n_tok; t += stride) {
    if (t >= end) {
      int64_t lo = 0, hi = n_seq;  // cu[lo] <= t < cu[hi]
      while (hi - lo > 1) {
        const int64_t mid = (lo + hi) >> 1;
        if (cu[mid] <= t) lo = mid; else hi = mid;
      }
      end = cu[lo + 1];
      v = vals[lo];
    }
    out[t] = v;
  }
}

// ---------------------------------------------------------------------------
// Grouped normalisation over arbitrary index lists (CSR), with optional trimmed
// statistics and clipping: unirl/algorithms/normalizers.py:32-59.  One lane per
// group.  Trimming drops the k smallest and k largest members from the
// statistics; membership is decided by rank (ties broken by position, i.e. a
// stable sort), so no per-lane sort buffer is needed.
// ---------------------------------------------------------------------------
struct NormArgs {
  const float* r;
  int64_t n;
  const int64_t* members;  // concatenated group members
  const int64_t* offsets;  // [n_groups + 1]
  int64_t n_groups;
  float eps;
  float trim_ratio;
  int use_global_std;
  int has_clip;
  float clip_max;
  float* out;
};

__global__ __launch_bounds__(kAdvThreads) void normalize_grouped_kernel(NormArgs A) {
  __shared__ double lds[kAdvThreads / kWave];
  float batch_std = 1.0f;
  if (A.use_global_std) {
    double s = 0.0;
    for (int64_t i = threadIdx.x; i < A.n; i += kAdvThreads) s += (double)A.r[i];
    s = block_sum<double>(s, lds);
    const double mean = s / (double)A.n;
    double q = 0.0;
    for (int64_t i = threadIdx.x; i < A.n; i += kAdvThreads) {
      const double d = (double)A.r[i] - mean;
      q += d * d;
    }
    q = block_sum<double>(q, lds);
    batch_std = (float)sqrt(q / (double)(A.n - 1)) + A.eps;
  }
  for (int64_t g = threadIdx.x; g < A.n_groups; g += kAdvThreads) {
    const int64_t lo = A.offsets[g], hi = A.offsets[g + 1];
    const int64_t m = hi - lo;
    if (m <= 0) continue;
    int64_t k = 0;
    if (A.trim_ratio > 0.0f && m > 2) {
      k = (int64_t)((double)m * (double)A.trim_ratio);  // int(len * ratio)
      if (!(k > 0 && 2 * k < m)) k = 0;
    }
    // pass 1: mean over the kept ranks
    double s = 0.0;
    int64_t kept = 0;
    for (int64_t a = lo; a < hi; ++a) {
      const float va = A.r[A.members[a]];
      bool keep = true;
      if (k > 0) {
        int64_t rank = 0;
        for (int64_t b = lo; b < hi; ++b) {
          const float vb = A.r[A.members[b]];
          rank += (vb < va || (vb == va && b < a)) ? 1 : 0;
        }
        keep = (rank >= k) && (rank < m - k);
      }
      if (keep) {
        s += (double)va;
        ++kept;
      }
    }
    const double mean = s / (double)kept;
    float scale = batch_std;
    if (!A.use_global_std) {
      double q = 0.0;
      for (int64_t a = lo; a < hi; ++a) {
        const float va = A.r[A.members[a]];
        bool keep = true;
        if (k > 0) {
          int64_t rank = 0;
          for (int64_t b = lo; b < hi; ++b) {
            const float vb = A.r[A.members[b]];
            rank += (vb < va || (vb == va && b < a)) ? 1 : 0;
          }
          keep = (rank >= k) && (rank < m - k);
        }
        if (keep) {
          const double d = (double)va - mean;
          q += d * d;
        }
      }
      scale = (float)sqrt(q / (double)(kept - 1)) + A.eps;  // one kept member -> NaN, as torch.std
    }
    const float mean_f = (float)mean;
    for (int64_t a = lo; a < hi; ++a) {
      float v = (A.r[A.members[a]] - mean_f) / scale;
      if (A.has_clip) v = nan_clamp(v, -A.clip_max, A.clip_max);  // torch.clamp keeps NaN
      A.out[A.members[a]] = v;
    }
  }
}

// out[b, :] = cast(src[group_of[b], :]): the batch of initial latents from one fp32 draw per
// noise group (unirl/sde/noise.py:78-97 stacks the shared draws; :187 casts as the last step).
struct ExpandArgs {
  const float* src;         // [U, D]
  const int64_t* group_of;  // [B], values in [0, U)
  int64_t U, D;
  void* out;                // [B, D]
  int dtype;
};

template <typename TO, int VEC>
__global__ __launch_bounds__(kGatherThreads) void expand_groups_kernel(ExpandArgs A) {
  const int64_t b = blockIdx.y;
  int64_t u = A.group_of[b];
  u = u < 0 ? 0 : (u >= A.U ? A.U - 1 : u);  // validated by the caller; never index outside src
  const float* __restrict__ s = A.src + u * A.D;
  TO* __restrict__ o = reinterpret_cast<TO*>(A.out) + b * A.D;
  const int64_t nvec = A.D / VEC;
  const int64_t stride = (int64_t)gridDim.x * kGatherThreads;
  for (int64_t i = (int64_t)blockIdx.x * kGatherThreads + threadIdx.x; i < nvec; i += stride) {
    float v[VEC];
    Vec<float, VEC>::load(s + i * VEC, v);
    Vec<TO, VEC>::store(o + i * VEC, v);
  }
}

template <typename TO>
static int launch_expand(const ExpandArgs& A, int64_t B, int vec, hipStream_t st) {
  int64_t nbx = (A.D / vec + kGatherThreads * 4 - 1) / (kGatherThreads * 4);
  if (nbx > 1024) nbx = 1024;
  if (nbx < 1) nbx = 1;
  dim3 grid((unsigned int)nbx, (unsigned int)B), block(kGatherThreads);
  if (vec == 4)
    hipLaunchKernelGGL((expand_groups_kernel<TO, 4>), grid, block, 0, st, A);
  else
    hipLaunchKernelGGL((expand_groups_kernel<TO, 1>), grid, block, 0, st, A);
  return (int)hipGetLastError();
}

}  // namespace unirl

using namespace unirl;

extern "C" int unirl_group_advantages(const float* rewards, int64_t n_groups, int64_t branch, int normalize,
                                      float eps, int scope_global, int use_global_std, float* adv_out,
                                      void* stream) {
  if (n_groups < 0 || branch < 0) return UNIRL_E_SHAPE;
  if (n_groups == 0 || branch == 0) return UNIRL_OK;
  if (!rewards || !adv_out) return UNIRL_E_NULL;
  if (!aligned_to(rewards, 4) || !aligned_to(adv_out, 4)) return UNIRL_E_ALIGN;
  AdvArgs A;
  A.r = rewards;
  A.n_groups = n_groups;
  A.branch = branch;
  A.normalize = normalize;
  A.scope_global = scope_global;
  A.use_global_std = use_global_std;
  A.eps = eps;
  A.out = adv_out;
  hipLaunchKernelGGL(group_advantages_kernel, dim3(1), dim3(kAdvThreads), 0, (hipStream_t)stream, A);
  return (int)hipGetLastError();
}

extern "C" int unirl_gather_steps(const void* src, int64_t B, int64_t S, int64_t inner_bytes,
                                  const int64_t* positions, int64_t n_pos, void* out, void* stream) {
  if (B < 0 || S < 0 || inner_bytes < 0 || n_pos < 0) return UNIRL_E_SHAPE;
  if (B == 0 || n_pos == 0 || inner_bytes == 0) return UNIRL_OK;
  if (!src || !positions || !out) return UNIRL_E_NULL;
  if (S == 0) return UNIRL_E_SHAPE;
  if (!aligned_to(positions, 8)) return UNIRL_E_ALIGN;
  hipStream_t st = (hipStream_t)stream;
  // widest word that divides the slice size and both base addresses
  int w = 16;
  while (w > 1 && (inner_bytes % w != 0 || !aligned_to(src, w) || !aligned_to(out, w))) w >>= 1;
  const int64_t inner = inner_bytes / w;
  int64_t nbx = (inner + kGatherThreads * 4 - 1) / (kGatherThreads * 4);
  if (nbx > 1024) nbx = 1024;
  if (nbx < 1) nbx = 1;
  const int64_t rows_total = B * n_pos;
  const int64_t per_launch = 32768;
  const int64_t b_per_launch = (per_launch / n_pos) > 0 ? (per_launch / n_pos) : 0;
  if (b_per_launch == 0) return UNIRL_E_LIMIT;  // more than 32768 positions
  (void)rows_total;
  for (int64_t b0 = 0; b0 < B; b0 += b_per_launch) {
    const int64_t nb = (B - b0 < b_per_launch) ? (B - b0) : b_per_launch;
    const char* s = reinterpret_cast<const char*>(src) + b0 * S * inner_bytes;
    char* o = reinterpret_cast<char*>(out) + b0 * n_pos * inner_bytes;
    dim3 grid((unsigned int)nbx, (unsigned int)(nb * n_pos)), block(kGatherThreads);
    switch (w) {
      case 16:
        hipLaunchKernelGGL((gather_steps_kernel<uint4>), grid, block, 0, st, reinterpret_cast<const uint4*>(s), S,
                           inner, positions, n_pos, reinterpret_cast<uint4*>(o));
        break;
      case 8:
        hipLaunchKernelGGL((gather_steps_kernel<uint2>), grid, block, 0, st, reinterpret_cast<const uint2*>(s), S,
                           inner, positions, n_pos, reinterpret_cast<uint2*>(o));
        break;
      case 4:
        hipLaunchKernelGGL((gather_steps_kernel<uint32_t>), grid, block, 0, st,
                           reinterpret_cast<const uint32_t*>(s), S, inner, positions, n_pos,
                           reinterpret_cast<uint32_t*>(o));
        break;
      case 2:
        hipLaunchKernelGGL((gather_steps_kernel<uint16_t>), grid, block, 0, st,
                           reinterpret_cast<const uint16_t*>(s), S, inner, positions, n_pos,
                           reinterpret_cast<uint16_t*>(o));
        break;
      default:
        hipLaunchKernelGGL((gather_steps_kernel<uint8_t>), grid, block, 0, st, reinterpret_cast<const uint8_t*>(s),
                           S, inner, positions, n_pos, reinterpret_cast<uint8_t*>(o));
        break;
    }
    const int rc = (int)hipGetLastError();
    if (rc != 0) return rc;
  }
  return UNIRL_OK;
}

extern "C" int unirl_expand_per_seq(const float* vals, const int64_t* cu_seqlens, int64_t n_seq, int64_t n_tok,
                                    float* out, void* stream) {
  if (n_seq < 0 || n_tok < 0) return UNIRL_E_SHAPE;
  if (n_tok == 0) return UNIRL_OK;
  if (!vals || !cu_seqlens || !out) return UNIRL_E_NULL;
  if (n_seq == 0) return UNIRL_E_SHAPE;
  if (!aligned_to(vals, 4) || !aligned_to(cu_seqlens, 8) || !aligned_to(out, 4)) return UNIRL_E_ALIGN;
  int64_t nb = (n_tok + kGatherThreads * 4 - 1) / (kGatherThreads * 4);
  if (nb > 4096) nb = 4096;
  hipLaunchKernelGGL(expand_per_seq_kernel, dim3((unsigned int)nb), dim3(kGatherThreads), 0, (hipStream_t)stream,
                     vals, cu_seqlens, n_seq, n_tok, out);
  return (int)hipGetLastError();
}

extern "C" int unirl_normalize_grouped(const float* rewards, int64_t n, const int64_t* members,
                                       const int64_t* offsets, int64_t n_groups, float eps, float trim_ratio,
                                       int use_global_std, int has_clip, float clip_max, float* out,
                                       void* stream) {
  if (n < 0 || n_groups < 0) return UNIRL_E_SHAPE;
  if (n == 0 || n_groups == 0) return UNIRL_OK;
  if (!rewards || !members || !offsets || !out) return UNIRL_E_NULL;
  if (!aligned_to(rewards, 4) || !aligned_to(out, 4) || !aligned_to(members, 8) || !aligned_to(offsets, 8))
    return UNIRL_E_ALIGN;
  NormArgs A;
  A.r = rewards;
  A.n = n;
  A.members = members;
  A.offsets = offsets;
  A.n_groups = n_groups;
  A.eps = eps;
  A.trim_ratio = trim_ratio;
  A.use_global_std = use_global_std;
  A.has_clip = has_clip;
  A.clip_max = clip_max;
  A.out = out;
  hipLaunchKernelGGL(normalize_grouped_kernel, dim3(1), dim3(kAdvThreads), 0, (hipStream_t)stream, A);
  return (int)hipGetLastError();
}

extern "C" int unirl_expand_groups(const float* src, int64_t U, int64_t D, const int64_t* group_of, int64_t B,
                                   void* out, int out_dtype, void* stream) {
  if (!dtype_ok(out_dtype)) return UNIRL_E_DTYPE;
  if (U < 0 || D < 0 || B < 0) return UNIRL_E_SHAPE;
  if (B == 0 || D == 0) return UNIRL_OK;
  if (U == 0) return UNIRL_E_SHAPE;
  if (!src || !group_of || !out) return UNIRL_E_NULL;
  const size_t so = dtype_size(out_dtype);
  if (!aligned_to(src, 4) || !aligned_to(group_of, 8) || !aligned_to(out, so)) return UNIRL_E_ALIGN;
  const int vec = (D % 4 == 0 && aligned_to(src, 16) && aligned_to(out, 4 * so)) ? 4 : 1;
  hipStream_t st = (hipStream_t)stream;
  const int64_t per_launch = 32768;  // grid.y limit is 65535
  for (int64_t b0 = 0; b0 < B; b0 += per_launch) {
    const int64_t nb = (B - b0 < per_launch) ? (B - b0) : per_launch;
    ExpandArgs A;
    A.src = src;
    A.group_of = group_of + b0;
    A.U = U;
    A.D = D;
    A.out = reinterpret_cast<char*>(out) + b0 * D * (int64_t)so;
    A.dtype = out_dtype;
    int rc = UNIRL_E_DTYPE;
    switch (out_dtype) {
      case UNIRL_F32: rc = launch_expand<float>(A, nb, vec, st); break;
      case UNIRL_BF16: rc = launch_expand<bf16_t>(A, nb, vec, st); break;
      case UNIRL_F16: rc = launch_expand<f16_t>(A, nb, vec, st); break;
    }
    if (rc != 0) return rc;
  }
  return UNIRL_OK;
}
