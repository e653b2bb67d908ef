// Gaussian KL between old and new transition means, reduced per (sample, step)
// row and thresholded into the Flow-DPPO trust-region mask.
//
// Replaces unirl/algorithms/flowdppo.py:
//   _gaussian_kl_div          :43-51   (p - q)**2 / (2 * sigma**2)
//   kl_per_sample / kl_mask   :92-96   mean over dims >= 2, then `< threshold`
// torch's type promotion is reproduced: with 16-bit means and an f32 sigma
// tensor, the subtraction and the square each round to the 16-bit dtype and
// only the division runs in f32.  The kernel sums the squares (f32 per lane,
// f64 across lanes and workgroups, fixed order) and divides once per row.
//
// HBM traffic: 2 * D * sizeof(T) bytes read per row, 5 bytes written per row.

#include <mutex>

#include "common_hip.h"
#include "dppo_body.h"
#include "unirl_internal.h"

namespace unirl {

constexpr int kKlThreads = 256;
// Rows (and partial slots) the allocation-free entry point accepts: 32768 doubles = 256 KiB per GPU.
constexpr int64_t kKlStaticRows = UNIRL_KL_STATIC_MAX_ROWS;

struct KlArgs {
  const void* p;
  const void* q;
  const float* sigma;
  int64_t n_sigma;
  int64_t row0;  // global index of the first row of this launch (for the sigma lookup)
  int64_t D;
  float threshold;
  float* kl;
  uint8_t* mask;
  float* elem_out;
  double* partials;
  int always_partials;  // store workgroup partials even when one workgroup covers a row
  UNIRL_TRACE_FIELD
};

__device__ __forceinline__ float kl_den(const KlArgs& A, int64_t row) {
  const float s = A.sigma[(A.row0 + row) % A.n_sigma];
  return 2.0f * (s * s);
}

__device__ __forceinline__ void kl_finish(const KlArgs& A, int64_t row, double q, float den) {
  const float kl = (float)((q / (double)den) / (double)A.D);
  A.kl[row] = kl;
  if (A.mask) A.mask[row] = (kl < A.threshold) ? 1 : 0;
}

template <typename T, int VEC, int ITEMS>
__global__ __launch_bounds__(kKlThreads) void gaussian_kl_kernel(KlArgs A) {
  __shared__ double lds[kKlThreads / kWave];
  UNIRL_TRACE_T0();
  const int64_t row = blockIdx.y;
  const int64_t D = A.D;
  const T* __restrict__ pp = reinterpret_cast<const T*>(A.p) + row * D;
  const T* __restrict__ qp = reinterpret_cast<const T*>(A.q) + row * D;
  const int64_t nvec = D / VEC;
  const int64_t stride = (int64_t)gridDim.x * kKlThreads;
  float acc = 0.0f;
  for (int64_t i0 = (int64_t)blockIdx.x * kKlThreads + threadIdx.x; i0 < nvec; i0 += stride * ITEMS) {
    float a[ITEMS][VEC], b[ITEMS][VEC];
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      const int64_t i = i0 + it * stride;
      if (i < nvec) {
        Vec<T, VEC>::load(pp + i * VEC, a[it]);
        Vec<T, VEC>::load(qp + i * VEC, b[it]);
      }
    }
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      const int64_t i = i0 + it * stride;
      if (i < nvec) {
#pragma unroll
        for (int k = 0; k < VEC; ++k) acc += kl_sq<T>(a[it][k], b[it][k]);
      }
    }
  }
  UNIRL_TRACE_MARK1();
  const double part = block_sum<double>((double)acc, lds);
  if (threadIdx.x != 0) return;
  if (gridDim.x == 1 && !A.always_partials) {
    kl_finish(A, row, part, kl_den(A, row));
  } else {
    A.partials[row * gridDim.x + blockIdx.x] = part;  // summed by gaussian_kl_finalize_kernel
  }
  UNIRL_TRACE_END(A.trace);
}

// One wavefront per row: adds the workgroup partials in index order, divides, thresholds.
__global__ __launch_bounds__(kKlThreads) void gaussian_kl_finalize_kernel(KlArgs A, int64_t R, unsigned int nblk) {
  UNIRL_TRACE_T0();
  const int64_t row = (int64_t)blockIdx.x * (kKlThreads / kWave) + threadIdx.x / kWave;
  if (row >= R) return;
  const float den = kl_den(A, row);  // issued with the partial loads, not after them
  const double q = wave_ordered_sum(A.partials + row * nblk, nblk);
  UNIRL_TRACE_MARK1();
  if ((threadIdx.x & (kWave - 1)) == 0) kl_finish(A, row, q, den);
  UNIRL_TRACE_END(A.trace);
}

template <typename T, int VEC>
__global__ __launch_bounds__(kKlThreads) void gaussian_kl_elem_kernel(KlArgs A) {
  const int64_t row = blockIdx.y;
  const int64_t D = A.D;
  const T* __restrict__ pp = reinterpret_cast<const T*>(A.p) + row * D;
  const T* __restrict__ qp = reinterpret_cast<const T*>(A.q) + row * D;
  float* __restrict__ op = A.elem_out + row * D;
  const float den = kl_den(A, row);
  const int64_t nvec = D / VEC;
  const int64_t stride = (int64_t)gridDim.x * kKlThreads;
  for (int64_t i = (int64_t)blockIdx.x * kKlThreads + threadIdx.x; i < nvec; i += stride) {
    float a[VEC], b[VEC], o[VEC];
    Vec<T, VEC>::load(pp + i * VEC, a);
    Vec<T, VEC>::load(qp + i * VEC, b);
#pragma unroll
    for (int k = 0; k < VEC; ++k) o[k] = kl_sq<T>(a[k], b[k]) / den;
    Vec<float, VEC>::store(op + i * VEC, o);
  }
}

// Backward of the element-wise form through autograd's own chain: out = sq / den (f32),
// sq = d*d and d = p - q in the means' dtype.  The incoming f32 gradient is divided by den and
// rounded to that dtype, multiplied by 2d there, and reaches p as is and q negated.
template <typename T, int VEC>
__global__ __launch_bounds__(kKlThreads) void gaussian_kl_elem_bwd_kernel(KlArgs A, const float* g, void* grad_p,
                                                                          void* grad_q) {
  const int64_t row = blockIdx.y;
  const int64_t D = A.D;
  const T* __restrict__ pp = reinterpret_cast<const T*>(A.p) + row * D;
  const T* __restrict__ qp = reinterpret_cast<const T*>(A.q) + row * D;
  const float* __restrict__ gp = g + row * D;
  T* __restrict__ op = grad_p ? reinterpret_cast<T*>(grad_p) + row * D : nullptr;
  T* __restrict__ oq = grad_q ? reinterpret_cast<T*>(grad_q) + row * D : nullptr;
  const float den = kl_den(A, row);
  const int64_t nvec = D / VEC;
  const int64_t stride = (int64_t)gridDim.x * kKlThreads;
  for (int64_t i = (int64_t)blockIdx.x * kKlThreads + threadIdx.x; i < nvec; i += stride) {
    float a[VEC], b[VEC], gg[VEC], o[VEC], n[VEC];
    Vec<T, VEC>::load(pp + i * VEC, a);
    Vec<T, VEC>::load(qp + i * VEC, b);
    Vec<float, VEC>::load(gp + i * VEC, gg);
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
      const float d = Elem<T>::round_trip(a[k] - b[k]);
      const float gs = Elem<T>::round_trip(gg[k] / den);
      o[k] = Elem<T>::round_trip(gs * (2.0f * d));
      n[k] = -o[k];
    }
    if (op) Vec<T, VEC>::store(op + i * VEC, o);
    if (oq) Vec<T, VEC>::store(oq + i * VEC, n);
  }
}

template <typename T>
static int launch_kl_elem_bwd(const KlArgs& A, int64_t R, int vec, const float* g, void* gp, void* gq,
                              hipStream_t st) {
  int64_t nblk = (A.D / vec + kKlThreads - 1) / kKlThreads;
  if (nblk > 2048) nblk = 2048;
  if (nblk < 1) nblk = 1;
  dim3 grid((unsigned int)nblk, (unsigned int)R), block(kKlThreads);
  if (vec == 4)
    hipLaunchKernelGGL((gaussian_kl_elem_bwd_kernel<T, 4>), grid, block, 0, st, A, g, gp, gq);
  else
    hipLaunchKernelGGL((gaussian_kl_elem_bwd_kernel<T, 1>), grid, block, 0, st, A, g, gp, gq);
  return (int)hipGetLastError();
}

static unsigned int kl_blocks_per_row(int64_t nvec, int items, int64_t R) {
  const int64_t per_pass = (int64_t)kKlThreads * items;
  int64_t nblk = (nvec + per_pass - 1) / per_pass;
  const int64_t cap = tune_int("UNIRL_KL_MAX_BLOCKS", 512);
  int64_t max_per_row = cap / (R > 0 ? R : 1);
  if (max_per_row < 1) max_per_row = 1;
  if (nblk > max_per_row) nblk = max_per_row;
  if (nblk > kMaxPartialBlocks) nblk = kMaxPartialBlocks;
  if (nblk < 1) nblk = 1;
  return (unsigned int)nblk;
}

template <typename T>
static int launch_kl(const KlArgs& A, int64_t R, int vec, unsigned int nblk, int items, hipStream_t st) {
  dim3 grid(nblk, (unsigned int)R), block(kKlThreads);
  if constexpr (sizeof(T) == 2) {
    if (vec == 8) {  // 16-byte loads of eight 16-bit values
      if (items >= 4)
        hipLaunchKernelGGL((gaussian_kl_kernel<T, 8, 4>), grid, block, 0, st, A);
      else if (items >= 2)
        hipLaunchKernelGGL((gaussian_kl_kernel<T, 8, 2>), grid, block, 0, st, A);
      else
        hipLaunchKernelGGL((gaussian_kl_kernel<T, 8, 1>), grid, block, 0, st, A);
      return (int)hipGetLastError();
    }
  }
  if (vec == 4) {
    if (items >= 4)
      hipLaunchKernelGGL((gaussian_kl_kernel<T, 4, 4>), grid, block, 0, st, A);
    else if (items >= 2)
      hipLaunchKernelGGL((gaussian_kl_kernel<T, 4, 2>), grid, block, 0, st, A);
    else
      hipLaunchKernelGGL((gaussian_kl_kernel<T, 4, 1>), grid, block, 0, st, A);
  } else {
    hipLaunchKernelGGL((gaussian_kl_kernel<T, 1, 2>), grid, block, 0, st, A);
  }
  return (int)hipGetLastError();
}

template <typename T>
static int launch_kl_elem(const KlArgs& A, int64_t R, int vec, hipStream_t st) {
  int64_t nblk = (A.D / vec + kKlThreads - 1) / kKlThreads;
  if (nblk > 2048) nblk = 2048;
  if (nblk < 1) nblk = 1;
  dim3 grid((unsigned int)nblk, (unsigned int)R), block(kKlThreads);
  if (vec == 4)
    hipLaunchKernelGGL((gaussian_kl_elem_kernel<T, 4>), grid, block, 0, st, A);
  else
    hipLaunchKernelGGL((gaussian_kl_elem_kernel<T, 1>), grid, block, 0, st, A);
  return (int)hipGetLastError();
}

// Launched with one wavefront for up to kDppoWaveMax elements, with a workgroup beyond.

__global__ __launch_bounds__(kKlThreads) void flowdppo_loss_kernel(DppoArgs A) {
  if (blockDim.x == kWave) {
    dppo_on_one_wave(A, A.kl);
    return;
  }
  __shared__ double lds[kKlThreads / kWave];
  __shared__ float ldsf[kKlThreads / kWave];
  DppoAcc s;
  // every wavefront makes the same number of trips as a whole (its counters are taken across the lanes)
  for (int64_t base = 0; base < A.n; base += kKlThreads) {
    const int64_t i = base + threadIdx.x;
    const bool valid = i < A.n;
    dppo_elem_of(A, i, valid, valid ? A.nw[i] : 0.0f, valid ? A.od[i] : 0.0f, valid ? A.adv[i] : 0.0f,
                 valid ? A.kl[i] : 0.0f, s);
  }
  double tot[D_SUMS];
#pragma unroll
  for (int v = 0; v < D_SUMS; ++v) tot[v] = block_sum<double>(s.acc[v], lds);
  // the wavefronts' counters (exact in fp64), carried by each wavefront's first lane
  unsigned long long cnt[C_VALS];
  const bool lead = (threadIdx.x & (kWave - 1)) == 0;
#pragma unroll
  for (int v = 0; v < C_VALS; ++v) cnt[v] = (unsigned long long)block_sum<double>(lead ? (double)s.cnt[v] : 0.0, lds);
  const float rmin = block_min(s.rmin, ldsf), rmax = block_max(s.rmax, ldsf), klmax = block_max(s.klmax, ldsf);
  if (threadIdx.x == 0) dppo_metrics(A, tot, cnt, rmin, rmax, klmax);
}

// KL finalize and the KL-ADV loss in one launch: the sixteen wavefronts of one workgroup add the
// streaming kernel's partials row by row (fixed order), leave the per-row KL in LDS, and the
// first wavefront runs the [B,S'] problem on it.  With one partial per lane a wavefront keeps the
// loads of four of its rows in flight at once: every trip to memory that waits for the one before
// costs about a microsecond here, and a row per trip made this kernel 5.5 us at 24 rows.
// R <= kDppoWaveMax.
constexpr int kDppoFinishThreads = 1024;
__global__ __launch_bounds__(kDppoFinishThreads) void flowdppo_finish_kernel(KlArgs K, DppoArgs A, unsigned int nblk) {
  __shared__ float lds_kl[kDppoWaveMax];
  UNIRL_TRACE_T0();
  const int wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  constexpr int kWaves = kDppoFinishThreads / kWave;
  const int64_t R = A.n;
  // the first wavefront's share of the [B,S'] problem is loaded now, with the partials, not after them
  float first[3] = {0.0f, 0.0f, 0.0f};
  if (wave == 0 && (int64_t)threadIdx.x < A.n) {
    first[0] = A.nw[threadIdx.x];
    first[1] = A.od[threadIdx.x];
    first[2] = A.adv[threadIdx.x];
  }
  auto finish_row = [&](int64_t row, double q, float den) {
    const float kl = (float)((q / (double)den) / (double)K.D);
    if (lane == 0) {
      K.kl[row] = kl;
      if (K.mask) K.mask[row] = (kl < K.threshold) ? 1 : 0;
      lds_kl[row] = kl;
    }
  };
  if (nblk <= kWave) {
    constexpr int kRows = 4;
    const unsigned int jl = (unsigned int)lane < nblk ? lane : nblk - 1;
    for (int64_t base = wave; base < R; base += kWaves * kRows) {
      double y[kRows];
      float den[kRows];
#pragma unroll
      for (int r = 0; r < kRows; ++r) {
        const int64_t row = base + r * kWaves;
        const int64_t rc = row < R ? row : R - 1;  // past the end: the last row again, dropped below
        y[r] = K.partials[rc * nblk + jl];
        den[r] = kl_den(K, rc);
      }
      __builtin_amdgcn_sched_barrier(0);  // every load issued before the first value is used
#pragma unroll
      for (int r = 0; r < kRows; ++r) {
        const int64_t row = base + r * kWaves;
        if (row < R) finish_row(row, wave_sum((unsigned int)lane < nblk ? y[r] : 0.0), den[r]);  // wave-uniform
      }
    }
  } else {
    // many partials per row means few rows (rows * nblk is capped by the launch): one row at a time
    for (int64_t row = wave; row < R; row += kWaves) {
      const float den = kl_den(K, row);  // issued with the partial loads, not after them
      finish_row(row, wave_ordered_sum(K.partials + row * nblk, nblk), den);
    }
  }
  UNIRL_TRACE_MARK1();
  __syncthreads();
  if (wave == 0) dppo_on_one_wave(A, lds_kl, first);
  UNIRL_TRACE_END(K.trace);
}

}  // namespace unirl

using namespace unirl;

extern "C" int unirl_flowdppo_loss(const float* new_logp, const float* old_logp, const float* advantages,
                                   const float* kl, int64_t n, float threshold, float* loss_elem, float* metrics,
                                   void* stream) {
  if (n < 0) return UNIRL_E_SHAPE;
  if (!metrics) return UNIRL_E_NULL;
  if (n > 0 && (!new_logp || !old_logp || !advantages || !kl || !loss_elem)) return UNIRL_E_NULL;
  if (!aligned_to(new_logp, 4) || !aligned_to(old_logp, 4) || !aligned_to(advantages, 4) || !aligned_to(kl, 4) ||
      !aligned_to(loss_elem, 4) || !aligned_to(metrics, 4))
    return UNIRL_E_ALIGN;
  DppoArgs A;
  A.nw = new_logp;
  A.od = old_logp;
  A.adv = advantages;
  A.kl = kl;
  A.n = n;
  A.threshold = threshold;
  A.loss_elem = loss_elem;
  A.metrics = metrics;
  A.grad_new = nullptr;
  A.grad_scale = 0.0f;
  hipLaunchKernelGGL(flowdppo_loss_kernel, dim3(1), dim3(n <= kDppoWaveMax ? kWave : kKlThreads), 0,
                     (hipStream_t)stream, A);
  return (int)hipGetLastError();
}

// Shared body of the two row-KL entry points; `partials` holds `capacity` doubles.
static int kl_mask_run(const void* p, const void* q, int dtype, const float* sigma, int64_t n_sigma, int64_t R,
                       int64_t D, float threshold, float* kl_out, uint8_t* mask_out, double* partials,
                       int64_t capacity, hipStream_t st) {
  const size_t sz = dtype_size(dtype);
  if (!aligned_to(p, sz) || !aligned_to(q, sz)) return UNIRL_E_ALIGN;
  int vec = 4;
  if (D % 4 != 0 || !aligned_to(p, 4 * sz) || !aligned_to(q, 4 * sz)) vec = 1;
  if (sz == 2 && D % 8 == 0 && aligned_to(p, 16) && aligned_to(q, 16)) vec = 8;
  const int items = (vec >= 4) ? (int)tune_int("UNIRL_KL_ITEMS", 2) : 2;
  const unsigned int nblk = kl_blocks_per_row(D / vec, items, R);
  int64_t per_launch = capacity / nblk;
  if (per_launch > 32768) per_launch = 32768;
  if (per_launch < 1) return UNIRL_E_LIMIT;
  for (int64_t r0 = 0; r0 < R; r0 += per_launch) {
    const int64_t nr = (R - r0 < per_launch) ? (R - r0) : per_launch;
    KlArgs A = {};
    A.p = offset_ptr(p, r0 * D, sz);
    A.q = offset_ptr(q, r0 * D, sz);
    A.sigma = sigma;
    A.n_sigma = n_sigma;
    A.row0 = r0;
    A.D = D;
    A.threshold = threshold;
    A.kl = kl_out + r0;
    A.mask = mask_out ? mask_out + r0 : nullptr;
    A.elem_out = nullptr;
    A.partials = partials;
    UNIRL_TRACE_SET(A, "kl", nblk * (unsigned int)nr);
    int rc = UNIRL_E_DTYPE;
    switch (dtype) {
      case UNIRL_F32: rc = launch_kl<float>(A, nr, vec, nblk, items, st); break;
      case UNIRL_BF16: rc = launch_kl<bf16_t>(A, nr, vec, nblk, items, st); break;
      case UNIRL_F16: rc = launch_kl<f16_t>(A, nr, vec, nblk, items, st); break;
    }
    if (rc != 0) return rc;
    if (nblk > 1) {
      const int per_block = kKlThreads / kWave;
      UNIRL_TRACE_SET(A, "kl_finalize", (unsigned int)((nr + per_block - 1) / per_block));
      hipLaunchKernelGGL(gaussian_kl_finalize_kernel, dim3((unsigned int)((nr + per_block - 1) / per_block)),
                         dim3(kKlThreads), 0, st, A, nr, nblk);
      rc = (int)hipGetLastError();
      if (rc != 0) return rc;
    }
  }
  return UNIRL_OK;
}

extern "C" int unirl_gaussian_kl_mask(const void* p, const void* q, int dtype, const float* sigma, int64_t n_sigma,
                                      int64_t R, int64_t D, float threshold, float* kl_out, uint8_t* mask_out,
                                      void* workspace, size_t workspace_bytes, void* stream) {
  if (!dtype_ok(dtype)) return UNIRL_E_DTYPE;
  if (R < 0 || D <= 0 || n_sigma <= 0) return UNIRL_E_SHAPE;
  if (R == 0) return UNIRL_OK;
  if (!p || !q || !sigma || !kl_out) return UNIRL_E_NULL;
  if (!workspace || workspace_bytes < kWorkspaceBytes) return UNIRL_E_WORKSPACE;
  return kl_mask_run(p, q, dtype, sigma, n_sigma, R, D, threshold, kl_out, mask_out, ws_partials(workspace),
                     kPartialCapacity, (hipStream_t)stream);
}

// ---------------------------------------------------------------------------
// The same call for callers that cannot allocate (a HIP graph under capture, a serving loop, a
// harness that forbids hipMalloc): the per-workgroup partials live in a static device array of
// this library instead of a caller-owned workspace.  Every GPU holds its own copy of the array
// at its own address, looked up once per device; host code only ever uses that address, never
// the array's name.  The kernels overwrite every partial they read back, so nothing needs
// clearing between calls; calls that overlap on one GPU share the array and race.
// The address used is the CURRENT device's (hipGetDevice): as for every launch, the current device
// must be the one that owns `stream` and the pointers -- a stream of another GPU is refused by the
// launch itself (invalid resource handle), so a foreign array address is never dereferenced.
// ---------------------------------------------------------------------------
static __device__ __align__(256) double scratch[kKlStaticRows];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
double* g_scratch_ptr[kMaxDevices];  // device address of `scratch` on each GPU, null until looked up

int kl_static_scratch(double** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return UNIRL_E_LIMIT;
  std::lock_guard<std::mutex> hold(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* addr = nullptr;
    e = hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!addr) return UNIRL_E_NULL;
    g_scratch_ptr[dev] = reinterpret_cast<double*>(addr);
  }
  *out = g_scratch_ptr[dev];
  return UNIRL_OK;
}
}  // namespace

extern "C" int unirl_gaussian_kl_mask_static(const void* p, const void* q, int dtype, const float* sigma,
                                             int64_t n_sigma, int64_t R, int64_t D, float threshold, float* kl_out,
                                             uint8_t* mask_out, void* stream) {
  if (!dtype_ok(dtype)) return UNIRL_E_DTYPE;
  if (R < 0 || D <= 0 || n_sigma <= 0) return UNIRL_E_SHAPE;
  if (R > kKlStaticRows) return UNIRL_E_LIMIT;  // the partials of every launch of the call fit the static array
  if (R == 0) return UNIRL_OK;
  if (!p || !q || !sigma || !kl_out) return UNIRL_E_NULL;
  double* partials = nullptr;
  const int rc = kl_static_scratch(&partials);
  if (rc != 0) return rc;
  return kl_mask_run(p, q, dtype, sigma, n_sigma, R, D, threshold, kl_out, mask_out, partials, kKlStaticRows,
                     (hipStream_t)stream);
}

extern "C" int unirl_flowdppo_step(const void* p, const void* q, int dtype, const float* sigma, int64_t n_sigma,
                                   int64_t R, int64_t D, const float* new_logp, const float* old_logp,
                                   const float* advantages, float threshold, float loss_scale, float* kl_out,
                                   float* loss_elem, float* grad_new, float* metrics, void* workspace,
                                   size_t workspace_bytes, void* stream) {
  if (!dtype_ok(dtype)) return UNIRL_E_DTYPE;
  if (R <= 0 || D <= 0 || n_sigma <= 0) return UNIRL_E_SHAPE;
  if (R > kDppoWaveMax) return UNIRL_E_LIMIT;
  if (!p || !q || !sigma || !kl_out || !new_logp || !old_logp || !advantages || !loss_elem || !metrics)
    return UNIRL_E_NULL;
  if (!workspace || workspace_bytes < kWorkspaceBytes) return UNIRL_E_WORKSPACE;
  const size_t sz = dtype_size(dtype);
  if (!aligned_to(p, sz) || !aligned_to(q, sz) || !aligned_to(new_logp, 4) || !aligned_to(old_logp, 4) ||
      !aligned_to(advantages, 4) || !aligned_to(kl_out, 4) || !aligned_to(loss_elem, 4) ||
      !aligned_to(grad_new, 4) || !aligned_to(metrics, 4))
    return UNIRL_E_ALIGN;
  int vec = 4;
  if (D % 4 != 0 || !aligned_to(p, 4 * sz) || !aligned_to(q, 4 * sz)) vec = 1;
  if (sz == 2 && D % 8 == 0 && aligned_to(p, 16) && aligned_to(q, 16)) vec = 8;
  const int items = (vec >= 4) ? (int)tune_int("UNIRL_KL_ITEMS", 2) : 2;
  const unsigned int nblk = kl_blocks_per_row(D / vec, items, R);
  if ((int64_t)nblk * R > kPartialCapacity) return UNIRL_E_LIMIT;
  hipStream_t st = (hipStream_t)stream;
  KlArgs K = {};
  K.p = p;
  K.q = q;
  K.sigma = sigma;
  K.n_sigma = n_sigma;
  K.D = D;
  K.threshold = threshold;
  K.kl = kl_out;
  K.partials = ws_partials(workspace);
  K.always_partials = 1;
  UNIRL_TRACE_SET(K, "kl", nblk * (unsigned int)R);
  int rc = UNIRL_E_DTYPE;
  switch (dtype) {
    case UNIRL_F32: rc = launch_kl<float>(K, R, vec, nblk, items, st); break;
    case UNIRL_BF16: rc = launch_kl<bf16_t>(K, R, vec, nblk, items, st); break;
    case UNIRL_F16: rc = launch_kl<f16_t>(K, R, vec, nblk, items, st); break;
  }
  if (rc != 0) return rc;
  DppoArgs A;
  A.nw = new_logp;
  A.od = old_logp;
  A.adv = advantages;
  A.kl = nullptr;  // read from LDS
  A.n = R;
  A.threshold = threshold;
  A.loss_elem = loss_elem;
  A.metrics = metrics;
  A.grad_new = grad_new;
  A.grad_scale = loss_scale / (float)R;  // d(loss_scale * mean(elem)) / d elem
  UNIRL_TRACE_SET(K, "dppo_finish", 1);
  hipLaunchKernelGGL(flowdppo_finish_kernel, dim3(1), dim3(kDppoFinishThreads), 0, st, K, A, nblk);
  return (int)hipGetLastError();
}

extern "C" int unirl_gaussian_kl_elem(const void* p, const void* q, int dtype, const float* sigma, int64_t n_sigma,
                                      int64_t R, int64_t D, float* out, void* stream) {
  if (!dtype_ok(dtype)) return UNIRL_E_DTYPE;
  if (R < 0 || D <= 0 || n_sigma <= 0) return UNIRL_E_SHAPE;
  if (R == 0) return UNIRL_OK;
  if (!p || !q || !sigma || !out) return UNIRL_E_NULL;
  const size_t sz = dtype_size(dtype);
  if (!aligned_to(p, sz) || !aligned_to(q, sz) || !aligned_to(out, 4)) return UNIRL_E_ALIGN;
  int vec = 4;
  if (D % 4 != 0 || !aligned_to(p, 4 * sz) || !aligned_to(q, 4 * sz) || !aligned_to(out, 16)) vec = 1;
  hipStream_t st = (hipStream_t)stream;
  const int64_t per_launch = 32768;
  for (int64_t r0 = 0; r0 < R; r0 += per_launch) {
    const int64_t nr = (R - r0 < per_launch) ? (R - r0) : per_launch;
    KlArgs A = {};
    A.p = offset_ptr(p, r0 * D, sz);
    A.q = offset_ptr(q, r0 * D, sz);
    A.sigma = sigma;
    A.n_sigma = n_sigma;
    A.row0 = r0;
    A.D = D;
    A.threshold = 0.0f;
    A.kl = nullptr;
    A.mask = nullptr;
    A.elem_out = out + r0 * D;
    A.partials = nullptr;
    int rc = UNIRL_E_DTYPE;
    switch (dtype) {
      case UNIRL_F32: rc = launch_kl_elem<float>(A, nr, vec, st); break;
      case UNIRL_BF16: rc = launch_kl_elem<bf16_t>(A, nr, vec, st); break;
      case UNIRL_F16: rc = launch_kl_elem<f16_t>(A, nr, vec, st); break;
    }
    if (rc != 0) return rc;
  }
  return UNIRL_OK;
}

extern "C" int unirl_gaussian_kl_elem_bwd(const void* p, const void* q, int dtype, const float* sigma,
                                          int64_t n_sigma, int64_t R, int64_t D, const float* g_out, void* grad_p,
                                          void* grad_q, void* stream) {
  if (!dtype_ok(dtype)) return UNIRL_E_DTYPE;
  if (R < 0 || D <= 0 || n_sigma <= 0) return UNIRL_E_SHAPE;
  if (R == 0 || (!grad_p && !grad_q)) return UNIRL_OK;
  if (!p || !q || !sigma || !g_out) return UNIRL_E_NULL;
  const size_t sz = dtype_size(dtype);
  if (!aligned_to(p, sz) || !aligned_to(q, sz) || !aligned_to(g_out, 4) || !aligned_to(grad_p, sz) ||
      !aligned_to(grad_q, sz))
    return UNIRL_E_ALIGN;
  int vec = 4;
  if (D % 4 != 0 || !aligned_to(p, 4 * sz) || !aligned_to(q, 4 * sz) || !aligned_to(g_out, 16) ||
      !aligned_to(grad_p, 4 * sz) || !aligned_to(grad_q, 4 * sz))
    vec = 1;
  hipStream_t st = (hipStream_t)stream;
  const int64_t per_launch = 32768;
  for (int64_t r0 = 0; r0 < R; r0 += per_launch) {
    const int64_t nr = (R - r0 < per_launch) ? (R - r0) : per_launch;
    KlArgs A = {};
    A.p = offset_ptr(p, r0 * D, sz);
    A.q = offset_ptr(q, r0 * D, sz);
    A.sigma = sigma;
    A.n_sigma = n_sigma;
    A.row0 = r0;
    A.D = D;
    const float* g = g_out + r0 * D;
    void* gp = const_cast<void*>(offset_ptr(grad_p, r0 * D, sz));
    void* gq = const_cast<void*>(offset_ptr(grad_q, r0 * D, sz));
    int rc = UNIRL_E_DTYPE;
    switch (dtype) {
      case UNIRL_F32: rc = launch_kl_elem_bwd<float>(A, nr, vec, g, gp, gq, st); break;
      case UNIRL_BF16: rc = launch_kl_elem_bwd<bf16_t>(A, nr, vec, g, gp, gq, st); break;
      case UNIRL_F16: rc = launch_kl_elem_bwd<f16_t>(A, nr, vec, g, gp, gq, st); break;
    }
    if (rc != 0) return rc;
  }
  return UNIRL_OK;
}
