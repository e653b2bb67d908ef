/*
 * unirl_hip.h -- C ABI of libunirl_hip.so: the per-sample RL-math hot path of
 * UniRL as single-pass fused HIP kernels for gfx950 (MI355X).
 *
 * The reference has no FFI layer: the path is eager torch inside plain Python
 * functions.  Each entry point below therefore names the Python function (file
 * and line in the reference tree) whose arithmetic it replaces; the Python
 * package `unirl_amd` keeps those functions' signatures and calls these entry
 * points through ctypes.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless its comment says "host";
 *   - tensors are dense and row-major; `B` is the leading (per-sample) extent
 *     and `D` the product of all remaining extents;
 *   - `dtype` arguments take UNIRL_F32 / UNIRL_BF16 / UNIRL_F16;
 *   - `stream` is a hipStream_t passed as void*; every call only enqueues work
 *     on it and returns (asynchronous, no host synchronisation);
 *   - `workspace` is caller-owned device memory of at least
 *     unirl_workspace_bytes() bytes.  A reducing entry point stores one fp64
 *     partial per workgroup there and a small second kernel, enqueued by the
 *     same call, adds them in a fixed order; nothing is carried from call to
 *     call and no initialisation is required.  Two calls that may overlap in
 *     time (different streams) need different workspaces;
 *   - the library allocates nothing, frees nothing and keeps no global state;
 *   - return value: 0 = ok, < 0 = invalid argument (UNIRL_E_*), > 0 = the
 *     hipError_t of a failed launch.  No C++ exception crosses this boundary.
 */
#ifndef UNIRL_HIP_H_
#define UNIRL_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* 2: typed gradient outputs in unirl_sde_step_logp_bwd; unirl_ratio_loss_fwd_bwd and
 * unirl_flowdppo_step added.  3: unirl_dpm2_step added.  4: unirl_gaussian_kl_mask_static
 * added.  5: unirl_sde_replay_logp, unirl_sde_replay_logp_bwd, unirl_lmhead_logp added.
 * 6: the unirl_calib_* measurement aids left the library (they live in the measurement build);
 * unirl_flowdppo_replay_step added; in-kernel sampling noise (struct unirl_rng in
 * unirl_sde_step_desc, two more arguments of unirl_sde_rollout_logp). */
#define UNIRL_ABI_VERSION 6

enum unirl_dtype { UNIRL_F32 = 0, UNIRL_BF16 = 1, UNIRL_F16 = 2 };

/* SDE transition family: unirl/sde/kernels.py:185 (flow), :239 (cps), :282 (dance). */
enum unirl_sde_kind { UNIRL_SDE_FLOW = 0, UNIRL_SDE_DANCE = 1, UNIRL_SDE_CPS = 2 };

enum unirl_status {
  UNIRL_OK = 0,
  UNIRL_E_NULL = -1,      /* a required pointer is NULL */
  UNIRL_E_SHAPE = -2,     /* negative / inconsistent extent */
  UNIRL_E_DTYPE = -3,     /* unknown dtype / kind / mode */
  UNIRL_E_WORKSPACE = -4, /* workspace missing or too small */
  UNIRL_E_ALIGN = -5,     /* pointer not aligned to its element size */
  UNIRL_E_LIMIT = -6      /* extent beyond a documented limit */
};

#define UNIRL_MAX_ROLLOUT_STEPS 64

int unirl_abi_version(void);
const char* unirl_status_string(int status);

/* Bytes of device workspace every reducing entry point expects. */
size_t unirl_workspace_bytes(void);
/* Optional: zero-fill a workspace (a fill kernel on `stream`); no entry point needs it. */
int unirl_workspace_init(void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------
 * One SDE transition + per-sample Gaussian log-prob.
 * Replaces StepStrategy.denoise -> SDEStrategy.step -> _finalize_logp
 * (unirl/sde/kernels.py:43-99, :154-177, :207-236, :255-279, :304-333).
 *
 *   noise_pred  [B,D] dtype_v          model velocity
 *   sample      [B,D] dtype_x          current latent; dtype_x is the
 *                                      "input dtype" of the round trip
 *   prev_sample [B,D] dtype_x or NULL  NULL = sampling, else replay
 *   noise       [B,D] f32 or NULL      sampling only; NULL = no noise term
 *   sigma, sigma_next  f32, one value (stride 0) or one per sample (stride 1)
 *   sigma_max_ptr      f32 device scalar or NULL (then sigma_max_val is used)
 *   eta                python-side float; eta < 1e-7 skips the log-prob
 *   prev_out    [B,D] f32 or NULL      prev_sample after the dtype round trip
 *   mean_out    [B,D] f32 or NULL      prev_sample_mean
 *   logp_out    [B]   f32 or NULL      mean over D of the element log-prob
 *                                      (logp_sum != 0: sum over D instead)
 * ---------------------------------------------------------------------- */
int unirl_sde_step_logp(const void* noise_pred, int dtype_v, const void* sample, int dtype_x,
                        const void* prev_sample, const float* noise, const float* sigma,
                        const float* sigma_next, int sigma_stride, const float* sigma_max_ptr,
                        float sigma_max_val, double eta, int kind, int64_t B, int64_t D,
                        float* prev_out, float* mean_out, float* logp_out, int logp_sum,
                        void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------
 * The same transition with strided, typed tensors, for the replay and rollout
 * loops that keep trajectories as [B, K, ...] stacks in a 16-bit dtype
 * (unirl/models/sd3/diffusion.py:366-406 writes `latents.to(trajectory_dtype)`
 * into a stack; :467-497 reads `segment.latents_at(k)` = latents[:, k] and
 * stacks log-probs [B, S'] and means `.to(trajectory_dtype)`).  Each tensor
 * names its dtype and the element distance between consecutive samples
 * (0 = D, densely packed), so `latents[:, k]` is read in place and prev, mean
 * and the log-prob column are written straight into their stacks.
 * prev_sample.ptr == NULL selects sampling; prev_sample.dtype must equal
 * sample.dtype.  Outputs are rounded to their dtype on store (prev has already
 * been rounded to sample.dtype, so storing it in that dtype is exact).
 * Other fields as in unirl_sde_step_logp. */
struct unirl_sde_tensor {
  const void* ptr;
  int dtype;             /* unirl_dtype */
  int64_t sample_stride; /* elements; 0 = D */
};
/* Sampling noise drawn inside the kernel instead of read from memory -- the reference draws it
 * inside FlowSDEStrategy.step with randn_tensor(generator=None) (unirl/sde/kernels.py:230-232),
 * i.e. from a generator no bit pattern of which has to be matched.  Counter-based: Philox-4x32-10
 * keyed by `seed`, counter {element index / 4, offset (+ the step index in a rollout)}, two
 * Box-Muller pairs per block; the draw of an element depends only on (seed, offset, step,
 * b * D + i), never on the launch shape.  The caller moves `offset` on between calls. */
struct unirl_rng {
  int enabled;
  uint64_t seed;
  uint64_t offset;
};
struct unirl_sde_step_desc {
  struct unirl_sde_tensor noise_pred, sample, prev_sample;
  const float* noise;    /* sampling only; NULL = no noise (or drawn in the kernel, see rng) */
  int64_t noise_stride;
  const float* sigma;
  const float* sigma_next;
  int sigma_stride;
  const float* sigma_max_ptr;
  float sigma_max_val;
  double eta;
  int kind;
  int64_t B, D;
  void* prev_out;        /* NULL = not wanted */
  int prev_dtype;
  int64_t prev_stride;
  void* mean_out;
  int mean_dtype;
  int64_t mean_stride;
  float* logp_out;       /* element b at logp_out[b * logp_stride] */
  int64_t logp_stride;   /* 0 = 1 */
  int logp_sum;
  struct unirl_rng rng;  /* sampling with noise == NULL: draw N(0,1) noise in the kernel */
  float* noise_out;      /* NULL, or f32 [B,D]: receives the drawn noise (one more write) */
  int64_t noise_out_stride; /* elements between samples; 0 = D */
};
int unirl_sde_step_logp_ex(const struct unirl_sde_step_desc* desc /* host */, void* workspace,
                           size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------
 * The replay of S recorded steps of every sample as ONE launch (+ its finalize)
 * over the B*S (sample, step) rows, instead of one call per step: the loop of
 * DiffusionStage.replay (unirl/models/sd3/diffusion.py:467-497, which ends in
 * stack(log_probs, dim=1) and stack(means, dim=1).to(trajectory_dtype)) for
 * velocities that are all known, e.g. from one model pass over the steps
 * stacked into the batch.  The consumer is the [B,S'] loss of
 * unirl/algorithms/flowdppo.py:286-320 / flowgrpo.py:160-193.
 *
 *   noise_pred  velocities; step j of sample b at
 *               ptr + b*sample_stride + j*noise_pred_step_stride elements
 *               (0 = dense [B,S,D]: S*D and D; [S,B,D] is sample_stride = D,
 *               step stride = B*D)
 *   latents     the trajectory stack [B,K,D] (segment.latents): slot k of
 *               sample b at ptr + b*sample_stride + k*latents_slot_stride
 *               (0 = K*slot stride and D).  Read in place, twice per row.
 *   slot_sample host int64 [S]: slot of the latent step j starts from
 *               (LatentSegment.latents_at(step), unirl/types/segments/latent.py:82-97)
 *   slot_prev   host int64 [S]: slot of the stored next latent (prev_sample)
 *   sigma, sigma_next  device f32 [S]: the step's sigma pair
 *   mean_out    [B,S,D] dense in mean_dtype, or NULL
 *   logp_out    [B,S] dense f32, or NULL (left untouched when eta < 1e-7)
 * Per row the arithmetic is unirl_sde_step_logp_ex's in replay mode, bit for
 * bit.  Limits: S <= UNIRL_MAX_ROLLOUT_STEPS, B*S <= 32768 (UNIRL_E_LIMIT).
 * ---------------------------------------------------------------------- */
struct unirl_sde_replay_desc {
  struct unirl_sde_tensor noise_pred;
  int64_t noise_pred_step_stride;
  struct unirl_sde_tensor latents;
  int64_t latents_slot_stride;
  int64_t K;
  const int64_t* slot_sample; /* host */
  const int64_t* slot_prev;   /* host */
  const float* sigma;
  const float* sigma_next;
  const float* sigma_max_ptr;
  float sigma_max_val;
  double eta;
  int kind;
  int64_t B, S, D;
  void* mean_out;
  int mean_dtype;
  float* logp_out;
  int logp_sum;
};
int unirl_sde_replay_logp(const struct unirl_sde_replay_desc* desc /* host */, void* workspace,
                          size_t workspace_bytes, void* stream);

/* Its backward with respect to the velocities (the latents are stored data) -- the gradient
 * autograd carries from `new_logp` into the model through the replay loop of
 * unirl/models/sd3/diffusion.py:467-497 and unirl/sde/kernels.py:200-228: g_logp f32 [B,S]
 * (NULL = 0), g_mean f32 [B,S,D] dense (NULL = 0; the Flow-DPPO loss sends none, its KL mask is
 * detached); grad_v in dtype_gv, laid out like noise_pred (same strides).  mean_out / logp_out
 * of the descriptor are ignored. */
int unirl_sde_replay_logp_bwd(const struct unirl_sde_replay_desc* desc /* host */, const float* g_logp,
                              const float* g_mean, void* grad_v, int dtype_gv, void* stream);

/* Backward of unirl_sde_step_logp with respect to noise_pred and sample, for
 * the autograd graph the reference builds through unirl/sde/kernels.py:225-228
 * and :200-204 (prev_sample is detached there).  Inputs as in the forward call;
 * g_logp [B] f32 (NULL = 0), g_mean [B,D] f32 (NULL = 0), g_prev [B,D] f32
 * (sampling only, NULL = 0).  Outputs grad_v / grad_x are [B,D] in the dtype
 * given for each (autograd hands a gradient back in its input's dtype, so a
 * bf16 noise_pred takes a bf16 gradient without a cast pass); either may be
 * NULL. */
int unirl_sde_step_logp_bwd(const void* noise_pred, int dtype_v, const void* sample, int dtype_x,
                            const void* prev_sample, const float* noise, const float* sigma,
                            const float* sigma_next, int sigma_stride, const float* sigma_max_ptr,
                            float sigma_max_val, double eta, int kind, int64_t B, int64_t D,
                            const float* g_logp, const float* g_mean, const float* g_prev,
                            int logp_sum, void* grad_v, int dtype_gv, void* grad_x, int dtype_gx,
                            void* stream);

/* ------------------------------------------------------------------------
 * S chained SDE transitions with the latent held in registers: the loop of
 * DiffusionStage.diffuse around StepStrategy.denoise
 * (unirl/models/sd3/diffusion.py:366-390) for velocities that are already
 * known.  Step k uses sigmas[k] -> sigmas[k+1] and etas[k].
 *
 *   x0          [B,D] dtype_x
 *   v_steps     host array of S device pointers, each [B,D] dtype_v
 *   noise_steps host array of S device pointers, each [B,D] f32 (entries may
 *               be NULL: no noise for that step, or noise drawn in the kernel
 *               when rng is given); NULL altogether with rng
 *   rng         host, NULL or the generator: a step without a noise pointer and
 *               with eta >= 1e-7 draws its noise in the kernel (step k uses
 *               offset + k); noise_out_steps: NULL, or host array of S device
 *               pointers (entries may be NULL), each f32 [B,D], receiving it
 *   sigmas      device f32 [S+1];  etas  host double [S]
 *   x_out       [B,D] f32  final latent
 *   traj_out    NULL or [S,B,D] f32: latent after every step
 *   logp_out    [B,S] f32; steps with eta < 1e-7 hold NaN
 * ---------------------------------------------------------------------- */
int unirl_sde_rollout_logp(const void* x0, int dtype_x, const void* const* v_steps, int dtype_v,
                           const float* const* noise_steps, const struct unirl_rng* rng /* host */,
                           float* const* noise_out_steps, const float* sigmas,
                           const double* etas, int S, const float* sigma_max_ptr,
                           float sigma_max_val, int kind, int64_t B, int64_t D, float* x_out,
                           float* traj_out, float* logp_out, int logp_sum, void* workspace,
                           size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------
 * One step of the deterministic DPM-Solver-2 sampler: DPM2Strategy.step ->
 * _dpm_step (unirl/sde/kernels.py:360-471).  No log-prob (the reference
 * returns None for it).  The caller keeps the solver's state -- the previous
 * step's x0 prediction -- and derives the step's scalar coefficients from the
 * sigma schedule the way the reference does (0-dim tensor arithmetic, float64
 * for the two DPM updates), rounded to f32:
 *   x0   = sample - sigma * model_output                      (:366-367)
 *   DDIM   (first / last step)  eps = (sample - one_minus_s*x0) / s;
 *                               prev = one_minus_t*x0 + sqrt_t2*eps   (:449-453)
 *   FIRST  (first order)        prev = c1*sample - c2*x0               (:391)
 *   SECOND (multistep)          D1 = inv_r0*(x0 - x0_prev);
 *                               prev = c1*sample - c2*x0 - half_c2*D1  (:416-425)
 * model_output / sample [n] in their dtypes (upcast in registers, as
 * StepStrategy.denoise's .float()); x0_prev f32 [n], SECOND only; x0_out and
 * prev_out f32 [n].  x0_out must not alias x0_prev.
 * ---------------------------------------------------------------------- */
enum unirl_dpm2_branch { UNIRL_DPM2_DDIM = 0, UNIRL_DPM2_FIRST = 1, UNIRL_DPM2_SECOND = 2 };
struct unirl_dpm2_coeffs {
  float sigma;                                 /* sigmas[step] */
  float one_minus_s, s, one_minus_t, sqrt_t2;  /* DDIM */
  float c1, c2;                                /* sigma_t/sigma_s, alpha_t*(exp(-h)-1) */
  float half_c2, inv_r0;                       /* SECOND */
};
int unirl_dpm2_step(const void* model_output, int dtype_v, const void* sample, int dtype_x,
                    const float* x0_prev, int branch, const struct unirl_dpm2_coeffs* coeffs /* host */,
                    int64_t n, float* x0_out, float* prev_out, void* stream);

/* ------------------------------------------------------------------------
 * Gaussian KL between transition means, reduced per (sample, step), and the
 * trust-region mask.  Replaces _gaussian_kl_div + the reduction and compare
 * of _flowdppo_kl_adv_loss (unirl/algorithms/flowdppo.py:43-51, :92-96).
 *
 *   p, q     [R,D] dtype       new / old means, R = B*S' rows
 *   sigma    f32 [n_sigma]     row r uses sigma[r % n_sigma]  (n_sigma = S'
 *                              for the reference's [1,S',1,1,1]; 1 = scalar)
 *   kl_out   [R] f32           mean over D of (p-q)^2 / (2 sigma^2), computed
 *                              with torch's type promotion: 16-bit inputs
 *                              subtract and square in that dtype, then divide
 *                              in f32
 *   mask_out [R] u8 or NULL    kl < threshold  (torch.bool layout)
 * ---------------------------------------------------------------------- */
int unirl_gaussian_kl_mask(const void* p, const void* q, int dtype, const float* sigma,
                           int64_t n_sigma, int64_t R, int64_t D, float threshold, float* kl_out,
                           uint8_t* mask_out, void* workspace, size_t workspace_bytes,
                           void* stream);

/* unirl_gaussian_kl_mask without a workspace and without any allocation.  It has no
 * counterpart in the reference; it exists for callers that cannot allocate device memory: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  The
 * per-workgroup partials go to a static device array inside the library (256 KiB, held by every
 * GPU the library runs on until the process ends) instead of a caller-owned workspace; its
 * address is looked up once per device, on the first call made with that device current, which
 * is best made outside a graph capture (make one call on each GPU at set-up).  The current
 * device must be the one that owns `stream`, p and q, as for any launch.  Same kernels, same
 * launch shape and bit-identical
 * results as unirl_gaussian_kl_mask.  Limit: R <= UNIRL_KL_STATIC_MAX_ROWS (UNIRL_E_LIMIT
 * beyond).  Every call on a GPU shares that GPU's array: calls that overlap in time on one GPU
 * (different streams or threads) race; calls ordered on one stream do not. */
#define UNIRL_KL_STATIC_MAX_ROWS 32768
int unirl_gaussian_kl_mask_static(const void* p, const void* q, int dtype, const float* sigma,
                                  int64_t n_sigma, int64_t R, int64_t D, float threshold,
                                  float* kl_out, uint8_t* mask_out, void* stream);

/* The [B,S'] part of _flowdppo_kl_adv_loss (unirl/algorithms/flowdppo.py:86-137) given the row
 * KLs from unirl_gaussian_kl_mask: ratio, the KL / advantage-sign masks,
 * loss_elem = where(keep, -A*ratio, 0) and the logged metrics.  All arrays are
 * f32 [n].  metrics [16] f32: 0 ratio_mean, 1 ratio_std, 2 ratio_min,
 * 3 ratio_max, 4 approx_kl, 5 kl_new_old_mean, 6 kl_new_old_max,
 * 7 kl_mask_fraction, 8 pos_rm_fraction, 9 neg_rm_fraction, 10 masked_fraction,
 * 11 unmasked_fraction, 12 mean(loss_elem).  d loss_elem / d new_logp equals
 * loss_elem itself, so no separate backward entry point exists. */
int unirl_flowdppo_loss(const float* new_logp, const float* old_logp, const float* advantages,
                        const float* kl, int64_t n, float threshold, float* loss_elem,
                        float* metrics, void* stream);

/* unirl_gaussian_kl_mask and unirl_flowdppo_loss as one call of two launches for
 * the loss step of FlowDPPO.compute_loss_and_backward
 * (unirl/algorithms/flowdppo.py:309-320):
 * the streaming KL kernel, then one workgroup that adds its partials row by
 * row and runs the [B,S'] problem on the result.  R = B*S' rows of D elements
 * in p / q; new_logp, old_logp, advantages, kl_out, loss_elem are f32 [R].
 * grad_new (NULL or f32 [R]) receives loss_scale * loss_elem / R, the gradient
 * `(loss_elem.mean() * loss_scale).backward()` leaves in new_logp.  Limit:
 * R <= 4096 (UNIRL_E_LIMIT beyond; use the two entry points above). */
int unirl_flowdppo_step(const void* p, const void* q, int dtype, const float* sigma,
                        int64_t n_sigma, int64_t R, int64_t D, const float* new_logp,
                        const float* old_logp, const float* advantages, float threshold,
                        float loss_scale, float* kl_out, float* loss_elem, float* grad_new,
                        float* metrics /* [16] f32, as unirl_flowdppo_loss */, void* workspace,
                        size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------
 * The forward of a Flow-DPPO micro-step straight from the model's velocities:
 * unirl_sde_replay_logp and unirl_flowdppo_step as ONE streaming pass plus one
 * finishing workgroup.  Replaces the replay loop of
 * unirl/models/sd3/diffusion.py:467-497 (per step: denoise with the stored
 * next latent -> log-prob and mean, stacked to [B,S'] / [B,S',...]) followed
 * by FlowDPPO.compute_loss_and_backward's loss (unirl/algorithms/flowdppo.py:
 * 286-320: gather the frozen old log-probs and means, _flowdppo_kl_adv_loss).
 * The new mean of every element is in registers while the log-prob residual is
 * summed; it is rounded to the trajectory dtype as the reference stores it
 * (`.to(trajectory_dtype)`) and the Gaussian-KL numerator against the old mean
 * is summed beside it with torch's type promotion (flowdppo.py:51), so the new
 * means are never written and never re-read: 4 reads per element and 2 launches,
 * where replay + KL take 5 reads, 1 write and 4 launches.
 *   desc        as unirl_sde_replay_logp; desc->logp_out (required) receives the
 *               new log-probs [B,S]; desc->mean_out only if the caller wants the
 *               means as well (NULL otherwise)
 *   old_means   [B,S,D] dense, in the dtype of desc->latents (the trajectory dtype)
 *   sigma_t     f32 [n_sigma_t], row r = b*S + j uses sigma_t[r % n_sigma_t]
 *               (FlowDPPO._compute_sigma_t, flowdppo.py:342-368)
 *   old_logp, advantages, kl_out, loss_elem   f32 [B*S]
 *   mask_out    NULL or u8 [B*S]: kl < threshold
 *   grad_logp   NULL or f32 [B*S]: loss_scale * loss_elem / (B*S), what
 *               `(loss_elem.mean() * loss_scale).backward()` leaves in the new
 *               log-probs; hand it to unirl_sde_replay_logp_bwd as g_logp
 *   metrics     f32 [16] as unirl_flowdppo_loss
 * Limits: B*S <= 2048 rows (UNIRL_E_LIMIT); eta >= 1e-7 (UNIRL_E_SHAPE: a
 * deterministic step has no log-prob).
 * ---------------------------------------------------------------------- */
int unirl_flowdppo_replay_step(const struct unirl_sde_replay_desc* desc /* host */,
                               const void* old_means, const float* sigma_t, int64_t n_sigma_t,
                               const float* old_logp, const float* advantages, float threshold,
                               float loss_scale, float* kl_out, uint8_t* mask_out,
                               float* loss_elem, float* grad_logp, float* metrics,
                               void* workspace, size_t workspace_bytes, void* stream);

/* Element-wise form of the same quantity (unirl/algorithms/flowdppo.py:51), f32 output [R,D]. */
int unirl_gaussian_kl_elem(const void* p, const void* q, int dtype, const float* sigma,
                           int64_t n_sigma, int64_t R, int64_t D, float* out, void* stream);

/* Its backward, for callers that differentiate _gaussian_kl_div (the reference's function is
 * plain torch and therefore differentiable; its own loss detaches the result).  g_out f32 [R,D];
 * grad_p / grad_q in the means' dtype, either may be NULL.  Follows autograd's chain through
 * the 16-bit subtraction and square (unirl/algorithms/flowdppo.py:51). */
int unirl_gaussian_kl_elem_bwd(const void* p, const void* q, int dtype, const float* sigma,
                               int64_t n_sigma, int64_t R, int64_t D, const float* g_out,
                               void* grad_p, void* grad_q, void* stream);

/* ------------------------------------------------------------------------
 * Token log-prob and entropy over the vocabulary.  Replaces _logp_chunk
 * (unirl/models/qwen3/ar.py:82-85) and the log_softmax(...).gather sites
 * (qwen3/ar.py:144-174, qwen_vl/ar.py:334-335, hunyuan_image3/ar.py:509-510).
 *
 *   logits   [rows, V] dtype, consecutive rows `row_stride` elements apart
 *   ids      [rows] int64      target token per row
 *   temperature                values <= 0 mean 1 (qwen3/ar.py:78)
 *   logp_out [rows] f32 or NULL   (x[id] - logsumexp(x)) with x = logits/T
 *   ent_out  [rows] f32 or NULL   -sum softmax(x) log_softmax(x)
 *   lse_out  [rows] f32 or NULL   logsumexp(x), kept for the backward
 * An id outside [0,V) yields NaN in logp_out for that row.
 * ---------------------------------------------------------------------- */
int unirl_token_logp_entropy(const void* logits, int dtype, int64_t rows, int64_t V,
                             int64_t row_stride, const int64_t* ids, float temperature,
                             float* logp_out, float* ent_out, float* lse_out, void* stream);

/* grad_logits[r, j] = g_logp[r] * (1[j == ids[r]] - softmax(x)[r, j]) / T in
 * `dtype`, the gradient autograd gives through unirl/models/qwen3/ar.py:83-85. */
int unirl_token_logp_bwd(const void* logits, int dtype, int64_t rows, int64_t V,
                         int64_t row_stride, const int64_t* ids, float temperature,
                         const float* lse, const float* g_logp, void* grad_logits,
                         int64_t grad_row_stride, void* stream);

/* ------------------------------------------------------------------------
 * The same three outputs straight from the hidden states: the lm_head GEMM with
 * the log-softmax statistics reduced in its epilogue, so the [rows, V] logits
 * of a replay chunk (unirl/models/qwen3/ar.py:82-99: `lm_head(h).float() / T`,
 * gather, logsumexp) are never written.  bf16 only, for a head in nn.Linear's
 * layout:
 *   hidden  bf16 [rows, K], consecutive rows ld_hidden elements apart
 *   weight  bf16 [V, K] (row v = the weights of vocabulary entry v), rows
 *           ld_weight elements apart;  bias bf16 [V] or NULL
 *   logits  = bf16(fp32 sum over K (+ bias)) -- one rounding to bf16, as a bf16
 *           Linear produces them; the statistics are taken from those values
 *   logits_out  NULL, or bf16 [rows, V] (rows ld_logits apart) to also receive
 *           the logits (validation; it costs the write this entry point exists
 *           to avoid)
 *   logp_out / ent_out / lse_out, ids, temperature: as unirl_token_logp_entropy
 * Requirements: K a multiple of 64; ld_hidden, ld_weight multiples of 8 and both
 * bases 16-byte aligned (UNIRL_E_SHAPE / UNIRL_E_ALIGN otherwise: use the
 * library GEMM and unirl_token_logp_entropy).  scratch: device memory of
 * unirl_lmhead_logp_scratch_bytes(rows, V) bytes (16 bytes per row and 128
 * columns), no initialisation needed, one call at a time.
 * Non-finite logits give NaN outputs for their row.
 * ---------------------------------------------------------------------- */
int unirl_lmhead_logp(const void* hidden, int64_t ld_hidden, const void* weight, int64_t ld_weight,
                      const void* bias, int64_t rows, int64_t V, int64_t K, const int64_t* ids,
                      float temperature, float* logp_out, float* ent_out, float* lse_out,
                      void* logits_out, int64_t ld_logits, void* scratch, size_t scratch_bytes,
                      void* stream);
/* Bytes of `scratch` unirl_lmhead_logp needs for this many rows and vocabulary entries. */
size_t unirl_lmhead_logp_scratch_bytes(int64_t rows, int64_t V);

/* ------------------------------------------------------------------------
 * dst[c][r] = src[r][c] for a [rows, cols] matrix of 2- or 4-byte elements
 * (rows ld_src elements apart; destination rows ld_dst apart).  Replaces the
 * `weight.t().contiguous()` a caller makes to hand the GEMM library the head's
 * weight as [K, V]: the gradient of the hidden states in the backward of
 * `lm_head` (unirl/models/qwen3/ar.py:82-99 under autograd), dL [rows, V] @ W
 * [V, K], runs 1.2 - 1.5 times faster on that layout.  16-byte accesses when
 * bases and leading dimensions allow them, element-wise otherwise.  Limit:
 * rows <= 4 194 240 (UNIRL_E_LIMIT).
 * ---------------------------------------------------------------------- */
int unirl_transpose_2d(const void* src, int64_t ld_src, void* dst, int64_t ld_dst, int64_t rows,
                       int64_t cols, int elem_bytes, void* stream);

/* ------------------------------------------------------------------------
 * Token-level ratio losses with every metric reduction fused in.
 * Replaces _grpo_clip_loss (unirl/algorithms/base.py:115-157), _drpo_loss
 * (unirl/algorithms/drpo.py:97-159), rollout_replay_logp_absdiff
 * (base.py:83-103), GRPO._expand_advantages_to_tokens (grpo.py:172-198) and
 * the aggregation in grpo.py:148-155 / drpo.py:318-330.
 *
 * Token layout (new_logp / old_logp are f32; n_tok = number of slots):
 *   padded  : seq_stride > 0: [n_seq, seq_stride]; `lengths` is int64 [n_seq]
 *             and row r holds lengths[r] valid tokens first
 *   packed  : seq_stride == 0: `lengths` is the int64 PREFIX SUM cu_seqlens
 *             [n_seq+1] (cu[0] = 0, cu[n_seq] = n_tok); sequence r owns tokens
 *             [cu[r], cu[r+1])
 *   flat    : lengths == NULL: one run of n_tok tokens (n_seq ignored); needs
 *             per-token advantages and token-mean aggregation
 * Advantages: adv_per_token != 0 -> one per token (same layout as the
 * log-probs); else one per sequence (requires lengths).
 * loss_mask: NULL or f32 per token, multiplied into the loss (drpo.py:319-321).
 * ---------------------------------------------------------------------- */
enum unirl_loss_kind { UNIRL_LOSS_GRPO = 0, UNIRL_LOSS_DRPO = 1 };
enum unirl_agg_mode {
  UNIRL_AGG_TOKEN_MEAN = 0,        /* sum over tokens / token count        */
  UNIRL_AGG_SEQ_MEAN_TOKEN_SUM = 1,/* mean_seq(sum_tok) / horizon           */
  UNIRL_AGG_SEQ_MEAN_TOKEN_MEAN = 2/* mean_seq(mean_tok), empty seq -> 0    */
};

/* Slots of the f32 metrics vector written by unirl_ratio_loss_fwd. */
enum unirl_metric_slot {
  UNIRL_M_LOSS = 0,           /* aggregated loss                              */
  UNIRL_M_RATIO_MEAN = 1,
  UNIRL_M_RATIO_STD = 2,      /* unbiased; 0 when fewer than two tokens       */
  UNIRL_M_RATIO_MIN = 3,
  UNIRL_M_RATIO_MAX = 4,
  UNIRL_M_CLIP_FRACTION = 5,  /* GRPO: mean(max(gt, lt))                      */
  UNIRL_M_CLIPFRAC_HI = 6,    /* GRPO clipfrac_gt_one / DRPO clipfrac_upper   */
  UNIRL_M_CLIPFRAC_LO = 7,    /* GRPO clipfrac_lt_one / DRPO clipfrac_lower   */
  UNIRL_M_APPROX_KL = 8,      /* GRPO 0.5*ld^2 ; DRPO (r-1)-ld                */
  UNIRL_M_PENALTY_MEAN = 9,   /* DRPO drpo_penalty_mean                       */
  UNIRL_M_ABSDIFF_MEAN = 10,  /* mean |new-old|                               */
  UNIRL_M_ABSDIFF_MAX = 11,
  UNIRL_M_NUM_TOKENS = 12,    /* valid-token count as f32                     */
  UNIRL_M_COUNT = 16
};

struct unirl_ratio_loss_params {
  int kind;            /* unirl_loss_kind                                     */
  int agg_mode;        /* unirl_agg_mode                                      */
  float clip_low;      /* GRPO clip_range                                     */
  float clip_high;     /* GRPO clip_range_high (= clip_low when symmetric)    */
  float drpo_epsilon;  /* DRPO epsilon                                        */
  int mu_weighted;     /* DRPO penalty weight mu = exp(old) (1) or 1 (0)      */
  float horizon;       /* UNIRL_AGG_SEQ_MEAN_TOKEN_SUM divisor                */
  int adv_per_token;
};

int unirl_ratio_loss_fwd(const float* new_logp, const float* old_logp, const float* advantages,
                         const int64_t* lengths, const float* loss_mask, int64_t n_seq,
                         int64_t seq_stride, int64_t n_tok,
                         const struct unirl_ratio_loss_params* params /* host */,
                         float* loss_per_elem /* NULL or same layout as new_logp */,
                         float* metrics /* [UNIRL_M_COUNT] f32 */, void* workspace,
                         size_t workspace_bytes, void* stream);

/* Backward of unirl_ratio_loss_fwd: what `(loss * loss_scale).backward()` leaves in new_logp
 * (unirl/algorithms/grpo.py:156, unirl/algorithms/drpo.py:331) through the token arithmetic of
 * unirl/algorithms/base.py:133-157 / unirl/algorithms/drpo.py:131-159.
 * grad_new = g_scale * w_tok * dloss/dnew, where w_tok is the aggregation
 * weight of the token (1/N, 1/(n_seq*horizon) or 1/(n_seq*len)), times
 * g_elem per token when that is not NULL (the caller reduced loss_per_elem
 * itself).  Padded slots past a sequence's length receive 0. */
int unirl_ratio_loss_bwd(const float* new_logp, const float* old_logp, const float* advantages,
                         const int64_t* lengths, const float* loss_mask, int64_t n_seq,
                         int64_t seq_stride, int64_t n_tok,
                         const struct unirl_ratio_loss_params* params /* host */,
                         const float* g_scale /* device scalar or NULL (=1) */,
                         const float* g_elem, int aggregate,
                         const float* n_valid /* device scalar: metrics[UNIRL_M_NUM_TOKENS]
                                                 of the forward; token-mean only */,
                         float* grad_new, void* stream);

/* Forward and backward of one training micro-step in a single pass over new / old:
 * the metrics of unirl_ratio_loss_fwd plus grad_new = loss_scale * w_tok * dloss/dnew,
 * i.e. what `(loss * loss_scale).backward()` leaves in new_logp.grad
 * (unirl/algorithms/grpo.py:134-160, drpo.py:310-334, flowgrpo.py:174-193).
 * n_valid: the token-mean denominator in the padded layout (every token inside
 * the lengths, masked or not) when the host knows it; < 0 lets the kernel sum
 * the lengths.  Ignored in the other layouts (n_tok).  Padded slots past a
 * sequence's length receive 0.  With n_tok == 0 both entry points write only the
 * metrics (count 0, the means NaN like torch's mean of nothing). */
int unirl_ratio_loss_fwd_bwd(const float* new_logp, const float* old_logp, const float* advantages,
                             const int64_t* lengths, const float* loss_mask, int64_t n_seq,
                             int64_t seq_stride, int64_t n_tok,
                             const struct unirl_ratio_loss_params* params /* host */,
                             float loss_scale, int64_t n_valid, float* grad_new,
                             float* metrics /* [UNIRL_M_COUNT] f32 */, void* workspace,
                             size_t workspace_bytes, void* stream);

/* out[t] = vals[r] for every token t of sequence r (packed layout, cu_seqlens
 * int64 [n_seq+1]): GRPO._expand_advantages_to_tokens
 * (unirl/algorithms/grpo.py:187-198) as one kernel. */
int unirl_expand_per_seq(const float* vals, const int64_t* cu_seqlens, int64_t n_seq,
                         int64_t n_tok, float* out, void* stream);

/* ------------------------------------------------------------------------
 * Group-normalised advantages.  Replaces RolloutTrack.compute_advantages
 * (unirl/types/rollout_resp.py:277-333) for n = n_groups * branch rewards in
 * group-by-parent order.
 *   scope_global  != 0: (r - mean_all) / (std_unbiased_all + eps)
 *   use_global_std!= 0: (r - mean_g)   / (std_unbiased_all + eps)
 *   otherwise          : (r - mean_g)   / sqrt(var_pop_g + eps)
 *   normalize == 0     : centring only
 * ---------------------------------------------------------------------- */
int unirl_group_advantages(const float* rewards, int64_t n_groups, int64_t branch, int normalize,
                           float eps, int scope_global, int use_global_std, float* adv_out,
                           void* stream);

/* Grouped normalisation over arbitrary index lists, normalize_grouped
 * (unirl/algorithms/normalizers.py:8-59).  `members` int64 concatenates the
 * groups' sample indices (each in [0,n), validated by the caller), `offsets`
 * int64 [n_groups+1] delimits them.  out must be zero-filled by the caller:
 * samples in no group keep 0.  Statistics: mean and unbiased std (+ eps) of
 * the group, of its trimmed core when trim_ratio > 0 (k = int(len*ratio)
 * members dropped from each end, only if len > 2 and 0 < 2k < len), or one
 * batch-wide unbiased std + eps when use_global_std != 0. */
int unirl_normalize_grouped(const float* rewards, int64_t n, const int64_t* members,
                            const int64_t* offsets, int64_t n_groups, float eps, float trim_ratio,
                            int use_global_std, int has_clip, float clip_max, float* out,
                            void* stream);

/* ------------------------------------------------------------------------
 * out[b, j, :] = src[b, positions[j], :] -- the copy behind gather_sde_field
 * (unirl/algorithms/base.py:70,80).  inner_bytes is the byte size of one
 * [b, s] slice; positions is a device int64 array with values in [0, S).
 * ---------------------------------------------------------------------- */
int unirl_gather_steps(const void* src, int64_t B, int64_t S, int64_t inner_bytes,
                       const int64_t* positions, int64_t n_pos, void* out, void* stream);

/* ------------------------------------------------------------------------
 * out[b, :] = cast(src[group_of[b], :]) -- the device half of the x_T noise
 * recipe (unirl/sde/noise.py:72-97, :178-187): the reference draws one fp32
 * CPU tensor per noise group, stacks one copy per SAMPLE on the host, and
 * uploads and casts the whole batch.  Here only the U unique draws cross PCIe
 * (src f32 [U, D]); this kernel replicates them to the B samples and applies
 * the final cast (round to nearest even) in the same pass.  group_of is a
 * device int64 [B] with values in [0, U).
 * ---------------------------------------------------------------------- */
int unirl_expand_groups(const float* src, int64_t U, int64_t D, const int64_t* group_of, int64_t B,
                        void* out, int out_dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* UNIRL_HIP_H_ */
