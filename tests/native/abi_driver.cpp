// A C++ program that uses the library the way a non-Python host would: hipMalloc'd buffers, the
// C ABI of include/unirl_hip.h, nothing else (no torch, no Python).  Each entry point of the hot
// path is called on small seeded inputs and checked against a float64 evaluation of the
// reference's formula written out below (file:line cited per check).  Exit status 0 = all
// checks passed; every check prints one line.  Test infrastructure, not part of the product.
//
// Build (tests/native/build.py):  hipcc --offload-arch=gfx950 -Iinclude abi_driver.cpp -L... -lunirl_hip

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

#include "unirl_hip.h"

namespace {

int g_failures = 0;

#define HIP_OK(call)                                                                  \
  do {                                                                                \
    hipError_t e_ = (call);                                                           \
    if (e_ != hipSuccess) {                                                           \
      std::printf("HIP error %d at %s:%d\n", (int)e_, __FILE__, __LINE__);           \
      std::exit(2);                                                                   \
    }                                                                                 \
  } while (0)

struct Rng {  // 64-bit LCG; uniform() in [0,1), normal() by Box-Muller
  uint64_t s;
  explicit Rng(uint64_t seed) : s(seed * 2862933555777941757ull + 3037000493ull) {}
  double uniform() {
    s = s * 6364136223846793005ull + 1442695040888963407ull;
    return (double)(s >> 11) * (1.0 / 9007199254740992.0);
  }
  double normal() {
    double u = uniform(), v = uniform();
    if (u < 1e-300) u = 1e-300;
    return std::sqrt(-2.0 * std::log(u)) * std::cos(6.283185307179586 * v);
  }
};

uint16_t to_bf16(float f) {  // round to nearest even
  uint32_t u;
  std::memcpy(&u, &f, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
float from_bf16(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}

template <typename T>
struct DevBuf {
  T* p = nullptr;
  size_t n = 0;
  explicit DevBuf(size_t count) : n(count) { HIP_OK(hipMalloc((void**)&p, (count ? count : 1) * sizeof(T))); }
  explicit DevBuf(const std::vector<T>& h) : DevBuf(h.size()) {
    if (n) HIP_OK(hipMemcpy(p, h.data(), n * sizeof(T), hipMemcpyHostToDevice));
  }
  ~DevBuf() { (void)hipFree(p); }
  std::vector<T> host() const {
    std::vector<T> h(n);
    if (n) HIP_OK(hipMemcpy(h.data(), p, n * sizeof(T), hipMemcpyDeviceToHost));
    return h;
  }
  DevBuf(const DevBuf&) = delete;
  DevBuf& operator=(const DevBuf&) = delete;
};

void expect_close(const char* what, double got, double ref, double rtol, double atol) {
  const double err = std::fabs(got - ref);
  if (!(err <= rtol * std::fabs(ref) + atol)) {
    std::printf("FAIL %s: got %.9g, expected %.9g\n", what, got, ref);
    ++g_failures;
  }
}
void expect_status(const char* what, int rc) {
  if (rc != 0) {
    std::printf("FAIL %s: status %d (%s)\n", what, rc, unirl_status_string(rc));
    ++g_failures;
  }
}

// logp = lf[id] - logsumexp(lf), lf = logits.float() / T  (unirl/models/qwen3/ar.py:82-85);
// entropy = logsumexp(lf) - sum softmax(lf) * lf.
void check_token_logp(hipStream_t st) {
  const int64_t rows = 7, V = 4099, stride = V + 5;
  const float T = 0.7f;
  Rng rng(11);
  std::vector<uint16_t> x((size_t)rows * stride);
  for (auto& v : x) v = to_bf16((float)(2.0 * rng.normal()));
  x[3 * stride + 17] = to_bf16(15.0f);
  std::vector<int64_t> ids(rows);
  for (auto& i : ids) i = (int64_t)(rng.uniform() * V);
  ids[3] = 17;
  DevBuf<uint16_t> dx(x);
  DevBuf<int64_t> dids(ids);
  DevBuf<float> dlp(rows), dent(rows), dlse(rows);
  expect_status("unirl_token_logp_entropy",
                unirl_token_logp_entropy(dx.p, UNIRL_BF16, rows, V, stride, dids.p, T, dlp.p, dent.p, dlse.p, st));
  HIP_OK(hipStreamSynchronize(st));
  const auto lp = dlp.host(), ent = dent.host(), lse = dlse.host();
  for (int64_t r = 0; r < rows; ++r) {
    double m = -1e300;
    std::vector<double> lf(V);
    for (int64_t j = 0; j < V; ++j) {
      lf[j] = (double)(from_bf16(x[r * stride + j]) / T);  // the division is fp32 in the reference
      m = std::fmax(m, lf[j]);
    }
    double s = 0.0, t = 0.0;
    for (int64_t j = 0; j < V; ++j) {
      const double e = std::exp(lf[j] - m);
      s += e;
      t += e * lf[j];
    }
    const double ref_lse = m + std::log(s);
    expect_close("token lse", lse[r], ref_lse, 1e-5, 1e-6);
    expect_close("token logp", lp[r], lf[ids[r]] - ref_lse, 1e-5, 2e-6);
    expect_close("token entropy", ent[r], ref_lse - t / s, 1e-5, 2e-6);
  }
  std::printf("token log-prob + entropy: checked %lld rows\n", (long long)rows);
}

// FlowSDEStrategy.step + compute_log_prob, sampling then replay (unirl/sde/kernels.py:207-236, :193-205, :154-177).
void check_sde_step(hipStream_t st, void* ws, size_t ws_bytes) {
  const int64_t B = 3, D = 1000;
  const double sigma = 0.84375006, sigma_next = 0.82258058, eta = 0.7, sigma_max = 0.98780483;
  Rng rng(12);
  std::vector<float> x(B * D), v(B * D), n(B * D);
  for (int64_t i = 0; i < B * D; ++i) {
    x[i] = (float)rng.normal();
    v[i] = (float)rng.normal();
    n[i] = (float)rng.normal();
  }
  const std::vector<float> sg = {(float)sigma}, sn = {(float)sigma_next};
  DevBuf<float> dx(x), dv(v), dn(n), dsg(sg), dsn(sn), dprev(B * D), dmean(B * D), dlp(B), dlp2(B);
  expect_status("unirl_sde_step_logp (sampling)",
                unirl_sde_step_logp(dv.p, UNIRL_F32, dx.p, UNIRL_F32, nullptr, dn.p, dsg.p, dsn.p, 0, nullptr,
                                    (float)sigma_max, eta, UNIRL_SDE_FLOW, B, D, dprev.p, dmean.p, dlp.p, 0, ws,
                                    ws_bytes, st));
  expect_status("unirl_sde_step_logp (replay)",
                unirl_sde_step_logp(dv.p, UNIRL_F32, dx.p, UNIRL_F32, dprev.p, nullptr, dsg.p, dsn.p, 0, nullptr,
                                    (float)sigma_max, eta, UNIRL_SDE_FLOW, B, D, nullptr, nullptr, dlp2.p, 0, ws,
                                    ws_bytes, st));
  HIP_OK(hipStreamSynchronize(st));
  const auto prev = dprev.host(), mean = dmean.host(), lp = dlp.host(), lp2 = dlp2.host();
  const double s = (double)sg[0], s1 = (double)sn[0], dt = s1 - s;
  const double stdv = std::sqrt(s / (1.0 - (s == 1.0 ? sigma_max : s))) * eta;
  const double a = 1.0 + stdv * stdv / (2.0 * s) * dt, b = 1.0 + stdv * stdv * (1.0 - s) / (2.0 * s);
  const double std_var = stdv * std::sqrt(-dt);
  for (int64_t r = 0; r < B; ++r) {
    double acc = 0.0;
    for (int64_t j = 0; j < D; ++j) {
      const int64_t i = r * D + j;
      const double m = (double)x[i] * a + (double)v[i] * b * dt;
      const double p = m + std_var * (double)n[i];
      expect_close("sde mean", mean[i], m, 2e-6, 2e-6);
      expect_close("sde prev", prev[i], p, 2e-6, 2e-6);
      const double d = (double)prev[i] - (double)mean[i];  // the log-prob sees the stored fp32 values
      acc += -(d * d) / (2.0 * std_var * std_var) - std::log(std_var) - 0.9189385332046727;
    }
    expect_close("sde log-prob (sampling)", lp[r], acc / (double)D, 2e-5, 2e-6);
    expect_close("sde log-prob (replay)", lp2[r], acc / (double)D, 2e-5, 2e-6);
  }
  std::printf("sde step + log-prob: checked %lld elements, sampling and replay\n", (long long)(B * D));
}

// _gaussian_kl_div and the mean / threshold of _flowdppo_kl_adv_loss (unirl/algorithms/flowdppo.py:43-51, :92-96):
// bf16 subtraction and square, fp32 division, mean over the row.
void check_kl(hipStream_t st, void* ws, size_t ws_bytes) {
  const int64_t R = 4, D = 2048;
  Rng rng(13);
  std::vector<uint16_t> p(R * D), q(R * D);
  for (int64_t i = 0; i < R * D; ++i) {
    const double base = rng.normal();
    p[i] = to_bf16((float)(base + 0.02 * rng.normal()));
    q[i] = to_bf16((float)(base + 0.02 * rng.normal()));
  }
  const std::vector<float> sig = {0.3f, 0.2f};
  std::vector<double> ref(R);
  for (int64_t r = 0; r < R; ++r) {
    const double den = 2.0 * (double)(sig[r % 2] * sig[r % 2]);
    double acc = 0.0;
    for (int64_t j = 0; j < D; ++j) {
      const float d = from_bf16(to_bf16(from_bf16(p[r * D + j]) - from_bf16(q[r * D + j])));
      acc += (double)from_bf16(to_bf16(d * d)) / den;
    }
    ref[r] = acc / (double)D;
  }
  const float thr = (float)(0.5 * (ref[0] + ref[1]));
  DevBuf<uint16_t> dp(p), dq(q);
  DevBuf<float> dsig(sig), dkl(R);
  DevBuf<uint8_t> dmask(R);
  expect_status("unirl_gaussian_kl_mask", unirl_gaussian_kl_mask(dp.p, dq.p, UNIRL_BF16, dsig.p, 2, R, D, thr, dkl.p,
                                                                 dmask.p, ws, ws_bytes, st));
  HIP_OK(hipStreamSynchronize(st));
  const auto kl = dkl.host();
  const auto mask = dmask.host();
  for (int64_t r = 0; r < R; ++r) {
    expect_close("gaussian kl", kl[r], ref[r], 1e-5, 1e-12);
    if (std::fabs(ref[r] - thr) > 1e-5 * thr && (int)mask[r] != (ref[r] < thr ? 1 : 0)) {
      std::printf("FAIL kl mask row %lld\n", (long long)r);
      ++g_failures;
    }
  }
  // the allocation-free entry (static scratch inside the library) gives the same bits, twice
  for (int call = 0; call < 2; ++call) {
    DevBuf<float> dkl2(R);
    DevBuf<uint8_t> dmask2(R);
    expect_status("unirl_gaussian_kl_mask_static", unirl_gaussian_kl_mask_static(dp.p, dq.p, UNIRL_BF16, dsig.p, 2, R, D,
                                                                                 thr, dkl2.p, dmask2.p, st));
    HIP_OK(hipStreamSynchronize(st));
    const auto kl2 = dkl2.host();
    const auto mask2 = dmask2.host();
    for (int64_t r = 0; r < R; ++r) {
      if (std::memcmp(&kl2[r], &kl[r], sizeof(float)) != 0 || mask2[r] != mask[r]) {
        std::printf("FAIL static-scratch kl row %lld call %d\n", (long long)r, call);
        ++g_failures;
      }
    }
  }
  std::printf("gaussian kl + mask: checked %lld rows\n", (long long)R);
}

// _grpo_clip_loss with the token-mean aggregation on a padded batch (unirl/algorithms/base.py:133-156,
// grpo.py:148-155), forward and the one-pass forward + backward.
void check_grpo(hipStream_t st, void* ws, size_t ws_bytes) {
  const int64_t n_seq = 5, L = 64;
  const double eps_lo = 0.2, eps_hi = 0.28;
  Rng rng(14);
  std::vector<float> nw(n_seq * L), od(n_seq * L), adv(n_seq);
  std::vector<int64_t> len = {64, 1, 17, 0, 40};
  for (int64_t i = 0; i < n_seq * L; ++i) {
    od[i] = (float)(-8.0 * rng.uniform());
    nw[i] = od[i] + (float)(0.3 * rng.normal());
  }
  for (auto& a : adv) a = (float)rng.normal();
  unirl_ratio_loss_params P;
  std::memset(&P, 0, sizeof(P));
  P.kind = UNIRL_LOSS_GRPO;
  P.agg_mode = UNIRL_AGG_TOKEN_MEAN;
  P.clip_low = (float)eps_lo;
  P.clip_high = (float)eps_hi;
  P.horizon = 8192.0f;
  P.adv_per_token = 0;
  DevBuf<float> dnw(nw), dod(od), dadv(adv), dmet(UNIRL_M_COUNT), dmet2(UNIRL_M_COUNT), dgrad(n_seq * L);
  DevBuf<int64_t> dlen(len);
  expect_status("unirl_ratio_loss_fwd", unirl_ratio_loss_fwd(dnw.p, dod.p, dadv.p, dlen.p, nullptr, n_seq, L, n_seq * L,
                                                             &P, nullptr, dmet.p, ws, ws_bytes, st));
  const float loss_scale = 0.5f;
  expect_status("unirl_ratio_loss_fwd_bwd",
                unirl_ratio_loss_fwd_bwd(dnw.p, dod.p, dadv.p, dlen.p, nullptr, n_seq, L, n_seq * L, &P, loss_scale, -1,
                                         dgrad.p, dmet2.p, ws, ws_bytes, st));
  HIP_OK(hipStreamSynchronize(st));
  const auto met = dmet.host(), met2 = dmet2.host(), grad = dgrad.host();
  const double lo = (double)(float)(1.0 - eps_lo), hi = (double)(float)(1.0 + eps_hi);
  double N = 0.0, loss = 0.0, rsum = 0.0, kl = 0.0, clip = 0.0;
  std::vector<double> gref(n_seq * L, 0.0);
  for (int64_t r = 0; r < n_seq; ++r) N += (double)len[r];
  for (int64_t r = 0; r < n_seq; ++r) {
    for (int64_t j = 0; j < len[r]; ++j) {
      const int64_t i = r * L + j;
      const double ld = (double)(nw[i] - od[i]), ratio = std::exp(ld), A = (double)adv[r];
      const double u = -A * ratio, c = -A * std::fmin(std::fmax(ratio, lo), hi);
      loss += std::fmax(u, c);
      rsum += ratio;
      kl += 0.5 * ld * ld;
      clip += (ratio - 1.0 > eps_hi || 1.0 - ratio > eps_lo) ? 1.0 : 0.0;
      const bool inside = ratio >= lo && ratio <= hi;
      gref[i] = (u >= c ? u : (inside ? c : 0.0)) * (double)loss_scale / N;  // ties do not occur on these inputs
    }
  }
  expect_close("grpo loss", met[UNIRL_M_LOSS], loss / N, 2e-5, 1e-6);
  expect_close("grpo ratio_mean", met[UNIRL_M_RATIO_MEAN], rsum / N, 1e-5, 0);
  expect_close("grpo approx_kl", met[UNIRL_M_APPROX_KL], kl / N, 2e-5, 1e-9);
  expect_close("grpo clip_fraction", met[UNIRL_M_CLIP_FRACTION], clip / N, 0, 1.5 / N);
  expect_close("grpo token count", met[UNIRL_M_NUM_TOKENS], N, 0, 0);
  for (int k = 0; k < UNIRL_M_COUNT; ++k)
    if (k <= UNIRL_M_NUM_TOKENS) expect_close("one-pass metrics equal the forward's", met2[k], met[k], 1e-6, 1e-9);
  for (int64_t i = 0; i < n_seq * L; ++i) expect_close("grpo grad_new", grad[i], gref[i], 3e-5, 1e-9);
  std::printf("grpo clipped-ratio loss: checked metrics and %lld gradients\n", (long long)(n_seq * L));
}

// RolloutTrack.compute_advantages (unirl/types/rollout_resp.py:314-333): (r - mean_g) / sqrt(var_pop_g + eps).
void check_advantages(hipStream_t st) {
  const int64_t G = 6, b = 5;
  Rng rng(15);
  std::vector<float> r(G * b);
  for (auto& v : r) v = rng.uniform() < 0.5 ? 0.0f : 1.0f;
  for (int64_t j = 0; j < b; ++j) r[2 * b + j] = 1.0f;  // an all-equal group: exactly 0
  DevBuf<float> dr(r), dout(G * b);
  expect_status("unirl_group_advantages", unirl_group_advantages(dr.p, G, b, 1, 1e-8f, 0, 0, dout.p, st));
  HIP_OK(hipStreamSynchronize(st));
  const auto out = dout.host();
  for (int64_t g = 0; g < G; ++g) {
    double m = 0.0, var = 0.0;
    for (int64_t j = 0; j < b; ++j) m += (double)r[g * b + j];
    m /= (double)b;
    for (int64_t j = 0; j < b; ++j) var += ((double)r[g * b + j] - m) * ((double)r[g * b + j] - m);
    var /= (double)b;
    for (int64_t j = 0; j < b; ++j)
      expect_close("group advantage", out[g * b + j], ((double)r[g * b + j] - m) / std::sqrt(var + 1e-8), 2e-5, 1e-6);
  }
  std::printf("group advantages: checked %lld rewards\n", (long long)(G * b));
}

// The replay loop of a diffusion stage as one call (unirl/models/sd3/diffusion.py:467-497): every
// (sample, step) transition reads its latent and its stored next latent from the trajectory stack.
// Checked against the single-step entry point called once per step on copies of the slots.
void check_sde_replay(hipStream_t st, void* ws, size_t ws_bytes) {
  const int64_t B = 2, K = 4, S = 2, D = 520;
  const double eta = 0.7, sigma_max = 0.98780483;
  Rng rng(15);
  std::vector<float> stack(B * K * D), v(B * S * D);
  for (auto& e : stack) e = (float)rng.normal();
  for (auto& e : v) e = (float)rng.normal();
  const std::vector<float> sg = {0.84375006f, 0.5f}, sn = {0.82258058f, 0.4f};
  const int64_t slot_x[2] = {2, 0}, slot_p[2] = {3, 1};
  DevBuf<float> dstack(stack), dv(v), dsg(sg), dsn(sn), dmean(B * S * D), dlp(B * S);
  unirl_sde_replay_desc d;
  std::memset(&d, 0, sizeof(d));
  d.noise_pred = {dv.p, UNIRL_F32, S * D};
  d.noise_pred_step_stride = D;
  d.latents = {dstack.p, UNIRL_F32, K * D};
  d.latents_slot_stride = D;
  d.K = K;
  d.slot_sample = slot_x;
  d.slot_prev = slot_p;
  d.sigma = dsg.p;
  d.sigma_next = dsn.p;
  d.sigma_max_ptr = nullptr;
  d.sigma_max_val = (float)sigma_max;
  d.eta = eta;
  d.kind = UNIRL_SDE_FLOW;
  d.B = B;
  d.S = S;
  d.D = D;
  d.mean_out = dmean.p;
  d.mean_dtype = UNIRL_F32;
  d.logp_out = dlp.p;
  d.logp_sum = 0;
  expect_status("unirl_sde_replay_logp", unirl_sde_replay_logp(&d, ws, ws_bytes, st));
  HIP_OK(hipStreamSynchronize(st));
  const auto mean = dmean.host(), lp = dlp.host();
  for (int64_t j = 0; j < S; ++j) {
    // the same step through the single-step entry point, on dense copies of the two slots
    std::vector<float> x(B * D), prev(B * D), vj(B * D);
    for (int64_t b = 0; b < B; ++b)
      for (int64_t i = 0; i < D; ++i) {
        x[b * D + i] = stack[(b * K + slot_x[j]) * D + i];
        prev[b * D + i] = stack[(b * K + slot_p[j]) * D + i];
        vj[b * D + i] = v[(b * S + j) * D + i];
      }
    DevBuf<float> dx(x), dprev(prev), dvj(vj), dm1(B * D), dl1(B);
    expect_status("unirl_sde_step_logp (one step of the replay)",
                  unirl_sde_step_logp(dvj.p, UNIRL_F32, dx.p, UNIRL_F32, dprev.p, nullptr, dsg.p + j, dsn.p + j, 0,
                                      nullptr, (float)sigma_max, eta, UNIRL_SDE_FLOW, B, D, nullptr, dm1.p, dl1.p, 0,
                                      ws, ws_bytes, st));
    HIP_OK(hipStreamSynchronize(st));
    const auto m1 = dm1.host(), l1 = dl1.host();
    for (int64_t b = 0; b < B; ++b) {
      expect_close("replay log-prob vs single step", lp[b * S + j], l1[b], 1e-6, 1e-7);
      for (int64_t i = 0; i < D; ++i)
        if (mean[(b * S + j) * D + i] != m1[b * D + i]) {
          std::printf("FAIL replay mean differs from the single step at (%lld,%lld,%lld)\n", (long long)b, (long long)j,
                      (long long)i);
          ++g_failures;
          break;
        }
    }
  }
  std::printf("batched replay: %lld x %lld transitions equal the single-step calls\n", (long long)B, (long long)S);
}

// The Flow-DPPO forward straight from the velocities (unirl/models/sd3/diffusion.py:467-497 followed by
// unirl/algorithms/flowdppo.py:43-51,86-137): the frozen policy's log-probs and means come from one replay
// call, the new policy's from the fused entry point, and the KL rows, masks, loss elements and gradient are
// checked against a float64 evaluation of the reference's formulas on the means the unfused replay writes.
void check_flowdppo_replay(hipStream_t st, void* ws, size_t ws_bytes) {
  const int64_t B = 3, K = 4, S = 2, D = 520, R = B * S;
  const double eta = 0.7, sigma_max = 0.98780483;
  Rng rng(16);
  std::vector<float> stack(B * K * D), v_old(B * S * D), v_new(B * S * D), adv(R);
  for (auto& e : stack) e = (float)rng.normal();
  for (auto& e : v_old) e = (float)rng.normal();
  for (int64_t r = 0; r < R; ++r) {
    const double bump = 0.002 + 0.03 * rng.uniform();  // the policy has moved by a different amount per row
    for (int64_t i = 0; i < D; ++i) v_new[r * D + i] = v_old[r * D + i] + (float)(bump * rng.normal());
    adv[r] = (float)rng.normal();
  }
  const std::vector<float> sg = {0.84375006f, 0.5f}, sn = {0.82258058f, 0.4f}, sig_t = {0.31f, 0.22f};
  const int64_t slot_x[2] = {2, 0}, slot_p[2] = {3, 1};
  DevBuf<float> dstack(stack), dvo(v_old), dvn(v_new), dsg(sg), dsn(sn), dst(sig_t), dadv(adv);
  DevBuf<float> old_mean(R * D), old_lp(R), new_mean(R * D), new_lp(R), lp_f(R), kl(R), elem(R), grad(R), met(16);
  DevBuf<uint8_t> mask(R);
  unirl_sde_replay_desc d;
  std::memset(&d, 0, sizeof(d));
  d.noise_pred = {dvo.p, UNIRL_F32, S * D};
  d.noise_pred_step_stride = D;
  d.latents = {dstack.p, UNIRL_F32, K * D};
  d.latents_slot_stride = D;
  d.K = K;
  d.slot_sample = slot_x;
  d.slot_prev = slot_p;
  d.sigma = dsg.p;
  d.sigma_next = dsn.p;
  d.sigma_max_val = (float)sigma_max;
  d.eta = eta;
  d.kind = UNIRL_SDE_FLOW;
  d.B = B;
  d.S = S;
  d.D = D;
  d.mean_dtype = UNIRL_F32;
  d.mean_out = old_mean.p;
  d.logp_out = old_lp.p;
  expect_status("unirl_sde_replay_logp (frozen policy)", unirl_sde_replay_logp(&d, ws, ws_bytes, st));
  d.noise_pred.ptr = dvn.p;
  d.mean_out = new_mean.p;
  d.logp_out = new_lp.p;
  expect_status("unirl_sde_replay_logp (new policy)", unirl_sde_replay_logp(&d, ws, ws_bytes, st));
  HIP_OK(hipStreamSynchronize(st));
  const auto om = old_mean.host(), nm = new_mean.host(), olp = old_lp.host(), nlp = new_lp.host();
  // float64 KL rows, and a threshold halfway between two of them so that both mask values occur
  std::vector<double> kl_ref(R);
  for (int64_t r = 0; r < R; ++r) {
    double q = 0.0;
    for (int64_t i = 0; i < D; ++i) {
      const double df = (double)nm[r * D + i] - (double)om[r * D + i];
      q += df * df;
    }
    const double s_t = sig_t[r % S];
    kl_ref[r] = q / (2.0 * s_t * s_t) / (double)D;
  }
  std::vector<double> sorted = kl_ref;
  std::sort(sorted.begin(), sorted.end());
  const float thr = (float)(0.5 * (sorted[R / 2 - 1] + sorted[R / 2]));
  const float loss_scale = 0.37f;
  d.mean_out = nullptr;  // the new means are not wanted: nothing but the partials is written
  d.logp_out = lp_f.p;
  expect_status("unirl_flowdppo_replay_step",
                unirl_flowdppo_replay_step(&d, old_mean.p, dst.p, S, old_lp.p, dadv.p, thr, loss_scale, kl.p, mask.p, elem.p,
                                           grad.p, met.p, ws, ws_bytes, st));
  HIP_OK(hipStreamSynchronize(st));
  const auto lpf = lp_f.host(), klg = kl.host(), el = elem.host(), gr = grad.host(), mt = met.host();
  const auto mk = mask.host();
  int kept = 0, low = 0;
  for (int64_t r = 0; r < R; ++r) {
    expect_close("fused step: new log-prob vs the replay's", lpf[r], nlp[r], 1e-6, 1e-7);
    expect_close("fused step: KL row", klg[r], kl_ref[r], 1e-5, 1e-12);
    const bool low_kl = kl_ref[r] < (double)thr;
    if ((mk[r] != 0) != low_kl) {
      std::printf("FAIL fused step: mask of row %lld\n", (long long)r);
      ++g_failures;
    }
    const double ratio = std::exp((double)nlp[r] - (double)olp[r]);
    const bool rm = !low_kl && ((ratio > 1.0 && adv[r] > 0.0f) || (ratio < 1.0 && adv[r] < 0.0f));
    const double loss = rm ? 0.0 : -(double)adv[r] * ratio;
    // a log-prob of magnitude L carries fp32 rounding of 6e-8 L, which the exponential turns into that much
    // relative error of the ratio
    const double tol = 1e-5 + 2e-7 * std::fabs((double)nlp[r]);
    expect_close("fused step: loss element", el[r], loss, tol, 1e-9);
    expect_close("fused step: gradient", gr[r], (double)loss_scale * loss / (double)R, tol, 1e-10);
    kept += rm ? 0 : 1;
    low += low_kl ? 1 : 0;
  }
  expect_close("fused step: kl_mask_fraction", mt[7], 1.0 - (double)low / (double)R, 1e-6, 1e-7);
  expect_close("fused step: unmasked_fraction", mt[11], (double)kept / (double)R, 1e-6, 1e-7);
  std::printf("fused Flow-DPPO replay step: %lld rows, %d below the KL threshold, %d kept\n", (long long)R, low, kept);
}

// Sampling noise drawn inside the step (the reference draws it inside FlowSDEStrategy.step,
// unirl/sde/kernels.py:219-233): the drawn noise, stored on request, fed back as a given noise tensor must
// reproduce the step bit for bit; the same (seed, offset) must give the same draw and another offset another;
// and the draw must look standard normal.
void check_sde_rng(hipStream_t st, void* ws, size_t ws_bytes) {
  const int64_t B = 4, D = 4096;
  Rng rng(17);
  std::vector<float> x(B * D), v(B * D);
  for (auto& e : x) e = (float)rng.normal();
  for (auto& e : v) e = (float)rng.normal();
  const std::vector<float> sg = {0.84375006f}, sn = {0.82258058f};
  DevBuf<float> dx(x), dv(v), dsg(sg), dsn(sn), prev_a(B * D), prev_b(B * D), nz_a(B * D), nz_b(B * D), nz_c(B * D), lp_a(B),
      lp_b(B);
  unirl_sde_step_desc d;
  std::memset(&d, 0, sizeof(d));
  d.noise_pred = {dv.p, UNIRL_F32, 0};
  d.sample = {dx.p, UNIRL_F32, 0};
  d.prev_sample = {nullptr, UNIRL_F32, 0};
  d.sigma = dsg.p;
  d.sigma_next = dsn.p;
  d.sigma_max_val = 0.98780483f;
  d.eta = 0.7;
  d.kind = UNIRL_SDE_FLOW;
  d.B = B;
  d.D = D;
  d.prev_dtype = UNIRL_F32;
  d.prev_out = prev_a.p;
  d.logp_out = lp_a.p;
  d.rng.enabled = 1;
  d.rng.seed = 20241125ull;
  d.rng.offset = 40ull;
  d.noise_out = nz_a.p;
  expect_status("unirl_sde_step_logp_ex (noise drawn in the kernel)", unirl_sde_step_logp_ex(&d, ws, ws_bytes, st));
  d.prev_out = nullptr;
  d.logp_out = nullptr;
  d.noise_out = nz_b.p;
  expect_status("unirl_sde_step_logp_ex (same seed and offset)", unirl_sde_step_logp_ex(&d, ws, ws_bytes, st));
  d.rng.offset = 41ull;
  d.noise_out = nz_c.p;
  expect_status("unirl_sde_step_logp_ex (next offset)", unirl_sde_step_logp_ex(&d, ws, ws_bytes, st));
  // the same step with the drawn noise handed over as a tensor
  d.rng.enabled = 0;
  d.noise = nz_a.p;
  d.noise_out = nullptr;
  d.prev_out = prev_b.p;
  d.logp_out = lp_b.p;
  expect_status("unirl_sde_step_logp_ex (given noise)", unirl_sde_step_logp_ex(&d, ws, ws_bytes, st));
  HIP_OK(hipStreamSynchronize(st));
  const auto na = nz_a.host(), nb = nz_b.host(), nc = nz_c.host(), pa = prev_a.host(), pb = prev_b.host();
  const auto la = lp_a.host(), lb = lp_b.host();
  if (std::memcmp(na.data(), nb.data(), na.size() * 4) != 0) {
    std::printf("FAIL drawn noise is not a function of (seed, offset)\n");
    ++g_failures;
  }
  if (std::memcmp(na.data(), nc.data(), na.size() * 4) == 0) {
    std::printf("FAIL another offset gave the same noise\n");
    ++g_failures;
  }
  if (std::memcmp(pa.data(), pb.data(), pa.size() * 4) != 0) {
    std::printf("FAIL the step from drawn noise differs from the step from the same noise given\n");
    ++g_failures;
  }
  for (int64_t b = 0; b < B; ++b) expect_close("log-prob from drawn noise vs given noise", la[b], lb[b], 1e-6, 1e-7);
  double m1 = 0.0, m2 = 0.0, cross = 0.0;
  const double n = (double)na.size();
  for (size_t i = 0; i < na.size(); ++i) {
    m1 += na[i];
    m2 += (double)na[i] * na[i];
    cross += (double)na[i] * nc[i];
  }
  const double se = 1.0 / std::sqrt(n);
  expect_close("drawn noise: mean", m1 / n, 0.0, 0.0, 5.0 * se);
  expect_close("drawn noise: variance", m2 / n, 1.0, 0.0, 5.0 * std::sqrt(2.0) * se);
  expect_close("drawn noise: correlation between two offsets", cross / n, 0.0, 0.0, 5.0 * se);
  std::printf("in-kernel noise: %lld draws reproducible, standard normal, step equal to the step from the same noise\n",
              (long long)na.size());
}

// lm_head + log-softmax with the logits never written (unirl/models/qwen3/ar.py:82-99), and the
// transposed copy of the weight used by its backward: against a float64 product of the same bf16
// operands rounded to bf16 (a logit one bf16 ulp off moves a log-prob by that ulp at most).
void check_lmhead(hipStream_t st) {
  const int64_t rows = 70, K = 128, V = 300;
  Rng rng(16);
  std::vector<uint16_t> h(rows * K), w(V * K);
  for (auto& e : h) e = to_bf16((float)rng.normal());
  for (auto& e : w) e = to_bf16((float)(0.2 * rng.normal()));
  std::vector<int64_t> ids(rows);
  for (auto& e : ids) e = (int64_t)(rng.uniform() * (double)V) % V;
  const float T = 0.8f;
  DevBuf<uint16_t> dh(h), dw(w), dwt(V * K);
  DevBuf<int64_t> dids(ids);
  DevBuf<float> dlp(rows), dent(rows), dlse(rows);
  const size_t sb = unirl_lmhead_logp_scratch_bytes(rows, V);
  DevBuf<unsigned char> scratch(sb);
  expect_status("unirl_lmhead_logp", unirl_lmhead_logp(dh.p, K, dw.p, K, nullptr, rows, V, K, dids.p, T, dlp.p, dent.p,
                                                       dlse.p, nullptr, 0, scratch.p, sb, st));
  expect_status("unirl_transpose_2d", unirl_transpose_2d(dw.p, K, dwt.p, V, V, K, 2, st));
  HIP_OK(hipStreamSynchronize(st));
  const auto lp = dlp.host(), ent = dent.host(), lse = dlse.host();
  const auto wt = dwt.host();
  for (int64_t v = 0; v < V; ++v)
    for (int64_t k = 0; k < K; ++k)
      if (wt[k * V + v] != w[v * K + k]) {
        std::printf("FAIL transpose at (%lld,%lld)\n", (long long)v, (long long)k);
        ++g_failures;
        v = V;
        break;
      }
  for (int64_t r = 0; r < rows; ++r) {
    std::vector<double> x(V);
    double m = -1e300;
    for (int64_t v = 0; v < V; ++v) {
      double acc = 0.0;
      for (int64_t k = 0; k < K; ++k) acc += (double)from_bf16(h[r * K + k]) * (double)from_bf16(w[v * K + k]);
      x[v] = (double)from_bf16(to_bf16((float)acc)) / (double)T;
      m = x[v] > m ? x[v] : m;
    }
    double sum = 0.0, tsum = 0.0;
    for (int64_t v = 0; v < V; ++v) {
      const double e = std::exp(x[v] - m);
      sum += e;
      tsum += e * x[v];
    }
    const double ref_lse = m + std::log(sum);
    expect_close("lm_head log-sum-exp", lse[r], ref_lse, 2e-3, 2e-3);
    expect_close("lm_head log-prob", lp[r], x[ids[r]] - ref_lse, 2e-3, 2.5e-2);  // + one bf16 ulp of a logit of <= 4
    expect_close("lm_head entropy", ent[r], ref_lse - tsum / sum, 2e-3, 2e-3);
  }
  std::printf("fused lm_head: checked %lld rows of %lld logits; transpose %lld x %lld exact\n", (long long)rows,
              (long long)V, (long long)V, (long long)K);
}

}  // namespace

int main() {
  int n_dev = 0;
  if (hipGetDeviceCount(&n_dev) != hipSuccess || n_dev < 1) {
    std::printf("no HIP device\n");
    return 3;
  }
  HIP_OK(hipSetDevice(0));
  if (unirl_abi_version() != UNIRL_ABI_VERSION) {
    std::printf("library ABI %d, header ABI %d\n", unirl_abi_version(), UNIRL_ABI_VERSION);
    return 4;
  }
  hipStream_t st;
  HIP_OK(hipStreamCreate(&st));
  const size_t ws_bytes = unirl_workspace_bytes();
  void* ws = nullptr;
  HIP_OK(hipMalloc(&ws, ws_bytes));
  check_token_logp(st);
  check_sde_step(st, ws, ws_bytes);
  check_kl(st, ws, ws_bytes);
  check_grpo(st, ws, ws_bytes);
  check_advantages(st);
  check_sde_replay(st, ws, ws_bytes);
  check_flowdppo_replay(st, ws, ws_bytes);
  check_sde_rng(st, ws, ws_bytes);
  check_lmhead(st);
  HIP_OK(hipStreamSynchronize(st));
  HIP_OK(hipFree(ws));
  HIP_OK(hipStreamDestroy(st));
  std::printf(g_failures ? "FAILED: %d checks\n" : "all checks passed\n", g_failures);
  return g_failures ? 1 : 0;
}
