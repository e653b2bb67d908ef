"""CPU oracle for the per-sample RL-math hot path.  TEST INFRASTRUCTURE ONLY.

This package restates, in plain eager torch on the CPU (fp32, the reference's
operation order) and in float64 brute-force form, the arithmetic of the
reference functions that ``unirl_amd`` replaces.  Nothing under ``unirl_amd/``
imports it; only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` do, and only as the checker.

Parity status.  The reference ships no tests, golden vectors or fixtures for any
of these functions, and the reference package cannot be imported in the build
container (its package ``__init__`` files pull in omegaconf / ray / diffusers,
which are absent).  The formula functions are pinned by what the mathematics
fixes (``tests/test_oracle_*``) and by an independent numpy float64 restatement
(``tests/golden/vectors.npz``); the control-flow functions are pinned by outputs
of the reference itself, produced by loading the two self-contained reference
files and two extracted definitions (``tests/golden/reference_vectors.npz``):

  sigma_schedule            closed form, end points, shift=1, six known answers
  sde_step / sde_denoise    scipy.stats.norm.logpdf, torch.distributions.Normal,
                            eta=0 Euler limit, dance == flow with std=eta,
                            float64 brute force, sigma==1 branch
  token_logp / entropy      torch.log_softmax, Categorical.entropy, uniform
                            logits, shift invariance, float64 brute force
  grpo_clip_loss / drpo_loss  on-policy invariants, autograd gradcheck in
                            float64, brute force over a grid around the clip edges
  gaussian_kl / flowdppo    torch.distributions.kl_divergence, exact power-of-two
                            cases, the mask truth table
  compute_advantages        reference-run vectors (all switches, root track,
                            singleton groups), numpy mean/var closed forms
  normalize_grouped/global  reference-run vectors (trimmed statistics, empty and
                            singleton groups, clip, global std)
  gather_sde_field          reference-run vectors (values and error text),
                            dictionary lookup

Parity unpinned: the entropy, which the reference does not compute anywhere
(defined as lse - sum softmax*lf, 0*log 0 = 0).

Reference line numbers are cited per function (paths relative to the reference
tree).
"""
