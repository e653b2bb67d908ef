"""unirl_amd -- the per-sample RL-math hot path of UniRL on MI355X (gfx950).

Fused HIP kernels behind a C ABI (``include/unirl_hip.h``, built by
``python -m unirl_amd.build``) and, on top of them, Python modules that keep the
reference's call signatures:

    unirl_amd.sde          StepStrategy.denoise, Flow/Dance/CPS strategies, sigma schedule
    unirl_amd.algorithms   _grpo_clip_loss, _drpo_loss, _flowdppo_kl_adv_loss, GRPO, DRPO, ...
    unirl_amd.models       token log-prob / entropy over the vocabulary
    unirl_amd.types        group-normalised advantages
    unirl_amd.ops          tensor-level wrappers of the raw entry points

Importing the package does not load the shared library; the first kernel call does,
and raises if it has not been built.  There is no CPU implementation.
"""

__version__ = "0.1.0"

__all__ = ["__version__"]
