"""Loss math of the RL algorithms: GRPO / DRPO (token level), FlowGRPO / FlowDPPO (diffusion)."""

from ._fused import fused_token_loss, fused_token_loss_backward
from .base import (
    AlgorithmStepResult,
    StageAlgorithm,
    _grpo_clip_loss,
    _resolve_clip_range_from_schedule,
    gather_sde_field,
    rollout_replay_logp_absdiff,
    typed_conditions,
)
from .drpo import DRPO, DRPOConfig, _drpo_loss
from .flowdppo import FlowDPPO, FlowDPPOConfig, _flowdppo_kl_adv_loss, _gaussian_kl_div
from .flowgrpo import FlowGRPO, FlowGRPOConfig
from .grpo import GRPO, GRPOConfig
from .normalizers import normalize_global, normalize_grouped

__all__ = [
    "AlgorithmStepResult",
    "DRPO",
    "DRPOConfig",
    "FlowDPPO",
    "FlowDPPOConfig",
    "FlowGRPO",
    "FlowGRPOConfig",
    "GRPO",
    "GRPOConfig",
    "StageAlgorithm",
    "fused_token_loss",
    "fused_token_loss_backward",
    "gather_sde_field",
    "normalize_global",
    "normalize_grouped",
    "rollout_replay_logp_absdiff",
    "typed_conditions",
]
