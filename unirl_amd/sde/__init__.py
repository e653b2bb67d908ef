"""Flow-matching SDE transition kernels and the sigma schedule."""

from .kernels import (
    STRATEGIES,
    CPSSDEStrategy,
    DanceSDEStrategy,
    DPM2Strategy,
    FlowSDEStrategy,
    SDEStrategy,
    StepStrategy,
    latents_at,
    replay_slots,
    sde_rollout,
)
from .noise import generate_latents, generate_shared_noise, regen_initial_noise
from .runtime import calculate_dynamic_mu, get_sigma_schedule

__all__ = [
    "CPSSDEStrategy",
    "DPM2Strategy",
    "DanceSDEStrategy",
    "FlowSDEStrategy",
    "SDEStrategy",
    "STRATEGIES",
    "StepStrategy",
    "calculate_dynamic_mu",
    "generate_latents",
    "generate_shared_noise",
    "get_sigma_schedule",
    "latents_at",
    "regen_initial_noise",
    "replay_slots",
    "sde_rollout",
]
