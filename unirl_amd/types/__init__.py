"""Layout contracts shared with the reference's rollout types."""

from .rollout_resp import RolloutTrack, compute_advantages

__all__ = ["RolloutTrack", "compute_advantages"]
