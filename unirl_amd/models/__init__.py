"""Model-side pieces of the hot path (the log-prob arithmetic only; no model forwards)."""

from .ar_logp import ARLogprobStep, chunked_replay_logp, token_entropy, token_logp, token_logp_entropy

__all__ = ["ARLogprobStep", "chunked_replay_logp", "token_entropy", "token_logp", "token_logp_entropy"]
