"""Token log-prob and entropy over the vocabulary (oracle; test infrastructure only).

Log-prob follows unirl/models/qwen3/ar.py:78-85: ``lf = logits.float()/T`` (T<=0
means 1), ``lf[tok] - logsumexp(lf)``.  The reference computes no entropy; it is
defined here as ``H = logsumexp(lf) - sum softmax(lf)*lf`` with ``0 * log 0 = 0``: a logit of
-inf (a masked token) has probability 0 and contributes nothing, the convention of
``torch.distributions.Categorical``.
"""

from __future__ import annotations

import math

import torch


def token_logp(logits: torch.Tensor, ids: torch.Tensor, temperature: float = 1.0) -> torch.Tensor:
    T = float(temperature) if float(temperature) > 0.0 else 1.0
    lf = logits.float() / T
    chosen = lf.gather(-1, ids.unsqueeze(-1)).squeeze(-1)
    return chosen - torch.logsumexp(lf, dim=-1)


def token_entropy(logits: torch.Tensor, temperature: float = 1.0) -> torch.Tensor:
    """Entropy of softmax(lf), lf as in token_logp (fp32 division), evaluated in float64
    (``lse - sum p*lf`` cancels badly in fp32 when one logit dominates) and returned as fp32."""
    T = float(temperature) if float(temperature) > 0.0 else 1.0
    lf = (logits.float() / T).double()
    lse = torch.logsumexp(lf, dim=-1)
    p = torch.softmax(lf, dim=-1)
    terms = torch.where(p == 0, torch.zeros_like(p), p * lf)  # p == 0 is False for NaN: NaN rows stay NaN
    return (lse - terms.sum(dim=-1)).clamp_min(0.0).float()  # clamp keeps NaN


def token_entropy_fp32(logits: torch.Tensor, temperature: float = 1.0) -> torch.Tensor:
    """The same quantity the way eager fp32 torch would compute it (CPU baseline timing)."""
    T = float(temperature) if float(temperature) > 0.0 else 1.0
    lf = logits.float() / T
    return torch.logsumexp(lf, dim=-1) - (torch.softmax(lf, dim=-1) * lf).sum(dim=-1)


def token_logp_entropy_chunked(logits, ids, temperature=1.0, chunk=512):
    """Row-chunked evaluation to bound the fp32 transient (the reference chunks the
    vocabulary projection the same way, qwen3/ar.py:88-96)."""
    lp, ent = [], []
    for s in range(0, logits.shape[0], chunk):
        lp.append(token_logp(logits[s : s + chunk], ids[s : s + chunk], temperature))
        ent.append(token_entropy(logits[s : s + chunk], temperature))
    return torch.cat(lp), torch.cat(ent)


def token_logp_entropy_f64(row, tok, temperature=1.0):
    """One row as python floats: (logp, entropy) in float64 arithmetic."""
    T = float(temperature) if float(temperature) > 0.0 else 1.0
    lf = [float(v) / T for v in row]
    m = max(lf)
    s = sum(math.exp(v - m) for v in lf)
    lse = m + math.log(s)
    ent = lse - sum(math.exp(v - lse) * v for v in lf)
    return lf[tok] - lse, ent
