"""Token log-probs (and entropy) from logits, fused.

Drop-in for the log-prob sites of the reference's AR stages:

* replay -- ``_logp_chunk`` inside ``_replay_aware_forward``
  (``unirl/models/qwen3/ar.py:78-99``): ``lf = lm_head(h).float() / T``,
  ``lf[tok] - logsumexp(lf)``, chunked over the response and checkpointed;
* sampling -- the behaviour log-prob of ``Qwen3ARStep.step``
  (``unirl/models/qwen3/ar.py:138-175``; same arithmetic in ``qwen_vl/ar.py:334-335``
  and ``hunyuan_image3/ar.py:509-510``).

The reference materialises ``.float()`` and ``/ T`` copies of the ``[B, chunk, V]``
logits and reads them again for the gather and the logsumexp; here the logits are
read once in their own dtype and only ``[B, chunk]`` floats are written.  Under
autograd the backward is one more pass that writes ``(onehot - softmax) * g / T``
in the logits' dtype, so the chunk needs no activation checkpoint of an fp32 copy.
"""

from __future__ import annotations

from typing import Callable, Dict, List, Optional, Tuple

import torch
import torch.nn.functional as F

from .. import ops


def _is_plain_linear(lm_head) -> bool:
    """True for an ``nn.Linear`` proper whose output nobody else can be holding: not a subclass
    (a quantised or custom Linear's autograd may save its output) and no forward hook (a hook
    sees, and may keep, the output).  Only then may a gradient be written over the logits."""
    from torch.nn.modules import module as _m

    return (
        type(lm_head) is torch.nn.Linear
        and not lm_head._forward_hooks
        and not lm_head._forward_hooks_with_kwargs
        and not _m._global_forward_hooks
    )


class _TokenLogpFn(torch.autograd.Function):
    """Log-prob (differentiable) and, on request, entropy (detached) from one pass over the logits."""

    @staticmethod
    def forward(ctx, logits: torch.Tensor, tokens: torch.Tensor, temperature: float, want_entropy: bool,
                consume: bool = False):
        logp, ent, lse = ops.token_logp_entropy(
            logits, tokens, temperature, want_logp=True, want_entropy=want_entropy, want_lse=True
        )
        ctx.save_for_backward(logits, tokens, lse)
        ctx.temperature = temperature
        # `consume`: the caller owns the logits and nobody reads them after this node's backward, so
        # the gradient may overwrite them (no second [rows, V] buffer)
        ctx.consume = bool(consume) and logits.is_contiguous() and logits.dtype in _KERNEL_DTYPES
        ctx.consumed = False
        if not want_entropy:
            return logp
        ctx.mark_non_differentiable(ent)
        return logp, ent

    @staticmethod
    def backward(ctx, g_logp, *_g_entropy):
        if ctx.consumed:
            raise RuntimeError(
                "the logits of this replay were overwritten by their gradient in the first backward; "
                "a second backward through the same graph needs chunked_replay_logp(..., keep_logits=False)"
            )
        logits, tokens, lse = ctx.saved_tensors
        ctx.consumed = ctx.consume
        grad = ops.token_logp_bwd(logits, tokens, ctx.temperature, lse, g_logp, in_place=ctx.consume)
        if ctx.consume:
            # the kernel wrote through a raw pointer: tell autograd, so that anything else that saved
            # these logits fails loudly instead of reading their gradient
            torch.autograd.graph.increment_version(logits)
        return grad, None, None, None, None


class _RecomputedChunkFn(torch.autograd.Function):
    """Log-probs of one chunk whose ``[B, chunk, V]`` logits are not kept for the backward.

    The reference wraps each chunk in ``torch.utils.checkpoint`` (``qwen3/ar.py:93-96``): the
    backward runs ``lm_head`` again and then the whole log-softmax forward and backward.  Here
    the forward keeps the per-token log-sum-exp (4 bytes a token), so the backward runs
    ``lm_head`` again and goes straight to the gradient kernel -- the recomputed logits are
    read once instead of twice -- and, for a plain ``nn.Linear`` head, the gradient overwrites
    the logits buffer.
    """

    @staticmethod
    def forward(ctx, hidden: torch.Tensor, tokens: torch.Tensor, lm_head, temperature: float, fused_head: bool, *params):
        del params  # listed only so autograd sees the head's parameters as inputs of this node
        ctx.autocast = (torch.is_autocast_enabled("cuda"), torch.get_autocast_dtype("cuda"))
        with torch.no_grad():
            if fused_head:
                # the head's GEMM with the log-softmax statistics in its epilogue: no logits at all
                logp, _, lse, _ = ops.lmhead_logp(hidden, lm_head.weight, lm_head.bias, tokens, temperature,
                                                  want_lse=True)
            else:
                logits = lm_head(hidden)
                logp, _, lse = ops.token_logp_entropy(
                    logits, tokens, temperature, want_logp=True, want_entropy=False, want_lse=True
                )
        ctx.save_for_backward(hidden, tokens, lse)
        ctx.lm_head, ctx.temperature = lm_head, temperature
        return logp

    @staticmethod
    def backward(ctx, g_logp):
        hidden, tokens, lse = ctx.saved_tensors
        enabled, dtype = ctx.autocast
        h = hidden.detach().requires_grad_(hidden.requires_grad)
        with torch.enable_grad(), torch.autocast("cuda", dtype=dtype, enabled=enabled):
            logits = ctx.lm_head(h)
        plain = _is_plain_linear(ctx.lm_head) and logits.is_contiguous()
        d_logits = ops.token_logp_bwd(
            logits.detach(), tokens, ctx.temperature, lse, g_logp, in_place=plain and logits.dtype in _KERNEL_DTYPES
        )
        # parameter gradients accumulate into .grad here, as under a re-entrant checkpoint
        torch.autograd.backward(logits, d_logits)
        n_params = len(ctx.needs_input_grad) - 5
        return (h.grad, None, None, None, None) + (None,) * n_params


_KERNEL_DTYPES = (torch.float32, torch.bfloat16, torch.float16)

def transpose_weight(weight: torch.Tensor) -> torch.Tensor:
    """A contiguous ``[K, V]`` copy of a head's ``[V, K]`` weight (``unirl_transpose_2d``: 0.3 ms for
    the Qwen3-4B head where torch's strided copy takes 6 ms)."""
    if weight.dim() == 2 and weight.is_cuda and weight.element_size() in (2, 4) and weight.stride(1) == 1:
        return ops.transpose_2d(weight)
    return weight.detach().t().contiguous()


class _TransposedOnce:
    """The ``[K, V]`` copy of the head's weight for ONE replay.

    The gradient of the hidden states is ``dL [rows, V] @ W [V, K]``, a product with both operands
    read across their rows; the GEMM library runs it at 0.65 - 0.75 of the speed it reaches on
    ``dL @ Wt.T`` with ``Wt`` stored ``[K, V]`` (measured on the MI355X, Qwen3-4B head: 7.3 against
    4.8 ms at 8192 rows, 1.84 against 1.51 ms at 2048).  The copy is made in the backward, by the
    first chunk that needs it, from the weight's values at that moment, shared by the replay's
    other chunks and dropped with the replay's graph.  Nothing outlives the replay, so no write
    to the weight can leave a stale copy behind -- in particular not one made through ``.data``
    (``p.data.copy_(...)``: EMA, weight sync and parameter injection all write that way), which
    changes neither the tensor's version counter nor its address and therefore cannot be seen by
    a cache that is keyed on them.  The price is one transposition per replay (0.3 ms against a
    backward of 11 ms at 8192 rows) instead of one per optimizer step.  A second backward through
    a retained graph remakes the copy if the version counter has moved in between."""

    __slots__ = ("weight", "version", "copy")

    def __init__(self, weight: torch.Tensor) -> None:
        self.weight, self.version, self.copy = weight, None, None

    def get(self) -> torch.Tensor:
        if self.copy is None or self.version != self.weight._version:
            self.copy, self.version = transpose_weight(self.weight), self.weight._version
        return self.copy

    def release(self) -> None:
        self.copy = None


class _LinearHeadChunkFn(torch.autograd.Function):
    """``lm_head`` (a plain ``nn.Linear``) and the log-probs of one chunk as a single node that also
    does the linear's backward: ``d_logits`` is written over the logits (kept from the forward, or
    rebuilt here -- the reference's per-chunk checkpoint, ``unirl/models/qwen3/ar.py:93-96``), and
    the two gradient GEMMs are issued in the operand layouts the GEMM library is fastest on."""

    @staticmethod
    def forward(ctx, hidden, tokens, weight, bias, temperature: float, keep: bool, fused_head: bool, transposed):
        # transposed: None, or the replay's _TransposedOnce plus whether this chunk runs last in the backward
        logits = None
        with torch.no_grad():
            if fused_head:
                # the head's GEMM with the log-softmax statistics in its epilogue: no logits at all
                logp, _, lse, _ = ops.lmhead_logp(hidden, weight, bias, tokens, temperature, want_lse=True)
            else:
                logits = F.linear(hidden, weight, bias)
                logp, _, lse = ops.token_logp_entropy(
                    logits, tokens, temperature, want_logp=True, want_entropy=False, want_lse=True
                )
        ctx.save_for_backward(hidden, tokens, lse, weight, bias, logits if keep else None)
        ctx.temperature, ctx.transposed = temperature, transposed
        ctx.consumed = False
        return logp

    @staticmethod
    def backward(ctx, g_logp):
        if ctx.consumed:
            raise RuntimeError(
                "the logits of this replay were overwritten by their gradient in the first backward; "
                "a second backward through the same graph needs chunked_replay_logp(..., keep_logits=False)"
            )
        hidden, tokens, lse, weight, bias, logits = ctx.saved_tensors
        if logits is None:
            logits = F.linear(hidden, weight, bias)
        else:
            ctx.consumed = True
        d_logits = ops.token_logp_bwd(logits, tokens, ctx.temperature, lse, g_logp, in_place=True)
        d2 = d_logits.reshape(-1, d_logits.shape[-1])
        g_hidden = g_weight = g_bias = None
        if ctx.needs_input_grad[0]:
            if ctx.transposed is not None:
                once, last = ctx.transposed
                g_hidden = torch.mm(d2, once.get().t()).view(hidden.shape)
                if last:
                    once.release()  # the replay's backward is complete: the copy's memory goes back now
            else:
                g_hidden = torch.mm(d2, weight).view(hidden.shape)
        if ctx.needs_input_grad[2]:
            g_weight = torch.mm(d2.t(), hidden.reshape(-1, hidden.shape[-1]))
        if bias is not None and ctx.needs_input_grad[3]:
            g_bias = d2.sum(dim=0)
        return g_hidden, None, g_weight, g_bias, None, None, None, None


def token_logp(logits: torch.Tensor, tokens: torch.Tensor, temperature: float = 1.0) -> torch.Tensor:
    """fp32 ``log_softmax(logits.float() / T)[..., tokens]`` with shape ``logits.shape[:-1]``.

    ``temperature <= 0`` means 1 (greedy decoding reports the untempered log-prob).
    Differentiable w.r.t. ``logits``.
    """
    T = float(temperature) if float(temperature) > 0.0 else 1.0
    if torch.is_grad_enabled() and logits.requires_grad:
        return _TokenLogpFn.apply(logits, tokens, T, False)
    logp, _, _ = ops.token_logp_entropy(logits, tokens, T, want_logp=True, want_entropy=False)
    return logp


def token_logp_entropy(
    logits: torch.Tensor, tokens: torch.Tensor, temperature: float = 1.0
) -> Tuple[torch.Tensor, torch.Tensor]:
    """``(log-prob of tokens, entropy of softmax(logits / T))`` per row, both fp32, one pass.

    The log-prob is differentiable w.r.t. ``logits``; the entropy is returned detached.
    """
    T = float(temperature) if float(temperature) > 0.0 else 1.0
    if torch.is_grad_enabled() and logits.requires_grad:
        return _TokenLogpFn.apply(logits, tokens, T, True)
    logp, ent, _ = ops.token_logp_entropy(logits, tokens, T, want_logp=True, want_entropy=True)
    return logp, ent


def token_entropy(logits: torch.Tensor, temperature: float = 1.0) -> torch.Tensor:
    """Entropy of ``softmax(logits.float() / T)`` per row (fp32, detached)."""
    T = float(temperature) if float(temperature) > 0.0 else 1.0
    _, ent, _ = ops.token_logp_entropy(logits, None, T, want_logp=False, want_entropy=True)
    return ent


#: all of a replay's logits are kept for the backward (no second ``lm_head`` pass) up to this size
KEEP_LOGITS_BYTES = 4 << 30
#: replays of at least this many rows compute the hidden states' gradient on a transposed copy of the weight
TRANSPOSED_HEAD_MIN_ROWS = 4096


def chunked_replay_logp(
    lm_head: Callable[[torch.Tensor], torch.Tensor],
    resp_hidden: torch.Tensor,
    response_tokens: torch.Tensor,
    temperature: float = 1.0,
    chunk: Optional[int] = None,
    keep_logits: Optional[bool] = None,
    fused_head: Optional[bool] = None,
    transposed_head: Optional[bool] = None,
) -> torch.Tensor:
    """Padded ``[B, T_max]`` fp32 log-probs of ``response_tokens`` under ``lm_head(resp_hidden)``.

    Chunked like the reference (``chunk = max(64, 2048 // B)`` there) so that the
    ``[B, chunk, V]`` logits block -- the only large transient -- stays bounded.  The default
    here is twice that, ``max(64, 4096 // B)``: the block is consumed by the fused kernel in the
    dtype ``lm_head`` produced (2 bytes per logit where the reference's fp32 copies hold 10), so
    it is still less than half the reference's transient, and the head's GEMMs run measurably
    faster on the larger block.  Under autograd
    the logits of a chunk are dropped and recomputed in the backward, like the reference's
    per-chunk checkpoint (``keep_logits=True`` keeps them instead: no second ``lm_head``
    pass, ``B * T_max * V`` elements of memory; an ``nn.Linear`` head's kept logits are overwritten
    by their gradient in the backward, so a second backward through the same graph raises).
    Left at ``None``, the logits of an
    ``nn.Linear`` head are kept when all of them together take at most ``KEEP_LOGITS_BYTES``
    (4 GiB, below what the reference's checkpointed chunks hold in fp32 transients) and
    recomputed otherwise; kept logits allow chunks
    of ``8192 // B`` rows.  The recomputing path is taken when ``resp_hidden`` or a parameter of
    an ``nn.Module`` head requires grad; a bare callable whose captured weights alone require
    grad keeps its logits.

    ``fused_head`` computes the forward with ``unirl_lmhead_logp``: the head's GEMM with the
    log-softmax statistics reduced in its epilogue, so no logits exist in the forward at all (the
    backward rebuilds each chunk's logits with ``lm_head`` as above).  It needs a plain bf16
    ``nn.Linear`` head, bf16 hidden states on the same device, a hidden size that is a multiple
    of 64 and no autocast (``True`` raises otherwise).  Measured on the MI355X with Qwen3-4B's head
    it is faster than the library GEMM plus the token kernel from 64 to 8192 rows per chunk and
    holds 6 % of the transient memory.  Left at ``None`` it is used wherever it applies and the
    logits are not kept: without autograd (scoring a rollout) and on the recomputing path.  Its
    bf16 logits differ from the library GEMM's in about 0.02 % of the entries by one bf16 ulp (a
    different fp32 summation order), as two library versions would.

    For a plain ``nn.Linear`` head on hidden states of its own dtype (no autocast) the head and
    its backward run inside one autograd node, which issues the gradient GEMMs itself.
    ``transposed_head`` lets it compute the hidden states' gradient on a ``[K, V]`` copy of the
    weight: the GEMM library is 1.2 - 1.5 times faster on that layout.  The copy is made once per
    replay, in its backward, from the weight's values at that moment (``V * K`` elements held while
    the backward runs), and dropped with it: no copy survives a replay, so a weight written between
    replays in any way -- an optimizer step, or a write through ``.data`` that no version counter
    records -- is always read afresh.  Left at ``None`` it is used for replays of at least
    ``TRANSPOSED_HEAD_MIN_ROWS`` rows.
    """
    bsz, t_max = int(resp_hidden.size(0)), int(response_tokens.size(1))
    if t_max == 0:
        return resp_hidden.new_zeros((bsz, 0), dtype=torch.float32)
    if keep_logits is None:
        keep_logits = (
            _is_plain_linear(lm_head)
            and bsz * t_max * lm_head.out_features * lm_head.weight.element_size() <= KEEP_LOGITS_BYTES
        )
    fused_ok = (
        _is_plain_linear(lm_head) and ops.lmhead_logp_supported(resp_hidden, lm_head.weight, lm_head.bias)
        and not torch.is_autocast_enabled("cuda")
    )
    if fused_head is None:
        # kept logits come from the library GEMM; everywhere else nothing needs them in the forward
        trains = fused_ok and torch.is_grad_enabled() and (
            resp_hidden.requires_grad or any(p.requires_grad for p in lm_head.parameters()))
        fused_head = fused_ok and not (trains and keep_logits)
    if fused_head:
        if not fused_ok:
            raise ValueError(
                "fused_head needs a plain bf16 nn.Linear head, bf16 hidden states on the same HIP device, a hidden "
                "size that is a multiple of 64, and no autocast"
            )
        keep_logits = False
    rows_per_chunk = 8192 if keep_logits else 4096
    step = int(chunk) if chunk is not None else max(64, rows_per_chunk // max(1, bsz))
    T = float(temperature) if float(temperature) > 0.0 else 1.0
    params = tuple(lm_head.parameters()) if isinstance(lm_head, torch.nn.Module) else ()
    wants_grad = torch.is_grad_enabled() and (resp_hidden.requires_grad or any(p.requires_grad for p in params))
    # a plain Linear on operands of its own dtype: the head and its backward run inside one node
    own_linear = (
        wants_grad and _is_plain_linear(lm_head) and not torch.is_autocast_enabled("cuda")
        and resp_hidden.dtype == lm_head.weight.dtype and resp_hidden.dtype in _KERNEL_DTYPES
        and resp_hidden.is_cuda and lm_head.weight.device == resp_hidden.device
        and (lm_head.bias is None or lm_head.bias.dtype == resp_hidden.dtype)
    )
    if transposed_head is None:
        transposed_head = bsz * t_max >= TRANSPOSED_HEAD_MIN_ROWS
    recompute = not keep_logits and wants_grad
    once = _TransposedOnce(lm_head.weight) if (own_linear and transposed_head and resp_hidden.requires_grad) else None
    parts: List[torch.Tensor] = []
    for s in range(0, t_max, step):
        h, tok = resp_hidden[:, s : s + step, :], response_tokens[:, s : s + step]
        if own_linear:
            # autograd runs the chunks' backwards in reverse order of creation: the first chunk is the last
            parts.append(_LinearHeadChunkFn.apply(h, tok, lm_head.weight, lm_head.bias, T, bool(keep_logits), fused_head,
                                                  None if once is None else (once, s == 0)))
        elif recompute:
            parts.append(_RecomputedChunkFn.apply(h, tok, lm_head, T, fused_head, *params))
        elif fused_head:
            parts.append(ops.lmhead_logp(h, lm_head.weight, lm_head.bias, tok, T)[0])
        else:
            logits = lm_head(h)
            if _is_plain_linear(lm_head) and torch.is_grad_enabled() and logits.requires_grad:
                # a plain Linear's output is saved by nothing but this node: its gradient may take its place
                parts.append(_TokenLogpFn.apply(logits, tok, T, False, True))
            else:
                parts.append(token_logp(logits, tok, temperature))
    return torch.cat(parts, dim=1)


class ARLogprobStep:
    """Per-token sampling step: pick the next token and report its log-prob under the
    temperature-scaled full softmax (before top-k / top-p truncation), as
    ``Qwen3ARStep.step`` does.  Token selection uses torch's sampling primitives; the
    log-prob is the fused kernel."""

    def __init__(self, *, temperature: float = 1.0, top_p: float = 1.0, top_k: int = 0) -> None:
        self.temperature = float(temperature)
        self.top_p = float(top_p)
        self.top_k = int(top_k)

    def step(self, logits: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        if logits.dim() != 2:
            raise ValueError(f"ARLogprobStep.step: expected logits shape [B, vocab], got {tuple(logits.shape)}")
        if self.temperature <= 0.0:
            token_id = logits.argmax(dim=-1)
            return token_id, token_logp(logits, token_id, 1.0)
        scaled = logits.float() / self.temperature
        if 0 < self.top_k < scaled.shape[-1]:
            kth = torch.topk(scaled, self.top_k, dim=-1).values[..., -1, None]
            scaled = scaled.masked_fill(scaled < kth, float("-inf"))
        if self.top_p < 1.0:
            sorted_vals, sorted_idx = torch.sort(scaled, dim=-1, descending=True)
            cum = torch.softmax(sorted_vals, dim=-1).cumsum(dim=-1)
            drop = torch.zeros_like(cum, dtype=torch.bool)
            drop[..., 1:] = cum[..., :-1] > self.top_p
            sorted_vals = sorted_vals.masked_fill(drop, float("-inf"))
            scaled = torch.full_like(scaled, float("-inf")).scatter(-1, sorted_idx, sorted_vals)
        token_id = torch.multinomial(torch.softmax(scaled, dim=-1), num_samples=1).squeeze(-1)
        return token_id, token_logp(logits, token_id, self.temperature)


__all__ = ["ARLogprobStep", "chunked_replay_logp", "token_entropy", "token_logp", "token_logp_entropy"]
