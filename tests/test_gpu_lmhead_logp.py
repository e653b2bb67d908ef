"""The lm_head GEMM with the log-softmax statistics in its epilogue (logits never written) against
the oracle on lm_head(h): `lm_head(h).float() / T`, gather, logsumexp (unirl/models/qwen3/ar.py:82-85)."""

import math

import pytest
import torch

from oracle import token_logp as otok
from tests._util import assert_close

pytestmark = pytest.mark.gpu

BF16_LOGP_RTOL = 2e-3  # bf16 path


def reference_logits(h, w, b):
    """What a bf16 Linear holds: the fp32 sum over K (+ bias), rounded once to bf16.  Evaluated in
    float64 so that the comparison is against the correctly rounded value."""
    acc = h.double() @ w.double().t()
    if b is not None:
        acc = acc + b.double()
    return acc.float().bfloat16()


def make(rows, K, V, seed, bias=False, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    h = torch.randn(rows, K, generator=g).bfloat16()
    w = (scale * torch.randn(V, K, generator=g) / math.sqrt(K)).bfloat16()
    b = (0.5 * torch.randn(V, generator=g)).bfloat16() if bias else None
    ids = torch.randint(0, V, (rows,), generator=g)
    return h, w, b, ids


def check_against_oracle(dev, h, w, b, ids, T, what):
    """Kernel logits == correctly rounded reference logits except for fp32-summation-order flips of one
    bf16 ulp (counted); statistics == oracle on the kernel's own logits (tight) and on the reference
    logits (bf16 tolerance, rows with a flipped target logit excepted and counted)."""
    from unirl_amd import ops

    lp, ent, lse, logits = ops.lmhead_logp(h.to(dev), w.to(dev), None if b is None else b.to(dev), ids.to(dev), T,
                                           want_entropy=True, want_lse=True, want_logits=True)
    ref_logits = reference_logits(h, w, b)
    got = logits.cpu()
    diff = (got.float() - ref_logits.float()).abs()
    ulp = torch.maximum(got.float().abs(), ref_logits.float().abs()) * 2.0 ** -7
    # a sum that nearly cancels carries the fp32 rounding of its terms, which may exceed an ulp of
    # the small result: bound it by 2^-20 of the sum of the terms' magnitudes
    slack = (h.double().abs() @ w.double().abs().t()).float() * 2.0 ** -20
    assert bool((diff <= ulp + slack).all()), f"{what}: a logit is off by more than one bf16 ulp"
    flipped = diff > 0
    frac = float(flipped.float().mean())
    assert frac < 2e-2, f"{what}: {frac:.2%} of the logits differ from the correctly rounded sum"
    # statistics on the kernel's own logits: the fp32 bar
    own_lp = otok.token_logp(got, ids, T)
    own_ent = otok.token_entropy(got, T)
    own_lse = torch.logsumexp(got.float() / T, dim=-1)
    assert_close(lp, own_lp, 1e-5, 2e-6, f"{what}: log-prob vs oracle on the same logits")
    assert_close(lse, own_lse, 1e-5, 2e-6, f"{what}: logsumexp vs oracle on the same logits")
    assert_close(ent, own_ent, 1e-5, 1e-6, f"{what}: entropy vs oracle on the same logits")
    # and against the oracle on the reference's logits
    ref_lp = otok.token_logp(ref_logits, ids, T)
    target_flipped = flipped[torch.arange(len(ids)), ids]
    ok = ~target_flipped
    assert int(target_flipped.sum()) <= max(2, len(ids) // 50), f"{what}: too many flipped target logits"
    assert_close(lp.cpu()[ok], ref_lp[ok], BF16_LOGP_RTOL, 2e-3, f"{what}: log-prob vs oracle on lm_head(h)")
    return frac, int(target_flipped.sum())


@pytest.mark.parametrize("rows,K,V,bias", [(64, 256, 1024, False), (130, 128, 300, True), (1, 64, 129, False),
                                           (257, 192, 1000, True), (128, 2560, 640, False),
                                           # the 256 x 256 tile: exact fit, ragged rows and columns, one K step
                                           (512, 64, 256, False), (300, 128, 700, True), (1000, 320, 513, True),
                                           (255, 128, 257, False), (256, 64, 1, False)])
@pytest.mark.parametrize("T", [1.0, 0.7])
def test_small_heads_match_oracle(dev, rows, K, V, bias, T):
    h, w, b, ids = make(rows, K, V, seed=rows + K + V, bias=bias, scale=4.0)
    check_against_oracle(dev, h, w, b, ids, T, f"rows={rows} K={K} V={V} bias={bias} T={T}")


def test_without_logits_gives_the_same_statistics(dev):
    from unirl_amd import ops

    h, w, b, ids = make(200, 320, 5000, seed=5, bias=True, scale=3.0)
    a = ops.lmhead_logp(h.to(dev), w.to(dev), b.to(dev), ids.to(dev), 0.9, want_entropy=True, want_lse=True,
                        want_logits=True)
    c = ops.lmhead_logp(h.to(dev), w.to(dev), b.to(dev), ids.to(dev), 0.9, want_entropy=True, want_lse=True)
    assert c[3] is None
    for x, y in zip(a[:3], c[:3]):
        assert torch.equal(x, y)
    # [B, S, K] hidden states and [B, S] ids keep their leading shape
    lp3, _, _, _ = ops.lmhead_logp(h.to(dev).view(4, 50, 320), w.to(dev), b.to(dev), ids.to(dev).view(4, 50), 0.9)
    assert tuple(lp3.shape) == (4, 50) and torch.equal(lp3.reshape(-1), c[0])


@pytest.mark.parametrize("rows,V", [(300, 1024), (64, 700)])
def test_masked_vocabulary_entries_stay_finite(dev, rows, V):
    """A -inf bias masks vocabulary entries.  The reference's logsumexp and the token kernel give finite
    log-probs and entropies for the other entries (0 * log 0 = 0); so must the fused head, in whole
    tiles (V = 1024: every 16-column piece of the first tile is masked before any finite logit is met)
    and in the ragged last tile."""
    from unirl_amd import ops

    h, w, _, ids = make(rows, 128, V, 77)
    b = torch.zeros(V).bfloat16()
    b[:300] = float("-inf")          # whole 16-column pieces, and more than one 256-column tile's first half
    b[517::7] = float("-inf")        # scattered single entries
    ids = torch.where(torch.isinf(b.float()[ids]), torch.full_like(ids, 301), ids)  # targets on live entries
    lp, ent, lse, logits = ops.lmhead_logp(h.to(dev), w.to(dev), b.to(dev), ids.to(dev), 0.9, want_entropy=True,
                                           want_lse=True, want_logits=True)
    got = logits.cpu()
    assert bool(torch.isinf(got.float()[:, :300]).all())
    assert bool(torch.isfinite(lp).all()) and bool(torch.isfinite(ent).all()) and bool(torch.isfinite(lse).all())
    assert_close(lp, otok.token_logp(got, ids, 0.9), 1e-5, 2e-6, "log-prob with masked entries")
    assert_close(lse, torch.logsumexp(got.float() / 0.9, dim=-1), 1e-5, 2e-6, "logsumexp with masked entries")
    assert_close(ent, otok.token_entropy(got, 0.9), 1e-5, 1e-6, "entropy with masked entries")
    # and the two paths chunked_replay_logp may take agree
    lp2, ent2, _ = ops.token_logp_entropy(logits, ids.to(dev), 0.9, want_logp=True, want_entropy=True)
    assert_close(lp, lp2.cpu(), 1e-5, 2e-6, "fused head vs token kernel on the same logits")
    assert_close(ent, ent2.cpu(), 1e-5, 1e-6, "fused head vs token kernel: entropy")


def test_out_of_range_id_and_argument_errors(dev):
    from unirl_amd import ops

    h, w, _, ids = make(8, 64, 256, seed=6)
    ids[3] = -100
    ids[5] = 256
    lp, _, _, _ = ops.lmhead_logp(h.to(dev), w.to(dev), None, ids.to(dev))
    assert torch.isnan(lp[3]) and torch.isnan(lp[5]) and bool(torch.isfinite(lp[[0, 1, 2, 4, 6, 7]]).all())
    with pytest.raises(ValueError):
        ops.lmhead_logp(h.float().to(dev), w.to(dev), None, ids.to(dev))        # not bf16
    with pytest.raises(ValueError):
        ops.lmhead_logp(h[:, :48].contiguous().to(dev), w[:, :48].contiguous().to(dev), None, ids.to(dev))  # K % 64
    with pytest.raises(ValueError):
        ops.lmhead_logp(h.to(dev), w.to(dev), None, ids[:4].to(dev))


@pytest.mark.parametrize("rows", [64, 2048])
def test_qwen3_head_shape(dev, rows):
    """Qwen3-4B's head: bf16 Linear(2560, 151936).  The weights are drawn on the device; the
    reference logits come from the float64 product on the device as well (chunked over V)."""
    from unirl_amd import ops

    K, V, T = 2560, 151936, 1.0
    g = torch.Generator(device=dev).manual_seed(7)
    w = (torch.randn(V, K, generator=g, device=dev) * (3.0 / math.sqrt(K))).bfloat16()
    h = torch.randn(rows, K, generator=g, device=dev).bfloat16()
    ids = torch.randint(0, V, (rows,), generator=g, device=dev)
    lp, ent, lse, logits = ops.lmhead_logp(h, w, None, ids, T, want_entropy=True, want_lse=True, want_logits=True)
    lp2, ent2, lse2, none = ops.lmhead_logp(h, w, None, ids, T, want_entropy=True, want_lse=True)
    assert none is None and torch.equal(lp, lp2) and torch.equal(ent, ent2) and torch.equal(lse, lse2)
    # logits against the correctly rounded float64 product, 8192 columns at a time
    n_flip, worst = 0, 0.0
    ref_logits = torch.empty_like(logits)
    for c0 in range(0, V, 8192):
        blk = (h.double() @ w[c0 : c0 + 8192].double().t()).float().bfloat16()
        ref_logits[:, c0 : c0 + 8192] = blk
        d = (logits[:, c0 : c0 + 8192].float() - blk.float()).abs()
        ulp = torch.maximum(blk.float().abs(), logits[:, c0 : c0 + 8192].float().abs()) * 2.0 ** -7
        slack = (h.float().abs() @ w[c0 : c0 + 8192].float().abs().t()) * 2.0 ** -20  # see check_against_oracle
        assert bool((d <= ulp + slack).all()), "a logit is off by more than one bf16 ulp"
        n_flip += int((d > 0).sum())
    frac = n_flip / logits.numel()
    print(f"rows={rows}: {frac:.3%} of the logits differ by one bf16 ulp from the correctly rounded product")
    assert frac < 2e-2
    # statistics: oracle (CPU) on a row sample of the kernel's own logits, fp32 bar
    sample = torch.arange(0, rows, max(1, rows // 64))[:64]
    own = logits[sample.to(dev)].cpu()
    assert_close(lp[sample.to(dev)], otok.token_logp(own, ids[sample.to(dev)].cpu(), T), 1e-5, 2e-6, "log-prob")
    assert_close(ent[sample.to(dev)], otok.token_entropy(own, T), 1e-5, 1e-6, "entropy")
    # all rows on the device in float64, from the kernel's logits
    lf = logits.double() / T
    ref_lse = torch.logsumexp(lf, dim=-1)
    ref_lp_own = lf.gather(-1, ids.unsqueeze(-1)).squeeze(-1) - ref_lse
    assert_close(lse, ref_lse, 1e-5, 2e-6, "logsumexp, all rows")
    assert_close(lp, ref_lp_own, 1e-5, 2e-6, "log-prob, all rows, own logits")
    # against lm_head(h) as the reference computes it (correctly rounded bf16 logits): bf16 bar,
    # rows whose target logit flipped by one ulp counted apart
    lf_ref = ref_logits.double() / T
    ref_lp = lf_ref.gather(-1, ids.unsqueeze(-1)).squeeze(-1) - torch.logsumexp(lf_ref, dim=-1)
    tgt_flip = logits.gather(-1, ids.unsqueeze(-1)).squeeze(-1) != ref_logits.gather(-1, ids.unsqueeze(-1)).squeeze(-1)
    print(f"rows={rows}: {int(tgt_flip.sum())} target logits flipped by one bf16 ulp")
    assert int(tgt_flip.sum()) <= max(2, rows // 50)
    assert_close(lp[~tgt_flip], ref_lp[~tgt_flip], BF16_LOGP_RTOL, 2e-3, "log-prob vs oracle on lm_head(h)")


def test_chunked_replay_with_the_fused_head(dev):
    """chunked_replay_logp(fused_head=True): same log-probs as the library-GEMM path up to one-ulp flips
    of single bf16 logits, same gradients (the backward is the same recompute), and no [B, chunk, V]
    transient in the forward."""
    from unirl_amd import models

    B, T_max, H, V, T = 2, 300, 256, 20000, 0.8
    g = torch.Generator().manual_seed(21)
    # no bias, like the LM heads this path serves: with one, the library adds it to the already rounded
    # bf16 product (two roundings) where the fused kernel adds it in fp32 and rounds once, which is
    # what test_small_heads_match_oracle holds it to
    head = torch.nn.Linear(H, V, bias=False).to(dev).to(torch.bfloat16)
    with torch.no_grad():
        head.weight.copy_((3.0 / math.sqrt(H) * torch.randn(V, H, generator=g)).to(dev))
    hidden = torch.randn(B, T_max, H, generator=g).bfloat16().to(dev)
    toks = torch.randint(0, V, (B, T_max), generator=g).to(dev)
    up = torch.randn(B, T_max, generator=g).to(dev)

    def run(fused):
        head.zero_grad(set_to_none=True)
        h = hidden.clone().requires_grad_(True)
        torch.cuda.synchronize()
        torch.cuda.reset_peak_memory_stats()
        base = torch.cuda.memory_allocated()
        out = models.chunked_replay_logp(head, h, toks, T, chunk=128, keep_logits=False, fused_head=fused)
        fwd_peak = torch.cuda.max_memory_allocated() - base
        (out * up).sum().backward()
        return out.detach(), h.grad.float(), head.weight.grad.float(), fwd_peak

    out_f, gh_f, gw_f, peak_f = run(True)
    out_u, gh_u, gw_u, peak_u = run(False)
    # a flipped target logit moves a log-prob by one bf16 ulp of that logit (<= 2^-7 * 16 here); everything
    # else moves by the tiny change of the log-sum-exp
    close = (out_f - out_u).abs() <= 2e-3 * out_u.abs() + 2e-3
    assert int((~close).sum()) <= 3, f"{int((~close).sum())} log-probs differ beyond one-ulp flips"
    assert float((out_f - out_u).abs().max()) < 0.2
    assert float((gh_f - gh_u).norm() / gh_u.norm()) < 1e-2
    assert float((gw_f - gw_u).norm() / gw_u.norm()) < 1e-2
    # the unfused forward holds a [B, chunk, V] bf16 block, the fused one only its tile states
    assert peak_f < peak_u / 2, (peak_f, peak_u)
    # no-grad call takes the fused kernel too
    with torch.no_grad():
        out_ng = models.chunked_replay_logp(head, hidden, toks, T, chunk=128, fused_head=True)
    assert torch.equal(out_ng, out_f)
    with pytest.raises(ValueError, match="fused_head"):
        models.chunked_replay_logp(head.float(), hidden.float(), toks, T, fused_head=True)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32, torch.int16, torch.int32])
def test_transpose_2d_is_exact(dev, dtype):
    """unirl_transpose_2d: bit-exact against torch's transposed copy for whole tiles, ragged edges, one
    row / one column, strided source rows and a base off the 16-byte grid (element-wise path)."""
    from unirl_amd import ops

    g = torch.Generator().manual_seed(30)
    for rows, cols in ((64, 64), (128, 192), (1, 1), (1, 300), (300, 1), (65, 127), (200, 72), (7, 1000), (513, 66)):
        if dtype.is_floating_point:
            src = torch.randn(rows, cols, generator=g).to(dtype).to(dev)
        else:
            src = torch.randint(-30000, 30000, (rows, cols), generator=g).to(dtype).to(dev)
        out = ops.transpose_2d(src)
        assert out.shape == (cols, rows) and out.is_contiguous()
        assert torch.equal(out, src.t().contiguous()), (rows, cols)
        # rows of a wider buffer, starting one element in: a leading dimension and a base that rule out
        # 16-byte loads
        wide = torch.zeros(rows, cols + 3, dtype=dtype, device=dev)
        view = wide[:, 1 : 1 + cols]
        view.copy_(src)
        assert torch.equal(ops.transpose_2d(view), src.t().contiguous()), (rows, cols, "strided")
    with pytest.raises(ValueError):
        ops.transpose_2d(torch.zeros(4, 4, dtype=torch.float64, device=dev))
    with pytest.raises(ValueError):
        ops.transpose_2d(torch.zeros(4, 4, 4, device=dev))


def test_transpose_2d_head_sized(dev):
    """The Qwen3-4B head's weight, [151936, 2560] bf16 (778 MB)."""
    from unirl_amd import ops

    w = torch.randn(151936, 2560, device=dev, dtype=torch.bfloat16)
    wt = ops.transpose_2d(w)
    assert torch.equal(wt, w.t().contiguous())


def test_chunked_replay_picks_the_fused_head_where_no_logits_are_kept(dev):
    """Left to itself, the replay of a plain bf16 head runs the fused kernel without autograd and on the
    recomputing path, and the library GEMM where it keeps the logits for the backward."""
    from unirl_amd import models, ops

    B, T_max, H, V = 2, 40, 64, 500
    g = torch.Generator().manual_seed(22)
    head = torch.nn.Linear(H, V, bias=False).to(dev).to(torch.bfloat16)
    hidden = torch.randn(B, T_max, H, generator=g).bfloat16().to(dev)
    toks = torch.randint(0, V, (B, T_max), generator=g).to(dev)
    fused = ops.lmhead_logp(hidden, head.weight, None, toks, 1.0)[0]
    with torch.no_grad():
        assert torch.equal(models.chunked_replay_logp(head, hidden, toks), fused)
        unfused = models.chunked_replay_logp(head, hidden, toks, fused_head=False)
    h = hidden.clone().requires_grad_(True)
    kept = models.chunked_replay_logp(head, h, toks)                       # fits the budget: logits kept, library GEMM
    assert torch.equal(kept.detach(), unfused)
    dropped = models.chunked_replay_logp(head, h, toks, keep_logits=False)  # nothing kept: fused forward
    assert torch.equal(dropped.detach(), fused)
    dropped.sum().backward()
    g_fused = h.grad.clone()
    h.grad = None
    kept.sum().backward()
    assert float((g_fused.float() - h.grad.float()).norm() / h.grad.float().norm()) < 2e-2
    # a head the fused kernel does not take (fp32) falls back silently when left to itself
    head32 = torch.nn.Linear(H, V).to(dev)
    with torch.no_grad():
        out32 = models.chunked_replay_logp(head32, hidden.float(), toks)
    assert out32.dtype == torch.float32 and bool(torch.isfinite(out32).all())
