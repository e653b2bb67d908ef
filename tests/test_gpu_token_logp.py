"""GPU parity of the fused token log-prob / entropy kernel against the CPU oracle."""

import math

import pytest
import torch

from oracle import token_logp as otok
from tests._util import BF16_RTOL, FP32_RTOL, assert_close

pytestmark = pytest.mark.gpu


def logits(rows, V, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    x = (2 * torch.randn(rows, V, generator=g)).to(dtype)
    ids = torch.randint(0, V, (rows,), generator=g)
    return x, ids


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("V", [1, 7, 1000, 4099, 50257, 151936])
@pytest.mark.parametrize("T", [1.0, 0.7])
def test_logp_entropy_match_oracle(dev, dtype, V, T):
    from unirl_amd import models

    rows = 9
    x, ids = logits(rows, V, V + int(T * 10), dtype)
    if V > 20:
        x[3, 17] = 15.0  # spiked row
        ids[3] = 17
    ref_lp, ref_ent = otok.token_logp(x, ids, T), otok.token_entropy(x, T)
    lp, ent = models.token_logp_entropy(x.to(dev), ids.to(dev), T)
    assert lp.dtype == ent.dtype == torch.float32 and lp.shape == ent.shape == (rows,)
    # eager fp32 `x[tok] - logsumexp(x)` itself carries ~|x| * 2^-24 absolute error; allow for it
    assert_close(lp, ref_lp, FP32_RTOL, 2e-6, "logp")
    assert_close(ent, ref_ent, FP32_RTOL, 1e-6, "entropy")
    # against float64 truth the kernel is accurate in pure relative terms, also on the spiked row
    for r in (0, 3):
        b_lp, b_ent = otok.token_logp_entropy_f64(x[r].float().tolist(), int(ids[r]), T)
        assert abs(float(lp[r]) - b_lp) <= 2e-6 * abs(b_lp) + 1e-9, (r, float(lp[r]), b_lp)
        assert abs(float(ent[r]) - b_ent) <= 2e-6 * abs(b_ent) + 1e-9, (r, float(ent[r]), b_ent)


def test_leading_dims_and_temperature_rules(dev):
    from unirl_amd import models

    x, ids = logits(24, 333, 1, torch.bfloat16)
    x3, ids3 = x.reshape(2, 12, 333), ids.reshape(2, 12)
    lp = models.token_logp(x3.to(dev), ids3.to(dev), 0.7)
    assert lp.shape == (2, 12)
    assert_close(lp, otok.token_logp(x3, ids3, 0.7), FP32_RTOL, 2e-6, "3-d logits")
    # T <= 0 means 1
    assert torch.equal(models.token_logp(x.to(dev), ids.to(dev), 0.0), models.token_logp(x.to(dev), ids.to(dev), 1.0))
    assert torch.equal(models.token_logp(x.to(dev), ids.to(dev), -2.0), models.token_logp(x.to(dev), ids.to(dev), 1.0))
    assert_close(models.token_entropy(x.to(dev), 0.7), otok.token_entropy(x, 0.7), FP32_RTOL, 1e-6, "entropy only")


def test_row_views_strides_and_misalignment(dev):
    from unirl_amd import models, ops

    x, ids = logits(12, 1003, 2, torch.bfloat16)  # 2006-byte rows: every other row is misaligned
    xd = x.to(dev)
    assert_close(models.token_logp(xd, ids.to(dev)), otok.token_logp(x, ids), FP32_RTOL, 2e-6, "odd V")
    # a column slice keeps the row stride of the parent: no copy is needed
    sub, sub_ref = xd[:, 5:905], x[:, 5:905]
    sub_ids = ids % 900
    lp, ent, _ = ops.token_logp_entropy(sub, sub_ids.to(dev), 1.0)
    assert_close(lp, otok.token_logp(sub_ref, sub_ids), FP32_RTOL, 2e-6, "strided rows")
    assert_close(ent, otok.token_entropy(sub_ref), FP32_RTOL, 1e-6, "strided rows entropy")
    # transposed logits are made contiguous by the wrapper
    xt = x.t().contiguous().to(dev).t()
    assert_close(models.token_logp(xt, ids.to(dev)), otok.token_logp(x, ids), FP32_RTOL, 2e-6, "transposed")
    # the shifted logits of a training step, [B, S, V][:, :-1], are read in place: one launch per
    # batch entry, no flattened copy
    x3, ids3 = logits(3 * 7, 1003, 4, torch.bfloat16)
    x3, ids3 = x3.reshape(3, 7, 1003), ids3.reshape(3, 7)
    x3d = x3.to(dev)
    shifted, sh_ids = x3d[:, :-1], ids3[:, 1:]
    assert not shifted.is_contiguous()
    blocks = list(ops._row_blocks(shifted, 1003))
    assert len(blocks) == 3 and all(b.data_ptr() == x3d[k].data_ptr() for k, b in enumerate(blocks))
    lp, ent, _ = ops.token_logp_entropy(shifted, sh_ids.to(dev), 0.7)
    assert lp.shape == (3, 6)
    assert_close(lp, otok.token_logp(x3[:, :-1], sh_ids, 0.7), FP32_RTOL, 2e-6, "shifted logits")
    assert_close(ent, otok.token_entropy(x3[:, :-1], 0.7), FP32_RTOL, 1e-6, "shifted logits entropy")
    assert len(list(ops._row_blocks(x3d, 1003))) == 1 and len(list(ops._row_blocks(xd[:, 5:905], 900))) == 1
    # and their backward, through autograd: the gradient of the slice lands in the parent
    leaf = x3.float().requires_grad_(True)
    w = torch.randn(3, 6, generator=torch.Generator().manual_seed(1))
    (otok.token_logp(leaf[:, :-1], sh_ids, 0.7) * w).sum().backward()
    leaf_d = x3.float().to(dev).requires_grad_(True)
    (models.token_logp(leaf_d[:, :-1], sh_ids.to(dev), 0.7) * w.to(dev)).sum().backward()
    assert_close(leaf_d.grad, leaf.grad, 1e-5, 1e-6 * float(leaf.grad.abs().max()), "grad through the shifted view")
    assert float(leaf_d.grad[:, -1].abs().sum()) == 0.0


def test_uniform_peaked_and_minus_inf(dev):
    from unirl_amd import models

    V = 151936
    x = torch.zeros(4, V, dtype=torch.bfloat16)
    ids = torch.tensor([5, V - 1, 7, 0])
    x[2, 7] = 60.0
    x[3, 100:] = float("-inf")  # masked vocabulary tail
    lp, ent = models.token_logp_entropy(x.to(dev), ids.to(dev))
    assert abs(float(lp[0]) + math.log(V)) < 1e-5 and abs(float(ent[1]) - math.log(V)) < 1e-5
    assert abs(float(lp[2])) < 1e-6 and 0.0 <= float(ent[2]) < 1e-6
    assert abs(float(lp[3]) + math.log(100)) < 1e-5 and abs(float(ent[3]) - math.log(100)) < 1e-5
    ref = torch.distributions.Categorical(logits=x[3].float()).entropy()
    assert abs(float(ent[3]) - float(ref)) < 1e-5


def test_out_of_range_id_gives_nan_not_a_fault(dev):
    from unirl_amd import models

    x, ids = logits(4, 100, 3, torch.float32)
    ids[1], ids[2] = 100, -1
    lp = models.token_logp(x.to(dev), ids.to(dev)).cpu()
    assert torch.isnan(lp[1]) and torch.isnan(lp[2]) and torch.isfinite(lp[0]) and torch.isfinite(lp[3])


def test_out_of_range_id_gets_a_zero_gradient_row(dev):
    """A padding id (e.g. -100) has no log-prob; its row of the gradient is zero, whatever the
    upstream gradient holds (NaN included), and the other rows are untouched by it."""
    from unirl_amd import ops

    V = 1000
    x, ids = logits(6, V, 9, torch.bfloat16)
    bad = ids.clone()
    bad[1], bad[4] = -100, V
    xd = x.to(dev)
    _, _, lse = ops.token_logp_entropy(xd, bad.to(dev), 1.0, want_logp=False, want_entropy=False, want_lse=True)
    g = torch.randn(6)
    g[4] = float("nan")
    grad = ops.token_logp_bwd(xd, bad.to(dev), 1.0, lse, g.to(dev)).float().cpu()
    assert torch.count_nonzero(grad[1]) == 0 and torch.count_nonzero(grad[4]) == 0
    good = ops.token_logp_bwd(xd, ids.to(dev), 1.0, lse, torch.nan_to_num(g).to(dev)).float().cpu()
    keep = [0, 2, 3, 5]
    assert torch.equal(grad[keep], good[keep])
    # in place on the same buffer gives the same bits
    buf = xd.clone()
    ops.token_logp_bwd(buf, bad.to(dev), 1.0, lse, g.to(dev), in_place=True)
    assert torch.equal(buf.float().cpu(), grad)


def test_all_minus_inf_row_has_lse_minus_inf(dev):
    """torch.logsumexp of a row of -inf is -inf (and the log-prob -inf - (-inf) = NaN)."""
    from unirl_amd import ops

    x = torch.randn(3, 500)
    x[1] = float("-inf")
    ids = torch.tensor([3, 4, 5])
    lp, ent, lse = ops.token_logp_entropy(x.to(dev), ids.to(dev), 1.0, want_lse=True)
    ref = torch.logsumexp(x, dim=-1)
    assert float(lse[1]) == float("-inf") and torch.isnan(lp[1]) and torch.isnan(ent[1])
    assert torch.allclose(lse.cpu()[[0, 2]], ref[[0, 2]], rtol=1e-6)


def test_shape_errors(dev):
    from unirl_amd import models

    x, ids = logits(4, 100, 4, torch.float32)
    with pytest.raises(ValueError):
        models.token_logp(x.to(dev), ids[:3].to(dev))
    assert models.token_logp(x[:0].to(dev), ids[:0].to(dev)).shape == (0,)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("T", [1.0, 0.7])
def test_backward_matches_autograd_of_oracle(dev, dtype, T):
    from unirl_amd import models

    x, ids = logits(6, 2051, 5, dtype)
    g = torch.randn(6, generator=torch.Generator().manual_seed(6))
    xr = x.clone().requires_grad_(True)
    (otok.token_logp(xr, ids, T) * g).sum().backward()
    xg = x.to(dev).requires_grad_(True)
    (models.token_logp(xg, ids.to(dev), T) * g.to(dev)).sum().backward()
    assert xg.grad.dtype == dtype and xg.grad.shape == x.shape
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    assert_close(xg.grad.float(), xr.grad.float(), tol, tol * float(xr.grad.float().abs().max()) * 0.1, "grad")
    # log-prob with the entropy beside it: one pass, same gradient, entropy detached
    xe = x.to(dev).requires_grad_(True)
    lp, ent = models.token_logp_entropy(xe, ids.to(dev), T)
    assert not ent.requires_grad and lp.requires_grad
    (lp * g.to(dev)).sum().backward()
    assert torch.equal(xe.grad, xg.grad)
    assert torch.equal(ent, models.token_entropy(x.to(dev), T))


def test_chunked_replay_matches_reference_chunk_loop(dev):
    from unirl_amd import models

    g = torch.Generator().manual_seed(7)
    B, T_max, H, V = 3, 150, 32, 1000
    hidden = torch.randn(B, T_max, H, generator=g).bfloat16()
    W = (0.2 * torch.randn(V, H, generator=g)).bfloat16()
    toks = torch.randint(0, V, (B, T_max), generator=g)
    Wd = W.to(dev)
    got = models.chunked_replay_logp(lambda h: h @ Wd.t(), hidden.to(dev), toks.to(dev), temperature=0.7, chunk=64)
    assert got.shape == (B, T_max) and got.dtype == torch.float32
    # oracle on the logits the device GEMM produced (the GEMM itself is not under test)
    lg = (hidden.to(dev) @ Wd.t()).cpu()
    ref = otok.token_logp(lg, toks, 0.7)
    assert_close(got, ref, FP32_RTOL, 2e-6, "chunked replay")
    assert models.chunked_replay_logp(lambda h: h @ Wd.t(), hidden[:, :0].to(dev), toks[:, :0].to(dev)).shape == (B, 0)


def test_sampling_step_reports_full_softmax_logprob(dev):
    from unirl_amd import models

    x, _ = logits(16, 500, 8, torch.bfloat16)
    torch.manual_seed(0)
    tok, lp = models.ARLogprobStep(temperature=0.7, top_p=0.9, top_k=50).step(x.to(dev))
    assert_close(lp, otok.token_logp(x, tok.cpu(), 0.7), FP32_RTOL, 2e-6, "behaviour logp")
    tok, lp = models.ARLogprobStep(temperature=0.0).step(x.to(dev))
    assert torch.equal(tok.cpu(), x.float().argmax(-1))
    assert_close(lp, otok.token_logp(x, tok.cpu(), 1.0), FP32_RTOL, 2e-6, "greedy logp")
    with pytest.raises(ValueError):
        models.ARLogprobStep().step(x.reshape(2, 8, 500).to(dev))


def test_config2_full_shape(dev):
    """bf16 [8192, 151936], 1% of rows with one +15 spike (seed 1002): parity on a row sample against
    the CPU oracle, and on every row through properties and a chunked eager computation on the device."""
    from unirl_amd import models

    rows, V = 8192, 151936
    g = torch.Generator(device=dev).manual_seed(1002)
    x = torch.empty(rows, V, dtype=torch.bfloat16, device=dev)
    for s in range(0, rows, 512):  # generate in slabs: the fp32 normals are a transient
        x[s : s + 512] = (2 * torch.randn(512, V, generator=g, device=dev)).bfloat16()
    spiked = torch.randperm(rows, generator=g, device=dev)[:82]
    cols = torch.randint(0, V, (82,), generator=g, device=dev)
    x[spiked, cols] = 15.0
    ids = torch.randint(0, V, (rows,), generator=g, device=dev)
    ids[spiked[:41]] = cols[:41]  # half of the spiked rows are asked for their spike

    lp, ent = models.token_logp_entropy(x, ids, 1.0)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(lp).all()) and bool(torch.isfinite(ent).all())
    assert bool((lp <= 0).all()) and bool((ent >= 0).all()) and bool((ent <= math.log(V) + 1e-5).all())

    sample = torch.cat([spiked[:8], torch.arange(0, rows, 683, device=dev)]).cpu()
    xs, ids_s = x[sample.to(dev)].cpu(), ids[sample.to(dev)].cpu()
    assert_close(lp[sample.to(dev)], otok.token_logp(xs, ids_s), FP32_RTOL, 2e-6, "config-2 logp sample")
    assert_close(ent[sample.to(dev)], otok.token_entropy(xs), FP32_RTOL, 1e-6, "config-2 entropy sample")

    # every row, against eager torch on the device in fp64 slabs
    for s in range(0, rows, 256):
        lf = x[s : s + 256].double()
        ref = lf.gather(-1, ids[s : s + 256, None])[:, 0] - torch.logsumexp(lf, -1)
        assert_close(lp[s : s + 256], ref, 2e-6, 1e-7, f"rows {s}..")
    # determinism
    lp2, ent2 = models.token_logp_entropy(x, ids, 1.0)
    assert torch.equal(lp, lp2) and torch.equal(ent, ent2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_chunked_replay_recomputes_logits_in_backward(dev, dtype):
    """Training path of the chunked replay: the chunk's logits are dropped after the forward and
    rebuilt in the backward (the reference's per-chunk checkpoint).  Gradients of the hidden states
    and of the head's weight and bias against autograd through the reference's chunk function."""
    from unirl_amd import models

    g = torch.Generator().manual_seed(11)
    B, T_max, H, V, T = 3, 150, 32, 1000, 0.7
    hidden = torch.randn(B, T_max, H, generator=g)
    toks = torch.randint(0, V, (B, T_max), generator=g)
    upstream = torch.randn(B, T_max, generator=g)
    head = torch.nn.Linear(H, V)
    with torch.no_grad():
        head.weight.copy_(0.2 * torch.randn(V, H, generator=g))
        head.bias.copy_(0.1 * torch.randn(V, generator=g))

    # reference chunk function (qwen3/ar.py:82-85) on the CPU, fp32
    h_ref = hidden.clone().requires_grad_(True)
    lf = head(h_ref).float() / T
    ref = lf.gather(-1, toks.unsqueeze(-1)).squeeze(-1) - torch.logsumexp(lf, dim=-1)
    (ref * upstream).sum().backward()
    ref_grads = (h_ref.grad.clone(), head.weight.grad.clone(), head.bias.grad.clone())
    head.zero_grad()

    def run(keep):
        hd = torch.nn.Linear(H, V).to(dev).to(dtype)
        with torch.no_grad():
            hd.weight.copy_(head.weight.to(dtype))
            hd.bias.copy_(head.bias.to(dtype))
        h = hidden.to(dev).to(dtype).requires_grad_(True)
        out = models.chunked_replay_logp(hd, h, toks.to(dev), temperature=T, chunk=64, keep_logits=keep)
        (out * upstream.to(dev)).sum().backward()
        return out.detach().cpu(), (h.grad.float().cpu(), hd.weight.grad.float().cpu(), hd.bias.grad.float().cpu())

    out_r, grads_r = run(False)
    out_k, grads_k = run(True)
    # dropping the logits changes nothing: same kernels on the same recomputed values
    assert torch.equal(out_r, out_k)
    for a, b in zip(grads_r, grads_k):
        assert torch.equal(a, b)
    if dtype == torch.float32:
        assert_close(out_r, ref.detach(), 1e-5, 2e-5, "log-probs")  # the GEMMs differ in summation order
        for name, a, b in zip(("hidden", "weight", "bias"), grads_r, ref_grads):
            assert_close(a, b, 1e-4, 1e-5 * float(b.abs().max()), f"{name} grad")
    else:
        for name, a, b in zip(("hidden", "weight", "bias"), grads_r, ref_grads):
            assert_close(a, b, 5e-2, 2e-2 * float(b.abs().max()), f"{name} grad (bf16 head)")

    # hidden states without grad, head parameters with: still the recomputing path, same result
    hd = torch.nn.Linear(H, V).to(dev)
    with torch.no_grad():
        hd.weight.copy_(head.weight)
        hd.bias.copy_(head.bias)
    out = models.chunked_replay_logp(hd, hidden.to(dev), toks.to(dev), temperature=T, chunk=64, keep_logits=False)
    assert "LinearHeadChunk" in type(out.grad_fn.next_functions[0][0]).__name__
    (out * upstream.to(dev)).sum().backward()
    assert_close(hd.weight.grad.cpu(), ref_grads[1], 1e-4, 1e-5 * float(ref_grads[1].abs().max()), "weight grad only")


def test_chunked_replay_keeps_logits_only_within_its_budget(dev, monkeypatch):
    """Left to itself the replay keeps an ``nn.Linear`` head's logits for the backward while all of them
    fit the byte budget and recomputes them beyond it; a bare callable's logits are never kept by default
    when the hidden states need a gradient."""
    from unirl_amd import models
    from unirl_amd.models import ar_logp

    B, T_max, H, V = 2, 40, 16, 300
    g = torch.Generator().manual_seed(12)
    head = torch.nn.Linear(H, V).to(dev)
    toks = torch.randint(0, V, (B, T_max), generator=g).to(dev)

    def path(lm_head):
        h = torch.randn(B, T_max, H, generator=g).to(dev).requires_grad_(True)
        out = models.chunked_replay_logp(lm_head, h, toks, chunk=16)
        return {type(fn).__name__ for fn, _ in out.grad_fn.next_functions}  # out = cat(per-chunk parts)

    # kept logits of a Linear head are overwritten by their gradient: a second backward says so
    h = torch.randn(B, T_max, H, generator=g).to(dev).requires_grad_(True)
    out = models.chunked_replay_logp(head, h, toks, chunk=16)
    out.sum().backward(retain_graph=True)
    with pytest.raises(RuntimeError, match="overwritten by their gradient"):
        out.sum().backward()
    head.zero_grad()

    # a Linear subclass, or a Linear with a forward hook, may hold its output elsewhere: its logits are
    # never overwritten, so the captured output still holds logits after the backward and a second
    # backward through the same graph works
    class MyLinear(torch.nn.Linear):
        pass

    sub = MyLinear(H, V).to(dev)
    hooked = torch.nn.Linear(H, V).to(dev)
    seen = []
    hooked.register_forward_hook(lambda mod, args, out: seen.append(out))
    for lm_head in (sub, hooked):
        assert not ar_logp._is_plain_linear(lm_head)
        h = torch.randn(B, T_max, H, generator=g).to(dev).requires_grad_(True)
        out = models.chunked_replay_logp(lm_head, h, toks, chunk=16, keep_logits=True)
        out.sum().backward(retain_graph=True)
        first = h.grad.clone()
        h.grad = None
        out.sum().backward()
        assert torch.equal(h.grad, first)
    assert ar_logp._is_plain_linear(head)
    captured = seen[0].detach()
    with torch.no_grad():
        again = torch.nn.functional.linear(h[:, :16].detach(), hooked.weight, hooked.bias)
    assert torch.allclose(captured, again), "a hooked head's captured logits were overwritten"

    def keeps(lm_head):
        """Whether the replay kept (and so consumed) its logits: then a second backward raises."""
        h = torch.randn(B, T_max, H, generator=g).to(dev).requires_grad_(True)
        out = models.chunked_replay_logp(lm_head, h, toks, chunk=16)
        out.sum().backward(retain_graph=True)
        try:
            out.sum().backward()
        except RuntimeError as e:
            assert "overwritten by their gradient" in str(e)
            return True
        return False

    assert B * T_max * V * 4 < ar_logp.KEEP_LOGITS_BYTES
    assert all("LinearHeadChunk" in n for n in path(head))  # a plain Linear: head and backward in one node
    assert keeps(head)
    monkeypatch.setattr(ar_logp, "KEEP_LOGITS_BYTES", B * T_max * V * 4 - 1)
    assert all("LinearHeadChunk" in n for n in path(head))
    assert not keeps(head)
    assert all("RecomputedChunk" in n for n in path(lambda h: h @ head.weight.t()))
    assert all("RecomputedChunk" in n for n in path(sub))


def test_chunked_replay_transposed_head_gradient(dev):
    """The hidden states' gradient computed on the transposed copy of the weight equals the plain
    product (another summation order), and the copy can never be stale: it is made inside each
    replay's backward and dropped with it, so the next replay reads the weight afresh however it was
    written in between -- in place (an optimizer step, which moves the version counter) or through
    `.data` (EMA, weight sync, parameter injection: neither the version nor the address changes)."""
    from unirl_amd import models
    from unirl_amd.models import ar_logp

    B, T_max, H, V = 2, 48, 32, 700
    g = torch.Generator().manual_seed(13)
    head = torch.nn.Linear(H, V).to(dev)
    toks = torch.randint(0, V, (B, T_max), generator=g).to(dev)
    hidden = torch.randn(B, T_max, H, generator=g).to(dev)
    up = torch.randn(B, T_max, generator=g).to(dev)

    def grads(transposed):
        head.zero_grad(set_to_none=True)
        h = hidden.clone().requires_grad_(True)
        out = models.chunked_replay_logp(head, h, toks, 0.9, chunk=16, transposed_head=transposed)
        (out * up).sum().backward()
        return out.detach(), h.grad, head.weight.grad.clone(), head.bias.grad.clone()

    def reference():
        h = hidden.clone().requires_grad_(True)
        lf = torch.nn.functional.linear(h, head.weight.detach(), head.bias.detach()).float() / 0.9
        ref = lf.gather(-1, toks.unsqueeze(-1)).squeeze(-1) - torch.logsumexp(lf, dim=-1)
        (ref * up).sum().backward()
        return h.grad

    writes = ("in place", ".data", "none")
    for how in writes:
        version, address = head.weight._version, head.weight.data_ptr()
        out_t, gh_t, gw_t, gb_t = grads(True)
        out_p, gh_p, gw_p, gb_p = grads(False)
        assert torch.equal(out_t, out_p) and torch.equal(gw_t, gw_p) and torch.equal(gb_t, gb_p)
        assert_close(gh_t, gh_p, 1e-5, 1e-6 * float(gh_p.abs().max()), f"hidden grad, transposed copy vs plain ({how})")
        assert_close(gh_t, reference(), 1e-4, 1e-5 * float(gh_p.abs().max()), "hidden grad vs autograd of the chain")
        fresh = 0.05 * torch.randn(V, H, generator=g).to(dev)
        if how == "in place":  # an optimizer step: the version moves on
            with torch.no_grad():
                head.weight.add_(fresh)
            assert head.weight._version != version
        elif how == ".data":   # invisible to a version / address check
            head.weight.data.copy_(head.weight.data + 8.0 * fresh)
            assert head.weight._version == version and head.weight.data_ptr() == address
    # a retained graph: the second backward meets a weight written in place in between and remakes the copy
    h = hidden.clone().requires_grad_(True)
    out = models.chunked_replay_logp(head, h, toks, 0.9, chunk=16, transposed_head=True, keep_logits=False)
    (out * up).sum().backward(retain_graph=True)
    first = h.grad.clone()
    h.grad = None
    (out * up).sum().backward()
    assert torch.equal(h.grad, first)
    # nothing is cached between replays, and by default small replays do not use the copy at all
    assert not hasattr(ar_logp, "_TRANSPOSED")
    calls = []
    real = ar_logp.transpose_weight
    ar_logp.transpose_weight = lambda w: (calls.append(1), real(w))[1]
    try:
        h = hidden.clone().requires_grad_(True)
        models.chunked_replay_logp(head, h, toks, 0.9, chunk=16).sum().backward()
        assert not calls and B * T_max < ar_logp.TRANSPOSED_HEAD_MIN_ROWS
        h = hidden.clone().requires_grad_(True)
        models.chunked_replay_logp(head, h, toks, 0.9, chunk=16, transposed_head=True).sum().backward()
        assert len(calls) == 1, "one transposition per replay, shared by its chunks"
    finally:
        ar_logp.transpose_weight = real
