"""GPU parity of the fused LM-head + log-prob / entropy kernels against the oracle (F.linear + log-softmax).

Tolerances follow the reference's own chunked-LM-head test for bf16 operands
(tests/backends/megatron/test_sft_chunked_ce.py:119-134): loss / log-probs 2e-3 abs, gradients 5e-3 abs
(+ one bf16 ulp of output rounding for the bf16 gradients).
"""

import math

import pytest
import torch
import torch.nn.functional as F

from oracle import policy as P
from tests.gpu_util import announce, require_gpu

pytestmark = pytest.mark.gpu

BF16_ULP = 2.0 ** -7


def _inputs(n, h, v, seed, w_scale=0.02):
    g = torch.Generator().manual_seed(seed)
    hid = torch.randn(n, h, generator=g).bfloat16()
    w = (torch.randn(v, h, generator=g) * w_scale).bfloat16()
    tok = torch.randint(0, v, (n,), generator=g)
    return hid, w, tok, g


def _oracle(hid, w, tok, wl, we, temperature):
    h32 = hid.float().requires_grad_()
    w32 = w.float().requires_grad_()
    logits = F.linear(h32, w32) / temperature
    ls = torch.log_softmax(logits, -1)
    lp = ls[torch.arange(hid.size(0)), tok]
    ent = -(ls.exp() * ls).sum(-1)
    ((lp * wl).sum() + (ent * we).sum()).backward()
    return lp.detach(), ent.detach(), h32.grad, w32.grad


@pytest.mark.parametrize("n,h,v,temperature", [
    (256, 64, 256, 1.0),        # exactly one tile
    (300, 128, 1000, 0.7),      # ragged tokens and ragged vocabulary
    (1024, 256, 5000, 1.0),     # several vocab tiles and splits
    (70, 4096, 1030, 1.0),      # production hidden size
    (301, 128, 700, 1.0),       # odd token count: odd slab stride, 2-byte stores in the backward slab
    (300, 128, 9000, 1.0),      # few tokens, 36 vocabulary tiles: 32 vocabulary splits per row block
    (600, 128, 5000, 0.9),      # 20 tiles: 16 splits, the last ones short or empty
])
def test_forward_backward_vs_oracle(n, h, v, temperature):
    from relax_amd.lm_head import lm_head_log_probs_and_entropy

    dev = require_gpu()
    announce("lmhead", n, h, v, temperature)
    hid, w, tok, g = _inputs(n, h, v, seed=n + v, w_scale=0.3 if h < 1024 else 0.05)
    # incoming gradients of the size a mean-reduced loss produces: the backward rounds d loss / d logits to bf16
    # (as autograd does in the reference when the LM head runs in bf16), so O(1) coefficients would put single
    # elements beyond an absolute 5e-3
    wl, we = torch.randn(n, generator=g) / 16, torch.randn(n, generator=g) / 32
    rlp, rent, rgh, rgw = _oracle(hid, w, tok, wl, we, temperature)
    hd, wd = hid.to(dev).requires_grad_(), w.to(dev).requires_grad_()
    lp, ent = lm_head_log_probs_and_entropy(hd, wd, tok.to(dev), temperature, with_entropy=True)
    assert lp.dtype == torch.float32 and lp.shape == (n,) and ent.shape == (n,)
    torch.testing.assert_close(lp.cpu(), rlp, atol=2e-3, rtol=0)
    torch.testing.assert_close(ent.cpu(), rent, atol=2e-3, rtol=0)
    ((lp * wl.to(dev)).sum() + (ent * we.to(dev)).sum()).backward()
    assert hd.grad.dtype == torch.bfloat16 and wd.grad.dtype == torch.bfloat16
    torch.testing.assert_close(hd.grad.float().cpu(), rgh, atol=5e-3, rtol=2 * BF16_ULP)
    torch.testing.assert_close(wd.grad.float().cpu(), rgw, atol=5e-3, rtol=2 * BF16_ULP)
    # deterministic
    lp2, _ = lm_head_log_probs_and_entropy(hid.to(dev), w.to(dev), tok.to(dev), temperature, with_entropy=True)
    assert torch.equal(lp2, lp.detach())


def _oracle_bf16_logits(hid, w, tok, wl, we, temperature):
    """The reference's numerics: F.linear in bf16 (logits rounded to bf16), then fp32 log-softmax
    (relax/backends/megatron/loss.py:405-409); gradients flow through the rounding unchanged."""
    h32 = hid.float().requires_grad_()
    w32 = w.float().requires_grad_()
    raw = F.linear(h32, w32)
    logits = (raw + (raw.bfloat16().float() - raw).detach()) / temperature
    ls = torch.log_softmax(logits, -1)
    lp = ls[torch.arange(hid.size(0)), tok]
    ent = -(ls.exp() * ls).sum(-1)
    ((lp * wl).sum() + (ent * we).sum()).backward()
    return lp.detach(), ent.detach(), h32.grad, w32.grad


@pytest.mark.parametrize("n,h,v,temperature", [
    (256, 64, 256, 1.0),
    (301, 128, 1000, 0.7),      # ragged vocabulary, odd token count (a half-filled token pair at the end)
    (1024, 256, 5000, 1.0),
    (70, 4096, 1030, 1.0),
    (300, 128, 9000, 1.0),      # 32 vocabulary splits per row block
])
def test_keep_logits_forward_backward_vs_bf16_logit_oracle(n, h, v, temperature):
    from relax_amd.lm_head import lm_head_log_probs_and_entropy

    dev = require_gpu()
    announce("lmhead keep_logits", n, h, v, temperature)
    hid, w, tok, g = _inputs(n, h, v, seed=3 * n + v, w_scale=0.3 if h < 1024 else 0.05)
    wl, we = torch.randn(n, generator=g) / 16, torch.randn(n, generator=g) / 32
    rlp, rent, rgh, rgw = _oracle_bf16_logits(hid, w, tok, wl, we, temperature)
    hd, wd = hid.to(dev).requires_grad_(), w.to(dev).requires_grad_()
    lp, ent = lm_head_log_probs_and_entropy(hd, wd, tok.to(dev), temperature, with_entropy=True, keep_logits=True)
    # a logit whose fp32 value sits on a bf16 rounding boundary may round the other way than on the CPU (different
    # summation order): one bf16 ulp of that logit, which only shows where it is the target or carries most of the mass
    close = lambda a, b, tol: ((a - b).abs() <= tol).float().mean().item()
    assert close(lp.detach().cpu(), rlp, 2e-3) >= 0.995, (lp.detach().cpu() - rlp).abs().max()
    torch.testing.assert_close(lp.detach().cpu(), rlp, atol=4e-2, rtol=0)
    torch.testing.assert_close(ent.detach().cpu(), rent, atol=2e-3, rtol=0)
    loss = (lp * wl.to(dev)).sum() + (ent * we.to(dev)).sum()
    loss.backward(retain_graph=True)
    torch.testing.assert_close(hd.grad.float().cpu(), rgh, atol=5e-3, rtol=2 * BF16_ULP)
    torch.testing.assert_close(wd.grad.float().cpu(), rgw, atol=5e-3, rtol=2 * BF16_ULP)
    with pytest.raises(RuntimeError, match="one backward pass"):
        loss.backward()


def test_kept_logits_slab_is_the_bf16_projection_and_stride_parity():
    """The slab the forward pass keeps equals bf16(hidden @ weight^T) transposed; an odd row stride (2-byte stores)
    and an even one (paired 4-byte stores) give the same bytes; the in-place backward equals the recomputing one
    evaluated on the same (rounded) logits to one bf16 ulp."""
    from relax_amd.lm_head import lmhead_dlogits_from_logits_t, lmhead_logprob_fwd

    dev = require_gpu()
    announce("lmhead kept slab")
    n, h, v = 333, 256, 777
    hid, w, tok, g = _inputs(n, h, v, seed=5, w_scale=0.2)
    hd, wd, td = hid.to(dev), w.to(dev), tok.to(dev)
    even = torch.full((v, 336), float("nan"), dtype=torch.bfloat16, device=dev)
    odd = torch.full((v, 335), float("nan"), dtype=torch.bfloat16, device=dev)
    out_e = lmhead_logprob_fwd(hd, wd, td, 1.0, True, logits_t=even)
    out_o = lmhead_logprob_fwd(hd, wd, td, 1.0, True, logits_t=odd)
    assert torch.equal(even[:, :n].view(torch.int16), odd[:, :n].view(torch.int16))
    assert torch.isnan(even[:, n:]).all() and torch.isnan(odd[:, n:]).all()  # padding columns untouched
    for a, b in zip(out_e, out_o):
        assert torch.equal(a, b)
    ref = F.linear(hid.float(), w.float())
    got = even[:, :n].t().float().cpu()
    assert ((got - ref).abs() <= ref.abs() * 2.0 ** -8 + 1e-5).all()  # half a bf16 ulp + fp32 summation order
    assert (got == ref.bfloat16().float()).float().mean() > 0.999
    # statistics of the rounded logits
    lp, ent, lse, spx = out_e
    ls = torch.log_softmax(got, -1)
    torch.testing.assert_close(lp.cpu(), ls[torch.arange(n), tok], atol=1e-4, rtol=0)
    torch.testing.assert_close(ent.cpu(), -(ls.exp() * ls).sum(-1), atol=1e-4, rtol=0)
    # in-place gradient against the closed form on the stored logits
    g_lp = (torch.randn(n, generator=g) / 8).to(dev)
    g_ent = (torch.randn(n, generator=g) / 8).to(dev)
    d_t = lmhead_dlogits_from_logits_t(even, n, td, lse, spx, g_lp, g_ent, 1.0)
    p = ls.exp()
    onehot = F.one_hot(tok, v).float()
    want = g_lp.cpu()[:, None] * (onehot - p) + g_ent.cpu()[:, None] * p * ((p * got).sum(-1, keepdim=True) - got)
    torch.testing.assert_close(d_t.t().float().cpu(), want, atol=1e-5, rtol=2 * BF16_ULP)


@pytest.mark.parametrize("n", [333, 257, 8 * 31 + 1])
def test_in_place_gradient_leaves_the_padding_zero_for_the_backward_gemms(n):
    """n % 8 != 0: relax_amd_lmhead_dlogits_from_logits_t writes whole 16-byte vectors of tokens; the lanes past the
    last token must be zeros, so that a slab whose padding was cleared once goes to relax_amd_lmhead_dweight /
    relax_amd_lmhead_dhidden as it is (their k loop runs over the padded token count) -- no clearing in between."""
    from relax_amd import lm_head as LM

    dev = require_gpu()
    announce("lmhead in-place gradient padding", n)
    h, v = 256, 777
    hid, w, tok, g = _inputs(n, h, v, seed=n, w_scale=0.2)
    hd, wd, td = hid.to(dev), w.to(dev), tok.to(dev)
    slab = LM.alloc_slab(v, n, dev)
    lp, ent, lse, spx = LM.lmhead_logprob_fwd(hd, wd, td, 1.0, True, logits_t=slab[:v])
    g_lp = (torch.randn(n, generator=g) / 8).to(dev)
    g_ent = (torch.randn(n, generator=g) / 8).to(dev)
    # the last token's coefficients are large: if they leaked into the padding lanes the products below would show it
    g_lp[-1], g_ent[-1] = 50.0, 50.0
    d_t = LM.lmhead_dlogits_from_logits_t(slab[:v], n, td, lse, spx, g_lp, g_ent, 1.0)
    assert (slab[:, n:] == 0).all() and (slab[v:] == 0).all()
    d = d_t.float()
    dw = torch.full((v, h), float("nan"), dtype=torch.float32, device=dev)
    LM.lmhead_dweight(slab, n, hd, v, dw)
    dh = torch.full((n, h), float("nan"), dtype=torch.float32, device=dev)
    LM.lmhead_dhidden(slab, n, wd, dh)
    want_dw, want_dh = d @ hd.float(), d.t() @ wd.float()
    torch.testing.assert_close(dw, want_dw, atol=2e-5 * max(1.0, want_dw.abs().max().item()), rtol=1e-5)
    torch.testing.assert_close(dh, want_dh, atol=2e-5 * max(1.0, want_dh.abs().max().item()), rtol=1e-5)


@pytest.mark.parametrize("n,h,v", [
    (256, 256, 256),       # one tile, two k-slice pairs
    (300, 128, 1000),      # ragged in every dimension, hidden size of half a tile
    (777, 384, 1111),      # one and a half tiles of hidden units; odd extents
    (1500, 512, 5000),     # several tiles either way
    (64, 4096, 640),       # production hidden size, fewer tokens than one k-slice pair
    (2048, 256, 8),        # a vocabulary shorter than one k-slice
])
def test_backward_gemms_vs_fp32_matmul(n, h, v):
    """relax_amd_lmhead_dhidden / relax_amd_lmhead_dweight (the two contractions of the gradient slab autograd runs
    through F.linear) against fp32 matmuls of the same bf16 operands: bf16 outputs to one rounding, fp32 outputs and
    fp32 accumulation to accumulation-order noise."""
    from relax_amd import lm_head as LM

    dev = require_gpu()
    announce("lmhead backward gemms", n, h, v)
    g = torch.Generator().manual_seed(n + 3 * v)
    hid = torch.randn(n, h, generator=g).bfloat16().to(dev)
    w = (torch.randn(v, h, generator=g) * 0.5).bfloat16().to(dev)
    d = (torch.randn(v, n, generator=g) * 0.25).bfloat16().to(dev)
    slab = LM.alloc_slab(v, n, dev)
    assert slab.shape == ((v + 127) // 128 * 128, (n + 127) // 128 * 128)
    slab[:v, :n] = d
    want_dh = d.float().t() @ w.float()
    want_dw = d.float() @ hid.float()
    # poisoned outputs: every element must be written, nothing beyond the valid extent
    dh = torch.full((n + 3, h + 8), 7.0, dtype=torch.bfloat16, device=dev)
    LM.lmhead_dhidden(slab, n, w, dh[:n, :h])
    assert (dh[n:] == 7).all() and (dh[:, h:] == 7).all()
    torch.testing.assert_close(dh[:n, :h].float(), want_dh, atol=1e-2 * want_dh.abs().max().item() * BF16_ULP,
                               rtol=BF16_ULP)
    dw = torch.full((v + 3, h + 8), 7.0, dtype=torch.bfloat16, device=dev)
    LM.lmhead_dweight(slab, n, hid, v, dw[:v, :h])
    assert (dw[v:] == 7).all() and (dw[:, h:] == 7).all()
    torch.testing.assert_close(dw[:v, :h].float(), want_dw, atol=1e-2 * want_dw.abs().max().item() * BF16_ULP,
                               rtol=BF16_ULP)
    # fp32 output, then accumulation of a second product on top of it
    dw32 = torch.full((v, h), float("nan"), dtype=torch.float32, device=dev)
    LM.lmhead_dweight(slab, n, hid, v, dw32)
    scale = max(1.0, want_dw.abs().max().item())
    torch.testing.assert_close(dw32, want_dw, atol=2e-5 * scale, rtol=1e-5)
    LM.lmhead_dweight(slab, n, hid, v, dw32, accumulate=True)
    torch.testing.assert_close(dw32, 2 * want_dw, atol=4e-5 * scale, rtol=1e-5)
    dh32 = torch.full((n, h), float("nan"), dtype=torch.float32, device=dev)
    LM.lmhead_dhidden(slab, n, w, dh32)
    torch.testing.assert_close(dh32, want_dh, atol=2e-5 * max(1.0, want_dh.abs().max().item()), rtol=1e-5)
    # clamped reads are multiplied by the slab's zero padding: non-finite values next to the operands' ends in memory
    # must not reach the result (the operands here are views into larger poisoned buffers)
    big_w = torch.full((v + 130, h), float("nan"), dtype=torch.bfloat16, device=dev)
    big_w[:v] = w
    big_h = torch.full((n + 130, h), float("inf"), dtype=torch.bfloat16, device=dev)
    big_h[:n] = hid
    LM.lmhead_dhidden(slab, n, big_w[:v], dh32)
    LM.lmhead_dweight(slab, n, big_h[:n], v, dw32)
    assert torch.isfinite(dh32).all() and torch.isfinite(dw32).all()
    torch.testing.assert_close(dw32, want_dw, atol=2e-5 * scale, rtol=1e-5)


def test_backward_gemm_argument_errors():
    from relax_amd import lm_head as LM
    from relax_amd._lib import KernelError

    dev = require_gpu()
    announce("lmhead backward gemm errors")
    w = torch.zeros(300, 128, dtype=torch.bfloat16, device=dev)
    hid = torch.zeros(200, 128, dtype=torch.bfloat16, device=dev)
    out_h = torch.zeros(200, 128, dtype=torch.bfloat16, device=dev)
    out_w = torch.zeros(300, 128, dtype=torch.bfloat16, device=dev)
    tight = torch.zeros(300, 200, dtype=torch.bfloat16, device=dev)  # neither rows nor columns padded to 128
    with pytest.raises(KernelError, match="ceil128"):
        LM.lmhead_dhidden(tight, 200, w, out_h)
    with pytest.raises(KernelError, match="ceil128"):
        LM.lmhead_dweight(tight, 200, hid, 300, out_w)
    slab = LM.alloc_slab(300, 200, dev)
    with pytest.raises(TypeError):
        LM.lmhead_dweight(slab, 200, hid, 300, out_w, accumulate=True)  # accumulation needs an fp32 output
    with pytest.raises(KernelError, match="ceil128"):
        LM.lmhead_dhidden(slab[:300], 200, w, out_h)  # rows not padded


def test_reference_shaped_case_temperature_and_labels():
    """Shape of the reference's own deferred-LM-head test (T=256, H=32, V=64, weight*0.02, temperature 0.7)."""
    from relax_amd.lm_head import lm_head_log_probs_and_entropy

    dev = require_gpu()
    announce("lmhead reference-shaped")
    torch.manual_seed(0)
    hid = torch.randn(256, 32).bfloat16()
    w = (torch.randn(64, 32) * 0.02).bfloat16()
    tok = torch.randint(0, 64, (256,))
    labels = F.pad(tok[1:], (0, 1), value=0)  # SFT alignment: labels are tokens[1:] + [0]
    want = P.lm_head_log_probs(hid, w, labels, temperature=0.7, sub_chunk=64)
    got, ent = lm_head_log_probs_and_entropy(hid.to(dev), w.to(dev), labels.to(dev), 0.7)
    assert ent is None
    torch.testing.assert_close(got.cpu(), want, atol=2e-3, rtol=0)


def test_slabbed_backward_accumulates_dweight(monkeypatch):
    import relax_amd.lm_head as LH

    dev = require_gpu()
    announce("lmhead slabbed backward")
    monkeypatch.setattr(LH, "BACKWARD_SLAB", 256)
    n, h, v = 700, 64, 900
    hid, w, tok, g = _inputs(n, h, v, seed=3, w_scale=0.3)
    wl = torch.randn(n, generator=g) / 16
    rlp, _, rgh, rgw = _oracle(hid, w, tok, wl, torch.zeros(n), 1.0)
    hd, wd = hid.to(dev).requires_grad_(), w.to(dev).requires_grad_()
    lp, _ = LH.lm_head_log_probs_and_entropy(hd, wd, tok.to(dev))
    (lp * wl.to(dev)).sum().backward()
    torch.testing.assert_close(hd.grad.float().cpu(), rgh, atol=5e-3, rtol=2 * BF16_ULP)
    torch.testing.assert_close(wd.grad.float().cpu(), rgw, atol=5e-3, rtol=2 * BF16_ULP)


@pytest.mark.parametrize("n,h,v,temperature,slab,scale", [
    (700, 64, 900, 1.0, 256, 1.0),       # three slabs, the last one short: dweight accumulated in fp32
    (300, 128, 1000, 0.7, 8192, 1.0),    # one slab
    (1100, 256, 5000, 1.0, 512, 0.25),   # the upstream gradient the caller announced
    (513, 128, 700, 1.3, 384, 1.0),      # a last slab of one token
])
def test_token_local_step_vs_oracle(n, h, v, temperature, slab, scale):
    """``lm_head_token_local_step`` (one projection: every slab's logits become their gradient in place, inside
    forward) with a PPO-clip surrogate + entropy bonus as the token-local loss, against the oracle's F.linear ->
    log-softmax -> same loss in fp32 autograd, and against the two-projection path of ``FusedLMHeadLogProb``."""
    from relax_amd.lm_head import lm_head_log_probs_and_entropy, lm_head_token_local_step

    dev = require_gpu()
    announce("lmhead token-local step", n, h, v, temperature, slab, scale)
    hid, w, tok, g = _inputs(n, h, v, seed=n + v, w_scale=0.3 if h < 1024 else 0.05)
    adv = torch.randn(n, generator=g)
    noise = torch.randn(n, generator=g) * 0.3      # a third of the tokens end up clipped
    mask = (torch.rand(n, generator=g) > 0.2).float()
    denom = mask.sum().clamp_min(1)

    def surrogate(lp, ent, old, a, m, d):
        ratio = torch.exp(lp - old)
        pg = torch.maximum(-a * ratio, -a * ratio.clamp(0.8, 1.28))
        return ((pg - 0.01 * ent) * m).sum() / d

    # oracle, in the reference's numerics: logits rounded to bf16 (F.linear in the weight dtype), fp32 log-softmax
    h32, w32 = hid.float().requires_grad_(), w.float().requires_grad_()
    raw = F.linear(h32, w32)
    lp_unrounded = torch.log_softmax(raw.detach() / temperature, -1)[torch.arange(n), tok]
    ls = torch.log_softmax((raw + (raw.bfloat16().float() - raw).detach()) / temperature, -1)
    rlp = ls[torch.arange(n), tok]
    rent = -(ls.exp() * ls).sum(-1)
    old = rlp.detach() + noise
    want = surrogate(rlp, rent, old, adv, mask, denom)
    (want * scale).backward()

    old_d, adv_d, mask_d, denom_d = old.to(dev), adv.to(dev), mask.to(dev), denom.to(dev)

    def token_loss(b, e, lp, ent):
        return surrogate(lp, ent, old_d[b:e], adv_d[b:e], mask_d[b:e], denom_d)

    hd, wd = hid.to(dev).requires_grad_(), w.to(dev).requires_grad_()
    loss, lp, ent = lm_head_token_local_step(hd, wd, tok.to(dev), token_loss, temperature, with_entropy=True,
                                             slab_tokens=slab, assumed_grad_scale=scale)
    assert loss.requires_grad and not lp.requires_grad and not ent.requires_grad
    torch.testing.assert_close(lp.cpu(), rlp.detach(), atol=2e-3, rtol=0)
    torch.testing.assert_close(ent.cpu(), rent.detach(), atol=2e-3, rtol=0)
    assert abs(loss.item() - want.item()) < 2e-3
    (loss * scale).backward()
    torch.testing.assert_close(hd.grad.float().cpu(), h32.grad, atol=5e-3, rtol=2 * BF16_ULP)
    torch.testing.assert_close(wd.grad.float().cpu(), w32.grad, atol=5e-3, rtol=2 * BF16_ULP)
    with pytest.raises(RuntimeError, match="cannot run twice"):
        (loss * scale).backward()

    # the two-projection path, on a loss without clip boundaries (the two paths' log-probs differ by the bf16
    # rounding of the kept logits, which moves tokens across a clip boundary): gradients equal up to that rounding
    def smooth(lp, ent, a, m, d):
        return ((-a * lp - 0.01 * ent) * m).sum() / d

    h1, w1 = hid.to(dev).requires_grad_(), w.to(dev).requires_grad_()
    loss1, _, _ = lm_head_token_local_step(
        h1, w1, tok.to(dev), lambda b, e, lp, ent: smooth(lp, ent, adv_d[b:e], mask_d[b:e], denom_d), temperature,
        with_entropy=True, slab_tokens=slab)
    loss1.backward()
    h2, w2 = hid.to(dev).requires_grad_(), w.to(dev).requires_grad_()
    lp2, ent2 = lm_head_log_probs_and_entropy(h2, w2, tok.to(dev), temperature, with_entropy=True)
    smooth(lp2, ent2, adv_d, mask_d, denom_d).backward()
    torch.testing.assert_close(h1.grad.float(), h2.grad.float(), atol=5e-3, rtol=2 * BF16_ULP)
    torch.testing.assert_close(w1.grad.float(), w2.grad.float(), atol=5e-3, rtol=2 * BF16_ULP)

    # an upstream gradient other than the announced one: backward rescales what forward produced
    h3, w3 = hid.to(dev).requires_grad_(), w.to(dev).requires_grad_()
    loss3, _, _ = lm_head_token_local_step(h3, w3, tok.to(dev), token_loss, temperature, with_entropy=True,
                                           slab_tokens=slab, assumed_grad_scale=scale)
    (loss3 * (3.0 * scale)).backward()
    torch.testing.assert_close(h3.grad.float(), 3.0 * hd.grad.float(), atol=1e-6, rtol=2 * BF16_ULP)
    torch.testing.assert_close(w3.grad.float(), 3.0 * wd.grad.float(), atol=1e-6, rtol=2 * BF16_ULP)

    # without gradients: the plain forward, no slab of logits (so nothing is rounded to bf16 on the way)
    with torch.no_grad():
        loss4, lp4, _ = lm_head_token_local_step(hid.to(dev), w.to(dev), tok.to(dev), token_loss, temperature,
                                                 with_entropy=True, slab_tokens=slab)
    assert not loss4.requires_grad and torch.isfinite(loss4)
    torch.testing.assert_close(lp4.cpu(), lp_unrounded, atol=2e-3, rtol=0)


def test_token_local_step_empty_input_and_weight_only_gradient():
    from relax_amd.lm_head import lm_head_token_local_step

    dev = require_gpu()
    announce("lmhead token-local step: empty / weight-only")
    hid, w, tok, g = _inputs(300, 128, 640, seed=11, w_scale=0.3)
    coef = (torch.randn(300, generator=g) / 16).to(dev)
    wd = w.to(dev).requires_grad_()
    loss, lp, ent = lm_head_token_local_step(hid.to(dev)[:0], wd, tok.to(dev)[:0], lambda b, e, lp, _: lp.sum())
    assert ent is None and lp.numel() == 0 and loss.item() == 0
    loss.backward()
    assert wd.grad is not None and not wd.grad.any()
    # only the weight wants a gradient
    wd.grad = None
    loss, _, _ = lm_head_token_local_step(hid.to(dev), wd, tok.to(dev), lambda b, e, lp, _: (lp * coef[b:e]).sum(),
                                          slab_tokens=128)
    loss.backward()
    _, _, _, rgw = _oracle(hid, w, tok, coef.cpu(), torch.zeros(300), 1.0)
    torch.testing.assert_close(wd.grad.float().cpu(), rgw, atol=5e-3, rtol=2 * BF16_ULP)


def test_argument_errors():
    from relax_amd.lm_head import lm_head_log_probs_and_entropy, lmhead_logprob_fwd

    dev = require_gpu()
    hid = torch.randn(8, 48, device=dev).bfloat16()  # hidden size not a multiple of 128: the raw op refuses ...
    w = torch.randn(16, 48, device=dev).bfloat16()
    tok = torch.zeros(8, dtype=torch.long, device=dev)
    with pytest.raises(Exception, match="multiple of 128"):
        lmhead_logprob_fwd(hid, w, tok)
    lp, _ = lm_head_log_probs_and_entropy(hid, w, tok)  # ... and the wrapper pads
    want = torch.log_softmax(hid.float() @ w.float().t(), -1)[:, 0]
    torch.testing.assert_close(lp, want, atol=2e-3, rtol=0)
    with pytest.raises(TypeError, match="bfloat16"):
        lm_head_log_probs_and_entropy(hid.float(), w, tok)


def test_full_size_forward_and_gradient_properties():
    """The benchmark shape (hidden [32768, 4096] x weight [151936, 4096]): sampled rows against a library fp32
    matmul + log_softmax, range properties for every row, and gradient identities that hold at any size --
    sum_v dlogits = 0 makes dhidden orthogonal to nothing in particular, but the weight gradient of a constant shift is
    zero: sum_v dweight[v, :] = sum_n dlogits_rowsum[n] * hidden[n, :] = 0."""
    from relax_amd.lm_head import lm_head_log_probs_and_entropy

    dev = require_gpu()
    n, h, v = 32768, 4096, 151936
    announce("lmhead full size", n, h, v)
    g = torch.Generator(device=dev).manual_seed(0)
    hid = torch.randn(n, h, device=dev, generator=g).bfloat16().requires_grad_()
    w = (torch.randn(v, h, device=dev, generator=g) * 0.02).bfloat16().requires_grad_()
    tok = torch.randint(0, v, (n,), device=dev, generator=g)
    lp, ent = lm_head_log_probs_and_entropy(hid, w, tok, 1.0, True, False)
    assert torch.isfinite(lp).all() and (lp <= 0).all()
    assert (ent >= 0).all() and (ent <= math.log(v) + 1e-3).all()
    idx = torch.arange(0, n, n // 64, device=dev)
    ref = torch.log_softmax(hid.detach()[idx].float() @ w.detach().float().t(), -1)
    torch.testing.assert_close(lp.detach()[idx], ref[torch.arange(idx.numel(), device=dev), tok[idx]], atol=2e-3, rtol=0)
    torch.testing.assert_close(ent[idx], -(ref.exp() * ref).sum(-1), atol=2e-3, rtol=0)
    del ref
    adv = torch.randn(n, device=dev, generator=g) / n
    (-(adv * lp)).sum().backward()
    assert torch.isfinite(hid.grad).all() and torch.isfinite(w.grad).all()
    # a uniform shift of every logit changes no log-prob: the weight gradient summed over the vocabulary vanishes
    col = w.grad.float().sum(0)
    assert col.abs().max().item() < 2e-3 * max(1.0, w.grad.float().abs().sum(0).max().item())
    # sampled rows of dhidden against the closed form  dh_n = -adv_n * (w[tok_n] - sum_v p_v w_v)
    pick = idx[:8]
    p = torch.softmax(hid.detach()[pick].float() @ w.detach().float().t(), -1)
    want = -adv[pick, None] * (w.detach()[tok[pick]].float() - p @ w.detach().float())
    torch.testing.assert_close(hid.grad[pick].float(), want, atol=2e-3 * want.abs().max().item(), rtol=2 * BF16_ULP)

    # the same step with one projection (four slabs of 8192 rows whose logits become their gradient in place): the
    # same identities, and gradients that agree with the two-projection ones up to the bf16 rounding of the logits
    from relax_amd.lm_head import lm_head_token_local_step

    hid2, w2 = hid.detach().clone().requires_grad_(), w.detach().clone().requires_grad_()
    loss, lp2, ent2 = lm_head_token_local_step(hid2, w2, tok, lambda b, e, lp_, _: -(adv[b:e] * lp_).sum(), 1.0,
                                               with_entropy=True)
    # its statistics come from the logits rounded to bf16 (the reference's numerics: F.linear in bf16, then .float())
    ref = torch.log_softmax((hid.detach()[idx] @ w.detach().t()).float(), -1)
    torch.testing.assert_close(lp2[idx], ref[torch.arange(idx.numel(), device=dev), tok[idx]], atol=2e-3, rtol=0)
    torch.testing.assert_close(ent2[idx], -(ref.exp() * ref).sum(-1), atol=2e-3, rtol=0)
    del ref
    assert (lp2 - lp.detach()).abs().max().item() < 4e-2  # one bf16 ulp of a target logit of magnitude < 8
    assert abs(loss.item() + (adv * lp.detach()).sum().item()) < 2e-3
    loss.backward()
    col = w2.grad.float().sum(0)
    assert col.abs().max().item() < 2e-3 * max(1.0, w2.grad.float().abs().sum(0).max().item())
    torch.testing.assert_close(hid2.grad[pick].float(), want, atol=2e-3 * want.abs().max().item(), rtol=2 * BF16_ULP)
    scale_h, scale_w = hid.grad.float().abs().max().item(), w.grad.float().abs().max().item()
    torch.testing.assert_close(hid2.grad.float(), hid.grad.float(), atol=2e-2 * scale_h, rtol=4 * BF16_ULP)
    for r0 in range(0, v, 16384):  # in pieces: a full fp32 copy of both weight gradients is 5 GB
        torch.testing.assert_close(w2.grad[r0:r0 + 16384].float(), w.grad[r0:r0 + 16384].float(), atol=2e-2 * scale_w,
                                   rtol=4 * BF16_ULP)


def test_sft_losses_plain_and_with_deferred_lm_head_vs_oracle():
    """sft_loss_function on logits and sft_loss_function_chunked on hidden states + LM-head weight (handed over as a
    module, a bound forward or the tensor) against the oracle's F.linear -> log-softmax -> sample-mean composition,
    forward and gradients; loss_function dispatch for ``loss_type="sft"``."""
    import relax_amd
    from oracle import reducers as R
    from relax_amd.cp_utils import get_sum_of_sample_mean

    dev = require_gpu()
    announce("sft losses")
    g = torch.Generator().manual_seed(4)
    tot, resp, h, v = [7, 12, 5], [7, 5, 5], 128, 300     # SFT-shaped and RL-shaped samples mixed
    t = sum(tot)
    hid = torch.randn(1, t, h, generator=g).bfloat16()
    head = torch.nn.Linear(h, v, bias=False)
    with torch.no_grad():
        head.weight.copy_(torch.randn(v, h, generator=g) * 0.1)
    head = head.bfloat16()
    toks = [torch.randint(0, v, (n,), generator=g) for n in tot]
    masks = [(torch.rand(r, generator=g) > 0.2).float() for r in resp]
    batch = dict(unconcat_tokens=toks, total_lengths=tot, response_lengths=resp, loss_masks=masks)
    args = P.make_args(loss_type="sft", sft_chunked_logits=True, rollout_temperature=0.9, global_batch_size=3)
    # oracle: materialised logits in the weight dtype, fp32 log-softmax, sample mean
    hc, wc = hid.clone().requires_grad_(), head.weight.detach().clone().requires_grad_()
    lps = []
    for (b, e, _), tk, r in zip(P.response_row_ranges(tot, resp), toks, resp):
        tg = F.pad(tk[1:], (0, 1), value=0) if r == tk.numel() else tk[-r:]
        lps.append(P.lm_head_log_probs(hc[0, b:e], wc, tg, temperature=0.9, sub_chunk=4))
    want = -R.make_reducer(resp, masks)(torch.cat(lps))
    want.backward()
    dbatch = dict(unconcat_tokens=[x.to(dev) for x in toks], total_lengths=tot, response_lengths=resp,
                  loss_masks=[m.to(dev) for m in masks])
    dhead = torch.nn.Linear(h, v, bias=False).bfloat16().to(dev)
    with torch.no_grad():
        dhead.weight.copy_(head.weight)
    for handle, single in ((dhead, "auto"), (dhead.forward, "off"), (dhead.weight, "auto")):
        # "auto": the one-projection step (each token's weight in the loss read off the reducer); "off": log-probs
        # from the forward kernel, backward through a second projection
        args.relax_amd_single_pass = single
        hd = hid.to(dev).requires_grad_()
        dhead.weight.grad = None
        loss, log = relax_amd.sft_loss_function_chunked(args, dbatch, hd, None, lm_head_forward=handle)
        loss.backward()
        # the oracle rounds the logits to bf16 before the softmax (as F.linear in the weight dtype does); the kernel
        # keeps fp32 accumulators: 2e-3 per sample mean, three samples summed
        assert abs(loss.item() - want.item()) < 2e-3 * len(resp) and abs(log["loss"].item() - loss.item()) == 0
        torch.testing.assert_close(hd.grad.float().cpu(), hc.grad.float(), atol=5e-3, rtol=2 * BF16_ULP)
        torch.testing.assert_close(dhead.weight.grad.float().cpu(), wc.grad.float(), atol=5e-3, rtol=2 * BF16_ULP)
    # a caller's own reducer (not known to be a fixed weighted sum) keeps log-probs-through-autograd: same results
    args.relax_amd_single_pass = "auto"
    lib_reducer = get_sum_of_sample_mean(tot, resp, dbatch["loss_masks"], False)
    hd = hid.to(dev).requires_grad_()
    dhead.weight.grad = None
    loss, _ = relax_amd.sft_loss_function_chunked(args, dbatch, hd, lambda x: lib_reducer(x),
                                                  lm_head_forward=dhead.forward)
    loss.backward()
    assert abs(loss.item() - want.item()) < 2e-3 * len(resp)
    torch.testing.assert_close(hd.grad.float().cpu(), hc.grad.float(), atol=5e-3, rtol=2 * BF16_ULP)
    # the same loss from materialised logits
    logits = (hid[0].to(dev) @ dhead.weight.detach().t()).float().unsqueeze(0).requires_grad_()
    loss2, _ = relax_amd.sft_loss_function(args, dbatch, logits, None)
    assert abs(loss2.item() - want.item()) < 2e-3 * len(resp)
    # loss_function: Megatron scaling (num_microbatches / global_batch_size) and the logging dict
    hd = hid.to(dev).requires_grad_()
    dhead.weight.grad = None
    scaled, normalizer, logd = relax_amd.loss_function(args, dbatch, 2, hd, lm_head_forward=dhead.forward)
    assert abs(scaled.item() - want.item() * 2 / 3) < 2e-3 * len(resp) and logd["keys"] == ["loss"] and int(normalizer) == 1
    scaled.backward()  # the step produced its gradients for the scale loss_function applies
    torch.testing.assert_close(hd.grad.float().cpu(), hc.grad.float() * 2 / 3, atol=5e-3, rtol=2 * BF16_ULP)
    torch.testing.assert_close(dhead.weight.grad.float().cpu(), wc.grad.float() * 2 / 3, atol=5e-3, rtol=2 * BF16_ULP)
    with pytest.raises(NotImplementedError, match="expose the LM-head weight"):
        relax_amd.sft_loss_function_chunked(args, dbatch, hd, None, lm_head_forward=lambda x: x)


def test_model_forward_under_bypass_feeds_the_fused_loss_end_to_end():
    """A small model run under ``bypass_output_layer`` returns hidden states; ``loss_function`` with the yielded handle
    gives the loss and the gradients (LM-head weight and the layers below it) of the same model run normally with
    materialised logits, to the bf16 tolerances of the reference's chunked-LM-head test."""
    import relax_amd
    from relax_amd.model import bypass_output_layer

    dev = require_gpu()
    announce("bypass end to end")

    class Head(torch.nn.Module):
        def __init__(self, h, v):
            super().__init__()
            self.weight = torch.nn.Parameter(torch.randn(v, h) * 0.1)

        def forward(self, input_, weight=None, runtime_gather_output=None):
            return F.linear(input_, self.weight if weight is None else weight), None

    class Tiny(torch.nn.Module):
        def __init__(self, v, h):
            super().__init__()
            self.embed = torch.nn.Embedding(v, h)
            self.mix = torch.nn.Linear(h, h)
            self.output_layer = Head(h, v)

        def forward(self, tokens):
            x = torch.tanh(self.mix(self.embed(tokens)))
            return self.output_layer(x)[0]

    torch.manual_seed(3)
    v, h, tot, resp = 300, 128, [9, 14, 6], [9, 6, 6]
    model = Tiny(v, h).bfloat16().to(dev)
    g = torch.Generator().manual_seed(8)
    toks = [torch.randint(0, v, (n,), generator=g).to(dev) for n in tot]
    masks = [(torch.rand(r, generator=g) > 0.2).float().to(dev) for r in resp]
    batch = dict(unconcat_tokens=toks, total_lengths=tot, response_lengths=resp, loss_masks=masks)
    args = P.make_args(loss_type="sft", sft_chunked_logits=True, global_batch_size=3)
    packed = torch.cat(toks).unsqueeze(0)

    logits = model(packed).float()
    want, _, _ = relax_amd.loss_function(P.make_args(loss_type="sft", global_batch_size=3), batch, 1, logits)
    want.backward()
    ref_grads = {k: p.grad.clone() for k, p in model.named_parameters()}
    model.zero_grad()

    with bypass_output_layer(model) as head:
        hidden = model(packed)
        assert hidden.shape == (1, sum(tot), h) and hidden.dtype == torch.bfloat16
        loss, _, log = relax_amd.loss_function(args, batch, 1, hidden, lm_head_forward=head)
    loss.backward()
    assert abs(loss.item() - want.item()) < 2e-3 * len(resp)
    for k, p in model.named_parameters():
        torch.testing.assert_close(p.grad.float(), ref_grads[k].float(), atol=5e-3, rtol=4 * BF16_ULP, msg=k)
    assert torch.equal(model(packed).float(), logits)  # the layer projects again once the block is left
