"""GPU parity of the log-prob / entropy kernels against the oracle, through the C ABI (ctypes).

Tolerances: fp32 inputs 2e-5 abs (fp32 accumulation, different summation order); bf16 / fp16 inputs 2e-3 abs on
log-probs, entropy and gradients (the bound the benchmark states); indices and masks exact.
"""

import math

import pytest
import torch

from oracle import logprob as O
from tests.gpu_util import announce, require_gpu, spiked_logits

pytestmark = pytest.mark.gpu


def _oracle(x_cpu, tok_cpu, wl, we, inv_t=1.0):
    x = x_cpu.clone().requires_grad_()
    xs = x.float() * inv_t if inv_t != 1.0 else x
    lp, ent = O.calculate_log_probs_and_entropy(xs, tok_cpu, None, with_entropy=True)
    ((lp.squeeze(-1) * wl).sum() + (ent * we).sum()).backward()
    return lp.squeeze(-1).detach(), ent.detach(), x.grad


@pytest.mark.parametrize("key", ["logprob_single_rank", "logprob_two_shards"])
def test_reference_literals(literals, key):
    import relax_amd

    dev = require_gpu()
    fx = literals[key]
    announce("literals", key)
    x = torch.tensor(fx["logits"], device=dev, requires_grad=True)
    tok = torch.tensor(fx["tokens"], device=dev)
    wl, we = torch.tensor(fx["logprob_weights"]), torch.tensor(fx["entropy_weights"])
    for chunk in (-1, 1, 2, 8):
        x.grad = None
        lp, ent = relax_amd.calculate_log_probs_and_entropy(x, tok, None, with_entropy=True, chunk_size=chunk)
        assert lp.shape == (len(fx["tokens"]), 1) and lp.dtype == torch.float32
        ((lp.squeeze(-1) * wl.to(dev)).sum() + (ent * we.to(dev)).sum()).backward()
        rlp, rent, rg = _oracle(torch.tensor(fx["logits"]), torch.tensor(fx["tokens"]), wl, we)
        torch.testing.assert_close(lp.squeeze(-1).cpu(), rlp, atol=2e-6, rtol=0)
        torch.testing.assert_close(ent.cpu(), rent, atol=2e-6, rtol=0)
        torch.testing.assert_close(x.grad.cpu(), rg, atol=2e-6, rtol=0)


@pytest.mark.parametrize(
    "n,v,dtype,scale,tol",
    [
        (64, 1003, torch.float32, 2.0, 2e-5),      # unaligned stride -> scalar path
        (48, 4096, torch.float32, 2.0, 2e-5),      # vector path, exact multiple of the unroll
        (33, 32000, torch.float32, 2.0, 2e-5),     # first benchmark configuration's vocabulary
        (40, 4100, torch.bfloat16, 3.0, 2e-3),     # vector path + remainder vectors + scalar tail (4100 % 8 = 4)
        (24, 151936, torch.bfloat16, 3.0, 2e-3),   # headline vocabulary, spiked rows
        (24, 151936, torch.float16, 3.0, 2e-3),
        (24, 151936, torch.float32, 3.0, 2e-5),    # what stock Megatron hands the custom-loss hook (loss.py:92-97)
        (3, 7, torch.bfloat16, 1.0, 2e-3),
    ],
)
@pytest.mark.parametrize("inv_t", [1.0, 1 / 0.7])
def test_forward_backward_vs_oracle(n, v, dtype, scale, tol, inv_t):
    from relax_amd import ops

    dev = require_gpu()
    announce("fwd/bwd", n, v, dtype, inv_t)
    x = spiked_logits(n, v, scale, dtype, seed=n + v, device=dev)
    g = torch.Generator().manual_seed(7)
    tok = torch.randint(0, v, (n,), generator=g)
    wl, we = torch.randn(n, generator=g), torch.randn(n, generator=g) * 0.3
    wl[0] = 0.0
    we[0] = 0.0  # a zero-gradient row must come back exactly zero
    lp, ent, lse, spx = ops.logprob_entropy_fwd(x, tok.to(dev), None, inv_t, True)
    d = ops.logprob_entropy_bwd(x, tok.to(dev), lse, spx, wl.to(dev), we.to(dev), inv_temperature=inv_t)
    rlp, rent, rg = _oracle(x.cpu(), tok, wl, we, inv_t)
    assert lp.dtype == torch.float32 and d.dtype == dtype and d.shape == x.shape
    torch.testing.assert_close(lp.cpu(), rlp, atol=tol, rtol=0)
    torch.testing.assert_close(ent.cpu(), rent, atol=tol, rtol=0)
    # gradients come back in the logits dtype: allow one ulp of that dtype's output rounding on top of the bound
    ulp = {torch.float32: 0.0, torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10}[dtype]
    torch.testing.assert_close(d.float().cpu(), rg.float(), atol=tol, rtol=ulp)
    assert d[0].abs().max().item() == 0.0
    # run-to-run determinism (forward-only pass and training pass must agree bit for bit)
    lp2, ent2, _, _ = ops.logprob_entropy_fwd(x, tok.to(dev), None, inv_t, True)
    assert torch.equal(lp, lp2) and torch.equal(ent, ent2)
    # a forward without entropy returns the same log-probs
    lp3, ent3, _, spx3 = ops.logprob_entropy_fwd(x, tok.to(dev), None, inv_t, False)
    assert ent3 is None and spx3 is None
    # (its scan leaves the sum of p * x out; the maximum and the sum of exponentials are the same arithmetic)
    assert torch.equal(lp3, lp) and torch.equal(_, lse)


def test_keep_mask_reference_literal_and_random_rows(literals):
    """log_prob_keep_mask: the reference test's literal case, then random rows in every dtype (the target is kept
    whatever the mask says; entropy ignores the mask), values and gradients against the oracle."""
    import relax_amd

    dev = require_gpu()
    fx = literals["logprob_single_rank"]
    announce("keep mask literal")
    keep = torch.tensor(fx["keep_mask"])
    wl, we = torch.tensor(fx["logprob_weights"]), torch.tensor(fx["entropy_weights"])
    xc = torch.tensor(fx["logits"], requires_grad=True)
    tok = torch.tensor(fx["tokens"])
    lp, ent = O.calculate_log_probs_and_entropy(xc, tok, None, with_entropy=True, log_prob_keep_mask=keep)
    ((lp.squeeze(-1) * wl).sum() + (ent * we).sum()).backward()
    xd = torch.tensor(fx["logits"], device=dev, requires_grad=True)
    glp, gent = relax_amd.calculate_log_probs_and_entropy(xd, tok.to(dev), None, with_entropy=True,
                                                          log_prob_keep_mask=keep.to(dev))
    ((glp.squeeze(-1) * wl.to(dev)).sum() + (gent * we.to(dev)).sum()).backward()
    torch.testing.assert_close(glp.cpu(), lp.detach(), atol=2e-6, rtol=0)
    torch.testing.assert_close(gent.cpu(), ent.detach(), atol=2e-6, rtol=0)
    torch.testing.assert_close(xd.grad.cpu(), xc.grad, atol=2e-6, rtol=0)
    for n, v, dtype, tol in ((9, 1003, torch.float32, 3e-5), (6, 151936, torch.bfloat16, 2e-3),
                             (7, 4104, torch.float16, 2e-3)):
        announce("keep mask", n, v, dtype)
        g = torch.Generator().manual_seed(v)
        x = (torch.randn(n, v, generator=g) * 3).to(dtype)
        tok = torch.randint(0, v, (n,), generator=g)
        keep = torch.rand(n, v, generator=g) < 0.3
        keep[0] = True                       # nothing masked: must equal the unmasked path
        keep[1] = False                      # everything masked: only the target survives, log-prob 0
        wl, we = torch.randn(n, generator=g), torch.randn(n, generator=g)
        xc = x.clone().float().requires_grad_()
        lp, ent = O.calculate_log_probs_and_entropy(xc, tok, None, with_entropy=True, log_prob_keep_mask=keep)
        ((lp.squeeze(-1) * wl).sum() + (ent * we).sum()).backward()
        xd = x.to(dev).requires_grad_()
        glp, gent = relax_amd.calculate_log_probs_and_entropy(xd, tok.to(dev), None, with_entropy=True,
                                                              log_prob_keep_mask=keep.to(dev))
        ((glp.squeeze(-1) * wl.to(dev)).sum() + (gent * we.to(dev)).sum()).backward()
        torch.testing.assert_close(glp.cpu(), lp.detach(), atol=tol, rtol=0)
        torch.testing.assert_close(gent.cpu(), ent.detach(), atol=tol, rtol=0)
        ulp = {torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10, torch.float32: 1e-5}[dtype]
        torch.testing.assert_close(xd.grad.float().cpu(), xc.grad, atol=tol, rtol=ulp)
        assert abs(glp[1].item()) < 1e-6
        plain, _ = relax_amd.calculate_log_probs_and_entropy(x.to(dev), tok.to(dev), None, with_entropy=False)
        assert abs(plain[0].item() - glp[0].item()) < 1e-5
        # metric-only entropy: no entropy gradient reaches the logits
        xd2 = x.to(dev).requires_grad_()
        l2, e2 = relax_amd.calculate_log_probs_and_entropy(xd2, tok.to(dev), None, with_entropy=True,
                                                           log_prob_keep_mask=keep.to(dev), with_entropy_grad=False)
        assert not e2.requires_grad
        l2.sum().backward()


def test_autograd_function_semantics(literals):
    import relax_amd

    dev = require_gpu()
    announce("autograd semantics")
    fx = literals["logprob_single_rank"]
    x = torch.tensor(fx["logits"], device=dev, requires_grad=True)
    tok = torch.tensor(fx["tokens"], device=dev)
    lp, ent = relax_amd.calculate_log_probs_and_entropy(x, tok, None, with_entropy=True, with_entropy_grad=False)
    assert lp.requires_grad and not ent.requires_grad
    lp, ent = relax_amd.calculate_log_probs_and_entropy(x, tok, None, with_entropy=False)
    assert ent is None
    empty = torch.zeros(0, 4, device=dev)
    lp, ent = relax_amd.calculate_log_probs_and_entropy(empty, torch.zeros(0, dtype=torch.long, device=dev), None, True)
    assert lp.shape == (0,) and ent.shape == (0,)
    # bf16 logits: fp32 outputs, gradient in the logits dtype
    xb = torch.randn(5, 64, device=dev).bfloat16().requires_grad_()
    lp, _ = relax_amd.calculate_log_probs_and_entropy(xb, torch.randint(0, 64, (5,), device=dev), None)
    assert lp.dtype == torch.float32
    lp.sum().backward()
    assert xb.grad.dtype == torch.bfloat16
    # inputs are never written
    before = xb.detach().clone()
    relax_amd.calculate_log_probs_and_entropy(xb, torch.randint(0, 64, (5,), device=dev), None, True)
    assert torch.equal(before, xb.detach())


def test_strided_rows_row_ids_and_inverse_map():
    from relax_amd import ops

    dev = require_gpu()
    announce("row maps")
    t_rows, v = 23, 520
    big = torch.randn(t_rows, v + 8, device=dev)
    x = big[:, :v]  # row stride v+8: still 16-byte aligned rows
    begins = torch.tensor([2, 9, 15], device=dev)
    lens = [3, 4, 5]
    cu = torch.tensor([0, 3, 7, 12], device=dev)
    row_ids, sample_ids, inv = ops.build_row_maps(begins, cu, 12, t_rows)
    want_rows = [2, 3, 4, 9, 10, 11, 12, 15, 16, 17, 18, 19]
    assert row_ids.tolist() == want_rows
    assert sample_ids.tolist() == [0] * 3 + [1] * 4 + [2] * 5
    want_inv = [-1] * t_rows
    for k, r in enumerate(want_rows):
        want_inv[r] = k
    assert inv.tolist() == want_inv
    tok = torch.randint(0, v, (12,), device=dev)
    lp, ent, lse, spx = ops.logprob_entropy_fwd(x, tok, row_ids, 1.0, True)
    ref = torch.log_softmax(x[want_rows].double(), -1)
    torch.testing.assert_close(lp.double(), ref[torch.arange(12), tok], atol=2e-5, rtol=0)
    g = torch.randn(12, device=dev)
    d = ops.logprob_entropy_bwd(x, tok, lse, spx, g, None, token_of_row=inv)
    assert d.shape == (t_rows, v)
    untouched = [r for r in range(t_rows) if r not in want_rows]
    assert d[untouched].abs().max().item() == 0.0
    p = ref.exp()
    want = -p * g.double()[:, None]
    want[torch.arange(12), tok] += g.double()
    torch.testing.assert_close(d[want_rows].double(), want, atol=2e-5, rtol=0)


def test_invalid_target_gives_nan_not_a_fault():
    from relax_amd import ops

    dev = require_gpu()
    announce("invalid target")
    x = torch.randn(4, 64, device=dev)
    tok = torch.tensor([0, 64, -1, 63], device=dev)
    lp, _, _, _ = ops.logprob_entropy_fwd(x, tok, None, 1.0, True)
    assert torch.isnan(lp[1]) and torch.isnan(lp[2]) and torch.isfinite(lp[0]) and torch.isfinite(lp[3])


def test_full_size_properties_headline_shape():
    """Size-independent properties at the benchmark's vocabulary on a 4096-row slab, plus an oracle spot check."""
    from relax_amd import ops

    dev = require_gpu()
    n, v = 4096, 151936
    announce("full-size properties", n, v)
    g = torch.Generator(device=dev).manual_seed(0)
    x = (torch.randn(n, v, device=dev, generator=g) * 3.0).bfloat16()
    tok = torch.randint(0, v, (n,), device=dev, generator=g)
    lp, ent, lse, spx = ops.logprob_entropy_fwd(x, tok, None, 1.0, True)
    assert (lp <= 0).all() and (ent >= 0).all() and (ent <= math.log(v) + 1e-3).all()
    # shift invariance: adding a constant representable in bf16 steps changes nothing beyond rounding of x itself
    glp = torch.randn(n, device=dev, generator=g)
    gen = torch.randn(n, device=dev, generator=g) * 0.1
    d = ops.logprob_entropy_bwd(x, tok, lse, spx, glp, gen)
    rowsum = d.float().sum(-1)
    assert rowsum.abs().max().item() < 5e-2  # sum_v dlogits = 0 up to bf16 rounding of 151936 terms
    idx = torch.arange(0, n, 128, device=dev)
    xs = x[idx].cpu()
    rlp, rent = O.calculate_log_probs_and_entropy(xs, tok[idx].cpu(), None, with_entropy=True)
    torch.testing.assert_close(lp[idx].cpu(), rlp.squeeze(-1), atol=2e-3, rtol=0)
    torch.testing.assert_close(ent[idx].cpu(), rent, atol=2e-3, rtol=0)


@pytest.mark.parametrize("v,dtype,n", [(151936, torch.bfloat16, 700), (8 * (18 * 1024 + 1), torch.bfloat16, 300),
                                       (128256, torch.float16, 600), (131072, torch.bfloat16, 40),
                                       (100352, torch.bfloat16, 1100), (8 * (16 * 1024 - 1), torch.float16, 300),
                                       (163840, torch.bfloat16, 300), (8 * (19 * 1024 + 1), torch.float16, 520),
                                       (32000, torch.float32, 1500), (4 * (8 * 1024 - 1), torch.float32, 700),
                                       (64000, torch.bfloat16, 900), (65536, torch.float16, 600),
                                       (50304, torch.float32, 700), (65536, torch.float32, 500)])
def test_backward_burst_form_equals_row_per_workgroup_kernel_bitwise(v, dtype, n):
    """The three kernels behind relax_amd_logprob_entropy_bwd, switched with relax_amd_set_kernel_choice (the default:
    one-shot workgroups that take 4 KB of a row each; the row-per-workgroup loop; the persistent burst form), on every
    row shape the burst form is built for (and the ends of two of them), with rows that score no token, tokens
    without gradient (zero rows, in runs and scattered), a device-side gradient scale and targets on a row's first and
    last element: bit-identical gradients."""
    from relax_amd import ops

    dev = require_gpu()
    announce("backward: burst form vs row-per-workgroup", v, dtype, n)
    g = torch.Generator().manual_seed(v + n)
    x = (torch.randn(n, v, generator=g) * 2).to(dtype).to(dev)
    scores = torch.rand(n, generator=g) > 0.2
    idx = torch.cumsum(scores.int(), 0) - 1
    token_of_row = torch.where(scores, idx, torch.full_like(idx, -1)).int().to(dev)
    row_ids = torch.nonzero(scores).flatten().int().to(dev)
    n_tok = int(scores.sum())
    tok = torch.randint(0, v, (n_tok,), generator=g)
    tok[:3] = torch.tensor([0, v - 1, v - 2])
    tok = tok.to(dev)
    lp, ent, lse, spx = ops.logprob_entropy_fwd(x, tok, row_ids, 0.8, True)
    glp = torch.randn(n_tok, generator=g)
    gen = torch.randn(n_tok, generator=g) * 0.1
    dead = torch.rand(n_tok, generator=g) < 0.25
    dead[n_tok // 2:n_tok // 2 + 12] = True
    glp[dead] = 0.0
    gen[dead] = 0.0
    scale = torch.tensor([0.37], device=dev)
    outs = {}
    for kind in ("cached", "resident", "auto"):
        ops.set_kernel_choice({"cached": "two_walk"}.get(kind, kind))
        for with_ent in (True, False):
            d = ops.logprob_entropy_bwd(x, tok, lse, spx, glp.to(dev), gen.to(dev) if with_ent else None,
                                        token_of_row=token_of_row, grad_scale_dev=scale, inv_temperature=0.8)
            torch.cuda.synchronize()
            outs[kind, with_ent] = d.view(torch.int16 if dtype != torch.float32 else torch.int32)
    for with_ent in (True, False):
        assert torch.equal(outs["resident", with_ent], outs["cached", with_ent]), with_ent
        assert torch.equal(outs["auto", with_ent], outs["cached", with_ent]), with_ent
        assert outs["resident", with_ent].any()
    zero_rows = torch.ones(n, dtype=torch.bool)
    zero_rows[row_ids.cpu().long()[~dead]] = False
    assert not outs["resident", True][zero_rows.to(dev)].any()


# ------------------------------------------------------------------------------------------------- top-K selection


def _check_topk_rows(x, k, row_ids=None):
    """values equal torch.topk's exactly and are sorted; every index is valid, distinct and points at its value;
    where a value is strictly greater than the k-th value the index must be among torch's."""
    from relax_amd import ops

    vals, idx = ops.topk_rows(x, row_ids, k)
    rows = x if row_ids is None else x[row_ids.long()]
    want = torch.topk(rows.float(), k, dim=-1)
    got_v, want_v = vals, want.values
    same = (got_v == want_v) | (torch.isnan(got_v) & torch.isnan(want_v))
    assert same.all(), (got_v[~same][:5], want_v[~same][:5])
    assert idx.dtype == torch.int64 and (idx >= 0).all() and (idx < x.size(1)).all()
    gathered = torch.gather(rows.float(), 1, idx)
    ok = (gathered == got_v) | (torch.isnan(gathered) & torch.isnan(got_v))
    assert ok.all()
    assert (torch.sort(idx, dim=1).values.diff(dim=1) > 0).all() or k == 1  # distinct
    kth = want_v[:, -1:]
    strict = got_v > kth
    for r in range(min(rows.size(0), 64)):  # set equality above the threshold (ties at the threshold may differ)
        assert set(idx[r][strict[r]].tolist()) == set(want.indices[r][want_v[r] > kth[r]].tolist())
    return vals, idx


@pytest.mark.parametrize("n,v,k,dtype", [
    (64, 151936, 64, torch.bfloat16),    # the production vocabulary: many equal bf16 values around the threshold
    (33, 151936, 8, torch.float32),      # what stock Megatron hands over
    (50, 32003, 100, torch.float16),     # rows that are not 16-byte aligned (scalar loads)
    (40, 4104, 512, torch.float32),      # the largest k
    (17, 1000, 1, torch.bfloat16),       # k = 1: the arg-max
    (9, 700, 700, torch.float32),        # k = vocabulary: a full sort... of at most 512 -> uses 512 below
])
def test_topk_rows_equals_torch_topk(n, v, k, dtype):
    dev = require_gpu()
    announce("topk rows", n, v, k, dtype)
    k = min(k, 512)
    g = torch.Generator(device=dev).manual_seed(n + v + k)
    x = (torch.randn((n, v), device=dev, generator=g) * 3).to(dtype)
    _check_topk_rows(x, k)
    # through a row map: the last rows first, some rows twice
    row_ids = torch.cat([torch.arange(n - 1, -1, -2, device=dev), torch.tensor([0, 0], device=dev)]).int()
    _check_topk_rows(x, k, row_ids)


@pytest.mark.parametrize("n,v,k,dtype,temperature", [
    (96, 151936, 64, torch.bfloat16, 1.0),    # the production row: one read serves both
    (40, 151936, 8, torch.float32, 0.7),      # fp32 rows of the same vocabulary
    (50, 65536, 512, torch.float16, 1.0),     # a short row for the fused kernel, the largest k
    (44, 8 * 7168, 64, torch.bfloat16, 1.0),  # the shortest row the fused kernel takes (1024-thread workgroups from here on)
    (36, 32000, 32, torch.float32, 1.0),      # fp32 rows of the small benchmark vocabulary: 8000 vectors, likewise
    (50, 32003, 100, torch.float16, 1.0),     # rows that are not 16-byte aligned: the two passes run one after the other
    (30, 4104, 16, torch.bfloat16, 1.3),      # a short row: likewise
])
def test_logprob_entropy_topk_one_read_equals_the_two_passes(n, v, k, dtype, temperature):
    """``logprob_entropy_topk_fwd`` (log-probs, entropy and the top-K ids of the same rows from one read) against the
    two separate launches: log-prob / entropy / lse / spx bit for bit, top-K values exactly, indices pointing at their
    values; through a row map as well; rows with long runs of equal values or an infinite logit (which the shortcut
    hands to the general kernel) included."""
    from relax_amd import ops

    dev = require_gpu()
    announce("logprob + topk one read", n, v, k, dtype, temperature)
    g = torch.Generator(device=dev).manual_seed(n + v + k)
    x = (torch.randn((n, v), device=dev, generator=g) * 3).to(dtype)
    x[3] = 1.5        # a constant row: every element ties
    x[5, : v // 2] = x[5, 0]  # half a row of equal values above most of the rest
    x[5, 0: v // 2] = 9.0
    x[7, 11] = float("inf")   # an infinite logit: log-prob and entropy are NaN in both kernels, the selection still exact
    x[9, v // 3:] = float("-inf")  # most of a row at -inf
    tok = torch.randint(0, v, (n,), device=dev, generator=g)
    inv_t = 1.0 / temperature
    for row_ids in (None, torch.cat([torch.arange(n - 1, -1, -2, device=dev), torch.tensor([0, 5, 5, 3], device=dev)]).int()):
        t = tok if row_ids is None else tok[: row_ids.numel()]
        lp, ent, lse, spx, vals, idx = ops.logprob_entropy_topk_fwd(x, t, row_ids, inv_t, k, True, with_values=True)
        lp2, ent2, lse2, spx2 = ops.logprob_entropy_fwd(x, t, row_ids, inv_t, True)
        for one, two in ((lp, lp2), (ent, ent2), (lse, lse2), (spx, spx2)):
            assert torch.equal(one.isnan(), two.isnan()) and torch.equal(one.nan_to_num(), two.nan_to_num())
        assert lp[~lp.isnan()].numel() >= lp.numel() - 3
        vals2, idx2 = ops.topk_rows(x, row_ids, k)
        rows = x if row_ids is None else x[row_ids.long()]
        assert torch.equal(vals, vals2)
        assert torch.equal(vals, torch.topk(rows.float(), k, dim=-1).values)
        assert (idx >= 0).all() and (idx < v).all()
        assert torch.equal(torch.gather(rows.float(), 1, idx), vals)
        assert (torch.sort(idx, dim=1).values.diff(dim=1) > 0).all() or k == 1  # distinct
    # rows that are views into a wider matrix (row stride > vocabulary, still 16-byte aligned)
    wide = torch.full((n, v + 64), 50.0, device=dev, dtype=dtype)   # what lies beyond a row would win every selection
    wide[:, :v] = x
    lpw, entw, _, _, valsw, idxw = ops.logprob_entropy_topk_fwd(wide[:, :v], tok, None, inv_t, k, True, with_values=True)
    lpc, entc, _, _, valsc, idxc = ops.logprob_entropy_topk_fwd(x, tok, None, inv_t, k, True, with_values=True)
    assert torch.equal(lpw.nan_to_num(), lpc.nan_to_num()) and torch.equal(entw.nan_to_num(), entc.nan_to_num())
    assert torch.equal(valsw, valsc)
    plain = torch.ones(n, dtype=torch.bool, device=dev)
    plain[[3, 5]] = False  # rows with tens of thousands of exact ties: which of the tied entries leave is not fixed
    assert torch.equal(idxw[plain], idxc[plain])
    assert torch.equal(torch.gather(x.float(), 1, idxw), valsw)
    # without entropy and without values: the optional outputs are really optional
    lp3, ent3, lse3, spx3, vals3, idx3 = ops.logprob_entropy_topk_fwd(x, tok, None, inv_t, k, False)
    assert ent3 is None and spx3 is None and vals3 is None
    assert torch.equal(lp3.nan_to_num(), ops.logprob_entropy_fwd(x, tok, None, inv_t, False)[0].nan_to_num())


def test_topk_rows_on_tiny_vocabularies():
    """Rows shorter than one 16-byte vector, with a row stride that still allows vector loads: nothing may be read
    outside the row."""
    dev = require_gpu()
    announce("topk rows tiny")
    g = torch.Generator(device=dev).manual_seed(3)
    for v, k, dtype in ((5, 3, torch.bfloat16), (3, 3, torch.float32), (1, 1, torch.bfloat16), (9, 4, torch.float16)):
        wide = (torch.randn((12, 16), device=dev, generator=g) * 2).to(dtype)
        _check_topk_rows(wide[:, :v], k)  # row stride 16 elements: 16-byte aligned rows of v elements


def test_topk_rows_on_degenerate_rows():
    """Rows that defeat the first histogram: all values equal (every key shares all 32 bits), two distinct values,
    values that differ only in their low mantissa bits (three refinement passes), infinities, NaN (ordered above
    +inf as torch does), signed zeros, and a row whose k-th value is shared by thousands of entries."""
    dev = require_gpu()
    announce("topk rows degenerate")
    v, k = 20000, 50
    g = torch.Generator(device=dev).manual_seed(7)
    rows = [
        torch.full((v,), 1.25, device=dev),
        (torch.rand(v, device=dev, generator=g) > 0.999).float() * 3 - 1,
        1.0 + torch.arange(v, device=dev).float() * 2.0 ** -22,
        torch.randn(v, device=dev, generator=g),
        torch.randn(v, device=dev, generator=g),
        torch.zeros(v, device=dev),
        torch.randn(v, device=dev, generator=g).round(),
    ]
    rows[3][5], rows[3][77], rows[3][4000] = float("inf"), float("-inf"), float("inf")
    rows[4][123], rows[4][19999] = float("nan"), float("nan")
    rows[5][::2] = -0.0
    x = torch.stack(rows)
    vals, idx = _check_topk_rows(x, k)
    assert torch.isnan(vals[4, :2]).all() and set(idx[4, :2].tolist()) == {123, 19999}
    assert set(idx[3, :2].tolist()) == {5, 4000}
    assert (vals[0] == 1.25).all() and (vals[2] == x[2, -k:].flip(0)).all()
    _check_topk_rows(x.bfloat16(), k)
    _check_topk_rows(x, 512)


def test_get_log_probs_and_entropy_with_topk_uses_one_launch_and_matches_torch():
    """``with_topk=True`` (loss.py:434-446): per-sample ``topk_token_ids`` [R_i, k], the rows' k largest logits."""
    import relax_amd
    from oracle import policy as P

    dev = require_gpu()
    announce("with_topk")
    tot, resp, v, k = [9, 6, 12], [4, 3, 7], 3000, 5
    g = torch.Generator().manual_seed(12)
    logits = (torch.randn(1, sum(tot), v, generator=g) * 2).to(dev)
    toks = [torch.randint(0, v, (n,), generator=g).to(dev) for n in tot]
    args = P.make_args(rollout_temperature=0.7, opd_log_prob_top_k=k)
    _, out = relax_amd.get_log_probs_and_entropy(logits, args=args, unconcat_tokens=toks, total_lengths=tot,
                                                 response_lengths=resp, with_topk=True)
    assert [tuple(t.shape) for t in out["topk_token_ids"]] == [(r, k) for r in resp]
    for (b, e, _), ids in zip(P.response_row_ranges(tot, resp), out["topk_token_ids"]):
        assert torch.equal(ids, torch.topk(logits[0, b:e], k, dim=-1).indices)
