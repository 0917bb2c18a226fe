"""Pins oracle.logprob against the reference's literal vectors, library routines and invariants (CPU)."""

import math

import pytest
import torch

from oracle import logprob as O


def _weighted_loss(lp, ent, wl, we):
    out = (lp.squeeze(-1) * wl).sum()
    if ent is not None:
        out = out + (ent * we).sum()
    return out


@pytest.mark.parametrize("key", ["logprob_single_rank", "logprob_two_shards"])
@pytest.mark.parametrize("use_mask", [False, True])
def test_literals_match_library_closed_forms(literals, key, use_mask):
    fx = literals[key]
    x = torch.tensor(fx["logits"], dtype=torch.float32, requires_grad=True)
    tok = torch.tensor(fx["tokens"])
    keep = torch.tensor(fx["keep_mask"]) if use_mask else None
    wl, we = torch.tensor(fx["logprob_weights"]), torch.tensor(fx["entropy_weights"])
    lp, ent = O.calculate_log_probs_and_entropy(x, tok, None, with_entropy=True, log_prob_keep_mask=keep)
    _weighted_loss(lp, ent, wl, we).backward()

    # independent statement: library log_softmax / Categorical entropy + autograd (fp64)
    x64 = torch.tensor(fx["logits"], dtype=torch.float64, requires_grad=True)
    rows = torch.arange(len(fx["tokens"]))
    lx = x64
    if use_mask:
        lx = x64.masked_fill(~keep, float("-inf"))
        lx = lx.clone()
        lx[rows, tok] = x64[rows, tok]
    lp_ref = torch.log_softmax(lx, -1)[rows, tok]
    ent_ref = torch.distributions.Categorical(logits=x64).entropy()
    ((lp_ref * wl.double()).sum() + (ent_ref * we.double()).sum()).backward()
    assert lp.shape == (len(fx["tokens"]), 1) and lp.dtype == torch.float32
    torch.testing.assert_close(lp.squeeze(-1).double(), lp_ref.detach(), atol=2e-6, rtol=0)
    torch.testing.assert_close(ent.double(), ent_ref.detach(), atol=2e-6, rtol=0)
    torch.testing.assert_close(x.grad.double(), x64.grad, atol=2e-6, rtol=0)


@pytest.mark.parametrize("chunk", [-1, 1, 2, 8])
def test_chunk_size_independence_strict(literals, chunk):
    fx = literals["logprob_single_rank"]
    x = torch.tensor(fx["logits"])
    tok = torch.tensor(fx["tokens"])
    keep = torch.tensor(fx["keep_mask"])
    a = O.calculate_log_probs_and_entropy(x, tok, None, with_entropy=True, log_prob_keep_mask=keep)
    b = O.calculate_log_probs_and_entropy(x, tok, None, with_entropy=True, chunk_size=chunk, log_prob_keep_mask=keep)
    torch.testing.assert_close(a[0], b[0], atol=fx["atol"], rtol=0)
    torch.testing.assert_close(a[1], b[1], atol=fx["atol"], rtol=0)


def test_empty_input_shapes():
    x = torch.zeros(0, 4)
    lp, ent = O.calculate_log_probs_and_entropy(x, torch.zeros(0, dtype=torch.long), None, with_entropy=True)
    assert lp.shape == (0,) and ent.shape == (0,)
    lp, ent = O.calculate_log_probs_and_entropy(x, torch.zeros(0, dtype=torch.long), None, with_entropy=False)
    assert lp.shape == (0,) and ent is None


def test_entropy_not_differentiable_without_entropy_grad(literals):
    fx = literals["logprob_single_rank"]
    x = torch.tensor(fx["logits"], requires_grad=True)
    lp, ent = O.calculate_log_probs_and_entropy(
        x, torch.tensor(fx["tokens"]), None, with_entropy=True, with_entropy_grad=False
    )
    assert lp.requires_grad and not ent.requires_grad


def test_gradcheck_fp64_explicit_backward():
    torch.manual_seed(1)
    x = torch.randn(5, 7, dtype=torch.float64, requires_grad=True)
    tok = torch.randint(0, 7, (5,))

    def f(z):
        lp, ent = O._LogProbEntropy.apply(z, tok, None, True, True)
        return lp.squeeze(-1), ent

    # the oracle upcasts with .float(); run gradcheck on an fp64 clone of the same formulas instead
    saved = O.forward_values(x.detach(), tok, None, True)
    g_lp, g_ent = torch.randn(5), torch.randn(5)
    explicit = O.backward_values(saved, tok, g_lp, g_ent).double()
    lp64 = torch.log_softmax(x, -1)[torch.arange(5), tok]
    p = torch.softmax(x, -1)
    ent64 = -(p * torch.log_softmax(x, -1)).sum(-1)
    ((lp64 * g_lp.double()).sum() + (ent64 * g_ent.double()).sum()).backward()
    torch.testing.assert_close(explicit, x.grad, atol=5e-6, rtol=0)


def test_invariants_shift_range_rowsum():
    torch.manual_seed(2)
    v = 257
    x = (torch.randn(9, v) * 3).requires_grad_()
    tok = torch.randint(0, v, (9,))
    lp, ent = O.calculate_log_probs_and_entropy(x, tok, None, with_entropy=True)
    lp2, ent2 = O.calculate_log_probs_and_entropy(x.detach() + 11.5, tok, None, with_entropy=True)
    torch.testing.assert_close(lp, lp2, atol=2e-5, rtol=0)
    torch.testing.assert_close(ent, ent2, atol=2e-5, rtol=0)
    assert (ent >= 0).all() and (ent <= math.log(v) + 1e-5).all() and (lp <= 0).all()
    (lp.sum() * 0.7 + (ent * torch.randn(9)).sum()).backward()
    assert x.grad.sum(-1).abs().max() < 1e-5  # both gradient terms sum to zero over the vocab


def test_uniform_row_closed_form():
    v = 64
    lp, ent = O.calculate_log_probs_and_entropy(torch.zeros(2, v), torch.tensor([3, 9]), None, with_entropy=True)
    torch.testing.assert_close(lp.squeeze(-1), torch.full((2,), -math.log(v)), atol=1e-6, rtol=0)
    torch.testing.assert_close(ent, torch.full((2,), math.log(v)), atol=1e-6, rtol=0)


def test_bf16_input_returns_fp32_and_grad_in_input_dtype():
    torch.manual_seed(3)
    x = torch.randn(4, 33).bfloat16().requires_grad_()
    tok = torch.randint(0, 33, (4,))
    lp, ent = O.calculate_log_probs_and_entropy(x, tok, None, with_entropy=True)
    assert lp.dtype == torch.float32 and ent.dtype == torch.float32
    lp.sum().backward()
    assert x.grad.dtype == torch.bfloat16
