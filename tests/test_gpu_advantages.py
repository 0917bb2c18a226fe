"""GPU parity of group-normalised rewards, broadcast returns, whitening and the reverse-KL kernels vs the oracle.

Advantages: 1e-6 relative (the stated bound); error behaviour as the reference's tests assert it.
"""

from types import SimpleNamespace

import numpy as np
import pytest
import torch

from oracle import advantages as A
from oracle import opd as D
from tests.gpu_util import announce, require_gpu

pytestmark = pytest.mark.gpu


class _Sample:
    def __init__(self, reward, group):
        self.reward, self.group_index = reward, group

    def get_reward_value(self, args):
        return self.reward


def _args(est="grpo", n=4, std=True, norm=True):
    return SimpleNamespace(advantage_estimator=est, n_samples_per_prompt=n, grpo_std_normalization=std,
                           rewards_normalization=norm, custom_reward_post_process_path=None)


def test_post_process_rewards_literals(literals):
    from relax_amd.utils import post_process_rewards

    require_gpu()
    announce("post_process_rewards literals")
    fx = literals["group_rewards"]
    r = fx["grpo_binary"]["rewards"]
    raw, got = post_process_rewards(_args("grpo", 4), [_Sample(x, 0) for x in r])
    arr = np.asarray(r, dtype=np.float32)
    np.testing.assert_allclose(got, (arr - arr.mean()) / (arr.std(ddof=1) + 1e-6), rtol=1e-6, atol=1e-6)
    assert raw == r
    _, got = post_process_rewards(_args("rloo", 4), [_Sample(x, 0) for x in r])
    np.testing.assert_allclose(got, fx["rloo_binary"]["expected"], rtol=1e-6)
    b = fx["rpp_baseline"]
    _, got = post_process_rewards(_args("reinforce_plus_plus_baseline", 2),
                                  [_Sample(x, g) for x, g in zip(b["rewards"], b["groups"])])
    assert got == b["expected"]
    m = literals["grpo_micro_fixture"]
    _, got = post_process_rewards(_args("grpo", 2, std=False),
                                  [_Sample(x, g) for x, g in zip(m["raw_rewards"], m["group_indices"])])
    assert got == m["normalized_rewards"]
    with pytest.raises(ValueError, match="3 samples, expected 4"):
        post_process_rewards(_args("grpo", 4), [_Sample(1.0, 0)] * 3)
    with pytest.raises(ValueError, match="group_index is required"):
        post_process_rewards(_args("grpo", 1), [_Sample(1.0, None)])
    with pytest.raises(ValueError, match="non-finite"):
        post_process_rewards(_args("rloo", 2), [_Sample(1.0, 0), _Sample(float("nan"), 0)])
    raw, got = post_process_rewards(_args("grpo", 4, norm=False), [_Sample(x, 0) for x in r])
    assert got == r


def test_group_rewards_first_config_shape_vs_oracle():
    """64 prompts x 8 responses, Bernoulli(0.4) rewards, interleaved group order."""
    from relax_amd.utils import post_process_rewards

    require_gpu()
    announce("group rewards 512")
    g = torch.Generator().manual_seed(0)
    rewards = torch.bernoulli(torch.full((512,), 0.4), generator=g).tolist()
    groups = torch.randperm(512, generator=g).remainder(64).tolist()
    for est, std in (("grpo", True), ("grpo", False), ("rloo", True), ("cispo", True)):
        _, got = post_process_rewards(_args(est, 8, std), [_Sample(r, gi) for r, gi in zip(rewards, groups)])
        want = A.group_normalise(rewards, groups, 8, est, std)
        np.testing.assert_allclose(got, want.numpy(), rtol=1e-6, atol=1e-7)


def test_rloo_leave_one_out_bruteforce_and_errors():
    from relax_amd.ppo_utils import compute_rloo_leave_one_out_rewards as rloo

    dev = require_gpu()
    announce("rloo standalone")
    for gsz in (2, 3, 5, 8):
        torch.manual_seed(gsz)
        r = torch.randn(gsz, dtype=torch.float64)
        want = torch.tensor([r[i].item() - (r.sum().item() - r[i].item()) / (gsz - 1) for i in range(gsz)], dtype=torch.float64)
        got = rloo(r.to(dev))
        assert got.dtype == torch.float64
        torch.testing.assert_close(got.cpu(), want, atol=1e-12, rtol=0)
    torch.testing.assert_close(rloo(torch.tensor([3.0, 1.0], device=dev)).cpu(), torch.tensor([2.0, -2.0]))
    assert rloo(torch.full((4,), 2.5, device=dev)).abs().max().item() == 0
    with pytest.raises(ValueError, match="1-D"):
        rloo(torch.zeros(2, 2, device=dev))
    with pytest.raises(ValueError, match=">= 2"):
        rloo(torch.zeros(1, device=dev))
    with pytest.raises(ValueError, match="non-finite"):
        rloo(torch.tensor([1.0, float("inf")], device=dev))


def test_grpo_returns_and_advantages_and_whitening(literals):
    import relax_amd
    from relax_amd.distributed_utils import distributed_masked_whiten
    from relax_amd.ppo_utils import get_grpo_returns

    dev = require_gpu()
    announce("returns / whiten")
    fx = literals["grpo_returns"]
    like = [torch.randn(3, device=dev), torch.randn(2, 2, dtype=torch.float64, device=dev)]
    out = get_grpo_returns(torch.tensor(fx["rewards"], device=dev), like)
    assert out[0].dtype == torch.float32 and out[1].dtype == torch.float64 and out[1].shape == (2, 2)
    assert (out[0] == 1.5).all() and (out[1] == -0.25).all()

    g = torch.Generator().manual_seed(1)
    lens = [int(x) for x in torch.randint(1, 300, (37,), generator=g)]
    rewards = torch.randn(37, generator=g).tolist()
    masks = [(torch.rand(n, generator=g) > 0.2).float() for n in lens]
    lps = [torch.zeros(n) for n in lens]
    for normalize in (False, True):
        args = SimpleNamespace(advantage_estimator="grpo", use_rollout_logprobs=False, normalize_advantages=normalize)
        data = dict(log_probs=[x.to(dev) for x in lps], rewards=rewards, loss_masks=[m.to(dev) for m in masks])
        relax_amd.compute_advantages_and_returns(args, data)
        want_adv, want_ret = A.advantages_and_returns(rewards, lps, masks, normalize)
        for a, b in zip(data["advantages"], want_adv):
            torch.testing.assert_close(a.cpu(), b, rtol=2e-5 if normalize else 1e-6, atol=1e-6)
        for a, b in zip(data["returns"], want_ret):
            torch.testing.assert_close(a.cpu(), b, rtol=1e-6, atol=0)

    v = torch.randn(5000, generator=g)
    m = (torch.rand(5000, generator=g) > 0.3).float()
    got = distributed_masked_whiten(v.to(dev), m.to(dev))
    torch.testing.assert_close(got.cpu(), A.masked_whiten(v, m), rtol=2e-5, atol=2e-6)
    got = distributed_masked_whiten(v.to(dev), m.to(dev), shift_mean=False)
    torch.testing.assert_close(got.cpu(), A.masked_whiten(v, m, shift_mean=False), rtol=2e-5, atol=2e-6)
    one = distributed_masked_whiten(torch.tensor([3.0, 5.0], device=dev), torch.tensor([1.0, 0.0], device=dev))
    torch.testing.assert_close(one.cpu(), A.masked_whiten(torch.tensor([3.0, 5.0]), torch.tensor([1.0, 0.0])), rtol=1e-5, atol=0)
    with pytest.raises(ValueError, match="zero"):
        distributed_masked_whiten(v.to(dev), torch.zeros(5000, device=dev))


def test_advantages_service_method_returns_nested_tensors():
    from relax_amd.advantages import Advantages

    dev = require_gpu()
    announce("advantages service method")
    svc = Advantages(SimpleNamespace(advantage_estimator="rloo", use_rollout_logprobs=False, kl_coef=0.0))
    data = dict(log_probs=[torch.zeros(3, device=dev), torch.zeros(5, device=dev)], rewards=[0.5, -1.0],
                loss_masks=[torch.ones(3, device=dev), torch.ones(5, device=dev)])
    out = svc.compute_advantages_and_returns(data)
    assert out["advantages"].is_nested and [t.tolist() for t in out["advantages"].unbind()] == [[0.5] * 3, [-1.0] * 5]
    assert svc.compute_advantages_and_returns({}) is None


@pytest.mark.parametrize("n,v,dtype,tol", [(17, 1003, torch.float32, 2e-5), (12, 4104, torch.bfloat16, 2e-3),
                                           (10, 151936, torch.bfloat16, 2e-3)])
def test_full_vocab_reverse_kl_vs_oracle(n, v, dtype, tol):
    from relax_amd.opd_utils import compute_opd_kl_full_vocab, reduce_opd_loss

    dev = require_gpu()
    announce("reverse KL", n, v, dtype)
    g = torch.Generator().manual_seed(n)
    s = (torch.randn(n, v, generator=g) * 3).to(dtype)
    t = (s.float() + torch.randn(n, v, generator=g)).to(dtype)
    lens = [n // 2, n - n // 2]
    masks = [(torch.rand(k, generator=g) > 0.15).float() for k in lens]
    sc = s.clone().requires_grad_()
    want = D.full_vocab_reverse_kl(sc, t)
    want_loss = D.reduce_token_mean(want, lens, masks)
    want_loss.backward()
    sd = s.to(dev).requires_grad_()
    got = compute_opd_kl_full_vocab(sd, t.to(dev))
    loss = reduce_opd_loss({"response_lengths": lens, "loss_masks": [m.to(dev) for m in masks]}, got)
    loss.backward()
    torch.testing.assert_close(got.detach().cpu(), want.detach(), atol=tol, rtol=0)
    assert abs(loss.item() - want_loss.item()) < tol
    assert sd.grad.dtype == dtype
    torch.testing.assert_close(sd.grad.float().cpu(), sc.grad.float(), atol=tol, rtol=2.0 ** -7 if dtype == torch.bfloat16 else 0)
    assert (got >= -tol).all()
    same = compute_opd_kl_full_vocab(s.to(dev), s.to(dev))
    assert same.abs().max().item() < 1e-5


@pytest.mark.gpu
@pytest.mark.parametrize("n,v,dtype,tol", [
    (33, 1000, torch.float32, 3e-5),        # scalar tail, 256-thread variant
    (64, 151936, torch.bfloat16, 2e-3),     # the production vocabulary, 1024-thread variant
    (17, 32003, torch.float16, 2e-3),       # rows that are not 16-byte aligned
])
def test_fused_opd_loss_matches_oracle_and_two_launch_path(n, v, dtype, tol):
    """One-launch forward + backward of the masked token-mean reverse KL: same loss, per-token KL and student
    gradient as the oracle and as the separate forward / backward launches; an upstream gradient other than 1 is
    applied to the stored gradient."""
    from relax_amd.opd_utils import compute_opd_kl_full_vocab, opd_loss_full_vocab, reduce_opd_loss

    dev = require_gpu()
    announce("fused OPD loss", n, v, dtype)
    g = torch.Generator().manual_seed(n + v)
    s = (torch.randn(n, v, generator=g) * 3).to(dtype)
    t = (s.float() + torch.randn(n, v, generator=g)).to(dtype)
    lens = [n // 3, n - n // 3]
    masks = [(torch.rand(k, generator=g) > 0.3).float() for k in lens]
    sc = s.clone().requires_grad_()
    want = D.full_vocab_reverse_kl(sc, t)
    want_loss = D.reduce_token_mean(want, lens, masks)
    (2.5 * want_loss).backward()
    batch = {"response_lengths": lens, "loss_masks": [m.to(dev) for m in masks]}
    sd = s.to(dev).requires_grad_()
    loss, kl = opd_loss_full_vocab(batch, sd, t.to(dev))
    (2.5 * loss).backward()
    torch.testing.assert_close(kl.cpu(), want.detach(), atol=tol, rtol=0)
    assert abs(loss.item() - want_loss.item()) < tol
    assert sd.grad.dtype == dtype and sd.grad.shape == s.shape
    ulp = {torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10, torch.float32: 1e-5}[dtype]
    torch.testing.assert_close(sd.grad.float().cpu(), sc.grad.float(), atol=tol, rtol=ulp)
    # masked tokens: zero gradient rows, KL still reported
    dead = torch.cat(masks) == 0
    assert dead.any() and (sd.grad[dead.to(dev)] == 0).all()
    # against the two-launch path on the same device
    s2 = s.to(dev).requires_grad_()
    kl2 = compute_opd_kl_full_vocab(s2, t.to(dev))
    loss2 = reduce_opd_loss(batch, kl2)
    (2.5 * loss2).backward()
    torch.testing.assert_close(kl, kl2.detach(), atol=2e-6 if dtype == torch.float32 else 1e-5, rtol=1e-6)
    torch.testing.assert_close(sd.grad.float(), s2.grad.float(), atol=tol * 1e-2, rtol=2 * ulp)
    # no-grad call falls back to the forward-only kernel
    with torch.no_grad():
        loss3, kl3 = opd_loss_full_vocab(batch, s.to(dev), t.to(dev))
    assert abs(loss3.item() - loss2.item()) < 1e-6
    assert torch.equal(kl3, kl2.detach())


def test_opd_token_mean_literal(literals):
    from relax_amd.opd_utils import compute_opd_kl, reduce_opd_loss

    dev = require_gpu()
    fx = literals["opd_token_mean"]
    got = reduce_opd_loss({"response_lengths": fx["lengths"], "loss_masks": [torch.tensor(m, device=dev) for m in fx["masks"]]},
                          torch.tensor(fx["values"], device=dev))
    assert got.item() == fx["expected"]
    s, t = torch.tensor([-0.5, -2.0], device=dev), torch.tensor([-1.0, -0.3], device=dev)
    torch.testing.assert_close(compute_opd_kl(s, t, "reverse_kl"), s - t)
    d = s - t
    torch.testing.assert_close(compute_opd_kl(s, t, "low_var_kl"), torch.exp(-d) - 1 + d, atol=1e-6, rtol=1e-6)
