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


@pytest.mark.parametrize("v,dtype,n", [(151936, torch.bfloat16, 700), (152064, torch.float16, 300),
                                       (128256, torch.bfloat16, 520), (131072, torch.float16, 515),
                                       (100352, torch.bfloat16, 1030), (102400, torch.bfloat16, 40),
                                       (163840, torch.bfloat16, 300), (8 * (19 * 1024 + 3), torch.float16, 530)])
def test_register_resident_reverse_kl_step_equals_two_walk_kernel_bitwise(v, dtype, n):
    """The three kernels behind relax_amd_reverse_kl_step_fused, switched with relax_amd_set_kernel_choice, for every
    row shape the register-resident ones are built for (partial and full last vector positions), with more rows than
    workgroups (several rows per persistent workgroup, uneven counts), fewer rows than workgroups, and rows without
    gradient (zero rows, KL still reported) scattered and in runs.  KL, both log-sum-exps and the gradient must be
    bit-identical, and a few rows are checked against the oracle."""
    from relax_amd import ops

    dev = require_gpu()
    announce("resident reverse KL vs two-walk", v, dtype, n)
    gen = torch.Generator(device=dev).manual_seed(v + n)
    s = (torch.randn((n, v), device=dev, generator=gen) * 3).to(dtype)
    t = (s.float() + torch.randn((n, v), device=dev, generator=gen)).to(dtype)
    s[1, 7] = 40.0       # a row dominated by one entry
    t[2] = s[2]          # KL == 0
    g = (torch.rand(n, device=dev, generator=gen) > 0.2).float() * torch.rand(n, device=dev, generator=gen)
    g[n // 2:n // 2 + 9] = 0.0
    g[-1] = 0.0
    results = {}
    try:
        for kind in ("cached", "resident", "auto", "auto_again"):
            ops.set_kernel_choice({"cached": "two_walk", "resident": "resident"}.get(kind, "auto"))
            kl, ls, lt, d = ops.reverse_kl_step_fused(s, t, g, 0.75)
            torch.cuda.synchronize()
            results[kind] = dict(kl=kl, lse_s=ls, lse_t=lt, d=d.view(torch.int16))
    finally:
        ops.set_kernel_choice("auto")
    for kind in ("resident", "auto", "auto_again"):  # auto: one-shot workgroups, eight to a row
        for key, want in results["cached"].items():
            got = results[kind][key]
            assert torch.equal(got, want), (kind, key, (got.float() - want.float()).abs().max())
    d = results["resident"]["d"].view(dtype)
    live = g != 0
    live[2] = False  # identical rows: every gradient entry is p_s * 0
    assert (d[g == 0] == 0).all() and d[live].float().abs().sum(-1).min().item() > 0
    assert abs(results["resident"]["kl"][2].item()) < 1e-5
    rows = [0, 1, 2, n - 2]
    sc = s[rows].cpu().requires_grad_()
    want = D.full_vocab_reverse_kl(sc, t[rows].cpu())
    (want * (0.75 * g[rows].cpu())).sum().backward()
    torch.testing.assert_close(results["resident"]["kl"][rows].cpu(), want.detach(), atol=2e-3, rtol=0)
    ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
    torch.testing.assert_close(d[rows].float().cpu(), sc.grad.float(), atol=2e-3, rtol=ulp)


@pytest.mark.parametrize("v,dtype,n", [(50304, torch.bfloat16, 700), (64000, torch.bfloat16, 300),
                                       (65536, torch.float16, 9), (8 * 7169, torch.float16, 515),
                                       (248320, torch.bfloat16, 150), (202048, torch.float16, 130),
                                       (256000, torch.bfloat16, 70), (262144, torch.float16, 20),
                                       # one lane, and all lanes but one, at the partial vector position
                                       (8 * (30 * 1024 + 1), torch.float16, 40), (8 * (31 * 1024 + 1023), torch.bfloat16, 40),
                                       (8 * (6 * 1024 + 1), torch.bfloat16, 300), (8 * (7 * 1024 + 1023), torch.float16, 300)])
def test_one_shot_reverse_kl_step_on_short_rows_equals_two_walk_kernel_bitwise(v, dtype, n):
    """Rows of 6145 .. 8192 sixteen-byte vectors and of more than 20 vectors per thread (vocabularies of 200 k - 262 k
    entries: eighteen teacher vectors per thread in LDS, two waves per SIMD), which only the two-walk kernel and the
    one-shot workgroups (the default) are built for: KL, both log-sum-exps and the gradient bit-identical, twice in a row (the second launch finds
    the first one's words in the exchange ring)."""
    from relax_amd import ops

    dev = require_gpu()
    announce("one-shot reverse KL vs two-walk, short rows", v, dtype, n)
    gen = torch.Generator(device=dev).manual_seed(v + n)
    s = (torch.randn((n, v), device=dev, generator=gen) * 3).to(dtype)
    t = (s.float() + torch.randn((n, v), device=dev, generator=gen)).to(dtype)
    s[0, v - 1] = 30.0
    g = (torch.rand(n, device=dev, generator=gen) > 0.2).float() * torch.rand(n, device=dev, generator=gen)
    g[-1] = 0.0
    results = {}
    try:
        for kind in ("two_walk", "auto", "auto_again"):
            ops.set_kernel_choice("two_walk" if kind == "two_walk" else "auto")
            kl, ls, lt, d = ops.reverse_kl_step_fused(s, t, g, 1.25)
            torch.cuda.synchronize()
            results[kind] = dict(kl=kl, lse_s=ls, lse_t=lt, d=d.view(torch.int16))
    finally:
        ops.set_kernel_choice("auto")
    for kind in ("auto", "auto_again"):
        for key, want in results["two_walk"].items():
            assert torch.equal(results[kind][key], want), (kind, key)
    assert (results["auto"]["d"][g == 0] == 0).all() and torch.isfinite(results["auto"]["kl"]).all()
    rows = [0, n - 2]
    sc = s[rows].cpu().requires_grad_()
    want = D.full_vocab_reverse_kl(sc, t[rows].cpu())
    (want * (1.25 * g[rows].cpu())).sum().backward()
    torch.testing.assert_close(results["auto"]["kl"][rows].cpu(), want.detach(), atol=2e-3, rtol=0)
    ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
    torch.testing.assert_close(results["auto"]["d"].view(dtype)[rows].float().cpu(), sc.grad.float(), atol=2e-3, rtol=ulp)


@pytest.mark.parametrize("seed", range(12))
def test_one_shot_reverse_kl_step_on_random_layouts_equals_two_walk_kernel_bitwise(seed):
    """Random row counts (from a single row up to more than the exchange ring's 4096 slots), row lengths from every
    family the one-shot kernel is built for (and their neighbours by one vector), both 16-bit types, random runs of
    rows without gradient: the default kernel choice against the two-walk kernel, every output bit for bit."""
    from relax_amd import ops

    dev = require_gpu()
    gen = torch.Generator(device=dev).manual_seed(2000 + seed)
    cpu = torch.Generator().manual_seed(2000 + seed)
    nvecs = [6 * 1024 + 1, 7 * 1024 + 832, 8 * 1024, 12 * 1024 + 256, 15 * 1024 + 1023, 16 * 1024, 18 * 1024 + 560,
             19 * 1024 + 5, 20 * 1024, 24 * 1024 + 680, 30 * 1024 + 320, 31 * 1024 + 256, 32 * 1024]
    nvec = nvecs[seed % len(nvecs)] if seed < len(nvecs) else nvecs[int(torch.randint(0, len(nvecs), (1,), generator=cpu))]
    dtype = [torch.bfloat16, torch.float16][seed % 2]
    v = nvec * 8
    budget = 1_200_000_000 // (v * 2 * 2)
    n = [1, 7, 9, 63][seed % 4] if seed % 3 == 0 else int(torch.randint(64, max(65, min(budget, 6000)), (1,), generator=cpu))
    if seed == 1:
        n = 4400  # more rows than the ring has slots
    announce("one-shot reverse KL, random layout", seed, v, dtype, n)
    s = (torch.randn((n, v), device=dev, generator=gen) * 3).to(dtype)
    t = (s.float() + torch.randn((n, v), device=dev, generator=gen)).to(dtype)
    g = (torch.rand(n, device=dev, generator=gen) > 0.3).float() * torch.rand(n, device=dev, generator=gen)
    if n > 20:
        g[n // 3:n // 3 + 11] = 0.0
    results = {}
    try:
        for kind in ("two_walk", "auto"):
            ops.set_kernel_choice(kind)
            kl, ls, lt, d = ops.reverse_kl_step_fused(s, t, g, 0.5)
            torch.cuda.synchronize()
            results[kind] = dict(kl=kl, lse_s=ls, lse_t=lt, d=d.view(torch.int16))
        assert ops.last_kernel("reverse_kl_step_fused") == "reverse_kl_split"
    finally:
        ops.set_kernel_choice("auto")
    for key, want in results["two_walk"].items():
        assert torch.equal(results["auto"][key], want), (seed, key)
    assert torch.isfinite(results["auto"]["kl"]).all()


def test_one_shot_reverse_kl_step_gives_up_a_wait_that_cannot_succeed_and_recovers():
    """Failure handling of the exchange between the workgroups of a row, forced from the host
    (relax_amd_set_exchange_wait): with the awaited tag offset by one no wait can succeed; every workgroup gives up
    after a few looks, the row's KL and log-sum-exps come back NaN, every kernel exits normally, and the next launch
    with the defaults restored is exact again."""
    from relax_amd import ops
    from relax_amd._lib import check, lib

    dev = require_gpu()
    announce("one-shot reverse KL: give-up path")
    v, n = 151936, 120
    gen = torch.Generator(device=dev).manual_seed(3)
    s = (torch.randn((n, v), device=dev, generator=gen) * 2).bfloat16()
    t = (s.float() + torch.randn((n, v), device=dev, generator=gen)).bfloat16()
    g = torch.rand(n, device=dev, generator=gen)

    def run():
        out = ops.reverse_kl_step_fused(s, t, g, 1.0)
        torch.cuda.synchronize()
        return out

    ops.set_kernel_choice("two_walk")
    want = run()
    ops.set_kernel_choice("auto")
    check(lib.relax_amd_set_exchange_wait(4, 1))
    try:
        kl, ls, lt, d = run()
    finally:
        check(lib.relax_amd_set_exchange_wait(0, 0))
    assert torch.isnan(kl).all() and torch.isnan(ls).all() and torch.isnan(lt).all()
    got = run()
    for a, b in zip(got, want):
        assert torch.equal(a.view(torch.int16) if a.dtype == torch.bfloat16 else a, b.view(torch.int16) if b.dtype == torch.bfloat16 else b)


def test_default_reverse_kl_step_replayed_from_a_captured_graph():
    """The default reverse-KL step tags the partial sums its workgroups exchange with a counter that a small kernel in
    front of the launch advances on the device, so a captured launch gets fresh tags on every replay: three replays on
    fresh rows, with eager launches between them, each bit-identical to the two-walk kernel on the same inputs."""
    from relax_amd import ops

    dev = require_gpu()
    announce("reverse-KL step under graph capture")
    v, n = 100352, 260
    gen = torch.Generator(device=dev).manual_seed(17)
    s = torch.empty((n, v), device=dev, dtype=torch.bfloat16)
    t = torch.empty((n, v), device=dev, dtype=torch.bfloat16)
    g = torch.rand(n, device=dev, generator=gen)
    g[5] = 0.0

    def fresh():
        s.copy_(torch.randn((n, v), device=dev, generator=gen) * 3)
        t.copy_(s.float() + torch.randn((n, v), device=dev, generator=gen))

    def run():
        kl, ls, lt, d = ops.reverse_kl_step_fused(s, t, g, 1.0)
        return dict(kl=kl, lse_s=ls, lse_t=lt, d=d.view(torch.int16))

    fresh()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()  # warm-up outside the capture (the library looks its exchange buffer up on first use)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = run()
    try:
        for rep in range(3):
            fresh()
            graph.replay()
            torch.cuda.synchronize()
            got = {k: x.clone() for k, x in captured.items()}
            eager = run()  # an eager launch between the replays
            ops.set_kernel_choice("two_walk")
            want = run()
            ops.set_kernel_choice("auto")
            torch.cuda.synchronize()
            for key in want:
                assert torch.equal(got[key], want[key]), (rep, key)
                assert torch.equal(eager[key], want[key]), (rep, key, "eager")
            assert not torch.isnan(got["kl"]).any()
    finally:
        ops.set_kernel_choice("auto")


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


@pytest.mark.parametrize("n,v,k,dtype,tol", [
    (19, 1003, 7, torch.float32, 3e-5),
    (8, 151936, 32, torch.bfloat16, 2e-3),
    (5, 4104, 300, torch.float16, 2e-3),      # K larger than a workgroup pass, repeated ids
])
def test_topk_log_probs_vs_oracle(n, v, k, dtype, tol):
    """compute_log_probs_on_topk_token_ids: values, sentinels, out-of-range ids, repeated ids and the dense gradient."""
    from relax_amd.opd_utils import compute_log_probs_on_topk_token_ids
    from relax_amd.ppo_utils import calculate_log_probs_and_entropy

    dev = require_gpu()
    announce("top-K log-probs", n, v, k, dtype)
    g = torch.Generator().manual_seed(n * k)
    x = (torch.randn(n, v, generator=g) * 3).to(dtype)
    ids = torch.randint(0, v, (n, k), generator=g)
    ids[0, 0] = -1                      # sentinel
    ids[1, 1] = v + 5                   # outside the vocabulary
    ids[2, 2] = ids[2, 3]               # repeated id: both gradients land on the same logit
    up = torch.randn(n, k, generator=g)
    up[3] = 0.0                         # a row without incoming gradient
    xc = x.clone().float().requires_grad_()
    want = D.log_probs_on_topk_ids(xc, ids)
    (want.masked_fill(ids < 0, 0.0) * up).sum().backward()
    xd = x.to(dev).requires_grad_()
    got = compute_log_probs_on_topk_token_ids(xd, ids.to(dev), None)
    assert got.dtype == torch.float32 and got.shape == (n, k)
    assert torch.isinf(got[0, 0]) and got[0, 0] < 0
    fin = ids >= 0
    torch.testing.assert_close(got.cpu()[fin], want.detach()[fin], atol=tol, rtol=0)
    (got.masked_fill((ids < 0).to(dev), 0.0) * up.to(dev)).sum().backward()
    ulp = {torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10, torch.float32: 1e-5}[dtype]
    torch.testing.assert_close(xd.grad.float().cpu(), xc.grad, atol=tol, rtol=2 * ulp)
    assert (xd.grad[3] == 0).all()
    # reusing the log-sum-exp of a log-prob forward gives the same values without a row scan
    from relax_amd import ops
    _, _, lse, _ = ops.logprob_entropy_fwd(x.to(dev), torch.zeros(n, dtype=torch.long, device=dev), with_entropy=False)
    again = compute_log_probs_on_topk_token_ids(x.to(dev), ids.to(dev), None, lse=lse)
    torch.testing.assert_close(again[fin.to(dev)], got.detach()[fin.to(dev)], atol=2e-6, rtol=0)
    assert compute_log_probs_on_topk_token_ids(x[:0].to(dev), ids[:0].to(dev), None).shape == (0, k)


@pytest.mark.parametrize("kl_type,alpha", [("reverse_kl", 0.5), ("forward_kl", 0.5), ("jsd", 0.3), ("jsd", 0.0),
                                           ("jsd", 1.0), ("low_var_kl", 0.5)])
@pytest.mark.parametrize("norm_mode", ["tail", "norm", "trunc"])
@pytest.mark.parametrize("masked,clamp", [(False, None), (True, None), (False, -6.0), (True, -6.0)])
def test_opd_kl_topk_vs_oracle(kl_type, alpha, norm_mode, masked, clamp):
    """compute_opd_kl_topk on [R, K] log-probs: every KL type x normalisation x union mask x clamp, values and
    gradient w.r.t. the student log-probs."""
    from relax_amd.opd_utils import compute_opd_kl_topk

    dev = require_gpu()
    r, k, v = 37, 70, 400
    g = torch.Generator().manual_seed(7)
    full_s = torch.log_softmax(torch.randn(r, v, generator=g) * 2, -1)
    full_t = torch.log_softmax(torch.randn(r, v, generator=g) * 2, -1)
    s, t = full_s[:, :k].contiguous(), full_t[:, :k].contiguous()
    mask = None
    if masked:
        ksz = torch.randint(1, k + 1, (r,), generator=g)
        mask = torch.arange(k).unsqueeze(0) < ksz.unsqueeze(1)
    up = torch.randn(r, generator=g)
    sc = s.clone().requires_grad_()
    if mask is None:
        want = D.opd_kl_topk(sc, t, kl_type, alpha, norm_mode, clamp)
    else:
        # Row by row on the valid prefix, where the mask is a no-op and (the tail bin being cut off with the
        # padding) "tail" reads as "trunc".  The masked formulation itself is pinned against this one on the CPU; its
        # autograd gradient is NaN for "norm" (0 * (-inf - -inf) reaches the log-sum-exp), which no kernel should copy.
        mode = "trunc" if norm_mode == "tail" else norm_mode
        want = torch.cat([D.opd_kl_topk(sc[i:i + 1, :n], t[i:i + 1, :n], kl_type, alpha, mode, clamp)
                          for i, n in enumerate(ksz.tolist())])
        torch.testing.assert_close(want.detach(), D.opd_kl_topk(s, t, kl_type, alpha, norm_mode, clamp, mask),
                                   atol=1e-5, rtol=1e-5)
    (want * up).sum().backward()
    sd = s.to(dev).requires_grad_()
    got = compute_opd_kl_topk(sd, t.to(dev), kl_type, alpha, norm_mode, clamp, None if mask is None else mask.to(dev))
    (got * up.to(dev)).sum().backward()
    scale = max(1.0, want.detach().abs().max().item())
    torch.testing.assert_close(got.detach().cpu(), want.detach(), atol=2e-5 * scale, rtol=2e-5)
    gscale = max(1.0, sc.grad.abs().max().item())
    torch.testing.assert_close(sd.grad.cpu(), sc.grad, atol=2e-5 * gscale, rtol=2e-4)


@pytest.mark.parametrize("v,dtype,n", [(151936, torch.bfloat16, 300), (4100 * 8, torch.float16, 200),
                                       (32000, torch.float32, 300), (8 * 255, torch.bfloat16, 50)])
def test_reverse_kl_backward_chunk_form_equals_row_per_workgroup_kernel_bitwise(v, dtype, n):
    """The two kernels behind relax_amd_reverse_kl_bwd (one-shot workgroups that take 4 KB of a row each, the default;
    the row-per-workgroup loop), with tokens without gradient and a device-side scale: bit-identical gradients."""
    from relax_amd import ops

    dev = require_gpu()
    announce("reverse KL backward: chunk form vs row loop", v, dtype, n)
    gen = torch.Generator().manual_seed(v + n)
    s = (torch.randn(n, v, generator=gen) * 2).to(dtype).to(dev)
    t = (s.float().cpu() + torch.randn(n, v, generator=gen)).to(dtype).to(dev)
    kl, ls, lt, s, t = ops.reverse_kl_fwd(s, t)
    g = torch.rand(n, generator=gen)
    g[::4] = 0.0
    g[n // 2:n // 2 + 7] = 0.0
    scale = torch.tensor([0.61], device=dev)
    outs = {}
    for kind in ("two_walk", "auto"):
        ops.set_kernel_choice(kind)
        d = ops.reverse_kl_bwd(s, t, kl, ls, lt, g.to(dev), 0.75, scale)
        torch.cuda.synchronize()
        outs[kind] = d.view(torch.int16 if dtype != torch.float32 else torch.int32)
    assert torch.equal(outs["auto"], outs["two_walk"])
    assert outs["auto"].any() and not outs["auto"][(g == 0).to(dev)].any()


def test_opd_kl_two_dimensional_reverse_kl_is_the_elementwise_log_ratio():
    """compute_opd_kl on [R, K] inputs with ``reverse_kl`` returns s - t element by element (opd_utils.py:1126-1138),
    after the lower clamp, with -inf - -inf = NaN at the padding of a union mask like the reference."""
    from relax_amd.opd_utils import compute_opd_kl

    dev = require_gpu()
    announce("opd kl 2-D reverse_kl")
    g = torch.Generator().manual_seed(3)
    s = (-torch.rand(5, 7, generator=g) * 9).to(dev)
    t = (-torch.rand(5, 7, generator=g) * 9).to(dev)
    assert torch.equal(compute_opd_kl(s, t, "reverse_kl"), s - t)
    assert torch.equal(compute_opd_kl(s.bfloat16(), t, "reverse_kl", log_prob_min_clamp=-4.0),
                       s.bfloat16().float().clamp_min(-4.0) - t.clamp_min(-4.0))
    mask = torch.rand(5, 7, generator=g).to(dev) > 0.3
    got = compute_opd_kl(s, t, "reverse_kl", mask=mask)
    assert torch.equal(got[mask], (s - t)[mask]) and torch.isnan(got[~mask]).all()
    with pytest.raises(ValueError, match="Unknown opd_kl_type"):
        compute_opd_kl(s, t, "forward_kl")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_sparse_row_add_patches_rows_in_place(dtype):
    """The sparse half of the gathered log-probs' gradient: K (id, value) pairs per token plus one at the target are
    added to the token's logits row in place; an id equal to the target gets both additions, ids outside the vocabulary
    (sentinels, ids of another shard) and zero values are skipped, other rows and elements are untouched."""
    from relax_amd import ops

    dev = require_gpu()
    announce("sparse row add", dtype)
    g = torch.Generator().manual_seed(5)
    rows, v, n, k = 9, 50, 6, 4
    d0 = torch.randn(rows, v, generator=g).to(dtype)
    row_ids = torch.tensor([7, 0, 3, 4, 8, 1], dtype=torch.int32)
    ids = torch.randint(0, v, (n, k), generator=g)
    ids[0, 1], ids[2, 0], ids[3, 3] = -1, v + 5, -1
    targets = torch.randint(0, v, (n,), generator=g)
    ids[4, 2] = targets[4]  # a gathered id that equals the target
    vals = torch.randn(n, k, generator=g)
    vals[5, 0] = 0.0
    tvals = torch.randn(n, generator=g)
    want = d0.float().clone()
    for t in range(n):
        for j in range(k):
            if 0 <= ids[t, j] < v:
                r, c = row_ids[t], ids[t, j]
                want[r, c] = (want[r, c] + vals[t, j] * 0.5).to(dtype).float()
        r, c = row_ids[t], targets[t]
        want[r, c] = (want[r, c] + tvals[t] * 0.5).to(dtype).float()
    d = d0.to(dev)
    ops.sparse_row_add(d, row_ids.to(dev), ids.to(dev), vals.to(dev), targets.to(dev), tvals.to(dev), scale=0.5)
    assert torch.equal(d.float().cpu(), want)


def test_opd_kl_topk_argument_checks():
    from relax_amd.opd_utils import compute_opd_kl, compute_opd_kl_topk

    dev = require_gpu()
    s = torch.zeros(3, 4, device=dev) - 2.0
    with pytest.raises(ValueError, match="Unknown opd_kl_type"):
        compute_opd_kl_topk(s, s, "nope")
    with pytest.raises(ValueError, match="jsd_alpha"):
        compute_opd_kl_topk(s, s, "jsd", 1.5)
    assert compute_opd_kl_topk(s[:0], s[:0]).shape == (0,)
    # identical distributions: zero divergence in every mode
    for kt in ("reverse_kl", "forward_kl", "jsd", "low_var_kl"):
        assert compute_opd_kl(s, s, "jsd" if kt != "low_var_kl" else kt).abs().max().item() < 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_reinforce_pp_returns_and_baseline_vs_oracle(dtype):
    """One-launch REINFORCE++ returns: the reference test's cases, then random ragged sequences (longer than one
    64-token chunk, fully masked ones, masked NaN/inf) -- bit-exact against the sequential oracle."""
    from relax_amd.ppo_utils import get_reinforce_plus_plus_baseline_advantages, get_reinforce_plus_plus_returns

    dev = require_gpu()
    announce("REINFORCE++ returns", dtype)
    got = get_reinforce_plus_plus_returns(
        torch.tensor([1.0], dtype=dtype), [torch.tensor([0.5, 12345.0, -0.25], dtype=dtype, device=dev)],
        [torch.tensor([1.0, 0.0, 1.0], dtype=dtype, device=dev)], [3], [3], 0.1, 0.5)
    torch.testing.assert_close(got[0].cpu(), torch.tensor([0.20625, 0.0, 1.025], dtype=dtype), atol=1e-6, rtol=1e-6)
    g = torch.Generator().manual_seed(11)
    lens = [1, 63, 64, 65, 200, 5, 1000]
    kls = [torch.randn(n, generator=g, dtype=dtype) for n in lens]
    masks = [(torch.rand(n, generator=g) > 0.3).to(dtype) for n in lens]
    masks[5] = torch.zeros(5, dtype=dtype)                     # fully masked sequence
    kls[4][masks[4] == 0] = float("nan")                       # garbage outside the mask
    kls[6][masks[6] == 0] = float("inf")
    rewards = torch.randn(len(lens), generator=g, dtype=dtype)
    for gamma in (1.0, 0.97):
        want = A.reinforce_pp_returns(rewards, kls, masks, 0.05, gamma)
        got = get_reinforce_plus_plus_returns(rewards, [k.to(dev) for k in kls], [m.to(dev) for m in masks], lens, lens,
                                              0.05, gamma)
        for a, b, k in zip(got, want, kls):
            assert a.dtype == dtype and a.shape == k.shape
            assert torch.equal(a.cpu(), b), (a.cpu() - b).abs().max()
    base = get_reinforce_plus_plus_baseline_advantages(rewards, [k.to(dev) for k in kls], [m.to(dev) for m in masks])
    for a, b in zip(base, A.reinforce_pp_baseline_advantages(rewards, kls, masks)):
        assert torch.equal(a.cpu(), b)
    with pytest.raises(ValueError, match="same number of responses"):
        get_reinforce_plus_plus_returns(torch.tensor([0.0, 1.0]), [torch.ones(1, device=dev)], [torch.ones(1, device=dev)],
                                        [1], [1], 0.1, 1.0)
    with pytest.raises(ValueError, match="must have the same shape"):
        get_reinforce_plus_plus_returns(torch.tensor([0.0]), [torch.ones(2, device=dev)], [torch.ones(1, device=dev)],
                                        [1], [1], 0.1, 1.0)
    with pytest.raises(ValueError, match="must match"):
        get_reinforce_plus_plus_baseline_advantages(torch.tensor([1.0]), [torch.ones(2, device=dev)], [torch.ones(1, device=dev)])


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_gae_vs_oracle_and_padded_forms(dtype):
    from relax_amd.ppo_utils import (chunked_gae, get_advantages_and_returns, get_advantages_and_returns_batch,
                                     vanilla_gae)

    dev = require_gpu()
    announce("GAE", dtype)
    g = torch.Generator().manual_seed(5)
    lens = [3, 2, 64, 65, 257, 1]
    vals = [torch.randn(n, generator=g, dtype=dtype) for n in lens]
    rews = [torch.randn(n, generator=g, dtype=dtype) for n in lens]
    adv, ret = get_advantages_and_returns_batch([n + 3 for n in lens], lens, [v.to(dev) for v in vals],
                                                [r.to(dev) for r in rews], 0.99, 0.95)
    for a, r_, v, rw in zip(adv, ret, vals, rews):
        wa, wr = A.gae(v, rw, 0.99, 0.95)
        assert a.shape == v.shape and a.dtype == dtype
        assert torch.equal(a.cpu(), wa) and torch.equal(r_.cpu(), wr)
    a1, r1 = get_advantages_and_returns(6, 3, vals[0].to(dev), rews[0].to(dev), 0.99, 0.95)
    assert torch.equal(a1, adv[0]) and torch.equal(r1, ret[0]) and not a1.requires_grad
    # [B, T] padded forms: rows are independent sequences of length T
    rw2, v2 = torch.randn(3, 257, generator=g, dtype=dtype), torch.randn(3, 257, generator=g, dtype=dtype)
    av, rv = vanilla_gae(rw2.to(dev), v2.to(dev), 0.99, 0.95)
    ac, rc = chunked_gae(rw2.to(dev), v2.to(dev), 0.99, 0.95, chunk_size=32)
    for i in range(3):
        wa, wr = A.gae(v2[i], rw2[i], 0.99, 0.95)
        assert torch.equal(av[i].cpu(), wa) and torch.equal(rv[i].cpu(), wr)
    assert torch.equal(av, ac) and torch.equal(rv, rc)


def test_masked_normalize_and_estimator_dispatch():
    """distributed_masked_normalize on one rank, and compute_advantages_and_returns for the ppo / REINFORCE++
    estimators against the oracle's composition of the same pieces."""
    import relax_amd
    from relax_amd.distributed_utils import distributed_masked_normalize

    dev = require_gpu()
    g = torch.Generator().manual_seed(3)
    x = torch.randn(5000, generator=g)
    m = (torch.rand(5000, generator=g) > 0.4).float()
    x[m == 0] = float("nan")
    out, mean, var, cnt = distributed_masked_normalize(x.to(dev), m.to(dev))
    wo, wm, wv, wc = A.masked_normalize(x, m)
    assert cnt.item() == wc.item()
    torch.testing.assert_close(mean.cpu(), wm, atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(var.cpu(), wv, atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(out.cpu(), wo, atol=2e-6, rtol=2e-6)
    with pytest.raises(ValueError, match="same shape"):
        distributed_masked_normalize(x[:3].to(dev), m[:2].to(dev))
    lens = [4, 70, 9]
    lps = [torch.randn(n, generator=g) * 0.1 - 1 for n in lens]
    refs = [lp + 0.05 * torch.randn(n, generator=g) for lp, n in zip(lps, lens)]
    masks = [(torch.rand(n, generator=g) > 0.2).float() for n in lens]
    rewards = [0.5, -1.0, 2.0]
    kl = [lp - rf for lp, rf in zip(lps, refs)]  # k1
    args = SimpleNamespace(advantage_estimator="reinforce_plus_plus", use_rollout_logprobs=False, kl_coef=0.1,
                           kl_loss_type="k1", gamma=0.9, lambd=0.95, normalize_advantages=True)
    data = dict(log_probs=[t.to(dev) for t in lps], ref_log_probs=[t.to(dev) for t in refs], rewards=rewards,
                loss_masks=[t.to(dev) for t in masks], response_lengths=lens, total_lengths=lens)
    relax_amd.compute_advantages_and_returns(args, data)
    want_ret = A.reinforce_pp_returns(torch.tensor(rewards), kl, masks, 0.1, 0.9)
    for a, b in zip(data["returns"], want_ret):
        torch.testing.assert_close(a.cpu(), b, atol=1e-6, rtol=1e-6)
    white, wm, wv, wc = A.masked_normalize(torch.cat(want_ret), torch.cat(masks))
    torch.testing.assert_close(torch.cat(data["advantages"]).cpu(), white, atol=2e-6, rtol=2e-5)
    assert data["reinforce_pp_valid_token_count"][0].item() == wc.item() and len(data["reinforce_pp_zero_variance"]) == 3
    args.advantage_estimator, args.normalize_advantages = "ppo", False
    vals = [torch.randn(n, generator=g) for n in lens]
    data = dict(log_probs=[t.to(dev) for t in lps], ref_log_probs=[t.to(dev) for t in refs], rewards=rewards,
                values=[t.to(dev) for t in vals], loss_masks=[t.to(dev) for t in masks], response_lengths=lens,
                total_lengths=lens)
    relax_amd.compute_advantages_and_returns(args, data)
    for i, n in enumerate(lens):
        tok_r = -0.1 * kl[i]
        tok_r[-1] += rewards[i]
        wa, wr = A.gae(vals[i], tok_r, 0.9, 0.95)
        torch.testing.assert_close(data["advantages"][i].cpu(), wa, atol=2e-6, rtol=2e-6)
        torch.testing.assert_close(data["returns"][i].cpu(), wr, atol=2e-6, rtol=2e-6)


def test_full_size_reverse_kl_properties():
    """The distillation benchmark shape (16384 x 151936, bf16): KL >= 0, KL(s || s) = 0, every gradient row sums to
    zero (a uniform shift of the student's logits changes nothing), masked rows are exactly zero, and the one-launch
    step agrees with the separate forward / backward launches."""
    from relax_amd.opd_utils import compute_opd_kl_full_vocab, opd_loss_full_vocab, reduce_opd_loss

    dev = require_gpu()
    n, v = 16384, 151936
    announce("reverse KL full size", n, v)
    g = torch.Generator(device=dev).manual_seed(0)
    s = torch.empty((n, v), dtype=torch.bfloat16, device=dev)
    t = torch.empty_like(s)
    for b in range(0, n, 2048):
        x = torch.randn((2048, v), device=dev, generator=g) * 3.0
        s[b:b + 2048] = x.to(torch.bfloat16)
        t[b:b + 2048] = (x + torch.randn((2048, v), device=dev, generator=g)).to(torch.bfloat16)
    del x
    mask = (torch.rand(n, device=dev, generator=g) >= 0.15).float()
    batch = {"loss_masks": [mask], "response_lengths": [n]}
    sd = s.clone().requires_grad_()
    loss, kl = opd_loss_full_vocab(batch, sd, t)
    loss.backward()
    assert (kl >= -1e-3).all() and torch.isfinite(kl).all()
    assert abs(loss.item() - (kl * mask).sum().item() / mask.sum().item()) < 1e-5
    rows = sd.grad.float().sum(-1)
    assert rows.abs().max().item() < 1e-6  # gradients are O(1/n): bf16 rounding of 151936 terms stays far below
    assert (sd.grad[mask == 0] == 0).all() and (sd.grad[mask != 0].float().abs().sum(-1) > 0).all()
    s2 = s.clone().requires_grad_()
    kl2 = compute_opd_kl_full_vocab(s2, t)
    reduce_opd_loss(batch, kl2).backward()
    torch.testing.assert_close(kl, kl2.detach(), atol=1e-5, rtol=1e-6)
    torch.testing.assert_close(sd.grad.float(), s2.grad.float(), atol=1e-9, rtol=2.0 ** -6)
    same = compute_opd_kl_full_vocab(s[:256], s[:256])
    assert same.abs().max().item() < 1e-5


@pytest.mark.parametrize("selection", ["sampled", "union"])
def test_opd_advantage_shaping_vs_oracle(selection):
    """compute_advantages_and_returns with ``use_opd``: the per-token distillation signal is subtracted from the GRPO
    advantages (and replaces them entirely with ``opd_only_reward``)."""
    import relax_amd

    dev = require_gpu()
    g = torch.Generator().manual_seed(9)
    lens, k = [5, 8, 3], 6
    lps = [torch.randn(n, generator=g) * 0.1 - 1 for n in lens]
    data = dict(log_probs=lps, rewards=[0.5, -1.0, 2.0], loss_masks=[torch.ones(n) for n in lens],
                response_lengths=lens, total_lengths=lens,
                rollout_log_probs=[lp + 0.01 * torch.randn(n, generator=g) for lp, n in zip(lps, lens)],
                teacher_log_probs=[lp + 0.3 * torch.randn(n, generator=g) for lp, n in zip(lps, lens)],
                opd_topk_student_log_probs=[torch.log_softmax(torch.randn(n, 40, generator=g), -1)[:, :k].contiguous() for n in lens],
                opd_topk_teacher_log_probs=[torch.log_softmax(torch.randn(n, 40, generator=g), -1)[:, :k].contiguous() for n in lens],
                opd_topk_ksz=[torch.randint(1, k + 1, (n,), generator=g) for n in lens])
    for only in (False, True):
        args = SimpleNamespace(advantage_estimator="grpo", use_rollout_logprobs=False, kl_coef=0.0, use_opd=True,
                               opd_only_reward=only, opd_kl_coef=0.3, opd_kl_type="reverse_kl" if selection == "sampled" else "jsd",
                               opd_jsd_alpha=0.3, opd_norm_mode="tail", opd_log_prob_min_clamp=None,
                               opd_token_selection=selection, opd_per_token_clip=0.5, normalize_advantages=False)
        want = [torch.zeros(n) if only else torch.full((n,), r) for n, r in zip(lens, data["rewards"])]
        D.apply_to_advantages(args, data, want)
        dd = {key: ([t.to(dev) for t in val] if isinstance(val, list) and isinstance(val[0], torch.Tensor) else val)
              for key, val in data.items()}
        relax_amd.compute_advantages_and_returns(args, dd)
        for a, b in zip(dd["advantages"], want):
            torch.testing.assert_close(a.cpu(), b, atol=2e-6, rtol=2e-6)
        for r_, n, r in zip(dd["returns"], lens, data["rewards"]):
            assert torch.equal(r_.cpu(), torch.zeros(n) if only else torch.full((n,), r))


def test_reinforce_pp_baseline_wiring_literals():
    """The literal case of the reference's wiring test
    (tests/backends/megatron/test_reinforce_plus_plus_wiring.py:45-79): rewards [1, -1], masks [[1, 0], [1, 1]],
    gamma 1, no KL, normalisation on."""
    import relax_amd

    dev = require_gpu()
    announce("reinforce++ baseline wiring literals")
    args = SimpleNamespace(use_rollout_logprobs=False, kl_coef=0.0, kl_loss_type="k2",
                           advantage_estimator="reinforce_plus_plus_baseline", gamma=1.0, use_opd=False,
                           normalize_advantages=True)
    data = {"log_probs": [torch.zeros(2, device=dev), torch.zeros(2, device=dev)], "ref_log_probs": None,
            "rewards": [1.0, -1.0], "values": None, "response_lengths": [2, 2],
            "loss_masks": [torch.tensor([1.0, 0.0], device=dev), torch.tensor([1.0, 1.0], device=dev)],
            "total_lengths": [2, 2]}
    relax_amd.compute_advantages_and_returns(args, data)
    for got, want in zip(data["returns"], [[1.0, 0.0], [-1.0, -1.0]]):
        torch.testing.assert_close(got.cpu(), torch.tensor(want), atol=1e-6, rtol=1e-6)
    for got, want in zip(data["advantages"], [[2.0 ** 0.5, 0.0], [-(0.5 ** 0.5), -(0.5 ** 0.5)]]):
        torch.testing.assert_close(got.cpu(), torch.tensor(want), atol=1e-6, rtol=1e-6)
    assert data["reinforce_pp_valid_token_count"][0].item() == 3
    assert data["reinforce_pp_zero_variance"][0].item() == 0
    assert isinstance(data["reinforce_pp_advantage_raw_mean"][0], torch.Tensor)
