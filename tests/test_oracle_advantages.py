"""Pins oracle.advantages / oracle.opd / oracle.policy against reference literals and brute force (CPU)."""

import math

import numpy as np
import pytest
import torch

from oracle import advantages as A
from oracle import opd as D
from oracle import policy as P
from oracle import reducers as R


def test_rloo_literals_and_bruteforce(literals):
    fx = literals["group_rewards"]
    torch.testing.assert_close(A.rloo_leave_one_out(torch.tensor(fx["rloo_pair"]["rewards"])), torch.tensor(fx["rloo_pair"]["expected"]))
    got = A.rloo_leave_one_out(torch.tensor(fx["rloo_binary"]["rewards"], dtype=torch.float64))
    torch.testing.assert_close(got, torch.tensor(fx["rloo_binary"]["expected"], dtype=torch.float64))
    assert A.rloo_leave_one_out(torch.full((4,), 2.5)).abs().max() == 0
    for g in (2, 3, 5, 8):
        torch.manual_seed(g)
        r = torch.randn(g, dtype=torch.float64)
        want = [r[i].item() - (r.sum().item() - r[i].item()) / (g - 1) for i in range(g)]
        torch.testing.assert_close(A.rloo_leave_one_out(r), torch.tensor(want, dtype=torch.float64), atol=1e-12, rtol=0)
    with pytest.raises(ValueError, match="1-D"):
        A.rloo_leave_one_out(torch.zeros(2, 2))
    with pytest.raises(ValueError, match=">= 2"):
        A.rloo_leave_one_out(torch.zeros(1))
    for bad in (float("nan"), float("inf"), -float("inf")):
        with pytest.raises(ValueError, match="non-finite"):
            A.rloo_leave_one_out(torch.tensor([1.0, bad]))


def test_group_normalise_literals(literals):
    fx = literals["group_rewards"]
    r = fx["grpo_binary"]["rewards"]
    got = A.group_normalise(r, [0, 0, 0, 0], 4, "grpo", True)
    arr = np.asarray(r, dtype=np.float32)
    want = (arr - arr.mean()) / (arr.std(ddof=1) + 1e-6)
    np.testing.assert_allclose(got.numpy(), want, atol=1e-6)
    got = A.group_normalise(r, [0, 0, 0, 0], 4, "rloo")
    np.testing.assert_allclose(got.numpy(), [(4 / 3) * (x - 0.5) for x in r], atol=1e-6)
    b = fx["rpp_baseline"]
    got = A.group_normalise(b["rewards"], b["groups"], 2, "reinforce_plus_plus_baseline")
    assert got.tolist() == b["expected"]
    with pytest.raises(ValueError, match="3 samples, expected 4"):
        A.group_normalise([1.0, 2.0, 3.0], [0, 0, 0], 4)
    # interleaved groups keep input order
    got = A.group_normalise([1.0, 10.0, 3.0, 12.0], [0, 1, 0, 1], 2, "grpo", False)
    assert got.tolist() == [-1.0, -1.0, 1.0, 1.0]


def test_grpo_micro_fixture_end_to_end(literals):
    fx = literals["grpo_micro_fixture"]
    norm = A.group_normalise(fx["raw_rewards"], fx["group_indices"], 2, "grpo", std_norm=False)
    assert norm.tolist() == fx["normalized_rewards"]
    like = [torch.zeros(n) for n in fx["response_lengths"]]
    adv, ret = A.advantages_and_returns(norm.tolist(), like)
    assert torch.cat(adv).tolist() == fx["advantages"] and torch.cat(ret).tolist() == fx["advantages"]

    # policy composition with log-probs forced through fabricated logits is covered on the GPU side; here the
    # composition is checked by substituting per-token values (entropy 0.5, lp constant, old = 0)
    from oracle import losses as L

    masks = [torch.ones(2) for _ in range(4)]
    red = R.make_reducer(fx["response_lengths"], masks)
    advt = torch.tensor(fx["advantages"])
    for lp_val, want in ((0.0, None), (0.5, fx["lp_half_case"])):
        lp = torch.full((8,), lp_val)
        ppo_kl = torch.zeros(8) - lp
        pg, cf = L.policy_clip(ppo_kl, advt, *fx["eps"])
        ent = torch.full((8,), fx["entropy"])
        loss = red(pg) - fx["entropy_coef"] * red(ent)
        if want is None:
            assert abs(red(pg).item()) < 1e-7 and abs(red(ent).item() - 2.0) < 1e-7
            assert abs(loss.item() - fx["default_loss"]) < 1e-7
        else:
            assert abs(red(pg).item() - want["pg_loss"]) < 1e-5
            assert abs(red(cf).item() - want["pg_clipfrac"]) < 1e-7
            assert abs(red(ppo_kl).item() - want["ppo_kl"]) < 1e-6
            assert abs(loss.item() - want["loss"]) < 1e-5


def test_grpo_returns_shapes_dtypes(literals):
    fx = literals["grpo_returns"]
    like = [torch.randn(3), torch.randn(2, 2, dtype=torch.float64)]
    out = A.grpo_returns(torch.tensor(fx["rewards"]), like)
    assert out[0].shape == (3,) and out[0].dtype == torch.float32 and (out[0] == 1.5).all()
    assert out[1].shape == (2, 2) and out[1].dtype == torch.float64 and (out[1] == -0.25).all()


def test_masked_whiten_textbook_and_edges():
    torch.manual_seed(0)
    v = torch.randn(100)
    m = (torch.rand(100) > 0.3).float()
    got = A.masked_whiten(v, m)
    sel = v[m.bool()].double().numpy()
    want = (v.double().numpy() - sel.mean()) / np.sqrt(sel.var(ddof=1) + 1e-8)
    np.testing.assert_allclose(got.numpy(), want, rtol=2e-5, atol=2e-5)
    assert got[~m.bool()].abs().sum() > 0  # values outside the mask are transformed, not zeroed
    one = A.masked_whiten(torch.tensor([3.0, 5.0]), torch.tensor([1.0, 0.0]))  # n == 1: no Bessel, var = 0
    np.testing.assert_allclose(one.numpy(), [0.0, 2.0 / math.sqrt(1e-8)], rtol=1e-4)
    keep = A.masked_whiten(v, m, shift_mean=False)
    np.testing.assert_allclose(keep.numpy(), want + sel.mean(), rtol=2e-5, atol=2e-5)
    with pytest.raises(ValueError, match="zero"):
        A.masked_whiten(v, torch.zeros(100))


def test_full_vocab_reverse_kl_equals_textbook_in_all_norm_modes():
    torch.manual_seed(1)
    s = torch.randn(6, 50) * 2
    t = s + torch.randn(6, 50)
    ps = torch.softmax(s.double(), -1)
    want = (ps * (torch.log_softmax(s.double(), -1) - torch.log_softmax(t.double(), -1))).sum(-1)
    for mode in ("tail", "norm", "trunc"):
        got = D.full_vocab_reverse_kl(s, t, mode)
        torch.testing.assert_close(got.double(), want, atol=5e-6, rtol=0)
    assert (want >= 0).all()
    torch.testing.assert_close(D.full_vocab_reverse_kl(s, s), torch.zeros(6), atol=1e-6, rtol=0)


def test_opd_sampled_token_forms_and_tail_bin():
    s, t = torch.tensor([-0.5, -2.0]), torch.tensor([-1.0, -0.3])
    torch.testing.assert_close(D.opd_kl(s, t, "reverse_kl"), s - t)
    d = s - t
    torch.testing.assert_close(D.opd_kl(s, t, "low_var_kl"), torch.exp(-d) - 1 + d)
    # top-2 of a 3-way distribution: tail bin must restore the exact 3-way KL
    ps, pt = torch.tensor([[0.5, 0.3, 0.2]]), torch.tensor([[0.2, 0.5, 0.3]])
    got = D.opd_kl_topk(ps[:, :2].log(), pt[:, :2].log(), "reverse_kl", norm_mode="tail")
    want = (ps * (ps.log() - pt.log())).sum(-1)
    torch.testing.assert_close(got, want, atol=1e-6, rtol=0)
    got = D.opd_kl_topk(ps[:, :2].log(), pt[:, :2].log(), "forward_kl", norm_mode="tail")
    torch.testing.assert_close(got, (pt * (pt.log() - ps.log())).sum(-1), atol=1e-6, rtol=0)


def test_reinforce_pp_returns_reference_cases_by_hand():
    """The input cases of the reference's own test (tests/utils/training/test_reinforce_plus_plus.py:45-127) with the
    expected returns worked out by hand."""
    kls = [torch.tensor([0.2], dtype=torch.float64), torch.tensor([0.1, 9999.0, -0.3], dtype=torch.float64),
           torch.tensor([0.2, -0.4, 0.7, -8888.0, 0.5], dtype=torch.float64)]
    masks = [torch.tensor([1.0], dtype=torch.float64), torch.tensor([1.0, 0.0, 1.0], dtype=torch.float64),
             torch.tensor([1.0, 1.0, 1.0, 0.0, 1.0], dtype=torch.float64)]
    got = A.reinforce_pp_returns(torch.tensor([1.5, -0.25, 2.0], dtype=torch.float64), kls, masks, 0.2, 1.0)
    # gamma = 1: reverse cumulative sums of r = -0.2 * kl (valid tokens) with the reward on the last valid token
    want = [[1.5 - 0.04], [-0.02 + (0.06 - 0.25), 0.0, 0.06 - 0.25],
            [-0.04 + 0.08 - 0.14 + (2.0 - 0.1), 0.08 - 0.14 + 1.9, -0.14 + 1.9, 0.0, 1.9]]
    for g, w in zip(got, want):
        torch.testing.assert_close(g, torch.tensor(w, dtype=torch.float64), atol=1e-12, rtol=0)
    # discounting, masked garbage in the middle: r = [-0.05, 0, 1.025]
    got = A.reinforce_pp_returns(torch.tensor([1.0], dtype=torch.float64),
                                 [torch.tensor([0.5, 12345.0, -0.25], dtype=torch.float64)],
                                 [torch.tensor([1.0, 0.0, 1.0], dtype=torch.float64)], 0.1, 0.5)
    torch.testing.assert_close(got[0], torch.tensor([0.20625, 0.0, 1.025], dtype=torch.float64), atol=1e-12, rtol=0)
    # fully masked NaN / inf -> exact zeros; non-finite values outside the mask never leak
    got = A.reinforce_pp_returns(torch.tensor([0.0]), [torch.tensor([float("nan"), float("inf")])], [torch.zeros(2)], 0.1, 1.0)
    assert torch.equal(got[0], torch.zeros(2))
    got = A.reinforce_pp_returns(torch.tensor([1.0], dtype=torch.float64),
                                 [torch.tensor([0.5, float("nan"), -0.25, float("inf")], dtype=torch.float64)],
                                 [torch.tensor([1.0, 0.0, 1.0, 0.0], dtype=torch.float64)], 0.1, 1.0)
    torch.testing.assert_close(got[0], torch.tensor([-0.05 + 1.025, 0.0, 1.025, 0.0], dtype=torch.float64), atol=1e-12, rtol=0)
    base = A.reinforce_pp_baseline_advantages(
        torch.tensor([1.0, -1.0], dtype=torch.float64),
        [torch.tensor([5.0, 9999.0, -7.0], dtype=torch.float64), torch.tensor([-123.0, float("nan")], dtype=torch.float64)],
        [torch.tensor([1.0, 0.0, 1.0], dtype=torch.float64), torch.tensor([0.0, 1.0], dtype=torch.float64)])
    assert base[0].tolist() == [1.0, 0.0, 1.0] and base[1].tolist() == [0.0, -1.0]


def test_gae_textbook_sum_and_masked_normalize_moments():
    torch.manual_seed(0)
    r, v = torch.randn(37, dtype=torch.float64), torch.randn(37, dtype=torch.float64)
    gamma, lam = 0.99, 0.95
    adv, ret = A.gae(v, r, gamma, lam)
    nxt = torch.cat([v[1:], torch.zeros(1, dtype=torch.float64)])
    delta = r + gamma * nxt - v
    want = torch.stack([sum((gamma * lam) ** l * delta[t + l] for l in range(37 - t)) for t in range(37)])
    torch.testing.assert_close(adv, want, atol=1e-12, rtol=1e-12)
    torch.testing.assert_close(ret, want + v, atol=1e-12, rtol=1e-12)
    # lambda = 1, gamma = 1: advantage = reward-to-go minus the value
    adv, _ = A.gae(v, r, 1.0, 1.0)
    torch.testing.assert_close(adv, torch.flip(torch.cumsum(torch.flip(r, [0]), 0), [0]) - v, atol=1e-12, rtol=1e-12)
    x = torch.randn(200)
    m = (torch.rand(200) > 0.3).float()
    x[m == 0] = float("nan")
    out, mean, var, cnt = A.masked_normalize(x, m)
    sel = x[m != 0].double().numpy()
    assert cnt.item() == len(sel)
    np.testing.assert_allclose(mean.item(), sel.mean(), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(var.item(), sel.var(ddof=0), rtol=1e-5)
    np.testing.assert_allclose(out[m != 0].numpy(), (sel - sel.mean()) / np.sqrt(sel.var(ddof=0)), rtol=2e-5, atol=2e-5)
    assert (out[m == 0] == 0).all()
    const, _, var0, _ = A.masked_normalize(torch.full((5,), 3.0), torch.ones(5))
    assert var0.item() == 0 and (const == 0).all()


def test_opd_union_mask_and_jsd_closed_forms():
    """The union path's padding mask: padded entries drop out, the tail bin is cut off with them, and the masked
    result equals the unmasked one on the row's valid prefix; JSD against its textbook definition."""
    torch.manual_seed(3)
    s = torch.log_softmax(torch.randn(4, 12), -1)[:, :6]
    t = torch.log_softmax(torch.randn(4, 12), -1)[:, :6]
    ksz = torch.tensor([6, 4, 1, 3])
    mask = torch.arange(6).unsqueeze(0) < ksz.unsqueeze(1)
    for kl_type, alpha in (("reverse_kl", 0.0), ("forward_kl", 1.0), ("jsd", 0.25), ("low_var_kl", 0.0)):
        for mode in ("norm", "trunc"):
            got = D.opd_kl_topk(s, t, kl_type, alpha, mode, None, mask)
            for i, n in enumerate(ksz.tolist()):
                want = D.opd_kl_topk(s[i:i + 1, :n], t[i:i + 1, :n], kl_type, alpha, mode)
                torch.testing.assert_close(got[i:i + 1], want, atol=1e-6, rtol=1e-6)
        # with a mask the tail bin does not contribute: "tail" degenerates to "trunc"
        torch.testing.assert_close(D.opd_kl_topk(s, t, kl_type, alpha, "tail", None, mask),
                                   D.opd_kl_topk(s, t, kl_type, alpha, "trunc", None, mask))
    # generalised JSD on complete distributions: (1-a) KL(p || m) + a KL(q || m), m = (1-a) p + a q
    p, q = torch.softmax(torch.randn(5, 9).double(), -1), torch.softmax(torch.randn(5, 9).double(), -1)
    a = 0.3
    m = (1 - a) * p + a * q
    want = (1 - a) * (p * (p / m).log()).sum(-1) + a * (q * (q / m).log()).sum(-1)
    got = D.opd_kl_topk(p.log().float(), q.log().float(), "jsd", a, "trunc")
    torch.testing.assert_close(got.double(), want, atol=1e-6, rtol=1e-5)
    # clamping from below bounds the log-ratio
    lo = D.opd_kl(torch.tensor([-50.0]), torch.tensor([-1.0]), "reverse_kl", min_clamp=-10.0)
    assert lo.item() == -9.0


def test_log_probs_on_topk_ids_against_log_softmax():
    torch.manual_seed(5)
    x = torch.randn(7, 40) * 3
    ids = torch.randint(0, 40, (7, 5))
    ids[0, 0], ids[1, 1] = -1, 45
    got = D.log_probs_on_topk_ids(x, ids)
    ref = torch.log_softmax(x.double(), -1)
    ok = (ids >= 0) & (ids < 40)
    torch.testing.assert_close(got[ok].double(), ref.gather(-1, ids.clamp(0, 39))[ok], atol=2e-6, rtol=0)
    assert got[0, 0] == float("-inf")
    torch.testing.assert_close(got[1, 1].double(), -torch.logsumexp(x[1].double(), -1), atol=2e-6, rtol=0)
    assert D.log_probs_on_topk_ids(x[:0], ids[:0]).shape == (0, 5)


def test_response_slicing_literal_and_bruteforce(literals):
    fx = literals["response_slicing"]
    logits = torch.tensor(fx["logits"])
    toks = [torch.tensor(fx["tokens"])]
    (chunk, targets), = list(P.iter_responses(logits, toks, fx["total_lengths"], fx["response_lengths"]))
    assert torch.equal(chunk, logits[0, fx["expected_rows"]]) and targets.tolist() == fx["expected_targets"]
    # brute-force enumeration: token at absolute position p (>=1) is scored by logits row p-1
    tot, resp = [5, 3, 7, 4], [2, 3, 1, 3]  # second sample is SFT-shaped (response == total)
    ranges = P.response_row_ranges(tot, resp)
    base = 0
    for (b, e, sft), t, r in zip(ranges, tot, resp):
        if sft:
            assert (b, e) == (base, base + t)
        else:
            want_rows = [base + p - 1 for p in range(t - r, t)]
            assert list(range(b, e)) == want_rows
        base += t


def test_get_log_probs_entropy_grad_wiring(literals):
    fx = literals["response_slicing"]
    for coef in (0.0, 0.01):
        logits = torch.tensor(fx["logits"], requires_grad=True)
        _, out = P.get_log_probs_and_entropy(
            logits, args=P.make_args(entropy_coef=coef), unconcat_tokens=[torch.tensor(fx["tokens"])],
            total_lengths=fx["total_lengths"], response_lengths=fx["response_lengths"], with_entropy=True,
        )
        assert out["entropy"][0].requires_grad == (coef != 0)
        want = torch.log_softmax(logits[0, :2], -1)[torch.arange(2), torch.tensor(fx["expected_targets"])]
        torch.testing.assert_close(out["log_probs"][0], want, atol=1e-6, rtol=0)


def test_lm_head_log_probs_vs_library():
    torch.manual_seed(0)
    h = torch.randn(4, 3, requires_grad=True)
    w = torch.randn(5, 3, requires_grad=True)
    labels = torch.tensor([4, 1, 3, 0])
    wts = torch.tensor([0.25, -0.5, 1.5, 0.75])
    lp = P.lm_head_log_probs(h, w, labels, temperature=0.7, sub_chunk=2)
    (lp * wts).sum().backward()
    h2, w2 = h.detach().clone().requires_grad_(), w.detach().clone().requires_grad_()
    want = torch.log_softmax(torch.nn.functional.linear(h2, w2) / 0.7, -1)[torch.arange(4), labels]
    (want * wts).sum().backward()
    torch.testing.assert_close(lp, want, atol=1e-6, rtol=0)
    torch.testing.assert_close(h.grad, h2.grad, atol=1e-6, rtol=0)
    torch.testing.assert_close(w.grad, w2.grad, atol=1e-6, rtol=0)


def test_policy_loss_function_composition_against_direct_autograd():
    """ppo + k3 (+unbiased) + entropy coef; compared with a flat fp64 restatement written with library routines."""
    torch.manual_seed(5)
    tot, resp, v = [6, 4, 5], [3, 2, 4], 11
    t = sum(tot)
    logits = torch.randn(1, t, v, requires_grad=True)
    toks = [torch.randint(0, v, (n,)) for n in tot]
    masks = [torch.tensor([1.0, 0.0, 1.0]), torch.tensor([1.0, 1.0]), torch.tensor([0.0, 1.0, 1.0, 1.0])]
    n = sum(resp)
    batch = dict(
        advantages=[torch.randn(r) for r in resp], log_probs=list(torch.split(torch.randn(n) * 0.1 - 2.3, resp)),
        ref_log_probs=list(torch.split(torch.randn(n) * 0.1 - 2.3, resp)), unconcat_tokens=toks,
        response_lengths=resp, total_lengths=tot, loss_masks=masks,
    )
    for unbiased in (False, True):
        args = P.make_args(eps_clip=0.2, eps_clip_high=0.28, use_kl_loss=True, kl_loss_coef=0.05, kl_loss_type="k3",
                           entropy_coef=0.02, use_unbiased_kl=unbiased)
        red = R.make_reducer(resp, masks)
        logits.grad = None
        loss, met = P.policy_loss_function(args, batch, logits, red)
        loss.backward()

        x = logits.detach().double().requires_grad_()
        rows, tg = [], []
        for (b, e, _), tk, r in zip(P.response_row_ranges(tot, resp), toks, resp):
            rows += list(range(b, e))
            tg += tk[-r:].tolist()
        ls = torch.log_softmax(x[0, rows], -1)
        lp = ls[torch.arange(n), torch.tensor(tg)]
        ent = -(ls.exp() * ls).sum(-1)
        old, ref = torch.cat(batch["log_probs"]).double(), torch.cat(batch["ref_log_probs"]).double()
        adv, m = torch.cat(batch["advantages"]).double(), torch.cat(masks).double()
        ratio = (lp - old).exp()
        pg = torch.maximum(-ratio * adv, -ratio.clamp(0.8, 1.28) * adv)
        d = lp - ref
        k3 = (-d).exp() - 1 + d
        if unbiased:
            k3 = ratio * k3
        seg = torch.tensor(sum(([i] * r for i, r in enumerate(resp)), []))
        den = torch.zeros(3, dtype=torch.float64).index_add_(0, seg, m).clamp_min(1)

        def sm(val):
            return torch.zeros(3, dtype=torch.float64).index_add(0, seg, val * m).div(den).sum()

        want = sm(pg) - 0.02 * sm(ent) + 0.05 * sm(k3)
        want.backward()
        assert abs(loss.item() - want.item()) < 1e-5
        torch.testing.assert_close(logits.grad.double(), x.grad, atol=1e-6, rtol=0)
        assert abs(met["kl_loss"].item() - sm(k3).item()) < 1e-5 and abs(met["entropy_loss"].item() - sm(ent).item()) < 1e-5


def test_loss_function_scaling_tail():
    torch.manual_seed(6)
    tot, resp, v = [4, 5], [2, 3], 7
    logits = torch.randn(1, 9, v)
    batch = dict(
        advantages=[torch.randn(r) for r in resp], log_probs=[torch.randn(r) for r in resp],
        unconcat_tokens=[torch.randint(0, v, (n,)) for n in tot], response_lengths=resp, total_lengths=tot,
        loss_masks=[torch.tensor([1, 1]), torch.tensor([1, 0, 1])],
    )
    a = P.make_args(global_batch_size=8)
    loss, norm, log = P.loss_function(a, batch, 4, logits, dp_world=2)
    raw, _ = P.policy_loss_function(a, batch, logits, R.make_reducer(resp, batch["loss_masks"]))
    assert abs(loss.item() - raw.item() * 4 / 8 * 2) < 1e-6 and norm.item() == 1 and log["values"][0].item() == 0
    assert log["keys"][:5] == ["loss", "pg_loss", "entropy_loss", "pg_clipfrac", "ppo_kl"]
    a = P.make_args(calculate_per_token_loss=True)
    loss, norm, log = P.loss_function(a, batch, 4, logits)
    assert norm.item() == 4 and norm.dtype == torch.int64 and log["values"][0].item() == 4
