"""Pins oracle.losses / oracle.reducers against the reference's literals, closed forms and brute force (CPU)."""

import math

import pytest
import torch

from oracle import losses as L
from oracle import reducers as R


def _t(x, dt=torch.float64):
    return torch.tensor(x, dtype=dt)


def test_ppo_clip_and_k2_response_mean_literal(literals):
    fx = literals["ppo_clip_k2_response_mean"]
    cur, old, ref, adv = _t(fx["current"]), _t(fx["old"]), _t(fx["reference"]), _t(fx["advantages"])
    masks = [torch.tensor(m) for m in fx["masks"]]
    lens = fx["response_lengths"]
    pg, _ = L.policy_clip(old - cur, adv, *fx["eps"])
    k2 = L.approx_kl(cur, ref, "k2")
    red = R.make_reducer(lens, masks)
    # independent: python loops over tokens
    exp_pg, exp_k2 = [], []
    for c, o, r, a in zip(fx["current"], fx["old"], fx["reference"], fx["advantages"]):
        ratio = math.exp(c - o)
        exp_pg.append(max(-ratio * a, -min(max(ratio, 0.8), 1.2) * a))
        exp_k2.append(0.5 * (c - r) ** 2)
    torch.testing.assert_close(pg, _t(exp_pg), atol=fx["tol"], rtol=fx["tol"])
    torch.testing.assert_close(k2.double(), _t(exp_k2), atol=fx["tol"], rtol=fx["tol"])

    def resp_mean(vals):
        out, off = 0.0, 0
        for n, m in zip(lens, fx["masks"]):
            out += sum(v * w for v, w in zip(vals[off : off + n], m)) / sum(m)
            off += n
        return out / len(lens)

    assert abs(float(red(pg)) / len(lens) - resp_mean(exp_pg)) < fx["tol"]
    assert abs(float(red(k2)) / len(lens) - resp_mean(exp_k2)) < fx["tol"]


def test_masked_tokens_do_not_change_reduction_but_nan_propagates(literals):
    fx = literals["masked_invariance"]
    masks = [torch.tensor(m) for m in fx["masks"]]
    red = R.make_reducer(fx["lengths"], masks)
    assert torch.equal(red(torch.tensor(fx["base"])), red(torch.tensor(fx["changed"])))
    bad = torch.tensor([1.0, float("nan"), 3.0, 4.0, float("inf")])
    assert torch.isnan(red(bad))
    assert torch.isnan(R.make_reducer(fx["lengths"], masks, per_token=True)(bad))


def test_clip_case_literal(literals):
    fx = literals["clip_case"]
    pg, cf = L.policy_clip(_t([fx["ppo_kl"]]), _t([fx["advantage"]]), *fx["eps"])
    assert cf.item() == fx["expected_clipfrac"]
    assert abs(pg.item() - (-1.2)) < 1e-12
    loss, cf = L.rloo_loss(_t([fx["rloo_log_prob"]]), _t([1.0]))
    assert abs(loss.item() - fx["rloo_expected_loss"]) < 1e-12 and cf.item() == fx["rloo_expected_clipfrac"]


def test_kl_estimators_literal(literals):
    fx = literals["kl_estimators"]
    for kind in ("k1", "k2", "k3", "low_var_kl"):
        lp, base = fx[kind]["lp"], fx[kind]["base"]
        got = L.approx_kl(torch.tensor(lp), torch.tensor(base), kind)
        for g, a, b in zip(got.tolist(), lp, base):
            d = a - b
            want = {"k1": d, "k2": d * d / 2, "k3": math.exp(-d) - 1 + d, "low_var_kl": min(10.0, math.exp(-d) - 1 + d)}[kind]
            assert abs(g - want) < fx["atol"] * max(1.0, abs(want))
        if kind in ("k2", "k3", "low_var_kl"):
            assert (got >= 0).all()
    assert L.approx_kl(torch.tensor(fx["low_var_kl"]["lp"]), torch.zeros(3), "low_var_kl")[0].item() == 10.0
    with pytest.raises(ValueError, match="Unknown kl_loss_type: unsupported"):
        L.approx_kl(torch.zeros(2), torch.zeros(2), "unsupported")


def test_unbiased_kl_multiplies_ratio():
    lp, base, ratio = torch.tensor([-0.5, -1.0]), torch.tensor([-0.7, -0.4]), torch.tensor([1.3, 0.6])
    torch.testing.assert_close(L.approx_kl(lp, base, "k3", ratio), ratio * L.approx_kl(lp, base, "k3"))


def test_ppo_clip_gradient_convention_bruteforce():
    # dloss/dlp = -A*r where unclipped branch is active (incl. inside the clamp range), else 0
    torch.manual_seed(0)
    lp = (torch.randn(200, dtype=torch.float64) * 0.3).requires_grad_()
    old = torch.randn(200, dtype=torch.float64) * 0.3
    adv = torch.randn(200, dtype=torch.float64)
    adv[:5] = 0.0
    loss, _ = L.policy_clip(old - lp, adv, 0.2, 0.28)
    loss.sum().backward()
    for i in range(200):
        r = math.exp(lp[i].item() - old[i].item())
        a = adv[i].item()
        inside = 0.8 <= r <= 1.28
        active = inside or (-r * a > -min(max(r, 0.8), 1.28) * a)
        want = -a * r if active else 0.0
        assert abs(lp.grad[i].item() - want) < 1e-12


def test_dual_clip_bruteforce():
    torch.manual_seed(1)
    kl = torch.randn(100, dtype=torch.float64)
    adv = torch.randn(100, dtype=torch.float64)
    loss, _ = L.policy_clip(kl, adv, 0.2, 0.2, 3.0)
    for i in range(100):
        r, a = math.exp(-kl[i].item()), adv[i].item()
        base = max(-r * a, -min(max(r, 0.8), 1.2) * a)
        want = min(-3.0 * a, base) if a < 0 else base
        assert abs(loss[i].item() - want) < 1e-12


def test_gspo_seq_kl_bruteforce_and_gradient():
    torch.manual_seed(2)
    lens = [3, 5, 1]
    lps = [torch.randn(n, dtype=torch.float64, requires_grad=True) for n in lens]
    olds = [torch.randn(n, dtype=torch.float64) for n in lens]
    masks = [torch.tensor([1.0, 0.0, 1.0]).double(), torch.ones(5).double(), torch.zeros(1).double()]
    out = L.gspo_seq_kl(lps, olds, masks)
    off = 0
    for lp, old, m in zip(lps, olds, masks):
        num = sum((o - l) * w for o, l, w in zip(old.tolist(), lp.tolist(), m.tolist()))
        k = num / max(sum(m.tolist()), 1.0)
        for j in range(len(lp)):
            assert abs(out[off + j].item() - k) < 1e-12
        off += len(lp)
    out.sum().backward()
    # d(sum_t k_i)/dlp_t = -R_i * m_t / clamp(sum m, 1)
    for lp, m, n in zip(lps, masks, lens):
        want = -n * m / max(m.sum().item(), 1.0)
        torch.testing.assert_close(lp.grad, want)


def test_cispo_bruteforce_and_gradient():
    torch.manual_seed(3)
    lp = torch.randn(300, dtype=torch.float64).requires_grad_()
    old = lp.detach() + torch.randn(300, dtype=torch.float64) * 0.5
    adv = torch.randn(300, dtype=torch.float64)
    adv[:4] = 0.0
    loss, cf = L.cispo(lp, old - lp, adv, 0.2, 0.28)
    loss.sum().backward()
    for i in range(300):
        r, a = math.exp(lp[i].item() - old[i].item()), adv[i].item()
        coef = min(r, 1.28) if a >= 0 else max(r, 0.8)  # A == 0 takes the upper-cap branch
        assert abs(loss[i].item() - (-coef * a * lp[i].item())) < 1e-12
        assert abs(lp.grad[i].item() - (-coef * a)) < 1e-12
        assert cf[i].item() == float((a >= 0 and r > 1.28) or (a < 0 and r < 0.8))


def test_per_token_path_literal(literals):
    fx = literals["per_token_loss_path"]
    masks = [_t(m) for m in fx["masks"]]
    lp = _t(fx["log_probs"]).requires_grad_()
    adv = _t(fx["advantages"])
    red = R.make_reducer(fx["response_lengths"], masks, per_token=True)
    loss, _ = L.rloo_loss(lp, adv)
    tok_sum = red(loss)
    n = R.num_tokens(masks)
    flat = torch.cat(masks)
    torch.testing.assert_close(tok_sum, -(adv * lp * flat).sum())
    assert n.item() == fx["expected_normalizer"]
    (tok_sum / n).backward()
    torch.testing.assert_close(lp.grad, -(adv * flat) / fx["expected_normalizer"])
    mean_red = R.make_reducer(fx["response_lengths"], masks)
    assert not torch.allclose(tok_sum / n, mean_red(loss.detach()) / 2)


def test_target_coordinate_masks_and_counts(literals):
    fx = literals["target_coordinate_masks"]
    m = torch.tensor(fx["mask"])
    red = R.make_reducer([4], [m], per_token=True)
    assert red(torch.tensor(fx["values"])).item() == fx["token_sum"]
    assert R.num_tokens([m]).item() == fx["count"] and R.num_tokens([m]).dtype == torch.int64
    shifted = torch.nn.functional.pad(torch.tensor(fx["sft_mask_in"]), (0, 1))[1:]
    assert shifted.tolist() == fx["sft_mask_out"] and int(shifted.sum()) == fx["sft_count"]


def test_fully_masked_sample_counts_as_one_token():
    masks = [torch.tensor([0, 0, 0]), torch.tensor([1, 1])]
    assert R.num_tokens(masks).item() == 3
    red = R.make_reducer([3, 2], masks)
    assert red(torch.tensor([5.0, 5.0, 5.0, 2.0, 4.0])).item() == 3.0  # 0/clamp(0,1) + 6/2


def test_supplied_sample_denominators():
    masks = [torch.tensor([1.0, 1.0]), torch.tensor([1.0, 0.0])]
    red = R.make_reducer([2, 2], masks, sample_denoms=[3, 3])
    assert abs(red(torch.tensor([3.0, 3.0, 6.0, 9.0])).item() - (6 / 3 + 6 / 3)) < 1e-6


def test_opd_token_mean_literal(literals):
    fx = literals["opd_token_mean"]
    masks = [torch.tensor(m) for m in fx["masks"]]
    assert R.token_mean(fx["lengths"], masks)(torch.tensor(fx["values"])).item() == fx["expected"]


def test_tis_bruteforce():
    torch.manual_seed(4)
    tr, ro = torch.randn(50), torch.randn(50)
    pg = torch.randn(50)
    out, met = L.vanilla_tis(pg, tr, ro, 0.0, 2.0)
    for i in range(50):
        t = math.exp(tr[i].item() - ro[i].item())
        w = min(max(t, 0.0), 2.0)
        assert abs(out[i].item() - pg[i].item() * w) < 1e-5 * max(1, abs(pg[i].item() * w))
        assert met["tis_clipfrac"][i].item() == float(t > 2.0)


def test_sapo_gate_value_at_ratio_one():
    loss, cf = L.sapo(torch.zeros(2), torch.tensor([1.0, -1.0]), 1.0, 1.05)
    assert abs(loss[0].item() + 2.0) < 1e-6 and abs(loss[1].item() - 2.0 / 1.05) < 1e-6 and cf.sum() == 0


def test_value_loss_hand_computed():
    """Clipped value loss, worked by hand for clip 0.5 and old values 0: (v, R) = (1, 0) -> clipped to 0.5, max(0.25, 1)
    = 1, counted as clipped; (0.2, 0) -> 0.04, not clipped; (1, 2) -> max((0.5 - 2)^2, (1 - 2)^2) = 2.25, clipped.
    One sample of three response tokens after a two-token prompt: the values sit on head rows 1..3."""
    from types import SimpleNamespace

    from oracle import policy as P

    head = torch.tensor([9.0, 1.0, 0.2, 1.0, 9.0]).reshape(1, 5, 1)
    batch = dict(values=[torch.zeros(3)], returns=[torch.tensor([0.0, 0.0, 2.0])], total_lengths=[5],
                 response_lengths=[3], loss_masks=[torch.ones(3)])
    assert torch.equal(P.get_values(head, [5], [3])[0], torch.tensor([1.0, 0.2, 1.0]))
    red = R.make_reducer([3], batch["loss_masks"], False)
    loss, met = P.value_loss_function(SimpleNamespace(value_clip=0.5), batch, head, red)
    assert abs(loss.item() - (1 + 0.04 + 2.25) / 3) < 1e-6
    assert abs(met["value_clipfrac"].item() - 2 / 3) < 1e-6 and abs(met["value_loss"].item() - loss.item()) < 1e-7


# ---- pins for the functions the reference has no test or fixture for: every expectation below is worked out with
# ---- Python floats in explicit per-token / per-sequence loops, or from a closed form that is not the oracle's code


def _opsm_by_loops(delta, lps, olds, advs, masks):
    """compute_opsm_mask (relax/utils/training/ppo_utils.py:142-180) as scalar loops over sequences and tokens."""
    keep, frac = [], 0.0
    for lp, old, adv, m in zip(lps, olds, advs, masks):
        num = sum((o - c) * w for c, o, w in zip(lp, old, m))
        cnt = max(sum(m), 1)
        seq_kl = num / cnt
        dropped = 0
        for a in adv:  # the drop test looks at every token of the sequence, masked or not
            d = 1 if (a < 0 and seq_kl > delta) else 0
            keep.append(1.0 - d)
            dropped += d
        frac += dropped / cnt
    return keep, frac


def test_opsm_mask_per_sequence_loops_and_edge_cases():
    # sequence 0: mean (old - cur) over its 4 unmasked tokens is exactly 0.5 == delta -> NOT dropped (strict >)
    # sequence 1: same mean 0.75 > delta, advantages negative / zero / positive -> only A < 0 tokens dropped,
    #             including the one whose loss mask is 0 (the fraction counts it, over 3 unmasked tokens)
    # sequence 2: fully masked -> sequence KL 0/1 = 0 -> nothing dropped, denominator clamps to 1
    # sequence 3: mean -0.25 (policy moved towards the samples) -> nothing dropped
    # sequence 4: one unmasked token far off-policy, all advantages negative -> all 3 dropped, fraction 3/1
    lps = [[0.0, 0.0, 0.0, 0.0], [-1.0, -1.0, -1.0, -1.0], [0.0, -3.0], [0.5, 0.5], [-2.0, 0.0, 0.0]]
    olds = [[0.5, 0.5, 0.5, 0.5], [-0.25, -0.25, -0.25, 5.0], [4.0, 4.0], [0.25, 0.25], [0.0, 0.0, 0.0]]
    advs = [[-1.0, -1.0, -1.0, -1.0], [-2.0, 0.0, 3.0, -0.5], [-1.0, -1.0], [-1.0, -1.0], [-1.0, -0.1, -7.0]]
    masks = [[1, 1, 1, 1], [1, 1, 1, 0], [0, 0], [1, 1], [1, 0, 0]]
    delta = 0.5
    want_keep, want_frac = _opsm_by_loops(delta, lps, olds, advs, masks)
    assert want_keep == [1, 1, 1, 1, 0, 1, 1, 0, 1, 1, 1, 1, 0, 0, 0]  # worked by hand, see the cases above
    assert abs(want_frac - (2 / 3 + 3.0)) < 1e-12
    for mask_dtype in (torch.float32, torch.int64):
        got, frac = L.opsm_mask(delta, [_t(x, torch.float32) for x in lps], [_t(x, torch.float32) for x in olds],
                                [_t(x, torch.float32) for x in advs], [torch.tensor(x, dtype=mask_dtype) for x in masks])
        assert got.tolist() == want_keep
        assert abs(frac.item() - want_frac) < 1e-6


@pytest.mark.parametrize("seed", range(4))
def test_opsm_mask_random_vs_loops(seed):
    g = torch.Generator().manual_seed(seed)
    lens = [int(x) for x in torch.randint(1, 9, (7,), generator=g)]
    lps = [torch.randn(n, generator=g, dtype=torch.float64) for n in lens]
    olds = [lp + 0.3 * torch.randn(lp.shape, generator=g, dtype=torch.float64) for lp in lps]
    advs = [torch.randn(n, generator=g, dtype=torch.float64) for n in lens]
    masks = [(torch.rand(n, generator=g) > 0.4).double() for n in lens]
    delta = 0.02
    want_keep, want_frac = _opsm_by_loops(delta, [x.tolist() for x in lps], [x.tolist() for x in olds],
                                          [x.tolist() for x in advs], [x.tolist() for x in masks])
    got, frac = L.opsm_mask(delta, lps, olds, advs, masks)
    assert got.tolist() == want_keep
    assert abs(frac.item() - want_frac) < 1e-12
    assert 0 < sum(want_keep) < len(want_keep)  # the case exercises both outcomes


def test_icepop_bruteforce_with_ratios_exactly_at_both_bounds():
    # icepop_function (relax/backends/megatron/loss.py:772-801): weight = ratio inside the CLOSED interval, else 0
    tr = torch.tensor([0.0, 0.0, -1.0, 1.0, 0.3, -0.2, 0.0])
    ro = torch.tensor([0.0, 0.0, 0.0, 0.0, 0.1, 0.1, 2.0])
    pg = torch.tensor([2.0, -3.0, 1.5, 0.5, -1.0, 4.0, 1.0])
    for lo, hi in ((1.0, 2.0), (0.5, 1.0), (0.5, 2.0), (0.0, 0.9)):
        out, met = L.icepop(pg, tr, ro, lo, hi)
        for i in range(tr.numel()):
            lr = tr[i].item() - ro[i].item()
            ratio = math.exp(lr)
            inside = lo <= ratio <= hi
            if lr == 0.0:  # exp(0) == 1 exactly: on the lower bound in the first pair, on the upper in the second
                assert ratio == 1.0 and inside == (lo <= 1.0 <= hi)
            w = ratio if inside else 0.0
            assert abs(out[i].item() - pg[i].item() * w) < 1e-6 * max(1.0, abs(pg[i].item() * w)), (lo, hi, i)
            assert met["tis_clipfrac"][i].item() == (0.0 if inside else 1.0)
            assert abs(met["tis"][i].item() - ratio) < 1e-6 * ratio
            assert abs(met["tis_abs"][i].item() - abs(ratio - 1)) < 1e-6
            assert abs(met["mismatch_kl"][i].item() + lr) < 1e-6
            assert abs(met["mismatch_k3_kl"][i].item() - (ratio - lr - 1)) < 1e-6
    # kept at the bound, dropped one ulp outside it
    one_up = torch.nextafter(torch.tensor(1.0), torch.tensor(2.0)).item()
    out, met = L.icepop(torch.ones(1), torch.zeros(1), torch.zeros(1), one_up, 2.0)
    assert out.item() == 0.0 and met["tis_clipfrac"].item() == 1.0
    out, met = L.icepop(torch.ones(1), torch.zeros(1), torch.zeros(1), 1.0, 1.0)
    assert out.item() == 1.0 and met["tis_clipfrac"].item() == 0.0


def test_icepop_gradient_flows_through_pg_loss_only_by_weight():
    tr = torch.tensor([0.2, -0.7, 0.05], dtype=torch.float64)
    ro = torch.tensor([0.0, 0.0, 0.0], dtype=torch.float64)
    pg = torch.tensor([1.0, 2.0, 3.0], dtype=torch.float64, requires_grad=True)
    out, _ = L.icepop(pg, tr, ro, 0.6, 1.2)
    out.sum().backward()
    want = [math.exp(0.2) if 0.6 <= math.exp(0.2) <= 1.2 else 0.0, 0.0, math.exp(0.05)]
    assert math.exp(-0.7) < 0.6 and math.exp(0.2) > 1.2 and want[0] == 0.0
    torch.testing.assert_close(pg.grad, _t(want), atol=1e-12, rtol=0)


def _sapo_by_loops(kl, adv, tau_pos, tau_neg):
    loss, cf, dloss_dkl = [], [], []
    for k, a in zip(kl, adv):
        r = math.exp(-k)
        tau = tau_pos if a > 0 else tau_neg  # A == 0 takes tau_neg (ppo_utils.py:247-251: `advantages > 0`)
        s = 1.0 / (1.0 + math.exp(-tau * (r - 1.0)))
        loss.append(-(4.0 / tau) * s * a)
        # 4 s (1 - s) = sech^2(x / 2): below 0.9 exactly when |x| > 2 atanh(sqrt(0.1))
        cf.append(1.0 if abs(tau * (r - 1.0)) > 2.0 * math.atanh(math.sqrt(0.1)) else 0.0)
        dloss_dkl.append(4.0 * s * (1.0 - s) * r * a)  # d/dkl of -(4/tau) sigma(tau (e^-kl - 1)) A
    return loss, cf, dloss_dkl


@pytest.mark.parametrize("taus", [(1.0, 1.05), (0.7, 2.0)])
def test_sapo_random_ratios_both_signs_zero_advantage_and_gradient(taus):
    g = torch.Generator().manual_seed(11)
    kl = torch.cat([0.6 * torch.randn(60, generator=g, dtype=torch.float64),
                    torch.tensor([0.0, 0.0, 0.0, 1.5, -1.5], dtype=torch.float64)])
    adv = torch.cat([torch.randn(60, generator=g, dtype=torch.float64),
                     torch.tensor([0.0, 2.0, -2.0, 0.0, 0.0], dtype=torch.float64)])
    want_loss, want_cf, want_grad = _sapo_by_loops(kl.tolist(), adv.tolist(), *taus)
    klg = kl.clone().requires_grad_()
    loss, cf = L.sapo(klg, adv, *taus)
    loss.sum().backward()
    torch.testing.assert_close(loss.detach(), _t(want_loss), atol=1e-12, rtol=1e-12)
    assert cf.tolist() == want_cf and 0 < sum(want_cf) < len(want_cf)
    torch.testing.assert_close(klg.grad, _t(want_grad), atol=1e-12, rtol=1e-12)
    # with respect to the current log-prob (kl = old - lp): -A * 4 sigma (1 - sigma) * r
    lp = (-kl).clone().requires_grad_()
    L.sapo(0.0 - lp, adv, *taus)[0].sum().backward()
    torch.testing.assert_close(lp.grad, -_t(want_grad), atol=1e-12, rtol=1e-12)


def test_sapo_temperature_pick_and_clip_fraction_threshold():
    # A == 0 and A < 0 use tau_neg, A > 0 uses tau_pos: visible at r = 1 where the gate is 2 / tau
    loss, _ = L.sapo(torch.zeros(3, dtype=torch.float64), _t([1e-30, -1e-30, 0.0]), 1.0, 4.0)
    assert loss[0].item() == -2.0 * 1e-30 and loss[1].item() == 0.5 * 1e-30 and loss[2].item() == 0.0
    # the zero-advantage token still reports its clip fraction with tau_neg: tau_neg*(r-1) = 4*0.2 -> weight 0.86
    r = 1.2
    _, cf = L.sapo(_t([-math.log(r)] * 2), _t([0.0, 1.0]), 1.0, 4.0)
    assert cf.tolist() == [1.0, 0.0]  # tau_pos*(r-1) = 0.2 -> weight 0.99
    # threshold: weight 4 s (1-s) < 0.9 <=> |tau (r-1)| > 0.6549...; 0.65 keeps, 0.66 counts
    x_star = 2.0 * math.atanh(math.sqrt(0.1))
    assert abs(x_star - 0.6549) < 1e-4
    for x, want in ((0.65, 0.0), (0.66, 1.0), (-0.65, 0.0), (-0.66, 1.0)):
        _, cf = L.sapo(_t([-math.log(1.0 + x)]), _t([1.0]), 1.0, 1.05)
        assert cf.item() == want, x


def test_seq_mean_token_sum_token_loop():
    # the aggregation of the packed varlen configuration: every sequence's masked token SUM, averaged over the B sequences
    # (fully masked sequences still count in B); the reference only has the plug-in point (loss.py:1062-1072)
    g = torch.Generator().manual_seed(5)
    lens = [5, 1, 8, 3, 4]
    masks = [(torch.rand(n, generator=g) > 0.35).double() for n in lens]
    masks[3] = torch.zeros(3, dtype=torch.float64)
    x = torch.randn(sum(lens), generator=g, dtype=torch.float64)
    total, off = 0.0, 0
    for n, m in zip(lens, masks):
        for t in range(n):
            total += x[off + t].item() * m[t].item()
        off += n
    want = total / len(lens)
    got = R.seq_mean_token_sum(lens, masks)(x)
    assert abs(got.item() - want) < 1e-12
    # hand-sized case: sums 1+2=3, 10 -> (3 + 10) / 2
    red = R.seq_mean_token_sum([3, 2], [torch.tensor([1.0, 1.0, 0.0]), torch.tensor([0.0, 1.0])])
    assert red(torch.tensor([1.0, 2.0, 100.0, -50.0, 10.0])).item() == 6.5
    # it differs from both reference reducers on ragged sequences (sample mean: 1.5 + 10; token sum: 13)
    masks2 = [torch.tensor([1.0, 1.0, 0.0]), torch.tensor([0.0, 1.0])]
    xs = torch.tensor([1.0, 2.0, 100.0, -50.0, 10.0])
    assert R.make_reducer([3, 2], masks2)(xs).item() == 11.5
    assert R.make_reducer([3, 2], masks2, per_token=True)(xs).item() == 13.0
    # gradient: m_t / B on every token
    xg = x.clone().requires_grad_()
    R.seq_mean_token_sum(lens, masks)(xg).backward()
    torch.testing.assert_close(xg.grad, torch.cat(masks) / len(lens), atol=0, rtol=0)
