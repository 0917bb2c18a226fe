"""Pins the distillation-loss composition of oracle.opd and the dispatch / scaling tail of oracle.policy (CPU).

Every expectation is worked out by scalar Python loops or by hand, never by calling the oracle's own helpers for
the quantity under test.  Reference: relax/utils/opd/opd_utils.py:1275-1455, relax/backends/megatron/loss.py:1247-1293
and :1565-1620, tests/backends/megatron/test_opd_loss_aggregation.py:36-49.
"""

import math

import pytest
import torch
import torch.nn.functional as F

from oracle import opd as D
from oracle import policy as P


# ---------------------------------------------------------------------------------------------------------------------
# scalar restatements used as the independent side
# ---------------------------------------------------------------------------------------------------------------------

def _tail(lps):
    """log(1 - sum exp lp) with the log-sum clamped to <= -1e-7 (opd_utils.py:1146-1149), in plain floats."""
    ls = min(math.log(sum(math.exp(v) for v in lps)), -1e-7)
    return math.log(-math.expm1(ls))


def _row_kl(s_row, t_row, alpha, norm_mode, n_valid=None):
    """One token's top-K divergence of the JSD family by a loop over the K entries (alpha 0 = reverse KL,
    1 = forward KL).  ``n_valid`` is the union path's per-row length: entries beyond it are padding and the tail
    bin is dropped with them."""
    k = len(s_row) if n_valid is None else n_valid
    s, t = list(s_row[:k]), list(t_row[:k])
    if norm_mode == "tail":
        s_all, t_all = s + [_tail(s)], t + [_tail(t)]
    elif norm_mode == "norm":
        zs, zt = math.log(sum(math.exp(v) for v in s)), math.log(sum(math.exp(v) for v in t))
        s_all, t_all = [v - zs for v in s], [v - zt for v in t]
    else:
        s_all, t_all = s, t
    if n_valid is not None:
        s_all, t_all = s_all[:k], t_all[:k]  # summed terms are cut back to the K columns: no tail bin
    if alpha == 0.0:
        return sum(math.exp(a) * (a - b) for a, b in zip(s_all, t_all))
    if alpha == 1.0:
        return sum(math.exp(b) * (b - a) for a, b in zip(s_all, t_all))
    out = 0.0
    for a, b in zip(s_all, t_all):
        mix = math.log((1 - alpha) * math.exp(a) + alpha * math.exp(b))
        out += (1 - alpha) * math.exp(a) * (a - mix) + alpha * math.exp(b) * (b - mix)
    return out


def _topk_rows(r, k, seed):
    """[r, k] log-probs of k tokens that hold ~80 % of the mass, so the tail bin is well away from its clamp."""
    g = torch.Generator().manual_seed(seed)
    p = torch.softmax(torch.randn(r, k + 3, generator=g, dtype=torch.float64), dim=-1)
    return p[:, :k].log()


def _batch(resp, masks):
    return {"response_lengths": resp, "loss_masks": [torch.tensor(m, dtype=torch.float64) for m in masks]}


# ---------------------------------------------------------------------------------------------------------------------
# reduce_token_mean (opd_utils.py:1355-1365)
# ---------------------------------------------------------------------------------------------------------------------

def test_reduce_token_mean_reference_literal(literals):
    fx = literals["opd_token_mean"]  # (1 + 1 + 10 + 0) / (1 + 1 + 1 + 0) = 12 / 3
    got = D.reduce_token_mean(torch.tensor(fx["values"]), fx["lengths"], [torch.tensor(m, dtype=torch.float32) for m in fx["masks"]])
    assert got.item() == fx["expected"] == 4.0


def test_reduce_token_mean_is_one_ratio_over_the_whole_micro_batch_not_a_mean_of_sample_means():
    vals = torch.tensor([2.0, 4.0, 6.0, 100.0, 8.0])
    masks = [torch.tensor([1.0, 1.0, 1.0]), torch.tensor([0.0, 1.0])]
    # token mean: (2 + 4 + 6 + 8) / 4 = 5; a mean of sample means would give (4 + 8) / 2 = 6
    assert D.reduce_token_mean(vals, [3, 2], masks).item() == 5.0
    # all masked: the denominator is clamped to one, the numerator is zero
    zero = [torch.zeros(3), torch.zeros(2)]
    assert D.reduce_token_mean(vals, [3, 2], zero).item() == 0.0
    # the clamp is on the whole count, not per sample: a fully masked sample adds nothing to the denominator
    assert D.reduce_token_mean(vals, [3, 2], [torch.tensor([1.0, 1.0, 0.0]), torch.zeros(2)]).item() == 3.0
    # gradient = mask / count
    v = vals.clone().requires_grad_()
    D.reduce_token_mean(v, [3, 2], masks).backward()
    assert v.grad.tolist() == [0.25, 0.25, 0.25, 0.0, 0.25]


# ---------------------------------------------------------------------------------------------------------------------
# policy_opd_loss (opd_utils.py:1368-1455)
# ---------------------------------------------------------------------------------------------------------------------

def _opd_args(**kw):
    base = dict(opd_loss_coef=0.7, opd_kl_type="reverse_kl", opd_jsd_alpha=0.5, opd_norm_mode="tail",
                opd_log_prob_min_clamp=None, opd_token_selection="sampled", opd_per_token_clip=None, opd_is_clip=None)
    base.update(kw)
    return P.make_args(**base)


def test_policy_opd_loss_none_returns():
    resp, masks = [2], [[1.0, 1.0]]
    lp, old = torch.tensor([-1.0, -2.0]), torch.tensor([-1.1, -2.2])
    b = _batch(resp, masks)
    b["teacher_log_probs"] = [torch.tensor([-1.5, -1.0])]
    # coefficient zero: nothing, whatever the batch holds
    assert D.policy_opd_loss(_opd_args(opd_loss_coef=0.0), b, lp, old, None) == (None, {})
    # sampled-token selection without the teacher's log-probs
    assert D.policy_opd_loss(_opd_args(), _batch(resp, masks), lp, old, None) == (None, {})
    nb = _batch(resp, masks)
    nb["teacher_log_probs"] = None
    assert D.policy_opd_loss(_opd_args(), nb, lp, old, None) == (None, {})
    # top-K selections need both arms, and an empty list counts as missing
    for sel in ("student_topk", "teacher_topk", "union"):
        a = _opd_args(opd_token_selection=sel)
        assert D.policy_opd_loss(a, _batch(resp, masks), lp, old, [_topk_rows(2, 3, 0)]) == (None, {})
        tb = _batch(resp, masks)
        tb["opd_topk_teacher_log_probs"] = [_topk_rows(2, 3, 1)]
        assert D.policy_opd_loss(a, tb, lp, old, None) == (None, {})
        assert D.policy_opd_loss(a, tb, lp, old, []) == (None, {})


def test_policy_opd_loss_sampled_token_clip_order_metrics_and_gradient_by_token_loops():
    resp, masks = [3, 2, 2], [[1.0, 0.0, 1.0], [1.0, 1.0], [0.0, 1.0]]
    lp0 = [-0.2, -3.0, -1.0, -0.5, -2.5, -0.1, -1.7]
    old0 = [-0.9, -3.1, -0.2, -0.5, -1.2, -2.0, -1.6]
    tea0 = [-1.4, -0.5, -1.3, -2.9, -0.4, -1.3, -0.2]
    tau, clip, coef = 0.9, 1.5, 0.7
    lp = torch.tensor(lp0, dtype=torch.float64, requires_grad=True)
    old = torch.tensor(old0, dtype=torch.float64)
    b = _batch(resp, masks)
    b["teacher_log_probs"] = list(torch.split(torch.tensor(tea0, dtype=torch.float64), resp))
    loss, met = D.policy_opd_loss(_opd_args(opd_loss_coef=coef, opd_per_token_clip=tau, opd_is_clip=clip), b, lp, old, None)
    loss.backward()

    flat_mask = [m for row in masks for m in row]
    num, over_tau, over_clip, grads = 0.0, 0, 0, []
    for a, o, t, m in zip(lp0, old0, tea0, flat_mask):
        kl = a - t  # reverse KL on the sampled token
        over_tau += kl > tau
        clipped = min(kl, tau)  # the per-token clip comes first ...
        ratio = math.exp(a - o)
        over_clip += ratio > clip
        w = min(ratio, clip)  # ... then the truncated importance ratio, a constant for the gradient
        num += clipped * w * m
        grads.append(coef * m * w * (1.0 if kl <= tau else 0.0) / sum(flat_mask))
    assert abs(loss.item() - coef * num / sum(flat_mask)) < 2e-7
    for g, want in zip(lp.grad.tolist(), grads):
        assert abs(g - want) < 2e-7
    # both fractions are plain means over every token, masked ones included (7 tokens, not 5)
    assert over_tau == 3 and over_clip == 2
    assert abs(met["opd_per_token_clip_frac"].item() - 3 / 7) < 1e-7
    assert abs(met["opd_is_clip_frac"].item() - 2 / 7) < 1e-7
    assert not met["opd_per_token_clip_frac"].requires_grad and not met["opd_is_clip_frac"].requires_grad
    assert list(met) == ["opd_per_token_clip_frac", "opd_is_clip_frac"]

    # one option at a time: only its own metric appears
    l1, m1 = D.policy_opd_loss(_opd_args(opd_per_token_clip=tau), b, lp.detach(), old, None)
    assert list(m1) == ["opd_per_token_clip_frac"]
    want = 0.7 * sum(min(a - t, tau) * m for a, t, m in zip(lp0, tea0, flat_mask)) / sum(flat_mask)
    assert abs(l1.item() - want) < 2e-7
    l2, m2 = D.policy_opd_loss(_opd_args(opd_is_clip=clip), b, lp.detach(), old, None)
    assert list(m2) == ["opd_is_clip_frac"]
    want = 0.7 * sum((a - t) * min(math.exp(a - o), clip) * m for a, o, t, m in zip(lp0, old0, tea0, flat_mask)) / sum(flat_mask)
    assert abs(l2.item() - want) < 2e-7
    l3, m3 = D.policy_opd_loss(_opd_args(), b, lp.detach(), old, None)
    assert m3 == {}
    assert abs(l3.item() - 0.7 * sum((a - t) * m for a, t, m in zip(lp0, tea0, flat_mask)) / sum(flat_mask)) < 2e-7


def test_policy_opd_loss_sampled_low_var_and_clamp():
    resp, masks = [2, 1], [[1.0, 1.0], [1.0]]
    lp0, tea0 = [-0.3, -30.0, -2.0], [-1.0, -2.0, -40.0]
    b = _batch(resp, masks)
    b["teacher_log_probs"] = list(torch.split(torch.tensor(tea0, dtype=torch.float64), resp))
    lp, old = torch.tensor(lp0, dtype=torch.float64), torch.zeros(3, dtype=torch.float64)
    loss, _ = D.policy_opd_loss(_opd_args(opd_kl_type="low_var_kl", opd_log_prob_min_clamp=-10.0, opd_loss_coef=1.0),
                                b, lp, old, None)
    want = 0.0
    for a, t in zip(lp0, tea0):
        d = max(a, -10.0) - max(t, -10.0)
        want += math.exp(-d) - 1 + d
    assert abs(loss.item() - want / 3) < 1e-6 * want


@pytest.mark.parametrize("sel", ["student_topk", "teacher_topk", "union"])
@pytest.mark.parametrize("kl_type,alpha", [("reverse_kl", 0.5), ("forward_kl", 0.5), ("jsd", 0.3)])
@pytest.mark.parametrize("norm_mode", ["tail", "norm", "trunc"])
def test_policy_opd_loss_topk_branches_by_row_loops(sel, kl_type, alpha, norm_mode):
    resp, k = [3, 2], 4
    masks = [[1.0, 1.0, 0.0], [1.0, 1.0]]
    student = [_topk_rows(3, k, 10), _topk_rows(2, k, 11)]
    teacher = [_topk_rows(3, k, 12), _topk_rows(2, k, 13)]
    ksz = [torch.tensor([4, 2, 3]), torch.tensor([1, 4])]
    lp0 = [-0.2, -1.0, -0.4, -0.9, -0.3]
    old0 = [-0.9, -0.8, -0.2, -0.5, -1.5]
    b = _batch(resp, masks)
    b["opd_topk_teacher_log_probs"] = teacher
    b["opd_topk_ksz"] = ksz  # read on the union path only
    tau, clip, coef = 0.05, 1.3, 0.4
    a = _opd_args(opd_loss_coef=coef, opd_token_selection=sel, opd_kl_type=kl_type, opd_jsd_alpha=alpha,
                  opd_norm_mode=norm_mode, opd_per_token_clip=tau, opd_is_clip=clip)
    loss, met = D.policy_opd_loss(a, b, torch.tensor(lp0, dtype=torch.float64), torch.tensor(old0, dtype=torch.float64), student)

    al = {"reverse_kl": 0.0, "forward_kl": 1.0}.get(kl_type, alpha)
    per = []
    for i in range(len(resp)):
        for r in range(resp[i]):
            nv = int(ksz[i][r]) if sel == "union" else None
            per.append(_row_kl(student[i][r].tolist(), teacher[i][r].tolist(), al, norm_mode, nv))
    flat_mask = [m for row in masks for m in row]
    num = sum(min(v, tau) * min(math.exp(x - o), clip) * m for v, x, o, m in zip(per, lp0, old0, flat_mask))
    assert abs(loss.item() - coef * num / sum(flat_mask)) < 2e-7
    assert abs(met["opd_per_token_clip_frac"].item() - sum(v > tau for v in per) / 5) < 1e-7
    assert abs(met["opd_is_clip_frac"].item() - sum(math.exp(x - o) > clip for x, o in zip(lp0, old0)) / 5) < 1e-7


def test_policy_opd_loss_union_mask_is_not_read_by_the_fixed_k_selections():
    resp, k = [2], 3
    student, teacher = [_topk_rows(2, k, 20)], [_topk_rows(2, k, 21)]
    b = _batch(resp, [[1.0, 1.0]])
    b["opd_topk_teacher_log_probs"] = teacher
    b["opd_topk_ksz"] = [torch.tensor([1, 2])]
    lp = torch.zeros(2, dtype=torch.float64)
    fixed, _ = D.policy_opd_loss(_opd_args(opd_token_selection="teacher_topk"), b, lp, lp, student)
    union, _ = D.policy_opd_loss(_opd_args(opd_token_selection="union"), b, lp, lp, student)
    want_fixed = sum(_row_kl(student[0][r].tolist(), teacher[0][r].tolist(), 0.0, "tail") for r in range(2)) / 2
    want_union = sum(_row_kl(student[0][r].tolist(), teacher[0][r].tolist(), 0.0, "tail", n) for r, n in enumerate([1, 2])) / 2
    assert abs(fixed.item() - 0.7 * want_fixed) < 2e-7 and abs(union.item() - 0.7 * want_union) < 2e-7
    assert abs(want_fixed - want_union) > 1e-3
    # a ``None`` length entry leaves that sample unmasked
    b["opd_topk_ksz"] = [None]
    again, _ = D.policy_opd_loss(_opd_args(opd_token_selection="union"), b, lp, lp, student)
    assert abs(again.item() - fixed.item()) < 2e-7


def test_policy_opd_loss_teacher_side_carries_no_gradient():
    resp = [2]
    student = [_topk_rows(2, 3, 30).requires_grad_()]
    teacher = [_topk_rows(2, 3, 31).requires_grad_()]
    b = _batch(resp, [[1.0, 1.0]])
    b["opd_topk_teacher_log_probs"] = teacher
    lp = torch.zeros(2, dtype=torch.float64)
    loss, _ = D.policy_opd_loss(_opd_args(opd_token_selection="student_topk"), b, lp, lp, student)
    loss.backward()
    assert teacher[0].grad is None and student[0].grad.abs().sum() > 0


# ---------------------------------------------------------------------------------------------------------------------
# apply_to_advantages (opd_utils.py:1275-1351)
# ---------------------------------------------------------------------------------------------------------------------

def test_apply_to_advantages_sampled_tokens_by_loops_and_no_clip_on_this_branch():
    a = P.make_args(opd_kl_coef=0.3, opd_kl_type="reverse_kl", opd_token_selection="sampled", opd_per_token_clip=0.01)
    stu = [torch.tensor([-0.5, -1.0, -4.0]), torch.tensor([-2.0])]
    tea = [torch.tensor([-0.7, -0.2, -0.1]), torch.tensor([-5.0])]
    adv0 = [[1.0, -1.0, 0.5], [2.0]]
    adv = [torch.tensor(x) for x in adv0]
    held = adv[0]
    D.apply_to_advantages(a, {"rollout_log_probs": stu, "teacher_log_probs": tea}, adv)
    for i in range(2):
        for j, base in enumerate(adv0[i]):
            # the per-token clip (0.01 here) is not applied to sampled tokens: -4.0 - -0.1 = -3.9, -0.5 + 0.7 = 0.2
            want = base - 0.3 * (stu[i][j].item() - tea[i][j].item())
            assert abs(adv[i][j].item() - want) < 1e-6
    assert adv[0] is not held and held.tolist() == adv0[0]  # list entries are replaced, not mutated

    # missing arm or zero coefficient: untouched
    same = [torch.tensor(x) for x in adv0]
    D.apply_to_advantages(a, {"rollout_log_probs": stu}, same)
    assert [t.tolist() for t in same] == adv0
    D.apply_to_advantages(P.make_args(opd_kl_coef=0.0, opd_kl_type="reverse_kl", opd_token_selection="sampled"),
                          {"rollout_log_probs": stu, "teacher_log_probs": tea}, same)
    assert [t.tolist() for t in same] == adv0


@pytest.mark.parametrize("sel", ["teacher_topk", "union"])
@pytest.mark.parametrize("kl_type,alpha,norm_mode", [("reverse_kl", 0.5, "tail"), ("jsd", 0.25, "norm"), ("forward_kl", 0.5, "trunc")])
def test_apply_to_advantages_topk_by_row_loops_with_clip_and_detach(sel, kl_type, alpha, norm_mode):
    k, resp = 4, [3, 2]
    stu = [_topk_rows(3, k, 40).requires_grad_(), _topk_rows(2, k, 41).requires_grad_()]
    tea = [_topk_rows(3, k, 42), _topk_rows(2, k, 43)]
    ksz = [torch.tensor([2, 4, 1]), torch.tensor([3, 3])]
    adv0 = [[0.5, -0.5, 1.5], [0.0, -2.0]]
    adv = [torch.tensor(x, dtype=torch.float64) for x in adv0]
    tau, coef = 0.04, 0.6
    a = P.make_args(opd_kl_coef=coef, opd_kl_type=kl_type, opd_jsd_alpha=alpha, opd_norm_mode=norm_mode,
                    opd_token_selection=sel, opd_per_token_clip=tau)
    D.apply_to_advantages(a, {"opd_topk_student_log_probs": stu, "opd_topk_teacher_log_probs": tea, "opd_topk_ksz": ksz}, adv)
    al = {"reverse_kl": 0.0, "forward_kl": 1.0}.get(kl_type, alpha)
    clipped_any = False
    for i in range(2):
        assert not adv[i].requires_grad  # the term is detached
        for r in range(resp[i]):
            nv = int(ksz[i][r]) if sel == "union" else None
            v = _row_kl(stu[i][r].tolist(), tea[i][r].tolist(), al, norm_mode, nv)
            clipped_any |= v > tau
            assert abs(adv[i][r].item() - (adv0[i][r] - coef * min(v, tau))) < 2e-7
    assert clipped_any

    # no clip configured: the raw term
    adv = [torch.tensor(x, dtype=torch.float64) for x in adv0]
    a.opd_per_token_clip = None
    D.apply_to_advantages(a, {"opd_topk_student_log_probs": stu, "opd_topk_teacher_log_probs": tea, "opd_topk_ksz": ksz}, adv)
    nv = int(ksz[0][0]) if sel == "union" else None
    v = _row_kl(stu[0][0].tolist(), tea[0][0].tolist(), al, norm_mode, nv)
    assert abs(adv[0][0].item() - (adv0[0][0] - coef * v)) < 2e-7

    # a missing top-K arm leaves the advantages as they were
    adv = [torch.tensor(x, dtype=torch.float64) for x in adv0]
    D.apply_to_advantages(a, {"opd_topk_teacher_log_probs": tea}, adv)
    assert [t.tolist() for t in adv] == adv0


# ---------------------------------------------------------------------------------------------------------------------
# sft_loss_function (loss.py:1247-1293) and the dispatch / scaling tail of loss_function (loss.py:1515-1620)
# ---------------------------------------------------------------------------------------------------------------------

def _sft_case():
    torch.manual_seed(11)
    tot, v = [4, 3], 9
    toks = [torch.randint(0, v, (n,)) for n in tot]
    logits = torch.randn(1, sum(tot), v, dtype=torch.float64)
    masks = [torch.tensor([1.0, 1.0, 0.0, 1.0], dtype=torch.float64), torch.tensor([1.0, 1.0, 1.0], dtype=torch.float64)]
    batch = dict(unconcat_tokens=toks, total_lengths=tot, response_lengths=list(tot), loss_masks=masks)
    return tot, v, toks, logits, masks, batch


def _sft_by_cross_entropy(tot, toks, logits, masks, per_token):
    """Row t of a sample scores token t + 1; the last row's target is the pad id 0 (sft_utils.py:23-40).  Library
    cross-entropy per row, then the masked reduction written as a loop."""
    total, off = 0.0, 0
    for n, tk, m in zip(tot, toks, masks):
        tgt = torch.cat([tk[1:], torch.zeros(1, dtype=tk.dtype)])
        ce = F.cross_entropy(logits[0, off:off + n], tgt, reduction="none")
        s = sum(ce[j].item() * m[j].item() for j in range(n))
        total += s if per_token else s / max(m.sum().item(), 1.0)
        off += n
    return total


@pytest.mark.parametrize("per_token", [False, True])
def test_sft_loss_function_against_library_cross_entropy_on_shifted_targets(per_token):
    from oracle import reducers as R

    tot, v, toks, logits, masks, batch = _sft_case()
    x = logits.clone().requires_grad_()
    loss, log = P.sft_loss_function(P.make_args(), batch, x, R.make_reducer(tot, masks, per_token))
    want = _sft_by_cross_entropy(tot, toks, logits, masks, per_token)
    assert abs(loss.item() - want) < 1e-6
    assert list(log) == ["loss"] and abs(log["loss"].item() - want) < 1e-6 and not log["loss"].requires_grad
    loss.backward()
    # masked row and rows outside nothing: row 2 of sample 0 is masked -> zero gradient there
    assert x.grad[0, 2].abs().sum().item() == 0.0 and x.grad[0, 0].abs().sum().item() > 0


def test_sft_loss_function_empty_batch_keeps_the_graph():
    from oracle import reducers as R

    logits = torch.zeros(1, 0, 5, requires_grad=True)
    batch = dict(unconcat_tokens=[torch.zeros(0, dtype=torch.long)], total_lengths=[0], response_lengths=[0],
                 loss_masks=[torch.zeros(0)])
    loss, _ = P.sft_loss_function(P.make_args(), batch, logits, R.make_reducer([0], batch["loss_masks"], False))
    assert float(loss) == 0.0 and loss.requires_grad


def test_loss_function_dispatches_on_loss_type():
    tot, v, toks, logits, masks, batch = _sft_case()
    a = P.make_args(loss_type="sft", global_batch_size=2)
    loss, norm, log = P.loss_function(a, batch, 1, logits)
    assert log["keys"] == ["loss"]
    assert abs(loss.item() - _sft_by_cross_entropy(tot, toks, logits, masks, False) * 1 / 2) < 1e-6
    with pytest.raises(KeyError):
        P.loss_function(P.make_args(loss_type="no_such_loss"), batch, 1, logits)
    # an explicit callable wins over loss_type
    called = {}

    def custom(args, b, lg, red):
        called["yes"] = True
        return torch.tensor(3.0), {"loss": torch.tensor(3.0), "extra": 7.0}

    loss, norm, log = P.loss_function(a, batch, 4, logits, dp_world=2, func=custom)
    assert called and loss.item() == 3.0 * 4 / 2 * 2 and log["keys"] == ["loss", "extra"]
    assert log["values"].tolist() == [0.0, 3.0, 7.0]  # python scalars in the log become tensors


def _three_token_case():
    """Two samples, three response tokens, V = 2 with logits chosen so that every log-prob is log(1/2): with
    old = log(1/2) the ratio is one, nothing clips and the policy loss per token is -A."""
    tot, resp = [3, 2], [2, 1]
    logits = torch.zeros(1, 5, 2, dtype=torch.float64)
    toks = [torch.tensor([0, 1, 0]), torch.tensor([1, 1])]
    half = math.log(0.5)
    batch = dict(
        unconcat_tokens=toks, total_lengths=tot, response_lengths=resp,
        loss_masks=[torch.tensor([1.0, 1.0], dtype=torch.float64), torch.tensor([1.0], dtype=torch.float64)],
        advantages=[torch.tensor([1.0, 3.0], dtype=torch.float64), torch.tensor([-4.0], dtype=torch.float64)],
        log_probs=[torch.full((2,), half, dtype=torch.float64), torch.full((1,), half, dtype=torch.float64)],
    )
    return batch, logits


def test_loss_function_sample_mean_scale_by_hand():
    batch, logits = _three_token_case()
    # sum of sample means of -A: -(1 + 3) / 2 + 4 / 1 = 2
    a = P.make_args(global_batch_size=8)
    loss, norm, log = P.loss_function(a, batch, 4, logits, dp_world=2)
    assert abs(loss.item() - 2.0 * 4 / 8 * 2) < 1e-6
    assert norm.item() == 1 and log["values"][0].item() == 0
    assert abs(log["values"][log["keys"].index("pg_loss") + 1].item() - 2.0) < 1e-6  # metrics are not rescaled
    # a batch-supplied global batch size replaces the configured one
    batch["dynamic_global_batch_size"] = 16
    loss, _, _ = P.loss_function(a, batch, 4, logits, dp_world=2)
    assert abs(loss.item() - 2.0 * 4 / 16 * 2) < 1e-6
    # an explicit scale replaces the whole factor (micro-batch count, batch size and world size all unused)
    batch["__loss_scale__"] = 0.125
    loss, norm, log = P.loss_function(a, batch, 4, logits, dp_world=2)
    assert abs(loss.item() - 2.0 * 0.125) < 1e-6 and norm.item() == 1
    # per-token mode ignores every one of them: token sum of -A = -1 - 3 + 4 = 0 -> use entropy to get a non-zero
    a = P.make_args(global_batch_size=8, calculate_per_token_loss=True, entropy_coef=-1.0)
    loss, norm, log = P.loss_function(a, batch, 4, logits, dp_world=2)
    assert abs(loss.item() - 3 * math.log(2.0)) < 1e-6  # pg 0 + 1.0 * sum of three entropies ln 2
    assert norm.item() == 3 and log["values"][0].item() == 3


@pytest.mark.parametrize("per_token", [False, True])
def test_loss_function_dummy_micro_batch_by_hand(per_token):
    batch, logits = _three_token_case()
    batch["__is_dummy__"] = True
    batch["__loss_scale__"] = 5.0  # ignored on a dummy micro-batch
    x = logits.clone().requires_grad_()
    a = P.make_args(global_batch_size=8, calculate_per_token_loss=per_token)
    loss, norm, log = P.loss_function(a, batch, 4, x, dp_world=2)
    assert loss.item() == 0.0 and loss.requires_grad  # zero, but still attached to the graph
    loss.backward()
    assert x.grad.abs().sum().item() == 0.0
    assert log["keys"][:5] == ["loss", "pg_loss", "entropy_loss", "pg_clipfrac", "ppo_kl"]
    assert log["values"].abs().sum().item() == 0.0 and log["values"].numel() == len(log["keys"]) + 1
    # the normaliser: zero tokens in per-token mode (so the step's token total skips this micro-batch), one otherwise
    assert norm.item() == (0 if per_token else 1)

    batch["__is_dummy__"] = False
    loss, norm, log = P.loss_function(a, batch, 4, logits, dp_world=2)
    assert norm.item() == (3 if per_token else 1) and log["values"].abs().sum().item() > 0
