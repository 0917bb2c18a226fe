"""Oracle: per-token policy losses and KL estimators (autograd-differentiable).

Test infrastructure only.  All functions are plain torch ops so autograd gives
the same gradient conventions as the reference (ties of ``torch.maximum`` split
half/half, ``clamp`` passes gradient at its closed bounds).
"""

from __future__ import annotations

import torch


def approx_kl(lp: torch.Tensor, base: torch.Tensor, kind: str, importance_ratio: torch.Tensor | None = None):
    """relax/utils/training/ppo_utils.py:100-139 (k1 / k2 / k3 / low_var_kl)."""
    d = lp.float() - base.float()
    if kind == "k1":
        out = d
    elif kind == "k2":
        out = d**2 / 2.0
    elif kind in ("k3", "low_var_kl"):
        nd = -d
        out = nd.exp() - 1 - nd
    else:
        raise ValueError(f"Unknown kl_loss_type: {kind}")
    if importance_ratio is not None:
        out = importance_ratio * out
    if kind == "low_var_kl":
        out = torch.clamp(out, min=-10, max=10)
    return out


def policy_clip(ppo_kl, adv, eps_lo: float, eps_hi: float, eps_c: float | None = None):
    """PPO clipped surrogate, ppo_utils.py:372-396.  Returns (loss [N], clipfrac [N])."""
    r = (-ppo_kl).exp()
    a = -r * adv
    b = -r.clamp(1 - eps_lo, 1 + eps_hi) * adv
    loss = torch.maximum(a, b)
    clipfrac = torch.gt(b, a).float()
    if eps_c is not None:
        assert eps_c > 1.0
        c = -eps_c * adv
        loss = torch.where(adv < 0, torch.min(c, loss), loss)
    return loss, clipfrac


def gspo_seq_kl(lps: list, olds: list, masks: list) -> torch.Tensor:
    """Sequence-level KL broadcast to tokens, ppo_utils.py:183-209.

    k_i = sum((old-lp)*m) / clamp_min(sum m, 1), expanded over sample i's tokens.
    """
    out = []
    for lp, old, m in zip(lps, olds, masks, strict=False):
        k = ((old - lp) * m).sum() / torch.clamp_min(m.sum(), 1)
        out.append(k.expand_as(lp))
    return torch.cat(out, dim=0)


def cispo(lp, ppo_kl, adv, eps_lo: float, eps_hi: float):
    """CISPO, ppo_utils.py:273-333: loss = -sg(coef)*sg(A)*lp; coef clipped by sign of A (A>=0 -> upper cap)."""
    r = torch.exp(-ppo_kl)
    hi, lo = 1.0 + eps_hi, 1.0 - eps_lo
    coef = torch.where(adv >= 0, torch.clamp(r, max=hi), torch.clamp(r, min=lo))
    loss = -(coef.detach() * adv.detach() * lp)
    clipfrac = ((adv >= 0) & (r > hi)).float() + ((adv < 0) & (r < lo)).float()
    return loss, clipfrac


def rloo_loss(lp, adv):
    """Unclipped REINFORCE term, ppo_utils.py:336-369."""
    return -(adv.detach() * lp), torch.zeros_like(lp)


def sapo(ppo_kl, adv, tau_pos: float, tau_neg: float):
    """Soft gate (4/tau)*sigmoid(tau*(r-1)), ppo_utils.py:212-270."""
    r = torch.exp(-ppo_kl)
    tau = torch.where(adv > 0, torch.full_like(adv, tau_pos), torch.full_like(adv, tau_neg))
    s = torch.sigmoid(tau * (r - 1.0))
    loss = -((4.0 / tau) * s * adv)
    clipfrac = ((4.0 * s * (1.0 - s)) < 0.9).float()
    return loss, clipfrac


def opsm_mask(delta: float, lps: list, olds: list, advs: list, masks: list):
    """Off-policy sequence mask, ppo_utils.py:142-180.  Returns (mask [N], clipfrac scalar)."""
    parts = []
    frac = torch.tensor(0.0)
    for lp, old, a, m in zip(lps, olds, advs, masks, strict=False):
        seq_kl = ((old - lp) * m).sum() / torch.clamp_min(m.sum(), 1)
        drop = ((a < 0) & (seq_kl > delta)).float()
        frac = frac + drop.sum() / torch.clamp_min(m.sum(), 1)
        parts.append(1 - drop)
    return torch.cat(parts, dim=0), frac


def vanilla_tis(pg_loss, train_lp, rollout_lp, clip_low: float, clip_high: float):
    """Truncated importance sampling weights + metrics, relax/backends/megatron/loss.py:741-769."""
    log_ratio = train_lp - rollout_lp
    tis = torch.exp(log_ratio)
    w = torch.clamp(tis, min=clip_low, max=clip_high)
    metrics = {
        "tis": tis.detach().clone(),
        "tis_clipfrac": (w != tis).float(),
        "tis_abs": (tis - 1).abs().detach(),
        "mismatch_kl": (-log_ratio).detach(),
        "mismatch_k3_kl": (tis - log_ratio - 1).detach(),
    }
    return pg_loss * w, metrics


def icepop(pg_loss, train_lp, rollout_lp, clip_low: float, clip_high: float):
    """relax/backends/megatron/loss.py:772-801: importance ratios outside [clip_low, clip_high] get weight zero."""
    log_ratio = train_lp - rollout_lp
    tis = torch.exp(log_ratio)
    w = torch.where((tis >= clip_low) & (tis <= clip_high), tis, torch.zeros_like(tis))
    metrics = {
        "tis": tis.detach().clone(),
        "tis_clipfrac": (w != tis).float(),
        "tis_abs": (tis - 1).abs().detach(),
        "mismatch_kl": (-log_ratio).detach(),
        "mismatch_k3_kl": (tis - log_ratio - 1).detach(),
    }
    return pg_loss * w, metrics


# ---- M2PO: second-moment trust region (ppo_utils.py:404-460)


def m2po_delta_sq(ppo_kl, adv):
    """Squared log-ratio of the tokens a clip would act on (ppo_utils.py:426-430): positive advantage with a ratio
    above one, negative advantage with a ratio below one (margins of 1e-12)."""
    ratio = (-ppo_kl).exp()
    harmful = ((adv > 1e-12) & (ratio > 1.0 + 1e-12)) | ((adv < -1e-12) & (ratio < 1.0 - 1e-12))
    return ppo_kl[harmful].pow(2)


def m2po_solve_tau(sorted_delta2, target_sum: float):
    """(tau, second moment after capping) for ascending ``sorted_delta2`` (ppo_utils.py:404-423): the cap is the
    largest data value whose capped sum stays below ``target_sum``; the scan runs in Python floats over the fp32
    values and their fp32 running sum, like the reference's."""
    n = sorted_delta2.numel()
    total = float(sorted_delta2.sum().item())
    if target_sum >= total - 1e-12:
        return 100000.0, total / n
    if target_sum <= 1e-12:
        return 0.0, 0.0
    values = [float(x) for x in sorted_delta2.tolist()]
    running = [float(x) for x in torch.cumsum(sorted_delta2, dim=0).tolist()]
    for k in range(n):
        above = n - k - 1
        if (values[k] - 1e-12) * above + running[k] >= target_sum - 1e-12:
            if k == 0:
                return 0.0, running[-1] / n
            after = (values[k - 1] * (above + 1) + running[k - 1]) / n
            return max(values[k - 1] - 1e-12, 0.0) ** 0.5, after
    return 100000.0, total / n


def m2po_clip_bounds(ppo_kl, adv, kl2_budget: float):
    """(ratio lower bound, ratio upper bound, M2 before, M2 after) -- kpo_clip_harmful_tokens, ppo_utils.py:433-445."""
    import math

    d2 = m2po_delta_sq(ppo_kl, adv)
    n = d2.numel()
    if n == 0:
        return 0.0, 100000.0, 0.0, 0.0
    m2_now = float(d2.sum().detach().item() / n)
    if m2_now <= kl2_budget + 1e-12:
        return 0.0, 100000.0, m2_now, m2_now
    tau, m2_after = m2po_solve_tau(torch.sort(d2)[0], kl2_budget * float(n))
    return math.exp(-tau), math.exp(tau), m2_now, m2_after


def m2po(ppo_kl, adv, kl2_budget: float, miniclip_low: float = 0.3, miniclip_high: float = 0.5):
    """compute_m2po_loss, ppo_utils.py:448-463: PPO-clip with margins max(adaptive, floor).  Returns
    (pg_losses, clipfrac, M2 before, M2 after, eps_low, eps_high)."""
    lo, hi, m2_now, m2_after = m2po_clip_bounds(ppo_kl, adv, kl2_budget)
    eps_low = max(1.0 - lo, miniclip_low)
    eps_high = max(hi - 1.0, miniclip_high)
    ratio = (-ppo_kl).exp()
    l1 = -adv * ratio
    l2 = -adv * ratio.clamp(1.0 - eps_low, 1.0 + eps_high)
    return torch.maximum(l1, l2), (l2 > l1).float(), m2_now, m2_after, eps_low, eps_high
