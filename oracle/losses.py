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
