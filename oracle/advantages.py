"""Oracle: group-normalised rewards, broadcast returns, advantage whitening.

Test infrastructure only.
"""

from __future__ import annotations

import torch

GROUP_NORM_ESTIMATORS = ("grpo", "gspo", "sapo", "cispo", "reinforce_plus_plus_baseline", "rloo")
STD_NORM_ESTIMATORS = ("grpo", "gspo", "sapo", "cispo")


def rloo_leave_one_out(group_rewards: torch.Tensor) -> torch.Tensor:
    """relax/utils/training/ppo_utils.py:664-705: G/(G-1) * (r - mean r), with the reference's input checks."""
    if group_rewards.dim() != 1:
        raise ValueError(f"expects a 1-D tensor (one group), got shape {tuple(group_rewards.shape)}")
    g = group_rewards.shape[0]
    if g < 2:
        raise ValueError(f"RLOO requires n_samples_per_prompt >= 2 (group size {g})")
    if not torch.isfinite(group_rewards).all():
        raise ValueError(f"RLOO group contains non-finite reward(s): {group_rewards}")
    return (g / (g - 1)) * (group_rewards - group_rewards.mean())


def group_normalise(raw, group_index, n_samples_per_prompt: int, estimator: str = "grpo", std_norm: bool = True):
    """relax/utils/utils.py:199-238: fp32 group centring, optional /(std_ddof1 + 1e-6), or RLOO.

    raw: list[float]; group_index: list[int] (interleaving allowed).  Returns fp32 tensor [B] in input order.
    """
    r = torch.tensor(raw, dtype=torch.float)
    where: dict[int, list[int]] = {}
    for pos, g in enumerate(group_index):
        if g is None:
            raise ValueError("Sample.group_index is required for group reward normalization.")
        where.setdefault(g, []).append(pos)
    out = torch.empty_like(r)
    for g, pos in where.items():
        if len(pos) != n_samples_per_prompt:
            raise ValueError(f"Reward group {g} has {len(pos)} samples, expected {n_samples_per_prompt}.")
        gr = r[pos]
        if estimator == "rloo":
            gr = rloo_leave_one_out(gr)
        else:
            gr = gr - gr.mean()
            if estimator in STD_NORM_ESTIMATORS and std_norm:
                gr = gr / (gr.std() + 1e-6)
        out[pos] = gr
    return out


def grpo_returns(rewards: torch.Tensor, like: list) -> list:
    """ppo_utils.py:654-661: ones_like(kl_i) * rewards[i]."""
    return [torch.ones_like(k) * rewards[i] for i, k in enumerate(like)]


def masked_whiten(values: torch.Tensor, mask: torch.Tensor, shift_mean: bool = True, epsilon: float = 1e-8):
    """relax/utils/distributed_utils.py:98-158 on a single rank (the all-reduce is the identity).

    Stats are packed into an fp32 vector (:128-132); Bessel correction applies when the masked count >= 2;
    values outside the mask are transformed too (not zeroed).
    """
    stats = torch.tensor(
        [(values * mask).sum(), ((values**2) * mask).sum(), mask.sum()], dtype=torch.float32, device=values.device
    )
    s1, s2, cnt = stats
    if cnt.item() == 0:
        raise ValueError("The global mask sum across all participating GPUs is zero.")
    mean = s1 / cnt
    var = s2 / cnt - mean**2
    if cnt.item() >= 2:
        var = var * (cnt / (cnt - 1))
    out = (values - mean) * torch.rsqrt(var + epsilon)
    if not shift_mean:
        out = out + mean
    return out


def advantages_and_returns(rewards, shapes_like: list, masks: list | None = None, normalize: bool = False):
    """GRPO-family branch of relax/backends/megatron/loss.py:574-591,651-738.

    rewards: list[float] already group-normalised; shapes_like: per-sample [R_i] tensors giving shape/dtype
    (the KL values never enter the GRPO-family advantage).  Returns (advantages list, returns list).
    """
    kl = [torch.zeros_like(x, dtype=torch.float32) for x in shapes_like]
    rw = torch.tensor(rewards, dtype=torch.float32)
    returns = grpo_returns(rw, kl)
    adv = list(returns)
    if normalize:
        flat = masked_whiten(torch.cat(adv), torch.cat(masks))
        adv = list(torch.split(flat, [a.size(0) for a in adv]))
    return adv, returns


def reinforce_pp_returns(rewards, kl: list, loss_masks: list, kl_coef: float, gamma: float) -> list:
    """relax/utils/training/ppo_utils.py:708-804 on one context-parallel rank: token rewards ``-kl_coef * kl`` on
    valid tokens (selected, not multiplied, so masked NaN cannot leak), the sequence reward on the last valid token,
    ``G_t = r_t + gamma * G_{t+1}`` evaluated right to left, zero outside the mask and for fully masked sequences."""
    if not (len(kl) == len(loss_masks) == len(rewards)):
        raise ValueError("rewards, kl, loss_masks must contain the same number of responses.")
    out = []
    for i, (k, m) in enumerate(zip(kl, loss_masks)):
        if k.shape != m.shape:
            raise ValueError(f"KL and loss mask for response {i} must have the same shape")
        valid = m != 0
        if not bool(valid.any()):
            out.append(torch.zeros_like(k))
            continue
        r = -kl_coef * torch.where(valid, k, torch.zeros_like(k))
        r[int(valid.nonzero()[-1])] += rewards[i]
        g = torch.zeros_like(r)
        run = 0.0
        for t in range(r.numel() - 1, -1, -1):
            run = r[t] + gamma * run
            g[t] = run
        out.append(torch.where(valid, g, torch.zeros_like(g)))
    return out


def reinforce_pp_baseline_advantages(rewards, like: list, loss_masks: list) -> list:
    """ppo_utils.py:807-843: the (already group-centred) reward on every valid token, zero elsewhere."""
    return [torch.where(m != 0, torch.ones_like(k) * r, torch.zeros_like(k)) for k, r, m in zip(like, rewards, loss_masks)]


def gae(values: torch.Tensor, rewards: torch.Tensor, gamma: float, lambd: float):
    """ppo_utils.py:846-906 / vanilla_gae :1026-1047 for one response: ``delta_t = r_t + gamma V_{t+1} - V_t``,
    ``A_t = delta_t + gamma*lambd*A_{t+1}`` right to left (V past the end = 0), returns = A + V."""
    n = values.numel()
    adv = torch.zeros_like(values)
    last = torch.zeros((), dtype=values.dtype)
    for t in range(n - 1, -1, -1):
        nxt = values[t + 1] if t < n - 1 else 0.0
        delta = rewards[t] + gamma * nxt - values[t]
        last = delta + gamma * lambd * last
        adv[t] = last
    return adv, adv + values


def masked_normalize(values: torch.Tensor, mask: torch.Tensor, variance_floor: float = 1e-8):
    """relax/utils/distributed_utils.py:161-213 on one rank: population moments (ddof = 0) over mask != 0, output
    zero outside the mask.  Returns (normalized, mean, variance, count)."""
    work = torch.float64 if values.dtype == torch.float64 else torch.float32
    v = values.to(work)
    valid = mask != 0
    count = valid.to(work).sum().clamp_min(1)
    mean = torch.where(valid, v, torch.zeros_like(v)).sum() / count
    centred = torch.where(valid, v - mean, torch.zeros_like(v))
    var = (centred.square().sum() / count).clamp_min(0.0)
    out = torch.where(valid, (v - mean) * torch.rsqrt(var.clamp_min(variance_floor)), torch.zeros_like(v))
    return out, mean, var, valid.to(work).sum()
