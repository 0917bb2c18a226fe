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
