"""Drop-in counterparts of the hot-path functions of ``relax/utils/training/ppo_utils.py`` (same names, argument
meaning and error behaviour), running on the gfx950 kernels.

Reference lines (paths relative to the reference checkout):
  calculate_log_probs_and_entropy      relax/utils/training/ppo_utils.py:1192-1243 (+ :480-629)
  compute_approx_kl                    :100-139
  compute_policy_loss                  :372-396
  compute_gspo_kl                      :183-209
  compute_cispo_loss                   :273-333
  compute_rloo_loss                    :336-369
  compute_sapo_loss                    :212-270
  compute_opsm_mask                    :142-180
  get_grpo_returns                     :654-661
  compute_rloo_leave_one_out_rewards   :664-705
"""

from __future__ import annotations

import torch

from . import ops


def _single_rank(tp_group) -> None:
    if tp_group is not None and hasattr(tp_group, "size") and tp_group.size() > 1:
        raise NotImplementedError("relax_amd runs the full vocabulary on one GPU; vocab-parallel groups are not supported")


def calculate_log_probs_and_entropy(
    logits,
    tokens,
    tp_group=None,
    with_entropy: bool = False,
    chunk_size: int = -1,
    log_prob_keep_mask=None,
    with_entropy_grad: bool = True,
):
    """Returns ``(log_prob [N,1] fp32, entropy [N] fp32 | None)``.

    ``chunk_size`` is accepted for signature compatibility and has no effect: the kernel streams each row once and
    holds no [chunk, V] temporaries, so there is nothing to chunk.  Results do not depend on it.
    """
    _single_rank(tp_group)
    if logits.size(0) == 0:
        return logits.new_zeros((0,)), (logits.new_zeros((0,)) if with_entropy else None)
    if log_prob_keep_mask is not None:
        # the log-prob's softmax only sees the kept vocabulary entries (and the target); the entropy sees the row
        if log_prob_keep_mask.shape != logits.shape:
            raise ValueError(f"log_prob_keep_mask {tuple(log_prob_keep_mask.shape)} must match the logits "
                             f"{tuple(logits.shape)}")
        keep = log_prob_keep_mask.to(device=logits.device, dtype=torch.uint8).contiguous()
        lp, ent = ops.LogProbEntropyMasked.apply(logits, tokens, keep, 1.0, bool(with_entropy),
                                                 bool(with_entropy_grad))
        return lp.unsqueeze(-1), (ent if with_entropy else None)
    lp, ent = ops.LogProbEntropy.apply(logits, tokens, None, None, 1.0, bool(with_entropy), bool(with_entropy_grad))
    return lp.unsqueeze(-1), (ent if with_entropy else None)


# ---------------------------------------------------------------------------------------------- per-token losses


def _cu_single(n: int, device) -> torch.Tensor:
    return torch.tensor([0, n], dtype=torch.int64, device=device)


class _TokenLoss(torch.autograd.Function):
    """Per-token (loss, clipfrac) of one policy-loss flavour; differentiable w.r.t. ``lp`` and/or ``ppo_kl``.

    The kernel sees log_prob = lp (or -ppo_kl with old = 0 when only ``ppo_kl`` is given) over a single pseudo-sample
    with unit mask and unit denominators, so its gradient coefficient is exactly d loss_t / d lp_t.
    """

    @staticmethod
    def forward(ctx, kind, lp, ppo_kl, adv, eps_lo, eps_hi, eps_c, tau_pos, tau_neg):
        shape = adv.shape
        n = adv.numel()
        dev = adv.device
        in_dtype = (lp if lp is not None else ppo_kl).dtype
        if lp is not None and ppo_kl is not None:
            # CISPO: loss uses lp directly and the (detached) ratio exp(-ppo_kl): old = lp + ppo_kl
            cur = lp.reshape(-1).float()
            old = cur + ppo_kl.reshape(-1).float()
        elif lp is not None:
            cur, old = lp.reshape(-1).float(), None
        else:
            cur = (-ppo_kl.reshape(-1)).float()
            old = torch.zeros_like(cur)
        out = ops.policy_loss(
            log_prob=cur, old_log_prob=old, advantages=adv.reshape(-1), loss_mask=torch.ones(n, device=dev),
            cu_resp=_cu_single(n, dev), loss_kind=kind, eps_clip=eps_lo, eps_clip_high=eps_hi, eps_clip_c=eps_c,
            tau_pos=tau_pos, tau_neg=tau_neg, per_token_outputs=True,
        )
        ctx.save_for_backward(out["coef_log_prob"])
        ctx.lp_given, ctx.kl_given, ctx.shape, ctx.in_dtype = lp is not None, ppo_kl is not None, shape, in_dtype
        clip = out["clipfrac_tok"].reshape(shape)
        ctx.mark_non_differentiable(clip)
        return out["pg_loss_tok"].reshape(shape).to(in_dtype), clip

    @staticmethod
    def backward(ctx, g_loss, _g_clip):
        (coef,) = ctx.saved_tensors
        g = (g_loss.reshape(-1).float() * coef).reshape(ctx.shape).to(ctx.in_dtype)
        g_lp = g if ctx.lp_given else None
        # with only ppo_kl given the kernel differentiated w.r.t. lp = -ppo_kl
        g_kl = (-g) if (ctx.kl_given and not ctx.lp_given) else None
        return None, g_lp, g_kl, None, None, None, None, None, None


def compute_policy_loss(ppo_kl, advantages, eps_clip, eps_clip_high, eps_clip_c=None):
    if eps_clip_c is not None:
        assert eps_clip_c > 1.0, (
            f"The lower bound of the clip_ratio_c for dual-clip PPO should be greater than 1.0, but get the value: {eps_clip_c}."
        )
    return _TokenLoss.apply("ppo", None, ppo_kl, advantages, eps_clip, eps_clip_high, eps_clip_c, 1.0, 1.05)


def compute_cispo_loss(log_probs, ppo_kl, advantages, eps_clip, eps_clip_high):
    return _TokenLoss.apply("cispo", log_probs, ppo_kl.detach(), advantages, eps_clip, eps_clip_high, None, 1.0, 1.05)


def compute_rloo_loss(log_probs, advantages):
    return _TokenLoss.apply("rloo", log_probs, None, advantages, 0.2, 0.2, None, 1.0, 1.05)


def compute_sapo_loss(ppo_kl, advantages, tau_pos, tau_neg):
    return _TokenLoss.apply("sapo", None, ppo_kl, advantages, 0.2, 0.2, None, tau_pos, tau_neg)


class _ApproxKL(torch.autograd.Function):
    @staticmethod
    def forward(ctx, lp, base, kind):
        n, dev = lp.numel(), lp.device
        out = ops.policy_loss(
            log_prob=lp.reshape(-1), ref_log_prob=base.reshape(-1), advantages=torch.zeros(n, device=dev),
            loss_mask=torch.ones(n, device=dev), cu_resp=_cu_single(n, dev), loss_kind="rloo", kl_kind=kind,
            kl_coef=1.0, per_token_outputs=True,
        )
        ctx.save_for_backward(out["coef_log_prob"])
        ctx.shape = lp.shape
        return out["kl_tok"].reshape(lp.shape)

    @staticmethod
    def backward(ctx, g):
        (coef,) = ctx.saved_tensors
        gl = (g.reshape(-1) * coef).reshape(ctx.shape)
        return gl, -gl, None


def compute_approx_kl(log_probs, log_probs_base, kl_loss_type: str, importance_ratio=None):
    if kl_loss_type not in ("k1", "k2", "k3", "low_var_kl"):
        raise ValueError(f"Unknown kl_loss_type: {kl_loss_type}")
    if importance_ratio is None:
        return _ApproxKL.apply(log_probs, log_probs_base, kl_loss_type)
    # an arbitrary caller-supplied ratio tensor: estimator from the kernel, ratio and clamp composed on [N] vectors
    base_kind = "k3" if kl_loss_type == "low_var_kl" else kl_loss_type
    kl = importance_ratio * _ApproxKL.apply(log_probs, log_probs_base, base_kind)
    if kl_loss_type == "low_var_kl":
        kl = torch.clamp(kl, min=-10, max=10)
    return kl


class _SeqKL(torch.autograd.Function):
    """k_i = sum((old - lp) * m) / clamp_min(sum m, 1) per sample, expanded to the sample's tokens."""

    @staticmethod
    def forward(ctx, lp, old, mask, cu_resp, n_tokens):
        num = ops.segment_sum(mask, cu_resp, values=(old - lp))
        den = ops.segment_sum(mask, cu_resp).clamp_min(1.0)
        inv = (1.0 / den).float()
        ctx.save_for_backward(mask, cu_resp, inv)
        ctx.n = n_tokens
        return ops.broadcast_per_sample((num / den).float(), cu_resp, n_tokens)

    @staticmethod
    def backward(ctx, g):
        mask, cu_resp, inv = ctx.saved_tensors
        gsum = ops.segment_sum(torch.ones_like(g), cu_resp, values=g).float()
        per = ops.broadcast_per_sample(gsum * inv, cu_resp, ctx.n) * mask.float()
        return -per, per, None, None, None


def compute_gspo_kl(full_log_probs, full_old_log_probs, local_log_probs, loss_masks):
    lens = [int(x.numel()) for x in local_log_probs]
    dev = full_log_probs[0].device
    cu = torch.tensor([0] + lens, dtype=torch.int64).cumsum(0).to(dev)
    return _SeqKL.apply(torch.cat(full_log_probs).float(), torch.cat(full_old_log_probs).float(),
                        torch.cat(loss_masks).float(), cu, sum(lens))


def compute_opsm_mask(args, full_log_probs, full_old_log_probs, advantages, loss_masks):
    lens = [int(x.numel()) for x in full_log_probs]
    dev = advantages[0].device
    n = sum(lens)
    cu = torch.tensor([0] + lens, dtype=torch.int64).cumsum(0).to(dev)
    adv = torch.cat(advantages).float()
    out = ops.policy_loss(
        log_prob=torch.cat(full_log_probs).detach(), old_log_prob=torch.cat(full_old_log_probs).detach(),
        advantages=adv, loss_mask=torch.cat(loss_masks), cu_resp=cu, loss_kind="rloo", use_opsm=True,
        opsm_delta=args.opsm_delta, per_token_outputs=True,
    )
    # rloo pg = -(A*lp)*w: recover the 0/1 weight without dividing by zero-valued products
    seq_kl = _SeqKL.apply(torch.cat(full_log_probs).detach().float(), torch.cat(full_old_log_probs).float(),
                          torch.cat(loss_masks).float(), cu, n)
    drop = ((adv < 0) & (seq_kl > args.opsm_delta)).float()
    return 1 - drop, out["metrics"][_metric_slot("opsm_clipfrac")]


def _metric_slot(name: str) -> int:
    from ._lib import METRIC_SLOTS

    return METRIC_SLOTS.index(name)


# ------------------------------------------------------------------------------------------------- advantages


def get_grpo_returns(rewards, kl):
    """``ones_like(kl[i]) * rewards[i]`` per sample: one broadcast launch over the packed layout."""
    if len(kl) == 0:
        return []
    lens = [int(k.numel()) for k in kl]
    dev = kl[0].device
    cu = torch.tensor([0] + lens, dtype=torch.int64).cumsum(0).to(dev)
    flat = ops.broadcast_per_sample(rewards.to(dev).float(), cu, sum(lens))
    outs = []
    for piece, like in zip(torch.split(flat, lens), kl, strict=True):
        outs.append(piece.reshape(like.shape).to(like.dtype))
    return outs


def compute_rloo_leave_one_out_rewards(group_rewards):
    if group_rewards.dim() != 1:
        raise ValueError(
            f"compute_rloo_leave_one_out_rewards expects a 1-D tensor (one group), got shape "
            f"{tuple(group_rewards.shape)}. A 2-D input would be silently treated as a single oversized group and "
            f"produce wrong results."
        )
    g = group_rewards.shape[0]
    if g < 2:
        raise ValueError(
            f"RLOO requires n_samples_per_prompt >= 2 (group size {g} makes the leave-one-out baseline undefined: "
            f"division by G-1=0)."
        )
    if not torch.isfinite(group_rewards).all():
        raise ValueError(f"RLOO group contains non-finite reward(s): {group_rewards}. All rewards must be finite.")
    out, _ = ops.group_rewards(group_rewards, torch.zeros(g, dtype=torch.int32, device=group_rewards.device), "rloo")
    return out
