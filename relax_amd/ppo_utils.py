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
  get_reinforce_plus_plus_returns / _baseline_advantages   :708-843
  get_advantages_and_returns(_batch), vanilla_gae, chunked_gae   :846-1189
"""

from __future__ import annotations

from itertools import accumulate as _accumulate

import torch

from . import _lib, ops
from ._lib import check, lib
from ._staging import upload_int64


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


def _scan_dtype(t: torch.Tensor):
    """(torch dtype, ABI code) the recurrences run in: fp64 stays fp64, everything else is evaluated in fp32."""
    return (torch.float64, _lib.F64) if t.dtype == torch.float64 else (torch.float32, _lib.F32)


def _pack(parts, dtype, dev):
    return torch.cat([p.reshape(-1) for p in parts]).to(device=dev, dtype=dtype) if len(parts) > 1 else \
        parts[0].reshape(-1).to(device=dev, dtype=dtype)


def get_reinforce_plus_plus_returns(rewards, kl, loss_masks, response_lengths, total_lengths, kl_coef: float,
                                    gamma: float):
    """Discounted REINFORCE++ returns, one launch for the whole batch (ppo_utils.py:708-804, cp_size == 1):
    ``G_t = r_t + gamma * G_{t+1}`` with ``r_t = -kl_coef * kl_t`` on valid tokens and the sequence reward added at
    the last valid token; masked tokens (and fully masked sequences) get 0, and masked NaN/inf never leak."""
    n = len(rewards)
    if not (len(kl) == n and len(loss_masks) == n and len(response_lengths) == n and len(total_lengths) == n):
        raise ValueError(
            "rewards, kl, loss_masks, response_lengths, and total_lengths must contain the same number of responses.")
    for i, (k, m) in enumerate(zip(kl, loss_masks)):
        if k.shape != m.shape:
            raise ValueError(f"KL and loss mask for response {i} must have the same shape, got {k.shape} and {m.shape}.")
    if n == 0:
        return []
    dev = kl[0].device
    ops._need_gpu(kl[0])
    dtype, code = _scan_dtype(kl[0])
    lens = [int(k.numel()) for k in kl]
    cu = upload_int64([0] + list(_accumulate(lens)), dev)
    flat_kl, flat_mask = _pack(kl, dtype, dev), _pack(loss_masks, dtype, dev)
    rw = torch.as_tensor(rewards).to(device=dev, dtype=dtype).contiguous()
    out = torch.empty_like(flat_kl)
    check(lib.relax_amd_reinforce_pp_returns(ops._p(flat_kl), ops._p(flat_mask), ops._p(rw), code, ops._p(cu), n,
                                             float(kl_coef), float(gamma), ops._p(out), ops._stream()))
    return [piece.reshape(k.shape).to(k.dtype) for piece, k in zip(torch.split(out, lens), kl)]


def get_reinforce_plus_plus_baseline_advantages(rewards, kl, loss_masks):
    """``rewards[i]`` broadcast over sample i's valid tokens, 0 elsewhere (ppo_utils.py:807-843); ``kl`` only
    supplies shapes, so non-finite values in it are harmless."""
    if not (len(rewards) == len(kl) == len(loss_masks)):
        raise ValueError("rewards, token shapes, and loss_masks must contain the same number of responses.")
    for i, (k, m) in enumerate(zip(kl, loss_masks)):
        if k.shape != m.shape:
            raise ValueError(f"Token shape and loss mask for response {i} must match, got {k.shape} and {m.shape}.")
    if len(kl) == 0:
        return []
    dev = kl[0].device
    lens = [int(k.numel()) for k in kl]
    rw = torch.as_tensor(rewards).to(dev)
    if kl[0].dtype == torch.float64:
        # the broadcast kernel is fp32; fp64 callers (the reference's own tests) keep every bit of the reward
        flat = torch.repeat_interleave(rw.to(torch.float64), torch.tensor(lens, device=dev))
    else:
        flat = ops.broadcast_per_sample(rw.float(), upload_int64([0] + list(_accumulate(lens)), dev), sum(lens))
    mask = torch.cat([m.reshape(-1) for m in loss_masks]).to(dev)
    out = torch.where(mask != 0, flat, torch.zeros((), dtype=flat.dtype, device=dev))
    return [piece.reshape(k.shape).to(k.dtype) for piece, k in zip(torch.split(out, lens), kl)]


def get_advantages_and_returns_batch(total_lengths, response_lengths, values_list, rewards_list, gamma, lambd,
                                     chunked: bool = True, padded_total_lengths=None):
    """GAE for a batch of responses in one launch (ppo_utils.py:909-1023, cp_size == 1).  Every sequence is scanned in
    the order of ``vanilla_gae``; ``chunked`` is accepted for signature compatibility (the reference's chunked scan is
    a faster evaluation of the same recurrence and agrees with the sequential one to 1e-5)."""
    b = len(response_lengths)
    assert b == len(values_list)
    assert b == len(rewards_list)
    if b == 0:
        return [], []
    dev = values_list[0].device
    ops._need_gpu(values_list[0])
    dtype, code = _scan_dtype(values_list[0])
    lens = [int(r) for r in response_lengths]
    cu = upload_int64([0] + list(_accumulate(lens)), dev)
    v = _pack([x[:n] for x, n in zip(values_list, lens)], dtype, dev)
    r = _pack([x[:n] for x, n in zip(rewards_list, lens)], dtype, dev)
    adv, ret = torch.empty_like(v), torch.empty_like(v)
    check(lib.relax_amd_gae(ops._p(v), ops._p(r), code, ops._p(cu), b, float(gamma), float(lambd), ops._p(adv),
                            ops._p(ret), ops._stream()))
    out_dtype = values_list[0].dtype
    return ([a.to(out_dtype) for a in torch.split(adv, lens)], [x.to(out_dtype) for x in torch.split(ret, lens)])


def get_advantages_and_returns(total_len: int, response_len: int, values, rewards, gamma: float, lambd: float):
    """One response (ppo_utils.py:846-906): ``(advantages.detach(), returns)``."""
    adv, ret = get_advantages_and_returns_batch([total_len], [response_len], [values], [rewards], gamma, lambd)
    return adv[0].detach(), ret[0]


def vanilla_gae(rewards, values, gamma: float, lambd: float):
    """``[B, T]`` padded form (ppo_utils.py:1026-1047): every row is one sequence of length T."""
    b, t = rewards.shape
    adv, ret = get_advantages_and_returns_batch([t] * b, [t] * b, list(values), list(rewards), gamma, lambd)
    return torch.stack(adv), torch.stack(ret)


def chunked_gae(rewards, values, gamma: float, lambd: float, chunk_size: int = 128):
    """Same recurrence as :func:`vanilla_gae`; the chunk size has no effect here."""
    return vanilla_gae(rewards, values, gamma, lambd)


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
