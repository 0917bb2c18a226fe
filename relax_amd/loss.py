"""Drop-in counterparts of the hot-path functions of ``relax/backends/megatron/loss.py`` at context-parallel
size 1 in the packed ("thd") layout, running on the gfx950 kernels.

Reference lines (paths relative to the reference checkout):
  get_responses                   relax/backends/megatron/loss.py:49-191
  get_log_probs_and_entropy       :290-463
  compute_advantages_and_returns  :532-738
  policy_loss_function            :824-1185
  loss_function                   :1443-1620

Where the reference loops over samples in Python and runs ~10 full [R, V] fp32 passes per sample, these functions
build the packed row maps once and issue one forward launch and one backward launch for the whole micro-batch.
``policy_loss_function`` is usable as ``--loss-type custom_loss --custom-loss-function-path
relax_amd.loss.policy_loss_function``; ``get_log_probs_and_entropy`` as the ``f`` of ``forward_only``.
"""

from __future__ import annotations

from argparse import Namespace
from collections.abc import Iterator
from typing import Any

import torch

from . import ops
from ._lib import METRIC_SLOTS
from ._staging import upload_int64
from .cp_utils import (PerSampleDivisorReducer, get_cp_local_num_tokens, get_sum_of_sample_mean,
                       sample_denominators)
from .ppo_utils import get_grpo_returns

_SLOT = {k: i for i, k in enumerate(METRIC_SLOTS)}
GRPO_FAMILY = ("grpo", "gspo", "sapo", "cispo", "rloo")


def _check_logits(logits: torch.Tensor, args, max_seq_lens=None) -> torch.Tensor:
    """[1, T, V] (packed, "thd") or [B, S, V] (padded, "bshd") -> [rows, V] (loss.py:94-99).  fp32 is what stock
    Megatron hands over; bf16 / fp16 logits are accepted as well."""
    assert logits.dtype in (torch.float32, torch.bfloat16, torch.float16), f"{logits.dtype}"
    assert len(logits.shape) == 3, f"{logits.shape}"
    if getattr(args, "qkv_format", "thd") == "thd":
        assert logits.size(0) == 1, f"{logits.shape}"
        return logits.squeeze(0)
    assert max_seq_lens is not None
    return logits.reshape(-1, logits.size(-1))


def _padded_starts(args, max_seq_lens):
    """``max_seq_lens`` when the batch is in the padded "bshd" layout (sample i starts at row max_seq_lens[i] * i),
    None for the packed layout, where a sample starts where the previous one ends."""
    return None if getattr(args, "qkv_format", "thd") == "thd" else max_seq_lens


def response_row_begins(total_lengths, response_lengths, max_seq_lens=None) -> tuple[list[int], list[bool]]:
    """First logits row of each sample's response (loss.py:103-125): RL samples are scored by the previous
    position's logits (start - 1); the SFT convention (response == total) uses start (sft_utils.py:23-40).  With
    ``max_seq_lens`` (padded layout, loss.py:112-114) sample i's rows begin at ``max_seq_lens[i] * i``."""
    begins, sft = [], []
    end = 0
    for i, (total, resp) in enumerate(zip(total_lengths, response_lengths, strict=False)):
        end = max_seq_lens[i] * i + total if max_seq_lens is not None else end + total
        start = end - resp
        is_sft = resp == total
        begins.append(start if is_sft else start - 1)
        sft.append(is_sft)
    return begins, sft


def get_responses(
    logits: torch.Tensor,
    *,
    args: Namespace,
    unconcat_tokens: list[torch.Tensor],
    total_lengths: list[int],
    response_lengths: list[int],
    max_seq_lens=None,
    padded_total_lengths=None,
    apply_temperature: bool = True,
    dynamic_cp_size=None,
    dynamic_cp_rank=None,
) -> Iterator[tuple[torch.Tensor, torch.Tensor]]:
    """Yields per-sample ``(logits rows [R, V], target ids [R])`` views.  Kept for callers that want the slices;
    the fused functions below do not iterate samples.  Temperature is applied per chunk like the reference."""
    flat = _check_logits(logits, args, max_seq_lens)
    begins, sft = response_row_begins(total_lengths, response_lengths, _padded_starts(args, max_seq_lens))
    for b, is_sft, toks, resp in zip(begins, sft, unconcat_tokens, response_lengths, strict=False):
        chunk = flat[b : b + resp]
        targets = torch.nn.functional.pad(toks[1:], (0, 1), value=0) if is_sft else toks[-resp:]
        if apply_temperature and args.rollout_temperature != 1.0:
            chunk = chunk / args.rollout_temperature
        yield chunk, targets


class PackedLayout:
    """Device-side description of one packed micro-batch: response offsets, row maps and packed target ids."""

    def __init__(self, device, n_rows: int, unconcat_tokens, total_lengths, response_lengths, need_inverse: bool,
                 max_seq_lens=None):
        self.response_lengths = [int(r) for r in response_lengths]
        self.n_samples = len(self.response_lengths)
        self.n_tokens = sum(self.response_lengths)
        begins, sft = response_row_begins(total_lengths, response_lengths, max_seq_lens)
        for b, r in zip(begins, self.response_lengths):
            if r > 0 and (b < 0 or b + r > n_rows):
                raise IndexError(f"response rows [{b}, {b + r}) fall outside the {n_rows} logits rows")
        cu = [0]
        for r in self.response_lengths:
            cu.append(cu[-1] + r)
        # where each sample's targets sit in the back-to-back token ids: the last `response` tokens, or (SFT layout)
        # the tokens shifted by one with a final zero
        src_begin, src_end, pos = [], [], 0
        for toks, is_sft, resp in zip(unconcat_tokens, sft, self.response_lengths, strict=False):
            n_tok = int(toks.numel())
            if resp > n_tok:
                raise ValueError(f"response length {resp} exceeds the sample's {n_tok} tokens")
            src_begin.append(pos + 1 if is_sft else pos + n_tok - resp)
            src_end.append(pos + n_tok)
            pos += n_tok
        b = self.n_samples
        dev = upload_int64(begins + cu + src_begin + src_end, device)
        self.row_begin, self.cu_resp = dev[:b], dev[b : 2 * b + 1]
        self.row_ids, self.sample_ids, self.token_of_row = ops.build_row_maps(
            self.row_begin, self.cu_resp, self.n_tokens, n_rows, want_inverse=need_inverse
        )
        self.targets = torch.empty(self.n_tokens, dtype=torch.int64, device=device)
        if self.n_tokens:
            packed = torch.cat([t.reshape(-1) for t in unconcat_tokens]) if b > 1 else unconcat_tokens[0].reshape(-1)
            packed = packed.to(device=device, dtype=torch.int64)
            ops.gather_targets(packed, dev[2 * b + 1 : 3 * b + 1], dev[3 * b + 1 :], self.cu_resp, self.targets)

    def split(self, flat: torch.Tensor) -> list[torch.Tensor]:
        return list(torch.split(flat, self.response_lengths))


def get_log_probs_and_entropy(
    logits: torch.Tensor,
    *,
    args: Namespace,
    unconcat_tokens: list[torch.Tensor],
    total_lengths: list[int],
    response_lengths: list[int],
    with_entropy: bool = False,
    with_topk: bool = False,
    topk_k=None,
    gather_topk_token_ids=None,
    non_loss_data: bool = True,
    max_seq_lens=None,
    padded_total_lengths=None,
    dynamic_cp_size=None,
    dynamic_cp_rank=None,
    lm_head_forward=None,
    **_: Any,
) -> tuple[torch.Tensor, dict[str, list[torch.Tensor]]]:
    """One packed launch over every response token; returns ``(empty, {"log_probs": [...], "entropy": [...]})``
    with per-sample ``[R_i]`` fp32 views, differentiable w.r.t. ``logits``."""
    assert non_loss_data
    topk_k_arg = topk_k
    if lm_head_forward is not None:
        return _deferred_lm_head_log_probs(logits, args, unconcat_tokens, total_lengths, response_lengths,
                                           with_entropy, lm_head_forward, max_seq_lens)
    flat = _check_logits(logits, args, max_seq_lens)
    want_grad = with_entropy and getattr(args, "entropy_coef", 0.0) != 0
    needs_bwd = torch.is_grad_enabled() and logits.requires_grad
    lay = PackedLayout(flat.device, flat.size(0), unconcat_tokens, total_lengths, response_lengths, needs_bwd,
                       _padded_starts(args, max_seq_lens))
    inv_t = 1.0 / float(getattr(args, "rollout_temperature", 1.0))
    lse = None
    topk_ids = None
    topk_k = None
    if with_topk:
        topk_k = topk_k_arg if topk_k_arg is not None else getattr(args, "opd_log_prob_top_k", 1)
        topk_k = min(max(int(topk_k), 1), int(flat.size(-1)))
    if lay.n_tokens == 0:
        lp = flat.new_zeros((0,), dtype=torch.float32)
        ent = lp
    elif not needs_bwd and with_topk and topk_k <= ops.TOPK_ROWS_MAX_K and flat.size(-1) <= ops.TOPK_ROWS_MAX_VOCAB:
        # the actor's forward-only pass that also collects its top-K ids: one read of the logits serves the softmax
        # scan and the selection (the selection does not depend on the temperature)
        lp, ent, lse, _, _, topk_ids = ops.logprob_entropy_topk_fwd(ops._rows(flat), lay.targets, lay.row_ids, inv_t,
                                                                    topk_k, bool(with_entropy))
    elif not needs_bwd:
        # forward-only (the ActorFwd / Reference passes): the launch's log-sum-exps stay at hand, so that a top-K gather
        # below costs K loads per row instead of another scan of the logits
        lp, ent, lse, _ = ops.logprob_entropy_fwd(ops._rows(flat), lay.targets, lay.row_ids, inv_t, bool(with_entropy))
    else:
        lp, ent = ops.LogProbEntropy.apply(
            flat, lay.targets, lay.row_ids, lay.token_of_row, inv_t, bool(with_entropy), bool(want_grad)
        )
    res = {"log_probs": lay.split(lp)}
    if with_entropy:
        res["entropy"] = lay.split(ent)
    if with_topk:
        # diagnostic student-side top-K ids (loss.py:436-438): a library selection over each sample's own rows
        k = topk_k
        if topk_ids is not None:
            res["topk_token_ids"] = lay.split(topk_ids)
        elif lay.n_tokens and k <= ops.TOPK_ROWS_MAX_K and flat.size(-1) <= ops.TOPK_ROWS_MAX_VOCAB:
            # one launch over every response row (the selection does not depend on the temperature)
            _, ids = ops.topk_rows(flat, lay.row_ids, k, with_values=False)
            res["topk_token_ids"] = lay.split(ids)
        else:  # very large k: the library's selection, sample by sample like the reference
            begins, _ = response_row_begins(total_lengths, response_lengths, _padded_starts(args, max_seq_lens))
            res["topk_token_ids"] = [torch.topk(flat[b:b + r], k=k, dim=-1).indices
                                     for b, r in zip(begins, lay.response_lengths)]
    if gather_topk_token_ids is not None:
        res["topk_log_probs"] = _gathered_topk_log_probs(flat, lay, gather_topk_token_ids, inv_t, lse)
    return torch.empty((0,), device=logits.device), res


def lm_head_weight_of(lm_head_forward) -> torch.Tensor:
    """The ``[V, H]`` weight behind a deferred LM head.  The reference hands the loss the captured
    ``output_layer.forward`` (relax/backends/megatron/model.py:93-181) and calls it per 1024-row sub-chunk; a fused
    kernel needs the operand itself, which a bound method, a module or a plain tensor all give up."""
    if isinstance(lm_head_forward, torch.Tensor):
        return lm_head_forward
    owner = getattr(lm_head_forward, "__self__", lm_head_forward)
    weight = getattr(owner, "weight", None)
    if not isinstance(weight, torch.Tensor) or weight.dim() != 2:
        raise NotImplementedError(
            "lm_head_forward must expose the LM-head weight (a bound forward of a module with .weight, the module "
            "itself, or the weight tensor): an opaque callable cannot be fused")
    if getattr(owner, "bias", None) is not None:
        raise NotImplementedError("a deferred LM head with a bias is not supported")
    return weight


def _deferred_rows(hidden, weight, args, unconcat_tokens, total_lengths, response_lengths, max_seq_lens):
    """``([T, H] rows of the hidden states, PackedLayout of their response tokens)`` for a deferred LM head: ``hidden``
    is ``[1, T, H]`` packed, ``[B, S, H]`` padded, or ``[T, H]``."""
    padded = _padded_starts(args, max_seq_lens)
    if hidden.dim() == 3 and padded is not None:
        rows = hidden.reshape(-1, hidden.size(-1))  # [B, S, H]: sample i starts at row max_seq_lens[i] * i
    elif hidden.dim() == 3:
        if hidden.size(0) != 1:
            raise ValueError(f"expected packed hidden states [1, T, H], got {tuple(hidden.shape)}")
        rows = hidden[0]
    else:
        rows = hidden
    if rows.dim() != 2 or rows.size(1) != weight.size(1):
        raise ValueError(f"hidden states {tuple(hidden.shape)} do not match the LM-head weight {tuple(weight.shape)}")
    if not rows.is_cuda:
        raise RuntimeError("relax_amd kernels need ROCm device tensors (no CPU fallback)")
    lay = PackedLayout(rows.device, rows.size(0), unconcat_tokens, total_lengths, response_lengths, False, padded)
    return rows, lay


def _deferred_lm_head_log_probs(hidden, args, unconcat_tokens, total_lengths, response_lengths, with_entropy,
                                lm_head_forward, max_seq_lens=None):
    """Deferred-LM-head branch of get_log_probs_and_entropy (loss.py:391-419): ``hidden`` is ``[1, T, H]`` (or
    ``[T, H]``) and the ``[T, V]`` logits are never formed.  The response rows of all samples go through the fused
    LM-head kernel in one launch; unlike the reference's chunked path entropy is available as well."""
    from .lm_head import lm_head_log_probs_and_entropy

    weight = lm_head_weight_of(lm_head_forward)
    rows, lay = _deferred_rows(hidden, weight, args, unconcat_tokens, total_lengths, response_lengths, max_seq_lens)
    if lay.n_tokens == 0:
        lp = rows.new_zeros((0,), dtype=torch.float32)
        ent = lp
    else:
        picked = rows.index_select(0, lay.row_ids.to(torch.int64)).to(weight.dtype)  # [N, H]: megabytes, not [N, V]
        want_grad = with_entropy and getattr(args, "entropy_coef", 0.0) != 0
        lp, ent = lm_head_log_probs_and_entropy(picked, weight, lay.targets,
                                                float(getattr(args, "rollout_temperature", 1.0)),
                                                with_entropy=bool(with_entropy), with_entropy_grad=bool(want_grad))
    res = {"log_probs": lay.split(lp)}
    if with_entropy:
        res["entropy"] = lay.split(ent)
    return torch.empty((0,), device=hidden.device), res


def sft_loss_function_chunked(args: Namespace, batch: dict, hidden_states: torch.Tensor, sum_of_sample_mean=None, *,
                              lm_head_forward):
    """SFT loss with the LM head deferred into the loss (loss.py:1386-1428): ``-sum_of_sample_mean(log_probs)`` with
    the log-probs taken straight from hidden states and the LM-head weight.  ``sum_of_sample_mean`` may be None: the
    reference's reducer is then rebuilt from the batch."""
    if sum_of_sample_mean is None:
        sum_of_sample_mean = get_sum_of_sample_mean(
            batch["total_lengths"], batch["response_lengths"], batch["loss_masks"],
            bool(getattr(args, "calculate_per_token_loss", False)), sample_denoms=batch.get("sample_index_mask_sums"))
    if torch.is_grad_enabled() and getattr(args, "relax_amd_single_pass", "auto") not in (False, "off") \
            and getattr(sum_of_sample_mean, "relax_amd_linear", False):
        loss = _sft_chunked_single_projection(args, batch, hidden_states, sum_of_sample_mean, lm_head_forward)
        if loss is not None:
            return loss, {"loss": loss.clone().detach()}
    _, out = get_log_probs_and_entropy(
        hidden_states, args=args, unconcat_tokens=batch["unconcat_tokens"], total_lengths=batch["total_lengths"],
        response_lengths=batch["response_lengths"], with_entropy=False, lm_head_forward=lm_head_forward,
        max_seq_lens=batch.get("max_seq_lens"))
    log_probs = torch.cat(out["log_probs"], dim=0)
    loss = -sum_of_sample_mean(log_probs)
    if log_probs.numel() == 0:
        loss = loss + 0 * hidden_states.sum()
    return loss, {"loss": loss.clone().detach()}


def _sft_chunked_single_projection(args, batch, hidden_states, sum_of_sample_mean, lm_head_forward):
    """The training step of the chunked SFT loss with one projection instead of two: the reducer is linear in the
    log-probs (every reducer of cp_utils.py:125-162 is a sum of masked per-sample means or token sums; this library's
    reducers say so with ``relax_amd_linear``, any other callable keeps the two-projection path), so each
    token's weight in the loss is known before its log-prob is, and the LM-head step can turn every slab of logits
    into its gradient straight away (``lm_head.lm_head_token_local_step``).  The weights are read off the reducer
    itself, as its gradient; the value returned is the reducer's own.  None when nothing needs a gradient."""
    from .lm_head import lm_head_token_local_step

    weight = lm_head_weight_of(lm_head_forward)
    if not (hidden_states.requires_grad or weight.requires_grad):
        return None
    rows, lay = _deferred_rows(hidden_states, weight, args, batch["unconcat_tokens"], batch["total_lengths"],
                               batch["response_lengths"], batch.get("max_seq_lens"))
    if lay.n_tokens == 0:
        return None
    probe = torch.zeros(lay.n_tokens, dtype=torch.float32, device=rows.device, requires_grad=True)
    with torch.enable_grad():
        token_weight, = torch.autograd.grad(sum_of_sample_mean(probe), probe)
    picked = rows.index_select(0, lay.row_ids.to(torch.int64)).to(weight.dtype)  # [N, H]

    def token_loss(begin, end, log_prob, _entropy):
        return -(log_prob * token_weight[begin:end]).sum()

    loss, log_probs, _ = lm_head_token_local_step(
        picked, weight, lay.targets, token_loss, float(getattr(args, "rollout_temperature", 1.0)),
        assumed_grad_scale=expected_grad_scale(batch))
    # the value in the reducer's own order of summation; the gradient is the step's
    return (-sum_of_sample_mean(log_probs)).detach().to(loss.dtype) + (loss - loss.detach())


def _sft_single_pass(args: Namespace, batch: dict, logits: torch.Tensor):
    """The SFT loss as one launch of the fused step: ``-sum_of_sample_mean(lp)`` is the REINFORCE surrogate
    ``-A * lp`` with unit advantages and no KL or entropy term, so forward scan and dlogits share one pass over the
    logits (one HBM read and one write per row instead of two reads and a write)."""
    flat = _check_logits(logits, args, batch.get("max_seq_lens"))
    dev = flat.device
    lay = PackedLayout(dev, flat.size(0), batch["unconcat_tokens"], batch["total_lengths"], batch["response_lengths"],
                       True, _padded_starts(args, batch.get("max_seq_lens")))
    if lay.n_tokens == 0:
        return None
    per_token = bool(getattr(args, "calculate_per_token_loss", False))
    masks = [m.to(dev) for m in batch["loss_masks"]]
    denom = None if per_token else sample_denominators(masks, lay, batch.get("sample_index_mask_sums"))
    kw = dict(
        old_log_prob=None, ref_log_prob=None, train_log_prob=None, rollout_log_prob=None,
        advantages=torch.ones(lay.n_tokens, dtype=torch.float32, device=dev), loss_mask=_cat_f32(masks, dev),
        sample_denom=denom, pg_sample_denom=None, loss_kind="rloo", kl_kind=None, unbiased_kl=False, use_opsm=False,
        use_tis=False, mismatch_metrics=False, abs_diff_from_old=2, eps_clip=0.2, eps_clip_high=0.2, entropy_coef=0.0,
        kl_coef=0.0, tis_lo=0.0, tis_hi=2.0, opsm_delta=1e-4, tau_pos=1.0, tau_neg=1.05)
    inv_t = 1.0 / float(getattr(args, "rollout_temperature", 1.0))
    loss, _metrics, _lp, _ent, _ = _SinglePassPolicyLoss.apply(flat, lay, inv_t, kw, expected_grad_scale(batch))
    return loss


def sft_loss_function(args: Namespace, batch: dict, logits: torch.Tensor, sum_of_sample_mean=None):
    """Negative log-likelihood of the response tokens (loss.py:1247-1293): ``-sum_of_sample_mean(log_probs)``.
    ``sum_of_sample_mean`` may be None: the reference's reducer is then rebuilt from the batch, and when a gradient
    is wanted the whole loss runs as one launch (``args.relax_amd_single_pass = "off"`` keeps the separate log-prob
    forward / backward launches)."""
    if sum_of_sample_mean is None and torch.is_grad_enabled() and logits.requires_grad \
            and getattr(args, "relax_amd_single_pass", "auto") not in (False, "off"):
        loss = _sft_single_pass(args, batch, logits)
        if loss is not None:
            return loss, {"loss": loss.clone().detach()}
    _, out = get_log_probs_and_entropy(
        logits, args=args, unconcat_tokens=batch["unconcat_tokens"], total_lengths=batch["total_lengths"],
        response_lengths=batch["response_lengths"], with_entropy=False, max_seq_lens=batch.get("max_seq_lens"))
    log_probs = torch.cat(out["log_probs"], dim=0)
    if sum_of_sample_mean is None:
        sum_of_sample_mean = get_sum_of_sample_mean(
            batch["total_lengths"], batch["response_lengths"], batch["loss_masks"],
            bool(getattr(args, "calculate_per_token_loss", False)), sample_denoms=batch.get("sample_index_mask_sums"))
    loss = -sum_of_sample_mean(log_probs)
    if log_probs.numel() == 0:
        loss = loss + 0 * logits.sum()
    return loss, {"loss": loss.clone().detach()}


def _pack_topk_ids(flat, lay, gather_topk_token_ids):
    """Per-sample ``[R_i, K_i]`` id tensors -> (one ``[N, K_max]`` int64 tensor padded with the -1 sentinel, the
    per-sample widths); ``(None, widths)`` when there is nothing to gather."""
    dev = flat.device
    per_sample, widths = [], []
    for i, r in enumerate(lay.response_lengths):
        ids = gather_topk_token_ids[i] if i < len(gather_topk_token_ids) else None
        if ids is None or ids.numel() == 0:
            per_sample.append(None)
            widths.append(0)
            continue
        if ids.dim() != 2 or ids.size(0) != r:
            raise ValueError(f"top-K ids of sample {i} must be [{r}, K], got {tuple(ids.shape)}")
        per_sample.append(ids.to(device=dev, dtype=torch.long))
        widths.append(int(ids.size(1)))
    k_max = max(widths) if widths else 0
    if k_max == 0 or lay.n_tokens == 0:
        return None, widths
    if all(w == k_max for w in widths):  # the usual case, every sample with the same K: one concatenation
        return (per_sample[0] if len(per_sample) == 1 else torch.cat(per_sample, dim=0)).contiguous(), widths
    packed = torch.full((lay.n_tokens, k_max), -1, dtype=torch.long, device=dev)
    pos = 0
    for ids, r, w in zip(per_sample, lay.response_lengths, widths):
        if w:
            packed[pos:pos + r, :w] = ids
        pos += r
    return packed, widths


def _trim_topk(out, flat, lay, widths):
    """``[N, K_max]`` gathered log-probs -> per-sample ``[R_i, K_i]`` views."""
    if out is None:
        return [flat.new_zeros((r, 0)) for r in lay.response_lengths]
    pieces = torch.split(out, lay.response_lengths)
    return [p[:, :w] if w else flat.new_zeros((r, 0)) for p, r, w in zip(pieces, lay.response_lengths, widths)]


def _gathered_topk_log_probs(flat, lay, gather_topk_token_ids, inv_t, lse=None):
    """Per-sample ``[R_i, K_i]`` log-probs at the given vocabulary ids (compute_opd_topk_log_probs,
    relax/utils/opd/opd_utils.py:1005-1019) in one packed launch: samples with fewer ids (the union path) are padded
    with the -1 sentinel, which yields -inf and no gradient, and trimmed again afterwards.  ``lse`` (the rows'
    log-sum-exps from a log-prob launch over the same rows) spares the gather its own scan of the logits."""
    from .opd_utils import TopKLogProbs

    packed, widths = _pack_topk_ids(flat, lay, gather_topk_token_ids)
    out = None if packed is None else TopKLogProbs.apply(flat, packed, inv_t, lse, lay.row_ids, lay.token_of_row,
                                                         torch.is_grad_enabled() and flat.requires_grad)
    return _trim_topk(out, flat, lay, widths)


# ------------------------------------------------------------------------------------------ fused policy loss


class _FusedPolicyLoss(torch.autograd.Function):
    """logits [T, V] -> scalar loss, two-launch form.  Forward: one log-prob/entropy launch + the policy-loss
    launches; backward: one dlogits launch fed with the stored d loss / d lp and d loss / d entropy coefficients."""

    @staticmethod
    def forward(ctx, flat, lay, inv_t, kw):
        lp, ent, lse, spx = ops.logprob_entropy_fwd(flat, lay.targets, lay.row_ids, inv_t, True)
        lp_visible = bool(kw.get("lp_requires_grad", False))
        gather_ids = kw.get("gather_topk_ids")
        kw = {k: v for k, v in kw.items() if k not in ("lp_requires_grad", "gather_topk_ids")}
        out = ops.policy_loss(log_prob=lp, entropy=ent, cu_resp=lay.cu_resp, **kw)
        metrics = out["metrics"]
        entropy_grad = kw.get("entropy_coef", 0.0) != 0
        if gather_ids is not None:
            # log-probs at the given vocabulary ids (the top-K distillation term): K loads per row next to the
            # log-sum-exp just computed; their gradient comes back to this function's one dlogits launch
            topk_lp = torch.empty(gather_ids.shape, dtype=torch.float32, device=flat.device)
            stride = flat.stride(0) if flat.size(0) > 1 else flat.size(1)
            ops.check(ops.lib.relax_amd_topk_logprob_fwd(
                ops._p(flat), ops._code(flat), gather_ids.size(0), flat.size(1), stride, ops._p(lay.row_ids),
                ops._p(gather_ids), gather_ids.size(1), float(inv_t), ops._p(lse), ops._p(topk_lp), None,
                ops._stream()))
        else:
            topk_lp = lp.new_zeros(0)
        ctx.save_for_backward(flat, lay.targets, lse, spx if entropy_grad else None, out["coef_log_prob"],
                              out["coef_entropy"] if entropy_grad else None, lay.token_of_row, gather_ids,
                              lay.row_ids if gather_ids is not None else None)
        ctx.inv_t = inv_t
        # ``lp_requires_grad``: further loss terms built on the returned log-probs (the distillation term) send their
        # gradient back here, where it joins the policy loss's coefficient before the one dlogits launch
        hidden = [metrics, ent] + ([] if lp_visible else [lp]) + ([] if gather_ids is not None else [topk_lp])
        ctx.mark_non_differentiable(*hidden)
        return metrics[_SLOT["loss"]].clone(), metrics, lp, ent, topk_lp

    @staticmethod
    def backward(ctx, g_loss, _gm, g_lp, _gent, g_topk):
        flat, targets, lse, spx, c_lp, c_ent, token_of_row, gather_ids, row_ids = ctx.saved_tensors
        scale = g_loss.reshape(1).to(torch.float32).contiguous()
        sparse = None
        if gather_ids is None:
            g_topk = None
        if g_lp is not None or g_topk is not None:
            c_lp = c_lp * scale
            c_ent = None if c_ent is None else c_ent * scale
            scale = None
            if g_lp is not None:
                c_lp = c_lp + g_lp.reshape(-1).to(torch.float32)
            if g_topk is not None:
                # d log p[id_k] / d logits = onehot(id_k) - p: the -p parts of all K join the log-prob coefficient
                # (whose own onehot, at the target, is taken back below); the onehots are K sparse additions
                g_k = torch.where(gather_ids >= 0, g_topk.to(torch.float32), torch.zeros((), device=flat.device))
                total = g_k.sum(dim=-1)
                c_lp = c_lp + total
                sparse = (g_k, -total)
        d = ops.logprob_entropy_bwd(flat, targets, lse, spx, c_lp, c_ent, token_of_row=token_of_row,
                                    grad_scale_dev=scale, inv_temperature=ctx.inv_t)
        if sparse is not None:
            ops.sparse_row_add(d, row_ids, gather_ids, sparse[0], targets, sparse[1], scale=ctx.inv_t)
        return d, None, None, None


GRAD_SCALE_KEY = "relax_amd_grad_scale"


def expected_grad_scale(batch) -> float:
    """The upstream gradient the loss is expected to receive in backward (``batch["relax_amd_grad_scale"]``, set by
    ``loss_function`` from its own scaling; 1 when the loss is differentiated as returned)."""
    hint = batch.get(GRAD_SCALE_KEY)
    if hint is None:
        return 1.0
    hint = float(hint)
    return hint if (hint == hint and hint != 0.0 and abs(hint) != float("inf")) else 1.0


class _SinglePassPolicyLoss(torch.autograd.Function):
    """logits [T, V] -> scalar loss, single-launch form: each workgroup scans its row and at once walks it again
    (out of registers or cache) to write dlogits for the upstream gradient ``assumed_scale`` the caller expects, so
    HBM sees one read and one write per row.  The backward compares the actual upstream gradient with the assumed one
    on the device: a no-op kernel when they agree, one more pass over dlogits (and a second rounding of 16-bit
    gradients) when they do not."""

    @staticmethod
    def forward(ctx, flat, lay, inv_t, kw, assumed_scale=1.0):
        out, lp, ent, _lse, _spx, dlogits = ops.actor_step_fused(
            flat, lay.targets, lay.token_of_row, lay.sample_ids, lay.n_tokens, inv_t, float(assumed_scale),
            cu_resp=lay.cu_resp, **kw)
        metrics = out["metrics"]
        topk = kw.get("topk_distill")
        if topk is not None:
            # the top-K distillation term: its multiple of each row's softmax left with the launch, the K one-hot
            # parts are added here (d log p[id] / d logits = (onehot(id) - p) / T)
            ops.sparse_row_add(dlogits, lay.row_ids, topk["ids"], out["topk_grad"],
                               scale=float(inv_t) * float(assumed_scale))
            topk_kl = out["topk_kl"]
        else:
            topk_kl = lp.new_zeros(0)
        ctx.dlogits = dlogits
        ctx.assumed_scale = float(assumed_scale)
        ctx.mark_non_differentiable(metrics, lp, ent, topk_kl)
        ctx.set_materialize_grads(False)  # no zero tensors for the outputs nothing differentiates (three fills a step)
        return metrics[_SLOT["loss"]].clone(), metrics, lp, ent, topk_kl

    @staticmethod
    def backward(ctx, g_loss, _gm, _glp, _gent, _gkl):
        if g_loss is None:  # the loss itself took no part in what was differentiated
            return None, None, None, None, None
        d = ctx.dlogits
        if d is None:
            raise RuntimeError("the single-pass policy loss holds its gradient once: backward cannot run twice")
        ctx.dlogits = None
        factor = g_loss.reshape(1).to(torch.float32)
        if ctx.assumed_scale != 1.0:
            factor = factor / ctx.assumed_scale
        ops.scale_rows_inplace(d, factor.contiguous())
        return d, None, None, None, None


def _sampled_opd_kernel_args(args, batch, loss_mask, dev):
    """(kernel arguments, teacher log-probs [N]) that put the gradient of the sampled-token distillation term
    (relax/utils/opd/opd_utils.py:1368-1455: ``opd_loss_coef * token_mean(signal)``) into the single launch, or None
    when the term is not of that kind (top-K selections, no teacher log-probs).  ``extra_coef_log_prob`` holds each
    token's weight ``opd_loss_coef * mask / clamp_min(sum mask, 1)``; the plain ``reverse_kl`` signal (lp - teacher)
    has derivative 1 and needs nothing else, ``low_var_kl`` and the clamp / clips are applied by the kernel."""
    if getattr(args, "opd_token_selection", "sampled") in ("student_topk", "teacher_topk", "union"):
        return None
    kl_type = getattr(args, "opd_kl_type", "reverse_kl")
    if kl_type not in ("reverse_kl", "low_var_kl"):
        return None
    teacher = batch.get("teacher_log_probs")
    if teacher is None:
        return None
    teacher = torch.cat([t.reshape(-1) for t in teacher]).to(device=dev, dtype=torch.float32)
    if teacher.numel() != loss_mask.numel():
        return None
    clamp, tau, is_clip = (getattr(args, k, None) for k in ("opd_log_prob_min_clamp", "opd_per_token_clip",
                                                            "opd_is_clip"))
    out = {"extra_coef_log_prob": loss_mask * (float(args.opd_loss_coef) / torch.clamp_min(loss_mask.sum(), 1))}
    if tau is not None or is_clip is not None:
        # the clip-fraction metrics are plain means over every response token, masked ones included: the launch then
        # scans the rows of masked tokens as well (it skips them otherwise)
        out["read_masked_rows"] = True
    if kl_type != "reverse_kl" or any(v is not None for v in (clamp, tau, is_clip)):
        out["distill"] = dict(teacher=teacher, kl_kind="k1" if kl_type == "reverse_kl" else "k3", min_clamp=clamp,
                              token_clip=tau, is_clip=is_clip)
    return out, teacher


def _topk_opd_kernel_args(args, batch, lay, packed_ids, widths, loss_mask, dev):
    """Kernel arguments that put the top-K distillation term (relax/utils/opd/opd_utils.py:1368-1455 with the
    ``student_topk`` / ``teacher_topk`` / ``union`` selections) into the single launch, or None when the batch or the
    options do not fit it (then the two-launch path takes the step and reports what is wrong with them).
    ``packed_ids`` / ``widths`` as ``_pack_topk_ids`` returns them; ``extra_coef_log_prob`` holds each token's weight
    ``opd_loss_coef * mask / clamp_min(sum mask, 1)``."""
    from ._lib import FUSED_TOPK_MAX
    from .opd_utils import opd_topk_kernel_modes

    teacher = batch.get("opd_topk_teacher_log_probs")
    if packed_ids is None or not teacher or packed_ids.size(1) > FUSED_TOPK_MAX or len(teacher) != len(widths) \
            or min(widths) == 0:
        return None
    try:
        mode, alpha, norm = opd_topk_kernel_modes(args.opd_kl_type, float(args.opd_jsd_alpha),
                                                  getattr(args, "opd_norm_mode", "tail"))
    except ValueError:
        return None
    clamp, tau, is_clip = (getattr(args, k, None) for k in ("opd_log_prob_min_clamp", "opd_per_token_clip",
                                                            "opd_is_clip"))
    n, k = packed_ids.shape
    resp = lay.response_lengths
    if any(t is None or tuple(t.shape) != (r, w) for t, r, w in zip(teacher, resp, widths)):
        return None
    ksz = batch.get("opd_topk_ksz") if args.opd_token_selection == "union" else None
    uniform = all(w == k for w in widths)
    if uniform:
        t_packed = torch.cat([t.to(device=dev, dtype=torch.float32) for t in teacher], dim=0)
        width = None
    else:
        t_packed = torch.zeros((n, k), dtype=torch.float32, device=dev)
        pos = 0
        for t, r, w in zip(teacher, resp, widths):
            t_packed[pos:pos + r, :w] = t.to(device=dev, dtype=torch.float32)
            pos += r
        width = torch.repeat_interleave(torch.tensor(widths, dtype=torch.int32, device=dev),
                                        torch.tensor(resp, dtype=torch.int64, device=dev))
    valid = None
    if ksz is not None and any(i < len(ksz) and ksz[i] is not None for i in range(len(resp))):
        valid = torch.full((n,), -1, dtype=torch.int32, device=dev)
        pos = 0
        for i, r in enumerate(resp):
            if i < len(ksz) and ksz[i] is not None:
                valid[pos:pos + r] = ksz[i].to(device=dev, dtype=torch.int32).reshape(-1)
            pos += r
    return {
        "extra_coef_log_prob": loss_mask * (float(args.opd_loss_coef) / torch.clamp_min(loss_mask.sum(), 1)),
        "topk_distill": dict(ids=packed_ids, teacher=t_packed.detach(), width=width, valid=valid, kl_mode=mode,
                             norm_mode=norm, alpha=alpha, min_clamp=clamp, token_clip=tau, is_clip=is_clip),
        # the clip-fraction metrics average over masked tokens too: their rows are then scanned as well
        "read_masked_rows": tau is not None or is_clip is not None,
    }


def _single_pass_ok(args, flat, kw, needs_bwd) -> bool:
    mode = getattr(args, "relax_amd_single_pass", "auto")
    if mode in (False, "off") or not needs_bwd:
        return False
    if kw["loss_kind"] == "gspo" or kw["use_opsm"]:
        return False  # sequence-coupled gradients need the per-sequence reduction between forward and backward
    return True


def _cat_f32(parts, device):
    """Per-sample tensors -> one packed fp32 vector on ``device`` (one concatenation, one conversion)."""
    if parts is None:
        return None
    if isinstance(parts, torch.Tensor):
        return parts.to(device=device, dtype=torch.float32).reshape(-1)
    if len(parts) == 1:
        return parts[0].reshape(-1).to(device=device, dtype=torch.float32)
    first = parts[0]
    if all(p.device == first.device and p.dtype == first.dtype and p.dim() == 1 for p in parts):
        return torch.cat(parts).to(device=device, dtype=torch.float32)
    return torch.cat([p.to(device=device).reshape(-1) for p in parts]).to(torch.float32)


def _cat_fields_f32(device, n_tokens: int, **fields):
    """Several per-sample lists -> packed fp32 vectors, ``{name: [N] tensor | None}``.  When every list holds 1-D fp32
    tensors on ``device`` that add up to ``n_tokens`` elements, all of them are packed by ONE concatenation and the
    results are views of its output (a batch arrives as a handful of such lists, and each concatenation is a launch of
    its own that costs more than it moves); anything else falls back to one ``_cat_f32`` per field."""
    live = {k: v for k, v in fields.items() if v is not None}
    simple = len(live) > 1 and all(
        isinstance(v, (list, tuple)) and len(v) > 0 and all(
            torch.is_tensor(t) and t.dim() == 1 and t.dtype == torch.float32 and t.device == device for t in v)
        and sum(int(t.numel()) for t in v) == n_tokens for v in live.values())
    if not simple:
        return {k: _cat_f32(v, device) for k, v in fields.items()}
    packed = torch.cat([t for v in live.values() for t in v])
    out = {k: None for k in fields}
    for i, k in enumerate(live):
        out[k] = packed[i * n_tokens:(i + 1) * n_tokens]
    return out


def load_function(path: str):
    """``"pkg.module.fn"`` -> the function object (relax/utils/misc.py:30-38)."""
    import importlib

    module_path, _, attr = path.rpartition(".")
    return getattr(importlib.import_module(module_path), attr)


def _tis_terms(args, pg_loss, train_log_probs, rollout_log_probs):
    ratio_log = torch.cat(train_log_probs, dim=0) - torch.cat(rollout_log_probs, dim=0)
    tis = torch.exp(ratio_log)
    metrics = {"tis": tis, "tis_abs": (tis - 1).abs(), "mismatch_kl": -ratio_log, "mismatch_k3_kl": tis - ratio_log - 1}
    return tis, metrics


def vanilla_tis_function(args, *, pg_loss, train_log_probs, rollout_log_probs, loss_masks, **kwargs):
    """Truncated importance sampling, loss.py:741-769: weights ``clamp(exp(train - rollout), tis_clip_low, tis_clip)``.
    Returns ``(pg_loss * weights, loss_masks, per-token metrics)``; the plug-in signature of
    ``--custom-tis-function-path``."""
    tis, metrics = _tis_terms(args, pg_loss, train_log_probs, rollout_log_probs)
    weights = torch.clamp(tis, min=args.tis_clip_low, max=args.tis_clip)
    metrics["tis_clipfrac"] = (weights != tis).float()
    return pg_loss * weights, loss_masks, {k: v.clone().detach() for k, v in metrics.items()}


def icepop_function(args, *, pg_loss, train_log_probs, rollout_log_probs, loss_masks, **kwargs):
    """loss.py:772-801: like the truncated weights, but ratios outside ``[tis_clip_low, tis_clip]`` are zeroed."""
    tis, metrics = _tis_terms(args, pg_loss, train_log_probs, rollout_log_probs)
    weights = torch.where((tis >= args.tis_clip_low) & (tis <= args.tis_clip), tis, torch.zeros_like(tis))
    metrics["tis_clipfrac"] = (weights != tis).float()
    return pg_loss * weights, loss_masks, {k: v.clone().detach() for k, v in metrics.items()}


def _mask_safe(reducer, loss_masks):
    """REINFORCE++ reductions select the valid tokens first (loss.py:804-821), so a non-finite value under a zero mask
    cannot reach the sum as ``NaN * 0``."""
    valid = torch.cat([m.reshape(-1) != 0 for m in loss_masks], dim=0)

    def reduce_valid_tokens(values):
        v = valid.to(device=values.device)
        if values.shape[0] != v.numel():
            raise ValueError("REINFORCE++ reducer expected one value per response token, "
                             f"got {values.shape[0]} values for {v.numel()} mask elements.")
        return reducer(torch.where(v, values, torch.zeros_like(values)))

    return reduce_valid_tokens


def _composed_policy_loss_function(args: Namespace, batch: dict, logits: torch.Tensor, sum_of_sample_mean=None):
    """The policy loss as the reference composes it (loss.py:824-1185), step by step, for the configurations that hand
    per-token tensors to user code: ``--custom-tis-function-path`` (importance weights / rejection masks) and
    ``--custom-pg-loss-reducer-function-path``.  The ``[N, V]`` work is still one packed log-prob / entropy launch
    (forward) and one dlogits launch (backward); everything between them acts on ``[N]`` vectors through the
    differentiable token-loss kernels of ``ppo_utils`` and plain tensor arithmetic, so arbitrary Python can sit in the
    middle."""
    from . import ppo_utils as PU
    from .opd_utils import compute_policy_opd_loss, resolve_opd_gather_topk_token_ids

    est = args.advantage_estimator
    pp = est in ("reinforce_plus_plus", "reinforce_plus_plus_baseline")
    response_lengths, total_lengths = batch["response_lengths"], batch["total_lengths"]
    masks = batch["loss_masks"]
    per_token = bool(getattr(args, "calculate_per_token_loss", False))

    def reducer_for(loss_masks):
        red = get_sum_of_sample_mean(total_lengths, response_lengths, loss_masks, per_token,
                                     sample_denoms=batch.get("sample_index_mask_sums"))
        return _mask_safe(red, loss_masks) if pp else red

    reduce = sum_of_sample_mean if sum_of_sample_mean is not None else reducer_for(masks)
    if pp and sum_of_sample_mean is not None:
        reduce = _mask_safe(reduce, masks)
    dev = logits.device
    adv = batch["advantages"]
    adv = adv.to(dev).float() if isinstance(adv, torch.Tensor) else torch.cat([a.to(dev) for a in adv]).float()
    _, out = get_log_probs_and_entropy(
        logits, args=args, unconcat_tokens=batch["unconcat_tokens"], total_lengths=total_lengths,
        response_lengths=response_lengths, with_entropy=True, max_seq_lens=batch.get("max_seq_lens"),
        gather_topk_token_ids=resolve_opd_gather_topk_token_ids(args, batch))
    lps = out["log_probs"]
    true_on_policy = getattr(args, "true_on_policy_mode", False)
    if true_on_policy:
        olds = [x.detach() for x in lps]
    else:
        olds = [x.to(dev) for x in (batch["rollout_log_probs"] if args.use_rollout_logprobs else batch["log_probs"])]
    masks_dev = [m.to(dev) for m in masks]
    adv_list = list(torch.split(adv, response_lengths))
    if getattr(args, "use_opsm", False):
        opsm_mask, opsm_clipfrac = PU.compute_opsm_mask(args, lps, olds, adv_list, masks_dev)
    lp, old = torch.cat(lps), torch.cat(olds).float()
    ppo_kl = PU.compute_gspo_kl(lps, olds, lps, masks_dev) if est == "gspo" else old - lp
    if est == "sapo":
        pg_loss, pg_clipfrac = PU.compute_sapo_loss(ppo_kl, adv, args.sapo_tau_pos, args.sapo_tau_neg)
    elif est == "cispo":
        pg_loss, pg_clipfrac = PU.compute_cispo_loss(lp, ppo_kl, adv, args.eps_clip, args.eps_clip_high)
    elif est == "rloo":
        pg_loss, pg_clipfrac = PU.compute_rloo_loss(lp, adv)
    elif est in ("grpo", "gspo", "ppo") or pp:
        pg_loss, pg_clipfrac = PU.compute_policy_loss(ppo_kl, adv, args.eps_clip, args.eps_clip_high)
    else:
        raise NotImplementedError(f"advantage_estimator {est} is not supported. ")
    if getattr(args, "use_opsm", False):
        pg_loss = pg_loss * opsm_mask

    mismatch = bool(getattr(args, "get_mismatch_metrics", False) or getattr(args, "use_tis", False))
    tis_metrics, metric_reduce = None, reduce
    pg_masks = masks
    if mismatch:
        assert "rollout_log_probs" in batch, "rollout_log_probs must be provided for TIS"
        ois = (-ppo_kl).exp()
        train = [x.detach() for x in lps] if true_on_policy else [x.to(dev) for x in batch["log_probs"]]
        path = getattr(args, "custom_tis_function_path", None)
        tis_func = load_function(path) if path is not None else vanilla_tis_function
        pg_loss, pg_masks, tis_metrics = tis_func(
            args=args, pg_loss=pg_loss, train_log_probs=train,
            rollout_log_probs=[x.to(dev) for x in batch["rollout_log_probs"]], loss_masks=masks_dev,
            total_lengths=total_lengths, response_lengths=response_lengths)
        reduce = reducer_for(pg_masks)  # rejection masks change the numerators; denominators stay per logical sample
    path = getattr(args, "custom_pg_loss_reducer_function_path", None)
    if path is not None:
        pg_reduce = load_function(path)(total_lengths, response_lengths, pg_masks, per_token)
        if pp:
            pg_reduce = _mask_safe(pg_reduce, pg_masks)
    else:
        pg_reduce = reduce

    pg_loss = pg_reduce(pg_loss)
    pg_clipfrac = reduce(pg_clipfrac)
    kl_metric = reduce(ppo_kl)
    entropy_loss = reduce(torch.cat(out["entropy"], dim=0))
    loss = pg_loss - args.entropy_coef * entropy_loss
    use_kl = bool(getattr(args, "use_kl_loss", False))
    if use_kl:
        ref = torch.cat([x.to(dev) for x in batch["ref_log_probs"]], dim=0).float()
        ratio = torch.exp(lp - old) if getattr(args, "use_unbiased_kl", False) else None
        kl_loss = reduce(PU.compute_approx_kl(lp, ref, args.kl_loss_type, ratio))
        loss = loss + args.kl_loss_coef * kl_loss
    opd_loss, opd_reported = compute_policy_opd_loss(args=args, batch=batch, log_probs=lp, old_log_probs=old,
                                                     log_probs_and_entropy=out)
    if opd_loss is not None:
        loss = loss + opd_loss
    if lp.numel() == 0:
        loss = loss + 0 * logits.sum()

    reported = {"loss": loss.clone().detach(), "pg_loss": pg_loss.clone().detach(),
                "entropy_loss": entropy_loss.clone().detach(), "pg_clipfrac": pg_clipfrac.clone().detach(),
                "ppo_kl": kl_metric.clone().detach()}
    reported.update(opd_reported)
    if batch.get("rollout_log_probs") is not None:
        rollout = torch.cat([x.to(dev) for x in batch["rollout_log_probs"]], dim=0).float()
        if not args.use_rollout_logprobs:
            side = old
        elif batch.get("log_probs"):
            side = torch.cat([x.to(dev) for x in batch["log_probs"]], dim=0).float()
        else:
            side = lp.detach()
        reported["train_rollout_logprob_abs_diff"] = reduce((side - rollout).abs()).clone().detach()
        reported["train_rollout_prob_abs_diff"] = reduce((side.exp() - rollout.exp()).abs()).clone().detach()
    if use_kl:
        reported["kl_loss"] = kl_loss.clone().detach()
    if tis_metrics is not None:
        reported["ois"] = metric_reduce(ois).clone().detach()
        for k, v in tis_metrics.items():
            reported[k] = metric_reduce(v)  # over the tokens valid before any rejection (loss.py:1007-1014)
    if getattr(args, "use_opsm", False):
        reported["opsm_clipfrac"] = opsm_clipfrac
    return loss, reported


def policy_loss_function(args: Namespace, batch: dict, logits: torch.Tensor, sum_of_sample_mean=None):
    """Fused counterpart of loss.py:824-1185.  Returns ``(loss, metrics)`` with the reference's metric keys.

    ``sum_of_sample_mean`` is accepted for signature compatibility; the same reduction (per-sample masked mean with
    ``sample_index_mask_sums`` denominators, or the masked token sum when ``args.calculate_per_token_loss``) is
    evaluated inside the kernel from ``batch``.  A caller-specific reducer can be passed as
    ``batch["relax_amd_sample_denominators"]`` (per-sample divisors) or, for pg_loss only,
    ``batch["relax_amd_pg_sample_denominators"]``.  With ``args.custom_tis_function_path`` or
    ``args.custom_pg_loss_reducer_function_path`` set, the loss is composed step by step around the user's callables
    (``_composed_policy_loss_function``) instead of being evaluated inside one kernel.
    """
    flat = _check_logits(logits, args, batch.get("max_seq_lens"))
    dev = flat.device
    est = args.advantage_estimator
    response_lengths, total_lengths = batch["response_lengths"], batch["total_lengths"]
    if getattr(args, "custom_tis_function_path", None) is not None:
        return _composed_policy_loss_function(args, batch, logits, None)  # user code acts on per-token tensors
    hook_pg_denom = None
    reducer_path = getattr(args, "custom_pg_loss_reducer_function_path", None)
    if reducer_path is not None:
        # the built-in importance weights leave the loss masks as they are, so the masks the reference hands the
        # hook (loss.py:1065) are the batch's own in every case that reaches this point
        hook_reducer = load_function(reducer_path)(total_lengths, response_lengths, batch["loss_masks"],
                                                   bool(getattr(args, "calculate_per_token_loss", False)))
        if not isinstance(hook_reducer, PerSampleDivisorReducer):
            return _composed_policy_loss_function(args, batch, logits, None)  # an opaque callable: [N] tensors
        hook_pg_denom = hook_reducer.sample_divisors
    needs_bwd = torch.is_grad_enabled() and logits.requires_grad
    lay = PackedLayout(dev, flat.size(0), batch["unconcat_tokens"], total_lengths, response_lengths, needs_bwd,
                       _padded_starts(args, batch.get("max_seq_lens")))

    true_on_policy = getattr(args, "true_on_policy_mode", False)
    use_rollout = getattr(args, "use_rollout_logprobs", False)
    use_kl = bool(getattr(args, "use_kl_loss", False))
    mismatch = bool(getattr(args, "get_mismatch_metrics", False) or getattr(args, "use_tis", False))
    if mismatch:
        assert "rollout_log_probs" in batch, "rollout_log_probs must be provided for TIS"
    # the batch's per-sample lists, packed (one concatenation for all of them where their form allows)
    cat = _cat_fields_f32(
        dev, lay.n_tokens,
        old=None if true_on_policy else (batch["rollout_log_probs"] if use_rollout else batch["log_probs"]),
        rollout=batch.get("rollout_log_probs") if not (use_rollout and not true_on_policy) else None,
        ref=batch["ref_log_probs"] if use_kl else None, advantages=batch["advantages"], masks=batch["loss_masks"])
    old = cat["old"]
    rollout = cat["rollout"] if not (use_rollout and not true_on_policy) else old
    # train-engine log-probs: batch["log_probs"], or this step's own forward (kernel default) in true on-policy mode
    if true_on_policy or not batch.get("log_probs"):
        train = None
    else:  # the same packed vector as `old` unless that one holds the rollout engine's log-probs
        train = old if (old is not None and not use_rollout) else _cat_f32(batch["log_probs"], dev)
    # which log-probs the |train - rollout| metrics compare (loss.py:1125-1130): 1 = old, 0 = train, 2 = current
    if not use_rollout:
        abs_from = 2 if true_on_policy else 1
    else:
        abs_from = 0 if train is not None else 2
    masks = cat["masks"]
    per_token = bool(getattr(args, "calculate_per_token_loss", False))
    denom = batch.get("relax_amd_sample_denominators")
    if denom is None and not per_token:
        denom = sample_denominators(batch["loss_masks"], lay, batch.get("sample_index_mask_sums"))
    pg_denom = hook_pg_denom if hook_pg_denom is not None else batch.get("relax_amd_pg_sample_denominators")
    kw = dict(
        old_log_prob=old,
        ref_log_prob=cat["ref"],
        train_log_prob=train,
        rollout_log_prob=rollout,
        advantages=cat["advantages"],
        loss_mask=masks,
        sample_denom=None if denom is None else denom.to(device=dev, dtype=torch.float32),
        pg_sample_denom=None if pg_denom is None else pg_denom.to(device=dev, dtype=torch.float32),
        # REINFORCE++ trains with the PPO-clip surrogate; its mask-safe reduction is what the kernel does anyway
        loss_kind={"grpo": "ppo", "ppo": "ppo", "reinforce_plus_plus": "ppo",
                   "reinforce_plus_plus_baseline": "ppo"}.get(est, est),
        kl_kind=args.kl_loss_type if use_kl else None,
        unbiased_kl=bool(getattr(args, "use_unbiased_kl", False)) and use_kl,
        use_opsm=bool(getattr(args, "use_opsm", False)),
        use_tis=bool(getattr(args, "use_tis", False)) or bool(getattr(args, "get_mismatch_metrics", False)),
        mismatch_metrics=mismatch,
        abs_diff_from_old=abs_from,
        eps_clip=args.eps_clip,
        eps_clip_high=args.eps_clip_high,
        entropy_coef=float(getattr(args, "entropy_coef", 0.0)),
        kl_coef=float(getattr(args, "kl_loss_coef", 0.0)) if use_kl else 0.0,
        tis_lo=float(getattr(args, "tis_clip_low", 0.0)),
        tis_hi=float(getattr(args, "tis_clip", 2.0)),
        opsm_delta=float(getattr(args, "opsm_delta", 1e-4)),
        tau_pos=float(getattr(args, "sapo_tau_pos", 1.0)),
        tau_neg=float(getattr(args, "sapo_tau_neg", 1.05)),
    )
    if kw["loss_kind"] not in ("ppo", "gspo", "cispo", "rloo", "sapo"):
        raise NotImplementedError(f"advantage_estimator {est} is not supported. ")
    inv_t = 1.0 / float(getattr(args, "rollout_temperature", 1.0))
    if lay.n_tokens == 0:
        loss = 0 * logits.sum()
        zero = loss.detach().to(torch.float32)
        metrics = {k: zero.clone() for k in ("loss", "pg_loss", "entropy_loss", "pg_clipfrac", "ppo_kl")}
        if use_kl:
            metrics["kl_loss"] = zero.clone()
        return loss, metrics
    opd_on = float(getattr(args, "opd_loss_coef", 0.0) or 0.0) != 0.0
    opd_gather = None
    if opd_on:
        from .opd_utils import compute_policy_opd_loss, resolve_opd_gather_topk_token_ids

        opd_gather = resolve_opd_gather_topk_token_ids(args, batch)
    # a sampled-token distillation term needs nothing but this step's log-probs: it is built on the two-launch
    # function's output, and its gradient joins the policy loss's before the single dlogits launch
    # the same holds for the top-K selections: the log-probs at the given ids are K loads per row next to the row's
    # log-sum-exp, and their gradient is a multiple of the softmax plus K sparse additions
    opd_on_lp = opd_on and needs_bwd
    topk_widths = None
    if opd_on_lp:
        kw["lp_requires_grad"] = True
        if opd_gather is not None:
            kw["gather_topk_ids"], topk_widths = _pack_topk_ids(flat, lay, opd_gather)
    opd_in_kernel = topk_in_kernel = None
    if opd_on_lp and opd_gather is None and _single_pass_ok(args, flat, kw, needs_bwd):
        opd_in_kernel = _sampled_opd_kernel_args(args, batch, kw["loss_mask"], dev)
    elif opd_on_lp and _single_pass_ok(args, flat, kw, needs_bwd):
        topk_in_kernel = _topk_opd_kernel_args(args, batch, lay, kw.get("gather_topk_ids"), topk_widths,
                                               kw["loss_mask"], dev)
    topk_kl = None
    if topk_in_kernel is not None:
        # the top-K term as well: the kernel gathers the K logits of each row next to its log-sum-exp, evaluates the
        # per-token KL and its derivative, and folds the gradient into the one dlogits launch (plus K sparse additions)
        kw1 = {k: v for k, v in kw.items() if k not in ("lp_requires_grad", "gather_topk_ids")}
        loss, mvec, lp, ent, topk_kl = _SinglePassPolicyLoss.apply(flat, lay, inv_t, dict(kw1, **topk_in_kernel),
                                                                   expected_grad_scale(batch))
        topk_lp = None
    elif opd_in_kernel is not None:
        # the sampled-token term's gradient w.r.t. each log-prob is a per-token weight times the signal's derivative,
        # which the kernel evaluates next to the policy loss's: one launch; the term's value and metrics follow from
        # the launch's log-probs on [N] vectors
        kw.pop("lp_requires_grad", None)
        loss, mvec, lp, ent, _ = _SinglePassPolicyLoss.apply(flat, lay, inv_t, dict(kw, **opd_in_kernel[0]),
                                                             expected_grad_scale(batch))
        topk_lp = None
    elif not opd_on_lp and _single_pass_ok(args, flat, kw, needs_bwd):
        loss, mvec, lp, ent, _ = _SinglePassPolicyLoss.apply(flat, lay, inv_t, kw, expected_grad_scale(batch))
        topk_lp = None
    else:
        loss, mvec, lp, ent, topk_lp = _FusedPolicyLoss.apply(flat, lay, inv_t, kw)

    def m(name):
        return mvec[_SLOT[name]]

    opd_reported = {}
    loss_metric = m("loss")
    if topk_kl is not None:
        from .opd_utils import finish_policy_opd_loss

        with torch.no_grad():
            opd_value, opd_reported = finish_policy_opd_loss(args, batch, topk_kl, lp, old if old is not None else lp)
        loss = loss + opd_value
        loss_metric = loss.detach().clone()
    elif opd_in_kernel is not None:
        with torch.no_grad():
            if "distill" in opd_in_kernel[0]:
                opd_value, opd_reported = compute_policy_opd_loss(
                    args=args, batch=batch, log_probs=lp, old_log_probs=old if old is not None else lp,
                    log_probs_and_entropy={})
            else:  # plain reverse_kl: the term is the weighted sum of lp - teacher, and reports nothing of its own
                opd_value = (opd_in_kernel[0]["extra_coef_log_prob"] * (lp - opd_in_kernel[1])).sum()
        loss = loss + opd_value
        loss_metric = loss.detach().clone()
    elif opd_on:
        # The distillation term (loss.py:1102-1110) needs log-probs that autograd can see: the two-launch function's
        # own outputs when a gradient is wanted, a separate log-prob launch (with the top-K gather) otherwise.
        if opd_on_lp:
            lpe = {"log_probs": lay.split(lp)}
            if opd_gather is not None:
                lpe["topk_log_probs"] = _trim_topk(topk_lp if kw.get("gather_topk_ids") is not None else None, flat,
                                                   lay, topk_widths)
            opd_lp = lp
        else:
            _, lpe = get_log_probs_and_entropy(
                logits, args=args, unconcat_tokens=batch["unconcat_tokens"], total_lengths=total_lengths,
                response_lengths=response_lengths, with_entropy=False, max_seq_lens=batch.get("max_seq_lens"),
                gather_topk_token_ids=opd_gather)
            opd_lp = torch.cat(lpe["log_probs"])
        old_for_opd = old if old is not None else lp.detach()
        opd_loss, opd_reported = compute_policy_opd_loss(
            args=args, batch=batch, log_probs=opd_lp, old_log_probs=old_for_opd, log_probs_and_entropy=lpe)
        if opd_loss is not None:
            loss = loss + opd_loss
            loss_metric = loss.detach().clone()

    reported = {
        "loss": loss_metric,
        "pg_loss": m("pg_loss"),
        "entropy_loss": m("entropy_loss"),
        "pg_clipfrac": m("pg_clipfrac"),
        "ppo_kl": m("ppo_kl"),
    }
    if rollout is not None:
        reported["train_rollout_logprob_abs_diff"] = m("train_rollout_logprob_abs_diff")
        reported["train_rollout_prob_abs_diff"] = m("train_rollout_prob_abs_diff")
    if use_kl:
        reported["kl_loss"] = m("kl_loss")
    if mismatch:
        for k in ("ois", "tis", "tis_clipfrac", "tis_abs", "mismatch_kl", "mismatch_k3_kl"):
            reported[k] = m(k)
    reported.update(opd_reported)
    if kw["use_opsm"]:
        reported["opsm_clipfrac"] = m("opsm_clipfrac")
    return loss, reported


def get_values(logits: torch.Tensor, *, args: Namespace, unconcat_tokens, total_lengths, response_lengths,
               with_entropy: bool = False, non_loss_data: bool = True, max_seq_lens=None, padded_total_lengths=None,
               **_: Any):
    """Counterpart of loss.py:466-518: the value head's output ``[1, T, 1]`` at every response token, as per-sample
    ``[R_i]`` views of one packed gather (the same row map as the log-prob path; no temperature), differentiable
    w.r.t. ``logits``.  Returns ``(empty, {"values": [...]})``."""
    assert logits.dim() == 3 and logits.size(-1) == 1, f"{logits.shape}"
    padded = _padded_starts(args, max_seq_lens)
    assert logits.size(0) == 1 or padded is not None, f"{logits.shape}"
    flat = logits.reshape(-1)
    lay = PackedLayout(flat.device, flat.size(0), unconcat_tokens, total_lengths, response_lengths, False, padded)
    values = flat.index_select(0, lay.row_ids.to(torch.int64)) if lay.n_tokens else flat[:0]
    return torch.empty((0,), device=flat.device), {"values": lay.split(values)}


def value_loss_function(args: Namespace, batch: dict, logits: torch.Tensor, sum_of_sample_mean=None):
    """Counterpart of loss.py:1188-1244: PPO's clipped value loss ``max((v_clipped - R)^2, (v - R)^2)`` with
    ``v_clipped = v_old + clamp(v - v_old, +-value_clip)``, reduced like the policy loss; metrics ``value_loss`` and
    ``value_clipfrac``.  The work is ``[N]``-sized (one value per response token); the reduction is the masked
    per-sample kernel behind ``get_sum_of_sample_mean`` when no reducer is passed in."""
    dev = logits.device
    old_values = _cat_f32(batch["values"], dev)
    _, out = get_values(logits, args=args, unconcat_tokens=batch["unconcat_tokens"],
                        total_lengths=batch["total_lengths"], response_lengths=batch["response_lengths"],
                        max_seq_lens=batch.get("max_seq_lens"), padded_total_lengths=batch.get("padded_total_lengths"))
    values = torch.cat([v.flatten() for v in out["values"]], dim=0)
    returns = _cat_f32(batch["returns"], dev)
    if sum_of_sample_mean is None:
        sum_of_sample_mean = get_sum_of_sample_mean(
            batch["total_lengths"], batch["response_lengths"], [m.to(dev) for m in batch["loss_masks"]],
            bool(getattr(args, "calculate_per_token_loss", False)), sample_denoms=batch.get("sample_index_mask_sums"))
    clip = float(args.value_clip)
    clipfrac = torch.abs(values - old_values) > clip
    clipped = old_values + (values - old_values).clamp(-clip, clip)
    loss = torch.max((clipped - returns) ** 2, (values - returns) ** 2)
    loss = sum_of_sample_mean(loss)
    clipfrac = sum_of_sample_mean(clipfrac.float())
    if values.numel() == 0:
        loss = loss + 0 * values.sum()
    return loss, {"value_loss": loss.clone().detach(), "value_clipfrac": clipfrac.clone().detach()}


def mtp_only_loss_function(args: Namespace, batch: dict, hidden_states: torch.Tensor, sum_of_sample_mean=None):
    """loss.py:1431-1440: no language loss of its own; a zero that keeps the graph (and the multi-token-prediction
    auxiliary loss attached to it) alive."""
    del args, batch, sum_of_sample_mean
    loss = 0.0 * hidden_states.sum()
    return loss, {"loss": loss.detach()}


def _upstream_scale_hint(args, batch, num_microbatches, dp_world_size):
    """The gradient the loss returned by ``loss_function``'s inner function will receive in backward, as far as it
    is known on the host: this function's own factor (loss.py:1572-1586: ``__loss_scale__``, or
    ``num_microbatches / global_batch_size * dp_world_size``; none in per-token mode) times the factor the training
    schedule applies to the returned loss before ``backward()``.  The latter is ``args.relax_amd_schedule_loss_scale``
    when set; otherwise ``1 / num_microbatches`` in sample-mean mode (Megatron's ``forward_step_calc_loss`` divides
    the loss by the returned normalizer, 1, and by the number of micro-batches) and 1 in per-token mode (Megatron
    normalises the gradients by the token count later).  None when unknown without a device read; a wrong value
    costs one rescaling pass in backward, never correctness."""
    if batch.get("__is_dummy__", False):
        return None
    per_token = bool(getattr(args, "calculate_per_token_loss", False))
    own = 1.0
    if not per_token:
        explicit = batch.get("__loss_scale__", None)
        if explicit is not None:
            if isinstance(explicit, torch.Tensor):
                if explicit.is_cuda or explicit.numel() != 1:
                    return None
                explicit = explicit.item()
            own = float(explicit)
        else:
            gbs = batch.get("dynamic_global_batch_size", getattr(args, "global_batch_size", 1))
            if isinstance(gbs, torch.Tensor):
                if gbs.is_cuda:
                    return None
                gbs = gbs.item()
            own = float(num_microbatches) / float(gbs) * float(dp_world_size)
    schedule = getattr(args, "relax_amd_schedule_loss_scale", None)
    if schedule is None:
        schedule = 1.0 if per_token else 1.0 / max(int(num_microbatches), 1)
    return own * float(schedule)


def loss_function(args: Namespace, batch: dict, num_microbatches: int, logits: torch.Tensor, *, lm_head_forward=None,
                  dp_world_size: int = 1):
    """Counterpart of loss.py:1443-1620 on one GPU: token count, the loss selected by ``args.loss_type``
    (``policy_loss``; ``sft``, with the LM head deferred into the loss when ``args.sft_chunked_logits`` and an
    ``lm_head_forward`` are given), Megatron gradient-accumulation scaling, and the ``{"keys", "values"}`` logging
    dict."""
    loss_type = getattr(args, "loss_type", "policy_loss")
    if loss_type not in ("policy_loss", "value_loss", "sft", "custom_loss"):
        raise ValueError(f"Unknown loss type: {loss_type}")
    per_token = bool(getattr(args, "calculate_per_token_loss", False))
    # the micro-batch's token count (loss.py:1504) is what per-token mode returns as its normalizer; in sample-mean
    # mode nothing reads it, and its five small launches are left out
    num_tokens = None
    if per_token:
        num_tokens = get_cp_local_num_tokens(batch["total_lengths"], batch["response_lengths"], batch["loss_masks"])
    reducer = None
    if getattr(args, "mtp_only_training", False):
        func = mtp_only_loss_function
    elif loss_type == "policy_loss":
        func = policy_loss_function
    elif loss_type == "value_loss":
        func = value_loss_function
    elif loss_type == "custom_loss":  # loss.py:1530-1531: the plug-in gets the reducer the built-in losses use
        reducer = get_sum_of_sample_mean(batch["total_lengths"], batch["response_lengths"], batch["loss_masks"],
                                         bool(getattr(args, "calculate_per_token_loss", False)),
                                         sample_denoms=batch.get("sample_index_mask_sums"))
        func = load_function(args.custom_loss_function_path)
    elif getattr(args, "task_type", "causal_lm") == "seq_cls":
        raise NotImplementedError("sequence-classification SFT is outside the fused policy path")
    elif getattr(args, "sft_chunked_logits", False) and lm_head_forward is not None:
        from functools import partial

        func = partial(sft_loss_function_chunked, lm_head_forward=lm_head_forward)
    else:
        func = sft_loss_function
    hint = _upstream_scale_hint(args, batch, num_microbatches, dp_world_size)
    if hint is not None and func in (policy_loss_function, sft_loss_function):
        # the single-launch losses write dlogits during their forward pass, already multiplied by the upstream
        # gradient they expect; telling them the scale applied below saves a rescaling pass over dlogits in backward
        batch = dict(batch)
        batch[GRAD_SCALE_KEY] = hint
    if getattr(args, "recompute_loss_function", False):
        # loss.py:1535-1543: the loss is evaluated again during backward instead of keeping what it saved
        from torch.utils.checkpoint import checkpoint

        loss, log = checkpoint(func, args, batch, logits, reducer,
                               use_reentrant=getattr(args, "recompute_loss_function_use_reentrant", True))
    else:
        loss, log = func(args, batch, logits, reducer)
    is_dummy = batch.get("__is_dummy__", False)
    explicit = batch.get("__loss_scale__", None)
    gbs = batch.get("dynamic_global_batch_size", getattr(args, "global_batch_size", 1))
    if is_dummy:
        loss = 0.0 * loss
    elif not per_token:
        if explicit is not None:
            loss = loss * explicit
        elif all(isinstance(x, (int, float)) for x in (num_microbatches, gbs, dp_world_size)):
            # loss.py:1567 multiplies and divides step by step; with plain numbers the factor is formed on the host and
            # applied once (one launch forward, one backward, instead of three each; the value may differ from the
            # step-by-step one in the last bit)
            loss = loss * (num_microbatches / gbs * dp_world_size)
        else:
            loss = loss * num_microbatches / gbs * dp_world_size
    zero_count = torch.zeros((), dtype=torch.float32, device=logits.device)
    if per_token:
        effective = torch.zeros_like(num_tokens) if is_dummy else num_tokens
        denominator = effective.to(torch.float32)
    else:
        denominator = zero_count
    values = torch.stack([denominator] + [v.to(torch.float32) for v in log.values()])
    if is_dummy:
        values = torch.zeros_like(values)
    normalizer = effective if per_token else torch.ones((), dtype=torch.int64, device=logits.device)  # no host copy
    return loss, normalizer, {"keys": list(log.keys()), "values": values}


# ------------------------------------------------------------------------------------------------- advantages


def compute_advantages_and_returns(args: Namespace, rollout_data: dict) -> None:
    """Counterpart of loss.py:532-738 on one GPU.  GRPO family: broadcast the (already group-normalised) per-sample
    rewards over each response.  ``ppo``: token rewards ``-kl_coef * kl`` (+ the sequence reward on the last token)
    through GAE.  ``reinforce_plus_plus``: discounted returns; ``reinforce_plus_plus_baseline``: masked broadcast.
    With ``args.normalize_advantages`` the advantages are whitened (REINFORCE++: population-normalised, with the
    reference's ``reinforce_pp_*`` statistics) across the micro-batch.  Writes ``advantages`` / ``returns`` in place."""
    from .distributed_utils import distributed_masked_normalize, distributed_masked_whiten
    from .ppo_utils import (compute_approx_kl, get_advantages_and_returns_batch,
                            get_reinforce_plus_plus_baseline_advantages, get_reinforce_plus_plus_returns)

    log_probs = rollout_data.get("rollout_log_probs" if getattr(args, "use_rollout_logprobs", False) else "log_probs")
    ref_log_probs = rollout_data.get("ref_log_probs")
    values = rollout_data.get("values")
    rewards = rollout_data.get("rewards")
    loss_masks = rollout_data.get("loss_masks")
    est = args.advantage_estimator
    if est not in GRPO_FAMILY + ("ppo", "reinforce_plus_plus", "reinforce_plus_plus_baseline"):
        raise NotImplementedError(f"advantage_estimator {est} is not supported. ")
    xs = log_probs if log_probs is not None else values
    if xs is None:
        return
    dev = xs[0].device
    kl_coef = float(getattr(args, "kl_coef", 0.0) or 0.0)
    if kl_coef == 0 or not log_probs:
        # kl only supplies shape / dtype / device here (loss.py:574-577)
        kl = [torch.zeros(x.shape, dtype=torch.float32, device=dev) for x in xs]
    else:
        lens = [int(x.numel()) for x in log_probs]
        flat = compute_approx_kl(torch.cat([x.reshape(-1) for x in log_probs]),
                                 torch.cat([x.reshape(-1) for x in ref_log_probs]).to(dev),
                                 kl_loss_type=args.kl_loss_type)
        kl = list(torch.split(flat, lens))
    if est in GRPO_FAMILY:
        rw = torch.tensor(rewards, dtype=torch.float32, device=dev)
        returns = get_grpo_returns(rw, kl)
        advantages = list(returns)
    elif est == "ppo":
        token_rewards = []
        for reward, k in zip(rewards, kl, strict=False):
            k = k * (-kl_coef)
            k[-1] += reward
            token_rewards.append(k)
        advantages, returns = get_advantages_and_returns_batch(
            rollout_data.get("total_lengths"), rollout_data.get("response_lengths"), values, token_rewards,
            args.gamma, args.lambd)
    elif est == "reinforce_plus_plus":
        rw = torch.tensor(rewards, dtype=torch.float32, device=dev)
        returns = get_reinforce_plus_plus_returns(
            rewards=rw, kl=kl, loss_masks=loss_masks, response_lengths=rollout_data.get("response_lengths"),
            total_lengths=rollout_data.get("total_lengths"), kl_coef=kl_coef, gamma=args.gamma)
        advantages = list(returns)
    else:
        rw = torch.tensor(rewards, dtype=torch.float32, device=dev)
        advantages = get_reinforce_plus_plus_baseline_advantages(rewards=rw, kl=kl, loss_masks=loss_masks)
        returns = advantages
    if getattr(args, "use_opd", False):
        from .opd_utils import apply_opd_to_advantages

        if getattr(args, "opd_only_reward", False):  # pure distillation: drop every non-OPD contribution first
            advantages = [torch.zeros_like(a) for a in advantages]
            returns = [torch.zeros_like(r) for r in returns]
        advantages = list(advantages)
        apply_opd_to_advantages(args, rollout_data, advantages)
    if getattr(args, "normalize_advantages", False):
        flat = torch.cat(advantages)
        masks = torch.cat(loss_masks).to(dev)
        assert flat.size() == masks.size(), f"Shape mismatch before whitening: advantages {flat.size()}, masks {masks.size()}"
        is_rpp = est in ("reinforce_plus_plus", "reinforce_plus_plus_baseline")
        if is_rpp or masks.numel() > 0:
            if is_rpp:
                white, raw_mean, raw_var, count = distributed_masked_normalize(flat, masks, process_group=None)
                floor = torch.tensor(1e-8, device=dev, dtype=raw_var.dtype)
                norm_var = raw_var / torch.maximum(raw_var, floor)
                k = len(advantages)
                rollout_data["reinforce_pp_advantage_raw_mean"] = [raw_mean.detach()] * k
                rollout_data["reinforce_pp_advantage_raw_std"] = [raw_var.sqrt().detach()] * k
                rollout_data["reinforce_pp_advantage_normalized_mean"] = [torch.zeros_like(raw_mean)] * k
                rollout_data["reinforce_pp_advantage_normalized_std"] = [norm_var.sqrt().detach()] * k
                rollout_data["reinforce_pp_valid_token_count"] = [count.detach()] * k
                rollout_data["reinforce_pp_zero_variance"] = [(raw_var == 0).to(dtype=raw_var.dtype).detach()] * k
            else:
                white = distributed_masked_whiten(flat, masks, process_group=None, shift_mean=True)
            advantages = list(torch.split(white, [a.size(0) for a in advantages]))
    rollout_data["advantages"] = advantages
    rollout_data["returns"] = returns
