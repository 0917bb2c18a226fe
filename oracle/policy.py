"""Oracle: response slicing of packed logits and the policy-loss composition.

Test infrastructure only.  Context-parallel size 1, packed ("thd") layout.
"""

from __future__ import annotations

from types import SimpleNamespace

import torch
import torch.nn.functional as F

from . import losses, reducers
from .logprob import calculate_log_probs_and_entropy

DEFAULT_ARGS = dict(
    advantage_estimator="grpo",
    eps_clip=0.2,
    eps_clip_high=0.2,
    entropy_coef=0.0,
    use_kl_loss=False,
    kl_loss_coef=0.0,
    kl_loss_type="k1",
    use_unbiased_kl=False,
    use_rollout_logprobs=False,
    true_on_policy_mode=False,
    use_opsm=False,
    opsm_delta=1e-4,
    use_tis=False,
    get_mismatch_metrics=False,
    tis_clip=2.0,
    tis_clip_low=0.0,
    sapo_tau_pos=1.0,
    sapo_tau_neg=1.05,
    rollout_temperature=1.0,
    log_probs_chunk_size=-1,
    calculate_per_token_loss=False,
    global_batch_size=1,
    loss_type="policy_loss",
    sft_logits_chunk_size=1024,
    opd_loss_coef=0.0,
    opd_kl_type="reverse_kl",
    opd_jsd_alpha=0.5,
    opd_norm_mode="tail",
    opd_log_prob_min_clamp=None,
    opd_token_selection="sampled",
    opd_per_token_clip=None,
    opd_is_clip=None,
)


def make_args(**kw):
    d = dict(DEFAULT_ARGS)
    d.update(kw)
    return SimpleNamespace(**d)


def response_row_ranges(total_lengths, response_lengths, max_seq_lens=None):
    """Index arithmetic of relax/backends/megatron/loss.py:103-125 (cp_size == 1; packed "thd" layout, or with
    ``max_seq_lens`` the padded "bshd" layout flattened to rows, where sample i begins at max_seq_lens[i] * i).

    Returns per sample (row_begin, row_end, sft) where logits rows [row_begin, row_end) score the response
    tokens.  RL samples use the previous position's logits (start-1 .. end-1); the SFT convention
    (response == total) uses start .. end (relax/utils/sft_utils.py:23-40).
    """
    out = []
    end = 0
    for i, (total, resp) in enumerate(zip(total_lengths, response_lengths, strict=False)):
        end = max_seq_lens[i] * i + total if max_seq_lens is not None else end + total  # :112-117
        start = end - resp
        if resp == total:
            out.append((start, end, True))
        else:
            out.append((start - 1, end - 1, False))
    return out


def iter_responses(logits, tokens_list, total_lengths, response_lengths, temperature=1.0):
    """loss.py:49-191: yields ([R_i,V] logits / T, [R_i] target ids) per sample."""
    assert logits.dim() == 3 and logits.size(0) == 1, f"{logits.shape}"
    flat = logits.squeeze(0)
    for (b, e, sft), toks, resp in zip(
        response_row_ranges(total_lengths, response_lengths), tokens_list, response_lengths, strict=False
    ):
        chunk = flat[b:e]
        targets = F.pad(toks[1:], (0, 1), value=0) if sft else toks[-resp:]
        if temperature != 1.0:
            chunk = chunk / temperature
        yield chunk, targets


def get_log_probs_and_entropy(logits, *, args, unconcat_tokens, total_lengths, response_lengths, with_entropy=False,
                              gather_topk_token_ids=None, **_):
    """loss.py:290-463 without the CP branches; ``gather_topk_token_ids`` adds the per-sample ``topk_log_probs``
    (:440-441, compute_opd_topk_log_probs)."""
    from .opd import log_probs_on_topk_ids

    want_grad = with_entropy and getattr(args, "entropy_coef", 0.0) != 0  # :373
    lps, ents, topk = [], [], []
    for i, (chunk, targets) in enumerate(iter_responses(
        logits, unconcat_tokens, total_lengths, response_lengths, args.rollout_temperature
    )):
        lp, ent = calculate_log_probs_and_entropy(
            chunk,
            targets,
            None,
            with_entropy=with_entropy,
            with_entropy_grad=want_grad,
            chunk_size=args.log_probs_chunk_size,
        )
        lps.append(lp.squeeze(-1))
        ents.append(ent)
        if gather_topk_token_ids is not None:
            ids = gather_topk_token_ids[i] if i < len(gather_topk_token_ids) else None
            if ids is None or ids.numel() == 0:
                topk.append(chunk.new_zeros((chunk.size(0), 0)))
            else:
                topk.append(log_probs_on_topk_ids(chunk, ids))
    res = {"log_probs": lps}
    if with_entropy:
        res["entropy"] = ents
    if gather_topk_token_ids is not None:
        res["topk_log_probs"] = topk
    return torch.empty((0,)), res


def lm_head_log_probs(hidden, weight, targets, temperature=1.0, sub_chunk=1024):
    """Deferred LM head, loss.py:391-419: per sub-chunk logits = h W^T (in weight dtype) -> fp32 -> /T -> log-prob."""
    out = []
    for s in range(0, hidden.size(0), sub_chunk):
        e = min(s + sub_chunk, hidden.size(0))
        lg = F.linear(hidden[s:e].to(weight.dtype), weight).float()
        if temperature != 1.0:
            lg = lg / temperature
        lp, _ = calculate_log_probs_and_entropy(lg, targets[s:e], None, with_entropy=False)
        out.append(lp.squeeze(-1))
    return torch.cat(out, dim=0) if out else hidden.new_zeros((0,), dtype=torch.float32)


def policy_loss_function(args, batch, logits, reducer, pg_reducer=None, tis_fn=None, rebuild_reducer=None,
                         pg_reducer_factory=None):
    """Composition of loss.py:824-1185 (no CP).  Returns (loss, metrics dict).

    Plug-in points: ``tis_fn(pg_loss, train_lp, rollout_lp, masks) -> (pg_loss, masks, metrics)`` stands for
    ``--custom-tis-function-path`` (:1036-1040); when it is given, ``rebuild_reducer(masks)`` builds the reducer used
    after it (:1044-1059) while the importance-sampling metrics keep the original one (:1007-1014);
    ``pg_reducer_factory(masks)`` stands for ``--custom-pg-loss-reducer-function-path`` (:1062-1072)."""
    adv = torch.cat(batch["advantages"], dim=0) if isinstance(batch["advantages"], list) else batch["advantages"]
    resp, tot = batch["response_lengths"], batch["total_lengths"]
    if args.advantage_estimator in ("reinforce_plus_plus", "reinforce_plus_plus_baseline"):
        # loss.py:804-821, 864-865, 1056-1072: every reduction first selects the valid tokens, so a non-finite value
        # at a masked position cannot leak through ``NaN * 0``
        valid = torch.cat([m.reshape(-1) != 0 for m in batch["loss_masks"]], dim=0)

        def _safe(inner):
            return lambda values: inner(torch.where(valid, values, torch.zeros_like(values)))

        reducer = _safe(reducer)
        pg_reducer = _safe(pg_reducer) if pg_reducer is not None else None
    gather = batch.get("opd_topk_token_ids") if getattr(args, "opd_token_selection", None) in (
        "student_topk", "teacher_topk", "union") else None  # resolve_opd_gather_topk_token_ids, opd_utils.py:999-1003
    _, out = get_log_probs_and_entropy(
        logits, args=args, unconcat_tokens=batch["unconcat_tokens"], total_lengths=tot, response_lengths=resp,
        with_entropy=True, gather_topk_token_ids=gather,
    )
    lps = out["log_probs"]
    if args.true_on_policy_mode:
        olds = [x.detach() for x in lps]  # :893-899
    else:
        olds = batch["rollout_log_probs"] if args.use_rollout_logprobs else batch["log_probs"]  # :871

    if args.use_opsm:
        om, opsm_frac = losses.opsm_mask(args.opsm_delta, lps, olds, batch["advantages"], batch["loss_masks"])
    if args.advantage_estimator == "gspo":
        ppo_kl = losses.gspo_seq_kl(lps, olds, batch["loss_masks"])  # :961-967
        old = torch.cat(olds)
        lp = torch.cat(lps)
    else:
        old = torch.cat(olds)
        lp = torch.cat(lps)
        ppo_kl = old - lp  # :974

    est = args.advantage_estimator
    if est == "sapo":
        pg, clipfrac = losses.sapo(ppo_kl, adv, args.sapo_tau_pos, args.sapo_tau_neg)
    elif est == "cispo":
        pg, clipfrac = losses.cispo(lp, ppo_kl, adv, args.eps_clip, args.eps_clip_high)
    elif est == "rloo":
        pg, clipfrac = losses.rloo_loss(lp, adv)
    else:
        pg, clipfrac = losses.policy_clip(ppo_kl, adv, args.eps_clip, args.eps_clip_high)  # :1000
    if args.use_opsm:
        pg = pg * om

    tis_metrics = None
    metric_reducer = reducer
    pg_masks = batch["loss_masks"]
    if args.get_mismatch_metrics or args.use_tis:  # :1006-1059
        ois = (-ppo_kl).exp()
        train_side = torch.cat([x.detach() for x in lps]) if args.true_on_policy_mode else torch.cat(batch["log_probs"])
        if tis_fn is None:
            pg, tis_metrics = losses.vanilla_tis(
                pg, train_side, torch.cat(batch["rollout_log_probs"]), args.tis_clip_low, args.tis_clip
            )
        else:
            pg, pg_masks, tis_metrics = tis_fn(pg, train_side, torch.cat(batch["rollout_log_probs"]), pg_masks)
            reducer = rebuild_reducer(pg_masks)

    if pg_reducer_factory is not None:
        pg_reducer = pg_reducer_factory(pg_masks)
        if args.advantage_estimator in ("reinforce_plus_plus", "reinforce_plus_plus_baseline"):
            pg_reducer = _safe(pg_reducer)  # :1070-1071
    pg_red = pg_reducer if pg_reducer is not None else reducer
    pg_loss = pg_red(pg)
    pg_clipfrac = reducer(clipfrac)
    kl_metric = reducer(ppo_kl)
    ent = torch.cat(out["entropy"], dim=0)
    entropy_loss = reducer(ent)
    loss = pg_loss - args.entropy_coef * entropy_loss  # :1084
    metrics = {}
    if args.use_kl_loss:  # :1086-1100
        ref = torch.cat(batch["ref_log_probs"], dim=0)
        ratio = torch.exp(lp - old) if args.use_unbiased_kl else None
        kl = losses.approx_kl(lp, ref, args.kl_loss_type, ratio)
        kl_loss = reducer(kl)
        loss = loss + args.kl_loss_coef * kl_loss
    from .opd import policy_opd_loss

    opd_loss, opd_metrics = policy_opd_loss(args, batch, lp, old, out.get("topk_log_probs"))  # :1102-1110
    if opd_loss is not None:
        loss = loss + opd_loss
    if lp.numel() == 0:
        loss = loss + 0 * logits.sum()
    metrics.update(
        loss=loss.detach().clone(),
        pg_loss=pg_loss.detach().clone(),
        entropy_loss=entropy_loss.detach().clone(),
        pg_clipfrac=pg_clipfrac.detach().clone(),
        ppo_kl=kl_metric.detach().clone(),
    )
    metrics.update(opd_metrics)
    if batch.get("rollout_log_probs") is not None:  # :1115-1134
        roll = torch.cat(batch["rollout_log_probs"], dim=0)
        if not args.use_rollout_logprobs:
            side = old
        elif batch.get("log_probs"):
            side = torch.cat(batch["log_probs"], dim=0)
        else:
            side = lp.detach()
        metrics["train_rollout_logprob_abs_diff"] = reducer((side - roll).abs()).detach().clone()
        metrics["train_rollout_prob_abs_diff"] = reducer((torch.exp(side) - torch.exp(roll)).abs()).detach().clone()
    if args.use_kl_loss:
        metrics["kl_loss"] = kl_loss.detach().clone()
    if tis_metrics is not None:
        metrics["ois"] = metric_reducer(ois).detach().clone()
        for k, v in tis_metrics.items():
            metrics[k] = metric_reducer(v)
    if args.use_opsm:
        metrics["opsm_clipfrac"] = opsm_frac
    return loss, metrics


def sft_loss_function(args, batch, logits, reducer):
    """loss.py:1247-1293: negative reduced log-probability of the response tokens."""
    _, out = get_log_probs_and_entropy(logits, args=args, unconcat_tokens=batch["unconcat_tokens"],
                                       total_lengths=batch["total_lengths"], response_lengths=batch["response_lengths"])
    log_probs = torch.cat(out["log_probs"], dim=0)
    loss = -reducer(log_probs)
    if log_probs.numel() == 0:
        loss = loss + 0 * logits.sum()
    return loss, {"loss": loss.clone().detach()}


def loss_function(args, batch, num_microbatches, logits, dp_world: int = 1, func=None):
    """Scaling tail of loss.py:1488-1620 at cp = 1: returns (loss, normalizer, {"keys", "values"}).  The loss is
    picked by ``args.loss_type`` (:1515-1533) unless ``func`` is given; dummy micro-batches and an explicit
    ``__loss_scale__`` follow :1565-1586."""
    ntok = reducers.num_tokens(batch["loss_masks"])
    red = reducers.make_reducer(
        batch["response_lengths"], batch["loss_masks"], args.calculate_per_token_loss,
        batch.get("sample_index_mask_sums"),
    )
    if func is None:
        func = {"policy_loss": policy_loss_function, "sft": sft_loss_function,
                "value_loss": value_loss_function}[getattr(args, "loss_type", "policy_loss")]
    loss, log = func(args, batch, logits, red)
    dummy = batch.get("__is_dummy__", False)
    if dummy:
        loss = 0.0 * loss
    elif not args.calculate_per_token_loss:
        explicit = batch.get("__loss_scale__", None)
        if explicit is not None:
            loss = loss * explicit
        else:
            loss = loss * num_microbatches / batch.get("dynamic_global_batch_size", args.global_batch_size) * dp_world
    eff = torch.zeros_like(ntok) if dummy else ntok
    denom = eff if args.calculate_per_token_loss else torch.zeros_like(ntok)
    vals = torch.stack([denom] + [v if isinstance(v, torch.Tensor) else torch.tensor(v) for v in log.values()])
    if dummy:
        vals = torch.zeros_like(vals)
    norm = eff if args.calculate_per_token_loss else torch.tensor(1)
    return loss, norm, {"keys": list(log.keys()), "values": vals}


def get_values(logits, total_lengths, response_lengths):
    """loss.py:466-518: the value head's [1, T, 1] output over each sample's response rows (same slicing as the
    log-prob path, no temperature), squeezed to [R_i]."""
    assert logits.dim() == 3 and logits.size(0) == 1 and logits.size(-1) == 1
    flat = logits.squeeze(0)
    return [flat[b:e].squeeze(-1) for b, e, _sft in response_row_ranges(total_lengths, response_lengths)]


def value_loss_function(args, batch, logits, reducer):
    """loss.py:1188-1244: clipped value loss and its two metrics."""
    old = torch.cat(batch["values"], dim=0)
    values = torch.cat([v.flatten() for v in get_values(logits, batch["total_lengths"], batch["response_lengths"])])
    returns = torch.cat(batch["returns"], dim=0)
    clipfrac = torch.abs(values - old) > args.value_clip
    clipped = old + (values - old).clamp(-args.value_clip, args.value_clip)
    loss = reducer(torch.max((clipped - returns) ** 2, (values - returns) ** 2))
    frac = reducer(clipfrac.float())
    if values.numel() == 0:
        loss = loss + 0 * values.sum()
    return loss, {"value_loss": loss.clone().detach(), "value_clipfrac": frac.clone().detach()}
