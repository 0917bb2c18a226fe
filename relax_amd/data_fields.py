"""Wire formats on either side of the loss / log-prob / advantage path.

Inbound: which fields a training consumer pulls from the rollout data system (``build_data_fields``,
relax/utils/training/data_fields.py:6-82, with the on-policy-distillation schema of
relax/utils/opd/opd_main_worker.py:84-104, 272-278) and how the flat top-K lists that arrive are turned back into
``[R, K]`` tensors (``restore_opd_topk_rollout_fields``, opd_main_worker.py:281-326).

Outbound: per-sample outputs leave as jagged nested tensors on the host
(relax/backends/megatron/actor.py:2351-2363; relax/components/advantages.py:236-239).  The kernels here already
produce every per-token output as one packed ``[N]`` vector plus the ``cu`` offsets of the samples, and the per-sample
lists handed to the caller are views of it, so the packed vector crosses PCIe in one copy and becomes the nested
tensor's ``values`` directly instead of one device-to-host copy per sample.
"""

from __future__ import annotations

from argparse import Namespace

import torch

# on-policy-distillation transfer fields (opd_main_worker.py:84-104)
OPD_SAMPLED_TEACHER_LOG_PROBS = "teacher_log_probs"
OPD_SAMPLED_STUDENT_LOG_PROBS = "rollout_log_probs"
OPD_TOPK_TOKEN_IDS = "opd_topk_token_ids"
OPD_TOPK_TEACHER_LOG_PROBS = "opd_topk_teacher_log_probs"
OPD_TOPK_STUDENT_LOG_PROBS = "opd_topk_student_log_probs"  # only when OPD shapes the advantages
OPD_TOPK_K_LENGTHS = "opd_topk_ksz"  # only for the union selection
_TOPK_SELECTIONS = ("student_topk", "teacher_topk", "union")


def opd_transfer_schema(args: Namespace) -> list[str]:
    """Fields the distillation workers attach to a rollout batch (OpdManager.schema_opd_transfer_data,
    relax/engine/rollout/on_policy_distillation.py:163-169)."""
    selection = getattr(args, "opd_token_selection", "student_sampled")
    if selection == "student_sampled":
        return [OPD_SAMPLED_TEACHER_LOG_PROBS, OPD_SAMPLED_STUDENT_LOG_PROBS]
    if selection not in _TOPK_SELECTIONS:
        raise KeyError(selection)
    fields = [OPD_TOPK_TOKEN_IDS, OPD_TOPK_TEACHER_LOG_PROBS]
    if float(getattr(args, "opd_kl_coef", 0.0) or 0.0) != 0.0:
        fields.append(OPD_TOPK_STUDENT_LOG_PROBS)
    if selection == "union":
        fields.append(OPD_TOPK_K_LENGTHS)
    return fields


def consume_opd_train_data(data_fields: list[str], args: Namespace) -> None:
    """opd_utils.py:916-919: only the sglang teacher ships its fields with the training batch."""
    if getattr(args, "use_opd", False) and getattr(args, "opd_type", None) == "sglang":
        data_fields.extend(opd_transfer_schema(args))


def consume_opd_advantage_data(data_fields: list[str], args: Namespace) -> None:
    """opd_utils.py:922-925."""
    if getattr(args, "use_opd", False):
        data_fields.extend(opd_transfer_schema(args))


def _base_rollout_fields(args: Namespace) -> list[str]:
    fields = ["tokens", "total_lengths", "response_lengths", "loss_masks", "rollout_log_probs", "rewards",
              "sample_indices", "sample_index_mask_sums", "raw_reward", "group_index"]
    if getattr(args, "use_rollout_routing_replay", False):
        fields.append("rollout_routed_experts")
    if getattr(args, "multimodal_keys", None) is not None:
        fields.append("multimodal_train_inputs")
    return fields


def build_data_fields(args: Namespace, *, consumer: str = "actor") -> list[str]:
    """Field names a consumer (``actor``, and for PPO also ``critic`` / ``advantages``) requests for training; same
    lists in the same order as the reference."""
    if getattr(args, "loss_type", None) == "sft":
        fields = ["tokens", "total_lengths", "response_lengths", "loss_masks"]
        if getattr(args, "task_type", "causal_lm") == "seq_cls":
            fields.append("classification_labels")
        if args.multimodal_keys is not None:
            fields.append("multimodal_train_inputs")
        return fields

    ppo = getattr(args, "advantage_estimator", None) == "ppo"
    kl = getattr(args, "kl_coef", 0.0) != 0
    fields = _base_rollout_fields(args)
    if ppo and consumer == "critic":
        return fields
    if ppo and consumer == "advantages":
        fields.append("values")
        if kl:
            if not getattr(args, "use_rollout_logprobs", False) and not getattr(args, "true_on_policy_mode", False):
                fields.append("log_probs")
            fields.append("ref_log_probs")
        consume_opd_train_data(fields, args)
        return fields
    if ppo:
        if getattr(args, "fully_async", False) and not getattr(args, "hybrid", False):
            fields.extend(["advantages", "returns"])
        else:
            fields.append("values")
            if kl:
                fields.append("ref_log_probs")
        if (kl or getattr(args, "use_kl_loss", False)) and "ref_log_probs" not in fields:
            fields.append("ref_log_probs")
    consume_opd_train_data(fields, args)
    return fields


def restore_opd_topk_rollout_fields(rollout_data: dict, args: Namespace, device) -> None:
    """Flat per-sample lists of the top-K fields -> ``[R_i, K]`` tensors on ``device`` (union: ``[R_i, max K']``, the
    width recovered from the response length); the union's per-row K' lists -> int64 tensors.  In place."""
    selection = getattr(args, "opd_token_selection", None)
    top_k = int(getattr(args, "opd_log_prob_top_k", 0) or 0)
    if top_k <= 0 or selection not in _TOPK_SELECTIONS:
        return
    union = selection == "union"
    response_lengths = rollout_data.get("response_lengths", [])
    for key, dtype in ((OPD_TOPK_TOKEN_IDS, torch.long), (OPD_TOPK_TEACHER_LOG_PROBS, torch.float32),
                       (OPD_TOPK_STUDENT_LOG_PROBS, torch.float32)):
        if rollout_data.get(key) is None:
            continue
        restored = []
        for i, flat in enumerate(rollout_data[key]):
            if flat is None:
                restored.append(None)
                continue
            t = torch.as_tensor(flat, device=device, dtype=dtype)
            if union:
                rows = int(response_lengths[i]) if i < len(response_lengths) else 0
                if t.numel() == 0 or rows <= 0:
                    restored.append(t.reshape(0, 1))
                else:
                    restored.append(t.reshape(rows, t.numel() // rows))
            else:
                restored.append(t.reshape(-1, top_k))
        rollout_data[key] = restored
    if union and rollout_data.get(OPD_TOPK_K_LENGTHS) is not None:
        rollout_data[OPD_TOPK_K_LENGTHS] = [
            None if v is None else torch.as_tensor(v, device=device, dtype=torch.long)
            for v in rollout_data[OPD_TOPK_K_LENGTHS]]


def _packed_parent(items: list[torch.Tensor]):
    """(base, first element offset, total elements) when ``items`` are consecutive contiguous 1-D views of one
    tensor (what the loss / log-prob entry points return), else None."""
    if not items or any(t.dim() != 1 or not t.is_contiguous() for t in items):
        return None
    first = items[0]
    base = first._base if first._base is not None else first
    if base.dim() != 1 or not base.is_contiguous():
        return None
    expect = first.storage_offset()
    for t in items:
        tb = t._base if t._base is not None else t
        if tb is not base or t.dtype != base.dtype or t.storage_offset() != expect:
            return None
        expect += t.numel()
    return base, first.storage_offset() - base.storage_offset(), expect - first.storage_offset()


def jagged_to_host(items: list[torch.Tensor]) -> torch.Tensor:
    """Per-sample tensors -> one jagged nested tensor on the host, equal to
    ``torch.nested.as_nested_tensor([t.cpu() for t in items], layout=torch.jagged)`` (actor.py:2356-2360).

    1-D per-sample tensors that are consecutive views of one packed device vector are moved with a single copy; other
    inputs are concatenated on the device first (still one copy across PCIe)."""
    if not items:
        raise ValueError("jagged_to_host needs at least one tensor")
    lengths = [int(t.size(0)) for t in items]
    offsets = torch.zeros(len(items) + 1, dtype=torch.int64)
    torch.cumsum(torch.tensor(lengths, dtype=torch.int64), 0, out=offsets[1:])
    parent = _packed_parent(items)
    if parent is not None:
        base, start, total = parent
        values = base[start:start + total].detach().cpu()
    else:
        values = torch.cat([t.detach() for t in items], dim=0).cpu()
    return torch.nested.nested_tensor_from_jagged(values, offsets)


def to_transfer_payload(output_dict: dict) -> dict:
    """The dict ``_put_data_to_transfer_queue`` wraps into a TensorDict (actor.py:2355-2361): tensors moved to the host,
    per-sample lists turned into jagged nested tensors."""
    return {k: (jagged_to_host(list(v)) if isinstance(v, (list, tuple)) else v.detach().cpu())
            for k, v in output_dict.items()}


def advantages_payload(advantages: list[torch.Tensor], returns: list[torch.Tensor]) -> dict:
    """What the Advantages service returns (advantages.py:236-239): nested tensors of the per-sample vectors, on the
    device they were computed on."""
    return {"advantages": torch.nested.nested_tensor(list(advantages)),
            "returns": torch.nested.nested_tensor(list(returns))}
