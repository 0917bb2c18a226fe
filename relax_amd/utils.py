"""Drop-in counterpart of ``post_process_rewards`` (relax/utils/utils.py:180-240): group mean/std (GRPO family) and
leave-one-out (RLOO) reward normalisation by ``group_index``, computed by the gfx950 group-reward kernel."""

from __future__ import annotations

from typing import Any

import torch

from . import ops

_GROUP_NORM = ("grpo", "gspo", "sapo", "cispo", "reinforce_plus_plus_baseline", "rloo")
_STD_NORM = ("grpo", "gspo", "sapo", "cispo")


def post_process_rewards(args: Any, samples: list, device=None):
    """Returns ``(raw_rewards, normalised_rewards)`` as Python float lists in input order.

    ``samples`` are duck-typed: ``.group_index`` and ``.get_reward_value(args)``.  Error behaviour follows the
    reference: missing group index, wrong group size and (RLOO) non-finite rewards raise ``ValueError``.
    """
    if getattr(args, "custom_reward_post_process_path", None) is not None:
        # relax/utils/utils.py:186-192: the user's function decides; a 2-tuple is (raw, processed), anything else is
        # the processed rewards alone
        from .loss import load_function

        processed = load_function(args.custom_reward_post_process_path)(args, samples)
        if isinstance(processed, tuple) and len(processed) == 2:
            return processed
        return [s.get_reward_value(args) for s in samples], processed
    raw = [s.get_reward_value(args) for s in samples]
    if getattr(args, "agentic_custom_advantage_path", None) is not None:
        return raw, [s.custom_advantage for s in samples]
    if not (args.advantage_estimator in _GROUP_NORM and args.rewards_normalization):
        return raw, raw
    groups = []
    for s in samples:
        if s.group_index is None:
            raise ValueError("Sample.group_index is required for group reward normalization.")
        groups.append(int(s.group_index))
    if args.advantage_estimator == "rloo":
        mode = "rloo"
    elif args.advantage_estimator in _STD_NORM and args.grpo_std_normalization:
        mode = "center_std"
    else:
        mode = "center"
    dev = torch.device(device if device is not None else "cuda")
    r = torch.tensor(raw, dtype=torch.float).to(dev)
    g = torch.tensor(groups, dtype=torch.int32).to(dev)
    out, counts = ops.group_rewards(r, g, mode)
    counts = counts.tolist()
    seen = set()
    for pos, (gi, c) in enumerate(zip(groups, counts)):
        if gi in seen:
            continue
        seen.add(gi)
        if c != args.n_samples_per_prompt:
            raise ValueError(f"Reward group {gi} has {c} samples, expected {args.n_samples_per_prompt}.")
        if mode == "rloo":
            if c < 2:
                raise ValueError(f"RLOO requires n_samples_per_prompt >= 2 (group size {c} makes the leave-one-out baseline undefined: division by G-1=0).")
            positions = [p for p, gg in enumerate(groups) if gg == gi]
            bad = [p for p in positions if not torch.isfinite(torch.tensor(raw[p]))]
            if bad:
                raise ValueError(
                    f"RLOO group_index={gi} contains non-finite reward(s) at group position(s) "
                    f"{[positions.index(p) for p in bad]}, sample position(s) {bad}: {[raw[p] for p in bad]}."
                )
    return raw, out.tolist()
