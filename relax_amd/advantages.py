"""Counterpart of ``Advantages.compute_advantages_and_returns`` (relax/components/advantages.py:122-232) for the
GRPO estimator family: returns nested tensors of per-sample advantages / returns."""

from __future__ import annotations

from types import SimpleNamespace

import torch

from .loss import compute_advantages_and_returns as _fill


class Advantages:
    """Holds the estimator config; ``compute_advantages_and_returns(rollout_data)`` mirrors the service method."""

    def __init__(self, config):
        self.config = config

    def compute_advantages_and_returns(self, rollout_data: dict):
        cfg = self.config
        if rollout_data.get("log_probs") is None and rollout_data.get("values") is None and \
                rollout_data.get("rollout_log_probs") is None:
            return None
        data = dict(rollout_data)
        if data.get("log_probs") is None and data.get("values") is None:
            data["log_probs"] = data["rollout_log_probs"]  # shape template in true on-policy mode
        args = SimpleNamespace(
            advantage_estimator=cfg.advantage_estimator,
            use_rollout_logprobs=getattr(cfg, "use_rollout_logprobs", False),
            normalize_advantages=False,
        )
        _fill(args, data)
        return {
            "advantages": torch.nested.nested_tensor(data["advantages"]),
            "returns": torch.nested.nested_tensor(data["returns"]),
        }
