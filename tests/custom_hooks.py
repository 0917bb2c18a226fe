"""User-side plug-ins for the tests of the dotted-path hooks (``--custom-tis-function-path``,
``--custom-pg-loss-reducer-function-path``, ``--custom-loss-function-path``): plain tensor code of the kind a user of
the reference writes, with the reference's plug-in signatures (relax/backends/megatron/loss.py:1026-1040, 1062-1072,
1530-1531; ``--custom-reward-post-process-path``: relax/utils/utils.py:186-192)."""

import torch


def rejecting_tis(args, *, pg_loss, train_log_probs, rollout_log_probs, loss_masks, **kwargs):
    """Importance weights clamped to [0.9, 1.1]; tokens whose ratio leaves [0.8, 1.25] are rejected (mask -> 0)."""
    ratio = torch.exp(torch.cat(train_log_probs) - torch.cat(rollout_log_probs))
    keep = ((ratio >= 0.8) & (ratio <= 1.25)).to(pg_loss.dtype)
    lens = [m.numel() for m in loss_masks]
    masks = [m.to(pg_loss.dtype) * k for m, k in zip(loss_masks, torch.split(keep, lens))]
    metrics = {"tis": ratio.detach().clone(), "rejected": (1 - keep).detach()}
    return pg_loss * ratio.clamp(0.9, 1.1), masks, metrics


def token_mean_reducer(total_lengths, response_lengths, loss_masks, calculate_per_token_loss):
    """One global masked token mean (every token weighs the same, whatever its sample's length)."""
    mask = torch.cat([m.reshape(-1).float() for m in loss_masks])

    def reduce(values):
        m = mask.to(values.device)
        return (values * m).sum() / m.sum().clamp_min(1)

    return reduce


def negative_log_likelihood(args, batch, logits, sum_of_sample_mean):
    """A custom loss: plain masked NLL through the library's differentiable log-prob entry point."""
    import relax_amd

    _, out = relax_amd.get_log_probs_and_entropy(
        logits, args=args, unconcat_tokens=batch["unconcat_tokens"], total_lengths=batch["total_lengths"],
        response_lengths=batch["response_lengths"], with_entropy=False)
    loss = -sum_of_sample_mean(torch.cat(out["log_probs"]))
    return loss, {"loss": loss.clone().detach()}


def halved_rewards(args, samples):
    """A reward post-processor that returns the processed rewards only."""
    return [0.5 * s.get_reward_value(args) for s in samples]


def raw_and_centred_rewards(args, samples):
    """A reward post-processor that returns the (raw, processed) pair itself."""
    raw = [s.get_reward_value(args) for s in samples]
    mean = sum(raw) / len(raw)
    return raw, [r - mean for r in raw]
