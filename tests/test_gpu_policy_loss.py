"""GPU parity of the fused policy loss (custom_loss plug-in signature) against the oracle composition.

fp32 logits: loss / metrics / dlogits within 3e-5; bf16 logits within 2e-3 (the stated bound).  dlogits come back
in the logits dtype, so for bf16 the comparison also allows one bf16 ulp (2^-7 relative) of output rounding: an
element of magnitude ~2 cannot be represented more finely than 0.0078.  Token counts and row maps are exact.
"""

BF16_ULP = 2.0 ** -7

import pytest
import torch

from oracle import policy as P
from oracle import reducers as R
from tests.gpu_util import announce, require_gpu

pytestmark = pytest.mark.gpu


def _make_batch(seed, tot, resp, v, dtype=torch.float32, int_masks=False, sft_sample=None):
    g = torch.Generator().manual_seed(seed)
    t = sum(tot)
    logits = (torch.randn(1, t, v, generator=g) * 2).to(dtype)
    toks = [torch.randint(0, v, (n,), generator=g) for n in tot]
    n = sum(resp)
    masks = []
    for r in resp:
        m = (torch.rand(r, generator=g) > 0.3)
        masks.append(m.long() if int_masks else m.float())
    masks[0] = torch.zeros_like(masks[0])  # a fully masked sample exercises clamp_min(denominator, 1)
    base = -2.0 + 0.3 * torch.randn(n, generator=g)
    batch = dict(
        advantages=list(torch.split(torch.randn(n, generator=g), resp)),
        log_probs=list(torch.split(base, resp)),
        ref_log_probs=list(torch.split(base + 0.1 * torch.randn(n, generator=g), resp)),
        rollout_log_probs=list(torch.split(base + 0.05 * torch.randn(n, generator=g), resp)),
        unconcat_tokens=toks, response_lengths=resp, total_lengths=tot, loss_masks=masks,
    )
    return logits, batch


def _to_dev(batch, dev):
    out = {}
    for k, val in batch.items():
        if isinstance(val, list) and val and isinstance(val[0], torch.Tensor):
            out[k] = [x.to(dev) for x in val]
        else:
            out[k] = val
    return out


CASES = {
    "ppo": dict(),
    "ppo_k3_entropy": dict(eps_clip_high=0.28, use_kl_loss=True, kl_loss_coef=1e-3, kl_loss_type="k3", entropy_coef=0.01),
    "ppo_unbiased_low_var": dict(use_kl_loss=True, kl_loss_coef=0.05, kl_loss_type="low_var_kl", use_unbiased_kl=True),
    "ppo_k1": dict(use_kl_loss=True, kl_loss_coef=0.1, kl_loss_type="k1"),
    "ppo_k2_per_token": dict(use_kl_loss=True, kl_loss_coef=0.1, kl_loss_type="k2", calculate_per_token_loss=True),
    "gspo": dict(advantage_estimator="gspo", eps_clip=3e-4, eps_clip_high=4e-4),
    "gspo_wide": dict(advantage_estimator="gspo", eps_clip=0.2, eps_clip_high=0.2, entropy_coef=0.02),
    "cispo": dict(advantage_estimator="cispo", eps_clip=0.2, eps_clip_high=0.28),
    "rloo": dict(advantage_estimator="rloo"),
    "sapo": dict(advantage_estimator="sapo"),
    "opsm": dict(use_opsm=True, opsm_delta=-1.0),
    "tis": dict(use_tis=True, tis_clip=1.02, tis_clip_low=0.97),
    "true_on_policy": dict(true_on_policy_mode=True),
    "use_rollout_logprobs": dict(use_rollout_logprobs=True),
    "temperature": dict(rollout_temperature=0.7, entropy_coef=0.01),
    "reinforce_pp": dict(advantage_estimator="reinforce_plus_plus"),
    "reinforce_pp_baseline_k2": dict(advantage_estimator="reinforce_plus_plus_baseline", use_kl_loss=True,
                                     kl_loss_coef=0.1, kl_loss_type="k2"),
}


@pytest.mark.parametrize("name", sorted(CASES))
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-5), (torch.bfloat16, 2e-3)])
@pytest.mark.parametrize("single_pass", ["auto", "off"])
def test_policy_loss_function_vs_oracle(name, dtype, tol, single_pass):
    """Both kernel paths: the fused single-launch step ("auto" picks it whenever the loss is token-local) and the
    separate forward / backward launches ("off")."""
    import relax_amd

    dev = require_gpu()
    announce("policy_loss", name, dtype, single_pass)
    tot, resp, v = [9, 6, 12, 7], [4, 3, 7, 5], 264
    logits, batch = _make_batch(11, tot, resp, v, dtype)
    args = P.make_args(relax_amd_single_pass=single_pass, **CASES[name])
    # oracle on CPU (fp32 upcast of the same logits values)
    lo = logits.float().clone().requires_grad_()
    red = R.make_reducer(resp, batch["loss_masks"], args.calculate_per_token_loss)
    ob = dict(batch)
    want_loss, want_m = P.policy_loss_function(args, ob, lo, red)
    want_loss.backward()
    lg = logits.to(dev).requires_grad_()
    loss, met = relax_amd.policy_loss_function(args, _to_dev(batch, dev), lg, None)
    loss.backward()
    assert lg.grad.dtype == dtype and lg.grad.shape == logits.shape
    assert abs(loss.item() - want_loss.item()) < tol * max(1.0, abs(want_loss.item()))
    for k, w in want_m.items():
        assert k in met, f"missing metric {k}"
        assert abs(met[k].item() - float(w)) < tol * max(1.0, abs(float(w))), (k, met[k].item(), float(w))
    assert set(met) == set(want_m)
    torch.testing.assert_close(lg.grad.float().cpu(), lo.grad, atol=tol, rtol=BF16_ULP if dtype == torch.bfloat16 else 0)


AGG_CASES = {
    "gspo": dict(advantage_estimator="gspo", eps_clip=3e-4, eps_clip_high=4e-4),
    "gspo_wide_kl": dict(advantage_estimator="gspo", eps_clip=0.2, eps_clip_high=0.2, entropy_coef=0.02,
                         use_kl_loss=True, kl_loss_coef=0.05, kl_loss_type="k3"),
    "cispo": dict(advantage_estimator="cispo", eps_clip=0.2, eps_clip_high=0.28),
    "cispo_tis": dict(advantage_estimator="cispo", eps_clip=0.2, eps_clip_high=0.28, use_tis=True, tis_clip=1.02,
                      tis_clip_low=0.97, entropy_coef=0.01),
    "ppo_per_token": dict(calculate_per_token_loss=True, use_kl_loss=True, kl_loss_coef=0.1, kl_loss_type="k1"),
}


@pytest.mark.parametrize("name", sorted(AGG_CASES))
@pytest.mark.parametrize("route", ["all_terms", "pg_only_batch_key", "pg_only_reference_hook"])
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-5), (torch.bfloat16, 2e-3)])
@pytest.mark.parametrize("single_pass", ["auto", "off"])
def test_seq_mean_token_sum_aggregation_vs_oracle(name, route, dtype, tol, single_pass):
    """Sequence-mean-token-sum aggregation (every sequence's masked token sum, averaged over the B sequences) against
    ``oracle.reducers.seq_mean_token_sum``: loss, every metric and dlogits.  ``all_terms`` divides every reduced term
    by B (``relax_amd_sample_denominators``); the two ``pg_only`` routes reduce pg_loss that way and leave the other
    terms on the reference's sample-mean reducer, as ``--custom-pg-loss-reducer-function-path`` does
    (loss.py:1062-1076): once through the batch key, once through the reference's own hook returning a reducer that
    carries its divisors (which keeps the step on the fused launch)."""
    import relax_amd

    dev = require_gpu()
    announce("seq_mean_token_sum", name, route, dtype, single_pass)
    tot, resp, v = [9, 6, 12, 7, 15], [4, 3, 7, 5, 11], 264
    logits, batch = _make_batch(29, tot, resp, v, dtype)
    b = len(resp)
    per_token = bool(AGG_CASES[name].get("calculate_per_token_loss", False))
    if route == "all_terms" and per_token:
        pytest.skip("token-sum mode has no per-sample divisors for the other terms")
    kw = dict(relax_amd_single_pass=single_pass, **AGG_CASES[name])
    if route == "pg_only_reference_hook":
        kw["custom_pg_loss_reducer_function_path"] = "relax_amd.cp_utils.get_seq_mean_token_sum_reducer"
    args = P.make_args(**kw)
    masks = batch["loss_masks"]
    lo = logits.float().clone().requires_grad_()
    if route == "all_terms":
        want_loss, want_m = P.policy_loss_function(args, dict(batch), lo, R.seq_mean_token_sum(resp, masks))
    else:
        want_loss, want_m = P.policy_loss_function(args, dict(batch), lo, R.make_reducer(resp, masks, per_token),
                                                   pg_reducer_factory=lambda m: R.seq_mean_token_sum(resp, m))
    want_loss.backward()
    db = _to_dev(batch, dev)
    if route == "all_terms":
        db["relax_amd_sample_denominators"] = torch.full((b,), float(b), device=dev)
    elif route == "pg_only_batch_key":
        db["relax_amd_pg_sample_denominators"] = torch.full((b,), float(b), device=dev)
    lg = logits.to(dev).requires_grad_()
    calls = []
    if route == "pg_only_reference_hook":  # the hook must not push the step onto the composed path
        import relax_amd.loss as RL

        orig = RL._composed_policy_loss_function
        RL._composed_policy_loss_function = lambda *a, **k: calls.append(1) or orig(*a, **k)
    try:
        loss, met = relax_amd.policy_loss_function(args, db, lg, None)
    finally:
        if route == "pg_only_reference_hook":
            RL._composed_policy_loss_function = orig
    assert not calls
    loss.backward()
    assert abs(loss.item() - want_loss.item()) < tol * max(1.0, abs(want_loss.item()))
    assert set(met) == set(want_m)
    for k, w in want_m.items():
        assert abs(met[k].item() - float(w)) < tol * max(1.0, abs(float(w))), (k, met[k].item(), float(w))
    # dividing token sums by B instead of by the token count leaves gradient entries of magnitude ~100 on the wide-clip
    # GSPO case (sequence ratios far from one): fp32 rounding of those is relative, 1e-5 of the value
    torch.testing.assert_close(lg.grad.float().cpu(), lo.grad, atol=tol,
                               rtol=BF16_ULP if dtype == torch.bfloat16 else 1e-5)
    # the aggregation is not the sample mean in disguise: pg_loss differs from the reference reducer's
    lo2 = logits.float().clone().requires_grad_()
    _, plain = P.policy_loss_function(P.make_args(**AGG_CASES[name]), dict(batch), lo2,
                                      R.make_reducer(resp, masks, per_token))
    assert abs(float(plain["pg_loss"]) - float(want_m["pg_loss"])) > 10 * tol


def test_divisor_reducer_called_as_plain_closure_matches_token_loop():
    """The reducer object the hook returns is still the callable the reference expects (``reducer(x) -> scalar``)."""
    from relax_amd.cp_utils import get_seq_mean_token_sum_reducer

    dev = require_gpu()
    announce("divisor reducer as closure")
    g = torch.Generator().manual_seed(3)
    resp = [5, 1, 8, 3]
    masks = [(torch.rand(n, generator=g) > 0.4).float() for n in resp]
    masks[1] = torch.zeros(1)
    x = torch.randn(sum(resp), generator=g)
    want = R.seq_mean_token_sum(resp, masks)(x.double())
    red = get_seq_mean_token_sum_reducer([n + 2 for n in resp], resp, [m.to(dev) for m in masks], False)
    xd = x.to(dev).requires_grad_()
    got = red(xd)
    got.backward()
    assert abs(got.item() - want.item()) < 1e-6
    torch.testing.assert_close(xd.grad.cpu(), torch.cat(masks) / len(resp), atol=1e-7, rtol=0)


@pytest.mark.parametrize("single_pass", ["auto", "off"])
def test_reinforce_pp_masked_nonfinite_values_do_not_leak(single_pass):
    """REINFORCE++ reduces with a mask-safe reducer: NaN / inf advantages and old log-probs at masked tokens leave the
    loss, every metric and the gradient finite and equal to the oracle's."""
    import relax_amd

    dev = require_gpu()
    announce("reinforce++ mask-safe", single_pass)
    tot, resp, v = [9, 6, 12, 7], [4, 3, 7, 5], 264
    logits, batch = _make_batch(23, tot, resp, v)
    for key, bad in (("advantages", float("nan")), ("log_probs", float("inf")), ("ref_log_probs", float("nan"))):
        batch[key] = [torch.where(m != 0, x, torch.full_like(x, bad)) for x, m in zip(batch[key], batch["loss_masks"])]
    args = P.make_args(relax_amd_single_pass=single_pass, advantage_estimator="reinforce_plus_plus", use_kl_loss=True,
                       kl_loss_coef=0.1, kl_loss_type="k2")
    lo = logits.clone().requires_grad_()
    want_loss, want_m = P.policy_loss_function(args, dict(batch), lo, R.make_reducer(resp, batch["loss_masks"]))
    want_loss.backward()
    assert torch.isfinite(want_loss)
    # autograd still carries 0 * NaN into the logits rows of the masked tokens (the selected-out branch has a NaN local
    # derivative); the kernel writes exact zeros there, which is what a finite optimiser step needs
    clean = torch.isfinite(lo.grad[0]).all(-1)
    assert not clean.all() and clean.any()
    lg = logits.to(dev).requires_grad_()
    loss, met = relax_amd.policy_loss_function(args, _to_dev(batch, dev), lg, None)
    loss.backward()
    assert abs(loss.item() - want_loss.item()) < 3e-5
    for k, w in want_m.items():
        assert abs(met[k].item() - float(w)) < 3e-5 * max(1.0, abs(float(w))), (k, met[k].item(), float(w))
    got = lg.grad[0].cpu()
    assert torch.isfinite(got).all() and (got[~clean] == 0).all()
    torch.testing.assert_close(got[clean], lo.grad[0][clean], atol=3e-5, rtol=0)


@pytest.mark.parametrize("v,dtype", [(151936, torch.bfloat16), (32000, torch.float32), (4096, torch.float16),
                                     (40960, torch.bfloat16), (100000, torch.bfloat16), (4100, torch.bfloat16),
                                     (1003, torch.float32), (20000, torch.float32),
                                     # what stock Megatron hands the custom-loss hook (loss.py:92-97)
                                     (151936, torch.float32)])
def test_single_pass_matches_two_launch_path_at_real_vocabularies(v, dtype):
    """Every workgroup width of the fused kernel (256 / 512 / 1024 threads), the scalar-tail and the unaligned
    scalar path, an upstream gradient != 1 and the one-shot backward."""
    import relax_amd

    dev = require_gpu()
    announce("single pass vs two launch", v, dtype)
    tot, resp = [9, 6, 12, 7], [4, 3, 7, 5]
    logits, batch = _make_batch(17, tot, resp, v, dtype)
    db = _to_dev(batch, dev)
    outs = {}
    for mode in ("auto", "off"):
        args = P.make_args(relax_amd_single_pass=mode, eps_clip_high=0.28, use_kl_loss=True, kl_loss_coef=1e-3,
                           kl_loss_type="k3", entropy_coef=0.01)
        lg = logits.to(dev).requires_grad_()
        loss, met = relax_amd.policy_loss_function(args, db, lg, None)
        (loss * 3.0).backward(retain_graph=True)
        outs[mode] = (loss.detach(), {k: x.clone() for k, x in met.items()}, lg.grad.clone())
        if mode == "auto":
            with pytest.raises(RuntimeError, match="cannot run twice"):
                loss.backward()
    assert torch.equal(outs["auto"][0], outs["off"][0])  # same forward arithmetic, same reduction order
    for k in outs["auto"][1]:
        torch.testing.assert_close(outs["auto"][1][k], outs["off"][1][k], atol=1e-6, rtol=1e-6)
    ulp = {torch.float32: 1e-6, torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10}[dtype]
    torch.testing.assert_close(outs["auto"][2].float(), outs["off"][2].float(), atol=1e-6, rtol=ulp)
    # and against the oracle
    lo = logits.float().clone().requires_grad_()
    oargs = P.make_args(eps_clip_high=0.28, use_kl_loss=True, kl_loss_coef=1e-3, kl_loss_type="k3", entropy_coef=0.01)
    want, _ = P.policy_loss_function(oargs, dict(batch), lo, R.make_reducer(resp, batch["loss_masks"]))
    (want * 3.0).backward()
    tol = 3e-5 if dtype == torch.float32 else 2e-3
    assert abs(outs["auto"][0].item() - want.item()) < tol * max(1.0, abs(want.item()))
    torch.testing.assert_close(outs["auto"][2].float().cpu(), lo.grad, atol=tol, rtol=max(ulp, 1e-5))


def test_sample_index_mask_sums_int_masks_and_sft_row():
    import relax_amd

    dev = require_gpu()
    announce("policy_loss denominators / int masks / sft-shaped sample")
    tot, resp, v = [6, 5, 8], [3, 5, 4], 96  # second sample: response == total (SFT convention)
    logits, batch = _make_batch(5, tot, resp, v, torch.float32, int_masks=True)
    batch["sample_index_mask_sums"] = [7, 7, 3]
    args = P.make_args(entropy_coef=0.01)
    lo = logits.clone().requires_grad_()
    red = R.make_reducer(resp, batch["loss_masks"], False, batch["sample_index_mask_sums"])
    want_loss, want_m = P.policy_loss_function(args, dict(batch), lo, red)
    want_loss.backward()
    lg = logits.to(dev).requires_grad_()
    loss, met = relax_amd.policy_loss_function(args, _to_dev(batch, dev), lg, None)
    loss.backward()
    assert abs(loss.item() - want_loss.item()) < 3e-5
    torch.testing.assert_close(lg.grad.cpu(), lo.grad, atol=3e-5, rtol=0)


def test_loss_function_scaling_and_exact_token_count():
    import relax_amd

    dev = require_gpu()
    announce("loss_function tail")
    tot, resp, v = [9, 6, 12], [4, 3, 7], 64
    logits, batch = _make_batch(3, tot, resp, v, torch.float32, int_masks=True)
    for per_token in (False, True):
        args = P.make_args(global_batch_size=8, calculate_per_token_loss=per_token)
        want_loss, want_norm, want_log = P.loss_function(args, dict(batch), 4, logits, dp_world=2)
        loss, norm, log = relax_amd.loss_function(args, _to_dev(batch, dev), 4, logits.to(dev), dp_world_size=2)
        assert log["keys"] == want_log["keys"]
        assert int(norm.item()) == int(want_norm.item())  # exact
        torch.testing.assert_close(log["values"].cpu(), want_log["values"].float(), atol=3e-5, rtol=1e-5)
        assert abs(loss.item() - want_loss.item()) < 3e-5 * max(1, abs(want_loss.item()))
    n = relax_amd.cp_utils.get_cp_local_num_tokens(tot, resp, [m.to(dev) for m in batch["loss_masks"]])
    assert n.dtype == torch.int64 and n.item() == R.num_tokens(batch["loss_masks"]).item()


@pytest.mark.parametrize("loss_type", ["policy_loss", "sft"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("schedule", ["megatron", "as_returned", "explicit_scale", "per_token"])
def test_loss_function_scale_reaches_the_single_launch(loss_type, dtype, schedule, monkeypatch):
    """``loss_function`` multiplies the loss by ``num_microbatches / global_batch_size * dp`` (or ``__loss_scale__``)
    and the training schedule divides by the number of micro-batches, so the upstream gradient of the fused
    single-launch loss is never 1 in training.  The scale is handed to the launch, which writes dlogits already
    multiplied by it: backward must find nothing left to rescale (factor 1) and the gradient must equal the
    two-launch path's, which applies the scale in its dlogits kernel, to one rounding of the output dtype.  When the
    schedule does something else than announced, backward rescales and the gradient is still right."""
    import relax_amd
    from relax_amd import ops

    dev = require_gpu()
    announce("loss_function scale into the single launch", loss_type, dtype, schedule)
    tot, resp, v = [9, 6, 12, 7], [4, 3, 7, 5], 4096
    logits, batch = _make_batch(53, tot, resp, v, dtype)
    if loss_type == "sft":
        tot = resp = [9, 6, 12, 7]
        logits, batch = _make_batch(53, tot, resp, v, dtype)
    nm, gbs, dp = 4, 32, 2
    kw = dict(loss_type=loss_type, global_batch_size=gbs, use_kl_loss=True, kl_loss_coef=0.01, kl_loss_type="k3",
              entropy_coef=0.01, calculate_per_token_loss=(schedule == "per_token"))
    bd = _to_dev(batch, dev)
    if schedule == "explicit_scale":
        bd["__loss_scale__"] = 0.3
    post = {"megatron": 1.0 / nm, "as_returned": 1.0, "explicit_scale": 1.0 / nm, "per_token": 1.0}[schedule]
    if schedule == "as_returned":
        kw["relax_amd_schedule_loss_scale"] = 1.0
    factors = []
    real = ops.scale_rows_inplace
    monkeypatch.setattr(ops, "scale_rows_inplace", lambda d, f: factors.append(f.clone()) or real(d, f))
    grads = {}
    for mode in ("auto", "off"):
        args = P.make_args(relax_amd_single_pass=mode, **kw)
        lg = logits.to(dev).requires_grad_()
        loss, _norm, _log = relax_amd.loss_function(args, bd, nm, lg, dp_world_size=dp)
        (loss * post).backward()
        grads[mode] = lg.grad.clone()
    assert len(factors) == 1  # only the single-launch path goes through the in-place rescale
    assert abs(factors[0].item() - 1.0) <= 2.0 ** -20, factors[0].item()
    ulp = {torch.float32: 2e-6, torch.bfloat16: 2.0 ** -8}[dtype]
    torch.testing.assert_close(grads["auto"].float(), grads["off"].float(), atol=1e-9, rtol=ulp)
    assert grads["auto"].abs().sum().item() > 0
    # oracle, same scaling
    lo = logits.float().clone().requires_grad_()
    oargs = P.make_args(**kw)
    ob = dict(batch)
    if schedule == "explicit_scale":
        ob["__loss_scale__"] = 0.3
    want, _, _ = P.loss_function(oargs, ob, nm, lo, dp_world=dp)
    (want * post).backward()
    tol = 3e-5 if dtype == torch.float32 else 2e-3
    torch.testing.assert_close(grads["auto"].float().cpu(), lo.grad, atol=tol, rtol=max(ulp, 1e-5))
    # a schedule that does not do what was announced: the backward rescales, the result is still right
    factors.clear()
    args = P.make_args(relax_amd_single_pass="auto", **kw)
    lg = logits.to(dev).requires_grad_()
    loss, _norm, _log = relax_amd.loss_function(args, bd, nm, lg, dp_world_size=dp)
    (loss * post * 7.0).backward()
    assert len(factors) == 1 and abs(factors[0].item() - 7.0) < 1e-5
    torch.testing.assert_close(lg.grad.float().cpu(), lo.grad * 7.0, atol=7 * tol,
                               rtol=max(2 * ulp, 1e-5))


@pytest.mark.parametrize("loss_type", ["policy_loss", "sft", "value_loss"])
@pytest.mark.parametrize("reentrant", [True, False])
def test_loss_function_recompute_gives_the_same_loss_and_gradient(loss_type, reentrant):
    """``--recompute-loss-function`` (loss.py:1535-1543): the loss runs under ``torch.utils.checkpoint`` -- once
    without autograd, once more during backward -- and must return the same loss, logging values and gradient, bit
    for bit, as the direct call."""
    import relax_amd

    dev = require_gpu()
    announce("loss_function recompute", loss_type, reentrant)
    tot, resp, v = [9, 6, 12, 7], [4, 3, 7, 5], 264
    logits, batch = _make_batch(41, tot, resp, v)
    n = sum(resp)
    g = torch.Generator().manual_seed(1)
    batch["values"] = list(torch.split(torch.randn(n, generator=g), resp))
    batch["returns"] = list(torch.split(torch.randn(n, generator=g), resp))
    x = torch.randn(1, sum(tot), 1, generator=g) if loss_type == "value_loss" else logits
    bd = _to_dev(batch, dev)
    results = []
    for recompute in (False, True):
        args = P.make_args(loss_type=loss_type, value_clip=0.3, global_batch_size=4, use_kl_loss=True,
                           kl_loss_coef=0.01, kl_loss_type="k3", entropy_coef=0.01,
                           recompute_loss_function=recompute, recompute_loss_function_use_reentrant=reentrant)
        xd = x.to(dev).requires_grad_()
        loss, _norm, log = relax_amd.loss_function(args, bd, 2, xd)
        loss.backward()
        results.append((loss.detach(), log["keys"], log["values"], xd.grad))
    (l0, k0, v0, g0), (l1, k1, v1, g1) = results
    assert k0 == k1 and torch.equal(l0, l1) and torch.equal(v0, v1) and torch.equal(g0, g1)
    assert g0.abs().sum().item() > 0


def test_mtp_only_training_dispatch():
    """``args.mtp_only_training`` (loss.py:1431-1440, 1512-1513): a zero loss that stays attached to its input."""
    import relax_amd

    dev = require_gpu()
    announce("mtp only")
    tot, resp, v = [9, 6], [4, 3], 64
    logits, batch = _make_batch(4, tot, resp, v)
    args = P.make_args(mtp_only_training=True, global_batch_size=2)
    hd = torch.randn(1, sum(tot), 16).to(dev).requires_grad_()
    loss, _norm, log = relax_amd.loss_function(args, _to_dev(batch, dev), 1, hd)
    loss.backward()
    assert loss.item() == 0 and log["keys"] == ["loss"] and not hd.grad.any() and hd.grad.shape == hd.shape


def test_get_log_probs_and_entropy_forward_only_matches_training_forward_bitwise():
    """The forward-only pass and the training forward must give identical log-probs for identical inputs."""
    import relax_amd

    dev = require_gpu()
    announce("forward_only vs train forward")
    tot, resp, v = [9, 6, 12, 7], [4, 3, 7, 5], 1000
    logits, batch = _make_batch(2, tot, resp, v, torch.bfloat16)
    args = P.make_args(entropy_coef=0.0)
    db = _to_dev(batch, dev)
    with torch.no_grad():
        _, out = relax_amd.get_log_probs_and_entropy(
            logits.to(dev), args=args, unconcat_tokens=db["unconcat_tokens"], total_lengths=tot,
            response_lengths=resp, with_entropy=True)
    assert [x.shape[0] for x in out["log_probs"]] == resp
    lg = logits.to(dev).requires_grad_()
    _, out2 = relax_amd.get_log_probs_and_entropy(
        lg, args=args, unconcat_tokens=db["unconcat_tokens"], total_lengths=tot, response_lengths=resp,
        with_entropy=True)
    for a, b in zip(out["log_probs"], out2["log_probs"]):
        assert torch.equal(a, b)
    assert not out2["entropy"][0].requires_grad and out2["log_probs"][0].requires_grad
    _, ref = P.get_log_probs_and_entropy(logits.float(), args=args, unconcat_tokens=batch["unconcat_tokens"],
                                         total_lengths=tot, response_lengths=resp, with_entropy=True)
    for a, b in zip(out["log_probs"], ref["log_probs"]):
        torch.testing.assert_close(a.cpu(), b, atol=2e-3, rtol=0)
    for a, b in zip(out["entropy"], ref["entropy"]):
        torch.testing.assert_close(a.cpu(), b, atol=2e-3, rtol=0)


def test_grpo_micro_fixture_through_the_kernels(literals):
    """Reference hand-derived fixture: loss = -0.02 at lp = old; fabricated logits give entropy != 0.5, so the
    per-token kernel is driven directly with the fixture's per-token values."""
    from relax_amd import ops

    dev = require_gpu()
    announce("grpo micro fixture")
    fx = literals["grpo_micro_fixture"]
    adv = torch.tensor(fx["advantages"], device=dev)
    cu = torch.tensor([0, 2, 4, 6, 8], device=dev)
    for lp_val, want in ((0.0, None), (0.5, fx["lp_half_case"])):
        out = ops.policy_loss(
            log_prob=torch.full((8,), lp_val, device=dev), old_log_prob=torch.zeros(8, device=dev), advantages=adv,
            loss_mask=torch.ones(8, device=dev), entropy=torch.full((8,), fx["entropy"], device=dev), cu_resp=cu,
            sample_denom=torch.full((4,), 2.0, device=dev), entropy_coef=fx["entropy_coef"], eps_clip=0.2, eps_clip_high=0.2)
        m = dict(zip(["loss", "pg_loss", "entropy_loss", "pg_clipfrac", "ppo_kl"], out["metrics"][:5].tolist()))
        if want is None:
            assert abs(m["loss"] - fx["default_loss"]) < 1e-6 and abs(m["pg_loss"]) < 1e-6
        else:
            for k in ("loss", "pg_loss", "pg_clipfrac", "ppo_kl", "entropy_loss"):
                assert abs(m[k] - want[k]) < 2e-5, (k, m[k])


def test_standalone_token_losses_vs_oracle():
    from oracle import losses as L
    from relax_amd import ppo_utils as K

    dev = require_gpu()
    announce("standalone token losses")
    g = torch.Generator().manual_seed(9)
    n = 777
    lp = (torch.randn(n, generator=g) * 0.4 - 1).requires_grad_()
    old = lp.detach() + torch.randn(n, generator=g) * 0.3
    adv = torch.randn(n, generator=g)
    adv[:6] = 0
    w = torch.randn(n, generator=g)
    lpd = lp.detach().to(dev).requires_grad_()

    def cmp(ref_pair, got_pair, ref_leaf, got_leaf):
        (ref_pair[0] * w).sum().backward()
        (got_pair[0] * w.to(dev)).sum().backward()
        torch.testing.assert_close(got_pair[0].detach().cpu(), ref_pair[0].detach(), atol=2e-5, rtol=1e-5)
        torch.testing.assert_close(got_pair[1].cpu(), ref_pair[1], atol=0, rtol=0)
        torch.testing.assert_close(got_leaf.grad.cpu(), ref_leaf.grad, atol=2e-5, rtol=1e-5)
        ref_leaf.grad = None
        got_leaf.grad = None

    kl = (old - lp.detach()).requires_grad_()
    kld = kl.detach().to(dev).requires_grad_()
    cmp(L.policy_clip(kl, adv, 0.2, 0.28), K.compute_policy_loss(kld, adv.to(dev), 0.2, 0.28), kl, kld)
    cmp(L.policy_clip(kl, adv, 0.2, 0.28, 3.0), K.compute_policy_loss(kld, adv.to(dev), 0.2, 0.28, 3.0), kl, kld)
    cmp(L.sapo(kl, adv, 1.0, 1.05), K.compute_sapo_loss(kld, adv.to(dev), 1.0, 1.05), kl, kld)
    cmp(L.cispo(lp, old - lp, adv, 0.2, 0.28), K.compute_cispo_loss(lpd, old.to(dev) - lpd, adv.to(dev), 0.2, 0.28), lp, lpd)
    cmp(L.rloo_loss(lp, adv), K.compute_rloo_loss(lpd, adv.to(dev)), lp, lpd)
    for kind in ("k1", "k2", "k3", "low_var_kl"):
        ref = L.approx_kl(lp, old, kind)
        got = K.compute_approx_kl(lpd, old.to(dev), kind)
        (ref * w).sum().backward()
        (got * w.to(dev)).sum().backward()
        torch.testing.assert_close(got.detach().cpu(), ref.detach(), atol=2e-5, rtol=1e-5)
        torch.testing.assert_close(lpd.grad.cpu(), lp.grad, atol=2e-5, rtol=1e-5)
        lp.grad = None
        lpd.grad = None
    with pytest.raises(AssertionError):
        K.compute_policy_loss(kld, adv.to(dev), 0.2, 0.2, 0.5)
    # sequence KL (GSPO) as a standalone, with gradient
    lens = [300, 77, 400]
    masks = [(torch.rand(k, generator=g) > 0.4).float() for k in lens]
    lps = list(torch.split(lp, lens))
    ref = L.gspo_seq_kl(lps, list(torch.split(old, lens)), masks)
    got = K.compute_gspo_kl(list(torch.split(lpd, lens)), [o.to(dev) for o in torch.split(old, lens)],
                            list(torch.split(lpd, lens)), [m.to(dev) for m in masks])
    (ref * w).sum().backward()
    (got * w.to(dev)).sum().backward()
    torch.testing.assert_close(got.detach().cpu(), ref.detach(), atol=2e-5, rtol=1e-5)
    torch.testing.assert_close(lpd.grad.cpu(), lp.grad, atol=2e-5, rtol=1e-5)


@pytest.mark.parametrize("per_token", [False, True])
def test_value_loss_function_vs_oracle_and_closed_forms(per_token):
    """The critic's loss (``--loss-type value_loss``): value-head output [1, T, 1] sliced to the response rows, clipped
    squared error, per-sample masked mean.  Against the oracle (values, loss, both metrics, gradient w.r.t. the value
    head's output, which is zero outside the response rows and under a zero mask), through ``loss_function``'s
    dispatch, and against two closed forms: a clip wider than every deviation gives the plain squared error with
    gradient 2 (v - R) m / denominator, and with old values equal to the new ones nothing is clipped."""
    import relax_amd
    from relax_amd.loss import loss_function

    dev = require_gpu()
    announce("value loss", per_token)
    tot, resp = [9, 6, 12, 7], [4, 3, 7, 5]
    _, batch = _make_batch(5, tot, resp, 8)
    g = torch.Generator().manual_seed(77)
    n = sum(resp)
    head = torch.randn(1, sum(tot), 1, generator=g)
    batch["values"] = list(torch.split(torch.randn(n, generator=g), resp))
    batch["returns"] = list(torch.split(torch.randn(n, generator=g), resp))
    args = P.make_args(loss_type="value_loss", value_clip=0.4, calculate_per_token_loss=per_token)
    red = R.make_reducer(resp, batch["loss_masks"], per_token)
    ho = head.clone().requires_grad_()
    want_loss, want_m = P.value_loss_function(args, batch, ho, red)
    want_loss.backward()
    bd = _to_dev(batch, dev)
    hd = head.to(dev).requires_grad_()
    _, vals = relax_amd.get_values(hd, args=args, unconcat_tokens=bd["unconcat_tokens"], total_lengths=tot,
                                   response_lengths=resp)
    for got, want in zip(vals["values"], P.get_values(head, tot, resp)):
        assert torch.equal(got.detach().cpu(), want)
    loss, met = relax_amd.value_loss_function(args, bd, hd, None)
    loss.backward()
    assert abs(loss.item() - want_loss.item()) < 3e-6 * max(1.0, abs(want_loss.item()))
    assert set(met) == {"value_loss", "value_clipfrac"}
    for k, w in want_m.items():
        assert abs(met[k].item() - float(w)) < 3e-6 * max(1.0, abs(float(w))), k
    assert 0 < want_m["value_clipfrac"].item()  # the case does clip
    torch.testing.assert_close(hd.grad.cpu(), ho.grad, atol=1e-6, rtol=1e-5)
    loss2, normalizer, log = loss_function(args, bd, 1, head.to(dev))
    assert log["keys"] == ["value_loss", "value_clipfrac"]
    scale = 1.0 if per_token else 1.0 / args.global_batch_size
    assert abs(loss2.item() - want_loss.item() * scale) < 3e-6 * max(1.0, abs(want_loss.item()))
    # closed forms
    wide = P.make_args(loss_type="value_loss", value_clip=1e9, calculate_per_token_loss=per_token)
    hd2 = head.to(dev).requires_grad_()
    loss3, met3 = relax_amd.value_loss_function(wide, bd, hd2, None)
    loss3.backward()
    rows = torch.cat([torch.arange(b, e) for b, e, _ in P.response_row_ranges(tot, resp)])
    v = head.reshape(-1)[rows]
    ret, mask = torch.cat(batch["returns"]), torch.cat(batch["loss_masks"])
    den = torch.cat([torch.full((r,), 1.0 if per_token else max(float(m.sum()), 1.0))
                     for r, m in zip(resp, batch["loss_masks"])])
    assert abs(loss3.item() - float((((v - ret) ** 2) * mask / den).sum())) < 1e-5
    assert met3["value_clipfrac"].item() == 0
    want_grad = torch.zeros(sum(tot))
    want_grad[rows] = 2 * (v - ret) * mask / den
    torch.testing.assert_close(hd2.grad.reshape(-1).cpu(), want_grad, atol=1e-6, rtol=1e-5)
    bd_same = dict(bd, values=[x.detach().clone() for x in vals["values"]])
    _, met4 = relax_amd.value_loss_function(args, bd_same, head.to(dev), None)
    assert met4["value_clipfrac"].item() == 0


@pytest.mark.parametrize("case", ["ppo_k3_entropy", "gspo", "cispo"])
def test_padded_bshd_layout_equals_packed_layout(case):
    """``qkv_format="bshd"``: logits [B, S, V] padded to S = max_seq_len rows per sample (loss.py:94-117).  The same
    samples laid out packed and padded give the same loss and metrics bit for bit, the same gradient on every real
    row and exact zeros on the padding; the response rows are the ones brute-force enumeration names."""
    import relax_amd
    from relax_amd.loss import response_row_begins

    dev = require_gpu()
    announce("bshd layout", case)
    tot, resp, v = [9, 6, 12, 7], [4, 3, 7, 5], 264
    s_max = 13
    logits, batch = _make_batch(17, tot, resp, v)
    begins, _ = response_row_begins(tot, resp, [s_max] * 4)
    want_rows = [s_max * i + t - r - 1 for i, (t, r) in enumerate(zip(tot, resp))]  # previous position scores a token
    assert begins == want_rows
    assert [b for b, _e, _s in P.response_row_ranges(tot, resp, [s_max] * 4)] == want_rows
    padded = torch.full((4, s_max, v), 7.0)  # padding rows hold junk that must not matter
    off = 0
    for i, t in enumerate(tot):
        padded[i, :t] = logits[0, off:off + t]
        off += t
    bd = _to_dev(batch, dev)
    args = P.make_args(**CASES[case])
    lg = logits.to(dev).requires_grad_()
    loss, met = relax_amd.policy_loss_function(args, bd, lg, None)
    loss.backward()
    args_b = P.make_args(qkv_format="bshd", **CASES[case])
    bd_b = dict(bd, max_seq_lens=[s_max] * 4)
    pg = padded.to(dev).requires_grad_()
    loss_b, met_b = relax_amd.policy_loss_function(args_b, bd_b, pg, None)
    loss_b.backward()
    assert loss_b.item() == loss.item()
    for k in met:
        assert met_b[k].item() == met[k].item(), k
    assert pg.grad.shape == padded.shape
    off = 0
    for i, t in enumerate(tot):
        assert torch.equal(pg.grad[i, :t], lg.grad[0, off:off + t])
        assert not pg.grad[i, t:].any()
        off += t
    _, out = relax_amd.get_log_probs_and_entropy(padded.to(dev), args=args_b, unconcat_tokens=bd["unconcat_tokens"],
                                                 total_lengths=tot, response_lengths=resp, with_entropy=True,
                                                 max_seq_lens=[s_max] * 4)
    _, ref = relax_amd.get_log_probs_and_entropy(logits.to(dev), args=args, unconcat_tokens=bd["unconcat_tokens"],
                                                 total_lengths=tot, response_lengths=resp, with_entropy=True)
    for a, b in zip(out["log_probs"] + out["entropy"], ref["log_probs"] + ref["entropy"]):
        assert torch.equal(a, b)
    chunks = list(relax_amd.get_responses(padded.to(dev), args=args_b, unconcat_tokens=bd["unconcat_tokens"],
                                          total_lengths=tot, response_lengths=resp, max_seq_lens=[s_max] * 4))
    for (chunk, _tk), b, r in zip(chunks, want_rows, resp):
        assert torch.equal(chunk.cpu(), padded.reshape(-1, v)[b:b + r])


def test_reducers_vs_oracle_literals(literals):
    from relax_amd import cp_utils

    dev = require_gpu()
    announce("reducers")
    fx = literals["ppo_clip_k2_response_mean"]
    masks = [torch.tensor(m, device=dev) for m in fx["masks"]]
    red = cp_utils.get_sum_of_sample_mean(fx["response_lengths"], fx["response_lengths"], masks)
    inv = literals["masked_invariance"]
    a = red(torch.tensor(inv["base"], device=dev))
    b = red(torch.tensor(inv["changed"], device=dev))
    assert torch.equal(a, b) and abs(a.item() - (1.0 + 3.5)) < 1e-6
    fx = literals["per_token_loss_path"]
    masks = [torch.tensor(m, device=dev, dtype=torch.float64) for m in fx["masks"]]
    lp = torch.tensor(fx["log_probs"], device=dev, requires_grad=True)
    adv = torch.tensor(fx["advantages"], device=dev)
    red = cp_utils.get_sum_of_sample_mean([3, 5], fx["response_lengths"], masks, calculate_per_token_loss=True)
    n = cp_utils.get_cp_local_num_tokens([3, 5], fx["response_lengths"], masks)
    assert n.item() == fx["expected_normalizer"]
    total = red(-(adv * lp))
    (total / n).backward()
    flat = torch.cat(masks).float()
    torch.testing.assert_close(total, -(adv * lp.detach() * flat).sum(), atol=1e-6, rtol=0)
    torch.testing.assert_close(lp.grad, -(adv * flat) / 5, atol=1e-7, rtol=0)
    fx = literals["target_coordinate_masks"]
    m = [torch.tensor(fx["mask"], device=dev)]
    red = cp_utils.get_sum_of_sample_mean([4], [4], m, calculate_per_token_loss=True)
    assert red(torch.tensor(fx["values"], device=dev)).item() == fx["token_sum"]
    assert cp_utils.get_cp_local_num_tokens([4], [4], m).item() == fx["count"]


def test_full_size_packed_varlen_gspo_and_cispo_properties():
    """Packed variable-length batch at the benchmark's vocabulary (8 sequences, 2k-6k tokens here to bound the test's
    memory; the kernels are per-row): sequence-level GSPO through the two-launch path and token-level CISPO through the
    fused launch.  Checks that hold at any size: finite loss, every dlogits row sums to ~0, masked rows are exactly
    zero, the CISPO loss is identical bit for bit on both paths, and GSPO's per-sequence ratio really is shared by the
    sequence (scaling one token's old log-prob moves every gradient row of that sequence, and no other)."""
    import relax_amd

    dev = require_gpu()
    v = 151936
    cpu = torch.Generator().manual_seed(0)
    lengths = [int(x) for x in torch.randint(2048, 6145, (8,), generator=cpu)]
    n = sum(lengths)
    announce("varlen full vocab", lengths)
    g = torch.Generator(device=dev).manual_seed(0)
    logits = (torch.randn((1, n, v), device=dev, generator=g) * 3.0).to(torch.bfloat16)
    masks = []
    for ln in lengths:
        m = torch.ones(ln)
        for _ in range(4):
            w = int(0.075 * ln)
            st = int(torch.randint(0, ln - w, (1,), generator=cpu))
            m[st:st + w] = 0.0
        masks.append(m.to(dev))
    toks = [torch.randint(0, v, (ln,), device=dev, generator=g) for ln in lengths]
    adv = torch.rand(8, generator=cpu) - 0.5
    batch = dict(unconcat_tokens=toks, total_lengths=lengths, response_lengths=lengths, loss_masks=masks,
                 advantages=[adv[i].to(dev).expand(ln).contiguous() for i, ln in enumerate(lengths)],
                 relax_amd_sample_denominators=torch.full((8,), 8.0, device=dev))
    base = P.make_args()
    with torch.no_grad():
        _, out = relax_amd.get_log_probs_and_entropy(logits, args=base, unconcat_tokens=toks, total_lengths=lengths,
                                                     response_lengths=lengths, with_entropy=False)
    batch["log_probs"] = [lp + 0.02 * torch.randn(lp.shape, device=dev, generator=g) for lp in out["log_probs"]]
    flat_mask = torch.cat(masks)
    results = {}
    for name, kw in (("gspo", dict(advantage_estimator="gspo", eps_clip=3e-4, eps_clip_high=4e-4)),
                     ("cispo", dict(advantage_estimator="cispo", eps_clip=0.2, eps_clip_high=0.28)),
                     ("cispo_two_launch", dict(advantage_estimator="cispo", eps_clip=0.2, eps_clip_high=0.28,
                                               relax_amd_single_pass="off"))):
        lg = logits.clone().requires_grad_()
        loss, met = relax_amd.policy_loss_function(P.make_args(**kw), batch, lg, None)
        loss.backward()
        assert torch.isfinite(loss) and all(torch.isfinite(x) for x in met.values())
        d = lg.grad[0]
        assert d.float().sum(-1).abs().max().item() < 2e-2
        assert (d[flat_mask == 0] == 0).all()
        results[name] = (loss.item(), d)
    assert results["cispo"][0] == results["cispo_two_launch"][0]
    torch.testing.assert_close(results["cispo"][1].float(), results["cispo_two_launch"][1].float(), atol=1e-6,
                               rtol=2 * BF16_ULP)
    # GSPO: perturb one token's old log-prob in sequence 3; only that sequence's gradient rows may change
    lo = [x.clone() for x in batch["log_probs"]]
    first_valid = int(torch.nonzero(masks[3])[0])
    lo[3][first_valid] += 0.5
    lg = logits.clone().requires_grad_()
    loss2, _ = relax_amd.policy_loss_function(P.make_args(advantage_estimator="gspo", eps_clip=3e-4, eps_clip_high=4e-4),
                                              dict(batch, log_probs=lo), lg, None)
    loss2.backward()
    changed = (lg.grad[0] != results["gspo"][1]).any(-1)
    start = sum(lengths[:3])
    inside = torch.zeros(n, dtype=torch.bool, device=dev)
    inside[start:start + lengths[3]] = True
    assert not changed[~inside].any()
    assert changed[inside & (flat_mask != 0)].float().mean().item() > 0.99


def test_full_size_actor_step_with_topk_distillation_term():
    """The headline shape (16 sequences x 4096 tokens, V = 151936, bf16, first 20 % of every sequence masked) with the
    top-64 distillation term in the single launch: the same loss and metrics as the two-launch path; one whole
    sequence's rows (4096) against the oracle's gradient for that sequence's share of the loss; for every row: masked
    rows exactly zero, gradient rows summing to zero up to the rounding of 151936 bf16 terms."""
    import relax_amd

    dev = require_gpu()
    seqs, seq_len, v, k = 16, 4096, 151936, 64
    n = seqs * seq_len
    announce("actor step + top-K distillation, full size", n, v, k)
    g = torch.Generator(device=dev).manual_seed(3)
    logits = torch.empty((1, n, v), dtype=torch.bfloat16, device=dev)
    for s0 in range(0, n, 2048):
        logits[0, s0:s0 + 2048] = (torch.randn((2048, v), device=dev, generator=g) * 3.0).bfloat16()
    toks = [torch.randint(0, v, (seq_len,), device=dev, generator=g) for _ in range(seqs)]
    mask = torch.ones(seq_len, device=dev)
    mask[: seq_len // 5] = 0.0
    kw = dict(eps_clip_high=0.28, use_kl_loss=True, kl_loss_coef=1e-3, kl_loss_type="k3", opd_loss_coef=0.5,
              opd_token_selection="teacher_topk", opd_kl_type="reverse_kl", opd_norm_mode="tail")
    args = P.make_args(**kw)
    with torch.no_grad():
        _, out = relax_amd.get_log_probs_and_entropy(logits, args=args, unconcat_tokens=toks,
                                                     total_lengths=[seq_len] * seqs,
                                                     response_lengths=[seq_len] * seqs, with_entropy=False)
    old = [lp + 0.05 * torch.randn(lp.shape, device=dev, generator=g) for lp in out["log_probs"]]
    ref = [lp + 0.05 * torch.randn(lp.shape, device=dev, generator=g) for lp in out["log_probs"]]
    total_unmasked = float(mask.sum().item()) * seqs
    batch = dict(
        unconcat_tokens=toks, total_lengths=[seq_len] * seqs, response_lengths=[seq_len] * seqs,
        loss_masks=[mask] * seqs, advantages=[torch.randn(seq_len, device=dev, generator=g) for _ in range(seqs)],
        log_probs=old, ref_log_probs=ref,
        relax_amd_sample_denominators=torch.full((seqs,), total_unmasked, device=dev),
        opd_topk_token_ids=[torch.randint(0, v, (seq_len, k), device=dev, generator=g) for _ in range(seqs)],
        opd_topk_teacher_log_probs=[torch.log_softmax(torch.randn(seq_len, k + 1, device=dev, generator=g), -1)[:, :k]
                                    .contiguous() for _ in range(seqs)])
    results = {}
    for mode in ("auto", "off"):
        lg = logits.detach().requires_grad_()
        loss, met = relax_amd.policy_loss_function(P.make_args(relax_amd_single_pass=mode, **kw), batch, lg, None)
        loss.backward()
        results[mode] = (loss.detach(), met, lg.grad)
        lg.grad = None
        if mode == "auto":
            d = results["auto"][2][0]
            flat_mask = mask.repeat(seqs)
            for s0 in range(0, n, 8192):
                rows = d[s0:s0 + 8192]
                assert rows.float().sum(-1).abs().max().item() < 5e-2
                assert (rows[flat_mask[s0:s0 + 8192] == 0] == 0).all()
            picked = 5
            sub_rows = d[picked * seq_len:(picked + 1) * seq_len].float().cpu()
            results["auto"] = (results["auto"][0], met, None)
            del d, lg, loss
            torch.cuda.empty_cache()
    assert abs(results["auto"][0].item() - results["off"][0].item()) < 1e-5 * max(1.0, abs(results["off"][0].item()))
    for key, w in results["off"][1].items():
        assert abs(results["auto"][1][key].item() - w.item()) < 1e-5 * max(1.0, abs(w.item())), key
    d_off = results["off"][2][0][picked * seq_len:(picked + 1) * seq_len].float().cpu()
    torch.testing.assert_close(sub_rows, d_off, atol=2e-9, rtol=2.0 ** -6)
    # the picked sequence against the oracle: its rows, its share of the token-mean loss
    sub_logits = logits[0, picked * seq_len:(picked + 1) * seq_len].float().cpu().unsqueeze(0).requires_grad_()
    sub = {key: [val[picked].cpu()] for key, val in batch.items()
           if isinstance(val, list) and torch.is_tensor(val[0])}
    sub.update(total_lengths=[seq_len], response_lengths=[seq_len])
    # the term's token mean runs over the whole batch's unmasked tokens: the sequence's share has weight 1 / seqs
    want, _ = P.policy_loss_function(P.make_args(**dict(kw, opd_loss_coef=kw["opd_loss_coef"] / seqs)), sub, sub_logits,
                                     R.make_reducer([seq_len], sub["loss_masks"], sample_denoms=[total_unmasked]))
    want.backward()
    torch.testing.assert_close(sub_rows, sub_logits.grad[0], atol=3e-9, rtol=2.0 ** -6)


def test_full_size_actor_step_plain_spiked_rows_through_loss_function():
    """The headline workload as the benchmark times it, all 65536 rows: bf16 logits ~ N(0, 3) with 5 % of the rows
    carrying one logit raised by 15, first 20 % of every sequence masked, PPO-clip 0.2 / 0.28 + k3 KL 1e-3, no
    distillation term, through loss_function (gradient-accumulation scale 1 / 16).  Runs the register-resident step
    without the top-K block.  The same loss and metrics as the two-launch path; one whole sequence (4096 rows, some 200
    of them spiked) against the oracle's log-probs, entropy and gradient; for every row: masked rows exactly zero,
    gradient rows summing to zero up to the rounding of 151936 bf16 terms."""
    import relax_amd

    dev = require_gpu()
    seqs, seq_len, v = 16, 4096, 151936
    n = seqs * seq_len
    announce("actor step, plain, spiked rows, full size", n, v)
    g = torch.Generator(device=dev).manual_seed(0)
    logits = torch.empty((1, n, v), dtype=torch.bfloat16, device=dev)
    spiked = torch.zeros(n, dtype=torch.bool, device=dev)
    for s0 in range(0, n, 2048):
        x = torch.randn((2048, v), device=dev, generator=g) * 3.0
        spike = torch.rand(2048, device=dev, generator=g) < 0.05
        cols = torch.randint(0, v, (2048,), device=dev, generator=g)
        x[spike, cols[spike]] += 15.0
        spiked[s0:s0 + 2048] = spike
        logits[0, s0:s0 + 2048] = x.bfloat16()
        del x
    toks = [torch.randint(0, v, (seq_len,), device=dev, generator=g) for _ in range(seqs)]
    mask = torch.ones(seq_len, device=dev)
    mask[: seq_len // 5] = 0.0
    kw = dict(eps_clip=0.2, eps_clip_high=0.28, use_kl_loss=True, kl_loss_coef=1e-3, kl_loss_type="k3",
              global_batch_size=seqs)
    args = P.make_args(**kw)
    with torch.no_grad():
        _, out = relax_amd.get_log_probs_and_entropy(logits, args=args, unconcat_tokens=toks,
                                                     total_lengths=[seq_len] * seqs,
                                                     response_lengths=[seq_len] * seqs, with_entropy=True)
    old = [lp + 0.05 * torch.randn(lp.shape, device=dev, generator=g) for lp in out["log_probs"]]
    ref = [lp + 0.1 * torch.randn(lp.shape, device=dev, generator=g) for lp in out["log_probs"]]
    total_unmasked = float(mask.sum().item()) * seqs
    batch = dict(
        unconcat_tokens=toks, total_lengths=[seq_len] * seqs, response_lengths=[seq_len] * seqs,
        loss_masks=[mask] * seqs, advantages=[torch.randn(seq_len, device=dev, generator=g) for _ in range(seqs)],
        log_probs=old, ref_log_probs=ref,
        relax_amd_sample_denominators=torch.full((seqs,), total_unmasked, device=dev))
    picked = 11
    rows = slice(picked * seq_len, (picked + 1) * seq_len)
    assert 100 < int(spiked[rows].sum().item()) < 400
    results = {}
    for mode in ("auto", "off"):
        lg = logits.detach().requires_grad_()
        loss, normalizer, log = relax_amd.loss_function(P.make_args(relax_amd_single_pass=mode, **kw), batch, 1, lg)
        loss.backward()
        met = dict(zip(log["keys"], log["values"][1:].tolist()))
        d = lg.grad[0]
        if mode == "auto":
            flat_mask = mask.repeat(seqs)
            for s0 in range(0, n, 8192):
                blk = d[s0:s0 + 8192]
                assert blk.float().sum(-1).abs().max().item() < 5e-2 / seqs
                assert (blk[flat_mask[s0:s0 + 8192] == 0] == 0).all()
                assert (blk[flat_mask[s0:s0 + 8192] != 0] != 0).any(dim=1).all()
        results[mode] = (loss.detach().item(), met, d[rows].float().cpu())
        assert float(normalizer) == 1
        del d, lg, loss
        torch.cuda.empty_cache()
    assert abs(results["auto"][0] - results["off"][0]) < 1e-6 * max(1.0, abs(results["off"][0]))
    for key, w in results["off"][1].items():
        assert abs(results["auto"][1][key] - w) < 1e-5 * max(1.0, abs(w)), key
    torch.testing.assert_close(results["auto"][2], results["off"][2], atol=2e-10, rtol=2.0 ** -6)
    # the picked sequence against the oracle: log-probs, entropy, its share of the token-mean loss, its rows' gradient
    sub_logits = logits[0, rows].float().cpu().unsqueeze(0).requires_grad_()
    sub = {key: [val[picked].cpu()] for key, val in batch.items() if isinstance(val, list) and torch.is_tensor(val[0])}
    sub.update(total_lengths=[seq_len], response_lengths=[seq_len])
    _, oo = P.get_log_probs_and_entropy(sub_logits.detach(), args=args, unconcat_tokens=sub["unconcat_tokens"],
                                        total_lengths=[seq_len], response_lengths=[seq_len], with_entropy=True)
    torch.testing.assert_close(out["log_probs"][picked].cpu(), oo["log_probs"][0], atol=2e-3, rtol=0)
    torch.testing.assert_close(out["entropy"][picked].cpu(), oo["entropy"][0], atol=2e-3, rtol=0)
    want, _ = P.policy_loss_function(args, sub, sub_logits,
                                     R.make_reducer([seq_len], sub["loss_masks"], sample_denoms=[total_unmasked]))
    (want / seqs).backward()  # loss_function's scale: num_microbatches / global_batch_size * dp = 1 / 16
    torch.testing.assert_close(results["auto"][2], sub_logits.grad[0], atol=3e-10, rtol=2.0 ** -6)
    hot = spiked[rows].cpu() & (mask.cpu() != 0)
    assert results["auto"][2][hot].abs().sum() > 0


def test_full_size_grpo_plumbing_case_rewards_to_dlogits():
    """The GRPO plumbing configuration at its stated size: 64 prompts x group 8 = 512 responses x 256 tokens, fp32
    logits [131072, 32000] ~ N(0, 2), Bernoulli(0.4) rewards, a trailing pad of 0..63 masked tokens per response,
    group-normalised advantages (mean / std, eps 1e-6), PPO-clip 0.2, old = lp + N(0, 0.05), token-mean.  Rewards ->
    advantages against the oracle for all 512 responses; log-probs, loss share and dlogits of 12 whole responses
    (3072 rows, picked across the batch) against the oracle run on those rows; for every row: masked rows exactly zero,
    gradient rows summing to zero."""
    from types import SimpleNamespace

    import relax_amd
    from oracle import advantages as A
    from relax_amd import utils as U

    dev = require_gpu()
    prompts, group, resp_len, v = 64, 8, 256, 32000
    seqs, n = prompts * group, prompts * group * resp_len
    announce("GRPO plumbing case, full size", n, v)
    cpu = torch.Generator().manual_seed(0)
    g = torch.Generator(device=dev).manual_seed(0)
    logits = torch.empty((1, n, v), dtype=torch.float32, device=dev)
    for s0 in range(0, n, 4096):
        logits[0, s0:s0 + 4096] = torch.randn((4096, v), device=dev, generator=g) * 2.0
    rewards = torch.bernoulli(torch.full((seqs,), 0.4), generator=cpu).tolist()
    pads = torch.randint(0, 64, (seqs,), generator=cpu).tolist()
    masks = []
    for pad in pads:
        m = torch.ones(resp_len)
        if pad:
            m[resp_len - pad:] = 0.0
        masks.append(m)
    kw = dict(advantage_estimator="grpo", eps_clip=0.2, eps_clip_high=0.2, rewards_normalization=True,
              grpo_std_normalization=True, n_samples_per_prompt=group, global_batch_size=seqs)
    args = P.make_args(**kw)
    samples = [SimpleNamespace(group_index=i // group, get_reward_value=(lambda _a, r=r: r))
               for i, r in enumerate(rewards)]
    # rewards -> group-normalised rewards -> per-token advantages
    raw, normed = U.post_process_rewards(args, samples, device=dev)
    want_normed = A.group_normalise(rewards, [i // group for i in range(seqs)], group, "grpo", True)
    assert raw == rewards
    torch.testing.assert_close(torch.tensor(normed), want_normed, rtol=1e-6, atol=1e-7)
    toks = [torch.randint(0, v, (resp_len,), device=dev, generator=g) for _ in range(seqs)]
    dmasks = [m.to(dev) for m in masks]
    with torch.no_grad():
        _, out = relax_amd.get_log_probs_and_entropy(logits, args=args, unconcat_tokens=toks,
                                                     total_lengths=[resp_len] * seqs,
                                                     response_lengths=[resp_len] * seqs, with_entropy=False)
    old = [lp + 0.05 * torch.randn(lp.shape, device=dev, generator=g) for lp in out["log_probs"]]
    data = dict(log_probs=old, rewards=normed, loss_masks=dmasks)
    relax_amd.compute_advantages_and_returns(args, data)
    adv = data["advantages"]
    for i in (0, 7, 8, 300, 511):
        assert torch.equal(adv[i].cpu(), torch.full((resp_len,), float(want_normed[i])))
    total_unmasked = float(sum(resp_len - pad for pad in pads))
    batch = dict(unconcat_tokens=toks, total_lengths=[resp_len] * seqs, response_lengths=[resp_len] * seqs,
                 loss_masks=dmasks, advantages=adv, log_probs=old,
                 relax_amd_sample_denominators=torch.full((seqs,), total_unmasked, device=dev))
    logits.requires_grad_()
    loss, met = relax_amd.policy_loss_function(args, batch, logits, None)
    loss.backward()
    assert torch.isfinite(loss) and all(torch.isfinite(x) for x in met.values())
    d = logits.grad[0]
    flat_mask = torch.cat(dmasks)
    for s0 in range(0, n, 16384):
        rows = d[s0:s0 + 16384]
        assert rows.sum(-1).abs().max().item() < 1e-6
        assert (rows[flat_mask[s0:s0 + 16384] == 0] == 0).all()
    # 12 whole responses against the oracle: their rows, their share of the token-mean loss, their gradient rows
    picked = [0, 1, 63, 64, 100, 255, 256, 301, 400, 448, 510, 511]
    rows = torch.cat([torch.arange(i * resp_len, (i + 1) * resp_len) for i in picked])
    sub_logits = logits.detach()[0, rows.to(dev)].cpu().unsqueeze(0).requires_grad_()
    sub = dict(unconcat_tokens=[toks[i].cpu() for i in picked], total_lengths=[resp_len] * len(picked),
               response_lengths=[resp_len] * len(picked), loss_masks=[masks[i] for i in picked],
               advantages=[adv[i].cpu() for i in picked], log_probs=[old[i].cpu() for i in picked])
    reducer = R.make_reducer([resp_len] * len(picked), sub["loss_masks"],
                             sample_denoms=[total_unmasked] * len(picked))
    want, want_met = P.policy_loss_function(args, sub, sub_logits, reducer)
    want.backward()
    torch.testing.assert_close(d[rows.to(dev)].cpu(), sub_logits.grad[0], atol=3e-9, rtol=2e-4)
    # the same 12 responses' share of the loss from the product: a second, small call on just those rows
    lg2 = logits.detach()[0, rows.to(dev)].unsqueeze(0).clone().requires_grad_()
    dsub = {k: ([x.to(dev) for x in val] if isinstance(val, list) and torch.is_tensor(val[0]) else val)
            for k, val in sub.items()}
    dsub["relax_amd_sample_denominators"] = torch.full((len(picked),), total_unmasked, device=dev)
    got, _ = relax_amd.policy_loss_function(args, dsub, lg2, None)
    assert abs(got.item() - want.item()) < 3e-5 * max(1.0, abs(want.item()))


def _cfg4_lengths():
    """The benchmark's packed lengths: 8 draws from U[2048, 32768], the longest halved until the total fits 131072."""
    cpu = torch.Generator().manual_seed(0)
    lengths = [int(x) for x in torch.randint(2048, 32769, (8,), generator=cpu)]
    while sum(lengths) > 131072:
        lengths[lengths.index(max(lengths))] //= 2
    return lengths, cpu


@pytest.mark.parametrize("estimator", ["gspo", "cispo"])
def test_cfg4_full_size_varlen_seq_mean_token_sum_vs_oracle(estimator):
    """The agentic packed configuration at its stated size: 8 sequences of 2k-32k tokens (129 579 rows x 151 936 bf16
    logits, 39.4 GB), 3-6 masked tool-output spans per sequence (~30 % of tokens), RLOO advantages over the group of
    8, GSPO (clip 3e-4 / 4e-4) or CISPO, sequence-mean-token-sum aggregation through the reference's reducer hook.

    Oracle comparison at full size: the per-token losses, the sequence-level ratio, the aggregation, every metric and
    d loss / d log-prob come from the oracle on the [N] log-prob vector (log-probs and entropy themselves are checked
    against the oracle's row arithmetic on sampled rows), and dlogits rows are checked on sampled rows against
    d loss / d log-prob * (onehot - softmax) computed on the CPU.  Plus the size-independent properties: every
    gradient row sums to zero, masked rows are exactly zero."""
    import relax_amd
    from oracle import advantages as OA
    from oracle import logprob as O

    dev = require_gpu()
    v = 151936
    lengths, cpu = _cfg4_lengths()
    n = sum(lengths)
    announce("cfg4 full size", estimator, lengths, n)
    assert 100000 < n <= 131072 and min(lengths) >= 2048 and max(lengths) <= 32768
    g = torch.Generator(device=dev).manual_seed(0)
    logits = torch.empty((1, n, v), dtype=torch.bfloat16, device=dev)
    for s0 in range(0, n, 2048):
        e0 = min(n, s0 + 2048)
        logits[0, s0:e0] = (torch.randn((e0 - s0, v), device=dev, generator=g) * 3.0).to(torch.bfloat16)
    masks = []
    for ln in lengths:
        m = torch.ones(ln)
        spans = int(torch.randint(3, 7, (1,), generator=cpu))
        for _ in range(spans):
            w = int(0.3 * ln / spans)
            st = int(torch.randint(0, ln - w, (1,), generator=cpu))
            m[st:st + w] = 0.0
        masks.append(m)
    frac_masked = 1.0 - sum(float(m.sum()) for m in masks) / n
    assert 0.15 < frac_masked < 0.35
    rewards = torch.rand(8, generator=cpu)
    shaped = OA.rloo_leave_one_out(rewards)
    toks = [torch.randint(0, v, (ln,), device=dev, generator=g) for ln in lengths]
    kw = dict(advantage_estimator=estimator, custom_pg_loss_reducer_function_path=
              "relax_amd.cp_utils.get_seq_mean_token_sum_reducer")
    kw.update(dict(eps_clip=3e-4, eps_clip_high=4e-4) if estimator == "gspo" else dict(eps_clip=0.2, eps_clip_high=0.28))
    args = P.make_args(**kw)
    with torch.no_grad():
        _, out = relax_amd.get_log_probs_and_entropy(logits, args=args, unconcat_tokens=toks, total_lengths=lengths,
                                                     response_lengths=lengths, with_entropy=True)
    lp_gpu = torch.cat(out["log_probs"])
    ent_gpu = torch.cat(out["entropy"])
    # old log-probs: a small per-sequence drift plus token noise, so that GSPO's sequence ratios straddle its clip range
    drift = (torch.rand(8, generator=cpu) - 0.5) * 1.2e-3
    old = [lp.cpu() + drift[i] + 0.02 * torch.randn(lp.shape, generator=cpu) for i, lp in enumerate(out["log_probs"])]
    batch = dict(unconcat_tokens=toks, total_lengths=lengths, response_lengths=lengths,
                 loss_masks=[m.to(dev) for m in masks],
                 advantages=[shaped[i].to(dev).expand(ln).contiguous() for i, ln in enumerate(lengths)],
                 log_probs=[o.to(dev) for o in old])
    logits.requires_grad_()
    loss, met = relax_amd.policy_loss_function(args, batch, logits, None)
    loss.backward()
    d = logits.grad[0]

    # (1) log-probs / entropy of sampled rows against the oracle's row arithmetic
    idx = torch.arange(0, n, 997, device=dev)
    # response == total: the reference's SFT convention, row t scores token t + 1 and the last row token 0
    all_toks = torch.cat([torch.cat([t[1:], t.new_zeros(1)]) for t in toks])
    xs = logits.detach()[0][idx].cpu()
    rlp, rent = O.calculate_log_probs_and_entropy(xs, all_toks[idx].cpu(), None, with_entropy=True)
    torch.testing.assert_close(lp_gpu[idx].cpu(), rlp.squeeze(-1), atol=2e-3, rtol=0)
    torch.testing.assert_close(ent_gpu[idx].cpu(), rent, atol=2e-3, rtol=0)

    # (2) the oracle's composition on the [N] vectors: loss, metrics, d loss / d log-prob
    from oracle import losses as L

    lp_cpu = lp_gpu.cpu().double().requires_grad_()
    lps = list(torch.split(lp_cpu, lengths))
    olds = [o.double() for o in old]
    adv = torch.cat([shaped[i].double().expand(ln) for i, ln in enumerate(lengths)])
    dmasks = [m.double() for m in masks]
    if estimator == "gspo":
        ppo_kl = L.gspo_seq_kl(lps, olds, dmasks)
        pg, clipfrac = L.policy_clip(ppo_kl, adv, args.eps_clip, args.eps_clip_high)
    else:
        ppo_kl = torch.cat(olds) - lp_cpu
        pg, clipfrac = L.cispo(lp_cpu, ppo_kl, adv, args.eps_clip, args.eps_clip_high)
    sample_mean = R.make_reducer(lengths, dmasks)
    want_pg = R.seq_mean_token_sum(lengths, dmasks)(pg)
    want_ent = sample_mean(ent_gpu.cpu().double())
    want_loss = want_pg - args.entropy_coef * want_ent
    want_loss.backward()
    want = {"loss": want_loss, "pg_loss": want_pg, "entropy_loss": want_ent, "pg_clipfrac": sample_mean(clipfrac),
            "ppo_kl": sample_mean(ppo_kl)}
    want = {k: float(w.detach()) for k, w in want.items()}
    assert set(met) == set(want)
    for k, w in want.items():
        assert abs(met[k].item() - w) < 2e-3 * max(1.0, abs(w)), (k, met[k].item(), w)
    assert abs(loss.item() - want["loss"]) < 2e-3 * max(1.0, abs(want["loss"]))
    if estimator == "gspo":  # the case exercises both sides of the clip
        assert 0.0 < want["pg_clipfrac"] / 8 < 1.0
    dlp = lp_cpu.grad.float()

    # (3) sampled dlogits rows: dlp_t * (onehot(target) - softmax(row)); rows of masked tokens are exactly zero
    p = torch.softmax(xs.float(), dim=-1)
    hot = torch.zeros_like(p)
    hot[torch.arange(idx.numel()), all_toks[idx].cpu()] = 1.0
    want_rows = dlp[idx.cpu()][:, None] * (hot - p)
    got_rows = d[idx].float().cpu()
    torch.testing.assert_close(got_rows, want_rows, atol=2e-3, rtol=BF16_ULP)
    assert want_rows.abs().max().item() > 1e-3  # the comparison is not of zeros
    flat_mask = torch.cat(masks).to(dev)
    for s0 in range(0, n, 8192):
        e0 = min(n, s0 + 8192)
        blk = d[s0:e0]
        assert (blk[flat_mask[s0:e0] == 0] == 0).all()
        assert blk.float().sum(-1).abs().max().item() < 5e-2
    assert torch.isfinite(loss)


def test_get_log_probs_and_entropy_topk_outputs_vs_oracle():
    """``gather_topk_token_ids`` (per-sample [R_i, K_i] ids, ragged K as on the union path, one sample without ids) and
    ``with_topk`` through the packed launch: values per sample, and the gradient of a loss that mixes the sampled-token
    log-probs with the gathered ones."""
    import relax_amd
    from oracle import opd as D

    dev = require_gpu()
    announce("packed top-K outputs")
    tot, resp, v = [9, 6, 12, 7], [4, 6, 7, 5], 300   # sample 1 is SFT-shaped (response == total)
    logits, batch = _make_batch(5, tot, resp, v)
    g = torch.Generator().manual_seed(1)
    widths = [5, 0, 3, 5]
    ids = [torch.randint(0, v, (r, w), generator=g) if w else None for r, w in zip(resp, widths)]
    ids[0][0, 0] = -1
    up = [torch.randn(r, w, generator=g) for r, w in zip(resp, widths)]
    args = P.make_args(rollout_temperature=0.8)
    lo = logits.clone().requires_grad_()
    want, loss_w = [], 0.0
    for i, (chunk, targets) in enumerate(P.iter_responses(lo, batch["unconcat_tokens"], tot, resp)):
        x = chunk / 0.8
        lp = torch.log_softmax(x, -1).gather(-1, targets[:, None]).squeeze(-1)
        loss_w = loss_w + lp.sum() * 0.01
        if ids[i] is None:
            want.append(torch.zeros(resp[i], 0))
            continue
        t = D.log_probs_on_topk_ids(x, ids[i])
        want.append(t.detach())
        loss_w = loss_w + (t.masked_fill(ids[i] < 0, 0.0) * up[i]).sum()
    loss_w.backward()
    lg = logits.to(dev).requires_grad_()
    _, out = relax_amd.get_log_probs_and_entropy(
        lg, args=args, unconcat_tokens=[t.to(dev) for t in batch["unconcat_tokens"]], total_lengths=tot,
        response_lengths=resp, with_entropy=False, with_topk=True, topk_k=4,
        gather_topk_token_ids=[None if x is None else x.to(dev) for x in ids])
    loss = sum(lp.sum() for lp in out["log_probs"]) * 0.01
    for i, t in enumerate(out["topk_log_probs"]):
        assert t.shape == (resp[i], widths[i])
        if widths[i]:
            fin = ids[i] >= 0
            torch.testing.assert_close(t.detach().cpu()[fin], want[i][fin], atol=3e-5, rtol=0)
            loss = loss + (t.masked_fill((ids[i] < 0).to(dev), 0.0) * up[i].to(dev)).sum()
    assert torch.isinf(out["topk_log_probs"][0][0, 0])
    loss.backward()
    torch.testing.assert_close(lg.grad.cpu(), lo.grad, atol=3e-5, rtol=1e-5)
    for i, (chunk, _) in enumerate(P.iter_responses(logits, batch["unconcat_tokens"], tot, resp)):
        got = out["topk_token_ids"][i].cpu()
        assert got.shape == (resp[i], 4)
        # same top-4 values (ties could permute the ids)
        torch.testing.assert_close(chunk.gather(-1, got), torch.topk(chunk, 4, dim=-1).values)


@pytest.mark.parametrize("case", ["sampled_plain", "sampled_clips", "sampled_clamped", "sampled_clips_all_tokens",
                                  "sampled_clamped_all_tokens", "student_topk_forward", "union_jsd",
                                  "teacher_topk_reverse_tail", "topk_low_var_clips_all_tokens",
                                  "topk_norm_clamped_clips_all_tokens", "topk_ragged_widths", "topk_clips_masked"])
@pytest.mark.parametrize("single_pass", ["auto", "off"])
def test_policy_loss_with_opd_term_vs_oracle(case, single_pass):
    """``opd_loss_coef != 0``: the distillation term (sampled-token or top-K, union mask, per-token and
    importance-ratio clips) added to the policy loss -- loss, metrics and dlogits against the oracle."""
    import relax_amd

    dev = require_gpu()
    announce("policy loss + OPD", case, single_pass)
    tot, resp, v = [9, 6, 12, 7], [4, 3, 7, 5], 264
    logits, batch = _make_batch(31, tot, resp, v)
    g = torch.Generator().manual_seed(2)
    kw = dict(relax_amd_single_pass=single_pass, opd_loss_coef=0.7, use_kl_loss=True, kl_loss_coef=0.01,
              kl_loss_type="k3")
    if case.endswith("_all_tokens"):
        # no masked token at all (with masked tokens the single launch scans their rows as well: the clip-fraction
        # metrics average over them)
        batch["loss_masks"] = [torch.ones_like(m) for m in batch["loss_masks"]]
        case = case[:-len("_all_tokens")]
    if case == "sampled_plain":  # linear in the log-probs: its gradient leaves with the single launch
        kw.update(opd_token_selection="sampled", opd_kl_type="reverse_kl")
        batch["teacher_log_probs"] = [lp + 0.2 * torch.randn(lp.shape, generator=g) for lp in batch["log_probs"]]
    elif case == "sampled_clamped":  # clamp from below on both log-probs, ratio clip, no old log-probs in the batch
        kw.update(opd_token_selection="sampled", opd_kl_type="reverse_kl", opd_log_prob_min_clamp=-1.5,
                  opd_is_clip=1.02, opd_per_token_clip=0.1)
        batch["teacher_log_probs"] = [lp + 0.2 * torch.randn(lp.shape, generator=g) for lp in batch["log_probs"]]
    elif case == "sampled_clips":
        kw.update(opd_token_selection="sampled", opd_kl_type="low_var_kl", opd_per_token_clip=0.02, opd_is_clip=1.01)
        batch["teacher_log_probs"] = [lp + 0.2 * torch.randn(lp.shape, generator=g) for lp in batch["log_probs"]]
    else:
        k = 6
        batch["opd_topk_token_ids"] = [torch.randint(0, v, (r, k), generator=g) for r in resp]
        batch["opd_topk_teacher_log_probs"] = [torch.log_softmax(torch.randn(r, v, generator=g), -1)[:, :k].contiguous()
                                               for r in resp]
        if case == "student_topk_forward":
            kw.update(opd_token_selection="student_topk", opd_kl_type="forward_kl", opd_norm_mode="tail")
        elif case == "teacher_topk_reverse_tail":
            kw.update(opd_token_selection="teacher_topk", opd_kl_type="reverse_kl", opd_norm_mode="tail")
        elif case == "topk_low_var_clips":  # every token unmasked: the clips are applied inside the single launch
            kw.update(opd_token_selection="teacher_topk", opd_kl_type="low_var_kl", opd_per_token_clip=8.0,
                      opd_is_clip=1.01, opd_log_prob_min_clamp=-9.0)
        elif case == "topk_norm_clamped_clips":
            kw.update(opd_token_selection="student_topk", opd_kl_type="jsd", opd_jsd_alpha=0.3, opd_norm_mode="norm",
                      opd_log_prob_min_clamp=-7.0, opd_per_token_clip=0.5, opd_is_clip=0.99)
        elif case == "topk_clips_masked":  # clips with masked tokens: the launch scans the masked rows as well
            kw.update(opd_token_selection="teacher_topk", opd_kl_type="reverse_kl", opd_per_token_clip=0.5)
        elif case == "topk_ragged_widths":  # samples with different K: packed to the widest, trimmed per token
            kw.update(opd_token_selection="teacher_topk", opd_kl_type="jsd", opd_jsd_alpha=0.6, opd_norm_mode="tail")
            for i, w in enumerate([6, 3, 5, 1]):
                batch["opd_topk_token_ids"][i] = batch["opd_topk_token_ids"][i][:, :w].contiguous()
                batch["opd_topk_teacher_log_probs"][i] = batch["opd_topk_teacher_log_probs"][i][:, :w].contiguous()
        else:
            kw.update(opd_token_selection="union", opd_kl_type="jsd", opd_jsd_alpha=0.4, opd_norm_mode="trunc",
                      opd_log_prob_min_clamp=-12.0)
            batch["opd_topk_ksz"] = [torch.randint(1, k + 1, (r,), generator=g) for r in resp]
    args = P.make_args(**kw)
    lo = logits.clone().requires_grad_()
    want_loss, want_m = P.policy_loss_function(args, dict(batch), lo, R.make_reducer(resp, batch["loss_masks"]))
    want_loss.backward()
    lg = logits.to(dev).requires_grad_()
    loss, met = relax_amd.policy_loss_function(args, _to_dev(batch, dev), lg, None)
    loss.backward()
    assert abs(loss.item() - want_loss.item()) < 3e-5 * max(1.0, abs(want_loss.item()))
    assert set(met) == set(want_m), (sorted(met), sorted(want_m))
    for key, w in want_m.items():
        assert abs(met[key].item() - float(w)) < 3e-5 * max(1.0, abs(float(w))), (key, met[key].item(), float(w))
    torch.testing.assert_close(lg.grad.cpu(), lo.grad, atol=3e-5, rtol=1e-5)


@pytest.mark.parametrize("v,dtype,k,variant", [(100352, torch.bfloat16, 64, "reverse_tail"),
                                               (100352, torch.bfloat16, 200, "union_jsd_clips"),
                                               (151936, torch.bfloat16, 64, "forward_norm"),
                                               (32000, torch.float32, 96, "low_var"),
                                               # K = 1, just past one wave's width, and the largest the launch takes:
                                               # how the one-shot kernel's workgroups share the gather of a row's ids
                                               (100352, torch.bfloat16, 1, "forward_norm"),
                                               (163840, torch.bfloat16, 65, "union_jsd_clips"),
                                               (151936, torch.bfloat16, 256, "reverse_tail"),
                                               # rows of 31 vectors per thread: sixteen of them in LDS, no persistent
                                               # kernel to compare with
                                               (248320, torch.bfloat16, 64, "reverse_tail"),
                                               # fp32 rows of 38 vectors per thread, sixteen of them in LDS
                                               (151936, torch.float32, 64, "union_jsd_clips"),
                                               # rows scanned by 512 virtual threads: four workgroups share a row and
                                               # the gather of its K ids
                                               (32000, torch.bfloat16, 70, "forward_norm")])
def test_topk_opd_term_in_the_register_resident_step(v, dtype, k, variant):
    """The top-K distillation term inside the single launch on the row shapes of the register-resident kernel (several
    rows per persistent workgroup, K below and above one wave's width, the union mask, clips): loss, metrics and
    dlogits against the two-launch path and against the oracle; the default kernel (one-shot workgroups sharing each
    row) and the persistent one bit for bit."""
    import relax_amd
    from relax_amd import ops

    dev = require_gpu()
    announce("top-K OPD in the resident step", v, dtype, k, variant)
    g = torch.Generator().manual_seed(v + k)
    n_samples = 12 if dtype != torch.float32 else 30
    tot = [int(x) for x in torch.randint(20, 60, (n_samples,), generator=g)]
    resp = [int(torch.randint(1, t, (1,), generator=g)) for t in tot]
    logits, batch = _make_batch(37, tot, resp, v, dtype)
    kw = dict(opd_loss_coef=0.6, eps_clip_high=0.28, use_kl_loss=True, kl_loss_coef=1e-3, kl_loss_type="k3",
              entropy_coef=0.01)
    batch["opd_topk_token_ids"] = [torch.stack([torch.randperm(v, generator=g)[:k] for _ in range(r)]) for r in resp]
    batch["opd_topk_teacher_log_probs"] = [torch.log_softmax(2 * torch.randn(r, 4 * k, generator=g), -1)[:, :k]
                                           .contiguous() for r in resp]
    if variant == "reverse_tail":
        kw.update(opd_token_selection="teacher_topk", opd_kl_type="reverse_kl", opd_norm_mode="tail")
        batch["loss_masks"][2] = torch.zeros_like(batch["loss_masks"][2])
    elif variant == "union_jsd_clips":
        kw.update(opd_token_selection="union", opd_kl_type="jsd", opd_jsd_alpha=0.4, opd_norm_mode="trunc",
                  opd_log_prob_min_clamp=-14.0, opd_per_token_clip=0.05, opd_is_clip=1.01)
        batch["opd_topk_ksz"] = [torch.randint(1, k + 1, (r,), generator=g) for r in resp]
        batch["loss_masks"][1] = torch.zeros_like(batch["loss_masks"][1])  # masked rows are scanned: clip metrics
    elif variant == "forward_norm":
        kw.update(opd_token_selection="student_topk", opd_kl_type="forward_kl", opd_norm_mode="norm")
    else:
        kw.update(opd_token_selection="teacher_topk", opd_kl_type="low_var_kl", opd_log_prob_min_clamp=-11.0)
    db = _to_dev(batch, dev)
    outs = {}
    for mode in ("auto", "off"):
        lg = logits.to(dev).requires_grad_()
        loss, met = relax_amd.policy_loss_function(P.make_args(relax_amd_single_pass=mode, **kw), db, lg, None)
        loss.backward()
        outs[mode] = (loss.detach(), met, lg.grad)
    # the persistent kernel, or for rows it is not built for the two-walk kernel, bit for bit
    has_resident = v <= 65536 if dtype == torch.float32 else 57352 <= v <= 163840
    ops.set_kernel_choice("resident" if has_resident else "two_walk")
    try:
        lg = logits.to(dev).requires_grad_()
        loss, met = relax_amd.policy_loss_function(P.make_args(relax_amd_single_pass="auto", **kw), db, lg, None)
        loss.backward()
    finally:
        ops.set_kernel_choice("auto")
    assert torch.equal(loss.detach(), outs["auto"][0]) and torch.equal(lg.grad, outs["auto"][2])
    for key, w in outs["auto"][1].items():
        assert torch.equal(met[key], w), key
    if variant == "reverse_tail":
        # the exchange of the one-shot kernel forced to give up from the host (triples and gathered logits alike):
        # NaN instead of a hang, and the launch after it exact again
        from relax_amd._lib import check, lib
        check(lib.relax_amd_set_exchange_wait(4, 1))
        try:
            lg = logits.to(dev).requires_grad_()
            loss, _ = relax_amd.policy_loss_function(P.make_args(relax_amd_single_pass="auto", **kw), db, lg, None)
            torch.cuda.synchronize()
        finally:
            check(lib.relax_amd_set_exchange_wait(0, 0))
        assert torch.isnan(loss).all()
        lg = logits.to(dev).requires_grad_()
        loss, _ = relax_amd.policy_loss_function(P.make_args(relax_amd_single_pass="auto", **kw), db, lg, None)
        loss.backward()
        assert torch.equal(loss.detach(), outs["auto"][0]) and torch.equal(lg.grad, outs["auto"][2])
    ulp = {torch.bfloat16: 2.0 ** -7, torch.float32: 1e-5}[dtype]
    assert abs(outs["auto"][0].item() - outs["off"][0].item()) < 1e-5 * max(1.0, abs(outs["off"][0].item()))
    assert set(outs["auto"][1]) == set(outs["off"][1])
    for key, w in outs["off"][1].items():
        assert abs(outs["auto"][1][key].item() - w.item()) < 1e-5 * max(1.0, abs(w.item())), key
    torch.testing.assert_close(outs["auto"][2].float(), outs["off"][2].float(), atol=2e-6, rtol=2 * ulp)
    lo = logits.float().clone().requires_grad_()
    want, want_m = P.policy_loss_function(P.make_args(**kw), dict(batch), lo, R.make_reducer(resp, batch["loss_masks"]))
    want.backward()
    tol = 2e-3 if dtype != torch.float32 else 5e-5
    assert abs(outs["auto"][0].item() - want.item()) < tol * max(1.0, abs(want.item()))
    for key, w in want_m.items():
        assert abs(outs["auto"][1][key].item() - float(w)) < tol * max(1.0, abs(float(w))), key
    torch.testing.assert_close(outs["auto"][2].float().cpu(), lo.grad, atol=tol, rtol=max(2 * ulp, 1e-5))


@pytest.mark.parametrize("k", [1, 63, 65, 256, 300])
def test_topk_opd_term_widths_of_the_single_launch(k, monkeypatch):
    """K = 1, around one wave's width, the largest K the single launch takes and one beyond it (two launches), with
    repeated ids in a row: loss, metrics and dlogits against the oracle, and which launches ran."""
    import relax_amd
    from relax_amd import ops

    dev = require_gpu()
    announce("top-K OPD widths", k)
    tot, resp, v = [9, 6, 12, 7], [4, 3, 7, 5], 3000
    logits, batch = _make_batch(41, tot, resp, v)
    g = torch.Generator().manual_seed(k)
    batch["opd_topk_token_ids"] = [torch.randint(0, v, (r, k), generator=g) for r in resp]
    batch["opd_topk_token_ids"][2][1, 0] = batch["opd_topk_token_ids"][2][1, k - 1]  # a repeated id (k > 1)
    batch["opd_topk_teacher_log_probs"] = [torch.log_softmax(torch.randn(r, 2 * k + 3, generator=g), -1)[:, :k]
                                           .contiguous() for r in resp]
    args = P.make_args(opd_loss_coef=0.7, opd_token_selection="teacher_topk", opd_kl_type="jsd", opd_jsd_alpha=0.5,
                       opd_norm_mode="trunc", use_kl_loss=True, kl_loss_coef=0.01, kl_loss_type="k3")
    calls = []
    for name in ("actor_step_fused", "logprob_entropy_fwd", "logprob_entropy_bwd"):
        real = getattr(ops, name)
        monkeypatch.setattr(ops, name, lambda *a, _n=name, _r=real, **kw: (calls.append(_n), _r(*a, **kw))[1])
    lo = logits.clone().requires_grad_()
    want_loss, want_m = P.policy_loss_function(args, dict(batch), lo, R.make_reducer(resp, batch["loss_masks"]))
    want_loss.backward()
    lg = logits.to(dev).requires_grad_()
    loss, met = relax_amd.policy_loss_function(args, _to_dev(batch, dev), lg, None)
    loss.backward()
    assert calls == (["actor_step_fused"] if k <= 256 else ["logprob_entropy_fwd", "logprob_entropy_bwd"]), calls
    assert abs(loss.item() - want_loss.item()) < 3e-5 * max(1.0, abs(want_loss.item()))
    assert set(met) == set(want_m)
    for key, w in want_m.items():
        assert abs(met[key].item() - float(w)) < 3e-5 * max(1.0, abs(float(w))), key
    torch.testing.assert_close(lg.grad.cpu(), lo.grad, atol=3e-5, rtol=1e-5)


@pytest.mark.parametrize("seed", range(24))
def test_topk_opd_term_random_option_sweep_vs_oracle(seed):
    """Random draws over the top-K term's options (KL family and jsd_alpha, norm mode, lower clamp, per-token and
    importance-ratio clips, selection with and without the union mask, ragged per-sample K, masked tokens and a fully
    masked sample, temperature, per-token-loss reduction) through the single launch: loss, metrics and dlogits against
    the oracle."""
    import relax_amd

    dev = require_gpu()
    g = torch.Generator().manual_seed(1000 + seed)

    def pick(options):
        return options[int(torch.randint(0, len(options), (1,), generator=g))]

    tot, resp = [9, 6, 12, 7, 5], [4, 3, 7, 5, 2]
    v = pick([264, 1000, 3001])
    k = pick([1, 3, 8, 70])
    logits, batch = _make_batch(50 + seed, tot, resp, v)
    kl_type = pick(["reverse_kl", "forward_kl", "jsd", "low_var_kl"])
    selection = pick(["teacher_topk", "student_topk", "union"])
    kw = dict(opd_loss_coef=pick([0.3, 1.0]), opd_token_selection=selection, opd_kl_type=kl_type,
              opd_jsd_alpha=pick([0.2, 0.5, 0.9]), opd_norm_mode=pick(["tail", "norm", "trunc"]),
              opd_log_prob_min_clamp=pick([None, -6.0, -12.0]), opd_per_token_clip=pick([None, 0.05, 2.0]),
              opd_is_clip=pick([None, 0.99, 1.05]), rollout_temperature=pick([1.0, 0.7]),
              calculate_per_token_loss=pick([False, True]), use_kl_loss=True, kl_loss_coef=0.01, kl_loss_type="k3",
              entropy_coef=pick([0.0, 0.01]))
    if selection == "union" and kw["opd_norm_mode"] == "norm":
        kw["opd_norm_mode"] = "tail"  # the reference's autograd returns NaN for masked entries under "norm"
    announce("top-K OPD option sweep", seed, v, k, kl_type, selection, kw["opd_norm_mode"])
    widths = [k] * len(resp)
    if pick([False, True]) and k > 1:
        widths = [int(torch.randint(1, k + 1, (1,), generator=g)) for _ in resp]
    batch["opd_topk_token_ids"] = [torch.stack([torch.randperm(v, generator=g)[:w] for _ in range(r)])
                                   for r, w in zip(resp, widths)]
    batch["opd_topk_teacher_log_probs"] = [torch.log_softmax(2 * torch.randn(r, 3 * w + 2, generator=g), -1)[:, :w]
                                           .contiguous() for r, w in zip(resp, widths)]
    if selection == "union":
        batch["opd_topk_ksz"] = [torch.randint(1, w + 1, (r,), generator=g) for r, w in zip(resp, widths)]
    if pick([False, True]):
        batch["loss_masks"][1] = torch.zeros_like(batch["loss_masks"][1])
    args = P.make_args(**kw)
    lo = logits.clone().requires_grad_()
    want_loss, want_m = P.policy_loss_function(args, dict(batch), lo, R.make_reducer(resp, batch["loss_masks"],
                                                                                     kw["calculate_per_token_loss"]))
    want_loss.backward()
    lg = logits.to(dev).requires_grad_()
    loss, met = relax_amd.policy_loss_function(args, _to_dev(batch, dev), lg, None)
    loss.backward()
    assert abs(loss.item() - want_loss.item()) < 5e-5 * max(1.0, abs(want_loss.item())), (loss.item(), want_loss.item())
    assert set(met) == set(want_m), (sorted(met), sorted(want_m))
    for key, w in want_m.items():
        assert abs(met[key].item() - float(w)) < 5e-5 * max(1.0, abs(float(w))), (key, met[key].item(), float(w))
    torch.testing.assert_close(lg.grad.cpu(), lo.grad, atol=5e-5, rtol=2e-5)


def test_linear_opd_term_rides_the_single_launch(monkeypatch):
    """Sampled-token distillation signals (plain reverse_kl: linear in the log-probs; low_var_kl or clipped: derivative
    evaluated by the kernel) and the top-K signals (evaluated by the kernel next to each row's log-sum-exp): one fused
    launch, no separate log-prob or dlogits launch; with clips on a batch that has masked tokens the launch scans the
    masked rows too (their clip-fraction metrics need those log-probs) and is still the only one."""
    import relax_amd
    from relax_amd import ops

    dev = require_gpu()
    announce("linear OPD term: launches")
    tot, resp, v = [9, 6, 12, 7], [4, 3, 7, 5], 264
    logits, batch = _make_batch(32, tot, resp, v)
    g = torch.Generator().manual_seed(4)
    batch["teacher_log_probs"] = [lp + 0.2 * torch.randn(lp.shape, generator=g) for lp in batch["log_probs"]]
    calls = []
    for name in ("actor_step_fused", "logprob_entropy_fwd", "logprob_entropy_bwd"):
        real = getattr(ops, name)
        monkeypatch.setattr(ops, name, lambda *a, _n=name, _r=real, **k: (calls.append(_n), _r(*a, **k))[1])
    ones = [torch.ones_like(m) for m in batch["loss_masks"]]
    for kl_type, clip, masks, want in (
            ("reverse_kl", None, None, ["actor_step_fused"]), ("low_var_kl", None, None, ["actor_step_fused"]),
            ("reverse_kl", 0.02, ones, ["actor_step_fused"]), ("reverse_kl", 0.02, None, ["actor_step_fused"])):
        calls.clear()
        case_batch = batch if masks is None else dict(batch, loss_masks=masks)
        args = P.make_args(opd_loss_coef=0.7, opd_token_selection="sampled", opd_kl_type=kl_type,
                           opd_per_token_clip=clip)
        lg = logits.to(dev).requires_grad_()
        loss, _ = relax_amd.policy_loss_function(args, _to_dev(case_batch, dev), lg, None)
        loss.backward()
        assert calls == want, (kl_type, clip, calls)
    k = 5
    batch["opd_topk_token_ids"] = [torch.randint(0, v, (r, k), generator=g) for r in resp]
    batch["opd_topk_teacher_log_probs"] = [torch.log_softmax(torch.randn(r, v, generator=g), -1)[:, :k].contiguous()
                                           for r in resp]
    for kl_type, clip, masks, want in (("reverse_kl", None, None, ["actor_step_fused"]),
                                       ("jsd", 0.5, ones, ["actor_step_fused"]),
                                       ("jsd", 0.5, None, ["actor_step_fused"])):
        calls.clear()
        case_batch = batch if masks is None else dict(batch, loss_masks=masks)
        args = P.make_args(opd_loss_coef=0.7, opd_token_selection="teacher_topk", opd_kl_type=kl_type,
                           opd_jsd_alpha=0.5, opd_norm_mode="tail", opd_per_token_clip=clip)
        lg = logits.to(dev).requires_grad_()
        loss, _ = relax_amd.policy_loss_function(args, _to_dev(case_batch, dev), lg, None)
        loss.backward()
        assert calls == want, ("top-K", kl_type, clip, calls)


def test_outputs_leave_as_one_packed_copy_in_the_reference_wire_format():
    """What the forward-only pass returns goes to the data system as jagged nested tensors on the host
    (relax/backends/megatron/actor.py:2351-2363): the per-sample lists are views of one packed vector, so the packed
    vector is what crosses PCIe, and the result equals the list-based construction of the reference."""
    import relax_amd
    from relax_amd import data_fields as DF

    dev = require_gpu()
    announce("wire format of forward-only outputs")
    tot, resp, v = [9, 6, 12, 7], [4, 3, 7, 5], 1000
    logits, batch = _make_batch(5, tot, resp, v, torch.bfloat16)
    db = _to_dev(batch, dev)
    ids = [torch.randint(0, v, (r, 3), device=dev) for r in resp]
    with torch.no_grad():
        _, out = relax_amd.get_log_probs_and_entropy(
            logits.to(dev), args=P.make_args(), unconcat_tokens=db["unconcat_tokens"], total_lengths=tot,
            response_lengths=resp, with_entropy=True, gather_topk_token_ids=ids)
    assert DF._packed_parent(out["log_probs"]) is not None and DF._packed_parent(out["entropy"]) is not None
    payload = DF.to_transfer_payload(out)
    for key, items in out.items():
        want = torch.nested.as_nested_tensor([t.cpu() for t in items], layout=torch.jagged)
        got = payload[key]
        assert got.is_nested and got.layout == torch.jagged and got.device.type == "cpu"
        for a, b in zip(got.unbind(), want.unbind()):
            assert a.dtype == b.dtype and torch.equal(a, b)


def test_callable_from_worker_threads_and_under_activation_checkpointing():
    """The reference runs this path from worker threads (ActorFwd / Advantages services: threading.Thread,
    asyncio.to_thread; relax/components/actor_fwd.py:56-66) and may wrap the loss in torch.utils.checkpoint
    (relax/backends/megatron/loss.py:1535-1543, the forward then runs twice): results must not depend on the calling
    thread, concurrent callers must not disturb each other, and the recomputed forward must be deterministic."""
    import threading

    import relax_amd
    from torch.utils.checkpoint import checkpoint

    dev = require_gpu()
    announce("worker threads + checkpoint")
    tot, resp, v = [40, 25, 33, 18], [20, 11, 30, 9], 3000
    logits, batch = _make_batch(31, tot, resp, v, torch.bfloat16)
    db = _to_dev(batch, dev)
    args = P.make_args(eps_clip_high=0.28, use_kl_loss=True, kl_loss_coef=1e-3, kl_loss_type="k3", entropy_coef=0.01)
    from relax_amd.cp_utils import get_sum_of_sample_mean

    red = get_sum_of_sample_mean(tot, resp, db["loss_masks"])

    def run():
        lg = logits.to(dev).requires_grad_()
        loss, metrics = relax_amd.policy_loss_function(args, db, lg, red)
        loss.backward()
        return loss.detach().clone(), lg.grad.clone(), {k: m.clone() for k, m in metrics.items()}

    want = run()
    results, errors = {}, []

    def worker(i):
        try:
            with torch.cuda.stream(torch.cuda.Stream(device=dev)):  # default priority; each thread its own stream
                for _ in range(5):
                    results[i] = run()
                torch.cuda.current_stream().synchronize()
        except Exception as exc:  # surfaced below: an exception inside a thread would otherwise be lost
            errors.append(exc)

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(3)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for i in range(3):
        loss, grad, metrics = results[i]
        assert torch.equal(loss, want[0]) and torch.equal(grad, want[1])
        assert all(torch.equal(metrics[k], want[2][k]) for k in want[2])

    lg = logits.to(dev).requires_grad_()
    loss = checkpoint(lambda x: relax_amd.policy_loss_function(args, db, x, red)[0], lg, use_reentrant=False)
    loss.backward()
    assert torch.equal(loss.detach(), want[0]) and torch.equal(lg.grad, want[1])


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-5), (torch.bfloat16, 2e-3)])
@pytest.mark.parametrize("per_token", [False, True])
def test_sft_loss_single_launch_equals_two_launch_path_and_oracle(dtype, tol, per_token):
    """sft_loss_function with a gradient wanted runs as one launch of the fused step (REINFORCE surrogate with unit
    advantages); ``relax_amd_single_pass="off"`` keeps the separate forward / backward launches.  Both against the
    oracle's -sum_of_sample_mean(log_probs), SFT-shaped (response == total) and RL-shaped samples mixed, a
    temperature other than 1, an upstream gradient other than 1; no-grad calls return the same loss."""
    import relax_amd

    dev = require_gpu()
    announce("sft single launch", dtype, per_token)
    tot, resp, v = [7, 12, 5, 9], [7, 5, 5, 4], 264
    logits, batch = _make_batch(19, tot, resp, v, dtype)
    lo = logits.float().clone().requires_grad_()
    oargs = P.make_args(loss_type="sft", rollout_temperature=0.8, calculate_per_token_loss=per_token)
    _, out = P.get_log_probs_and_entropy(lo, args=oargs, unconcat_tokens=batch["unconcat_tokens"], total_lengths=tot,
                                         response_lengths=resp)
    want = -R.make_reducer(resp, batch["loss_masks"], per_token)(torch.cat(out["log_probs"]))
    (1.7 * want).backward()
    bd = _to_dev(batch, dev)
    got = {}
    for mode in ("auto", "off"):
        args = P.make_args(loss_type="sft", rollout_temperature=0.8, calculate_per_token_loss=per_token,
                           relax_amd_single_pass=mode)
        lg = logits.to(dev).requires_grad_()
        loss, log = relax_amd.sft_loss_function(args, bd, lg, None)
        (1.7 * loss).backward()
        assert list(log) == ["loss"] and log["loss"].item() == loss.item()
        assert abs(loss.item() - want.item()) < tol * max(1.0, abs(want.item())), (mode, loss.item(), want.item())
        assert lg.grad.dtype == dtype
        torch.testing.assert_close(lg.grad.float().cpu(), lo.grad, atol=tol, rtol=BF16_ULP if dtype == torch.bfloat16 else 0)
        got[mode] = (loss.item(), lg.grad)
        with torch.no_grad():
            quiet, _ = relax_amd.sft_loss_function(args, bd, logits.to(dev), None)
        assert abs(quiet.item() - loss.item()) < 1e-6 * max(1.0, abs(loss.item()))
    assert abs(got["auto"][0] - got["off"][0]) < 1e-6 * max(1.0, abs(want.item()))
    torch.testing.assert_close(got["auto"][1].float(), got["off"][1].float(), atol=tol * 1e-2,
                               rtol=2 * BF16_ULP if dtype == torch.bfloat16 else 1e-5)


def test_sft_eval_step_sums_and_counts_vs_oracle():
    """The SFT evaluation callback (relax/engine/sft/eval/ppl.py:24-92): masked sum of negative log-probs and the
    exact token count per micro-batch, in the shapes and dtypes the forward-only harness stacks."""
    from relax_amd.sft_eval import compute_ppl_metrics, compute_sft_eval_step

    dev = require_gpu()
    announce("sft eval step")
    tot, resp, v = [9, 6, 12], [9, 3, 12], 500     # SFT-shaped samples (response == total) and one RL-shaped
    logits, batch = _make_batch(9, tot, resp, v, torch.bfloat16, int_masks=True)
    db = _to_dev(batch, dev)
    empty, out = compute_sft_eval_step(logits.to(dev), args=P.make_args(), unconcat_tokens=db["unconcat_tokens"],
                                       total_lengths=tot, response_lengths=resp, loss_masks=db["loss_masks"],
                                       dynamic_cp_size=None, dynamic_cp_rank=None, max_seq_lens=None)
    assert empty.shape == (0,) and empty.device.type == "cuda"
    s, n = out["sum_neg_log_prob"][0], out["num_tokens"][0]
    assert s.shape == (1,) and s.dtype == torch.float32 and n.shape == (1,) and n.dtype == torch.long
    _, ref = P.get_log_probs_and_entropy(logits.float(), args=P.make_args(), unconcat_tokens=batch["unconcat_tokens"],
                                         total_lengths=tot, response_lengths=resp)
    masks = torch.cat([m.float() for m in batch["loss_masks"]])
    want = -(torch.cat(ref["log_probs"]) * masks).sum()
    assert n.item() == int(masks.sum().item())
    assert abs(s.item() - want.item()) < 2e-3 * max(1, n.item())
    m = compute_ppl_metrics(s.item(), n.item())
    assert abs(m["eval/loss"] - want.item() / masks.sum().item()) < 2e-3


@pytest.mark.parametrize("case", ["vanilla_vs_fused", "icepop", "rejecting_tis_and_token_mean", "reinforce_pp_custom_reducer"])
def test_custom_tis_and_reducer_hooks(case):
    """``--custom-tis-function-path`` / ``--custom-pg-loss-reducer-function-path`` (loss.py:1036-1072): the loss is
    composed around the user's callables.  With the library's own ``vanilla_tis_function`` named as the custom
    function the composed path must reproduce the single-kernel path; the other cases are checked against the oracle's
    composition with the same plug-ins."""
    import relax_amd
    from oracle import losses as L

    dev = require_gpu()
    announce("custom hooks", case)
    tot, resp, v = [11, 8, 14, 9], [6, 5, 9, 4], 700
    logits, batch = _make_batch(41, tot, resp, v, torch.float32)
    db = _to_dev(batch, dev)
    base = dict(use_tis=True, tis_clip=1.05, tis_clip_low=0.95, use_kl_loss=True, kl_loss_coef=0.05, kl_loss_type="k3",
                entropy_coef=0.01, custom_tis_function_path=None, custom_pg_loss_reducer_function_path=None)
    oracle_kw = {}
    if case == "vanilla_vs_fused":
        args = P.make_args(**{**base, "custom_tis_function_path": "relax_amd.loss.vanilla_tis_function"})
    elif case == "icepop":
        args = P.make_args(**{**base, "custom_tis_function_path": "relax_amd.loss.icepop_function"})
        oracle_kw = dict(
            tis_fn=lambda pg, tr, ro, masks: (*L.icepop(pg, tr, ro, 0.95, 1.05)[:1], masks, L.icepop(pg, tr, ro, 0.95, 1.05)[1]),
            rebuild_reducer=lambda masks: R.make_reducer(resp, masks))
    elif case == "rejecting_tis_and_token_mean":
        from tests import custom_hooks as H

        args = P.make_args(**{**base, "custom_tis_function_path": "tests.custom_hooks.rejecting_tis",
                              "custom_pg_loss_reducer_function_path": "tests.custom_hooks.token_mean_reducer"})

        def tis_fn(pg, tr, ro, masks):
            return H.rejecting_tis(None, pg_loss=pg, train_log_probs=[tr], rollout_log_probs=[ro], loss_masks=masks)

        oracle_kw = dict(tis_fn=tis_fn, rebuild_reducer=lambda masks: R.make_reducer(resp, masks),
                         pg_reducer_factory=lambda masks: H.token_mean_reducer(tot, resp, masks, False))
    else:
        from tests import custom_hooks as H

        args = P.make_args(**{**base, "use_tis": False, "advantage_estimator": "reinforce_plus_plus",
                              "custom_pg_loss_reducer_function_path": "tests.custom_hooks.token_mean_reducer"})
        oracle_kw = dict(pg_reducer_factory=lambda masks: H.token_mean_reducer(tot, resp, masks, False))

    lg = logits.to(dev).requires_grad_()
    loss, metrics = relax_amd.policy_loss_function(args, db, lg, None)
    loss.backward()

    if case == "vanilla_vs_fused":
        fused_args = P.make_args(**base)
        lg2 = logits.to(dev).requires_grad_()
        want_loss, want_metrics = relax_amd.policy_loss_function(fused_args, db, lg2, None)
        want_loss.backward()
        want_grad = lg2.grad.cpu()
        want_metrics = {k: m.cpu() for k, m in want_metrics.items()}
        want_loss = want_loss.detach().cpu()
    else:
        lref = logits.clone().requires_grad_()
        want_loss, want_metrics = P.policy_loss_function(args, batch, lref, R.make_reducer(resp, batch["loss_masks"]),
                                                         **oracle_kw)
        want_loss.backward()
        want_grad, want_loss = lref.grad, want_loss.detach()
    assert set(metrics) == set(want_metrics), (sorted(metrics), sorted(want_metrics))
    torch.testing.assert_close(loss.detach().cpu(), want_loss, atol=3e-5, rtol=1e-5)
    for k in want_metrics:
        torch.testing.assert_close(metrics[k].cpu().float(), want_metrics[k].float(), atol=3e-5, rtol=1e-4, msg=k)
    torch.testing.assert_close(lg.grad.cpu(), want_grad, atol=3e-5, rtol=1e-4)


def test_custom_loss_function_path_dispatch():
    """``--loss-type custom_loss --custom-loss-function-path`` (loss.py:1530-1531): the plug-in is loaded by dotted path
    and called with the library's reducer; scaling and the logging dict are those of the built-in losses."""
    import relax_amd

    dev = require_gpu()
    announce("custom loss dispatch")
    tot, resp, v = [11, 8, 14], [6, 5, 9], 400
    logits, batch = _make_batch(43, tot, resp, v, torch.float32)
    db = _to_dev(batch, dev)
    args = P.make_args(loss_type="custom_loss", custom_loss_function_path="tests.custom_hooks.negative_log_likelihood",
                       global_batch_size=3)
    lg = logits.to(dev).requires_grad_()
    loss, norm, log = relax_amd.loss_function(args, db, 2, lg)
    loss.backward()
    lref = logits.clone().requires_grad_()
    _, out = P.get_log_probs_and_entropy(lref, args=args, unconcat_tokens=batch["unconcat_tokens"], total_lengths=tot,
                                         response_lengths=resp)
    want = -R.make_reducer(resp, batch["loss_masks"])(torch.cat(out["log_probs"])) * 2 / 3
    want.backward()
    torch.testing.assert_close(loss.detach().cpu(), want.detach(), atol=3e-5, rtol=1e-5)
    torch.testing.assert_close(lg.grad.cpu(), lref.grad, atol=3e-5, rtol=1e-4)
    assert log["keys"] == ["loss"] and int(norm) == 1


@pytest.mark.parametrize("v,dtype,n_samples", [(100352, torch.bfloat16, 18), (128256, torch.float16, 18),
                                                (131072, torch.bfloat16, 18), (151936, torch.bfloat16, 18),
                                                (163840, torch.bfloat16, 18), (160000, torch.float16, 18),
                                                (65536, torch.bfloat16, 18), (64000, torch.float16, 20),
                                                (90112, torch.bfloat16, 20), (32000, torch.float32, 40),
                                                (32768, torch.float32, 40), (50304, torch.float32, 30),
                                                (64000, torch.float32, 24), (65536, torch.float32, 24)])
def test_register_resident_step_over_many_rows_per_workgroup(v, dtype, n_samples):
    """More logits rows than persistent workgroups, so every workgroup of the register-resident kernel rolls several
    rows through its registers (prompt rows, fully masked samples and masked tokens in between), for every row shape
    the kernel is built for (7 / 12 / 15 / 18 / 19 full vectors per thread plus a partial one, 8 / 16 / 20 exactly; fp32 rows
    of 7 / 12 / 15 plus a partial one, 8 / 16 exactly) and one it is not (90112, 11 exactly: two-walk kernel): same loss bits as the two-launch path, gradients equal to it and to the oracle."""
    import relax_amd

    dev = require_gpu()
    announce("register-resident step, many rows", v, dtype, n_samples)
    g = torch.Generator().manual_seed(v + n_samples)
    tot = [int(x) for x in torch.randint(20, 60, (n_samples,), generator=g)]
    resp = [int(torch.randint(1, t, (1,), generator=g)) for t in tot]
    logits, batch = _make_batch(29, tot, resp, v, dtype)
    batch["loss_masks"][3] = torch.zeros_like(batch["loss_masks"][3])
    assert sum(tot) > 600  # more than two rows for each of the 256 persistent workgroups
    db = _to_dev(batch, dev)
    kw = dict(eps_clip_high=0.28, use_kl_loss=True, kl_loss_coef=1e-3, kl_loss_type="k3", entropy_coef=0.01)
    outs = {}
    for mode in ("auto", "off"):
        lg = logits.to(dev).requires_grad_()
        loss, met = relax_amd.policy_loss_function(P.make_args(relax_amd_single_pass=mode, **kw), db, lg, None)
        loss.backward()
        outs[mode] = (loss.detach(), met, lg.grad)
    assert torch.equal(outs["auto"][0], outs["off"][0])
    ulp = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7, torch.float32: 1e-5}[dtype]
    torch.testing.assert_close(outs["auto"][2].float(), outs["off"][2].float(), atol=1e-6, rtol=ulp)
    lo = logits.float().clone().requires_grad_()
    want, _ = P.policy_loss_function(P.make_args(**kw), dict(batch), lo, R.make_reducer(resp, batch["loss_masks"]))
    want.backward()
    tol = 2e-3
    assert abs(outs["auto"][0].item() - want.item()) < tol * max(1.0, abs(want.item()))
    torch.testing.assert_close(outs["auto"][2].float().cpu(), lo.grad, atol=tol, rtol=max(ulp, 1e-5))


@pytest.mark.parametrize("v,dtype,n_rows,values", [
    (100352, torch.bfloat16, 700, "plain"), (32000, torch.float32, 1500, "plain"), (151936, torch.bfloat16, 300, "plain"),
    # 16-bit rows scanned by 512 threads: no persistent kernel exists for them, the one-shot kernel does
    (32000, torch.bfloat16, 1500, "short"), (50304, torch.float16, 1000, "short"),
    # 16-bit rows of more than 20 vectors per thread: the one-shot kernel keeps twelve of them in LDS
    (202048, torch.bfloat16, 300, "short"), (262144, torch.float16, 200, "short"), (248320, torch.bfloat16, 200, "short"),
    # fp32 rows of 248320 entries (the Qwen3.5 vocabulary as stock Megatron hands it to the loss), upper halves
    (248320, torch.float32, 160, "widened_short"), (248320, torch.float32, 160, "mixed_short"),
    # long fp32 rows, kept in the registers as their upper halves: bf16 values widened to fp32 (what a bf16 output
    # layer followed by .float() delivers: one read of the row), fp32 values with low bits (the row is read again), and
    # rows of both kinds next to each other, one of them with a single low bit in its last element
    (151936, torch.float32, 600, "widened"), (151936, torch.float32, 600, "plain"), (151936, torch.float32, 600, "mixed")])
@pytest.mark.parametrize("pattern", ["all_dead", "one_live_last", "few_live", "random", "all_live_no_map",
                                     "zero_advantage"])
def test_register_resident_kernel_equals_two_walk_kernel_bitwise(pattern, v, dtype, n_rows, values):
    """The kernels behind relax_amd_actor_step_fused, switched with relax_amd_set_kernel_choice (two-walk, persistent
    register-resident, and the default: one-shot workgroups that share each row and exchange their partial sums
    through device memory, where built), on row / token layouts that stress the persistent loop of the
    register-resident one and the zero-row path of the others: no live row at all, a single live row at
    the very end, fewer live rows than workgroups, random prompt rows and masked tokens over several rows per
    workgroup, no row map (every row scores its own token), and tokens whose gradient coefficients vanish (zero
    rows without a look at the logits); on 16-bit rows of 12 and of 18 full vectors per thread plus a partial one and on
    fp32 rows of 32000 entries.  Every output must be bit-identical."""
    from relax_amd import ops

    dev = require_gpu()
    announce("resident vs two-walk", pattern, v, dtype)
    g = torch.Generator().manual_seed(len(pattern))
    logits = (torch.randn(n_rows, v, generator=g) * 2).to(dtype)
    no_resident = values.endswith("short")  # (RESIDENT fails for these rows by design)
    if values.startswith(("widened", "mixed")):
        logits = logits.bfloat16().to(dtype)
    if values.startswith("mixed"):
        other = torch.randn(n_rows // 3, v, generator=g) * 2
        logits[1::3][: other.size(0)] = other  # every third row keeps its low bits
        logits[2::3, -1] += 2.0 ** -14         # and the next one differs from a widened row in one bit of one element
    logits = logits.to(dev)
    if pattern == "all_live_no_map":
        token_of_row, n_tok = None, n_rows
    else:
        scores = torch.rand(n_rows, generator=g) > 0.25
        idx = torch.cumsum(scores.int(), 0) - 1
        token_of_row = torch.where(scores, idx, torch.full_like(idx, -1)).int().to(dev)
        n_tok = int(scores.sum())
    mask = (torch.rand(n_tok, generator=g) > 0.2).float()
    if pattern == "all_dead":
        mask.zero_()
    elif pattern == "one_live_last":
        mask.zero_()
        mask[-1] = 1.0
    elif pattern == "few_live":
        mask.zero_()
        mask[torch.randperm(n_tok, generator=g)[:37]] = 1.0
    adv = torch.randn(n_tok, generator=g)
    if pattern == "zero_advantage":
        adv[::3] = 0.0  # PPO-clip without KL or entropy terms: coefficient exactly zero
    base = -2.0 + 0.3 * torch.randn(n_tok, generator=g)
    lens = [n_tok // 3, n_tok - n_tok // 3]
    cu = torch.tensor([0, lens[0], n_tok], dtype=torch.int64, device=dev)
    sample_ids = torch.cat([torch.full((n,), i, dtype=torch.int32) for i, n in enumerate(lens)]).to(dev)
    kw = dict(advantages=adv.to(dev), loss_mask=mask.to(dev), cu_resp=cu, old_log_prob=base.to(dev),
              sample_denom=torch.tensor([max(1.0, mask[:lens[0]].sum().item()), max(1.0, mask[lens[0]:].sum().item())],
                                        device=dev),
              loss_kind="ppo", eps_clip=0.2, eps_clip_high=0.28)
    if pattern != "zero_advantage":
        kw.update(ref_log_prob=(base + 0.1 * torch.randn(n_tok, generator=g)).to(dev), kl_kind="k3", kl_coef=1e-3,
                  entropy_coef=0.01)
    targets = torch.randint(0, v, (n_tok,), generator=g).to(dev)
    results = {}
    for kind in ("cached", "resident", "auto", "auto_again"):
        if no_resident and kind == "resident":
            kind = "auto"
        ops.set_kernel_choice({"cached": "two_walk", "resident": "resident"}.get(kind, "auto"))
        out, lp, ent, lse, spx, d = ops.actor_step_fused(logits, targets, token_of_row, sample_ids, n_tok, 1.0, 1.0, **kw)
        torch.cuda.synchronize()
        results[kind] = dict(lp=lp, ent=ent, lse=lse, spx=spx, coef=out["coef_log_prob"],
                             d=d.view(torch.int16 if dtype != torch.float32 else torch.int32),
                             coef_ent=out["coef_entropy"], metrics=out["metrics"])
    for kind in ("resident", "auto", "auto_again"):
        if kind not in results:
            continue
        for key, want in results["cached"].items():
            got = results[kind][key]
            assert torch.equal(got, want), (kind, pattern, key, (got.float() - want.float()).abs().max())
    if pattern == "all_dead":
        assert not results["auto_again"]["d"].any() and not results["auto"]["d"].any()


@pytest.mark.parametrize("seed", range(16))
def test_one_shot_step_on_random_layouts_equals_two_walk_kernel_bitwise(seed):
    """Random row counts (from a single row up), row lengths from every family the one-shot kernel is built for (and
    their neighbours by one vector), element types, row maps with unscored rows, masks, temperatures and loss options:
    the default kernel choice against the two-walk kernel, every output bit for bit.  Small row counts leave most of
    the chip idle, large ones wrap the exchange ring's 4096 slots."""
    from relax_amd import ops

    dev = require_gpu()
    g = torch.Generator().manual_seed(1000 + seed)
    families = [(torch.bfloat16, 8, [18 * 1024 + 560, 12 * 1024 + 256, 20 * 1024, 16 * 1024, 15 * 1024 + 1023,
                                     7 * 1024 + 832, 8 * 1024, 7 * 512 + 416, 8 * 512, 12 * 512 + 144,
                                     24 * 1024 + 680, 31 * 1024 + 256, 32 * 1024]),
                (torch.float16, 8, [18 * 1024 + 1, 19 * 1024 + 5, 12 * 512 + 1, 30 * 1024 + 640, 24 * 1024 + 1]),
                (torch.float32, 4, [7 * 1024 + 832, 8 * 1024, 12 * 1024 + 3, 16 * 1024, 37 * 1024 + 96, 24 * 1024 + 512])]
    dtype, per_vec, nvecs = families[seed % 3]
    nvec = nvecs[int(torch.randint(0, len(nvecs), (1,), generator=g))]
    v = nvec * per_vec
    budget = 160_000_000 // (v * (4 if dtype == torch.float32 else 2))
    n_rows = [1, 7, 8, 9, 63][seed % 5] if seed < 10 else int(torch.randint(64, max(65, min(budget, 5000)), (1,), generator=g))
    announce("one-shot step, random layout", seed, v, dtype, n_rows)
    logits = (torch.randn(n_rows, v, generator=g) * 2).to(dtype)
    if dtype == torch.float32 and nvec > 20000 and seed % 2 == 0:
        logits = logits.bfloat16().float()  # widened rows: the upper-halves form reads them once
    logits = logits.to(dev)
    if seed % 4 == 3:
        token_of_row, n_tok = None, n_rows
    else:
        scores = torch.rand(n_rows, generator=g) > 0.3
        scores[int(torch.randint(0, n_rows, (1,), generator=g))] = True
        idx = torch.cumsum(scores.int(), 0) - 1
        token_of_row = torch.where(scores, idx, torch.full_like(idx, -1)).int().to(dev)
        n_tok = int(scores.sum())
    mask = (torch.rand(n_tok, generator=g) > 0.25).float()
    base = -11.0 + 0.3 * torch.randn(n_tok, generator=g)
    n_a = max(1, n_tok // 2)
    lens = [n_a, n_tok - n_a] if n_tok > 1 else [1]
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int64, device=dev)
    sample_ids = torch.cat([torch.full((n,), i, dtype=torch.int32) for i, n in enumerate(lens)]).to(dev)
    denom = torch.tensor([max(1.0, mask[sample_ids.cpu() == i].sum().item()) for i in range(len(lens))], device=dev)
    kw = dict(advantages=torch.randn(n_tok, generator=g).to(dev), loss_mask=mask.to(dev), cu_resp=cu,
              old_log_prob=base.to(dev), sample_denom=denom, loss_kind=["ppo", "cispo", "sapo"][seed % 3],
              eps_clip=0.2, eps_clip_high=0.28)
    if seed % 2 == 0:
        kw.update(ref_log_prob=(base + 0.1 * torch.randn(n_tok, generator=g)).to(dev),
                  kl_kind=["k1", "k2", "k3", "low_var_kl"][(seed // 2) % 4], kl_coef=1e-3)
    if seed % 3 != 1:
        kw.update(entropy_coef=0.01)
    targets = torch.randint(0, v, (n_tok,), generator=g).to(dev)
    inv_t = [1.0, 1.0 / 0.7][seed % 2]
    results = {}
    for kind in ("two_walk", "auto"):
        ops.set_kernel_choice(kind)
        out, lp, ent, lse, spx, d = ops.actor_step_fused(logits, targets, token_of_row, sample_ids, n_tok, inv_t, 1.0, **kw)
        torch.cuda.synchronize()
        results[kind] = dict(lp=lp, ent=ent, lse=lse, spx=spx, coef=out["coef_log_prob"], coef_ent=out["coef_entropy"],
                             d=d.view(torch.int16 if dtype != torch.float32 else torch.int32))
    ops.set_kernel_choice("auto")
    for key, want in results["two_walk"].items():
        got = results["auto"][key]
        if want is None:
            assert got is None
            continue
        assert torch.equal(got, want), (seed, key, (got.float() - want.float()).abs().max())
    assert not torch.isnan(results["auto"]["lp"]).any()


@pytest.mark.parametrize("v,dtype", [(151936, torch.bfloat16), (32000, torch.float32), (32000, torch.float16),
                                     (4 * (37 * 1024 + 96), torch.float32), (256000, torch.bfloat16)])
def test_log_probs_and_entropy_of_every_kernel_agree_bitwise_at_a_temperature(v, dtype):
    """The forward-only pass, the log-prob + top-K pass and the fused step in each of its kernels give one set of bits
    for log-prob, entropy, log-sum-exp and sum p*x at a temperature other than 1 (where a product of the temperature
    feeds the entropy's subtraction: written as separate operations the compiler fused it in some kernels and not in
    others).  This is what lets the reference's step-0 check see exactly zero KL between the passes."""
    from relax_amd import ops

    dev = require_gpu()
    announce("one set of bits at T = 0.7", v, dtype)
    g = torch.Generator().manual_seed(v)
    n = 300
    logits = (torch.randn(n, v, generator=g) * 2).to(dtype)
    if dtype == torch.float32 and v > 100000:
        logits = logits.bfloat16().float()
    logits = logits.to(dev)
    targets = torch.randint(0, v, (n,), generator=g).to(dev)
    inv_t = 1.0 / 0.7
    want = dict(zip(("lp", "ent", "lse", "spx"), ops.logprob_entropy_fwd(logits, targets, None, inv_t)))
    got = ops.logprob_entropy_topk_fwd(logits, targets, None, inv_t, 16)
    for key, t in zip(("lp", "ent", "lse", "spx"), got[:4]):
        assert torch.equal(t, want[key]), ("top-K forward", key)
    lp_only = ops.logprob_entropy_fwd(logits, targets, None, inv_t, with_entropy=False)
    assert torch.equal(lp_only[0], want["lp"]) and torch.equal(lp_only[2], want["lse"])
    base = want["lp"].cpu() + 0.05 * torch.randn(n, generator=g)
    kw = dict(advantages=torch.randn(n, generator=g).to(dev), loss_mask=torch.ones(n, device=dev),
              cu_resp=torch.tensor([0, n], dtype=torch.int64, device=dev), old_log_prob=base.to(dev),
              sample_denom=torch.tensor([float(n)], device=dev), loss_kind="ppo", eps_clip=0.2, eps_clip_high=0.28,
              entropy_coef=0.01)
    sample_ids = torch.zeros(n, dtype=torch.int32, device=dev)
    per_vec = 4 if dtype == torch.float32 else 8
    try:
        for kind in ("two_walk", "resident", "auto"):
            # no persistent kernel for rows scanned by 512 threads or of more than 20 vectors per thread
            if kind == "resident" and (v // per_vec < 7168 or (per_vec == 8 and v // per_vec > 20 * 1024)):
                continue
            ops.set_kernel_choice(kind)
            out, lp, ent, lse, spx, d = ops.actor_step_fused(logits, targets, None, sample_ids, n, inv_t, 1.0, **kw)
            torch.cuda.synchronize()
            for key, t in (("lp", lp), ("ent", ent), ("lse", lse), ("spx", spx)):
                assert torch.equal(t, want[key]), (kind, key, (t - want[key]).abs().max())
    finally:
        ops.set_kernel_choice("auto")


@pytest.mark.parametrize("v", [151936, 152064, 154880, 129280, 163840, 248320])
def test_vocabularies_of_the_reference_model_scripts_take_the_one_shot_kernels(v):
    """The vocabulary sizes the reference's model scripts name (scripts/models/*.sh: qwen3-*, qwen25-7B, glm4.7 / glm5,
    kimi-k2.6, qwen35-* / qwen36-* / qwen38-*, and 129280) in bf16 and in the fp32 stock Megatron hands a custom loss:
    the fused actor step, the fused reverse-KL step and the backward-only launch each report the kernel built for the
    shape (relax_amd_last_kernel), not the two-walk kernel that serves every shape."""
    from relax_amd import ops

    dev = require_gpu()
    announce("fast-path coverage", v)
    n = 24
    g = torch.Generator().manual_seed(v)
    mask = (torch.rand(n, generator=g) > 0.2).float()
    kw = dict(advantages=torch.randn(n, generator=g).to(dev), loss_mask=mask.to(dev),
              cu_resp=torch.tensor([0, n], dtype=torch.int64, device=dev),
              old_log_prob=(-12.0 + 0.3 * torch.randn(n, generator=g)).to(dev),
              sample_denom=torch.tensor([max(1.0, mask.sum().item())], device=dev), loss_kind="ppo", eps_clip=0.2,
              eps_clip_high=0.28)
    sample_ids = torch.zeros(n, dtype=torch.int32, device=dev)
    targets = torch.randint(0, v, (n,), generator=g).to(dev)
    for dtype in (torch.bfloat16, torch.float32):
        logits = (torch.randn(n, v, generator=g) * 2).to(dtype).to(dev)
        out, lp, ent, lse, spx, d = ops.actor_step_fused(logits, targets, None, sample_ids, n, 1.0, 1.0, **kw)
        assert ops.last_kernel("actor_step_fused") == "actor_step_split", (dtype, ops.last_kernel("actor_step_fused"))
        ops.logprob_entropy_bwd(logits, targets, lse, spx, torch.ones(n, device=dev), torch.zeros(n, device=dev))
        assert ops.last_kernel("logprob_entropy_bwd") == "logprob_entropy_bwd_chunk"
        assert torch.isfinite(lp[mask.to(dev) != 0]).all()
    s = (torch.randn(n, v, generator=g) * 2).bfloat16().to(dev)
    t = (torch.randn(n, v, generator=g) * 2).bfloat16().to(dev)
    kl, _, _, _ = ops.reverse_kl_step_fused(s, t, torch.ones(n, device=dev), 1.0)
    assert ops.last_kernel("reverse_kl_step_fused") == "reverse_kl_split"
    assert torch.isfinite(kl).all()
    ops.set_kernel_choice("two_walk")
    try:
        ops.actor_step_fused(logits, targets, None, sample_ids, n, 1.0, 1.0, **kw)
        assert ops.last_kernel("actor_step_fused") == "actor_step_fused"
    finally:
        ops.set_kernel_choice("auto")


def test_one_shot_step_gives_up_a_wait_that_cannot_succeed_and_recovers():
    """Failure handling of the exchange between the workgroups of a row, forced from the host
    (relax_amd_set_exchange_wait): with the tag a workgroup waits for offset by one, no wait can succeed; bounded to a
    few looks, every workgroup gives up, writes NaN log-probs / log-sum-exps for its row and exits normally.  The next
    launch with the defaults restored is exact again (tags moved on, nothing of the failed launch is mistaken for
    this one's)."""
    from relax_amd import ops
    from relax_amd._lib import check, lib

    dev = require_gpu()
    announce("one-shot step: give-up path")
    v, n = 100352, 200
    g = torch.Generator().manual_seed(11)
    logits = (torch.randn(n, v, generator=g) * 2).bfloat16().to(dev)
    mask = (torch.rand(n, generator=g) > 0.2).float()
    base = -11.0 + 0.3 * torch.randn(n, generator=g)
    kw = dict(advantages=torch.randn(n, generator=g).to(dev), loss_mask=mask.to(dev),
              cu_resp=torch.tensor([0, n], dtype=torch.int64, device=dev), old_log_prob=base.to(dev),
              sample_denom=torch.tensor([max(1.0, mask.sum().item())], device=dev), loss_kind="ppo", eps_clip=0.2,
              eps_clip_high=0.28, entropy_coef=0.01)
    sample_ids = torch.zeros(n, dtype=torch.int32, device=dev)
    targets = torch.randint(0, v, (n,), generator=g).to(dev)

    def run():
        out, lp, ent, lse, spx, d = ops.actor_step_fused(logits, targets, None, sample_ids, n, 1.0, 1.0, **kw)
        torch.cuda.synchronize()
        return lp, lse, d

    ops.set_kernel_choice("two_walk")
    want = run()
    ops.set_kernel_choice("auto")
    check(lib.relax_amd_set_exchange_wait(4, 1))
    try:
        lp, lse, d = run()
    finally:
        check(lib.relax_amd_set_exchange_wait(0, 0))
    live = (mask != 0).to(dev)
    assert torch.isnan(lp[live]).all() and torch.isnan(lse[live]).all()
    assert (lp[~live] == 0).all() and not d[~live].any()  # rows of masked tokens wait for nobody
    lp, lse, d = run()
    for got, w in zip((lp, lse, d.view(torch.int16)), (want[0], want[1], want[2].view(torch.int16))):
        assert torch.equal(got, w)
    assert lib.relax_amd_set_exchange_wait(-1, 0) != 0


def test_default_fused_step_replayed_from_a_captured_graph():
    """The default fused step tags the partial sums its workgroups exchange with a counter that a small kernel in front
    of the launch advances on the device, so a captured launch gets fresh tags on every replay: three replays on fresh
    logits, with eager launches between them, each bit-identical to the two-walk kernel on the same inputs."""
    from relax_amd import ops

    dev = require_gpu()
    announce("fused step under graph capture")
    v, n_rows = 100352, 300
    g = torch.Generator().manual_seed(5)
    scores = torch.rand(n_rows, generator=g) > 0.25
    idx = torch.cumsum(scores.int(), 0) - 1
    token_of_row = torch.where(scores, idx, torch.full_like(idx, -1)).int().to(dev)
    n_tok = int(scores.sum())
    mask = (torch.rand(n_tok, generator=g) > 0.2).float()
    base = -11.0 + 0.3 * torch.randn(n_tok, generator=g)
    kw = dict(advantages=torch.randn(n_tok, generator=g).to(dev), loss_mask=mask.to(dev),
              cu_resp=torch.tensor([0, n_tok], dtype=torch.int64, device=dev), old_log_prob=base.to(dev),
              ref_log_prob=(base + 0.1 * torch.randn(n_tok, generator=g)).to(dev), kl_kind="k3", kl_coef=1e-3,
              entropy_coef=0.01, sample_denom=torch.tensor([max(1.0, mask.sum().item())], device=dev),
              loss_kind="ppo", eps_clip=0.2, eps_clip_high=0.28)
    sample_ids = torch.zeros(n_tok, dtype=torch.int32, device=dev)
    targets = torch.randint(0, v, (n_tok,), generator=g).to(dev)
    logits = (torch.randn(n_rows, v, generator=g) * 2).bfloat16().to(dev)

    def run():
        out, lp, ent, lse, spx, d = ops.actor_step_fused(logits, targets, token_of_row, sample_ids, n_tok, 1.0, 1.0, **kw)
        return dict(lp=lp, ent=ent, lse=lse, coef=out["coef_log_prob"], d=d.view(torch.int16))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()  # warm-up outside the capture (the library looks its exchange buffer up on first use)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = run()
    for rep in range(3):
        logits.copy_((torch.randn(n_rows, v, generator=g) * 2).bfloat16())
        graph.replay()
        torch.cuda.synchronize()
        got = {k: t.clone() for k, t in captured.items()}
        eager = run()  # an eager launch between the replays
        ops.set_kernel_choice("two_walk")
        want = run()
        ops.set_kernel_choice("auto")
        torch.cuda.synchronize()
        for key in want:
            assert torch.equal(got[key], want[key]), (rep, key)
            assert torch.equal(eager[key], want[key]), (rep, key, "eager")
        assert not torch.isnan(got["lp"]).any()


@pytest.mark.parametrize("v", [128256, 129280, 131072, 152064, 163840, 4 * (31 * 1024 + 1), 4 * (38 * 1024 - 1),
                               100352, 102400, 4 * (24 * 1024 + 1)])
def test_long_fp32_rows_resident_as_upper_halves_equal_two_walk_kernel_and_oracle(v):
    """The other row shapes of the kernel that keeps long fp32 rows as their upper halves (24 / 31 / 37 full vector
    positions per thread plus a partial one, 25, 32 and 40 exactly; an odd number of positions leaves the last register
    quad half used; one lane or all lanes but one at the partial position): widened-bf16 rows and rows with low bits interleaved, every output bit-identical to the two-walk
    kernel's; log-probs, entropy and the gradient of the widened rows against the oracle."""
    from relax_amd import ops

    dev = require_gpu()
    announce("long fp32 rows, upper halves", v)
    n_rows = 330
    g = torch.Generator().manual_seed(v)
    logits = (torch.randn(n_rows, v, generator=g) * 2).bfloat16().float()
    logits[1::2] += torch.randn(n_rows // 2, v, generator=g) * 1e-3  # odd rows: real fp32 values
    logits = logits.to(dev)
    scores = torch.rand(n_rows, generator=g) > 0.2
    idx = torch.cumsum(scores.int(), 0) - 1
    token_of_row = torch.where(scores, idx, torch.full_like(idx, -1)).int().to(dev)
    n_tok = int(scores.sum())
    mask = (torch.rand(n_tok, generator=g) > 0.2).float()
    adv = torch.randn(n_tok, generator=g)
    base = -12.0 + 0.3 * torch.randn(n_tok, generator=g)
    targets = torch.randint(0, v, (n_tok,), generator=g)
    targets[:4] = torch.tensor([0, v - 1, v - 2, 4096 * ((v - 1) // 4096)])  # first / last elements, last position
    cu = torch.tensor([0, n_tok], dtype=torch.int64, device=dev)
    kw = dict(advantages=adv.to(dev), loss_mask=mask.to(dev), cu_resp=cu, old_log_prob=base.to(dev),
              ref_log_prob=(base + 0.1 * torch.randn(n_tok, generator=g)).to(dev), kl_kind="k3", kl_coef=1e-3,
              entropy_coef=0.01, sample_denom=torch.tensor([max(1.0, mask.sum().item())], device=dev),
              loss_kind="ppo", eps_clip=0.2, eps_clip_high=0.28)
    sample_ids = torch.zeros(n_tok, dtype=torch.int32, device=dev)
    results = {}
    for kind in ("two_walk", "resident", "auto"):  # auto: the one-shot form of the same kernel
        ops.set_kernel_choice(kind)
        out, lp, ent, lse, spx, d = ops.actor_step_fused(logits, targets.to(dev), token_of_row, sample_ids, n_tok, 1.0,
                                                         1.0, **kw)
        torch.cuda.synchronize()
        results[kind] = dict(lp=lp, ent=ent, lse=lse, spx=spx, coef=out["coef_log_prob"], d=d.view(torch.int32))
    for kind in ("resident", "auto"):
        for key, want in results["two_walk"].items():
            got = results[kind][key]
            assert torch.equal(got, want), (kind, key, (got.float() - want.float()).abs().max())
    # oracle on the scored rows: log-probs / entropy of every live token, gradient rows of a few tokens
    rows = torch.nonzero(scores).squeeze(1)
    x = logits[rows.to(dev)].cpu()
    ls = torch.log_softmax(x.double(), -1)
    want_lp = ls[torch.arange(n_tok), targets].float()
    want_ent = -(ls.exp() * ls).sum(-1).float()
    live = mask != 0
    torch.testing.assert_close(results["resident"]["lp"].cpu()[live], want_lp[live], atol=2e-5, rtol=0)
    torch.testing.assert_close(results["resident"]["ent"].cpu()[live], want_ent[live], atol=2e-5, rtol=0)
    d = results["resident"]["d"].view(torch.float32)
    coef, coef_ent = out["coef_log_prob"].cpu().double(), out["coef_entropy"].cpu().double()
    for t in [int(i) for i in torch.nonzero(live).squeeze(1)[:6]]:
        p = ls[t].exp()
        onehot = torch.zeros(v, dtype=torch.float64)
        onehot[targets[t]] = 1.0
        want = coef[t] * (onehot - p) + coef_ent[t] * p * ((p * x[t].double()).sum() - x[t].double())
        torch.testing.assert_close(d[rows[t]].cpu().double(), want, atol=2e-6, rtol=1e-4)


@pytest.mark.parametrize("v,dtype", [(8 * (18 * 1024 + 1), torch.bfloat16), (8 * (19 * 1024 - 1), torch.bfloat16),
                                     (8 * (19 * 1024 + 1), torch.bfloat16), (8 * 20 * 1024, torch.float16),
                                     (8 * (12 * 1024 + 1), torch.float16), (8 * (16 * 1024 - 1), torch.bfloat16),
                                     (4 * (7 * 1024 + 1), torch.float32), (4 * (8 * 1024 - 1), torch.float32),
                                     (8 * (7 * 1024 + 1), torch.bfloat16), (8 * 8 * 1024, torch.float16),
                                     (4 * (12 * 1024 + 1), torch.float32), (4 * (16 * 1024 - 1), torch.float32),
                                     # 512 virtual threads: one-shot kernel only
                                     (8 * (7 * 512 + 1), torch.bfloat16), (8 * 8 * 512, torch.float16),
                                     (8 * (13 * 512 - 1), torch.bfloat16)])
def test_register_resident_kernel_at_the_edges_of_its_row_shapes(v, dtype):
    """Row lengths at both ends of a built shape: one lane, or all lanes but one, hold a vector at the partially filled
    position.  Every output bit-identical to the two-walk kernel's."""
    from relax_amd import ops

    dev = require_gpu()
    announce("resident kernel, shape edges", v, dtype)
    n_rows = 600 if dtype != torch.float32 else 1200
    g = torch.Generator().manual_seed(v)
    logits = (torch.randn(n_rows, v, generator=g) * 2).to(dtype).to(dev)
    scores = torch.rand(n_rows, generator=g) > 0.2
    idx = torch.cumsum(scores.int(), 0) - 1
    token_of_row = torch.where(scores, idx, torch.full_like(idx, -1)).int().to(dev)
    n_tok = int(scores.sum())
    mask = (torch.rand(n_tok, generator=g) > 0.2).float()
    base = -2.0 + 0.3 * torch.randn(n_tok, generator=g)
    targets = torch.randint(0, v, (n_tok,), generator=g)
    targets[:4] = torch.tensor([0, v - 1, v - 2, v // 2])  # the row's first and last elements among the targets
    kw = dict(advantages=torch.randn(n_tok, generator=g).to(dev), loss_mask=mask.to(dev),
              cu_resp=torch.tensor([0, n_tok], dtype=torch.int64, device=dev), old_log_prob=base.to(dev),
              ref_log_prob=(base + 0.1 * torch.randn(n_tok, generator=g)).to(dev), kl_kind="k3", kl_coef=1e-3,
              entropy_coef=0.01, sample_denom=torch.tensor([max(1.0, mask.sum().item())], device=dev),
              loss_kind="ppo", eps_clip=0.2, eps_clip_high=0.28)
    sample_ids = torch.zeros(n_tok, dtype=torch.int32, device=dev)
    results = {}
    for kind in ("cached", "resident", "auto"):
        if kind == "resident" and v // (4 if dtype == torch.float32 else 8) < 7168:
            continue  # rows scanned by 512 threads have no persistent kernel
        ops.set_kernel_choice({"cached": "two_walk", "resident": "resident"}.get(kind, "auto"))
        out, lp, ent, lse, spx, d = ops.actor_step_fused(logits, targets.to(dev), token_of_row, sample_ids, n_tok, 1.0,
                                                         1.0, **kw)
        torch.cuda.synchronize()
        results[kind] = dict(lp=lp, ent=ent, lse=lse, spx=spx, coef=out["coef_log_prob"],
                             d=d.view(torch.int16 if dtype != torch.float32 else torch.int32))
    for kind in ("resident", "auto"):
        if kind not in results:
            continue
        for key, want in results["cached"].items():
            assert torch.equal(results[kind][key], want), (kind, key)
    assert results["auto"]["d"].any()


def test_forward_only_topk_gather_on_logits_that_require_grad():
    """The ActorFwd pass runs under ``torch.no_grad()`` on logits that may still carry ``requires_grad``: the top-K
    gather then reuses the log-prob launch's log-sum-exps and returns the same values as the differentiable path."""
    import relax_amd

    dev = require_gpu()
    announce("forward-only top-K gather")
    tot, resp, v, k = [9, 6, 12], [4, 3, 7], 3000, 6
    g = torch.Generator().manual_seed(21)
    logits = (torch.randn(1, sum(tot), v, generator=g) * 2).to(dev).requires_grad_()
    toks = [torch.randint(0, v, (n,), generator=g).to(dev) for n in tot]
    ids = [torch.randint(0, v, (r, k), generator=g).to(dev) for r in resp]
    args = P.make_args(rollout_temperature=0.8)
    kw = dict(args=args, unconcat_tokens=toks, total_lengths=tot, response_lengths=resp, with_entropy=True,
              gather_topk_token_ids=ids)
    with torch.no_grad():
        _, quiet = relax_amd.get_log_probs_and_entropy(logits, **kw)
    _, loud = relax_amd.get_log_probs_and_entropy(logits, **kw)
    for key in ("log_probs", "entropy", "topk_log_probs"):
        for a, b in zip(quiet[key], loud[key]):
            assert not a.requires_grad
            torch.testing.assert_close(a, b.detach(), atol=1e-6, rtol=1e-6)
    assert loud["topk_log_probs"][0].requires_grad
