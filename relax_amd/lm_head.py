"""Fused LM-head projection + log-prob / entropy on the gfx950 matrix cores.

Counterpart of the deferred-LM-head branch of ``get_log_probs_and_entropy`` (relax/backends/megatron/loss.py:391-419)
and ``_bypass_output_layer`` (relax/backends/megatron/model.py:93-181): instead of a callable that materialises
``[sub_chunk, V]`` logits per sub-chunk, the caller passes the hidden states and the LM-head weight and the
``[N, V]`` logits never reach HBM.  Unlike the reference's chunked path, entropy is available too.
"""

from __future__ import annotations

import ctypes as C

import torch

from . import _lib
from ._lib import check, lib
from . import ops
from .ops import _need_gpu, _p, _stream

# rows of the transposed-gradient slab the backward materialises at a time: [V, SLAB] bf16 (10 GB at V = 151936:
# sized for 288 GB of HBM, so the usual micro-batch is one slab and dweight needs no cross-slab accumulation)
BACKWARD_SLAB = 32768

# Largest [V, N] bf16 logits slab (bytes) the forward pass may keep for the backward pass when the caller leaves
# ``keep_logits`` undecided.  0 = never: the logits stay out of HBM and the backward pass projects a second time.
# Keeping them trades V * N * 2 bytes (10 GB at V = 151936, N = 32768) for one of the four GEMM-sized kernels of a step.
KEEP_LOGITS_MAX_BYTES = 0


def _bf16_rows(t: torch.Tensor, what: str) -> torch.Tensor:
    if t.dim() != 2:
        raise ValueError(f"{what} must be 2-D, got {tuple(t.shape)}")
    if t.dtype != torch.bfloat16:
        raise TypeError(f"{what} must be bfloat16 (got {t.dtype}); cast before calling, as the reference's "
                        f"_chunked_call casts the hidden states to the weight dtype")
    if t.stride(1) != 1 or t.stride(0) % 8 != 0 or t.data_ptr() % 16 != 0:
        t = t.contiguous()
    return t


def lmhead_logprob_fwd(hidden, weight, targets, inv_temperature: float = 1.0, with_entropy: bool = True,
                       logits_t=None):
    """Returns (log_prob, entropy | None, lse, spx | None), fp32 [N].  ``logits_t`` ([V, >= N] bf16, token contiguous),
    when given, receives the bf16 logits and the statistics are taken from those rounded values."""
    dev = _need_gpu(hidden, weight, targets)
    n, h = hidden.shape
    v = weight.size(0)
    if weight.size(1) != h:
        raise ValueError(f"hidden size mismatch: hidden {tuple(hidden.shape)} vs weight {tuple(weight.shape)}")
    kw = dict(dtype=torch.float32, device=dev)
    lp, lse = torch.empty(n, **kw), torch.empty(n, **kw)
    ent = torch.empty(n, **kw) if with_entropy else None
    spx = torch.empty(n, **kw) if with_entropy else None
    if n == 0:
        return lp, ent, lse, spx
    ws = torch.empty(lib.relax_amd_lmhead_workspace_bytes(n), dtype=torch.uint8, device=dev)
    with ops._timed("lmhead_logprob_fwd"):
        if logits_t is None:
            check(lib.relax_amd_lmhead_logprob_fwd(_p(hidden), _p(weight), _lib.BF16, n, h, v, hidden.stride(0),
                                                   weight.stride(0), _p(targets), float(inv_temperature), _p(ws),
                                                   _p(lp), _p(ent), _p(lse), _p(spx), _stream()))
        else:
            if logits_t.dtype != torch.bfloat16 or logits_t.dim() != 2 or logits_t.size(0) != v \
                    or logits_t.size(1) < n or logits_t.stride(1) != 1:
                raise ValueError(f"logits_t must be bf16 [V={v}, >= {n}] with contiguous tokens, "
                                 f"got {logits_t.dtype} {tuple(logits_t.shape)} strides {logits_t.stride()}")
            check(lib.relax_amd_lmhead_logprob_fwd_keep(_p(hidden), _p(weight), _lib.BF16, n, h, v, hidden.stride(0),
                                                        weight.stride(0), _p(targets), float(inv_temperature), _p(ws),
                                                        _p(lp), _p(ent), _p(lse), _p(spx), _p(logits_t),
                                                        logits_t.stride(0), _stream()))
    return lp, ent, lse, spx


def lmhead_dlogits_from_logits_t(logits_t, n, targets, lse, spx, g_lp, g_ent, inv_temperature: float):
    """Turns the kept bf16 logits ``[V, >= n]`` into d loss / d logits in place and returns the ``[V, n]`` view."""
    with ops._timed("lmhead_dlogits_inplace"):
        check(lib.relax_amd_lmhead_dlogits_from_logits_t(_p(logits_t), n, logits_t.size(0), logits_t.stride(0),
                                                         _p(targets), _p(lse), _p(spx), _p(g_lp), _p(g_ent), None,
                                                         float(inv_temperature), _stream()))
    return logits_t[:, :n]


def lmhead_dlogits_t(hidden, weight, targets, lse, spx, g_lp, g_ent, inv_temperature: float, out=None):
    """bf16 [V, n] slab of d loss / d logits for the ``n`` rows of ``hidden`` (transposed: token-contiguous)."""
    n, h = hidden.shape
    v = weight.size(0)
    if out is None:
        out = torch.empty((v, n), dtype=torch.bfloat16, device=hidden.device)
    with ops._timed("lmhead_dlogits_t"):
        check(lib.relax_amd_lmhead_dlogits_t(_p(hidden), _p(weight), _lib.BF16, n, h, v, hidden.stride(0),
                                             weight.stride(0), _p(targets), _p(lse), _p(spx), _p(g_lp), _p(g_ent),
                                             None, float(inv_temperature), _p(out), out.stride(0), _stream()))
    return out


def _ceil128(x: int) -> int:
    return (x + 127) // 128 * 128


def alloc_slab(vocab: int, n_tokens: int, device) -> torch.Tensor:
    """The bf16 gradient slab ``[ceil128(vocab), ceil128(n_tokens)]`` the backward GEMMs read, with its padding rows
    and columns cleared (the kernels that fill it never write there); ``slab[:vocab, :n_tokens]`` is the payload."""
    slab = torch.empty((_ceil128(vocab), _ceil128(n_tokens)), dtype=torch.bfloat16, device=device)
    if slab.size(0) > vocab:
        slab[vocab:].zero_()
    if slab.size(1) > n_tokens:
        slab[:, n_tokens:].zero_()
    return slab


GEMM_OUT_BF16, GEMM_OUT_F32, GEMM_OUT_F32_ACCUMULATE = 0, 1, 2


def _gemm_out(out: torch.Tensor, accumulate: bool) -> int:
    if out.dtype == torch.bfloat16 and not accumulate:
        return GEMM_OUT_BF16
    if out.dtype == torch.float32:
        return GEMM_OUT_F32_ACCUMULATE if accumulate else GEMM_OUT_F32
    raise TypeError(f"output must be bfloat16, or float32 (required to accumulate), got {out.dtype}")


def lmhead_dhidden(slab: torch.Tensor, n_tokens: int, weight: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """``out[n, h] = sum_v slab[v, n] * weight[v, h]`` on the matrix cores; ``slab`` as ``alloc_slab`` lays it out."""
    v, h = weight.shape
    with ops._timed("lmhead_dhidden_gemm"):
        check(lib.relax_amd_lmhead_dhidden(_p(slab), slab.size(0), slab.stride(0), _p(weight), weight.stride(0),
                                           n_tokens, h, v, _p(out), out.stride(0), _gemm_out(out, False), _stream()))
    return out


def lmhead_dweight(slab: torch.Tensor, n_tokens: int, hidden: torch.Tensor, vocab: int, out: torch.Tensor,
                   accumulate: bool = False) -> torch.Tensor:
    """``out[v, h] (+)= sum_n slab[v, n] * hidden[n, h]`` on the matrix cores."""
    with ops._timed("lmhead_dweight_gemm"):
        check(lib.relax_amd_lmhead_dweight(_p(slab), slab.stride(0), _p(hidden), hidden.stride(0), n_tokens,
                                           hidden.size(1), vocab, _p(out), out.stride(0), _gemm_out(out, accumulate),
                                           _stream()))
    return out


class FusedLMHeadLogProb(torch.autograd.Function):
    """(hidden [N,H] bf16, weight [V,H] bf16, targets [N]) -> (log_prob [N], entropy [N]).

    Backward recomputes the logits slab by slab on the matrix cores, emits d loss / d logits for the slab in bf16
    (never the full [N, V] tensor) and contracts it with the weight (dhidden) and the hidden states (dweight) with
    the library's own matrix-core kernels, which read the slab, the weight and the hidden states in the layouts they
    have; dweight is accumulated in fp32 across slabs.  With ``keep_logits`` the forward pass writes
    the bf16 logits, transposed, into the slab the backward pass needs anyway, and the backward pass turns them into
    the gradient in place instead of projecting again (one backward pass only: the slab is consumed).
    """

    @staticmethod
    def forward(ctx, hidden, weight, targets, inv_temperature, with_entropy, with_entropy_grad, keep_logits=False):
        with_entropy_grad = bool(with_entropy and with_entropy_grad)
        hidden, weight = _bf16_rows(hidden, "hidden"), _bf16_rows(weight, "weight")
        if targets.dtype != torch.int64 or not targets.is_contiguous():
            targets = targets.to(torch.int64).contiguous()
        n, v = hidden.size(0), weight.size(0)
        ctx.logits_t = None
        if keep_logits and n > 0 and (ctx.needs_input_grad[0] or ctx.needs_input_grad[1]):
            ctx.logits_t = alloc_slab(v, n, hidden.device)
        lp, ent, lse, spx = lmhead_logprob_fwd(hidden, weight, targets, inv_temperature, with_entropy,
                                               None if ctx.logits_t is None else ctx.logits_t[:v])
        ctx.save_for_backward(hidden, weight, targets, lse, spx if with_entropy_grad else None)
        ctx.inv_temperature = inv_temperature
        ctx.with_entropy_grad = with_entropy_grad
        if ent is None:
            ent = lp.new_zeros((0,))
        if not with_entropy_grad:
            ctx.mark_non_differentiable(ent)
        return lp, ent

    @staticmethod
    def backward(ctx, g_lp, g_ent):
        hidden, weight, targets, lse, spx = ctx.saved_tensors
        if g_lp is None:
            raise RuntimeError("FusedLMHeadLogProb expected a materialized grad_log_prob")
        g_lp = g_lp.reshape(-1).to(torch.float32).contiguous()
        if not ctx.with_entropy_grad or g_ent is None or g_ent.numel() == 0:
            g_ent = None
        else:
            g_ent = g_ent.reshape(-1).to(torch.float32).contiguous()
        n, h = hidden.shape
        v = weight.size(0)
        need_h, need_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        d_hidden = torch.empty_like(hidden) if need_h else None
        if n == 0:  # an empty micro-batch: nothing flows back
            return d_hidden, (torch.zeros_like(weight) if need_w else None), None, None, None, None, None
        if ctx.logits_t is not None:
            if ctx.logits_t is False:
                raise RuntimeError("FusedLMHeadLogProb(keep_logits=True) supports one backward pass: the kept logits "
                                   "were overwritten with their gradient by the first one")
            slab = ctx.logits_t
            lmhead_dlogits_from_logits_t(slab[:v], n, targets, lse, spx, g_lp, g_ent, ctx.inv_temperature)
            ctx.logits_t = False
            if need_h:
                lmhead_dhidden(slab, n, weight, d_hidden)
            d_weight = lmhead_dweight(slab, n, hidden, v, torch.empty_like(weight)) if need_w else None
            return d_hidden, d_weight, None, None, None, None, None
        slab = alloc_slab(v, min(n, BACKWARD_SLAB), hidden.device)
        single = n <= BACKWARD_SLAB
        d_weight = None
        if need_w:  # accumulated in fp32 when the micro-batch spans several slabs
            d_weight = torch.empty_like(weight) if single else torch.empty(weight.shape, dtype=torch.float32,
                                                                            device=weight.device)
        for s in range(0, n, BACKWARD_SLAB):
            e = min(n, s + BACKWARD_SLAB)
            cnt = e - s
            if s > 0 and cnt < slab.size(1):
                slab[:, cnt:_ceil128(cnt)].zero_()  # a shorter last slab: its padding columns hold the previous one
            lmhead_dlogits_t(hidden[s:e], weight, targets[s:e], lse[s:e], None if spx is None else spx[s:e],
                             g_lp[s:e], None if g_ent is None else g_ent[s:e], ctx.inv_temperature,
                             out=slab[:v, :cnt])
            if need_h:
                lmhead_dhidden(slab, cnt, weight, d_hidden[s:e])
            if need_w:
                lmhead_dweight(slab, cnt, hidden[s:e], v, d_weight, accumulate=s > 0)
        if need_w and not single:
            d_weight = d_weight.to(weight.dtype)
        return d_hidden, d_weight, None, None, None, None, None


def lm_head_log_probs_and_entropy(hidden, weight, tokens, temperature: float = 1.0, with_entropy: bool = False,
                                  with_entropy_grad: bool = True, keep_logits: bool | None = None):
    """``(log_prob [N] fp32, entropy [N] fp32 | None)`` of ``log_softmax(hidden @ weight.T / temperature)``.

    ``keep_logits``: True keeps a ``[V, N]`` bf16 copy of the logits between forward and backward (faster backward,
    V * N * 2 bytes), False never does, None decides by ``KEEP_LOGITS_MAX_BYTES``.

    The kernels consume the hidden size in pairs of 64-wide slices; other sizes are zero-padded here (zeros add nothing to
    the logits, and autograd through the padding returns gradients of the original shapes)."""
    pad = (-hidden.size(-1)) % 128
    if pad:
        hidden = torch.nn.functional.pad(hidden, (0, pad))
        weight = torch.nn.functional.pad(weight, (0, pad))
    if keep_logits is None:
        keep_logits = 2 * hidden.size(0) * weight.size(0) <= KEEP_LOGITS_MAX_BYTES
    lp, ent = FusedLMHeadLogProb.apply(hidden, weight, tokens, 1.0 / float(temperature), bool(with_entropy),
                                       bool(with_entropy_grad), bool(keep_logits))
    return lp, (ent if with_entropy else None)


# tokens per slab of the no-recompute step below: the bf16 logits of one slab, [V, STEP_SLAB] (2.5 GB at V = 151936),
# are the only logits in HBM at any time
STEP_SLAB = 8192


class _FusedLMHeadTokenLocalStep(torch.autograd.Function):
    """(hidden [N,H] bf16, weight [V,H] bf16, targets [N]) -> (loss, log_prob [N], entropy [N]) for a loss that is a
    sum of per-token terms whose weights do not depend on other tokens' log-probs (SFT, REINFORCE / PPO-clip with
    fixed normalisers): the whole step runs inside forward, one slab of tokens at a time, and never projects twice.

    Per slab: the forward kernel writes the slab's bf16 logits [V, slab] next to its log-probs / entropy; the caller's
    ``token_loss`` turns those log-probs into the slab's share of the loss, whose derivative w.r.t. them (autograd over
    [slab]-sized vectors) is the coefficient vector; the logits become d loss / d logits in place; dhidden of the slab
    and the slab's addition to dweight (fp32 across slabs) follow on the matrix cores.  Backward only rescales the two
    gradients when the upstream gradient differs from ``assumed_scale``.
    """

    @staticmethod
    def forward(ctx, hidden, weight, targets, inv_temperature, with_entropy, token_loss, slab_tokens, assumed_scale):
        hidden, weight = _bf16_rows(hidden, "hidden"), _bf16_rows(weight, "weight")
        if targets.dtype != torch.int64 or not targets.is_contiguous():
            targets = targets.to(torch.int64).contiguous()
        n, v = hidden.size(0), weight.size(0)
        need_h, need_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        slab_tokens = max(128, _ceil128(min(int(slab_tokens), max(n, 1))))
        dev = hidden.device
        lp_all = torch.empty(n, dtype=torch.float32, device=dev)
        ent_all = torch.empty(n if with_entropy else 0, dtype=torch.float32, device=dev)
        loss = torch.zeros((), dtype=torch.float32, device=dev)
        slab = alloc_slab(v, min(n, slab_tokens), dev) if (need_h or need_w) and n > 0 else None
        d_hidden = torch.empty_like(hidden) if need_h else None
        single = n <= slab_tokens
        d_weight = None
        if need_w:
            d_weight = torch.zeros_like(weight) if n == 0 else (
                torch.empty_like(weight) if single else torch.empty(weight.shape, dtype=torch.float32, device=dev))
        for s in range(0, n, slab_tokens):
            e = min(n, s + slab_tokens)
            cnt = e - s
            lp, ent, lse, spx = lmhead_logprob_fwd(hidden[s:e], weight, targets[s:e], inv_temperature, with_entropy,
                                                   None if slab is None else slab[:v])
            lp_all[s:e] = lp
            if with_entropy:
                ent_all[s:e] = ent
            with torch.enable_grad():
                lp_leaf = lp.detach().requires_grad_()
                ent_leaf = ent.detach().requires_grad_() if with_entropy else None
                part = token_loss(s, e, lp_leaf, ent_leaf)
                if slab is not None:
                    leaves = [lp_leaf] + ([ent_leaf] if with_entropy else [])
                    grads = torch.autograd.grad(part, leaves, allow_unused=True)
            loss = loss + part.detach().to(torch.float32)
            if slab is None:
                continue
            g_lp = grads[0] if grads[0] is not None else torch.zeros_like(lp)
            g_ent = grads[1] if with_entropy and grads[1] is not None else None
            if assumed_scale != 1.0:
                g_lp = g_lp * assumed_scale
                g_ent = None if g_ent is None else g_ent * assumed_scale
            g_lp = g_lp.to(torch.float32).contiguous()
            g_ent = None if g_ent is None else g_ent.to(torch.float32).contiguous()
            lmhead_dlogits_from_logits_t(slab[:v], cnt, targets[s:e], lse, spx if g_ent is not None else None, g_lp,
                                         g_ent, inv_temperature)
            if s > 0 and cnt < slab.size(1):
                # a shorter last slab: columns past its last 16-byte vector still hold the previous slab's gradient
                slab[:, (cnt + 7) // 8 * 8:_ceil128(cnt)].zero_()
            if need_h:
                lmhead_dhidden(slab, cnt, weight, d_hidden[s:e])
            if need_w:
                lmhead_dweight(slab, cnt, hidden[s:e], v, d_weight, accumulate=s > 0)
        if need_w and n > 0 and not single:
            d_weight = d_weight.to(weight.dtype)
        ctx.grads = (d_hidden, d_weight)
        ctx.assumed_scale = float(assumed_scale)
        ctx.mark_non_differentiable(lp_all, ent_all)
        return loss, lp_all, ent_all

    @staticmethod
    def backward(ctx, g_loss, _glp, _gent):
        if ctx.grads is None:
            raise RuntimeError("the fused LM-head step holds its gradients once: backward cannot run twice")
        d_hidden, d_weight = ctx.grads
        ctx.grads = None
        factor = g_loss.reshape(1).to(torch.float32)
        if ctx.assumed_scale != 1.0:
            factor = factor / ctx.assumed_scale
        factor = factor.contiguous()
        for d in (d_hidden, d_weight):
            if d is not None and d.numel():
                ops.scale_rows_inplace(d, factor)  # a no-op launch when the upstream gradient is the assumed one
        return d_hidden, d_weight, None, None, None, None, None, None


def lm_head_token_local_step(hidden, weight, tokens, token_loss, temperature: float = 1.0, with_entropy: bool = False,
                             slab_tokens: int | None = None, assumed_grad_scale: float = 1.0):
    """``(loss, log_prob [N], entropy [N] | None)`` of a token-local loss over ``log_softmax(hidden @ weight.T / T)``
    with the gradients w.r.t. ``hidden`` and ``weight`` produced inside this call (``loss.backward()`` then only hands
    them on), never more than ``slab_tokens`` rows of logits in HBM and no second projection.

    ``token_loss(begin, end, log_prob, entropy) -> 0-d tensor`` gives the share of rows ``[begin, end)`` in the loss,
    built from differentiable ``[end - begin]``-sized vector operations on the two leaves it is handed; the shares add
    up to the loss, so every normaliser inside it must be known up front (a token count, a per-sample mask sum: what
    the reference's reducers divide by, relax/backends/megatron/cp_utils.py:125-162).  SFT's
    ``-sum_of_sample_mean(log_probs)`` (loss.py:1386-1428) and a clipped policy-gradient surrogate with given old
    log-probs and advantages are of this kind; GSPO's sequence-level ratio is not.
    """
    pad = (-hidden.size(-1)) % 128
    if pad:
        hidden = torch.nn.functional.pad(hidden, (0, pad))
        weight = torch.nn.functional.pad(weight, (0, pad))
    loss, lp, ent = _FusedLMHeadTokenLocalStep.apply(
        hidden, weight, tokens, 1.0 / float(temperature), bool(with_entropy), token_loss,
        int(slab_tokens or STEP_SLAB), float(assumed_grad_scale))
    return loss, lp, (ent if with_entropy else None)
