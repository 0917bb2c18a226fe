"""The allocation-free LM-head forward (``relax_amd_lmhead_logprob_fwd_static``: workspace in a fixed array inside
the library) against ``relax_amd_lmhead_logprob_fwd`` with a caller workspace, through the C ABI.  Same kernels, so
the four outputs must be bit-identical; two calls in a row share the array, the second on a smaller input."""

import pytest
import torch

from tests.gpu_util import announce, require_gpu

pytestmark = pytest.mark.gpu

BF16 = 1  # RELAX_AMD_BF16


def _inputs(n, h, v, seed, dev):
    g = torch.Generator().manual_seed(seed)
    hidden = torch.randn(n, h, generator=g).bfloat16().to(dev)
    weight = (torch.randn(v, h, generator=g) * 0.05).bfloat16().to(dev)
    targets = torch.randint(0, v, (n,), generator=g).to(dev)
    return hidden, weight, targets


def _call(lib, static, hidden, weight, targets, inv_t):
    from relax_amd._lib import check

    n, h = hidden.shape
    v = weight.shape[0]
    dev = hidden.device
    # poisoned outputs: every element must be written by the call
    outs = [torch.full((n,), float("nan"), device=dev) for _ in range(4)]
    stream = torch.cuda.current_stream().cuda_stream
    common = (hidden.data_ptr(), weight.data_ptr(), BF16, n, h, v, hidden.stride(0), weight.stride(0),
              targets.data_ptr(), inv_t)
    if static:
        check(lib.relax_amd_lmhead_logprob_fwd_static(*common, *[o.data_ptr() for o in outs], stream))
    else:
        ws = torch.empty(max(1, lib.relax_amd_lmhead_workspace_bytes(n)), dtype=torch.uint8, device=dev)
        check(lib.relax_amd_lmhead_logprob_fwd(*common, ws.data_ptr(), *[o.data_ptr() for o in outs], stream))
    torch.cuda.synchronize()
    return outs


def test_static_scratch_forward_matches_workspace_forward_on_two_calls_in_a_row():
    from relax_amd._lib import check, lib

    dev = require_gpu()
    names = ("log_prob", "entropy", "lse", "spx")
    # first a larger input (several row blocks, vocabulary splits), then a smaller one that reuses the same array,
    # then an odd-sized one with a temperature
    for i, (n, h, v, seed, inv_t) in enumerate(((1500, 256, 5000, 1, 1.0), (300, 256, 5000, 2, 1.0),
                                                (777, 128, 1111, 3, 1.0 / 0.7))):
        announce("lmhead static scratch", n, h, v)
        hidden, weight, targets = _inputs(n, h, v, seed, dev)
        want = _call(lib, False, hidden, weight, targets, inv_t)
        got = _call(lib, True, hidden, weight, targets, inv_t)
        if i > 0:
            # what the entry point exists for: once the first call has resolved the array's address, a call takes no
            # device memory and gives none back -- neither through the runtime nor through torch's allocator
            outs = [torch.empty(n, device=dev) for _ in range(4)]
            stream = torch.cuda.current_stream().cuda_stream
            torch.cuda.synchronize()
            free_before, held_before = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated()
            reserved_before = torch.cuda.memory_reserved()
            for _ in range(3):
                check(lib.relax_amd_lmhead_logprob_fwd_static(
                    hidden.data_ptr(), weight.data_ptr(), BF16, n, h, v, hidden.stride(0), weight.stride(0),
                    targets.data_ptr(), inv_t, *[o.data_ptr() for o in outs], stream))
            torch.cuda.synchronize()
            assert torch.cuda.mem_get_info()[0] == free_before
            assert torch.cuda.memory_allocated() == held_before and torch.cuda.memory_reserved() == reserved_before
            assert torch.equal(outs[0], got[0])
        for name, a, b in zip(names, got, want):
            assert torch.isfinite(a).all(), name
            assert torch.equal(a, b), (name, n, (a - b).abs().max().item())
        # against plain torch on the same operands (the existing entry point's own parity bar: 2e-3)
        logits = (hidden.float() @ weight.float().t()) * inv_t
        lp = torch.log_softmax(logits, -1)
        ref_lp = lp.gather(1, targets[:, None]).squeeze(1)
        ref_ent = -(lp.exp() * lp).sum(-1)
        assert (got[0] - ref_lp).abs().max().item() < 2e-3
        assert (got[1] - ref_ent).abs().max().item() < 2e-3


def test_static_scratch_forward_rejects_sizes_beyond_its_array():
    from relax_amd._lib import KernelError, check, lib

    dev = require_gpu()
    announce("lmhead static scratch size limit")
    n = 32768 + 1
    hidden, weight, targets = _inputs(8, 128, 512, 4, dev)
    out = torch.zeros(8, device=dev)
    with pytest.raises(KernelError, match="32768"):
        check(lib.relax_amd_lmhead_logprob_fwd_static(
            hidden.data_ptr(), weight.data_ptr(), BF16, n, 128, 512, 128, 128, targets.data_ptr(), 1.0,
            out.data_ptr(), out.data_ptr(), out.data_ptr(), out.data_ptr(), None))
    # a zero-token call is a no-op
    check(lib.relax_amd_lmhead_logprob_fwd_static(None, None, BF16, 0, 128, 512, 128, 128, None, 1.0, None, None,
                                                  None, None, None))
