"""CPU checks of the C-ABI boundary: the shared library loads, exports every symbol the public header declares,
the ctypes struct mirrors the C layout, and argument validation / error plumbing work without a GPU."""

import ctypes as C
import os
import subprocess

import pytest
import torch

from relax_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    names = _lib.declared_symbols()
    assert len(names) >= 13 and "relax_amd_logprob_entropy_fwd" in names
    for n in names:
        assert hasattr(_lib.lib, n), f"{n} declared in include/relax_amd.h but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature"
    assert _lib.lib.relax_amd_version() == 2
    header = open(_lib.HEADER_PATH).read()
    assert "#define RELAX_AMD_ABI_VERSION 2" in header


def test_struct_layout_matches_c_header(tmp_path):
    src = tmp_path / "layout.c"
    src.write_text(
        '#include <stdio.h>\n#include <stddef.h>\n#include "relax_amd.h"\n'
        "int main(void){printf(\"%zu %zu %zu %zu %d %zu %zu %zu\\n\", sizeof(relax_amd_policy_loss_args),"
        " offsetof(relax_amd_policy_loss_args, n_samples), offsetof(relax_amd_policy_loss_args, eps_clip),"
        " offsetof(relax_amd_policy_loss_args, metrics), RELAX_AMD_NUM_METRICS,"
        " offsetof(relax_amd_policy_loss_args, extra_coef_log_prob),"
        " offsetof(relax_amd_policy_loss_args, distill_kl_kind),"
        " offsetof(relax_amd_policy_loss_args, distill_is_clip));"
        "printf(\"%zu %zu %zu %zu %d\\n\", offsetof(relax_amd_policy_loss_args, topk_ids),"
        " offsetof(relax_amd_policy_loss_args, topk_k), offsetof(relax_amd_policy_loss_args, topk_min_clamp),"
        " offsetof(relax_amd_policy_loss_args, topk_grad), RELAX_AMD_FUSED_TOPK_MAX);"
        "printf(\"%zu\\n\", offsetof(relax_amd_policy_loss_args, read_masked_rows));return 0;}\n"
    )
    exe = tmp_path / "layout"
    subprocess.check_call(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)])
    (size, off_n, off_eps, off_metrics, nmet, off_extra, off_kind, off_is, off_tk_ids, off_tk_k, off_tk_clamp,
     off_tk_grad, tk_max, off_masked) = map(int, subprocess.check_output([str(exe)]).split())
    S = _lib.PolicyLossArgs
    assert C.sizeof(S) == size
    assert S.n_samples.offset == off_n and S.eps_clip.offset == off_eps and S.metrics.offset == off_metrics
    assert S.extra_coef_log_prob.offset == off_extra and S.distill_kl_kind.offset == off_kind
    assert S.distill_is_clip.offset == off_is
    assert S.topk_ids.offset == off_tk_ids and S.topk_k.offset == off_tk_k
    assert S.topk_min_clamp.offset == off_tk_clamp and S.topk_grad.offset == off_tk_grad
    assert tk_max == _lib.FUSED_TOPK_MAX and S.read_masked_rows.offset == off_masked
    assert nmet == _lib.NUM_METRICS


def test_argument_validation_reports_errors_without_touching_the_gpu():
    L = _lib.lib
    rc = L.relax_amd_logprob_entropy_fwd(None, 0, 4, 0, 0, None, None, 1.0, None, None, None, None, None)
    assert rc == -1 and b"bad shape" in L.relax_amd_last_error()
    rc = L.relax_amd_logprob_entropy_fwd(None, 0, 4, 8, 8, None, None, 1.0, None, None, None, None, None)
    assert rc == -1 and b"NULL" in L.relax_amd_last_error()
    rc = L.relax_amd_logprob_entropy_fwd(C.c_void_p(16), 9, 4, 8, 8, None, C.c_void_p(16), 1.0, C.c_void_p(16), None, None, None, None)
    assert rc == -1 and b"dtype" in L.relax_amd_last_error()
    assert L.relax_amd_logprob_entropy_fwd(None, 0, 0, 8, 8, None, None, 1.0, None, None, None, None, None) == 0
    # the distillation fields of the policy-loss block are checked before anything is launched
    # a block that does not state its size (a client built against a shorter layout) is refused before any field
    # behind the old end is read
    short = _lib.PolicyLossArgs()
    short.metrics = short.sample_partials = short.cu_resp = 16
    assert L.relax_amd_policy_loss(C.byref(short), None) == -1 and b"struct_size" in L.relax_amd_last_error()
    short.struct_size = C.sizeof(_lib.PolicyLossArgs) - 8
    assert L.relax_amd_policy_loss(C.byref(short), None) == -1 and b"struct_size" in L.relax_amd_last_error()
    short.advantages = short.loss_mask = short.coef_log_prob = 16
    rc = L.relax_amd_actor_step_fused(C.c_void_p(16), 2, 4, 64, 64, None, None, C.c_void_p(16), 1.0, C.byref(short),
                                      1.0, C.c_void_p(16), C.c_void_p(16), C.c_void_p(16), C.c_void_p(16),
                                      C.c_void_p(16), 64, None)
    assert rc == -1 and b"struct_size" in L.relax_amd_last_error()
    # the process-wide kernel choice: returns the previous value, refuses unknown ones
    assert L.relax_amd_set_kernel_choice(1) == 0 and L.relax_amd_set_kernel_choice(2) == 1
    assert L.relax_amd_set_kernel_choice(7) == -1 and b"unknown choice" in L.relax_amd_last_error()
    assert L.relax_amd_set_kernel_choice(0) == 2
    a = _lib.new_policy_loss_args()
    a.metrics = a.sample_partials = a.cu_resp = 16
    a.distill_teacher_log_prob = 16
    assert L.relax_amd_policy_loss(C.byref(a), None) == -1 and b"extra_coef_log_prob" in L.relax_amd_last_error()
    a.extra_coef_log_prob, a.distill_kl_kind = 16, _lib.KL_KINDS["k2"]
    assert L.relax_amd_policy_loss(C.byref(a), None) == -1 and b"distill_kl_kind" in L.relax_amd_last_error()
    # ... and so is the top-K distillation block of the fused step
    f = _lib.new_policy_loss_args()
    f.advantages = f.loss_mask = f.coef_log_prob = f.topk_ids = 16
    p16 = C.c_void_p(16)

    def fused():
        return L.relax_amd_actor_step_fused(p16, 2, 4, 64, 64, None, None, p16, 1.0, C.byref(f), 1.0, p16, p16, p16,
                                            p16, p16, 64, None)

    assert fused() == -1 and b"extra_coef_log_prob" in L.relax_amd_last_error()
    f.extra_coef_log_prob = 16
    assert fused() == -1 and b"topk_teacher_log_prob" in L.relax_amd_last_error()
    f.topk_teacher_log_prob = f.topk_kl = f.topk_grad = 16
    f.topk_k = _lib.FUSED_TOPK_MAX + 1
    assert fused() == -1 and b"topk_k" in L.relax_amd_last_error()
    f.topk_k, f.topk_norm_mode = 8, 7
    assert fused() == -1 and b"topk_norm_mode" in L.relax_amd_last_error()
    rc = L.relax_amd_group_rewards(None, 0, None, 4, 7, None, None, None)
    assert rc == -1 and b"mode" in L.relax_amd_last_error()
    rc = L.relax_amd_masked_whiten(None, None, 0, 1, 1e-8, None, None, None, None)
    assert rc == -1
    with pytest.raises(ValueError):
        _lib.check(rc)
    assert L.relax_amd_whiten_partials(1) == 1 and L.relax_amd_whiten_partials(4097) == 2


def test_product_refuses_cpu_tensors():
    import relax_amd
    from relax_amd import ppo_utils

    with pytest.raises(RuntimeError, match="no CPU fallback"):
        relax_amd.calculate_log_probs_and_entropy(torch.randn(2, 4), torch.tensor([1, 2]), None)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ppo_utils.compute_policy_loss(torch.zeros(3), torch.ones(3), 0.2, 0.2)
    # shape-only paths need no device
    lp, ent = relax_amd.calculate_log_probs_and_entropy(torch.zeros(0, 4), torch.zeros(0, dtype=torch.long), None, True)
    assert lp.shape == (0,) and ent.shape == (0,)
    with pytest.raises(ValueError, match="Unknown kl_loss_type: unsupported"):
        ppo_utils.compute_approx_kl(torch.zeros(2), torch.zeros(2), "unsupported")


def test_host_index_arithmetic_matches_oracle_bruteforce():
    from oracle.policy import response_row_ranges
    from relax_amd.loss import response_row_begins

    tot, resp = [5, 3, 7, 4, 2], [2, 3, 1, 3, 0]
    begins, sft = response_row_begins(tot, resp)
    ranges = response_row_ranges(tot, resp)
    assert begins == [b for b, _, _ in ranges] and sft == [s for _, _, s in ranges]


def test_product_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "relax_amd")
    for fn in os.listdir(pkg):
        if fn.endswith(".py"):
            text = open(os.path.join(pkg, fn)).read()
            assert "import oracle" not in text and "from oracle" not in text, fn
