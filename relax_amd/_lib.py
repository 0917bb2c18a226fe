"""ctypes binding of ``librelax_amd.so`` (the C ABI declared in ``include/relax_amd.h``).

There is no CPU or PyTorch fallback: if the library has not been built the import of this module raises, and every
op raises when handed a tensor that is not on a ROCm device.
"""

from __future__ import annotations

import ctypes as C
import os
import re

# PyTorch ships its own copy of the HIP runtime (same soname as the system one).  It must be loaded BEFORE
# librelax_amd.so so that both bind to one runtime instance: streams and device pointers are only meaningful inside
# the runtime that created them, and a second instance reports "no ROCm-capable device".
import torch  # noqa: F401

HERE = os.path.dirname(os.path.abspath(__file__))
# RELAX_AMD_LIBRARY points at a build of the library kept somewhere else (same ABI); default: next to this file.
LIB_PATH = os.environ.get("RELAX_AMD_LIBRARY") or os.path.join(HERE, "librelax_amd.so")
HEADER_PATH = os.path.join(os.path.dirname(HERE), "include", "relax_amd.h")

F32, BF16, F16, F64 = 0, 1, 2, 3
LOSS_KINDS = {"ppo": 0, "gspo": 1, "cispo": 2, "rloo": 3, "sapo": 4}
KL_KINDS = {None: 0, "k1": 1, "k2": 2, "k3": 3, "low_var_kl": 4}
GROUP_MODES = {"center": 0, "center_std": 1, "rloo": 2}
OPD_JSD, OPD_LOW_VAR = 0, 1
METRIC_SLOTS = [
    "loss", "pg_loss", "entropy_loss", "pg_clipfrac", "ppo_kl", "kl_loss", "train_rollout_logprob_abs_diff",
    "train_rollout_prob_abs_diff", "ois", "tis", "tis_clipfrac", "tis_abs", "mismatch_kl", "mismatch_k3_kl",
    "opsm_clipfrac", "mask_sum",
]
NUM_METRICS = len(METRIC_SLOTS)

_vp, _i64, _i32, _f32 = C.c_void_p, C.c_int64, C.c_int32, C.c_float


class PolicyLossArgs(C.Structure):
    """Mirror of ``relax_amd_policy_loss_args``."""

    _fields_ = [
        ("struct_size", C.c_uint32), ("reserved", C.c_uint32),
        ("log_prob", _vp), ("old_log_prob", _vp), ("ref_log_prob", _vp), ("train_log_prob", _vp),
        ("rollout_log_prob", _vp), ("advantages", _vp), ("loss_mask", _vp), ("pg_loss_mask", _vp), ("entropy", _vp),
        ("cu_resp", _vp), ("sample_denom", _vp), ("pg_sample_denom", _vp),
        ("n_samples", _i64), ("n_tokens", _i64),
        ("loss_kind", _i32), ("kl_kind", _i32), ("unbiased_kl", _i32), ("use_opsm", _i32), ("use_tis", _i32),
        ("mismatch_metrics", _i32), ("abs_diff_from_old", _i32),
        ("eps_clip", _f32), ("eps_clip_high", _f32), ("eps_clip_c", _f32), ("entropy_coef", _f32), ("kl_coef", _f32),
        ("tis_lo", _f32), ("tis_hi", _f32), ("opsm_delta", _f32), ("tau_pos", _f32), ("tau_neg", _f32),
        ("coef_log_prob", _vp), ("coef_entropy", _vp), ("pg_loss_tok", _vp), ("clipfrac_tok", _vp),
        ("ppo_kl_tok", _vp), ("kl_tok", _vp), ("sample_partials", _vp), ("metrics", _vp),
        ("extra_coef_log_prob", _vp),
        ("distill_teacher_log_prob", _vp), ("distill_kl_kind", _i32),
        ("distill_min_clamp", _f32), ("distill_token_clip", _f32), ("distill_is_clip", _f32),
        ("topk_ids", _vp), ("topk_teacher_log_prob", _vp), ("topk_width", _vp), ("topk_valid", _vp),
        ("topk_k", _i32), ("topk_kl_mode", _i32), ("topk_norm_mode", _i32), ("topk_has_clamp", _i32),
        ("topk_jsd_alpha", _f32), ("topk_min_clamp", _f32), ("topk_kl", _vp), ("topk_grad", _vp),
        ("read_masked_rows", _i32),
    ]


def new_policy_loss_args() -> PolicyLossArgs:
    """A zeroed argument block with ``struct_size`` filled in (the library refuses a block without it)."""
    a = PolicyLossArgs()
    a.struct_size = C.sizeof(PolicyLossArgs)
    return a


FUSED_TOPK_MAX = 256
KERNEL_CHOICES = {"auto": 0, "two_walk": 1, "resident": 2}


SIGNATURES = {
    "relax_amd_version": (C.c_int, []),
    "relax_amd_last_error": (C.c_char_p, []),
    "relax_amd_last_kernel": (C.c_char_p, []),
    "relax_amd_set_kernel_choice": (C.c_int, [C.c_int]),
    "relax_amd_set_exchange_wait": (C.c_int, [C.c_int, C.c_int]),
    "relax_amd_logprob_entropy_fwd": (C.c_int, [_vp, C.c_int, _i64, _i64, _i64, _vp, _vp, _f32, _vp, _vp, _vp, _vp, _vp]),
    "relax_amd_logprob_entropy_bwd": (
        C.c_int, [_vp, C.c_int, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _f32, _vp, _f32, _vp, _i64, _vp]),
    "relax_amd_build_row_maps": (C.c_int, [_vp, _vp, _i64, _i64, _i64, _vp, _vp, _vp, _vp]),
    "relax_amd_policy_loss": (C.c_int, [C.POINTER(PolicyLossArgs), _vp]),
    "relax_amd_segment_sum": (C.c_int, [_vp, _vp, _vp, _i64, _vp, _vp]),
    "relax_amd_group_rewards": (C.c_int, [_vp, C.c_int, _vp, _i64, _i32, _vp, _vp, _vp]),
    "relax_amd_broadcast_per_sample": (C.c_int, [_vp, _vp, _i64, _vp, _vp]),
    "relax_amd_whiten_partials": (_i64, [_i64]),
    "relax_amd_masked_whiten": (C.c_int, [_vp, _vp, _i64, _i32, _f32, _vp, _vp, _vp, _vp]),
    "relax_amd_reverse_kl_fwd": (C.c_int, [_vp, _vp, C.c_int, _i64, _i64, _i64, _vp, _vp, _vp, _vp]),
    "relax_amd_actor_step_fused": (
        C.c_int, [_vp, C.c_int, _i64, _i64, _i64, _vp, _vp, _vp, _f32, C.POINTER(PolicyLossArgs), _f32, _vp, _vp, _vp,
                  _vp, _vp, _i64, _vp]),
    "relax_amd_scale_rows_inplace": (C.c_int, [_vp, C.c_int, _i64, _i64, _i64, _vp, _vp]),
    "relax_amd_lmhead_workspace_bytes": (_i64, [_i64]),
    "relax_amd_lmhead_logprob_fwd": (
        C.c_int, [_vp, _vp, C.c_int, _i64, _i64, _i64, _i64, _i64, _vp, _f32, _vp, _vp, _vp, _vp, _vp, _vp]),
    "relax_amd_lmhead_logprob_fwd_static": (
        C.c_int, [_vp, _vp, C.c_int, _i64, _i64, _i64, _i64, _i64, _vp, _f32, _vp, _vp, _vp, _vp, _vp]),
    "relax_amd_lmhead_dlogits_t": (
        C.c_int, [_vp, _vp, C.c_int, _i64, _i64, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _f32, _vp, _i64, _vp]),
    "relax_amd_lmhead_dhidden": (C.c_int, [_vp, _i64, _i64, _vp, _i64, _i64, _i64, _i64, _vp, _i64, C.c_int, _vp]),
    "relax_amd_lmhead_dweight": (C.c_int, [_vp, _i64, _vp, _i64, _i64, _i64, _i64, _vp, _i64, C.c_int, _vp]),
    "relax_amd_lmhead_logprob_fwd_keep": (
        C.c_int, [_vp, _vp, C.c_int, _i64, _i64, _i64, _i64, _i64, _vp, _f32, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _vp]),
    "relax_amd_lmhead_dlogits_from_logits_t": (
        C.c_int, [_vp, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _f32, _vp]),
    "relax_amd_reverse_kl_bwd": (C.c_int, [_vp, _vp, C.c_int, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _f32, _vp, _vp, _vp]),
    "relax_amd_reinforce_pp_returns": (C.c_int, [_vp, _vp, _vp, C.c_int, _vp, _i64, C.c_double, C.c_double, _vp, _vp]),
    "relax_amd_gae": (C.c_int, [_vp, _vp, C.c_int, _vp, _i64, C.c_double, C.c_double, _vp, _vp, _vp]),
    "relax_amd_masked_normalize": (C.c_int, [_vp, _vp, C.c_int, _i64, C.c_double, _vp, _vp, _vp]),
    "relax_amd_gather_targets": (C.c_int, [_vp, _vp, _vp, _vp, _i64, _vp, _vp]),
    "relax_amd_logprob_entropy_masked_fwd": (
        C.c_int, [_vp, C.c_int, _i64, _i64, _i64, _vp, _vp, _vp, _i64, _f32, _vp, _vp, _vp, _vp, _vp, _vp]),
    "relax_amd_logprob_entropy_masked_bwd": (
        C.c_int, [_vp, C.c_int, _i64, _i64, _i64, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _f32, _f32, _vp,
                  _i64, _vp]),
    "relax_amd_sparse_row_add": (
        C.c_int, [_vp, C.c_int, _i64, _i64, _i64, _vp, _vp, _vp, _i64, _vp, _vp, _f32, _vp]),
    "relax_amd_topk_rows": (C.c_int, [_vp, C.c_int, _i64, _i64, _i64, _vp, C.c_int, _vp, _vp, _vp, _vp]),
    "relax_amd_logprob_entropy_topk_fwd": (
        C.c_int, [_vp, C.c_int, _i64, _i64, _i64, _vp, _vp, _f32, C.c_int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "relax_amd_topk_logprob_fwd": (
        C.c_int, [_vp, C.c_int, _i64, _i64, _i64, _vp, _vp, _i64, _f32, _vp, _vp, _vp, _vp]),
    "relax_amd_topk_logprob_bwd": (
        C.c_int, [_vp, C.c_int, _i64, _i64, _i64, _vp, _vp, _i64, _f32, _vp, _vp, _vp, _i64, _vp]),
    "relax_amd_opd_kl_topk_fwd": (
        C.c_int, [_vp, _vp, _vp, _i64, _i64, C.c_int, C.c_int, _f32, C.c_int, _f32, _vp, _vp]),
    "relax_amd_opd_kl_topk_bwd": (
        C.c_int, [_vp, _vp, _vp, _i64, _i64, C.c_int, C.c_int, _f32, C.c_int, _f32, _vp, _vp, _vp]),
    "relax_amd_reverse_kl_step_fused": (
        C.c_int, [_vp, _vp, C.c_int, _i64, _i64, _i64, _vp, _f32, _vp, _vp, _vp, _vp, _vp]),
}


def declared_symbols(header_path: str = HEADER_PATH) -> list[str]:
    """Names of every function the public header declares."""
    text = open(header_path).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(relax_amd_[a-z0-9_]+)\s*\(", text)))


def _load() -> C.CDLL:
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build the HIP extension first (python relax_amd/build.py). "
            "relax_amd has no CPU or PyTorch fallback."
        )
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


class KernelError(RuntimeError):
    pass


def check(rc: int) -> None:
    if rc != 0:
        msg = lib.relax_amd_last_error().decode("utf-8", "replace")
        if rc == -1:
            raise ValueError(msg)
        raise KernelError(f"relax_amd error {rc}: {msg}")
