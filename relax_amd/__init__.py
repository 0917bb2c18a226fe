"""relax_amd: MI355X (gfx950) kernels behind Relax's log-prob / entropy / policy-loss / advantage functions.

Importing the package loads ``librelax_amd.so`` (built in-tree by ``python relax_amd/build.py``); it raises if the
library is missing -- there is no CPU or PyTorch fallback.
"""

from . import _lib  # noqa: F401  (fails loudly when the HIP extension has not been built)
from .loss import (  # noqa: F401
    compute_advantages_and_returns,
    get_log_probs_and_entropy,
    get_responses,
    get_values,
    loss_function,
    policy_loss_function,
    sft_loss_function,
    sft_loss_function_chunked,
    value_loss_function,
)
from .ppo_utils import calculate_log_probs_and_entropy  # noqa: F401

__version__ = "0.1.0"
