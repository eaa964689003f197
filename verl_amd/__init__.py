"""MI355X-native per-token scoring and SPEC-RL draft verification for verl.

Hand-written HIP kernels (gfx950) behind a C ABI (include/vrl.h), wrapped with
the names and argument conventions of verl.utils.torch_functional. Importing
this package never compiles or loads anything; the first call loads
``verl_amd/libvrl_hip.so`` (built by ``python -m verl_amd.build``) and raises if
it is not there.

Setting ``VERL_USE_EXTERNAL_MODULES=verl_amd.plugin`` makes verl import
``verl_amd.plugin`` at start-up (verl/__init__.py:49-52), which calls
``install()``.
"""

from . import rollout_corr
from .fused_linear import FusedLinearForPPO, fused_linear_for_ppo, linear_cross_entropy, lm_head_score_mfma
from .hook import install, uninstall
from .layout import expand_per_sequence, response_from_packed, response_slice, roll_labels, transpose_2d
from .spec_rl import (
    VerifyResult,
    draw_log_uniforms,
    fused_score_verify,
    spec_verify,
    thresh_offset_from_lenience,
    truncate_draft,
)
from .torch_functional import (
    calculate_sum_pi_squared_from_logits,
    entropy_from_logits,
    entropy_from_logits_with_chunking,
    fused_logprob_entropy,
    logprobs_from_logits,
    logprobs_from_logits_naive,
    logprobs_from_logits_v2,
    score_responses,
)
from .errors import check_errors

__version__ = "0.1.0"

__all__ = [
    "install",
    "uninstall",
    "FusedLinearForPPO",
    "fused_linear_for_ppo",
    "linear_cross_entropy",
    "lm_head_score_mfma",
    "VerifyResult",
    "draw_log_uniforms",
    "fused_score_verify",
    "spec_verify",
    "thresh_offset_from_lenience",
    "truncate_draft",
    "expand_per_sequence",
    "response_from_packed",
    "response_slice",
    "roll_labels",
    "transpose_2d",
    "calculate_sum_pi_squared_from_logits",
    "entropy_from_logits",
    "entropy_from_logits_with_chunking",
    "fused_logprob_entropy",
    "logprobs_from_logits",
    "logprobs_from_logits_naive",
    "logprobs_from_logits_v2",
    "score_responses",
    "check_errors",
]
