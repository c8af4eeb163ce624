"""MI355X-native GRPO/GSPO policy-loss path: fused lm_head + log-softmax
statistics, clipped-ratio losses, group advantages and packing helpers, as hand
written HIP kernels (gfx950) behind a C ABI, with Python mirrors of the
reference's ``chatlearn.algorithm.grpo_utils`` functions."""
from .fused import fused_linear_logprob_entropy, grpo_head_step  # noqa: F401

__all__ = ["fused_linear_logprob_entropy", "grpo_head_step"]
