"""Mirror of chatlearn/algorithm/grpo_utils/loss_gallery.py: same two functions,
same signatures, results from the fused HIP loss kernel.

Both functions are differentiable with respect to ``log_probs`` with torch's
sub-gradient conventions (ties of max/min split in halves, clamp passes the
gradient on the closed interval), because the kernel emits d loss / d log_prob
alongside the loss.
"""
from typing import List

import torch

from ... import ops
from ..._lib import LOSS_GRPO, LOSS_GSPO


class _PolicyLoss(torch.autograd.Function):
    @staticmethod
    def forward(ctx, log_probs, old_log_probs, adv, mode, loss_mask, diff_clip, pos_clip, neg_clip, final_clip):
        res = ops.policy_loss(log_probs.detach().float(), old_log_probs.detach().float(), adv, mode=mode,
                              loss_mask=loss_mask, diff_clip_ratio=diff_clip, pos_clip_ratio=pos_clip,
                              neg_clip_ratio=neg_clip, final_clip_ratio=final_clip, want_dloss=True,
                              want_flags3=(mode == LOSS_GSPO))
        # reference: assert not torch.isnan(loss).any(), "pg loss is nan"
        assert not int(res.flags.item()) & 1, "pg loss is nan"
        ctx.save_for_backward(res.dloss)
        ctx.in_dtype = log_probs.dtype
        out_dtype = torch.promote_types(torch.promote_types(log_probs.dtype, old_log_probs.dtype), adv.dtype)
        loss = res.loss.to(out_dtype)
        if mode == LOSS_GSPO:
            ctx.mark_non_differentiable(res.is_positive_clipped, res.is_negative_clipped, res.is_clipped)
            return loss, res.is_positive_clipped, res.is_negative_clipped, res.is_clipped
        return loss

    @staticmethod
    def backward(ctx, g, *_):
        (dloss,) = ctx.saved_tensors
        return (g.to(dloss.dtype) * dloss).to(ctx.in_dtype), None, None, None, None, None, None, None, None


def _adv_tensor(advantages, like):
    # torch.tensor(list) exactly as the reference does (loss_gallery.py:19,53): a list of numpy
    # float64 gives a float64 tensor, a list of Python floats a float32 one.
    return torch.tensor(advantages).to(like.device)


def calculate_grpo_loss(
    log_probs: torch.Tensor,
    old_log_probs: torch.Tensor,
    advantages: List[float],
    diff_clip_ratio: float = 10,
    pos_clip_ratio: float = 0.2,
    neg_clip_ratio: float = 0.2,
    final_clip_ratio: float = 3.0,
):
    """Token-level GRPO surrogate on padded [B, S] tensors (reference loss_gallery.py:6-33)."""
    adv = _adv_tensor(advantages, log_probs)
    loss = _PolicyLoss.apply(log_probs, old_log_probs, adv, LOSS_GRPO, None, diff_clip_ratio, pos_clip_ratio,
                             neg_clip_ratio, final_clip_ratio)
    return loss.contiguous()


def calculate_gspo_loss(
    log_probs: torch.Tensor,
    old_log_probs: torch.Tensor,
    advantages: List[float],
    diff_clip_ratio: float = 10,
    pos_clip_ratio: float = 1e-3,
    neg_clip_ratio: float = 1e-3,
    final_clip_ratio: float = 0.01,
    loss_mask: torch.Tensor = None
):
    """Sequence-level GSPO surrogate and its three clip masks (reference loss_gallery.py:35-74)."""
    adv = _adv_tensor(advantages, log_probs)
    loss, is_pos, is_neg, is_clip = _PolicyLoss.apply(
        log_probs, old_log_probs, adv, LOSS_GSPO, loss_mask, diff_clip_ratio, pos_clip_ratio, neg_clip_ratio,
        final_clip_ratio)
    return (loss.contiguous(), is_pos, is_neg, is_clip)
