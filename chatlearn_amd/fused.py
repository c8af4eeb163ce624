"""The seam the reference lacks: logprob / entropy straight from the final hidden
states and lm_head.weight, without the [T, V] logits tensor.

``fused_linear_logprob_entropy`` stands where the reference runs
``self.model(...).logits`` followed by ``logprobs_from_logits`` and
``entropy_from_logits_with_chunking`` (policy_trainer.py:216-228); it is
autograd-aware, so ``total_loss.backward()`` (policy_trainer.py:286) reaches
``hidden`` and ``weight`` through the fused backward kernels.

``grpo_head_step`` does a whole micro-batch of the head in three launches
groups - fused forward, fused loss (+ upstream gradients), fused backward -
for callers that own the training loop.
"""
from typing import Optional

import torch

from . import ops
from ._lib import LOSS_GRPO, LOSS_GSPO


class _FusedHead(torch.autograd.Function):
    @staticmethod
    def forward(ctx, hidden, weight, labels, temperature, need_entropy, dweight_buffer):
        lp, ent, _, lse = ops.lmhead_forward(hidden, weight, labels, temperature, need_entropy)
        ctx.save_for_backward(hidden, weight, labels, lse, ent if ent is not None else lse)
        ctx.set_materialize_grads(False)
        ctx.temperature = temperature
        ctx.has_entropy = ent is not None
        ctx.dweight_buffer = dweight_buffer
        if ent is None:
            ent = torch.zeros(0, device=hidden.device)
            ctx.mark_non_differentiable(ent)
        return lp, ent

    @staticmethod
    def backward(ctx, g_lp, g_ent):
        hidden, weight, labels, lse, ent = ctx.saved_tensors
        need_h, need_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        if g_lp is None and g_ent is None:
            return None, None, None, None, None, None
        if g_lp is None:
            g_lp = torch.zeros_like(lse)
        use_ent = ctx.has_entropy and g_ent is not None
        dh, dw = ops.lmhead_backward(
            hidden, weight, labels, lse, ent if use_ent else None, g_lp.float().contiguous(),
            g_ent.float().contiguous() if use_ent else None, ctx.temperature,
            need_dhidden=need_h, need_dweight=need_w, dweight=ctx.dweight_buffer,
            accumulate_dweight=ctx.dweight_buffer is not None)
        if dw is not None:
            # A caller-supplied fp32 main-grad buffer was accumulated in place; autograd gets no copy.
            dw = None if ctx.dweight_buffer is not None else dw.to(weight.dtype)
        return dh, dw, None, None, None, None


def fused_linear_logprob_entropy(hidden: torch.Tensor, weight: torch.Tensor, labels: torch.Tensor, *,
                                 temperature: float = 1.0, need_entropy: bool = True,
                                 dweight_buffer: Optional[torch.Tensor] = None):
    """(logprob fp32 [T], entropy fp32 [T]) of ``labels`` under softmax(hidden @ weight.T / temperature).

    hidden [T,H] and weight [V,H] share a dtype (bf16 or fp32), labels int64 [T].
    ``dweight_buffer``: optional fp32 [V,H] tensor that receives ``+= dW`` in the
    backward (the fp32 gradient accumulation FSDP2 does with ``reduce_dtype=fp32``);
    without it ``weight.grad`` gets dW cast to the weight dtype, as torch would.
    Leading dimensions of hidden/labels are flattened and restored.
    """
    lead = labels.shape
    h2 = hidden.reshape(-1, hidden.shape[-1])
    lp, ent = _FusedHead.apply(h2, weight, labels.reshape(-1), float(temperature), bool(need_entropy), dweight_buffer)
    lp = lp.reshape(lead)
    ent = ent.reshape(lead) if need_entropy else None
    return lp, ent


def grpo_head_step(hidden, weight, labels, old_logprob, ref_logprob, advantages, cu_seqlens, loss_mask, *,
                   n_tokens_total: float, fsdp_size: int = 1, use_group_sequence_policy=False,
                   pos_clip_ratio=0.2, neg_clip_ratio=0.2, diff_clip_ratio=10, final_clip_ratio=3,
                   kl_coef=0.0, entropy_coef=0.0, temperature=1.0, dweight: Optional[torch.Tensor] = None,
                   accumulate_dweight=False, need_dhidden=True, check_flags=True):
    """Forward + loss + backward of the head for one packed micro-batch, no autograd graph.

    Mirrors policy_trainer.py:216-286 on packed rows: returns a dict with the
    per-token ``logprob``/``entropy``, the loss scalars ``pg_loss_mean``,
    ``kl_loss_mean``, ``entropy_loss_mean``, ``total_loss`` (device fp64 scalars),
    ``dhidden`` and ``dweight``.  ``advantages`` is a device tensor [B].
    """
    lp, ent, _, lse = ops.lmhead_forward(hidden, weight, labels, temperature, need_entropy=True)
    scale = float(fsdp_size) / float(n_tokens_total)
    res = ops.policy_loss(
        lp, old_logprob, advantages, mode=LOSS_GSPO if use_group_sequence_policy else LOSS_GRPO,
        cu_seqlens=cu_seqlens, ref_logprob=ref_logprob, entropy=ent, loss_mask=loss_mask,
        diff_clip_ratio=diff_clip_ratio, pos_clip_ratio=pos_clip_ratio, neg_clip_ratio=neg_clip_ratio,
        final_clip_ratio=final_clip_ratio, kl_coef=kl_coef if kl_coef > 0 else 0.0,
        entropy_coef=entropy_coef if entropy_coef > 0 else 0.0, grad_scale=scale, want_dloss=False,
        want_upstream=True)
    dh, dw = ops.lmhead_backward(hidden, weight, labels, lse, ent, res.g_logprob, res.g_entropy, temperature,
                                 need_dhidden=need_dhidden, need_dweight=True, dweight=dweight,
                                 accumulate_dweight=accumulate_dweight)
    if check_flags:
        res.raise_on_flags()
    pg = res.sums[0] * scale
    kl = res.sums[1] * scale
    en = res.sums[2] * scale
    total = pg
    if entropy_coef > 0:
        total = total - entropy_coef * en
    if kl_coef > 0:
        total = total + kl_coef * kl
    return {"logprob": lp, "entropy": ent, "lse": lse, "pg_loss_mean": pg, "kl_loss_mean": kl,
            "entropy_loss_mean": en, "total_loss": total, "num_masked": res.sums[3],
            "per_token_loss": res.loss, "per_token_kl": res.kl, "dhidden": dh, "dweight": dw,
            "g_logprob": res.g_logprob}
