"""Mirror of the loss side of chatlearn/algorithm/grpo_utils/megatron_utils/train_helper.py
for one tensor-parallel and one context-parallel rank: the per-token logprob that
Megatron's vocab-parallel cross entropy yields, the vocab-parallel entropy, the
re-padding of packed outputs, ``_compute_all_losses`` and ``loss_func``.

Of the reference's ``get_batch`` only the packed (THD) branch is mirrored, as
``get_batch_packed``: one device pass replaces its per-sample Python loops.  The dense
branch ([1, 1, S, S] attention masks, position-id resets) and ``forward_step`` are
Megatron plumbing and stay with the caller; the loss functions here start where the
model has produced ``all_token_logits`` in Megatron's ``[s, b, V]`` (or
``[total_nnz, 1, V]``) layout.
"""
from dataclasses import dataclass
from typing import Any, Dict, Optional

import torch

from .... import ops
from ....bert_padding import pad_input
from ..loss_gallery import calculate_gspo_loss, calculate_grpo_loss
from ..trainer_utils import _StatsFromLogits


@dataclass
class PackedSeqParams:
    """Field-for-field stand-in for ``megatron.core.packed_seq_params.PackedSeqParams`` as the
    reference fills it (train_helper.py:304-310)."""
    qkv_format: str = 'thd'
    cu_seqlens_q: Optional[torch.Tensor] = None
    cu_seqlens_kv: Optional[torch.Tensor] = None
    max_seqlen_q: Optional[int] = None
    max_seqlen_kv: Optional[int] = None


def get_batch_packed(data_b: Dict[str, Any], is_training: bool, *, eod: int, tp_size: int = 1, cp_size: int = 1,
                     cp_rank: int = 0, device=None) -> Dict[str, Any]:
    """The packed branch of the reference's ``get_batch`` (train_helper.py:258-328, 400-420) for one
    raw batch ``data_b`` (``all_tokens`` [mbs, seq_length], ``prompt_token_length``,
    ``response_token_length``; for training also ``ref_logprobs``, ``old_logprobs``, ``advantages``
    and optionally ``loss_mask``).  Same keys and shapes as the reference returns; the sequence
    padding to ``tp*cp*2``, the unpadding, the label roll, the rolled packed loss mask and this
    context-parallel rank's share come from one device pass instead of O(mbs) Python loops."""
    tokens = data_b["all_tokens"].long()
    device = device or (tokens.device if tokens.is_cuda else torch.device("cuda", torch.cuda.current_device()))
    tokens = tokens.to(device)
    mbs, seqlen = tokens.shape
    packed = ops.thd_pack(tokens, data_b["prompt_token_length"], data_b["response_token_length"],
                          align=tp_size * cp_size * 2, pad_token=eod, cp_size=cp_size, cp_rank=cp_rank)
    max_padded = packed["max_seqlen_padded"]
    params = PackedSeqParams(qkv_format='thd', cu_seqlens_q=packed["cu_seqlens_padded"],
                             cu_seqlens_kv=packed["cu_seqlens_padded"], max_seqlen_q=max_padded,
                             max_seqlen_kv=max_padded)
    input_data = {
        "all_tokens": packed["tokens"].unsqueeze(0),
        "all_token_attention_mask": None,
        "all_token_loss_mask": None,
        "all_token_position_ids": None,
        "labels": packed["labels"].unsqueeze(0),
        'packed_seq_params': params,
        "ori_seq_len": max_padded,
        "ori_batch_size": mbs,
        "seq_indices": packed["seq_indices"].unsqueeze(0),
        "indices": packed["indices"],
        "num_tokens_on_this_cp_rank": packed["num_loss_tokens"],
        'pad_size': max_padded - seqlen,
    }
    if is_training:
        if "loss_mask" in data_b:
            loss_mask = data_b['loss_mask'].to(device).to(torch.int32).contiguous()
        else:
            as_i32 = lambda x: torch.as_tensor(x, dtype=torch.int32).to(device)
            _, loss_mask, _ = ops.build_masks(as_i32(data_b["prompt_token_length"]),
                                              as_i32(data_b["response_token_length"]), seqlen,
                                              want_position_ids=False)
        _, loss_mask = ops.shift_labels(None, loss_mask, zero_last=False)      # roll by -1 along the row
        input_data.update({
            "all_token_loss_mask": loss_mask,
            "advantages": data_b["advantages"],
            "ref_logprobs": data_b["ref_logprobs"].float().to(device),
            "old_logprobs": data_b["old_logprobs"].float().to(device),
        })
    return input_data


def language_model_logprob(labels: torch.Tensor, logits: torch.Tensor) -> torch.Tensor:
    """-1 * Megatron's ``compute_language_model_loss(labels, logits)`` at tp = 1: labels [b, s],
    logits [s, b, V]  ->  fp32 logprob [b, s] (reference train_helper.py:480-482)."""
    s, b, V = logits.shape
    lp, _ = _StatsFromLogits.apply(logits.reshape(s * b, V), labels.transpose(0, 1).reshape(-1), True, False)
    return lp.reshape(s, b).transpose(0, 1).contiguous()


def entropy_from_tensor_parallel_logits(logits: torch.Tensor) -> torch.Tensor:
    """fp32 entropy over the last dim; like the reference's autograd function it defines no backward
    (reference train_helper.py:605-635), so the result is detached."""
    _, ent = _StatsFromLogits.apply(logits.detach().reshape(-1, logits.shape[-1]), None, False, True)
    return ent.reshape(logits.shape[:-1])


def reduce_from_context_parallel_region(logprobs: torch.Tensor, is_packing: bool = False,
                                        inputs: Dict[str, Any] = None):
    """One context-parallel rank: re-pad packed rows to [B, S] and drop the padding columns
    (reference train_helper.py:213-230)."""
    if is_packing:
        logprobs = pad_input(logprobs.permute(1, 0), inputs['indices'], inputs['ori_batch_size'],
                             inputs['ori_seq_len']).squeeze(-1)
    return logprobs[:, :logprobs.shape[1] - inputs['pad_size']]


def _compute_all_losses(module_args, model, all_token_logits: torch.Tensor, labels: torch.Tensor,
                        training_inputs: Dict[str, Any]) -> Dict[str, torch.Tensor]:
    """All per-token loss tensors of one micro-batch (reference train_helper.py:465-547).
    ``model`` is unused (the reference only reaches through it for the cross entropy)."""
    del model
    forward_logprob = language_model_logprob(labels, all_token_logits)
    forward_logprob = reduce_from_context_parallel_region(forward_logprob, module_args.packing, training_inputs)
    old_logprobs = training_inputs["old_logprobs"]
    ref_logprobs = training_inputs["ref_logprobs"]
    advantages = training_inputs["advantages"]
    mask = training_inputs['all_token_loss_mask']
    if module_args.use_group_sequence_policy:
        pg_loss, is_positive_clipped, is_negative_clipped, is_clipped = calculate_gspo_loss(
            log_probs=forward_logprob, old_log_probs=old_logprobs, advantages=advantages,
            diff_clip_ratio=module_args.diff_clip_ratio, pos_clip_ratio=module_args.pos_clip_ratio,
            neg_clip_ratio=module_args.neg_clip_ratio, final_clip_ratio=module_args.final_clip_ratio,
            loss_mask=mask)
    else:
        pg_loss = calculate_grpo_loss(
            log_probs=forward_logprob, old_log_probs=old_logprobs, advantages=advantages,
            diff_clip_ratio=module_args.diff_clip_ratio, pos_clip_ratio=module_args.pos_clip_ratio,
            neg_clip_ratio=module_args.neg_clip_ratio, final_clip_ratio=module_args.final_clip_ratio)
    entropy_loss = entropy_from_tensor_parallel_logits(all_token_logits).permute(1, 0)
    entropy_loss = reduce_from_context_parallel_region(entropy_loss, module_args.packing, training_inputs)
    # k3 estimator with exp(k) forced to 1 outside the mask, and the reference's two assertions
    res = ops.policy_loss(forward_logprob.detach().float(), old_logprobs.float(),
                          torch.zeros(forward_logprob.shape[0], device=forward_logprob.device),
                          ref_logprob=ref_logprobs.float(), loss_mask=mask, want_dloss=False, want_kl=True)
    fl = int(res.flags.item())
    assert not fl & 2, "kl loss ratio has inf values"
    assert not fl & 4, "kl loss ratio has nan values"
    kl_loss = res.kl
    out = {'pg_loss': pg_loss, 'entropy_loss': entropy_loss, 'kl_loss': kl_loss}
    if module_args.use_group_sequence_policy:
        out.update({
            'is_positive_clipped': is_positive_clipped, 'is_negative_clipped': is_negative_clipped,
            'is_clipped': is_clipped, 'is_positive_clipped_sample_average': is_positive_clipped,
            'is_negative_clipped_sample_average': is_negative_clipped, 'is_clipped_sample_average': is_clipped})
    return out


def loss_func(inputs: Dict, losses: Dict[str, torch.Tensor]):
    """Masked reductions of the loss dict: (loss to back-propagate, number of unmasked tokens, report)
    (reference train_helper.py:426-463).  Only ``pg_loss`` keeps its gradient."""
    require_bp_keys = ['pg_loss']
    loss_mask = inputs["all_token_loss_mask"].float()
    total_loss_for_bp = 0
    reporting_losses = {}
    for key, loss in losses.items():
        if key not in require_bp_keys:
            loss = loss.detach()
        if key.endswith('_sample_average'):
            final_loss = (loss.float() * loss_mask).sum() / (1e-5 + loss_mask.sum())
        else:
            final_loss = (loss.float() * loss_mask).sum()
        if key in require_bp_keys:
            total_loss_for_bp = total_loss_for_bp + final_loss
        reporting_losses[key] = final_loss.detach().clone().to(torch.float)
    num_tokens = inputs.get('num_tokens_on_this_cp_rank', loss_mask.sum().clone().detach()).to(torch.int)
    reporting_losses["num_tokens"] = num_tokens
    reporting_losses["num_samples"] = torch.ones_like(num_tokens)
    return total_loss_for_bp, num_tokens, reporting_losses
