"""Mirror of the loss side of chatlearn/algorithm/grpo_utils/megatron_utils/train_helper.py
for one tensor-parallel and one context-parallel rank: the per-token logprob that
Megatron's vocab-parallel cross entropy yields, the vocab-parallel entropy, the
re-padding of packed outputs, ``_compute_all_losses`` and ``loss_func``.

Of the reference's ``get_batch`` only the packed (THD) branch is mirrored, as
``get_batch_packed``: one device pass replaces its per-sample Python loops.  The dense
branch ([1, 1, S, S] attention masks, position-id resets) and ``forward_step`` are
Megatron plumbing and stay with the caller; the loss functions here start where the
model has produced ``all_token_logits`` in Megatron's ``[s, b, V]`` (or
``[total_nnz, 1, V]``) layout - or, through ``compute_all_losses_from_hidden`` /
``logprobs_from_hidden``, one step earlier: at the decoder's final hidden states, before the
output layer, so that the logits are never written out.
"""
from dataclasses import dataclass
from typing import Any, Dict, Optional

import torch

from .... import ops
from ....bert_padding import index_first_axis, pad_input
from ....fused import AUTO, fused_linear_logprob_entropy
from ...._lib import LOSS_GRPO, LOSS_GSPO
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
            # the same rolled mask per packed token, built on the host from the host-side inputs: lets the
            # fused head find the rows that carry a gradient without reading anything back
            "packed_loss_mask_host": _packed_loss_mask_host(data_b, seqlen, tp_size * cp_size * 2) if cp_size == 1 else None,
            "advantages": data_b["advantages"],
            "ref_logprobs": data_b["ref_logprobs"].float().to(device),
            "old_logprobs": data_b["old_logprobs"].float().to(device),
        })
    return input_data


def _packed_loss_mask_host(data_b, seqlen: int, align: int) -> torch.Tensor:
    """CPU int32 [total padded tokens]: the training loss mask (response positions, or ``data_b['loss_mask']``)
    rolled left by one along its [mbs, seqlen] row, then laid out like the packed token row: sequence after
    sequence, each padded with zeros to a multiple of ``align``."""
    pl = [int(x) for x in data_b["prompt_token_length"]]
    rl = [int(x) for x in data_b["response_token_length"]]
    if "loss_mask" in data_b:
        m = data_b["loss_mask"].detach().cpu().to(torch.int32)
    else:
        m = torch.zeros(len(pl), seqlen, dtype=torch.int32)
        for i, (p, r) in enumerate(zip(pl, rl)):
            m[i, p:p + r] = 1
    m = torch.roll(m, shifts=-1, dims=1)
    rows = []
    for i, (p, r) in enumerate(zip(pl, rl)):
        padded = (p + r + align - 1) // align * align
        row = torch.zeros(padded, dtype=torch.int32)
        n = min(padded, seqlen)
        row[:n] = m[i, :n]
        rows.append(row)
    return torch.cat(rows) if rows else torch.zeros(0, dtype=torch.int32)


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


class _TokenLosses(torch.autograd.Function):
    """Every per-token quantity the Megatron loss dict holds that depends on the logprob, from ONE launch
    of the policy-loss kernel: the clipped surrogate (token- or sequence-level), the k3 KL with
    exp(k) forced to 1 outside the mask, and the three clip flags.  Only the surrogate carries a
    gradient (the kernel emits d loss / d logprob beside it); the reference's own loss_func detaches
    everything else (train_helper.py:441-449)."""

    @staticmethod
    def forward(ctx, logprob, old, ref, adv, mask, mode, clips):
        res = ops.policy_loss(logprob.detach().float(), old.float(), adv, mode=mode, ref_logprob=ref.float(),
                              loss_mask=mask, want_dloss=True, want_kl=True, want_flags3=(mode == LOSS_GSPO), **clips)
        bits = int(res.flags.item())       # the reference syncs here too (its three .any() assertions)
        assert not bits & 1, "pg loss is nan"
        assert not bits & 2, "kl loss ratio has inf values"
        assert not bits & 4, "kl loss ratio has nan values"
        ctx.save_for_backward(res.dloss)
        ctx.in_dtype = logprob.dtype
        # dtype of -A * ratio under torch's promotion: a list of numpy float64 advantages makes it float64
        surrogate = res.loss.to(torch.promote_types(torch.promote_types(logprob.dtype, old.dtype), adv.dtype))
        flags = (res.is_positive_clipped, res.is_negative_clipped, res.is_clipped) if mode == LOSS_GSPO else ()
        ctx.mark_non_differentiable(res.kl, *flags)
        return (surrogate, res.kl) + flags

    @staticmethod
    def backward(ctx, g_surrogate, *_):
        (dloss,) = ctx.saved_tensors
        g = None if g_surrogate is None else (g_surrogate.to(dloss.dtype) * dloss).to(ctx.in_dtype)
        return g, None, None, None, None, None, None


def _batch_rows(x: torch.Tensor, module_args, training_inputs):
    """[b, s] view of a per-token tensor: packed rows are scattered back to the padded batch."""
    return reduce_from_context_parallel_region(x, module_args.packing, training_inputs)


def _loss_dict(module_args, logprob: torch.Tensor, entropy: torch.Tensor,
               training_inputs: Dict[str, Any]) -> Dict[str, torch.Tensor]:
    """The loss dict from the [b, s] logprob (carrying the gradient) and the detached [b, s] entropy."""
    gspo = bool(module_args.use_group_sequence_policy)
    adv = torch.tensor(training_inputs["advantages"]).to(logprob.device)      # dtype rule of loss_gallery.py:19,53
    clips = {k: getattr(module_args, k) for k in ("diff_clip_ratio", "pos_clip_ratio", "neg_clip_ratio",
                                                  "final_clip_ratio")}
    surrogate, kl, *flags = _TokenLosses.apply(logprob, training_inputs["old_logprobs"],
                                               training_inputs["ref_logprobs"], adv,
                                               training_inputs['all_token_loss_mask'],
                                               LOSS_GSPO if gspo else LOSS_GRPO, clips)
    out = {'pg_loss': surrogate.contiguous(), 'entropy_loss': entropy, 'kl_loss': kl}
    if gspo:
        names = ('is_positive_clipped', 'is_negative_clipped', 'is_clipped')
        out.update(zip(names, flags))
        out.update(zip((n + '_sample_average' for n in names), flags))
    return out


def _compute_all_losses(module_args, model, all_token_logits: torch.Tensor, labels: torch.Tensor,
                        training_inputs: Dict[str, Any]) -> Dict[str, torch.Tensor]:
    """The per-token loss dict of one micro-batch (reference train_helper.py:465-547): keys ``pg_loss``,
    ``entropy_loss``, ``kl_loss`` and, for the sequence-level policy, the three clip flags twice (summed and
    sample-averaged by ``loss_func``).  ``model`` is unused: the reference only reaches through it for the
    cross entropy, which here is the softmax-statistics kernel on the given logits."""
    del model
    logprob = _batch_rows(language_model_logprob(labels, all_token_logits), module_args, training_inputs)
    entropy = _batch_rows(entropy_from_tensor_parallel_logits(all_token_logits).permute(1, 0), module_args,
                          training_inputs)
    return _loss_dict(module_args, logprob, entropy, training_inputs)


def _token_row_mask(module_args, training_inputs: Dict[str, Any], s: int, b: int):
    """(device mask, host mask) per row of the flattened [s * b, H] hidden states, from the [B, S] training
    mask: rows where it is zero get a zero upstream gradient through ``loss_func`` (which multiplies every
    entry by the mask, train_helper.py:451-455).  Packed rows are looked up through ``indices``."""
    mask = training_inputs['all_token_loss_mask']
    if module_args.packing:
        host = training_inputs.get("packed_loss_mask_host")
        if host is not None and host.numel() == s * b:
            return None, host
        B, S = training_inputs['ori_batch_size'], training_inputs['ori_seq_len']
        wide = mask.new_zeros(B, S)
        wide[:, :mask.shape[1]] = mask[:, :S]
        return index_first_axis(wide.reshape(B * S, 1).to(torch.int32), training_inputs['indices']).reshape(-1), None
    wide = mask.new_zeros(b, s)
    wide[:, :mask.shape[1]] = mask[:, :s]
    return wide.transpose(0, 1).reshape(-1).to(torch.int32), None


def compute_all_losses_from_hidden(module_args, hidden: torch.Tensor, output_weight: torch.Tensor,
                                   labels: torch.Tensor, training_inputs: Dict[str, Any], *, temperature: float = 1.0,
                                   dweight_buffer: Optional[torch.Tensor] = None, keep_logits_rows=AUTO,
                                   skip_masked_rows: bool = True) -> Dict[str, torch.Tensor]:
    """``_compute_all_losses`` with the output layer folded in (reference train_helper.py:465-547 together
    with the model's ``output_layer`` call that produces its logits, :585-594): ``hidden`` is what the
    decoder hands to the output layer at ``post_process``, ``[s, b, H]`` or ``[total_nnz, 1, H]``, and
    ``output_weight`` the ``[V, H]`` weight of that layer.  The same dict comes back - ``pg_loss`` carrying
    the gradient to ``hidden`` and ``output_weight`` through the fused backward, ``entropy_loss`` detached
    (the reference's entropy defines no backward, :605-635), ``kl_loss`` and the sequence-level clip flags -
    and goes into ``loss_func`` unchanged; the ``[*, V]`` logits are never written out.

    ``skip_masked_rows``: ``loss_func`` multiplies every entry by ``all_token_loss_mask``, so rows outside
    the mask get an exactly zero gradient; their logits are then not kept and the backward leaves them out.
    Pass False when the loss dict is consumed by something that does not apply the mask.
    ``dweight_buffer`` (fp32 [V, H], e.g. the weight's ``main_grad``) receives ``+= dW``."""
    s, b, H = hidden.shape
    flat_labels = labels.transpose(0, 1).reshape(-1)
    dev_mask = host_mask = None
    if skip_masked_rows:
        dev_mask, host_mask = _token_row_mask(module_args, training_inputs, s, b)
    lp, ent = fused_linear_logprob_entropy(hidden.reshape(s * b, H), output_weight, flat_labels,
                                           temperature=temperature, need_entropy=True, dweight_buffer=dweight_buffer,
                                           keep_logits_rows=keep_logits_rows, loss_mask=dev_mask,
                                           loss_mask_host=host_mask)
    logprob = _batch_rows(lp.reshape(s, b).transpose(0, 1), module_args, training_inputs)
    entropy = _batch_rows(ent.detach().reshape(s, b).permute(1, 0), module_args, training_inputs)
    return _loss_dict(module_args, logprob, entropy, training_inputs)


def logprobs_from_hidden(module_args, hidden: torch.Tensor, output_weight: torch.Tensor, labels: torch.Tensor,
                         inputs: Dict[str, Any], *, temperature: float = 1.0) -> torch.Tensor:
    """The no-grad branch of the reference's ``forward_step`` (train_helper.py:585-600): with labels the
    model returns -cross entropy per token, re-padded to [B, S]; here from the hidden states."""
    s, b, H = hidden.shape
    with torch.no_grad():
        lp, *_ = ops.lmhead_forward(hidden.reshape(s * b, H), output_weight, labels.transpose(0, 1).reshape(-1),
                                    temperature, need_entropy=False)
    return _batch_rows(lp.reshape(s, b).transpose(0, 1), module_args, inputs)


class _MaskedSums(torch.autograd.Function):
    """One launch reduces every tensor of the loss dict under the mask; the tensors listed in
    ``grad_slots`` get the gradient mask * g back."""

    @staticmethod
    def forward(ctx, mask, grad_slots, averaged, *tensors):
        sums, count = ops.masked_sums(tensors, mask, averaged)
        ctx.mask, ctx.grad_slots = mask, grad_slots
        ctx.like = [(t.dtype, t.shape) for t in tensors]
        ctx.mark_non_differentiable(count)
        return sums, count

    @staticmethod
    def backward(ctx, g_sums, _):
        grads = [None] * len(ctx.like)
        if g_sums is not None:
            g_sums = g_sums.float().contiguous()
            for j in ctx.grad_slots:
                dtype, shape = ctx.like[j]
                grads[j] = ops.masked_sums_backward(g_sums[j:j + 1], ctx.mask, dtype, shape)
        return (None, None, None) + tuple(grads)


BACKPROP_KEYS = ('pg_loss',)     # train_helper.py:441


def loss_func(inputs: Dict, losses: Dict[str, torch.Tensor]):
    """(loss to back-propagate, number of unmasked tokens, report) from the per-token loss dict
    (reference train_helper.py:426-463): every entry is summed under ``all_token_loss_mask`` (zeros and ones,
    as every mask the trainers build; it travels to the kernel as int32),
    the ``*_sample_average`` entries are divided by (1e-5 + number of unmasked tokens), only ``pg_loss``
    keeps its gradient.  All reductions run in one kernel launch."""
    names = list(losses)
    grad_slots = tuple(j for j, name in enumerate(names) if name in BACKPROP_KEYS and losses[name].requires_grad)
    averaged = tuple(name.endswith('_sample_average') for name in names)
    sums, count = _MaskedSums.apply(inputs["all_token_loss_mask"], grad_slots, averaged,
                                    *(losses[name] for name in names))
    report = {name: sums[j].detach().clone() for j, name in enumerate(names)}
    total = 0
    for j, name in enumerate(names):
        if name in BACKPROP_KEYS:
            total = total + sums[j]
    num_tokens = inputs.get('num_tokens_on_this_cp_rank', count[0]).to(torch.int)
    report["num_tokens"] = num_tokens
    report["num_samples"] = torch.ones_like(num_tokens)
    return total, num_tokens, report
