"""Mirror of chatlearn/algorithm/grpo_utils/trainer_utils.py: same names and
signatures.  Softmax statistics, masks, label shifts, unpad indices and row
gathers run in HIP kernels; list regrouping and right-padding of per-sample
tensors are host-side data marshalling, as in the reference."""
from collections import defaultdict
from typing import List, Any, Dict, Optional

import torch

from ... import ops
from ...bert_padding import index_first_axis
from .packing_utils import regroup_data_packing


def _work_device(t: torch.Tensor) -> torch.device:
    return t.device if t.is_cuda else torch.device("cuda", torch.cuda.current_device())


class _StatsFromLogits(torch.autograd.Function):
    """(logprob, entropy) fp32 from materialised logits, one fused pass per row."""

    @staticmethod
    def forward(ctx, logits2d, labels, want_lp, want_ent):
        lp, ent, lse = ops.softmax_stats(logits2d, labels, need_entropy=want_ent, need_logprob=want_lp)
        ctx.set_materialize_grads(False)
        none = torch.empty(0, device=logits2d.device)
        # the row statistics ride along (a few bytes per row) so that the backward reads each row once
        ctx.save_for_backward(logits2d, labels if labels is not None else none, lse, ent if want_ent else none)
        ctx.want = (want_lp, want_ent)
        empty = torch.empty(0, device=logits2d.device)
        outs = (lp if want_lp else empty, ent if want_ent else empty)
        if not want_lp:
            ctx.mark_non_differentiable(outs[0])
        if not want_ent:
            ctx.mark_non_differentiable(outs[1])
        return outs

    @staticmethod
    def backward(ctx, g_lp, g_ent):
        logits2d, labels, lse, ent = ctx.saved_tensors
        want_lp, want_ent = ctx.want
        g_lp = g_lp.float().contiguous() if (want_lp and g_lp is not None) else None
        g_ent = g_ent.float().contiguous() if (want_ent and g_ent is not None) else None
        if g_lp is None and g_ent is None:
            return None, None, None, None
        return ops.softmax_stats_backward(logits2d, labels if g_lp is not None else None, g_lp, g_ent, lse=lse,
                                          entropy=ent if g_ent is not None else None), None, None, None


def _flatten_logits(logits):
    return logits.reshape(-1, logits.shape[-1])


def entropy_from_logits(logits: torch.Tensor):
    """Calculate entropy from logits (reference trainer_utils.py:27-31); result in the logits' dtype."""
    _, ent = _StatsFromLogits.apply(_flatten_logits(logits), None, False, True)
    return ent.reshape(logits.shape[:-1]).to(logits.dtype)


def entropy_from_logits_with_chunking(logits: torch.Tensor, chunk_size: int = 512):
    """Entropy as fp32 [batch, seq] (reference trainer_utils.py:33-44).  The reference walks dim 1
    in ``chunk_size`` pieces only to bound memory; one fused pass per row needs no chunking."""
    del chunk_size
    _, ent = _StatsFromLogits.apply(_flatten_logits(logits), None, False, True)
    return ent.reshape(logits.shape[:-1])


def logprobs_from_logits(logits: torch.Tensor, labels: torch.Tensor) -> torch.Tensor:
    """log_softmax(logits)[labels] in the logits' dtype (reference trainer_utils.py:46-52)."""
    lp, _ = _StatsFromLogits.apply(_flatten_logits(logits), labels.reshape(-1), True, False)
    return lp.reshape(labels.shape).to(logits.dtype)


def sp_split(input_tensor: torch.Tensor, split_dim: int, sp_size: int, sp_local_rank: int):
    """split input by sp_size"""
    return torch.chunk(input_tensor, sp_size, split_dim)[sp_local_rank]


def generate_loss_mask_position_ids(
    tokens: torch.Tensor,
    prompt_token_length: List[int],
    response_token_length: List[int],
    prompt_position_ids: Optional[List[List[int]]] = None
):
    """attn_mask / loss_mask int32 [B,S] and position ids from the prompt and response lengths
    (reference trainer_utils.py:60-96).  The masks come from one kernel launch instead of a
    Python loop over the batch; results are returned on ``tokens.device``."""
    batch_size, seq_len = tokens.size()
    dev = _work_device(tokens)
    plen = torch.tensor(list(prompt_token_length), dtype=torch.int32).to(dev)
    rlen = torch.tensor(list(response_token_length), dtype=torch.int32).to(dev)
    if plen.numel() < batch_size:
        # rows without a length entry stay all-zero in the reference's loop
        pad = torch.zeros(batch_size - plen.numel(), dtype=torch.int32, device=dev)
        plen, rlen = torch.cat([plen, pad]), torch.cat([rlen, pad])
    attn_mask, loss_mask, position_ids = ops.build_masks(plen, rlen, seq_len, want_position_ids=not prompt_position_ids)
    attn_mask, loss_mask = attn_mask.to(tokens.device), loss_mask.to(tokens.device)
    if prompt_position_ids:
        # vision-language rows (reference trainer_utils.py:76-92): three position channels arrive as
        # Python lists; each is copied in and continued by counting up from its largest value
        position_ids = torch.zeros((3, batch_size, seq_len), dtype=torch.long, device=tokens.device)
        for b, channels in enumerate(prompt_position_ids):
            for ch in range(3):
                given = torch.as_tensor(channels[ch], dtype=torch.long)
                n = given.numel()
                position_ids[ch, b, :n] = given
                position_ids[ch, b, n:] = int(given.max()) + 1 + torch.arange(seq_len - n)
    else:
        position_ids = position_ids.to(tokens.device)
    return attn_mask, loss_mask, position_ids


def split_microbatch(
    data_list: List,
    micro_batch_size: int = None,
    max_train_token: int = None,
    process_group_list: List[Any] = None,
    offset: int = 0, packing: bool = False
):
    """Micro-batches of a mini-batch: token-budget bins when packing, else consecutive runs of
    ``micro_batch_size`` samples; every sample is tagged with its position ``id_in_list``
    (reference trainer_utils.py:98-119)."""
    assert micro_batch_size is not None or max_train_token is not None, \
        "At least one of micro_batch_size or max_train_token should be specified"
    if packing:
        return regroup_data_packing(data_list, process_group_list, max_train_token, offset)
    total = len(data_list)
    out = []
    for start in range(0, total, micro_batch_size):
        run = []
        for position in range(start, min(start + micro_batch_size, total)):
            data_list[position].update({'id_in_list': position})
            run.append(data_list[position])
        out.append(run)
    return out


def padding_tensor(tensor_list):
    """Stack tensors of different first-dimension lengths, zero-padded at the end of that dimension
    (reference trainer_utils.py:121-129)."""
    longest = max(t.shape[0] for t in tensor_list)
    padded = []
    for t in tensor_list:
        grown = t.new_zeros((longest,) + tuple(t.shape[1:]))
        grown[:t.shape[0]] = t
        padded.append(grown)
    return torch.stack(padded)


def batching(data_list: List[Dict[str, Any]]) -> Dict[str, Any]:
    """Per-key lists of a micro-batch; tensors are padded and stacked, the two vision keys are
    concatenated (reference trainer_utils.py:131-146)."""
    if len(data_list) == 0:
        return None
    batched_data = defaultdict(list)
    for key in data_list[0]:
        column = [sample[key] for sample in data_list]
        if key in ('pixel_values', 'image_grid_thw'):
            column = torch.cat(column, dim=0)
        elif isinstance(column[0], torch.Tensor):
            column = padding_tensor(column)
        batched_data[key] = column
    return batched_data


def split_and_unpadding(input_tensor: torch.Tensor, attention_mask: torch.Tensor) -> List[torch.Tensor]:
    valid_seq = torch.sum(attention_mask, dim=-1).cpu().tolist()
    return [input_tensor[i, :valid_seq[i]] for i in range(input_tensor.shape[0])]


def unpad_input(hidden_states, attention_mask):
    """
    Arguments:
        hidden_states: (batch, seqlen, ...) or, for vision-language position ids, (channel, batch, seqlen, ...)
        attention_mask: (batch, seqlen), bool / int, 1 means valid and 0 means not valid.
    Return:
        hidden_states: (total_nnz, ...), indices (total_nnz) int64, cu_seqlens (batch + 1) int32,
        max_seqlen_in_batch: int        (reference trainer_utils.py:155-194)
    """
    indices, cu_seqlens, _, max_seqlen_in_batch = ops.unpad_indices(attention_mask)
    if len(hidden_states.shape) > 3:
        channel_results = [
            index_first_axis(hidden_states[ch].reshape(-1, *hidden_states.shape[3:]), indices)
            for ch in range(hidden_states.shape[0])
        ]
        return torch.stack(channel_results), indices, cu_seqlens, max_seqlen_in_batch
    flat = hidden_states.reshape(-1, *hidden_states.shape[2:])
    return index_first_axis(flat, indices), indices, cu_seqlens, max_seqlen_in_batch
