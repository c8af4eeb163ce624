"""Oracle: masks, position ids, label shift, unpad / pad of packed batches.

Test infrastructure only; never imported by the product package.

Reference semantics restated here:
  * generate_loss_mask_position_ids         trainer_utils.py:60-96 (text and the three-channel
                                             vision-language position ids)
  * unpad_input                              trainer_utils.py:155-194 (incl. the channel-first 4-D branch)
  * index_first_axis / pad_input             flash-attn bert_padding (a row
    gather and its inverse scatter into zeros), call sites
    trainer_utils.py:179,190 and policy_trainer.py:239-248,350-355
  * split_and_unpadding                      trainer_utils.py:148-153
  * label roll / training-mask shift         policy_trainer.py:135,160-162
  * Megatron training-mask shift (no zeroing of the last column)
                                             train_helper.py:405-413

Integer work: every result here is compared bit-for-bit.
"""
import torch
import torch.nn.functional as F


def generate_loss_mask_position_ids(tokens, prompt_token_length, response_token_length, prompt_position_ids=None):
    """int32 attn/loss masks from the two length lists; position ids are a broadcast arange
    (trainer_utils.py:68-96, text-only branch) or, with ``prompt_position_ids`` (per sample three
    lists), a [3, B, S] tensor: each channel starts with the given list and continues counting up from
    its maximum + 1 (trainer_utils.py:76-92)."""
    loss_mask = torch.zeros_like(tokens, dtype=torch.int32)
    attn_mask = torch.zeros_like(tokens, dtype=torch.int32)
    for i, (p, r) in enumerate(zip(prompt_token_length, response_token_length)):
        loss_mask[i, p:p + r] = 1
        attn_mask[i, :p + r] = 1
    batch_size, seq_len = tokens.shape
    if prompt_position_ids:
        pos = torch.zeros((3, batch_size, seq_len), dtype=torch.long)
        for b, channels in enumerate(prompt_position_ids):
            for ch in range(3):
                sub = channels[ch]
                pos[ch, b, :len(sub)] = torch.tensor(sub)
                start = max(sub) + 1
                pos[ch, b, len(sub):] = torch.arange(start, start + (seq_len - len(sub)))
        return attn_mask, loss_mask, pos
    pos = torch.arange(seq_len, dtype=torch.long, device=tokens.device).unsqueeze(0).expand_as(tokens)
    return attn_mask, loss_mask, pos


def index_first_axis(x, indices):
    return x[indices]


def unpad_input(hidden_states, attention_mask):
    """trainer_utils.py:155-194; a tensor of more than three dimensions is (channel, batch, seqlen, ...)
    and is unpadded channel by channel (:176-187)."""
    seqlens = attention_mask.sum(dim=-1, dtype=torch.int32)
    indices = torch.nonzero(attention_mask.flatten(), as_tuple=False).flatten()
    max_seqlen = seqlens.max().item()
    cu_seqlens = F.pad(torch.cumsum(seqlens, dim=0, dtype=torch.int32), (1, 0))
    if hidden_states.dim() > 3:
        per_channel = [index_first_axis(hidden_states[ch].reshape(-1, *hidden_states.shape[3:]), indices)
                       for ch in range(hidden_states.shape[0])]
        return torch.stack(per_channel), indices, cu_seqlens, max_seqlen
    flat = hidden_states.reshape(-1, *hidden_states.shape[2:])
    return index_first_axis(flat, indices), indices, cu_seqlens, max_seqlen


def pad_input(x, indices, batch, seqlen):
    """Inverse of the gather: zeros [batch*seqlen, ...] with rows written at ``indices``."""
    out = torch.zeros(batch * seqlen, *x.shape[1:], dtype=x.dtype, device=x.device)
    out[indices] = x
    return out.reshape(batch, seqlen, *x.shape[1:])


def split_and_unpadding(input_tensor, attention_mask):
    """trainer_utils.py:148-153."""
    valid = torch.sum(attention_mask, dim=-1).cpu().tolist()
    return [input_tensor[i, :valid[i]] for i in range(input_tensor.shape[0])]


def shift_labels(tokens):
    """labels = roll(tokens, -1, dim 1) (policy_trainer.py:71,135)."""
    return torch.roll(tokens, shifts=-1, dims=1)


def shift_loss_mask_fsdp(loss_mask):
    """policy_trainer.py:160-162: roll left by one, zero the last column."""
    m = torch.roll(loss_mask, shifts=-1, dims=1)
    m[:, -1] = 0
    return m


def shift_loss_mask_megatron(loss_mask):
    """train_helper.py:405-413: roll left by one only."""
    return torch.roll(loss_mask, shifts=-1, dims=1)


def thd_partitioned_indices(cu_seqlens, total_tokens, world_size, rank):
    """Positions of a packed (THD) row that one context-parallel rank keeps.

    The reference calls TransformerEngine's ``tex.thd_get_partitioned_indices``
    (megatron_utils/train_helper.py:289-291); TransformerEngine (2.7 in the reference's
    images, docs/en/installation.md:28) is a third-party dependency that is not
    vendored, so this restates its published scheme: every
    sequence is cut into ``2 * world_size`` equal chunks and rank ``r`` keeps chunks
    ``r`` and ``2 * world_size - 1 - r`` (load balancing under a causal mask), in
    sequence order.  For ``world_size == 1`` this is ``arange(total_tokens)``, which
    is all the reference's own single-rank use needs; for more ranks the parity of
    this function with TransformerEngine is unpinned (no fixture of it exists in the
    reference) and only its defining properties are tested
    (tests/test_oracle_cpu.py::test_context_parallel_partition_properties): the ranks'
    index sets partition the row, each is ascending, and every rank gets the same
    amount of causal-attention work per sequence.
    """
    out = []
    for i in range(len(cu_seqlens) - 1):
        start, end = int(cu_seqlens[i]), int(cu_seqlens[i + 1])
        chunk = (end - start) // (2 * world_size)
        for c in (rank, 2 * world_size - 1 - rank):
            out.extend(range(start + c * chunk, start + (c + 1) * chunk))
    assert len(out) == total_tokens // world_size
    return torch.tensor(out, dtype=torch.int64)


def megatron_packed_batch(tokens, prompt_token_length, response_token_length, eod, tp_size=1, cp_size=1, cp_rank=0):
    """The packed branch of the Megatron trainer's ``get_batch`` (train_helper.py:258-328),
    written with the same loops on CPU tensors.  Returns the dict that branch builds
    (``packed_seq_params`` as a plain dict)."""
    tokens = tokens.long()
    mbs, seqlen = tokens.shape
    align_size = tp_size * cp_size * 2
    attn_mask = torch.zeros_like(tokens, dtype=torch.int32)
    for i, (p, r) in enumerate(zip(prompt_token_length, response_token_length)):
        attn_mask[i, : p + r] = 1
    seqlens_in_batch = attn_mask.sum(dim=-1, dtype=torch.int32)
    pad_size = (align_size - seqlens_in_batch % align_size) % align_size
    seqlens_in_batch_padded = seqlens_in_batch + pad_size
    width = int(seqlens_in_batch_padded.max())
    tokens_padded = torch.full((mbs, width), eod, dtype=tokens.dtype)
    attn_mask_for_padding = torch.zeros((mbs, width), dtype=tokens.dtype)
    for i in range(mbs):
        n, n_pad = int(seqlens_in_batch[i]), int(seqlens_in_batch_padded[i])
        tokens_padded[i, :n] = tokens[i, :n]
        attn_mask_for_padding[i, :n_pad] = 1
    packed, indices, cu_seqlens_padded, max_seqlen_in_batch = unpad_input(tokens_padded.unsqueeze(-1),
                                                                         attn_mask_for_padding)[:4]
    seq_indices = thd_partitioned_indices(cu_seqlens_padded, packed.shape[0], cp_size, cp_rank)
    tokens_rank = packed.index_select(0, seq_indices)
    labels = torch.roll(packed, shifts=-1, dims=0)
    labels_rank = labels.index_select(0, seq_indices)
    loss_mask = torch.zeros_like(packed, dtype=torch.int32)
    for i, (p, r) in enumerate(zip(prompt_token_length, response_token_length)):
        start = int(cu_seqlens_padded[i])
        loss_mask[start + p: start + p + r, 0] = 1
    loss_mask = torch.roll(loss_mask, shifts=-1, dims=0)
    loss_mask_rank = loss_mask.index_select(0, seq_indices)
    return {
        "all_tokens": tokens_rank.transpose(0, 1),
        "labels": labels_rank.transpose(0, 1),
        "packed_seq_params": {"qkv_format": "thd", "cu_seqlens_q": cu_seqlens_padded,
                              "cu_seqlens_kv": cu_seqlens_padded, "max_seqlen_q": max_seqlen_in_batch,
                              "max_seqlen_kv": max_seqlen_in_batch},
        "ori_seq_len": seqlens_in_batch_padded.max(),
        "ori_batch_size": mbs,
        "seq_indices": seq_indices.unsqueeze(0),
        "indices": indices,
        "num_tokens_on_this_cp_rank": loss_mask_rank.sum(),
        "pad_size": seqlens_in_batch_padded.max() - seqlen,
        "loss_mask_on_this_cp_rank": loss_mask_rank,
    }
