"""Oracle: masks, position ids, label shift, unpad / pad of packed batches.

Test infrastructure only; never imported by the product package.

Reference semantics restated here:
  * generate_loss_mask_position_ids (text)  trainer_utils.py:60-96
  * unpad_input                              trainer_utils.py:155-194
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


def generate_loss_mask_position_ids(tokens, prompt_token_length, response_token_length):
    """int32 attn/loss masks from the two length lists; position ids are a
    broadcast arange (trainer_utils.py:68-96, text-only branch)."""
    loss_mask = torch.zeros_like(tokens, dtype=torch.int32)
    attn_mask = torch.zeros_like(tokens, dtype=torch.int32)
    for i, (p, r) in enumerate(zip(prompt_token_length, response_token_length)):
        loss_mask[i, p:p + r] = 1
        attn_mask[i, :p + r] = 1
    seq_len = tokens.shape[1]
    pos = torch.arange(seq_len, dtype=torch.long, device=tokens.device).unsqueeze(0).expand_as(tokens)
    return attn_mask, loss_mask, pos


def index_first_axis(x, indices):
    return x[indices]


def unpad_input(hidden_states, attention_mask):
    """trainer_utils.py:155-194 (3-D branch)."""
    seqlens = attention_mask.sum(dim=-1, dtype=torch.int32)
    indices = torch.nonzero(attention_mask.flatten(), as_tuple=False).flatten()
    max_seqlen = seqlens.max().item()
    cu_seqlens = F.pad(torch.cumsum(seqlens, dim=0, dtype=torch.int32), (1, 0))
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
