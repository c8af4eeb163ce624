"""Oracle: the head's statistics when the vocabulary is split over tensor-parallel ranks.

Test infrastructure only; never imported by the product package.

Restated here, with the ranks simulated as a Python list of logit shards and the
all-reduces written as reductions over that list:

  * ``_VocabParallelEntropy.forward``            megatron_utils/train_helper.py:605-627
    (max all-reduce, sum-of-exponentials all-reduce, sum of p*z all-reduce).
  * vocab-parallel cross entropy.  The reference calls it through
    ``compute_language_model_loss`` (train_helper.py:480-482); the routine itself
    lives in Megatron-Core (third party, not vendored: the reference's scripts point
    at Pai-Megatron-Patch's Megatron-LM-250624 / -250908 snapshots).  Its published
    algorithm: all-reduce(MAX) of the shard maxima, subtract, each rank gathers the
    target logit if the label falls into its vocabulary range (else 0) and the
    gathered values are all-reduced (SUM), sum of exponentials all-reduced (SUM),
    loss = log(sum_exp) - target.

Pinned by: equality with the unsharded log_softmax / entropy for any sharding
(tests), which fixes signs, the masked gather and the max shift.
"""
import torch


def shard_ranges(vocab_size, n_shards):
    """Megatron's even vocabulary split: rank r owns [r*V/n, (r+1)*V/n) (V divisible by n)."""
    assert vocab_size % n_shards == 0
    per = vocab_size // n_shards
    return [(r * per, (r + 1) * per) for r in range(n_shards)]


def vocab_parallel_entropy(logit_shards):
    """Entropy per token from per-rank logit shards [..., V/n] (train_helper.py:605-627)."""
    shards = [s.float().clone() for s in logit_shards]
    logits_max = torch.stack([s.max(dim=-1)[0] for s in shards]).max(dim=0)[0]          # all_reduce MAX
    exp_shards = [(s - logits_max.unsqueeze(-1)).exp() for s in shards]
    sum_exp = torch.stack([e.sum(dim=-1) for e in exp_shards]).sum(dim=0)               # all_reduce SUM
    sm_times_logits = torch.stack([
        (e / sum_exp.unsqueeze(-1) * s0.float()).sum(dim=-1) for e, s0 in zip(exp_shards, logit_shards)
    ]).sum(dim=0)                                                                        # all_reduce SUM
    return logits_max + sum_exp.log() - sm_times_logits


def vocab_parallel_logprob(logit_shards, labels, ranges):
    """-cross_entropy per token from per-rank logit shards; labels are global ids."""
    shards = [s.float() for s in logit_shards]
    logits_max = torch.stack([s.max(dim=-1)[0] for s in shards]).max(dim=0)[0]
    target = torch.zeros_like(logits_max)
    sum_exp = torch.zeros_like(logits_max)
    for s, (lo, hi) in zip(shards, ranges):
        shifted = s - logits_max.unsqueeze(-1)
        inside = (labels >= lo) & (labels < hi)
        local = (labels - lo).clamp(0, hi - lo - 1)
        picked = shifted.gather(-1, local.unsqueeze(-1)).squeeze(-1)
        target = target + torch.where(inside, picked, torch.zeros_like(picked))        # all_reduce SUM
        sum_exp = sum_exp + shifted.exp().sum(dim=-1)                                    # all_reduce SUM
    return target - sum_exp.log()
