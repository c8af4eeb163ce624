"""Oracle: dynamic-batching bin packing and micro-batch regrouping.

Test infrastructure only; never imported by the product package.

Reference semantics restated here:
  * best-fit-decreasing packing            packing_utils.py:23-54
  * fixed-bin-count balancing              packing_utils.py:56-83
  * regroup into micro-batches             packing_utils.py:105-148
  * split_microbatch                       trainer_utils.py:98-123
  * padding_tensor / batching              trainer_utils.py:125-146

Integer work: every result here is compared bit-for-bit.
"""
import math
import warnings
from collections import defaultdict

import numpy as np
import torch
import torch.nn.functional as F


def _descending_stable(seq_len_list):
    """(index, length) pairs by length, longest first; equal lengths keep their
    original relative order (Python's sort is stable also with reverse=True),
    packing_utils.py:31-32,60-61."""
    return sorted(enumerate(seq_len_list), key=lambda kv: kv[1], reverse=True)


def bin_packing(seq_len_list, max_train_token):
    """packing_utils.py:23-54.  An item goes to the open bin with the least
    free space among those with STRICTLY more free space than the item needs
    (first such bin on equal free space); otherwise it opens a new bin.  An
    item longer than the cap only triggers a warning."""
    if sum(np.array(seq_len_list) > max_train_token) > 0:
        warnings.warn(
            f"Max length in microbatch exceeds max_token_in_seq, max length: {max(seq_len_list)}, "
            f"max_train_token: {max_train_token}")
    ids, lens = [], []
    for idx, need in _descending_stable(seq_len_list):
        pick, pick_free = None, None
        for b, members in enumerate(lens):
            free = max_train_token - sum(members)
            if free > need and (pick is None or free < pick_free):
                pick, pick_free = b, free
        if pick is None:
            ids.append([idx])
            lens.append([need])
        else:
            ids[pick].append(idx)
            lens[pick].append(need)
    return list(ids), list(lens)


def bin_packing_fix_bin(seq_len_list, bin_size):
    """packing_utils.py:56-83.  Longest first into the currently lightest of
    ``bin_size`` bins (first one on ties); bins are then ordered by total
    length, descending, where Python compares (total, list) tuples - so equal
    totals fall back to comparing the lists themselves.  The id lists and the
    length lists are sorted independently, as the reference does."""
    ids = [[] for _ in range(bin_size)]
    lens = [[] for _ in range(bin_size)]
    for idx, need in _descending_stable(seq_len_list):
        pick, pick_sum = None, None
        for b, members in enumerate(lens):
            tot = need + sum(members)
            if pick_sum is None or tot < pick_sum:
                pick, pick_sum = b, tot
        ids[pick].append(idx)
        lens[pick].append(need)
    totals = [sum(m) for m in lens]
    ids_sorted = [b for _, b in sorted(zip(totals, ids), reverse=True)]
    lens_sorted = [b for _, b in sorted(zip(totals, lens), reverse=True)]
    return ids_sorted, lens_sorted


def regroup_data_packing(data_list, process_group_list, max_train_token, offset):
    """packing_utils.py:105-148 on one rank: the MAX all-reduce of the bin
    count over each process group is the identity."""
    total = [d["prompt_token_length"] + d["response_token_length"] for d in data_list]
    first, _ = bin_packing(total, max_train_token)
    n_bins = len(first)
    bins, _ = bin_packing_fix_bin(total, n_bins)
    out = []
    for members in bins:
        out.append([])
        for sid in members:
            sample = data_list[sid]
            sample.update({"id_in_list": sid + offset})
            out[-1].append(sample)
    return out


def split_microbatch(data_list, micro_batch_size=None, max_train_token=None,
                     process_group_list=None, offset=0, packing=False):
    """trainer_utils.py:98-123."""
    assert micro_batch_size is not None or max_train_token is not None, \
        "At least one of micro_batch_size or max_train_token should be specified"
    if packing:
        return regroup_data_packing(data_list, process_group_list, max_train_token, offset)
    n = len(data_list)
    n_mb = math.ceil(n / micro_batch_size)
    out = [[] for _ in range(n_mb)]
    for i in range(n_mb):
        for sid in range(i * micro_batch_size, min((i + 1) * micro_batch_size, n)):
            data_list[sid].update({"id_in_list": sid})
            out[i].append(data_list[sid])
    return out


def padding_tensor(tensor_list):
    """trainer_utils.py:125-135: right-pad dim 0 with zeros to the longest, stack."""
    nd = tensor_list[0].dim()
    longest = max(t.shape[0] for t in tensor_list)
    return torch.stack([F.pad(t, (0, 0) * (nd - 1) + (0, longest - t.shape[0])) for t in tensor_list])


def batching(data_list):
    """trainer_utils.py:137-146."""
    if len(data_list) == 0:
        return None
    out = defaultdict(list)
    for key in data_list[0]:
        col = [d[key] for d in data_list]
        if key in ("pixel_values", "image_grid_thw"):
            col = torch.cat(col, dim=0)
        elif isinstance(col[0], torch.Tensor):
            col = padding_tensor(col)
        out[key] = col
    return out
