"""Mirror of chatlearn/algorithm/grpo_utils/packing_utils.py (dynamic-batching bin
packing).  The packing decisions run in the library's host-side C++ routines
(clgrpo_bin_packing / clgrpo_bin_packing_fix_bin); this file keeps the
reference's names, signatures and return shapes."""
from typing import Any, Dict, List, Union
import warnings

import torch

from ... import ops


def bin_packing(seq_len_list: List[int], max_train_token: int):
    """Best-fit-decreasing packing; returns (bins_id, bins_seqlen) as the reference does
    (packing_utils.py:23-54).  An item longer than the cap only warns."""
    if any(x > max_train_token for x in seq_len_list):
        warnings.warn(
            f"Max length in microbatch exceeds max_token_in_seq, max length: {max(seq_len_list)}, "
            f"max_train_token: {max_train_token}")
    bins_id = ops.bin_packing_ids(seq_len_list, max_train_token)
    bins_seqlen = [[seq_len_list[i] for i in b] for b in bins_id]
    return bins_id, bins_seqlen


def bin_packing_fix_bin(seq_len_list: List[int], bin_size: int):
    """Longest-first into the lightest of ``bin_size`` bins, bins ordered by total length
    descending (packing_utils.py:56-83).  As in the reference, the length lists are ordered by
    their own (total, list) key, independently of the id lists."""
    bins_id = ops.bin_packing_fix_bin_ids(seq_len_list, bin_size)
    lens = [[seq_len_list[i] for i in b] for b in bins_id]
    bins_seqlen = [b for _, b in sorted(((sum(b), b) for b in lens), reverse=True)]
    return bins_id, bins_seqlen


def regroup_data_from_list(data_all: Dict, data_position: List[int]):
    if isinstance(data_all, torch.Tensor):
        return data_all[torch.tensor(data_position)]
    if isinstance(data_all, list):
        return [data_all[item] for item in data_position]
    return None


def regroup_data_packing(
    data_list: List[Dict[str, Union[torch.Tensor, List[Any]]]],
    process_group_list: List[Any],
    max_train_token: int,
    offset: int
) -> List[Dict[str, Union[torch.Tensor, List[Any]]]]:
    """Split a list of samples into micro-batches of at most ``max_train_token`` tokens
    (packing_utils.py:105-148).  The bin count is MAX-reduced over each process group when
    torch.distributed is initialised; on a single process that reduction is the identity."""
    total_token_length = [d["prompt_token_length"] + d["response_token_length"] for d in data_list]
    bins_id, _ = bin_packing(seq_len_list=total_token_length, max_train_token=max_train_token)
    n_bins = len(bins_id)
    if torch.distributed.is_available() and torch.distributed.is_initialized() \
            and torch.distributed.get_world_size() > 1:
        dev = torch.device("cuda", torch.cuda.current_device()) if torch.cuda.is_available() else "cpu"
        t = torch.tensor(n_bins, device=dev)
        for pg in (process_group_list or [None]):
            torch.distributed.all_reduce(t, op=torch.distributed.ReduceOp.MAX, group=pg)
        n_bins = int(t.cpu().item())
    bins_id, _ = bin_packing_fix_bin(seq_len_list=total_token_length, bin_size=n_bins)
    regroup_data_list = []
    for micro_batch_id in bins_id:
        regroup_data_list.append([])
        for sample_id in micro_batch_id:
            packed_sample = data_list[sample_id]
            packed_sample.update({'id_in_list': sample_id + offset})
            regroup_data_list[-1].append(packed_sample)
    return regroup_data_list
