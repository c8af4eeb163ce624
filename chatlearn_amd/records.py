"""Host-side record formats and batch order either side of the policy-loss path.

* ``rollout_record``: the per-response sample dict the rollout engines emit
  (reference models/vllm_module.py:558-583, models/sglang_module.py:673-679,
  models/agent/agent_module.py:85-112) - the input of the reward and advantage stages.
* ``check_train_record``: what the trainer's pre-processing reads from a sample
  (algorithm/grpo_utils/policy_trainer.py:80-172, 187-365); raises a ValueError that names the
  field instead of failing deep inside batching.
* ``even_slice`` / ``slice_data_list_by_index`` (utils/utils.py:320-338) and
  ``minibatch_slice_index`` / ``iter_fixed_order`` (data/data.py:154-180): the order in which the
  replay buffer is cut into data-parallel shares and mini-batches, so that advantages computed
  over the episode line up with the mini-batches the trainer sees.

Pure host logic (lists and ints); nothing here touches the device.
"""
import copy
from typing import Any, Dict, Iterator, List, Optional, Sequence

import torch

ROLLOUT_FIELDS = ("all_tokens", "prompt_token_length", "response_token_length", "str_outputs")
TRAIN_FIELDS = ("all_tokens", "prompt_token_length", "response_token_length", "old_logprobs", "ref_logprobs",
                "advantages")


def rollout_record(input_data: Dict[str, Any], prompt_token_ids: Sequence[int], output_token_ids: Sequence[int],
                   str_outputs: Optional[str] = None, loss_mask: Optional[Sequence[int]] = None) -> Dict[str, Any]:
    """One response as the rollout stage hands it on: a deep copy of the prompt's input dict (it
    carries ``prompt_uid``, ``data_source``, ``ground_truth`` ...) updated with the token record.
    ``loss_mask`` (multi-turn agents) covers all tokens, prompt included."""
    data_obj = copy.deepcopy(input_data)
    prompt_token_ids, output_token_ids = list(prompt_token_ids), list(output_token_ids)
    data_obj.update({
        "all_tokens": torch.tensor(prompt_token_ids + output_token_ids),
        "response_token_length": len(output_token_ids),
        "prompt_token_length": len(prompt_token_ids),
        "str_outputs": str_outputs,
    })
    if loss_mask is not None:
        data_obj["loss_mask"] = torch.tensor(list(loss_mask))
        data_obj["all_token_length"] = len(prompt_token_ids) + len(output_token_ids)
    if "rollout_round" in data_obj:
        data_obj["rollout_round"] += 1
    return data_obj


def check_train_record(sample: Dict[str, Any], training: bool = True) -> None:
    """Validate one sample against what ``PolicyStep.preprocess_data_list`` will read."""
    need = TRAIN_FIELDS if training else TRAIN_FIELDS[:3]
    for key in need:
        if key not in sample:
            raise ValueError(f"sample lacks '{key}'")
    tokens = sample["all_tokens"]
    if not isinstance(tokens, torch.Tensor) or tokens.dim() != 1:
        raise ValueError("'all_tokens' must be a 1-D tensor")
    p, r = int(sample["prompt_token_length"]), int(sample["response_token_length"])
    if p < 0 or r < 0 or p + r != tokens.numel():
        raise ValueError(f"prompt_token_length + response_token_length = {p + r} but all_tokens has {tokens.numel()}")
    if "loss_mask" in sample and len(sample["loss_mask"]) != tokens.numel():
        raise ValueError("'loss_mask' must cover all tokens")
    if training:
        for key in ("old_logprobs", "ref_logprobs"):
            v = sample[key]
            if not isinstance(v, torch.Tensor) or v.dim() != 1 or v.numel() != tokens.numel():
                raise ValueError(f"'{key}' must be a 1-D tensor with one entry per token")
        float(sample["advantages"])


def even_slice(total_sample: int, total_slice: int) -> List[int]:
    """Boundaries of ``total_slice`` nearly equal consecutive slices; the first ``remainder`` slices
    are one longer (utils/utils.py:320-327)."""
    size, rem = divmod(total_sample, total_slice)
    return [i * size + min(i, rem) for i in range(total_slice)] + [total_sample]


def slice_data_list_by_index(batched_input: List[Any], index) -> List[Any]:
    """``index = (slice_id, total_slice)`` (utils/utils.py:329-338)."""
    bounds = even_slice(len(batched_input), index[1])
    return batched_input[bounds[index[0]]: bounds[index[0] + 1]]


def minibatch_slice_index(total_samples: int, dp_size: int, num_minibsz: int) -> List[int]:
    """Boundaries of the batches a fixed-size stream dataset yields: slice over the data-parallel
    ranks first, then every rank's share into ``num_minibsz`` mini-batches (data/data.py:160-167)."""
    dp = even_slice(total_samples, dp_size)
    out = [start + s for start, end in zip(dp[:-1], dp[1:]) for s in even_slice(end - start, num_minibsz)[:-1]]
    return out + [total_samples]


def iter_fixed_order(samples: List[Any], dp_size: int, num_minibsz: int) -> Iterator[List[Any]]:
    """The batches in the order ``StreamDataset.iter_fixed`` yields them (data/data.py:169-173)."""
    bounds = minibatch_slice_index(len(samples), dp_size, num_minibsz)
    for lo, hi in zip(bounds[:-1], bounds[1:]):
        yield samples[lo:hi]
