"""Mirror of chatlearn/algorithm/grpo_utils/advantage_compute.py.

The per-prompt reward pools stay in a host dict keyed by ``prompt_uid`` (they
carry over between calls until a group is complete, as in the reference); the
arithmetic - mean, population std, (r - mean) / (std + 1e-5), all-zero /
all-one flags - runs in one HIP launch over all samples, in float64.
"""
from collections import defaultdict
from typing import Any, Dict, List

import numpy as np
import torch

from ... import ops


def _mean_per_key(metric_list):
    # reference: chatlearn/utils/utils.py:364-405 (map, then numpy mean per key)
    if len(metric_list) == 0:
        return {}
    cols = {}
    for m in metric_list:
        for k, v in m.items():
            cols.setdefault(k, []).append(v)
    return {k: np.mean(v) for k, v in cols.items()}


class AdvantageComputer:
    """advantage computer"""
    def __init__(self, num_inference_per_prompt, device=None):
        self._metric_prefix = 'advantage_compute'
        self._metric_list = []
        self.rule_reward_buffer = defaultdict(list)
        self.num_inference_per_prompt = num_inference_per_prompt
        self._device = device

    def __call__(self, episode_replay_buffers: List[Dict[str, Any]]):
        buffers = episode_replay_buffers[-1].buffer
        for s in buffers:
            self.rule_reward_buffer[s['prompt_uid']].append(s["rule_reward"])
        if len(buffers) == 0:
            # the reference divides by len(...) == 0 here
            raise ZeroDivisionError("division by zero")

        # group index per sample, pools laid out group after group
        group_index = {}
        offsets = [0]
        pool = []
        for s in buffers:
            uid = s['prompt_uid']
            if uid not in group_index:
                group_index[uid] = len(group_index)
                pool.extend(float(x) for x in self.rule_reward_buffer[uid])
                offsets.append(len(pool))
        dev = self._device or torch.device("cuda", torch.cuda.current_device())
        rewards = torch.tensor([float(s["rule_reward"]) for s in buffers], dtype=torch.float64).to(dev)
        group_of = torch.tensor([group_index[s['prompt_uid']] for s in buffers], dtype=torch.int32).to(dev)
        adv, all_zero, all_one = ops.group_advantage(
            rewards, group_of, torch.tensor(pool, dtype=torch.float64).to(dev),
            torch.tensor(offsets, dtype=torch.int32).to(dev), eps=1e-5)
        adv = adv.cpu().numpy()
        all_wrong_list = all_zero.cpu().tolist()
        all_correct_list = all_one.cpu().tolist()
        for s, a in zip(buffers, adv):
            s['advantages'] = a  # numpy.float64, as in the reference

        self.rule_reward_buffer = defaultdict(
            list, {k: v for k, v in self.rule_reward_buffer.items() if len(v) < self.num_inference_per_prompt})
        all_correct_ratio = sum(all_correct_list) / len(all_correct_list)
        all_wrong_ratio = sum(all_wrong_list) / len(all_wrong_list)
        self._metric_list.append({"all_correct_ratio": all_correct_ratio, "all_wrong_ratio": all_wrong_ratio})
        return buffers

    def get_and_clear_metrics(self):
        if self._metric_list is None or len(self._metric_list) == 0:
            return self._metric_prefix, {}
        reduced_metrics = _mean_per_key(self._metric_list)
        self._metric_list = []
        return self._metric_prefix, reduced_metrics
