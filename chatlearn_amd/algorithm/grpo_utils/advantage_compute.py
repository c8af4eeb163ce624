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
        for s, a in zip(buffers, adv):
            s['advantages'] = a  # numpy.float64, as in the reference

        # groups that have all their responses are dropped from the pool (advantage_compute.py:40-41)
        kept = {uid: pool_ for uid, pool_ in self.rule_reward_buffer.items() if len(pool_) < self.num_inference_per_prompt}
        self.rule_reward_buffer = defaultdict(list, kept)
        n = float(len(buffers))
        self._metric_list.append({"all_correct_ratio": int(all_one.sum().item()) / n,
                                  "all_wrong_ratio": int(all_zero.sum().item()) / n})
        return buffers

    def get_and_clear_metrics(self):
        pending, self._metric_list = (self._metric_list or []), []
        return self._metric_prefix, (_mean_per_key(pending) if pending else {})
