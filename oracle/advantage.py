"""Oracle: group-wise reward -> advantage normalisation.

Test infrastructure only; never imported by the product package.

Reference semantics restated here:
  * AdvantageComputer.__call__ / metrics     advantage_compute.py:10-52
  * map_reduce_metrics (mean per key)        chatlearn/utils/utils.py:364-405
"""
from collections import defaultdict

import numpy as np


class _Buffer:
    """Stand-in for the replay-buffer object whose ``.buffer`` is the sample list
    (chatlearn/data/data.py:227 hands over a list of them)."""
    def __init__(self, samples):
        self.buffer = samples


def map_reduce_metrics(metric_list):
    if len(metric_list) == 0:
        return {}
    cols = {}
    for m in metric_list:
        for k, v in m.items():
            cols.setdefault(k, []).append(v)
    return {k: np.mean(v) for k, v in cols.items()}


class AdvantageComputer:
    """advantage_compute.py:10-52: population std (ddof=0) in float64, eps 1e-5;
    rewards of unfinished groups stay buffered between calls."""

    def __init__(self, num_inference_per_prompt):
        self._metric_prefix = "advantage_compute"
        self._metric_list = []
        self.rule_reward_buffer = defaultdict(list)
        self.num_inference_per_prompt = num_inference_per_prompt

    def __call__(self, episode_replay_buffers):
        samples = episode_replay_buffers[-1].buffer
        for s in samples:
            self.rule_reward_buffer[s["prompt_uid"]].append(s["rule_reward"])
        all_ones, all_zeros = [], []
        for s in samples:
            pool = self.rule_reward_buffer[s["prompt_uid"]]
            all_zeros.append(all(x == 0 for x in pool))
            all_ones.append(all(x == 1 for x in pool))
            s["advantages"] = (s["rule_reward"] - np.mean(pool)) / (np.std(pool) + 1e-5)
        self.rule_reward_buffer = defaultdict(
            list, {k: v for k, v in self.rule_reward_buffer.items()
                   if len(v) < self.num_inference_per_prompt})
        self._metric_list.append({"all_correct_ratio": sum(all_ones) / len(all_ones),
                                  "all_wrong_ratio": sum(all_zeros) / len(all_zeros)})
        return samples

    def get_and_clear_metrics(self):
        if not self._metric_list:
            return self._metric_prefix, {}
        red = map_reduce_metrics(self._metric_list)
        self._metric_list = []
        return self._metric_prefix, red
