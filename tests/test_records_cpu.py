"""Record formats and batch order (host logic) against hand-worked cases."""
import json
import os

import pytest
import torch

from chatlearn_amd import records

with open(os.path.join(os.path.dirname(__file__), "golden", "batch_order_cases.json")) as _f:
    GOLD = json.load(_f)


def test_even_slice_and_minibatch_order():
    for c in GOLD["even_slice"]:
        assert records.even_slice(c["n"], c["k"]) == c["want"]
    for c in GOLD["minibatch"]:
        assert records.minibatch_slice_index(c["n"], c["dp"], c["mb"]) == c["want"]
    samples = list(range(10))
    assert list(records.iter_fixed_order(samples, 2, 2)) == [[0, 1, 2], [3, 4], [5, 6, 7], [8, 9]]
    assert records.slice_data_list_by_index(samples, (1, 3)) == [4, 5, 6]
    # every sample lands in exactly one batch, in order
    for n, dp, mb in ((23, 3, 4), (5, 8, 2), (64, 8, 8)):
        flat = [x for b in records.iter_fixed_order(list(range(n)), dp, mb) for x in b]
        assert flat == list(range(n))


def test_rollout_record_and_validation():
    prompt = {"prompt_uid": "u1", "data_source": "openai/gsm8k", "ground_truth": "42", "rollout_round": 0}
    rec = records.rollout_record(prompt, [5, 6, 7], [8, 9], "ok")
    assert rec["all_tokens"].tolist() == [5, 6, 7, 8, 9]
    assert (rec["prompt_token_length"], rec["response_token_length"], rec["rollout_round"]) == (3, 2, 1)
    assert prompt["rollout_round"] == 0 and rec["prompt_uid"] == "u1"          # the prompt dict is copied
    records.check_train_record(rec, training=False)
    with pytest.raises(ValueError, match="old_logprobs"):
        records.check_train_record(rec, training=True)
    rec.update({"old_logprobs": torch.zeros(5), "ref_logprobs": torch.zeros(5), "advantages": 0.25})
    records.check_train_record(rec, training=True)
    rec["response_token_length"] = 3
    with pytest.raises(ValueError, match="all_tokens has 5"):
        records.check_train_record(rec)
    agent = records.rollout_record({}, [1, 2], [3, 4, 5], loss_mask=[0, 0, 1, 0, 1])
    assert agent["all_token_length"] == 5 and agent["loss_mask"].tolist() == [0, 0, 1, 0, 1]
    agent["loss_mask"] = torch.tensor([1, 1])
    with pytest.raises(ValueError, match="loss_mask"):
        records.check_train_record(agent, training=False)
