"""Bin packing: oracle and the library's host routines against hand-worked cases
(tests/golden/packing_cases.json), invariants, and each other on random inputs.
Integer results: every comparison is exact."""
import json
import os
import random
import warnings

import pytest

from oracle import packing as opk

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "packing_cases.json")) as f:
    GOLD = json.load(f)


@pytest.mark.parametrize("case", GOLD["bin_packing"], ids=lambda c: c["pins"][:40])
def test_oracle_bin_packing_golden(case):
    with warnings.catch_warnings(record=True) as w:
        warnings.simplefilter("always")
        ids, lens = opk.bin_packing(case["seq_len"], case["cap"])
    assert ids == case["ids"] and lens == case["lens"]
    assert bool(w) == bool(case.get("warns", False))


@pytest.mark.parametrize("case", GOLD["bin_packing_fix_bin"], ids=lambda c: c["pins"][:40])
def test_oracle_fix_bin_golden(case):
    ids, lens = opk.bin_packing_fix_bin(case["seq_len"], case["bins"])
    assert [list(b) for b in ids] == case["ids"] and [list(b) for b in lens] == case["lens"]


@pytest.mark.parametrize("case", GOLD["bin_packing"], ids=lambda c: c["pins"][:40])
def test_library_bin_packing_golden(lib, case):
    from chatlearn_amd.algorithm.grpo_utils import packing_utils as pk
    with warnings.catch_warnings(record=True) as w:
        warnings.simplefilter("always")
        ids, lens = pk.bin_packing(case["seq_len"], case["cap"])
    assert ids == case["ids"] and lens == case["lens"]
    assert bool(w) == bool(case.get("warns", False))


@pytest.mark.parametrize("case", GOLD["bin_packing_fix_bin"], ids=lambda c: c["pins"][:40])
def test_library_fix_bin_golden(lib, case):
    from chatlearn_amd.algorithm.grpo_utils import packing_utils as pk
    ids, lens = pk.bin_packing_fix_bin(case["seq_len"], case["bins"])
    assert ids == case["ids"] and lens == case["lens"]


def _random_lengths(rng, n, lo, hi, dup=False):
    vals = [rng.randint(lo, hi) for _ in range(n)]
    if dup and n > 3:
        for _ in range(n // 3):
            vals[rng.randrange(n)] = vals[rng.randrange(n)]
    return vals


@pytest.mark.parametrize("seed", range(6))
def test_library_matches_oracle_random(lib, seed):
    from chatlearn_amd.algorithm.grpo_utils import packing_utils as pk
    rng = random.Random(seed)
    n = rng.choice([1, 7, 64, 300, 512])
    lens = _random_lengths(rng, n, 1, 2048, dup=True)
    cap = rng.choice([2048, 4096, 16384])
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        assert pk.bin_packing(lens, cap) == opk.bin_packing(lens, cap)
    k = max(1, len(opk.bin_packing(lens, cap)[0]))
    a_ids, a_lens = pk.bin_packing_fix_bin(lens, k)
    b_ids, b_lens = opk.bin_packing_fix_bin(lens, k)
    assert a_ids == [list(x) for x in b_ids] and a_lens == [list(x) for x in b_lens]


@pytest.mark.parametrize("seed", range(4))
def test_packing_invariants(seed):
    rng = random.Random(100 + seed)
    lens = _random_lengths(rng, 200, 10, 1000)
    cap = 4096
    ids, blens = opk.bin_packing(lens, cap)
    flat = sorted(i for b in ids for i in b)
    assert flat == list(range(len(lens)))                    # every item exactly once
    assert all(sum(b) < cap for b in blens)                   # strict rule: a bin never reaches the cap
    assert all([lens[i] for i in b] == l for b, l in zip(ids, blens))
    k = len(ids)
    fids, flens = opk.bin_packing_fix_bin(lens, k)
    assert len(fids) == k and sorted(i for b in fids for i in b) == list(range(len(lens)))
    sums = [sum(lens[i] for i in b) for b in fids]
    assert sums == sorted(sums, reverse=True)
    assert max(sums) - min(sums) <= max(lens)                 # longest-first greedy balance bound
    assert opk.bin_packing(lens, cap) == (ids, blens)          # deterministic


def test_regroup_and_split_microbatch_match_oracle(lib):
    import copy
    from chatlearn_amd.algorithm.grpo_utils import trainer_utils as tu
    rng = random.Random(7)
    data = [{"prompt_token_length": rng.randint(10, 200), "response_token_length": rng.randint(10, 900), "k": i}
            for i in range(97)]
    a = tu.split_microbatch(copy.deepcopy(data), max_train_token=2048, packing=True, offset=5)
    b = opk.split_microbatch(copy.deepcopy(data), max_train_token=2048, packing=True, offset=5)
    assert a == b
    assert all(s["id_in_list"] == s["k"] + 5 for mb in a for s in mb)
    a = tu.split_microbatch(copy.deepcopy(data), micro_batch_size=8)
    b = opk.split_microbatch(copy.deepcopy(data), micro_batch_size=8)
    assert a == b and len(a) == 13 and len(a[-1]) == 1
    with pytest.raises(AssertionError):
        tu.split_microbatch(data)


def test_batching_matches_oracle():
    import torch
    from chatlearn_amd.algorithm.grpo_utils import trainer_utils as tu
    g = torch.Generator().manual_seed(0)
    data = [{"all_tokens": torch.randint(0, 100, (n,), generator=g), "old_logprobs": torch.randn(n, generator=g),
             "advantages": float(n), "prompt_token_length": n // 2} for n in (5, 9, 3)]
    a, b = tu.batching(data), opk.batching(data)
    assert a.keys() == b.keys()
    for k in a:
        if isinstance(a[k], torch.Tensor):
            assert a[k].shape == (3, 9) and torch.equal(a[k], b[k])
            assert (a[k][0, 5:] == 0).all()
        else:
            assert a[k] == b[k]
    assert tu.batching([]) is None
