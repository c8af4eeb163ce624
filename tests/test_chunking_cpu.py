"""Token chunking of a micro-batch (host logic of grpo_head_step)."""
import random

import numpy as np
import torch

from chatlearn_amd.fused import _token_chunks


def test_hand_worked_chunks():
    assert _token_chunks(16384, 16384, None) == [(0, 16384)]
    assert _token_chunks(16384, None, None) == [(0, 16384)]
    assert _token_chunks(20000, 16384, None) == [(0, 9984), (9984, 20000)]                # two about equal ranges cut on a multiple of 256, not 16384 + 3616
    assert _token_chunks(100, 30, None) == [(0, 25), (25, 50), (50, 75), (75, 100)]
    bounds = [0, 4000, 9000, 11000, 15169, 20000, 22000, 29588, 32768]
    assert _token_chunks(32768, 16384, bounds) == [(0, 11000), (11000, 22000), (22000, 32768)]
    # sequences longer than the cap get a range of their own
    assert _token_chunks(1000, 300, [0, 100, 500, 520, 1000]) == [(0, 100), (100, 500), (500, 520), (520, 1000)]


def test_chunk_properties_on_random_layouts():
    rng = random.Random(1)
    for _ in range(3000):
        T = rng.randint(1, 5000)
        cap = rng.randint(1, 3000)
        bounds = sorted({0, T} | {rng.randint(1, T) for _ in range(rng.randint(1, 40))}) if rng.random() < 0.7 else None
        ranges = _token_chunks(T, cap, bounds)
        assert ranges[0][0] == 0 and ranges[-1][1] == T
        assert all(a[1] == b[0] for a, b in zip(ranges, ranges[1:])) and all(hi > lo for lo, hi in ranges)
        if bounds is None:
            assert all(hi - lo <= cap for lo, hi in ranges)
            assert len(ranges) == -(-T // cap)                                             # as few as the cap allows
        else:
            assert all(hi in bounds for _, hi in ranges)
            for lo, hi in ranges:
                if hi - lo > cap:
                    assert not any(lo < x < hi for x in bounds)                            # a single long sequence


def test_chunks_bounded_by_kept_rows():
    """With the unmasked rows counted (only they keep logits) the bound is on those: fewer, longer token
    ranges; tokens or sequences without a kept row never open a range of their own."""
    live = np.array([1, 1, 0, 0, 1, 0, 1, 1, 0, 0, 0, 0])
    cum = np.concatenate([[0], np.cumsum(live)])
    assert _token_chunks(12, 3, None, cum) == [(0, 6), (6, 12)]                            # 3 + 2 kept rows, the masked tail rides along
    assert _token_chunks(12, 5, None, cum) == [(0, 12)]
    assert _token_chunks(12, 2, [0, 2, 4, 8, 12], cum) == [(0, 4), (4, 12)]                # sequence [2, 4) has no kept row
    rng = random.Random(2)
    for _ in range(2000):
        T = rng.randint(1, 4000)
        keep_p = rng.choice([0.05, 0.5, 0.75, 1.0])
        live = np.array([1 if rng.random() < keep_p else 0 for _ in range(T)])
        if rng.random() < 0.3:
            live[rng.randint(0, T - 1):] = 0                                               # masked tail
        cum = np.concatenate([[0], np.cumsum(live)])
        cap = rng.randint(1, 2500)
        bounds = sorted({0, T} | {rng.randint(1, T) for _ in range(rng.randint(1, 30))}) if rng.random() < 0.5 else None
        ranges = _token_chunks(T, cap, bounds, cum)
        assert ranges[0][0] == 0 and ranges[-1][1] == T
        assert all(a[1] == b[0] for a, b in zip(ranges, ranges[1:])) and all(hi > lo for lo, hi in ranges)
        rows = [int(cum[hi] - cum[lo]) for lo, hi in ranges]
        if bounds is None:
            assert all(r <= cap for r in rows)
            assert len(ranges) == max(1, -(-int(cum[T]) // cap))                           # as few as the cap allows
        else:
            assert all(hi in bounds for _, hi in ranges)
            for (lo, hi), r in zip(ranges, rows):
                if r > cap:
                    assert not any(lo < x < hi and cum[lo] < cum[x] < cum[hi] for x in bounds)
        if len(ranges) > 1:
            assert rows[-1] > 0 or bounds is not None                                      # no range for a tail without kept rows


def test_asked_number_of_ranges_and_launch_cost_choice():
    from chatlearn_amd.fused import _launch_cost, head_step_chunks
    # more ranges than the fewest: still a partition, still within the bound
    assert _token_chunks(1000, 600, None, None, n_ranges=4) == [(0, 256), (256, 512), (512, 768), (768, 1000)]
    assert len(_token_chunks(1000, 600, None, None, n_ranges=1)) == 2                      # never fewer than the bound needs
    rng = random.Random(3)
    for _ in range(500):
        T = rng.randint(10, 6000)
        cap = rng.randint(5, 3000)
        bounds = sorted({0, T} | {rng.randint(1, T) for _ in range(rng.randint(1, 30))}) if rng.random() < 0.5 else None
        fewest = _token_chunks(T, cap, bounds)
        for extra in (1, 2):
            r = _token_chunks(T, cap, bounds, None, n_ranges=len(fewest) + extra)
            assert r[0][0] == 0 and r[-1][1] == T and all(a[1] == b[0] for a, b in zip(r, r[1:]))
            assert all(hi > lo for lo, hi in r) and len(r) >= len(fewest)
            if bounds is None:
                assert all(hi - lo <= cap for lo, hi in r)
    H, V = 2048, 151936
    one, more = _launch_cost([(0, 16384)], None, H, V), _launch_cost([(0, 16640)], None, H, V)
    assert one < more < 1.1 * one                                                          # one more token block costs about 1/64 more, not a second round
    # a sequence-level micro-batch of 32768 tokens: the bound of 17408 rows allows two ranges; the choice
    # never takes more than two extra and every range ends on a sequence boundary
    cu = [0, 5000, 9000, 16000, 21000, 26000, 30000, 32768]
    import torch
    mask = torch.ones(32768, dtype=torch.int32)
    ranges = head_step_chunks(32768, 17408, True, cu, mask, shape=(H, V))
    assert 2 <= len(ranges) <= 4 and all(hi in cu for _, hi in ranges)
    assert ranges[0][0] == 0 and ranges[-1][1] == 32768
    # everything fits one range: one range, whatever the shape
    assert head_step_chunks(16384, 17408, False, None, None, shape=(4096, V)) == [(0, 16384)]


def test_library_launch_plans():
    """The forward picks its vocabulary splits so that the launch fills whole rounds of one workgroup per CU;
    the dhidden GEMM cuts its rows into a bulk launch of whole rounds before it cuts K.  594 vocabulary
    tiles (V = 151936), 256 CUs."""
    from chatlearn_amd import ops
    V = 151936
    assert ops.lmhead_forward_launch_plan(16384, V) == (64, 4, 149)                        # 64 blocks x 4 splits = 256 workgroups
    assert ops.lmhead_forward_launch_plan(8192, V) == (32, 8, 75)
    assert ops.lmhead_forward_launch_plan(16640, V) == (65, 35, 17)                        # 65 blocks: 2275 workgroups, 9 rounds of 17 tiles = 153 periods (ideal 151)
    for T in (1792, 5000, 12126, 17599, 20000, 33000, 65536, 100000):
        n_tb, sp, tps = ops.lmhead_forward_launch_plan(T, V)
        assert n_tb == -(-T // 256) and 1 <= sp <= 64 and sp * tps >= 594                  # every vocabulary tile is covered
        cost = -(-(n_tb * -(-594 // tps)) // 256) * tps
        assert cost <= 1.08 * n_tb * 594 / 256                                             # near the ideal n_tb * 594 / 256 tile periods
    assert ops.lmhead_forward_launch_plan(16640, V, cus=304) != ops.lmhead_forward_launch_plan(16640, V)
    # dhidden, H = 4096 (16 output tiles per 256 rows): 48 row tiles fill 3 rounds exactly; 50 row tiles run as
    # 48 without a K split plus 2 x 16 tiles cut into 8 K ranges
    assert ops.dhidden_launch_plan(12126, 4096, V, torch.bfloat16) == (0, 1)
    assert ops.dhidden_launch_plan(12700, 4096, V, torch.bfloat16) == (48, 8)
    assert ops.dhidden_launch_plan(1458, 1024, V, torch.float32) == (0, 10)                # 24 tiles: 10 K ranges fill 240 CUs
    # dW, H = 4096: 16 walks over 594 vocabulary tiles would be runs of 37 and 38; 592 tiles are walked in runs of 37
    # and the last 2 x 16 tiles are cut into 8 K ranges (256 work items).  Few tiles: one workgroup per tile, no walks
    assert ops.dweight_launch_plan(12126, 4096, V, torch.bfloat16) == (16, 592, 8)
    assert ops.dweight_launch_plan(5000, 4096, 32000, torch.bfloat16) == (16, 0, 1)        # 125 tiles, runs of 7 and 8: the 13 left-over tile rows would fill most CUs anyway
    assert ops.dweight_launch_plan(700, 512, 9001, torch.bfloat16) == (0, 0, 1)
    for rows, H, vocab in [(32767, 2048, V), (16384, 7168, 129280), (1457, 1024, V), (300, 4096, V), (65536, 4096, V)]:
        n_walk, bulk, ks = ops.dweight_launch_plan(rows, H, vocab, torch.bfloat16)
        n_mt = -(-vocab // 256)
        assert 0 <= bulk < n_mt and 1 <= ks <= 16
        if bulk:
            assert n_walk > 0 and bulk % n_walk == 0 and n_mt - bulk < n_walk              # equal runs, fewer tiles left than walks


def test_chunk_choice_on_random_layouts_is_always_a_partition():
    """head_step_chunks with the launch-cost choice switched on: whatever it picks is a partition into ranges
    within the bound (or single longer sequences), ending on sequence boundaries when asked to."""
    from chatlearn_amd.fused import head_step_chunks
    rng = random.Random(5)
    for _ in range(300):
        T = rng.randint(1, 40000)
        cap = rng.choice([256, 1000, 4096, 8192, 17408])
        seq = rng.random() < 0.5
        cu = sorted({0, T} | {rng.randint(1, T) for _ in range(rng.randint(0, 12))})
        mask = None
        if rng.random() < 0.6:
            mask = (torch.rand(T, generator=torch.Generator().manual_seed(rng.randint(0, 1 << 30))) < rng.choice([0.1, 0.7, 1.0])).int()
        ranges = head_step_chunks(T, cap, seq, cu, mask, shape=(rng.choice([1024, 2048, 4096, 7168]), rng.choice([32000, 129280, 151936])),
                                  chunk_hidden_bytes=rng.choice([None, 64 << 20, 256 << 20]))
        assert ranges[0][0] == 0 and ranges[-1][1] == T
        assert all(a[1] == b[0] for a, b in zip(ranges, ranges[1:])) and all(hi > lo for lo, hi in ranges)
        cum = None if mask is None else np.concatenate([[0], np.cumsum(mask.numpy() != 0)])
        for lo, hi in ranges:
            rows = (hi - lo) if cum is None else int(cum[hi] - cum[lo])
            if seq and len(ranges) > 1:
                assert hi in cu
                if rows > cap:
                    assert not any(lo < x < hi and (cum is None or cum[lo] < cum[x] < cum[hi]) for x in cu)
            elif not seq:
                assert rows <= cap


def test_bound_on_a_chunk_s_hidden_states():
    """Besides the bound on the kept rows, a chunk's hidden states stay below ``chunk_hidden_bytes`` when one is given: 32768 tokens
    at H = 7168 (448 MiB in 16-bit elements) are cut in two although every row's logits would fit one chunk,
    at H = 2048 (128 MiB) they are one chunk; fp32 counts 4 bytes per element; sequence-level ranges still end
    on sequence boundaries; without a shape or a bound nothing is cut."""
    from chatlearn_amd.fused import default_keep_rows, head_step_chunks
    CHUNK_HIDDEN_BYTES = 256 << 20
    keep = default_keep_rows(129280, torch.bfloat16)
    assert keep >= 32768
    assert head_step_chunks(32768, keep, False, None, None, shape=(7168, 129280), chunk_hidden_bytes=CHUNK_HIDDEN_BYTES) == \
        [(0, 16384), (16384, 32768)]
    assert head_step_chunks(32768, keep, False, None, None, shape=(7168, 129280)) == [(0, 32768)]
    assert head_step_chunks(32768, keep, False, None, None, shape=None, chunk_hidden_bytes=CHUNK_HIDDEN_BYTES) == [(0, 32768)]
    assert head_step_chunks(32768, default_keep_rows(151936, torch.bfloat16), False, None, None, shape=(2048, 151936),
                            chunk_hidden_bytes=CHUNK_HIDDEN_BYTES) == [(0, 32768)]
    assert len(head_step_chunks(32768, 1 << 20, False, None, None, shape=(4096, 32000), dtype=torch.float32,
                                chunk_hidden_bytes=CHUNK_HIDDEN_BYTES)) == 2
    cu = [0, 5000, 9000, 15000, 21000, 26000, 30000, 32768]
    mask = (torch.arange(32768) % 4 != 0).int()
    ranges = head_step_chunks(32768, keep, True, cu, mask, shape=(7168, 129280), chunk_hidden_bytes=CHUNK_HIDDEN_BYTES)
    assert len(ranges) >= 2 and ranges[0][0] == 0 and ranges[-1][1] == 32768 and all(hi in cu for _, hi in ranges)
    assert all(a[1] == b[0] for a, b in zip(ranges, ranges[1:]))
