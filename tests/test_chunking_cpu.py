"""Token chunking of a micro-batch (host logic of grpo_head_step)."""
import random

from chatlearn_amd.fused import _token_chunks


def test_hand_worked_chunks():
    assert _token_chunks(16384, 16384, None) == [(0, 16384)]
    assert _token_chunks(16384, None, None) == [(0, 16384)]
    assert _token_chunks(20000, 16384, None) == [(0, 10000), (10000, 20000)]              # two equal ranges, not 16384 + 3616
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
