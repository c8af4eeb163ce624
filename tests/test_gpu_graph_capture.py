"""The head path under HIP graph capture: forward with kept logits -> sequence-level loss with upstream
gradients -> backward, recorded once into a graph and replayed on fresh inputs.  The library issues
only kernel launches on the caller's stream (no allocation, memset or synchronisation of its own), so
the whole sequence is capturable; every replay must give the bits of an eager run on the same inputs.
Replays are separated by eager work and synchronisations of the test's own."""
import pytest
import torch

from chatlearn_amd import ops
from chatlearn_amd._lib import LOSS_GSPO

pytestmark = pytest.mark.gpu

T, H, V, B = 777, 256, 3001, 9


def _fresh(seed, dev):
    g = torch.Generator().manual_seed(seed)
    cuts = torch.sort(torch.randperm(T - 1, generator=g)[:B - 1] + 1).values
    cu = torch.cat([torch.zeros(1, dtype=torch.long), cuts, torch.tensor([T])]).to(torch.int32)
    x = {"hidden": (torch.randn(T, H, generator=g) * 0.7).to(torch.bfloat16),
         "weight": (torch.randn(V, H, generator=g) * 0.05).to(torch.bfloat16),
         "labels": torch.randint(0, V, (T,), generator=g),
         "noise": torch.randn(T, generator=g) * 1e-3,
         "adv": torch.randn(B, generator=g),
         "mask": (torch.rand(T, generator=g) < 0.8).int(),
         "cu": cu}
    return {k: v.to(dev).contiguous() for k, v in x.items()}


def _head(x, saved, dweight):
    lp, ent, _, lse = ops.lmhead_forward(x["hidden"], x["weight"], x["labels"], saved_logits=saved)
    old = lp + x["noise"]                      # behaviour policy close to the current one: both clip branches occur
    r = ops.policy_loss(lp, old, x["adv"], mode=LOSS_GSPO, cu_seqlens=x["cu"],
                        entropy=ent, loss_mask=x["mask"], pos_clip_ratio=4e-4, neg_clip_ratio=3e-4, entropy_coef=1e-3,
                        grad_scale=1.0 / T, want_upstream=True)
    dh, dw = ops.lmhead_backward(x["hidden"], x["weight"], x["labels"], lse, ent, r.g_logprob, r.g_entropy,
                                 dweight=dweight, accumulate_dweight=False, saved_logits=saved)
    return {"logprob": lp, "entropy": ent, "loss": r.loss, "sums": r.sums, "flags": r.flags, "dhidden": dh, "dweight": dw}


def test_head_path_replayed_from_a_graph_matches_eager_bit_for_bit(dev):
    static = _fresh(0, dev)
    saved = ops.saved_logits_buffer(T, V, torch.bfloat16, dev)
    dweight = torch.empty(V, H, dtype=torch.float32, device=dev)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        _head(static, saved, dweight)          # warm-up outside the capture: kernel attributes, allocator pools
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = _head(static, saved, dweight)
    torch.cuda.synchronize()

    for seed in (1, 2, 3):
        x = _fresh(seed, dev)
        for k in static:
            static[k].copy_(x[k])
        graph.replay()
        torch.cuda.synchronize()
        got = {k: v.clone() for k, v in out.items()}
        # eager work of the test's own between the replays, on the same inputs
        want = _head(x, ops.saved_logits_buffer(T, V, torch.bfloat16, dev), torch.empty(V, H, dtype=torch.float32, device=dev))
        torch.cuda.synchronize()
        for k in want:
            assert torch.equal(got[k], want[k]), f"replay with seed {seed}: {k} differs from the eager run"
        assert torch.isfinite(got["dweight"]).all() and float(got["dweight"].abs().sum()) > 0
