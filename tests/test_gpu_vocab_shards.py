"""Vocabulary-sharded head: per-shard records merged on the device must equal the unsharded
kernels and the oracle's restatement of the reference's three all-reduces; the sharded backward
must add up to the unsharded one."""
import pytest
import torch

from oracle import softmax_stats as osm
from oracle import vocab_parallel as ovp
from tests.util import assert_close_rel

pytestmark = pytest.mark.gpu


def _inputs(T, H, V, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    hidden = torch.randn(T, H, generator=g).to(dtype)
    weight = (torch.randn(V, H, generator=g) * 0.05).to(dtype)
    labels = torch.randint(0, V, (T,), generator=g)
    labels[0], labels[-1] = 0, V - 1
    return hidden, weight, labels


@pytest.mark.parametrize("T,H,V,n,dtype,temp", [
    (300, 256, 6000, 4, torch.float32, 1.0),
    (513, 128, 4096, 8, torch.bfloat16, 0.7),
    (700, 512, 9000, 3, torch.bfloat16, 1.0),
    (64, 64, 512, 2, torch.bfloat16, 1.0),
])
def test_sharded_forward_equals_unsharded_and_oracle(dev, T, H, V, n, dtype, temp):
    from chatlearn_amd import ops
    hidden, weight, labels = _inputs(T, H, V, dtype, seed=T + V)
    hd, wd, ld = hidden.to(dev), weight.to(dev), labels.to(dev)
    ranges = ovp.shard_ranges(V, n)
    records = torch.stack([ops.lmhead_forward_shard(hd, wd[lo:hi].contiguous(), ld, lo, temp) for lo, hi in ranges])
    lp, ent, mx, lse = ops.lmhead_merge_shards(records, ld, V, temp)
    # against the unsharded kernels (same arithmetic, different merge order)
    lp0, ent0, mx0, lse0 = ops.lmhead_forward(hd, wd, ld, temp)
    assert torch.equal(mx, mx0)
    for a, b, name in ((lp, lp0, "logprob"), (ent, ent0, "entropy"), (lse, lse0, "lse")):
        assert (a - b).abs().max().item() < 2e-5 * max(1.0, b.abs().max().item()), name
    # against the reference's reductions over the ranks, on the same bf16/fp32 operands in float64
    z = torch.nn.functional.linear(hidden.double(), weight.double()) / temp
    shards = [z[:, lo:hi] for lo, hi in ranges]
    r = 1e-5 if dtype == torch.float32 else 1e-2
    assert_close_rel(lp, ovp.vocab_parallel_logprob(shards, labels, ranges), r, "logprob vs vocab-parallel CE")
    assert_close_rel(ent, ovp.vocab_parallel_entropy(shards), r, "entropy vs _VocabParallelEntropy")
    # each record's last field is the target logit on the owning shard and zero elsewhere
    owner = labels // (V // n)
    zt = records[:, :, 3].cpu()
    for s in range(n):
        assert (zt[s][owner != s] == 0).all()
        assert (zt[s][owner == s] != 0).any() or (owner == s).sum() == 0


@pytest.mark.parametrize("with_saved", [False, True], ids=["recompute", "kept-logits"])
@pytest.mark.parametrize("T,H,V,n,dtype", [(300, 256, 6000, 4, torch.float32), (513, 128, 4096, 2, torch.bfloat16)])
def test_sharded_backward_adds_up(dev, T, H, V, n, dtype, with_saved):
    from chatlearn_amd import ops
    hidden, weight, labels = _inputs(T, H, V, dtype, seed=T + V + 7)
    g = torch.Generator().manual_seed(3)
    g_lp = torch.randn(T, generator=g)
    g_lp[torch.rand(T, generator=g) < 0.3] = 0.0
    g_ent = torch.randn(T, generator=g) * 0.1
    hd, wd, ld = hidden.to(dev), weight.to(dev), labels.to(dev)
    lp, ent, _, lse = ops.lmhead_forward(hd, wd, ld, 0.9)
    dh_sum = torch.zeros(T, H, dtype=torch.float32, device=dev)
    dw_rows = []
    for lo, hi in ovp.shard_ranges(V, n):
        ws = wd[lo:hi].contiguous()
        zbuf = None
        if with_saved:
            zbuf = ops.saved_logits_buffer(T, hi - lo, dtype, dev)
            ops.lmhead_forward_shard(hd, ws, ld, lo, 0.9, saved_logits=zbuf)
        dh, dw = ops.lmhead_backward(hd, ws, ld, lse, ent, g_lp.to(dev), g_ent.to(dev), 0.9, saved_logits=zbuf,
                                     vocab_begin=lo)
        dh_sum += dh.float()                                                            # the caller's all-reduce
        dw_rows.append(dw)
    rdh, rdw = osm.fused_head_backward_closed_form(hidden, weight, labels, g_lp, g_ent, 0.9)
    r = 1e-5 if dtype == torch.float32 else 1e-2
    assert_close_rel(dh_sum, rdh, r, "sum of shard dhidden")
    assert_close_rel(torch.cat(dw_rows), rdw, r, "concatenated shard dW")


def test_shard_entry_points_validate(dev):
    from chatlearn_amd import ops
    from chatlearn_amd._lib import ClgrpoError
    hidden, weight, labels = _inputs(64, 64, 512, torch.bfloat16, 1)
    with pytest.raises(ClgrpoError):
        ops.lmhead_forward_shard(hidden.to(dev), weight.to(dev), labels.to(dev), -5)
    with pytest.raises(ValueError):
        ops.lmhead_merge_shards(torch.zeros(2, 64, 3, device=dev), labels.to(dev), 512)
