"""Megatron-side loss helpers (tp = cp = 1) against the oracle."""
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from oracle import indexing as oi
from oracle import losses as ol
from oracle import softmax_stats as osm
from tests.util import assert_close_rel

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("packing", [False, True])
@pytest.mark.parametrize("gspo", [False, True])
def test_compute_all_losses_and_loss_func(dev, packing, gspo):
    from chatlearn_amd.algorithm.grpo_utils.megatron_utils import train_helper as th
    g = torch.Generator().manual_seed(11 + packing + 2 * gspo)
    B, S, V = 4, 40, 700
    lens = torch.tensor([40, 17, 33, 25])
    attn = (torch.arange(S).unsqueeze(0) < lens.unsqueeze(1)).int()
    mask = attn.clone()
    mask[:, :5] = 0
    mask = torch.roll(mask, -1, 1)                       # Megatron flavour: rolled, last column kept
    adv = [np.float64(x) for x in (0.7, -1.2, 0.0, 2.0)]
    if packing:
        idx = torch.nonzero(attn.flatten()).flatten()
        T = idx.numel()
        logits = torch.randn(T, 1, V, generator=g)
        labels = torch.randint(0, V, (1, T), generator=g)
        inputs = {"indices": idx, "ori_batch_size": B, "ori_seq_len": S, "pad_size": 0}
    else:
        logits = torch.randn(S, B, V, generator=g)
        labels = torch.randint(0, V, (B, S), generator=g)
        inputs = {"pad_size": 0}
    # oracle: logprob [b, s] from [s, b, V] logits, re-padded when packed
    z = logits.double().requires_grad_(True)
    lp = osm.logprobs_from_logits(z.transpose(0, 1), labels)                 # [b, s]
    ent = osm.vocab_parallel_entropy_tp1(logits).transpose(0, 1).double()    # [b, s]
    if packing:
        lp = oi.pad_input(lp.permute(1, 0), idx, B, S).squeeze(-1)
        ent = oi.pad_input(ent.permute(1, 0), idx, B, S).squeeze(-1)
    old = lp.detach().float() + torch.randn(B, S, generator=g) * (0.002 if gspo else 0.1)
    ref = lp.detach().float() + torch.randn(B, S, generator=g) * 0.1
    clip = dict(pos_clip_ratio=1e-3 if gspo else 0.2, neg_clip_ratio=1e-3 if gspo else 0.2, diff_clip_ratio=10,
                final_clip_ratio=3)
    want = ol.megatron_all_losses(lp, ent, old.double(), ref.double(), adv, mask, use_group_sequence_policy=gspo, **clip)
    w_total, w_n, w_rep = ol.megatron_loss_func(mask, want)
    w_total.backward()

    margs = SimpleNamespace(packing=packing, use_group_sequence_policy=gspo, **clip)
    d = lambda x: x.to(dev)
    inputs_d = {k: (d(v) if isinstance(v, torch.Tensor) else v) for k, v in inputs.items()}
    inputs_d.update({"old_logprobs": d(old), "ref_logprobs": d(ref), "advantages": adv, "all_token_loss_mask": d(mask)})
    zl = d(logits).requires_grad_(True)
    got = th._compute_all_losses(margs, None, zl, d(labels), inputs_d)
    assert set(got) == set(want)
    g_total, g_n, g_rep = th.loss_func(inputs_d, got)
    g_total.backward()
    assert int(g_n) == int(w_n) and g_rep.keys() == w_rep.keys()
    for k in ("pg_loss", "entropy_loss", "kl_loss"):
        assert_close_rel(got[k], want[k], 1e-5, k)
        assert g_rep[k].item() == pytest.approx(w_rep[k].item(), rel=1e-4, abs=1e-5), k
    if gspo:
        # the clip flags compare each sequence's ratio with the bounds: exact unless a ratio sits within
        # rounding of a bound, which this case excludes (checked in float64)
        delta = (lp.detach() - old.double()) * mask
        ratio = torch.exp(delta.sum(1) / (mask.sum(1) + 1e-8))
        assert torch.minimum((ratio - 1.001).abs(), (ratio - 0.999).abs()).min() > 1e-6
        for k in ("is_positive_clipped", "is_negative_clipped", "is_clipped"):
            assert torch.equal(got[k].cpu(), want[k]), k
            assert g_rep[k].item() == w_rep[k].item() and got[k].dtype == torch.bool
            assert g_rep[k + "_sample_average"].item() == pytest.approx(w_rep[k + "_sample_average"].item(), rel=1e-6)
    assert float(g_total) == pytest.approx(float(w_total), rel=1e-5)
    assert_close_rel(zl.grad, z.grad, 1e-5, "dlogits")
    # only pg_loss is back-propagated; the report entries are detached fp32 scalars
    assert g_total.requires_grad and not any(v.requires_grad for v in g_rep.values())
    assert all(v.dtype == torch.float32 for k, v in g_rep.items() if k not in ("num_tokens", "num_samples"))
    assert g_rep["num_tokens"].dtype == torch.int32 and int(g_rep["num_samples"]) == 1


def test_masked_sums_kernel_against_torch_and_edge_cases(dev):
    """The reduction behind loss_func: every dtype it accepts, the sample-average division, the token
    count, an all-zero mask, an empty input, and the gradient it hands back."""
    from chatlearn_amd import ops
    g = torch.Generator().manual_seed(3)
    n = 70001                                         # not a multiple of the workgroup size
    a32 = torch.randn(n, generator=g)
    a64 = torch.randn(n, generator=g, dtype=torch.float64)
    flag = torch.rand(n, generator=g) < 0.3
    mask = (torch.rand(n, generator=g) < 0.6).int()
    sums, count = ops.masked_sums([a32.to(dev), a64.to(dev), flag.to(dev), flag.to(dev)], mask.to(dev),
                                  (False, False, False, True))
    m = mask.double()
    cnt = float(m.sum())
    want = [float((a32.double() * m).sum()), float((a64.float().double() * m).sum()), float((flag.double() * m).sum()),
            float((flag.double() * m).sum()) / (1e-5 + cnt)]
    assert int(count) == int(cnt) and sums.dtype == torch.float32 and count.dtype == torch.int32
    assert sums.cpu().tolist() == pytest.approx(want, rel=1e-6, abs=1e-4)
    assert float(sums[2]) == want[2]                  # a count of flags is exact
    zero, c0 = ops.masked_sums([a32.to(dev)], torch.zeros(n, dtype=torch.int32, device=dev), (True,))
    assert float(zero[0]) == 0.0 and int(c0) == 0     # 0 / (1e-5 + 0)
    e, ce = ops.masked_sums([torch.empty(0, device=dev)], torch.empty(0, dtype=torch.int32, device=dev), (False,))
    assert float(e[0]) == 0.0 and int(ce) == 0
    for dt in (torch.float32, torch.float64):
        gr = ops.masked_sums_backward(torch.tensor([2.5], device=dev), mask.to(dev), dt, (n,))
        assert gr.dtype == dt and torch.equal(gr.cpu(), (2.5 * mask).to(dt))
