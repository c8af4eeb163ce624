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


def _fp64_head(hidden, weight, labels_sb):
    """fp64 logits [s, b, V] from hidden [s, b, H]; logprob / entropy [b, s] as the Megatron path forms them."""
    h = hidden.double().detach().requires_grad_(True)
    w = weight.double().detach().requires_grad_(True)
    z = torch.nn.functional.linear(h, w)                                   # [s, b, V]
    lp = osm.logprobs_from_logits(z.transpose(0, 1), labels_sb)            # [b, s]
    ent = osm.vocab_parallel_entropy_tp1(z.detach()).transpose(0, 1).double()
    return h, w, lp, ent


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("packing", [False, True])
@pytest.mark.parametrize("gspo", [False, True])
def test_compute_all_losses_from_hidden_and_loss_func(dev, packing, gspo, dtype):
    """The fused Megatron seam: decoder output + output-layer weight in, the loss dict and the loss_func
    triple out, gradients reaching hidden and weight - against megatron_all_losses + megatron_loss_func fed
    by the float64 head.  The loss stage of the oracle reads the kernel's own fp32 logprob values (its
    gradient still flows through the float64 head), so both sides take every clip decision on identical
    inputs and the clip flags compare exactly."""
    from chatlearn_amd.algorithm.grpo_utils.megatron_utils import train_helper as th
    g = torch.Generator().manual_seed(31 + packing + 2 * gspo)
    B, S, V, H = 4, 40, 700, 128
    lens = torch.tensor([40, 17, 33, 25])
    attn = (torch.arange(S).unsqueeze(0) < lens.unsqueeze(1)).int()
    mask = attn.clone()
    mask[:, :5] = 0
    mask = torch.roll(mask, -1, 1)
    adv = [np.float64(x) for x in (0.7, -1.2, 0.0, 2.0)]
    weight = (torch.randn(V, H, generator=g) * 0.1).to(dtype)
    if packing:
        idx = torch.nonzero(attn.flatten()).flatten()
        T = idx.numel()
        hidden = torch.randn(T, 1, H, generator=g).to(dtype)
        labels = torch.randint(0, V, (1, T), generator=g)
        inputs = {"indices": idx, "ori_batch_size": B, "ori_seq_len": S, "pad_size": 0}
    else:
        hidden = torch.randn(S, B, H, generator=g).to(dtype)
        labels = torch.randint(0, V, (B, S), generator=g)
        inputs = {"pad_size": 0}
    rtol = 1e-5 if dtype == torch.float32 else 1e-2
    clip = dict(pos_clip_ratio=1e-3 if gspo else 0.2, neg_clip_ratio=1e-3 if gspo else 0.2, diff_clip_ratio=10,
                final_clip_ratio=3)
    h64, w64, lp64, ent64 = _fp64_head(hidden, weight, labels)
    repad = (lambda x: oi.pad_input(x.permute(1, 0), idx, B, S).squeeze(-1)) if packing else (lambda x: x)
    lp_pad, ent_pad = repad(lp64), repad(ent64)
    old = lp_pad.detach().float() + torch.randn(B, S, generator=g) * (0.002 if gspo else 0.1)
    ref = lp_pad.detach().float() + torch.randn(B, S, generator=g) * 0.1

    margs = SimpleNamespace(packing=packing, use_group_sequence_policy=gspo, **clip)
    d = lambda x: x.to(dev)
    inputs_d = {k: (d(v) if isinstance(v, torch.Tensor) else v) for k, v in inputs.items()}
    inputs_d.update({"old_logprobs": d(old), "ref_logprobs": d(ref), "advantages": adv, "all_token_loss_mask": d(mask)})
    hd, wd = d(hidden).requires_grad_(True), d(weight).requires_grad_(True)
    got = th.compute_all_losses_from_hidden(margs, hd, wd, d(labels), inputs_d)
    g_total, g_n, g_rep = th.loss_func(inputs_d, got)
    g_total.backward()

    # the oracle's loss stage on the kernel's logprob values, gradient through the float64 head
    with torch.no_grad():
        lp_vals = th.logprobs_from_hidden(margs, hd.detach(), wd.detach(), d(labels), inputs_d).cpu().double()
    lp_in = lp_pad + (lp_vals - lp_pad).detach()
    want = ol.megatron_all_losses(lp_in, ent_pad, old.double(), ref.double(), adv, mask, use_group_sequence_policy=gspo, **clip)
    w_total, w_n, w_rep = ol.megatron_loss_func(mask, want)
    w_total.backward()

    assert set(got) == set(want) and int(g_n) == int(w_n) and g_rep.keys() == w_rep.keys()
    assert_close_rel(lp_vals, lp_pad.detach(), rtol, "logprob from hidden")
    assert_close_rel(got["entropy_loss"], ent_pad, rtol, "entropy_loss")
    assert not got["entropy_loss"].requires_grad and not got["kl_loss"].requires_grad
    for k in ("pg_loss", "kl_loss"):
        assert_close_rel(got[k], want[k], 1e-5, k)
        assert g_rep[k].item() == pytest.approx(w_rep[k].item(), rel=1e-4, abs=1e-5), k
    if gspo:
        for k in ("is_positive_clipped", "is_negative_clipped", "is_clipped"):
            assert torch.equal(got[k].cpu(), want[k]), k
            assert g_rep[k].item() == w_rep[k].item()
            assert g_rep[k + "_sample_average"].item() == pytest.approx(w_rep[k + "_sample_average"].item(), rel=1e-6)
    assert float(g_total) == pytest.approx(float(w_total), rel=1e-5)
    assert hd.grad.shape == hidden.shape and wd.grad.shape == weight.shape and wd.grad.dtype == dtype
    assert_close_rel(hd.grad, h64.grad, rtol, "d hidden")
    assert_close_rel(wd.grad, w64.grad, rtol, "d output weight")
    # rows outside the mask (in the flattened hidden order) get exactly zero
    live_sb = mask.reshape(-1)[idx] if packing else mask.transpose(0, 1).reshape(-1)
    assert (hd.grad.reshape(-1, H)[d(live_sb) == 0] == 0).all()
    # without the mask promise every row is back-propagated: same gradients
    hd2, wd2 = d(hidden).requires_grad_(True), d(weight).requires_grad_(True)
    got2 = th.compute_all_losses_from_hidden(margs, hd2, wd2, d(labels), inputs_d, skip_masked_rows=False,
                                             keep_logits_rows=None)
    th.loss_func(inputs_d, got2)[0].backward()
    assert_close_rel(hd2.grad, h64.grad, rtol, "d hidden (no mask promise, recompute)")
    assert_close_rel(wd2.grad, w64.grad, rtol, "d output weight (no mask promise, recompute)")


def test_fused_megatron_step_from_a_raw_batch(dev):
    """get_batch_packed -> (stand-in decoder) -> compute_all_losses_from_hidden -> loss_func on a raw batch with
    tp = 2 alignment: the host copy of the packed loss mask equals the device one, the number of tokens is the
    packed mask's sum, and the gradients equal those of the materialised-logits route."""
    from chatlearn_amd.algorithm.grpo_utils.megatron_utils import train_helper as th
    from chatlearn_amd.bert_padding import index_first_axis
    g = torch.Generator().manual_seed(5)
    B, S, V, H = 5, 48, 300, 64
    p, r = [3, 7, 1, 10, 5], [20, 30, 47, 9, 13]
    tokens = torch.randint(0, V, (B, S), generator=g)
    data_b = {"all_tokens": tokens, "prompt_token_length": p, "response_token_length": r,
              "ref_logprobs": -torch.rand(B, S, generator=g), "old_logprobs": -torch.rand(B, S, generator=g),
              "advantages": [np.float64(x) for x in (1.0, -0.5, 0.25, 0.0, -2.0)]}
    inputs = th.get_batch_packed(data_b, True, eod=0, tp_size=2, device=dev)
    T = inputs["all_tokens"].shape[1]
    want_mask = oi.megatron_packed_batch(tokens, p, r, 0, tp_size=2)["loss_mask_on_this_cp_rank"][:, 0]
    assert torch.equal(inputs["packed_loss_mask_host"], want_mask)
    wide = torch.zeros(B, inputs["ori_seq_len"], dtype=torch.int32, device=dev)
    wide[:, :S] = inputs["all_token_loss_mask"][:, :inputs["ori_seq_len"]]
    # the [B, S] training mask looked up per packed token differs from the packed mask only where a sequence's
    # last position wraps: the reference rolls the two masks along different rows (train_helper.py:296-300,413)
    per_token = index_first_axis(wide.reshape(-1, 1), inputs["indices"]).reshape(-1).cpu()
    assert per_token.numel() == T
    emb = (torch.randn(V, H, generator=g) * 0.5).to(dev)
    weight = (torch.randn(V, H, generator=g) * 0.2).to(dev)
    margs = SimpleNamespace(packing=True, use_group_sequence_policy=False, pos_clip_ratio=0.2, neg_clip_ratio=0.2,
                            diff_clip_ratio=10, final_clip_ratio=3)
    host_mask = inputs["packed_loss_mask_host"]
    assert torch.equal(host_mask, per_token)

    def run(fused, with_host_mask=True):
        inputs["packed_loss_mask_host"] = host_mask if with_host_mask else None    # None: rows looked up on the device
        w = weight.clone().requires_grad_(True)
        hidden = emb[inputs["all_tokens"][0]].unsqueeze(1).clone().requires_grad_(True)      # [T, 1, H]
        if fused:
            losses = th.compute_all_losses_from_hidden(margs, hidden, w, inputs["labels"], inputs)
        else:
            logits = torch.nn.functional.linear(hidden, w)
            losses = th._compute_all_losses(margs, None, logits, inputs["labels"], inputs)
        total, n, rep = th.loss_func(inputs, losses)
        total.backward()
        return total.detach(), int(n), rep, hidden.grad, w.grad
    t1, n1, rep1, dh1, dw1 = run(True)
    t2, n2, rep2, dh2, dw2 = run(True, with_host_mask=False)
    assert torch.equal(dh1, dh2) and torch.equal(dw1, dw2) and float(t1) == float(t2) and n1 == n2
    t0, n0, rep0, dh0, dw0 = run(False)
    assert n1 == n0 == int(want_mask.sum())
    assert float(t1) == pytest.approx(float(t0), rel=1e-5)
    for k in ("pg_loss", "entropy_loss", "kl_loss"):
        assert rep1[k].item() == pytest.approx(rep0[k].item(), rel=1e-4, abs=1e-5)
    assert_close_rel(dh1, dh0, 1e-5, "d hidden, fused against materialised logits")
    assert_close_rel(dw1, dw0, 1e-5, "d weight, fused against materialised logits")
