"""Policy-loss kernel and the loss_gallery mirrors against the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import losses as ol
from tests.util import assert_close_rel

pytestmark = pytest.mark.gpu


def _case(B, S, seed, spread=0.3):
    g = torch.Generator().manual_seed(seed)
    lp = torch.randn(B, S, generator=g) * 0.5 - 2.0
    old = lp + torch.randn(B, S, generator=g) * spread
    ref = lp + torch.randn(B, S, generator=g) * 0.2
    ent = torch.rand(B, S, generator=g) * 3
    mask = (torch.rand(B, S, generator=g) < 0.7).int()
    mask[:, -1] = 0
    adv = (torch.randn(B, generator=g) * 1.5)
    adv[0] = 0.0
    return lp, old, ref, ent, mask, adv


@pytest.mark.parametrize("adv_np", [False, True])
@pytest.mark.parametrize("B,S", [(1, 1), (5, 37), (32, 700)])
def test_grpo_mirror_value_grad_dtype(dev, B, S, adv_np):
    from chatlearn_amd.algorithm.grpo_utils.loss_gallery import calculate_grpo_loss
    lp, old, ref, ent, mask, adv = _case(B, S, B * S)
    # force every branch to appear: big positive / negative deltas, exact ties, final clip
    if S > 8:
        old[:, 0] = lp[:, 0]                     # ratio exactly 1 (tie of the two surrogates)
        old[:, 1] = lp[:, 1] - 11.0              # above diff_clip
        old[:, 2] = lp[:, 2] - 2.0               # ratio ~ 7.4: final clip for A < 0
        old[:, 3] = lp[:, 3] + 2.0
    advantages = [np.float64(a) for a in adv.tolist()] if adv_np else [float(a) for a in adv.tolist()]
    kw = dict(diff_clip_ratio=10, pos_clip_ratio=0.2, neg_clip_ratio=0.25, final_clip_ratio=3.0)
    a = lp.clone().requires_grad_(True)
    want = ol.calculate_grpo_loss(a, old, advantages, **kw)
    w = torch.randn(B, S, generator=torch.Generator().manual_seed(1)).to(want.dtype)
    (want * w).sum().backward()
    b = lp.to(dev).requires_grad_(True)
    got = calculate_grpo_loss(b, old.to(dev), advantages, **kw)
    assert got.dtype == want.dtype and got.shape == want.shape and got.is_contiguous()
    (got * w.to(dev)).sum().backward()
    rt = 1e-5
    assert_close_rel(got, want, rt, "grpo loss")
    assert_close_rel(b.grad, a.grad, rt, "grpo dloss/dlp")


@pytest.mark.parametrize("B,S", [(3, 11), (16, 900)])
def test_gspo_mirror_value_flags_grad(dev, B, S):
    from chatlearn_amd.algorithm.grpo_utils.loss_gallery import calculate_gspo_loss
    lp, old, ref, ent, mask, adv = _case(B, S, 7 * B + S, spread=0.02)
    old = lp + (old - lp) * 0.05 + torch.linspace(-4e-3, 4e-3, B).unsqueeze(1)   # sequence ratios around the clip range
    mask[1] = 0                                                                   # a fully masked sequence
    advantages = [np.float64(a) for a in adv.tolist()]
    kw = dict(diff_clip_ratio=10, pos_clip_ratio=4e-4, neg_clip_ratio=3e-4, final_clip_ratio=3.0, loss_mask=mask)
    a = lp.clone().requires_grad_(True)
    want = ol.calculate_gspo_loss(a, old, advantages, **kw)
    want[0].sum().backward()
    b = lp.to(dev).requires_grad_(True)
    kw["loss_mask"] = mask.to(dev)
    got = calculate_gspo_loss(b, old.to(dev), advantages, **kw)
    got[0].sum().backward()
    assert got[0].dtype == want[0].dtype
    assert_close_rel(got[0], want[0], 1e-5, "gspo loss")
    assert_close_rel(b.grad, a.grad, 1e-5, "gspo grad")
    # The three flags compare the per-sequence ratio with the clip bounds.  They are exact unless a
    # sequence's ratio lies within fp32 rounding of a bound, which this case excludes (checked here
    # in float64), so kernel and oracle must agree on every flag of every token.
    d64 = (lp.double() - old.double()) * mask
    ratio64 = torch.exp(d64.sum(1) / (mask.sum(1) + 1e-8))
    live = mask.sum(1) > 0
    margin = torch.minimum((ratio64 - (1 + 4e-4)).abs(), (ratio64 - (1 - 3e-4)).abs())[live].min()
    assert margin > 1e-6, "test case sits on a clip bound; pick another seed"
    for name, g_, w_ in zip(("pos", "neg", "clipped"), got[1:], want[1:]):
        assert g_.dtype == torch.bool and g_.shape == w_.shape
        assert torch.equal(g_.cpu(), w_), f"{name}: {int((g_.cpu() != w_).sum())} flags differ"
    if B >= 16:
        assert want[1].any() and want[2].any() and want[3].any()      # every flag occurs in the case


@pytest.mark.parametrize("mode", ["grpo", "gspo"])
@pytest.mark.parametrize("packed", [False, True])
def test_fused_loss_assembly_sums_flags_and_upstream_grads(dev, mode, packed):
    """clgrpo_policy_loss in one launch against policy_trainer.py:253-286 restated on [B,S]."""
    from chatlearn_amd import ops
    from chatlearn_amd._lib import LOSS_GRPO, LOSS_GSPO
    B, S = 9, 130
    lp, old, ref, ent, mask, adv = _case(B, S, 99, spread=0.1)
    lens = torch.randint(20, S + 1, (B,), generator=torch.Generator().manual_seed(3))
    valid = (torch.arange(S).unsqueeze(0) < lens.unsqueeze(1))
    mask = mask * valid.int()
    N, klc, enc = 555.0, 0.05, 0.01
    a = lp.clone().requires_grad_(True)
    e = ent.clone().requires_grad_(True)
    total, parts = ol.fsdp_policy_loss(a, e, old, ref, adv.tolist(), mask, N, entropy_coef=enc, kl_coef=klc,
                                       pos_clip_ratio=0.2, neg_clip_ratio=0.2, final_clip_ratio=3,
                                       use_group_sequence_policy=(mode == "gspo"))
    total.backward()
    if packed:
        sel = valid.flatten()
        f = lambda x: x.flatten()[sel].contiguous().to(dev)
        cu = torch.zeros(B + 1, dtype=torch.int32)
        cu[1:] = torch.cumsum(lens, 0)
        args = (f(lp), f(old), adv.to(dev))
        kw = dict(cu_seqlens=cu.to(dev), ref_logprob=f(ref), entropy=f(ent), loss_mask=f(mask))
    else:
        args = (lp.to(dev), old.to(dev), adv.to(dev))
        kw = dict(ref_logprob=ref.to(dev), entropy=ent.to(dev), loss_mask=mask.to(dev))
    res = ops.policy_loss(*args, mode=LOSS_GSPO if mode == "gspo" else LOSS_GRPO, kl_coef=klc, entropy_coef=enc,
                          grad_scale=1.0 / N, pos_clip_ratio=0.2, neg_clip_ratio=0.2, final_clip_ratio=3,
                          want_upstream=True, **kw)
    res.raise_on_flags()
    sums = res.sums.cpu()
    assert sums[0].item() / N == pytest.approx(parts["pg_loss_mean"].item(), rel=1e-5)
    assert sums[1].item() / N == pytest.approx(parts["kl_loss_mean"].item(), rel=1e-5)
    assert sums[2].item() / N == pytest.approx(parts["entropy_loss_mean"].item(), rel=1e-5)
    assert sums[3].item() == float(mask.sum())
    want_glp, want_gen = a.grad, e.grad
    if packed:
        want_glp, want_gen = want_glp.flatten()[sel], want_gen.flatten()[sel]
    assert_close_rel(res.g_logprob, want_glp, 1e-5, "g_logprob")
    assert_close_rel(res.g_entropy, want_gen, 1e-5, "g_entropy")
    # two runs give identical bits (fixed-order reductions)
    res2 = ops.policy_loss(*args, mode=LOSS_GSPO if mode == "gspo" else LOSS_GRPO, kl_coef=klc, entropy_coef=enc,
                           grad_scale=1.0 / N, pos_clip_ratio=0.2, neg_clip_ratio=0.2, final_clip_ratio=3,
                           want_upstream=True, **kw)
    assert torch.equal(res.sums, res2.sums) and torch.equal(res.g_logprob, res2.g_logprob)


def test_error_flags_raise_reference_messages(dev):
    from chatlearn_amd import ops
    from chatlearn_amd.algorithm.grpo_utils.loss_gallery import calculate_grpo_loss
    lp = torch.zeros(2, 4, device=dev)
    bad = lp.clone()
    bad[0, 1] = float("nan")
    with pytest.raises(AssertionError, match="pg loss is nan"):
        calculate_grpo_loss(bad, lp, [1.0, 1.0])
    adv = torch.ones(2, device=dev)
    mask = torch.ones(2, 4, dtype=torch.int32, device=dev)
    ref = lp.clone()
    ref[1, 2] = 500.0
    with pytest.raises(AssertionError, match="kl loss ratio has inf values"):
        ops.policy_loss(lp, lp, adv, ref_logprob=ref, loss_mask=mask).raise_on_flags()
    mask[1, 2] = 0                                     # masked-out positions do not trip the check
    ops.policy_loss(lp, lp, adv, ref_logprob=ref, loss_mask=mask).raise_on_flags()
    ref[0, 0] = float("nan")
    with pytest.raises(AssertionError, match="kl loss ratio has nan values"):
        ops.policy_loss(lp, lp, adv, ref_logprob=ref, loss_mask=mask).raise_on_flags()


def test_megatron_style_outputs(dev):
    """Per-token kl with exp(k) -> 1 at masked-out positions and masked sums (train_helper.py:465-547)."""
    from chatlearn_amd import ops
    B, S = 4, 50
    lp, old, ref, ent, mask, adv = _case(B, S, 5, spread=0.001)
    d = ol.megatron_all_losses(lp, ent, old, ref, adv.tolist(), mask, use_group_sequence_policy=True,
                               pos_clip_ratio=1e-3, neg_clip_ratio=1e-3, final_clip_ratio=3)
    total, n, rep = ol.megatron_loss_func(mask, d)
    from chatlearn_amd._lib import LOSS_GSPO
    res = ops.policy_loss(lp.to(dev), old.to(dev), adv.to(dev), mode=LOSS_GSPO, ref_logprob=ref.to(dev),
                          entropy=ent.to(dev), loss_mask=mask.to(dev), pos_clip_ratio=1e-3, neg_clip_ratio=1e-3,
                          final_clip_ratio=3, want_flags3=True)
    assert_close_rel(res.kl, d["kl_loss"], 1e-5, "kl per token")
    s = res.sums.cpu()
    assert s[0].item() == pytest.approx(rep["pg_loss"].item(), rel=1e-5)
    assert s[1].item() == pytest.approx(rep["kl_loss"].item(), rel=1e-4, abs=1e-7)
    assert s[2].item() == pytest.approx(rep["entropy_loss"].item(), rel=1e-5)
    assert int(s[3].item()) == int(n)
    assert s[6].item() == rep["is_clipped"].item()
