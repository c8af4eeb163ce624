"""Pins for the CPU oracle itself: closed forms, invariants, brute force on tiny
inputs and library routines, chosen so that a dropped term, a wrong sign or a
transposed operand fails at least one of them.  No GPU needed."""
import math

import numpy as np
import pytest
import torch

from oracle import advantage as oadv
from oracle import indexing as oidx
from oracle import losses as ol
from oracle import softmax_stats as osm

D = torch.float64


# ----------------------------------------------------------------- softmax statistics

def test_uniform_and_dominant_logits():
    V = 37
    z = torch.zeros(2, 3, V, dtype=D) + 1.7
    lab = torch.randint(0, V, (2, 3))
    assert torch.allclose(osm.logprobs_from_logits(z, lab), torch.full((2, 3), -math.log(V), dtype=D))
    assert torch.allclose(osm.entropy_from_logits(z), torch.full((2, 3), math.log(V), dtype=D))
    z = torch.zeros(1, 1, V, dtype=D)
    z[0, 0, 4] = 80.0
    assert abs(osm.logprobs_from_logits(z, torch.tensor([[4]])).item()) < 1e-12
    assert abs(osm.entropy_from_logits(z).item()) < 1e-12
    assert osm.logprobs_from_logits(z, torch.tensor([[5]])).item() == pytest.approx(-80.0)


def test_brute_force_rows():
    g = torch.Generator().manual_seed(0)
    z = torch.randn(2, 4, 11, generator=g, dtype=D) * 3
    lab = torch.randint(0, 11, (2, 4), generator=g)
    lp = osm.logprobs_from_logits(z, lab)
    ent = osm.entropy_from_logits(z)
    for b in range(2):
        for s in range(4):
            row = [float(x) for x in z[b, s]]
            zsum = sum(math.exp(x) for x in row)
            assert lp[b, s].item() == pytest.approx(row[int(lab[b, s])] - math.log(zsum), abs=1e-12)
            p = [math.exp(x) / zsum for x in row]
            assert ent[b, s].item() == pytest.approx(-sum(q * math.log(q) for q in p), abs=1e-12)


def test_shift_invariance_chunking_and_tp1_entropy():
    g = torch.Generator().manual_seed(1)
    z = torch.randn(2, 1100, 50, generator=g)
    lab = torch.randint(0, 50, (2, 1100), generator=g)
    assert torch.allclose(osm.logprobs_from_logits(z + 3.5, lab), osm.logprobs_from_logits(z, lab), atol=1e-5)
    e = osm.entropy_from_logits(z)
    ec = osm.entropy_from_logits_with_chunking(z, chunk_size=512)   # 1100 = 2 chunks + ragged tail
    assert ec.dtype == torch.float32 and torch.allclose(e, ec, atol=1e-6)
    assert torch.allclose(osm.vocab_parallel_entropy_tp1(z), e, atol=1e-5)
    assert torch.allclose(osm.entropy_from_logits(z + 2.0), e, atol=1e-4)


def test_fused_forward_equals_library_routes_and_temperature_is_weight_scaling():
    g = torch.Generator().manual_seed(2)
    h = torch.randn(9, 16, generator=g, dtype=D)
    w = torch.randn(23, 16, generator=g, dtype=D)
    lab = torch.randint(0, 23, (9,), generator=g)
    lp, ent, mx, lse = osm.fused_head_forward(h, w, lab, 0.7)
    z = (h @ w.t()) / 0.7
    assert torch.allclose(lp, torch.log_softmax(z, -1)[torch.arange(9), lab])
    assert torch.allclose(mx, z.max(-1).values) and torch.allclose(lse, torch.logsumexp(z, -1))
    lp2, ent2, _, _ = osm.fused_head_forward(h, w / 0.7, lab, 1.0)
    assert torch.allclose(lp, lp2) and torch.allclose(ent, ent2)
    # transposed-operand guard: a non-square case would not even multiply if W were used untransposed
    assert z.shape == (9, 23)


def test_backward_closed_form_equals_autograd_and_sums_to_zero():
    g = torch.Generator().manual_seed(3)
    h = torch.randn(7, 8, generator=g, dtype=D)
    w = torch.randn(13, 8, generator=g, dtype=D)
    lab = torch.randint(0, 13, (7,), generator=g)
    g_lp = torch.randn(7, generator=g, dtype=D)
    g_en = torch.randn(7, generator=g, dtype=D)
    for ge in (None, g_en):
        for temp in (1.0, 0.7):
            a = osm.fused_head_backward_closed_form(h, w, lab, g_lp, ge, temp)
            b = osm.fused_head_backward_autograd(h, w, lab, g_lp, ge, temp)
            assert torch.allclose(a[0], b[0], atol=1e-12) and torch.allclose(a[1], b[1], atol=1e-12)
            # sum_v dz[t, v] = 0  =>  the columns of dW sum to zero
            assert a[1].sum(0).abs().max() < 1e-12
    # finite differences on one entry: guards the sign of the whole thing
    eps = 1e-6
    hp = h.clone(); hp[2, 3] += eps
    f = lambda hh: (osm.fused_head_forward(hh, w, lab)[0] * g_lp).sum()
    dh, _ = osm.fused_head_backward_closed_form(h, w, lab, g_lp, None)
    assert ((f(hp) - f(h)) / eps).item() == pytest.approx(dh[2, 3].item(), rel=1e-4)


# ----------------------------------------------------------------- GRPO / GSPO

def _grpo_scalar(lp, old, A, dc=10, pos=0.2, neg=0.2, fc=3.0):
    r = math.exp(min(lp - old, dc))
    l1 = -A * r
    l2 = -A * min(max(r, 1 - neg), 1 + pos)
    return min(max(l1, l2), fc)


def test_grpo_every_branch_closed_form():
    lp = torch.tensor([[0.0, 0.5, -0.5, 0.1, 11.0, 2.0]], dtype=D, requires_grad=True)
    old = torch.zeros(1, 6, dtype=D)
    # A > 0 row
    loss = ol.calculate_grpo_loss(lp, old, [2.0])
    want = [_grpo_scalar(float(x), 0.0, 2.0) for x in lp[0]]
    assert torch.allclose(loss[0], torch.tensor(want, dtype=D))
    loss.sum().backward()
    g = lp.grad[0]
    assert g[0].item() == pytest.approx(-2.0)                       # lp == old: L = -A, dL = -A
    assert g[1].item() == 0.0                                       # ratio > 1+pos, A > 0: clipped, no grad
    assert g[2].item() == pytest.approx(-2.0 * math.exp(-0.5))      # ratio < 1-neg, A > 0: unclipped branch wins
    assert g[3].item() == pytest.approx(-2.0 * math.exp(0.1))       # inside the clip range
    assert g[4].item() == 0.0                                       # lp - old > diff_clip
    # A < 0 row
    lp2 = torch.tensor([[-0.5, 0.5, 1.0]], dtype=D, requires_grad=True)
    loss2 = ol.calculate_grpo_loss(lp2, torch.zeros(1, 3, dtype=D), [-1.0])
    assert loss2[0, 0].item() == pytest.approx(0.8)                 # ratio < 1-neg, A < 0: L = -A (1-neg)
    assert loss2[0, 1].item() == pytest.approx(math.exp(0.5))       # ratio > 1+pos, A < 0: unclipped wins
    loss2.sum().backward()
    assert lp2.grad[0, 0].item() == 0.0 and lp2.grad[0, 1].item() == pytest.approx(math.exp(0.5))
    # final clip: -A * ratio above the cap
    lp3 = torch.tensor([[2.0]], dtype=D, requires_grad=True)
    loss3 = ol.calculate_grpo_loss(lp3, torch.zeros(1, 1, dtype=D), [-1.0], final_clip_ratio=3.0)
    assert loss3.item() == 3.0
    loss3.sum().backward()
    assert lp3.grad.item() == 0.0


def test_grpo_dtype_quirk_and_nan_assert():
    lp = torch.zeros(2, 3)
    assert ol.calculate_grpo_loss(lp, lp, [0.5, 1.0]).dtype == torch.float32
    assert ol.calculate_grpo_loss(lp, lp, [np.float64(0.5), np.float64(1.0)]).dtype == torch.float64
    bad = lp.clone(); bad[0, 0] = float("nan")
    with pytest.raises(AssertionError, match="pg loss is nan"):
        ol.calculate_grpo_loss(bad, lp, [0.5, 1.0])


def test_gspo_sequence_ratio_and_flags():
    lp = torch.tensor([[0.2, 0.4, 9.0], [-0.3, -0.1, 5.0]], dtype=D, requires_grad=True)
    old = torch.zeros(2, 3, dtype=D)
    mask = torch.tensor([[1, 1, 0], [1, 1, 0]], dtype=torch.int32)
    loss, pos, neg, clip = ol.calculate_gspo_loss(lp, old, [1.0, -2.0], 10, 0.1, 0.1, 3.0, mask)
    r0, r1 = math.exp(0.3), math.exp(-0.2)          # exp(mean of the masked diffs); masked-out 9.0 / 5.0 ignored
    assert torch.allclose(loss[0], torch.full((3,), -1.0 * 1.1, dtype=D))          # clipped at 1+pos, A>0
    assert torch.allclose(loss[1], torch.full((3,), 2.0 * 0.9, dtype=D))           # clipped at 1-neg, A<0
    assert pos.tolist() == [[True] * 3, [False] * 3] and neg.tolist() == [[False] * 3, [True] * 3]
    assert clip.all()
    loss2, *_ = ol.calculate_gspo_loss(lp, old, [1.0, -2.0], 10, 0.5, 0.5, 3.0, mask)
    loss2.sum().backward()
    # every token of a sequence (masked or not) gets -A * ratio: no 1/|y| factor
    assert torch.allclose(lp.grad[0], torch.full((3,), -r0, dtype=D))
    assert torch.allclose(lp.grad[1], torch.full((3,), 2.0 * r1, dtype=D))
    assert torch.allclose(loss2[0], torch.full((3,), -r0, dtype=D))


def test_k3_kl_identities_and_asserts():
    lp = torch.tensor([-1.0, -2.0, -0.5], dtype=D, requires_grad=True)
    ref = torch.tensor([-1.0, -1.5, -2.5], dtype=D)
    kl = ol.k3_kl(ref, lp)
    assert kl[0].item() == 0.0 and (kl >= 0).all()
    kl.sum().backward()
    assert torch.allclose(lp.grad, 1 - torch.exp(ref - lp.detach()))
    assert ol.k3_kl(torch.tensor([50.0]), torch.tensor([0.0])).item() == 10.0      # clamp at 10
    with pytest.raises(AssertionError, match="inf"):
        ol.k3_kl(torch.tensor([500.0]), torch.tensor([0.0]))
    with pytest.raises(AssertionError, match="nan"):
        ol.k3_kl(torch.tensor([float("nan")]), torch.tensor([0.0]))


def test_fsdp_assembly_linearity_and_switches():
    g = torch.Generator().manual_seed(4)
    B, S = 3, 5
    lp = (torch.randn(B, S, generator=g) * 0.1 - 2).requires_grad_(True)
    old = lp.detach() + torch.randn(B, S, generator=g) * 0.05
    ref = lp.detach() + torch.randn(B, S, generator=g) * 0.1
    ent = torch.rand(B, S, generator=g) + 1
    mask = (torch.rand(B, S, generator=g) < 0.7).int()
    adv = [0.5, -1.0, 2.0]
    N = 11.0
    total, parts = ol.fsdp_policy_loss(lp, ent, old, ref, adv, mask, N, kl_coef=0.1, entropy_coef=0.01)
    pg = ol.calculate_grpo_loss(lp, old, adv)[mask.bool()].sum() / N
    kl = ol.k3_kl(ref, lp)[mask.bool()].sum() / N
    en = ent[mask.bool()].sum() / N
    assert total.item() == pytest.approx((pg - 0.01 * en + 0.1 * kl).item(), rel=1e-6)
    total0, _ = ol.fsdp_policy_loss(lp, ent, old, ref, adv, mask, N)                # both coefficients off
    assert total0.item() == pytest.approx(pg.item(), rel=1e-6)
    total2, _ = ol.fsdp_policy_loss(lp, ent, old, ref, adv, mask, N, fsdp_size=2)
    assert total2.item() == pytest.approx(2 * pg.item(), rel=1e-6)
    assert parts["pg_loss"].numel() == int(mask.sum())
    m = ol.fsdp_train_metrics([parts["pg_loss"]], [parts["entropy_loss"]], [parts["kl_loss"]], N)
    assert m["pg_loss"] == pytest.approx(pg.item(), rel=1e-6)
    assert m["entropy_loss"] == pytest.approx(ent[mask.bool()].mean().item(), rel=1e-6)


def test_megatron_losses_and_loss_func():
    g = torch.Generator().manual_seed(5)
    lp = torch.randn(2, 4, generator=g) * 0.1 - 1
    old, ref = lp + 0.01, lp - 0.02
    mask = torch.tensor([[1, 1, 0, 0], [1, 1, 1, 0]], dtype=torch.int32)
    ent = torch.rand(2, 4, generator=g)
    d = ol.megatron_all_losses(lp, ent, old, ref, [1.0, -1.0], mask, use_group_sequence_policy=True,
                               pos_clip_ratio=1e-3, neg_clip_ratio=1e-3)
    assert set(d) == {"pg_loss", "entropy_loss", "kl_loss", "is_positive_clipped", "is_negative_clipped",
                      "is_clipped", "is_positive_clipped_sample_average", "is_negative_clipped_sample_average",
                      "is_clipped_sample_average"}
    k = ref - lp
    assert torch.allclose(d["kl_loss"][0, 2:], (1 - k - 1)[0, 2:])        # masked-out: exp(k) replaced by 1
    total, n, rep = ol.megatron_loss_func(mask, d)
    assert int(n) == 5 and total.item() == pytest.approx((d["pg_loss"].float() * mask).sum().item())
    assert rep["is_clipped_sample_average"].item() == pytest.approx(
        (d["is_clipped"].float() * mask).sum().item() / (1e-5 + 5))


# ----------------------------------------------------------------- masks / unpad / pad

def test_masks_brute_force_and_shift():
    tokens = torch.arange(24).reshape(3, 8)
    p, r = [2, 0, 5], [3, 8, 9]            # last one overruns the row: slices truncate
    attn, loss, pos = oidx.generate_loss_mask_position_ids(tokens, p, r)
    for i in range(3):
        for s in range(8):
            assert attn[i, s].item() == int(s < p[i] + r[i])
            assert loss[i, s].item() == int(p[i] <= s < p[i] + r[i])
            assert pos[i, s].item() == s
    assert attn.dtype == torch.int32 and loss.dtype == torch.int32 and pos.dtype == torch.int64
    lab = oidx.shift_labels(tokens)
    assert lab[0].tolist() == [1, 2, 3, 4, 5, 6, 7, 0]                  # wraps inside the row
    sm = oidx.shift_loss_mask_fsdp(loss)
    assert sm[0].tolist() == [0, 1, 1, 1, 0, 0, 0, 0] and sm[1].tolist() == [1] * 7 + [0]
    assert oidx.shift_loss_mask_megatron(loss)[1].tolist() == [1] * 8   # no zeroing of the last column


def test_unpad_pad_roundtrip_and_invariants():
    g = torch.Generator().manual_seed(6)
    B, S, Hd = 4, 9, 3
    lens = [9, 0, 4, 1]
    mask = torch.zeros(B, S, dtype=torch.int32)
    for b, n in enumerate(lens):
        mask[b, :n] = 1
    x = torch.randn(B, S, Hd, generator=g)
    u, idx, cu, mx = oidx.unpad_input(x, mask)
    assert cu.tolist() == [0, 9, 9, 13, 14] and cu.dtype == torch.int32 and mx == 9
    assert idx.tolist() == [b * S + s for b in range(B) for s in range(lens[b])] and idx.dtype == torch.int64
    assert torch.equal(u, x.reshape(-1, Hd)[idx])
    back = oidx.pad_input(u, idx, B, S)
    assert torch.equal(back, x * mask.unsqueeze(-1))
    parts = oidx.split_and_unpadding(back[..., 0], mask)
    assert [t.numel() for t in parts] == lens


# ----------------------------------------------------------------- advantages

def _buf(samples):
    return [oadv._Buffer(samples)]


def test_advantage_bernoulli_closed_form_and_flags():
    G, k = 8, 3
    samples = [{"prompt_uid": "0_0", "rule_reward": 1.0 if i < k else 0.0} for i in range(G)]
    samples += [{"prompt_uid": "0_1", "rule_reward": 1.0} for _ in range(G)]
    samples += [{"prompt_uid": "0_2", "rule_reward": 0.0} for _ in range(G)]
    ac = oadv.AdvantageComputer(G)
    out = ac(_buf(samples))
    q = k / G
    assert out[0]["advantages"] == pytest.approx((1 - q) / (math.sqrt(q * (1 - q)) + 1e-5), rel=1e-12)
    assert out[G - 1]["advantages"] == pytest.approx((0 - q) / (math.sqrt(q * (1 - q)) + 1e-5), rel=1e-12)
    assert all(s["advantages"] == 0.0 for s in out[G:])            # all-equal rewards: exactly zero
    assert isinstance(out[0]["advantages"], np.float64)
    name, m = ac.get_and_clear_metrics()
    assert name == "advantage_compute" and m["all_correct_ratio"] == pytest.approx(1 / 3)
    assert m["all_wrong_ratio"] == pytest.approx(1 / 3)
    assert ac.get_and_clear_metrics() == ("advantage_compute", {})
    assert len(ac.rule_reward_buffer) == 0                           # complete groups are dropped


def test_advantage_carry_over_and_numpy_semantics():
    ac = oadv.AdvantageComputer(4)
    first = [{"prompt_uid": "7_1", "rule_reward": r} for r in (0.25, 1.0)]
    ac(_buf(first))
    assert first[0]["advantages"] == pytest.approx((0.25 - 0.625) / (np.std([0.25, 1.0]) + 1e-5))
    assert ac.rule_reward_buffer["7_1"] == [0.25, 1.0]               # incomplete group stays buffered
    second = [{"prompt_uid": "7_1", "rule_reward": r} for r in (0.5, 0.0)]
    ac(_buf(second))
    pool = [0.25, 1.0, 0.5, 0.0]
    assert second[0]["advantages"] == (0.5 - np.mean(pool)) / (np.std(pool) + 1e-5)   # ddof = 0, eps 1e-5
    assert "7_1" not in ac.rule_reward_buffer


@pytest.mark.parametrize("n", [1, 2, 3, 4, 6])
def test_vocab_parallel_oracle_equals_unsharded_for_any_split(n):
    """The rank-by-rank reductions (max, sum of exponentials, masked target gather, sum of p*z)
    must give the plain log_softmax gather and entropy however the vocabulary is cut; a wrong
    sign, a gather outside the owner's range or a missing max shift breaks one of them."""
    from oracle import vocab_parallel as ovp
    g = torch.Generator().manual_seed(n)
    z = torch.randn(9, 24, generator=g, dtype=torch.float64) * 4
    labels = torch.randint(0, 24, (9,), generator=g)
    labels[0], labels[1] = 0, 23
    ranges = ovp.shard_ranges(24, n)
    shards = [z[:, lo:hi] for lo, hi in ranges]
    assert torch.allclose(ovp.vocab_parallel_logprob(shards, labels, ranges).double(),
                          torch.log_softmax(z, -1).gather(1, labels[:, None]).squeeze(1), atol=1e-5)
    p = torch.softmax(z, -1)
    assert torch.allclose(ovp.vocab_parallel_entropy(shards).double(), -(p * p.log()).sum(-1), atol=1e-5)
    # uniform logits: entropy log V, logprob -log V whichever rank owns the label
    u = [torch.zeros(3, 24 // n) for _ in range(n)]
    assert torch.allclose(ovp.vocab_parallel_entropy(u), torch.full((3,), math.log(24.0)))
    assert torch.allclose(ovp.vocab_parallel_logprob(u, torch.tensor([0, 11, 23]), ranges),
                          torch.full((3,), -math.log(24.0)))


def test_megatron_packed_batch_oracle_against_hand_worked_cases():
    import json
    import os
    from oracle import indexing as oidx
    with open(os.path.join(os.path.dirname(__file__), "golden", "thd_pack_cases.json")) as f:
        gold = json.load(f)
    tokens = torch.tensor(gold["tokens"])
    for c in gold["cases"]:
        out = oidx.megatron_packed_batch(tokens, gold["prompt"], gold["response"], gold["eod"], tp_size=c["tp"],
                                         cp_size=c["cp"], cp_rank=c["rank"])
        assert out["packed_seq_params"]["cu_seqlens_q"].tolist() == c["cu_seqlens_padded"]
        assert out["indices"].tolist() == c["indices"]
        assert out["seq_indices"][0].tolist() == c["seq_indices"]
        assert out["all_tokens"][0].tolist() == c["all_tokens"]
        assert out["labels"][0].tolist() == c["labels"]
        assert out["loss_mask_on_this_cp_rank"][:, 0].tolist() == c["loss_mask"]
        assert int(out["num_tokens_on_this_cp_rank"]) == c["num_tokens"] and int(out["pad_size"]) == c["pad_size"]


@pytest.mark.parametrize("cp", [2, 4])
def test_context_parallel_partition_properties(cp):
    """What fixes the load-balanced split of a packed row over context-parallel ranks, without the
    library the reference calls for it: the ranks' index sets partition the row, each is ascending
    (sequence order is kept), each rank gets 1/cp of every sequence, and under a causal mask every
    rank does the same amount of attention work per sequence (rank r pairs chunk r with chunk
    2cp-1-r).  A literal case worked by hand closes the chunk numbering."""
    lens = [4 * cp, 8 * cp, 2 * cp]
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    total = cu[-1]
    parts = [oidx.thd_partitioned_indices(cu, total, cp, r) for r in range(cp)]
    assert sorted(torch.cat(parts).tolist()) == list(range(total))
    for part in parts:
        assert part.tolist() == sorted(part.tolist()) and len(part) == total // cp
    for s in range(len(lens)):
        work = []
        for part in parts:
            mine = [int(i) - cu[s] for i in part.tolist() if cu[s] <= i < cu[s + 1]]
            assert len(mine) == lens[s] // cp
            work.append(sum(pos + 1 for pos in mine))     # keys a causal query at `pos` attends to
        assert len(set(work)) == 1
    if cp == 2:
        # one sequence of 8 tokens, 4 chunks of 2: rank 0 keeps chunks 0 and 3, rank 1 chunks 1 and 2
        assert oidx.thd_partitioned_indices([0, 8], 8, 2, 0).tolist() == [0, 1, 6, 7]
        assert oidx.thd_partitioned_indices([0, 8], 8, 2, 1).tolist() == [2, 3, 4, 5]
