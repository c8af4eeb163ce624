"""Mask / index kernels, group advantages and statistics-from-logits against the
CPU oracle.  Integer outputs are compared bit for bit."""
import numpy as np
import pytest
import torch

from oracle import advantage as oadv
from oracle import indexing as oidx
from oracle import softmax_stats as osm
from tests.util import assert_close_rel

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("B,S", [(1, 1), (3, 8), (17, 700), (300, 33)])
def test_masks_and_shifts_bit_exact(dev, B, S):
    from chatlearn_amd import ops
    from chatlearn_amd.algorithm.grpo_utils import trainer_utils as tu
    g = torch.Generator().manual_seed(B * S)
    p = torch.randint(0, S + 1, (B,), generator=g).tolist()
    r = torch.randint(0, S + 3, (B,), generator=g).tolist()          # some overrun the row
    tokens = torch.randint(0, 1000, (B, S), generator=g)
    want = oidx.generate_loss_mask_position_ids(tokens, p, r)
    for src in (tokens, tokens.to(dev)):                              # CPU tokens come back on the CPU
        got = tu.generate_loss_mask_position_ids(src, p, r)
        for a, b in zip(got, want):
            assert a.dtype == b.dtype and a.device == src.device and torch.equal(a.cpu(), b)
    lab, sm = ops.shift_labels(tokens.to(dev), want[1].to(dev), zero_last=True)
    assert torch.equal(lab.cpu(), oidx.shift_labels(tokens))
    assert torch.equal(sm.cpu(), oidx.shift_loss_mask_fsdp(want[1].clone()))
    _, sm2 = ops.shift_labels(None, want[1].to(dev), zero_last=False)
    assert torch.equal(sm2.cpu(), oidx.shift_loss_mask_megatron(want[1]))


@pytest.mark.parametrize("B,S,Hd", [(1, 1, 1), (4, 9, 3), (64, 1000, 8), (700, 5, 1)])
def test_unpad_pad_bit_exact(dev, B, S, Hd):
    from chatlearn_amd.algorithm.grpo_utils import trainer_utils as tu
    from chatlearn_amd.bert_padding import pad_input
    g = torch.Generator().manual_seed(B + S)
    lens = torch.randint(0, S + 1, (B,), generator=g)
    lens[0] = S
    if B > 2:
        lens[1] = 0                                                   # an empty sequence
    mask = (torch.arange(S).unsqueeze(0) < lens.unsqueeze(1)).int()
    if B > 3:
        mask[3] = (torch.rand(S, generator=g) < 0.5).int()            # holes, not only right padding
    x = torch.randn(B, S, Hd, generator=g).to(torch.bfloat16)
    wu, widx, wcu, wmx = oidx.unpad_input(x, mask)
    u, idx, cu, mx = tu.unpad_input(x.to(dev), mask.to(dev))
    assert idx.dtype == torch.int64 and cu.dtype == torch.int32 and isinstance(mx, int)
    assert torch.equal(idx.cpu(), widx) and torch.equal(cu.cpu(), wcu) and mx == wmx
    assert torch.equal(u.cpu(), wu)
    back = pad_input(u, idx, B, S)
    assert torch.equal(back.cpu(), oidx.pad_input(wu, widx, B, S))
    assert torch.equal(back.cpu(), x * mask.unsqueeze(-1).to(x.dtype))
    # odd row sizes (2-byte rows) and int64 rows, as the trainer uses for tokens / position ids
    t = torch.randint(0, 1 << 40, (B, S, 1), generator=g)
    ut, *_ = tu.unpad_input(t.to(dev), mask.to(dev))
    assert torch.equal(ut.cpu(), t.reshape(-1, 1)[widx])
    # vision-language position ids: a leading channel dimension
    pos = torch.randint(0, 100, (3, B, S, 1), generator=g)
    up, *_ = tu.unpad_input(pos.to(dev), mask.to(dev))
    assert up.shape[0] == 3 and torch.equal(up[2].cpu(), pos[2].reshape(-1, 1)[widx])


def test_pad_input_is_differentiable(dev):
    from chatlearn_amd.bert_padding import index_first_axis, pad_input
    idx = torch.tensor([0, 2, 5, 7], device=dev)
    v = torch.randn(4, 1, device=dev, requires_grad=True)
    out = pad_input(v, idx, 2, 4)
    w = torch.arange(8., device=dev).reshape(2, 4, 1)
    (out * w).sum().backward()
    assert torch.equal(v.grad.flatten().cpu(), torch.tensor([0., 2., 5., 7.]))
    src = torch.randn(8, 3, device=dev, requires_grad=True)
    index_first_axis(src, idx).sum().backward()
    want = torch.zeros(8, 3)
    want[idx.cpu()] = 1
    assert torch.equal(src.grad.cpu(), want)


def _buf(s):
    return [oadv._Buffer(s)]


@pytest.mark.parametrize("reward_kind", ["bernoulli", "uniform"])
def test_advantage_computer_matches_oracle(dev, reward_kind):
    import copy
    from chatlearn_amd.algorithm.grpo_utils.advantage_compute import AdvantageComputer
    rng = np.random.default_rng(0)
    G = 8
    def batch(uids):
        out = []
        for u in uids:
            r = float(rng.random() < 0.3) if reward_kind == "bernoulli" else float(rng.random())
            out.append({"prompt_uid": u, "rule_reward": r})
        return out
    a, b = AdvantageComputer(G), oadv.AdvantageComputer(G)
    # first call: 5 complete groups (interleaved order) + one group with only 3 of its 8 responses
    uids = [f"0_{i % 5}" for i in range(5 * G)] + ["0_9"] * 3
    # second call: the rest of group 9 arrives, plus two new groups
    uids2 = ["0_9"] * 5 + ["1_0"] * G + ["1_1"] * G
    for u in (uids, uids2):
        s1 = batch(u)
        s2 = copy.deepcopy(s1)
        o1, o2 = a(_buf(s1)), b(_buf(s2))
        got = np.array([s["advantages"] for s in o1])
        want = np.array([s["advantages"] for s in o2])
        assert isinstance(o1[0]["advantages"], np.float64)
        assert np.array_equal(got, want), f"max diff {np.abs(got - want).max()}"   # float64, bit for bit
        assert dict(a.rule_reward_buffer) == dict(b.rule_reward_buffer)
    ma, mb = a.get_and_clear_metrics(), b.get_and_clear_metrics()
    assert ma[0] == mb[0] and ma[1].keys() == mb[1].keys()
    for k in ma[1]:
        assert ma[1][k] == pytest.approx(mb[1][k])


def test_group_advantage_large_pool_and_flags(dev):
    from chatlearn_amd import ops
    rng = np.random.default_rng(1)
    sizes = [1, 7, 8, 9, 32, 128, 129, 300]
    pool, offs, rewards, gid = [], [0], [], []
    for g, n in enumerate(sizes):
        vals = rng.random(n) if g % 2 else (rng.random(n) < 0.5).astype(np.float64)
        pool.extend(vals.tolist()); offs.append(len(pool))
        rewards.extend(vals.tolist()); gid.extend([g] * n)
    pool += [0.0] * 4; offs.append(len(pool)); rewards += [0.0] * 4; gid += [len(sizes)] * 4
    pool += [1.0] * 4; offs.append(len(pool)); rewards += [1.0] * 4; gid += [len(sizes) + 1] * 4
    adv, z, o = ops.group_advantage(torch.tensor(rewards, dtype=torch.float64, device=dev),
                                    torch.tensor(gid, dtype=torch.int32, device=dev),
                                    torch.tensor(pool, dtype=torch.float64, device=dev),
                                    torch.tensor(offs, dtype=torch.int32, device=dev))
    want = np.array([(r - np.mean(pool[offs[g]:offs[g + 1]])) / (np.std(pool[offs[g]:offs[g + 1]]) + 1e-5)
                     for r, g in zip(rewards, gid)])
    got = adv.cpu().numpy()
    small = np.array([offs[g + 1] - offs[g] <= 128 for g in gid])
    bad = np.nonzero((got != want) & small)[0]
    sizes_bad = sorted({offs[gid[i] + 1] - offs[gid[i]] for i in bad})
    assert bad.size == 0, (f"{bad.size} advantages differ from numpy in pools of sizes {sizes_bad}; "
                           f"max diff {np.abs(got - want)[bad].max():.3e}")   # numpy's summation order reproduced
    assert np.allclose(got, want, rtol=1e-12, atol=1e-12)
    assert z.cpu().tolist()[-8:] == [True] * 4 + [False] * 4 and o.cpu().tolist()[-8:] == [False] * 4 + [True] * 4
    assert (got[-8:] == 0).all()


@pytest.mark.parametrize("V", [1999, 6000], ids=["odd-V-elementwise", "V-16-byte-rows"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_stats_from_logits_mirrors(dev, dtype, V):
    from chatlearn_amd.algorithm.grpo_utils import trainer_utils as tu
    g = torch.Generator().manual_seed(4)
    B, S = 2, 300
    logits = (torch.randn(B, S, V, generator=g) * 2).to(dtype)
    labels = torch.randint(0, V, (B, S), generator=g)
    z64 = logits.double()
    rt = 1e-5 if dtype == torch.float32 else 1e-2
    ld = logits.to(dev).requires_grad_(True)
    lp = tu.logprobs_from_logits(ld, labels.to(dev))
    en = tu.entropy_from_logits_with_chunking(ld)
    en2 = tu.entropy_from_logits(ld)
    assert lp.dtype == dtype and en.dtype == torch.float32 and en2.dtype == dtype and lp.shape == (B, S)
    assert_close_rel(lp, osm.logprobs_from_logits(z64, labels), rt, "logprob")
    assert_close_rel(en, osm.entropy_from_logits(z64), rt, "entropy")
    w1 = torch.randn(B, S, generator=g)
    w2 = torch.randn(B, S, generator=g) * 0.1
    ((lp.float() * w1.to(dev)).sum() + (en * w2.to(dev)).sum()).backward()
    zr = z64.clone().requires_grad_(True)
    ((osm.logprobs_from_logits(zr, labels) * w1).sum() + (osm.entropy_from_logits(zr) * w2).sum()).backward()
    assert ld.grad.dtype == dtype
    assert_close_rel(ld.grad, zr.grad, rt, "dlogits")
    # a strided view along the row dimension (what slicing logits[:, a:b] produces)
    part = ld.detach()[:, 10:50]
    assert_close_rel(tu.entropy_from_logits_with_chunking(part), osm.entropy_from_logits(z64[:, 10:50]), rt, "slice")
    # a view whose rows are wider than the vocabulary slice it exposes (row stride > V), and the backward
    # without the forward's statistics (the kernel rebuilds them) giving the same d(logits)
    from chatlearn_amd import ops
    wide = ld.detach().reshape(B * S, V)
    half = wide[:, : (V // 16) * 8]
    lp_h, en_h, lse_h = ops.softmax_stats(half, labels.reshape(-1).to(dev) % half.shape[1])
    assert_close_rel(en_h, osm.entropy_from_logits(z64.reshape(B * S, V)[:, : half.shape[1]]), rt, "strided rows")
    gl = w1.reshape(-1).to(dev)
    ge = w2.reshape(-1).to(dev)
    lab_h = labels.reshape(-1).to(dev) % half.shape[1]
    d_with = ops.softmax_stats_backward(half, lab_h, gl, ge, lse=lse_h, entropy=en_h)
    d_without = ops.softmax_stats_backward(half, lab_h, gl, ge)
    assert_close_rel(d_with, d_without, 1e-5 if dtype == torch.float32 else 2 ** -7, "backward with / without kept statistics")


def test_stats_from_logits_with_masked_vocabulary_entries(dev):
    """Rows whose leading (or scattered) entries are -inf, as a vocabulary mask produces them: those entries
    contribute nothing to lse and logprob (torch's logsumexp semantics).  The entropy of such a row is NaN in
    the reference's formula (softmax * logits has 0 * -inf terms, trainer_utils.py:76-80) and NaN here."""
    from chatlearn_amd import ops
    g = torch.Generator().manual_seed(9)
    R, V = 37, 4096
    z = torch.randn(R, V, generator=g) * 3
    z[:20, :2100] = float("-inf")                   # every thread's first pieces are all -inf
    z[5, 3000:3500] = float("-inf")
    labels = torch.randint(2100, 3000, (R,), generator=g)
    lp, ent, lse = ops.softmax_stats(z.to(dev), labels.to(dev))
    z64 = z.double()
    want_lse = torch.logsumexp(z64, dim=-1)
    want_ent = want_lse - (torch.softmax(z64, dim=-1) * z64).sum(-1)       # the reference's expression
    assert torch.isfinite(lse).all()
    assert_close_rel(lse, want_lse, 1e-5, "lse")
    assert_close_rel(lp, z64.gather(1, labels[:, None])[:, 0] - want_lse, 1e-5, "logprob")
    assert torch.equal(torch.isnan(ent).cpu(), torch.isnan(want_ent)) and int(torch.isnan(want_ent).sum()) == 20
    assert_close_rel(ent[20:], want_ent[20:], 1e-5, "entropy of the unmasked rows")
