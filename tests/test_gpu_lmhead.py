"""Fused lm_head forward / backward (HIP, through the C ABI) against the CPU oracle
on identical seeded inputs.  Tolerances: 1e-5 relative in fp32, 1e-2 relative in
bf16 (relative to the largest magnitude of the compared tensor)."""
import math
import os

import pytest
import torch

from oracle import softmax_stats as osm
from tests.util import assert_close_rel, assert_contract, assert_rows_rel_l2

pytestmark = pytest.mark.gpu

RTOL = {torch.float32: 1e-5, torch.bfloat16: 1e-2}


def _inputs(T, H, V, dtype, seed, w_std=0.05):
    g = torch.Generator().manual_seed(seed)
    hidden = torch.randn(T, H, generator=g).to(dtype)
    weight = (torch.randn(V, H, generator=g) * w_std).to(dtype)
    labels = torch.randint(0, V, (T,), generator=g)
    # make sure the edges of the vocabulary are hit
    labels[0], labels[-1] = 0, V - 1
    return hidden, weight, labels


CASES = [
    # T, H, V, dtype, temperature
    (300, 256, 5000, torch.float32, 1.0),      # ragged T and V
    (1, 64, 257, torch.float32, 1.0),          # single token, V just past one tile
    (513, 128, 1000, torch.float32, 0.7),      # temperature
    (300, 256, 5000, torch.bfloat16, 1.0),
    (700, 512, 9001, torch.bfloat16, 0.7),
    (256, 1024, 4096, torch.bfloat16, 1.0),    # exact tiles
]


@pytest.mark.parametrize("T,H,V,dtype,temp", CASES)
def test_forward_matches_oracle(dev, T, H, V, dtype, temp):
    from chatlearn_amd import ops
    hidden, weight, labels = _inputs(T, H, V, dtype, seed=T + V)
    lp, ent, mx, lse = ops.lmhead_forward(hidden.to(dev), weight.to(dev), labels.to(dev), temp, need_entropy=True)
    rlp, rent, rmx, rlse = osm.fused_head_forward(hidden, weight, labels, temp, torch.float64)
    r = RTOL[dtype]
    assert_close_rel(lp, rlp, r, "logprob")
    assert_close_rel(ent, rent, r, "entropy")
    assert_close_rel(lse, rlse, r, "lse")
    assert_close_rel(mx, rmx, r, "rowmax")
    # the contract's elementwise form |err| <= atol + rtol |ref|, atol = rtol median|ref|, on every entry
    assert_contract(lp, rlp, r, "logprob")
    assert_contract(ent, rent, r, "entropy")
    assert (lp <= 1e-6).all() and (ent >= -1e-6).all() and (ent <= math.log(V) + 1e-4).all()


@pytest.mark.parametrize("T,H,V,dtype,temp", CASES)
@pytest.mark.parametrize("with_entropy", [False, True])
def test_backward_matches_oracle(dev, T, H, V, dtype, temp, with_entropy):
    from chatlearn_amd import ops
    hidden, weight, labels = _inputs(T, H, V, dtype, seed=T + V + 1)
    g = torch.Generator().manual_seed(5)
    g_lp = torch.randn(T, generator=g)
    g_lp[torch.rand(T, generator=g) < 0.3] = 0.0          # masked-out tokens
    g_ent = torch.randn(T, generator=g) * 0.1 if with_entropy else None
    hd, wd, ld = hidden.to(dev), weight.to(dev), labels.to(dev)
    lp, ent, _, lse = ops.lmhead_forward(hd, wd, ld, temp, need_entropy=True)
    dh, dw = ops.lmhead_backward(hd, wd, ld, lse, ent, g_lp.to(dev), g_ent.to(dev) if with_entropy else None, temp)
    rdh, rdw = osm.fused_head_backward_closed_form(hidden, weight, labels, g_lp, g_ent, temp)
    r = RTOL[dtype]
    assert dh.dtype == dtype and dw.dtype == torch.float32
    assert_close_rel(dh, rdh, r, "dhidden")
    assert_close_rel(dw, rdw, r, "dweight")
    assert_rows_rel_l2(dh.float(), rdh, r, "dhidden rows")
    assert_rows_rel_l2(dw, rdw, r, "dweight rows")
    if dtype == torch.float32:
        assert_contract(dh, rdh, r, "dhidden")
        # dW entries are sums over all tokens; where the terms cancel to far below the tensor's typical
        # magnitude, fp32 accumulation (any order) is further than 1e-5 from the float64 sum: at most 4 entries in
        # 10^5 on the MI355X
        assert_contract(dw, rdw, r, "dweight", min_frac=0.9999)


def test_backward_chunked_equals_unchunked_and_accumulates(dev):
    from chatlearn_amd import ops
    T, H, V = 900, 256, 3000
    hidden, weight, labels = _inputs(T, H, V, torch.bfloat16, seed=3)
    g_lp = torch.randn(T, generator=torch.Generator().manual_seed(1))
    hd, wd, ld, gd = hidden.to(dev), weight.to(dev), labels.to(dev), g_lp.to(dev)
    lp, ent, _, lse = ops.lmhead_forward(hd, wd, ld)
    dh1, dw1 = ops.lmhead_backward(hd, wd, ld, lse, None, gd)
    dh2, dw2 = ops.lmhead_backward(hd, wd, ld, lse, None, gd, chunk_tokens=256)
    # dhidden rows do not depend on the chunking beyond the fp32 summation order (split-K differs with M)
    assert_close_rel(dh2, dh1, 2 ** -7, "chunked dhidden")
    assert_close_rel(dw2, dw1, 1e-5, "chunked dW")   # only the fp32 summation order differs
    base = torch.ones(V, H, device=dev)
    _, dw3 = ops.lmhead_backward(hd, wd, ld, lse, None, gd, dweight=base, accumulate_dweight=True)
    assert dw3.data_ptr() == base.data_ptr()
    assert_close_rel(dw3 - 1.0, dw1, 1e-4, "accumulated dW")


def test_closed_forms(dev):
    """Uniform logits: lp = -log V, entropy = log V.  One dominant logit: lp -> 0, entropy -> 0."""
    from chatlearn_amd import ops
    T, H, V = 64, 64, 777
    hidden = torch.zeros(T, H, device=dev)
    weight = torch.randn(V, H, device=dev)
    labels = torch.randint(0, V, (T,), device=dev)
    lp, ent, _, lse = ops.lmhead_forward(hidden, weight, labels)
    assert torch.allclose(lp, torch.full_like(lp, -math.log(V)), atol=1e-5)
    assert torch.allclose(ent, torch.full_like(ent, math.log(V)), atol=1e-5)
    hidden = torch.zeros(T, H, device=dev)
    hidden[:, 0] = 1.0
    weight = torch.zeros(V, H, device=dev)
    weight[5, 0] = 60.0
    labels = torch.full((T,), 5, device=dev)
    lp, ent, _, _ = ops.lmhead_forward(hidden, weight, labels)
    assert lp.abs().max() < 1e-5 and ent.abs().max() < 1e-5


def test_autograd_function_matches_oracle_autograd(dev):
    from chatlearn_amd import fused_linear_logprob_entropy
    T, H, V = 260, 128, 1500
    hidden, weight, labels = _inputs(T, H, V, torch.float32, seed=11)
    h = hidden.to(dev).requires_grad_(True)
    w = weight.to(dev).requires_grad_(True)
    lp, ent = fused_linear_logprob_entropy(h.view(2, 130, H), w, labels.to(dev).view(2, 130), temperature=0.9)
    assert lp.shape == (2, 130) and ent.shape == (2, 130)
    g = torch.Generator().manual_seed(2)
    c_lp, c_ent = torch.randn(T, generator=g), torch.randn(T, generator=g)
    ((lp.reshape(-1) * c_lp.to(dev)).sum() + (ent.reshape(-1) * c_ent.to(dev)).sum()).backward()
    rdh, rdw = osm.fused_head_backward_autograd(hidden, weight, labels, c_lp, c_ent, 0.9)
    assert_close_rel(h.grad, rdh, 1e-5, "hidden.grad")
    assert_close_rel(w.grad, rdw, 1e-5, "weight.grad")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_autograd_kept_logits_mask_hint_and_second_backward(dev, dtype):
    """The seam keeps its logits for the backward by default; with the loss mask as a hint it keeps
    and back-propagates only the unmasked rows.  Both must give the gradients of the recomputing
    path, and a second backward through a retained graph (logits already consumed) must too."""
    from chatlearn_amd import fused_linear_logprob_entropy
    T, H, V = 300, 128, 2100
    hidden, weight, labels = _inputs(T, H, V, dtype, seed=13)
    g = torch.Generator().manual_seed(3)
    mask = (torch.rand(T, generator=g) < 0.6).to(torch.int32)
    c_lp = torch.randn(T, generator=g) * mask
    c_ent = torch.randn(T, generator=g) * 0.1 * mask

    def grads(retain=False, **kw):
        h = hidden.to(dev).requires_grad_(True)
        w = weight.to(dev).requires_grad_(True)
        lp, ent = fused_linear_logprob_entropy(h, w, labels.to(dev), temperature=0.8, **kw)
        loss = (lp * c_lp.to(dev)).sum() + (ent * c_ent.to(dev)).sum()
        loss.backward(retain_graph=retain)
        first = (h.grad.clone(), w.grad.clone())
        if retain:
            h.grad = w.grad = None
            loss.backward()
            return first, (h.grad, w.grad)
        return first

    ref_h, ref_w = grads(keep_logits_rows=None)                        # recompute in the backward
    rdh, rdw = osm.fused_head_backward_closed_form(hidden, weight, labels, c_lp, c_ent, 0.8)
    r = RTOL[dtype]
    assert_close_rel(ref_h, rdh, r, "recompute dh")
    cases = (("kept", {}), ("kept + mask hint", dict(loss_mask=mask.to(dev))),
             ("kept + host mask", dict(loss_mask_host=mask)),
             # more rows carry a gradient than may be kept: the first ones run from kept logits, the rest are
             # recomputed, and both parts add into one dW
             ("100 of 300 rows kept, no mask", dict(keep_logits_rows=100)),
             ("64 unmasked rows kept, the others recomputed", dict(keep_logits_rows=64, loss_mask=mask.to(dev))),
             ("64 kept, host mask", dict(keep_logits_rows=64, loss_mask_host=mask)),
             ("256 kept (one block), no mask", dict(keep_logits_rows=256)),
             ("nothing kept, host mask: only the unmasked rows are recomputed", dict(keep_logits_rows=None, loss_mask_host=mask)))
    assert int(mask.sum()) > 64
    for name, kw in cases:
        gh, gw = grads(**kw)
        assert_close_rel(gh, rdh, r, name + " dh")
        assert_close_rel(gw, rdw, r, name + " dW")
        if "mask" in name:
            assert (gh[mask.to(dev) == 0] == 0).all(), name
    # the hybrid with a caller's fp32 gradient buffer: both parts add to what it held
    main_grad = torch.full((V, H), 0.5, device=dev)
    h = hidden.to(dev).requires_grad_(True)
    w = weight.to(dev).requires_grad_(True)
    lp, ent = fused_linear_logprob_entropy(h, w, labels.to(dev), temperature=0.8, keep_logits_rows=64,
                                           loss_mask_host=mask, dweight_buffer=main_grad)
    ((lp * c_lp.to(dev)).sum() + (ent * c_ent.to(dev)).sum()).backward()
    assert w.grad is None
    assert_close_rel(main_grad - 0.5, rdw, r, "hybrid dW added to the main-grad buffer")
    with pytest.raises(ValueError, match="entries"):
        fused_linear_logprob_entropy(h, w, labels.to(dev), loss_mask_host=mask[:-1])
    (h1, w1), (h2, w2) = grads(retain=True, loss_mask=mask.to(dev))
    assert_close_rel(h2, rdh, r, "second backward dh")
    assert_close_rel(w2, rdw, r, "second backward dW")
    assert (h1[mask.to(dev) == 0] == 0).all()                          # masked rows get exactly zero
    # no gradient needed: nothing is kept, results identical
    with torch.no_grad():
        lp0, _ = fused_linear_logprob_entropy(hidden.to(dev), weight.to(dev), labels.to(dev), temperature=0.8)
    lp1, _ = fused_linear_logprob_entropy(hidden.to(dev).requires_grad_(True), weight.to(dev), labels.to(dev),
                                          temperature=0.8)
    assert torch.equal(lp0, lp1.detach())


def test_argument_errors(dev):
    from chatlearn_amd import ops
    from chatlearn_amd._lib import ClgrpoError
    h = torch.zeros(4, 48, device=dev)
    w = torch.zeros(10, 48, device=dev)
    with pytest.raises(ClgrpoError, match="ESHAPE"):
        ops.lmhead_forward(h, w, torch.zeros(4, dtype=torch.int64, device=dev))
    with pytest.raises(RuntimeError, match="GPU"):
        ops.lmhead_forward(torch.zeros(4, 64), torch.zeros(10, 64), None)
    # a label outside the vocabulary is flagged with NaN instead of a silent number
    h = torch.randn(4, 64, device=dev)
    w = torch.randn(10, 64, device=dev)
    lp, *_ = ops.lmhead_forward(h, w, torch.tensor([0, 9, 10, -1], device=dev))
    assert torch.isfinite(lp[:2]).all() and torch.isnan(lp[2:]).all()


@pytest.mark.parametrize("T,V", [(200, 16400), (1100, 16400), (1500, 16900), (1500, 20000)])
def test_backward_weight_gradient_with_walking_workgroups(dev, T, V):
    """A weight-gradient GEMM with many more 256 x 256 tiles than CUs runs with workgroups that walk
    runs of tiles (consecutive K loops streaming into each other); ragged V and T edges included, with and
    without the second launch over left-over tile rows (whose last tile holds 16 or 4 valid rows)."""
    from chatlearn_amd import ops
    H = 4096
    n_walk, bulk, ks = ops.dweight_launch_plan(T, H, V, torch.bfloat16)
    assert n_walk == 16
    # 65 and 67 vocabulary tiles: 64 walked in runs of 4, the last 1 or 3 tile rows cut into K ranges when the chunk is
    # long enough for that; 79 tiles: the 15 left-over tile rows fill most CUs, no second launch
    assert (bulk, ks) == {(200, 16400): (0, 1), (1100, 16400): (64, 2), (1500, 16900): (64, 3), (1500, 20000): (0, 1)}[(T, V)]
    hidden, weight, labels = _inputs(T, H, V, torch.bfloat16, seed=9, w_std=0.02)
    g = torch.Generator().manual_seed(6)
    g_lp = torch.randn(T, generator=g)
    g_ent = torch.randn(T, generator=g) * 0.1
    hd, wd, ld = hidden.to(dev), weight.to(dev), labels.to(dev)
    lp, ent, _, lse = ops.lmhead_forward(hd, wd, ld, 1.0)
    dh, dw = ops.lmhead_backward(hd, wd, ld, lse, ent, g_lp.to(dev), g_ent.to(dev), 1.0)
    rdh, rdw = osm.fused_head_backward_closed_form(hidden, weight, labels, g_lp, g_ent, 1.0)
    assert_close_rel(dh, rdh, 1e-2, "dhidden")
    assert_close_rel(dw, rdw, 1e-2, "dweight")
    # accumulate into an existing fp32 buffer
    base = torch.randn(V, H, generator=g)
    acc = base.clone().to(dev)
    ops.lmhead_backward(hd, wd, ld, lse, ent, g_lp.to(dev), g_ent.to(dev), 1.0, need_dhidden=False, dweight=acc,
                        accumulate_dweight=True)
    assert_close_rel(acc - base.to(dev), rdw, 1e-2, "accumulated dweight")


EDGE_SHAPES = [
    # T, H, V, dtype: tile edges in every dimension (tokens around 256, vocabulary around 32 / 64 / 256, the smallest H)
    (2, 64, 33, torch.bfloat16), (255, 64, 63, torch.bfloat16), (257, 128, 64, torch.bfloat16),
    (511, 64, 65, torch.bfloat16), (64, 192, 255, torch.bfloat16), (769, 64, 513, torch.bfloat16),
    (3, 32, 31, torch.float32), (256, 32, 256, torch.float32), (258, 96, 289, torch.float32),
]


@pytest.mark.parametrize("T,H,V,dtype", EDGE_SHAPES)
def test_edge_shapes_forward_and_both_backward_routes(dev, T, H, V, dtype):
    """Shapes that end inside a tile in every dimension: forward against the oracle, then the backward twice -
    recomputing the logit tiles, and from logits the forward kept - against the oracle's closed form."""
    from chatlearn_amd import ops
    hidden, weight, labels = _inputs(T, H, V, dtype, seed=7 * T + V, w_std=0.2)
    g = torch.Generator().manual_seed(T)
    g_lp, g_ent = torch.randn(T, generator=g), torch.randn(T, generator=g) * 0.1
    g_lp[::3] = 0.0
    hd, wd, ld = hidden.to(dev), weight.to(dev), labels.to(dev)
    r = RTOL[dtype]
    rlp, rent, _, rlse = osm.fused_head_forward(hidden, weight, labels, 1.0, torch.float64)
    rdh, rdw = osm.fused_head_backward_closed_form(hidden, weight, labels, g_lp, g_ent, 1.0)
    zbuf = ops.saved_logits_buffer(T, V, dtype, dev)
    for saved in (None, zbuf):
        lp, ent, _, lse = ops.lmhead_forward(hd, wd, ld, 1.0, need_entropy=True, saved_logits=saved)
        assert_close_rel(lp, rlp, r, "logprob")
        assert_close_rel(ent, rent, r, "entropy")
        assert_close_rel(lse, rlse, r, "lse")
        if saved is not None:
            z = ops.saved_logits_rowmajor(saved, T, V).double().cpu()
            assert_close_rel(z, hidden.double() @ weight.double().t(), 2 ** -10 if dtype != torch.float32 else 1e-5, "kept logits")
        dh, dw = ops.lmhead_backward(hd, wd, ld, lse, ent, g_lp.to(dev), g_ent.to(dev), 1.0, saved_logits=saved)
        route = "kept logits" if saved is not None else "recompute"
        assert_close_rel(dh, rdh, r, f"dhidden ({route})")
        assert_close_rel(dw, rdw, r, f"dweight ({route})")
        assert torch.isfinite(dh.float()).all() and torch.isfinite(dw).all()


def test_backward_option_combinations_agree(dev):
    """The backward's routes and options on one input: recompute or kept logits, one pass or token chunks,
    the caller's W^T buffer (fresh, then marked ready), dW written or added to.  All must give the gradients
    of the plain call (up to the fp32 summation order and, for kept logits, the half rounding of the logits)."""
    from chatlearn_amd import ops
    T, H, V = 1100, 192, 2500
    hidden, weight, labels = _inputs(T, H, V, torch.bfloat16, seed=21, w_std=0.1)
    g = torch.Generator().manual_seed(22)
    g_lp, g_ent = torch.randn(T, generator=g), torch.randn(T, generator=g) * 0.1
    g_lp[::4] = 0.0
    hd, wd, ld, gl, ge = hidden.to(dev), weight.to(dev), labels.to(dev), g_lp.to(dev), g_ent.to(dev)
    lp, ent, _, lse = ops.lmhead_forward(hd, wd, ld)
    dh0, dw0 = ops.lmhead_backward(hd, wd, ld, lse, ent, gl, ge)
    wt = ops.weight_t_buffer(wd)
    wt_ready = False
    for saved in (False, True):
        for chunk in (None, 256, 512):
            for accumulate in (False, True):
                zbuf = None
                if saved:
                    zbuf = ops.saved_logits_buffer(T, V, torch.bfloat16, dev)
                    ops.lmhead_forward(hd, wd, ld, saved_logits=zbuf)
                base = torch.full((V, H), 0.5, device=dev) if accumulate else None
                dh, dw = ops.lmhead_backward(hd, wd, ld, lse, ent, gl, ge, chunk_tokens=chunk, saved_logits=zbuf,
                                             weight_t=wt, weight_t_ready=wt_ready, dweight=base,
                                             accumulate_dweight=accumulate)
                wt_ready = True
                what = f"saved={saved} chunk={chunk} accumulate={accumulate}"
                assert_close_rel(dh, dh0, 2 ** -6, "dhidden " + what)
                assert_close_rel(dw - 0.5 if accumulate else dw, dw0, 2 ** -8, "dweight " + what)
    assert_close_rel(ops.weight_t_rowmajor(wt, H, V), wd.t().float(), 0.0, "W^T left in the caller's buffer")


@pytest.mark.parametrize("V", [777, 2100, 2500])
@pytest.mark.parametrize("accumulate", [False, True])
@pytest.mark.parametrize("saved", [False, True])
def test_weight_gradient_never_touches_memory_past_its_last_row(dev, V, accumulate, saved):
    """dW [V,H] handed in as the front of a larger buffer whose remainder holds a sentinel: a vocabulary that
    ends inside a 256-row tile (and not on a multiple of 8 rows) must leave every byte after row V alone,
    whether the GEMM writes dW or adds to it, and on both backward routes."""
    from chatlearn_amd import ops
    T, H = 520, 128
    hidden, weight, labels = _inputs(T, H, V, torch.bfloat16, seed=V, w_std=0.1)
    g_lp = torch.randn(T, generator=torch.Generator().manual_seed(V + 1))
    hd, wd, ld, gd = hidden.to(dev), weight.to(dev), labels.to(dev), g_lp.to(dev)
    guard_rows = 300                                   # more than one whole tile of rows behind the tensor
    sentinel = 1234.5
    buf = torch.full(((V + guard_rows) * H,), sentinel, device=dev)
    dw_view = buf[:V * H].view(V, H)
    if accumulate:
        dw_view.fill_(0.25)
    zbuf = ops.saved_logits_buffer(T, V, torch.bfloat16, dev) if saved else None
    lp, ent, _, lse = ops.lmhead_forward(hd, wd, ld, saved_logits=zbuf)
    _, dw = ops.lmhead_backward(hd, wd, ld, lse, None, gd, need_dhidden=False, dweight=dw_view,
                                accumulate_dweight=accumulate, saved_logits=zbuf)
    torch.cuda.synchronize()
    assert dw.data_ptr() == buf.data_ptr()
    assert (buf[V * H:] == sentinel).all(), "the weight-gradient GEMM wrote past row V"
    _, rdw = osm.fused_head_backward_closed_form(hidden, weight, labels, g_lp, None, 1.0)
    assert_close_rel(dw - 0.25 if accumulate else dw, rdw, 1e-2, "dweight")


def test_split_k_partials_stay_inside_their_buffer_and_many_ranges_agree(dev):
    """A dhidden GEMM with few output tiles and a long K (the vocabulary) is cut into many K ranges; the
    result must equal the oracle, and ragged T (the partial tiles' row count) must not disturb it."""
    from chatlearn_amd import ops
    for T, H, V, dtype in ((333, 256, 40000, torch.bfloat16), (130, 64, 30011, torch.float32)):
        hidden, weight, labels = _inputs(T, H, V, dtype, seed=T, w_std=0.05)
        g_lp = torch.randn(T, generator=torch.Generator().manual_seed(T + 2))
        hd, wd, ld = hidden.to(dev), weight.to(dev), labels.to(dev)
        lp, ent, _, lse = ops.lmhead_forward(hd, wd, ld)
        dh, dw = ops.lmhead_backward(hd, wd, ld, lse, None, g_lp.to(dev))
        rdh, rdw = osm.fused_head_backward_closed_form(hidden, weight, labels, g_lp, None, 1.0)
        assert_close_rel(dh, rdh, RTOL[dtype], "dhidden (split K)")
        assert_rows_rel_l2(dh.float(), rdh, RTOL[dtype], "dhidden rows (split K)")
        assert_close_rel(dw, rdw, RTOL[dtype], "dweight")


def test_kept_logits_beyond_the_half_range_stay_finite(dev):
    """Kept logits of 16-bit inputs are IEEE half.  A raw logit past the half range (|z| > 65504) is kept as
    the largest half instead of infinity, so the gradients the backward rebuilds from the kept logits stay
    finite; every other token's gradient equals the recomputing route's (the saturated token's own
    probabilities are formed from the saturated value and are not compared)."""
    from chatlearn_amd import ops
    T, H, V = 64, 64, 300
    g = torch.Generator().manual_seed(8)
    hidden = torch.randn(T, H, generator=g).bfloat16()
    weight = (torch.randn(V, H, generator=g) * 0.1).bfloat16()
    hidden[:, 0] = 0.0             # only token 3 reaches the two huge weight entries below
    hidden[3, :] = 0.0
    hidden[3, 0] = 300.0
    weight[7, 0] = 300.0           # z[3, 7] = 90000 > 65504
    weight[9, 0] = -300.0          # z[3, 9] = -90000
    labels = torch.randint(0, V, (T,), generator=g)
    labels[3] = 7
    hd, wd, ld = hidden.to(dev), weight.to(dev), labels.to(dev)
    g_lp = torch.randn(T, generator=g).to(dev)
    zbuf = ops.saved_logits_buffer(T, V, torch.bfloat16, dev)
    lp, ent, _, lse = ops.lmhead_forward(hd, wd, ld, saved_logits=zbuf)
    z = ops.saved_logits_rowmajor(zbuf, T, V)
    assert torch.isfinite(z).all()
    assert float(z[3, 7]) == 65504.0 and float(z[3, 9]) == -65504.0
    dh, dw = ops.lmhead_backward(hd, wd, ld, lse, None, g_lp, saved_logits=zbuf)
    assert torch.isfinite(dh.float()).all() and torch.isfinite(dw).all()
    dh0, dw0 = ops.lmhead_backward(hd, wd, ld, lse, None, g_lp)
    others = [t for t in range(T) if t != 3]
    assert_close_rel(dh[others], dh0[others], 2 ** -6, "dhidden of the other tokens, kept against recomputed")
    # token 3's hidden row is zero outside column 0, so it reaches dW through that column only
    assert_close_rel(dw[:, 1:], dw0[:, 1:], 2 ** -6, "dweight outside the saturated token's column")


def _random_shapes(n, seed):
    """Seeded shapes that end anywhere inside a tile: tokens 1..1400, vocabulary 2..3300, H a multiple of the slab."""
    import random
    rnd = random.Random(seed)
    out = []
    for i in range(n):
        dtype = torch.bfloat16 if i % 3 else torch.float32
        slab = 64 if dtype == torch.bfloat16 else 32
        out.append((rnd.randint(1, 1400), slab * rnd.randint(1, 6), rnd.randint(2, 3300), dtype,
                    rnd.choice([1.0, 0.6, 1.7]), rnd.choice([None, 256, 512]), rnd.random() < 0.5))
    return out


@pytest.mark.parametrize("T,H,V,dtype,temp,chunk,with_entropy",
                         _random_shapes(int(os.environ.get("CLGRPO_FUZZ_CASES", "14")), seed=2024))   # more cases on request
def test_random_shapes_both_backward_routes(dev, T, H, V, dtype, temp, chunk, with_entropy):
    """Random shapes, temperatures, chunkings and gradient masks: forward and both backward routes against the
    oracle's float64 closed form, to the tolerance of the dtype."""
    from chatlearn_amd import ops
    hidden, weight, labels = _inputs(T, H, V, dtype, seed=T * 31 + V, w_std=0.15)
    g = torch.Generator().manual_seed(T + H + V)
    g_lp = torch.randn(T, generator=g)
    g_lp[torch.rand(T, generator=g) < 0.4] = 0.0
    g_ent = torch.randn(T, generator=g) * 0.1 if with_entropy else None
    if with_entropy:
        g_ent[g_lp == 0] = 0.0          # a masked token carries neither gradient
    hd, wd, ld = hidden.to(dev), weight.to(dev), labels.to(dev)
    r = RTOL[dtype]
    rlp, rent, _, rlse = osm.fused_head_forward(hidden, weight, labels, temp, torch.float64)
    rdh, rdw = osm.fused_head_backward_closed_form(hidden, weight, labels, g_lp, g_ent, temp)
    zbuf = ops.saved_logits_buffer(T, V, dtype, dev)
    for saved in (None, zbuf):
        lp, ent, _, lse = ops.lmhead_forward(hd, wd, ld, temp, need_entropy=True, saved_logits=saved)
        assert_close_rel(lp, rlp, r, "logprob")
        assert_close_rel(ent, rent, r, "entropy")
        # the kept-logits route transforms the whole buffer in one go: chunking applies to the recompute route
        dh, dw = ops.lmhead_backward(hd, wd, ld, lse, ent, g_lp.to(dev), g_ent.to(dev) if with_entropy else None, temp,
                                     saved_logits=saved, chunk_tokens=chunk if saved is None else None)
        route = "kept logits" if saved is not None else "recompute"
        assert_close_rel(dh, rdh, r, f"dhidden ({route})")
        assert_close_rel(dw, rdw, r, f"dweight ({route})")
        assert (dh[g_lp.to(dev) == 0] == 0).all(), "rows without a gradient get an exactly zero dhidden"
