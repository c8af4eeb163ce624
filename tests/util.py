"""Shared helpers for the parity tests."""
import torch


def assert_close_rel(got, want, rtol, what=""):
    """|got - want| <= rtol * max(|want|) elementwise-max: a relative bound scaled by the
    tensor's own magnitude, so entries near zero do not make the test meaningless."""
    got = got.detach().double().cpu()
    want = want.detach().double().cpu()
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    assert torch.isfinite(got).all(), f"{what}: non-finite values"
    scale = want.abs().max().clamp_min(1e-30)
    err = (got - want).abs().max()
    assert err <= rtol * scale, f"{what}: max err {err:.3e} > {rtol:.1e} * {scale:.3e}"
    return float(err / scale)


def contract_report(got, want, rtol):
    """The tolerance contract of this path, elementwise: |got - want| <= atol + rtol * |want| with
    atol = rtol * median|want| (the median over the entries of ``want`` that are not exactly zero, so
    that a tensor that is mostly structural zeros - masked rows - does not get atol = 0 for its live
    part).  Returns the fraction of entries inside the bound and the worst absolute / relative errors
    (relative ones over entries with |want| > atol / rtol, i.e. above the median).  Runs where ``want``
    lives, so full-size tensors stay on the device."""
    want = want.detach().double()
    got = got.detach().to(want.device).double()
    assert got.shape == want.shape, f"shape {tuple(got.shape)} vs {tuple(want.shape)}"
    a = want.abs().flatten()
    nz = a[a > 0]
    med = float(nz.float().median()) if nz.numel() else 0.0
    atol = rtol * med
    err = (got - want).abs().flatten()
    inside = err <= atol + rtol * a
    big = a > med
    rel = (err[big] / a[big]) if bool(big.any()) else err.new_zeros(1)
    return {"frac_within": float(inside.double().mean()) if a.numel() else 1.0, "atol": atol,
            "max_abs_err": float(err.max()) if a.numel() else 0.0,
            "max_rel_err_above_median": float(rel.max()), "median_abs_ref": med, "n": int(a.numel()),
            "finite": bool(torch.isfinite(got).all())}


def assert_contract(got, want, rtol, what="", min_frac=1.0):
    """Every entry (or at least ``min_frac`` of them) inside |got - want| <= atol + rtol * |want|,
    atol = rtol * median|want|.  Prints the report (max abs / max rel error against the oracle)."""
    r = contract_report(got, want, rtol)
    print(f"[parity] {what}: within {r['frac_within']:.6f} of {r['n']} entries at rtol {rtol:g} (atol {r['atol']:.3e}), "
          f"max abs err {r['max_abs_err']:.3e}, max rel err above the median {r['max_rel_err_above_median']:.3e}")
    assert r["finite"], f"{what}: non-finite values"
    assert r["frac_within"] >= min_frac, (f"{what}: only {r['frac_within']:.6f} of the entries are within "
                                          f"atol {r['atol']:.3e} + {rtol:g} * |ref| (need {min_frac})")
    return r


def assert_rows_rel_l2(got, want, rtol, what=""):
    """Per-row relative L2 error: ||got_r - want_r|| <= rtol * (||want_r|| + median row norm).  A row's
    own magnitude sets its scale, so a few large rows cannot hide errors in the others."""
    want = want.detach().double()
    got = got.detach().to(want.device).double()
    assert got.shape == want.shape and want.dim() == 2, f"{what}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    wn = want.norm(dim=1)
    en = (got - want).norm(dim=1)
    nz = wn[wn > 0]
    med = nz.float().median().double() if nz.numel() else wn.new_zeros(())
    ratio = en / (wn + med).clamp_min(1e-300)
    worst = float(ratio.max()) if ratio.numel() else 0.0
    print(f"[parity] {what}: worst row-relative L2 error {worst:.3e} (bound {rtol:g})")
    assert worst <= rtol, f"{what}: row {int(ratio.argmax())} has relative L2 error {worst:.3e} > {rtol:g}"
    return worst


def oracle_head_step(hidden, weight, labels, old, ref, adv, cu, mask, *, n_tok, temperature=1.0, kl_coef=0.0,
                     entropy_coef=0.0, gspo=False, pos=0.2, neg=0.2, diff=10, final=3, dtype=torch.float64,
                     logprob_values=None):
    """The reference's micro-batch loop body (policy_trainer.py:216-286) on a packed row, restated with
    the oracle: fp64 head, re-padding to [B,S], reference loss assembly, autograd to hidden and W."""
    from oracle import indexing as oi
    from oracle import losses as ol
    from oracle import softmax_stats as osm
    h = hidden.to(dtype).detach().requires_grad_(True)
    w = weight.to(dtype).detach().requires_grad_(True)
    z = torch.nn.functional.linear(h, w) / temperature
    lp = osm.logprobs_from_logits(z, labels)
    lp_exact = lp.detach()
    if logprob_values is not None:
        # The loss stage reads these values (e.g. the kernel's own fp32 logprob) while the gradient still
        # flows through the oracle's float64 graph: every clip decision is then made on identical inputs.
        lp = lp + (logprob_values.to(dtype) - lp).detach()
    ent = osm.entropy_from_logits(z)
    lens = (cu[1:] - cu[:-1]).long()
    B, S = lens.numel(), int(lens.max())
    attn = (torch.arange(S).unsqueeze(0) < lens.unsqueeze(1))
    idx = torch.nonzero(attn.flatten(), as_tuple=False).flatten()
    pad = lambda x: oi.pad_input(x.unsqueeze(-1), idx, B, S).squeeze(-1)
    total, parts = ol.fsdp_policy_loss(pad(lp), pad(ent), pad(old.to(dtype)), pad(ref.to(dtype)), adv.to(dtype).tolist(),
                                       pad(mask), n_tok, entropy_coef=entropy_coef, kl_coef=kl_coef,
                                       pos_clip_ratio=pos, neg_clip_ratio=neg, diff_clip_ratio=diff,
                                       final_clip_ratio=final, use_group_sequence_policy=gspo)
    total.backward()
    return {"logprob": lp_exact, "entropy": ent.detach(), "total_loss": total.detach(), "parts": parts,
            "dhidden": h.grad, "dweight": w.grad}
