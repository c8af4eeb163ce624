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


def oracle_head_step(hidden, weight, labels, old, ref, adv, cu, mask, *, n_tok, temperature=1.0, kl_coef=0.0,
                     entropy_coef=0.0, gspo=False, pos=0.2, neg=0.2, diff=10, final=3, dtype=torch.float64):
    """The reference's micro-batch loop body (policy_trainer.py:216-286) on a packed row, restated with
    the oracle: fp64 head, re-padding to [B,S], reference loss assembly, autograd to hidden and W."""
    from oracle import indexing as oi
    from oracle import losses as ol
    from oracle import softmax_stats as osm
    h = hidden.to(dtype).detach().requires_grad_(True)
    w = weight.to(dtype).detach().requires_grad_(True)
    z = torch.nn.functional.linear(h, w) / temperature
    lp = osm.logprobs_from_logits(z, labels)
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
    return {"logprob": lp.detach(), "entropy": ent.detach(), "total_loss": total.detach(), "parts": parts,
            "dhidden": h.grad, "dweight": w.grad}
