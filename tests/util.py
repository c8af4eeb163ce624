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
