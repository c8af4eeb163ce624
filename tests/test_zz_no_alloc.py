"""clgrpo_policy_loss_static, the entry point that allocates nothing (its scratch memory is an array
built into the library), against clgrpo_policy_loss on identical inputs: same bits in every output,
on two calls in a row, the second with a smaller input.  Called through the C ABI directly."""
import ctypes as C

import pytest
import torch

from chatlearn_amd import _lib

pytestmark = pytest.mark.gpu


def _inputs(n, B, seed, dev):
    g = torch.Generator().manual_seed(seed)
    cuts = torch.sort(torch.randperm(n - 1, generator=g)[:B - 1] + 1).values
    cu = torch.cat([torch.zeros(1, dtype=torch.long), cuts, torch.tensor([n])]).to(torch.int32)
    lp = torch.randn(n, generator=g) * 0.5 - 2.0
    x = {"cu": cu, "lp": lp, "old": lp + torch.randn(n, generator=g) * 0.002, "ref": lp + torch.randn(n, generator=g) * 0.1,
         "ent": torch.rand(n, generator=g) * 3, "mask": (torch.rand(n, generator=g) < 0.7).int(),
         "adv": torch.randn(B, generator=g, dtype=torch.float64)}
    return {k: v.to(dev).contiguous() for k, v in x.items()}


def _run(entry, x, n, B, mode, with_workspace):
    dev = x["lp"].device
    f32 = dict(dtype=torch.float32, device=dev)
    out = {"loss": torch.empty(n, dtype=torch.float64, device=dev), "dloss": torch.empty(n, dtype=torch.float64, device=dev),
           "kl": torch.empty(n, **f32), "pos": torch.empty(n, dtype=torch.uint8, device=dev),
           "neg": torch.empty(n, dtype=torch.uint8, device=dev), "clip": torch.empty(n, dtype=torch.uint8, device=dev),
           "g_lp": torch.empty(n, **f32), "g_ent": torch.empty(n, **f32),
           "sums": torch.full((8,), -1.0, dtype=torch.float64, device=dev),
           "flags": torch.full((1,), -1, dtype=torch.int32, device=dev)}
    ws = None
    if with_workspace:
        ws = torch.empty(_lib.lib().clgrpo_policy_loss_workspace_bytes(n, B), dtype=torch.uint8, device=dev)
    p = lambda t: None if t is None else t.data_ptr()
    a = _lib.PolicyLossArgs(mode, _lib.F64, n, B, 0, p(x["cu"]), p(x["lp"]), p(x["old"]), p(x["ref"]), p(x["ent"]),
                            p(x["mask"]), p(x["adv"]), 10.0, 4e-4, 3e-4, 3.0, 1e-3, 1e-3, 1.0 / n, p(out["loss"]),
                            p(out["dloss"]), p(out["kl"]), p(out["pos"]), p(out["neg"]), p(out["clip"]), p(out["g_lp"]),
                            p(out["g_ent"]), p(out["sums"]), p(out["flags"]), p(ws), ws.numel() if ws is not None else 0, 0)
    stream = torch.cuda.current_stream(dev).cuda_stream
    _lib.check(getattr(_lib.lib(), entry)(C.byref(a), _lib.vp(stream or 0)))
    torch.cuda.synchronize()
    return out


def test_static_scratch_entry_point_equals_the_workspace_one_on_two_calls_in_a_row(dev):
    lib = _lib.lib()
    assert lib.clgrpo_policy_loss_static_max_sequences() == 65536
    # first call: the multi-block kernels run and both the sequence means and the per-block partial sums
    # live in the built-in scratch; second call: a smaller input (at most 4096 tokens: one workgroup,
    # sequence means only) that finds the first call's contents in the array
    for n, B, seed in ((300001, 3000, 1), (3000, 7, 2)):
        x = _inputs(n, B, seed, dev)
        for mode in (_lib.LOSS_GSPO, _lib.LOSS_GRPO):
            want = _run("clgrpo_policy_loss", x, n, B, mode, with_workspace=True)
            got = _run("clgrpo_policy_loss_static", x, n, B, mode, with_workspace=False)
            for k in want:
                assert torch.equal(got[k], want[k]), f"{k} differs (n={n}, mode={mode})"
            assert int(want["flags"]) == 0 and float(want["sums"][3]) == float(x["mask"].sum())


def test_static_scratch_entry_point_refuses_more_sequences_than_its_scratch_holds(dev):
    lib = _lib.lib()
    a = _lib.PolicyLossArgs()
    a.mode, a.compute_dtype, a.n, a.B = _lib.LOSS_GRPO, _lib.F32, 70000, 65537
    rc = lib.clgrpo_policy_loss_static(C.byref(a), None)
    assert rc == -6 and "65536" in lib.clgrpo_last_error_string().decode()
