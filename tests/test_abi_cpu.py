"""The C-ABI library loads, exports every symbol include/clgrpo.h declares, and
rejects bad arguments before any launch (so these run without a GPU)."""
import ctypes as C
import os
import re

import pytest

from chatlearn_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "clgrpo.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(clgrpo_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound(lib):
    names = _declared()
    assert len(names) >= 19
    for n in names:
        assert hasattr(lib, n), f"{n} declared in clgrpo.h but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature"
    assert sorted(_lib.SIGNATURES) == names
    assert lib.clgrpo_version() >= 100


def test_struct_sizes_match_header_layout():
    # 64-bit pointers and int64 fields, natural alignment
    assert C.sizeof(_lib.LmheadFwdArgs) == 3 * 8 + 3 * 8 + 4 + 4 + 4 * 8 + 8 + 8 + 8 + 8 + 8 + 8
    assert C.sizeof(_lib.LmheadBwdArgs) == 7 * 8 + 3 * 8 + 4 + 4 + 2 * 8 + 8 + 8 + 8 + 8 + 8 + 8 + 8 + 8
    assert C.sizeof(_lib.RowsArgs) == 6 * 8
    assert C.sizeof(_lib.MaskedSumsArgs) == 8 + 8 + 16 * 8 + 16 * 4 + 16 * 4 + 3 * 8


def _err(lib):
    return lib.clgrpo_last_error_string().decode()


def test_validation_before_launch(lib):
    a = _lib.LmheadFwdArgs()
    assert lib.clgrpo_lmhead_fwd(C.byref(a), None) == -1 and "positive" in _err(lib)      # EINVAL: T=H=V=0
    a.T, a.H, a.V, a.dtype = 8, 100, 50, _lib.BF16
    assert lib.clgrpo_lmhead_fwd(C.byref(a), None) == -3 and "multiple of 64" in _err(lib)  # ESHAPE
    a.H, a.dtype = 128, 7
    assert lib.clgrpo_lmhead_fwd(C.byref(a), None) == -2                                     # EDTYPE
    a.dtype = _lib.BF16
    assert lib.clgrpo_lmhead_fwd(C.byref(a), None) == -4 and "hidden" in _err(lib)          # ENULL
    assert lib.clgrpo_lmhead_fwd(None, None) == -4
    # one 16-byte record per token and vocabulary split, at most 64 splits whatever the device's CU count
    assert lib.clgrpo_lmhead_fwd_workspace_bytes(16384, 4096, 151936, _lib.BF16) == 64 * 16384 * 16
    assert lib.clgrpo_lmhead_fwd_workspace_bytes(100, 128, 700, _lib.BF16) == 3 * 100 * 16          # 3 vocabulary tiles
    wt_kept = lib.clgrpo_lmhead_bwd_workspace_bytes(1024, 128, 1000, _lib.BF16, 0, 3)
    b = _lib.LmheadBwdArgs()
    b.T, b.H, b.V, b.dtype = 8, 128, 50, _lib.F32
    assert lib.clgrpo_lmhead_bwd(C.byref(b), None) == -4
    full = lib.clgrpo_lmhead_bwd_workspace_bytes(1024, 128, 1000, _lib.BF16, 0, 0)
    half = lib.clgrpo_lmhead_bwd_workspace_bytes(1024, 128, 1000, _lib.BF16, 512, 0)
    saved = lib.clgrpo_lmhead_bwd_workspace_bytes(1024, 128, 1000, _lib.BF16, 0, 1)
    assert 0 < half < full and saved == full - 1024 * 1024 * 2   # minus the [T][ld] d(logits) buffer
    assert wt_kept == saved - 256 * 1024 * 2                       # minus the workspace's own W^T (H rounded up to 256 rows)
    assert lib.clgrpo_saved_logits_ld(151936) == 151936 and lib.clgrpo_saved_logits_ld(1000) == 1024
    p = _lib.PolicyLossArgs()
    p.mode = 5
    assert lib.clgrpo_policy_loss(C.byref(p), None) == -1
    p.mode, p.compute_dtype, p.n, p.B, p.S = 0, _lib.F32, 10, 3, 4
    assert lib.clgrpo_policy_loss(C.byref(p), None) == -3 and "B*S" in _err(lib)
    r = _lib.RowsArgs()
    r.n_idx, r.row_bytes = 4, 8
    assert lib.clgrpo_gather_rows(C.byref(r), None) == -4
    u = _lib.UnpadIndicesArgs()
    assert lib.clgrpo_unpad_indices(C.byref(u), None) == -1
    assert lib.clgrpo_bin_packing(None, 3, 10, None, None, None) == -4
    assert lib.clgrpo_bin_packing_fix_bin(None, 0, 0, None, None) == -1


def test_product_package_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "chatlearn_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith(".py"):
                src = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle\b", src, flags=re.M), f"{f} imports the oracle"


def test_cpu_tensors_are_refused():
    import torch
    from chatlearn_amd import ops
    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.lmhead_forward(torch.zeros(2, 64), torch.zeros(4, 64), None)
    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.softmax_stats(torch.zeros(2, 64), None)


def test_missing_library_fails_loudly(tmp_path):
    """No fallback: with the shared object absent the first call that needs it raises and names the
    build command (checked in a fresh interpreter so the loaded library of this process stays)."""
    import subprocess
    import sys
    code = (
        "import os, torch\n"
        f"os.environ['CLGRPO_LIB_PATH'] = {str(tmp_path / 'nowhere.so')!r}\n"
        "from chatlearn_amd import ops\n"
        "try:\n"
        "    ops.bin_packing_ids([3, 2, 1], 4)\n"
        "except RuntimeError as e:\n"
        "    assert 'python -m chatlearn_amd.build' in str(e) and 'no fallback' in str(e), str(e)\n"
        "    print('raised')\n"
    )
    repo = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, "-c", code], cwd=repo, capture_output=True, text=True, timeout=120)
    assert out.returncode == 0 and "raised" in out.stdout, out.stderr[-500:]
