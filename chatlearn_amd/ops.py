"""Torch-tensor front end of the C ABI: allocates outputs / workspaces with torch
(device memory and streams are all torch is used for) and calls libclgrpo.so.

Every function here requires device tensors and the built library; nothing
falls back to torch arithmetic.
"""
import ctypes as C
from typing import Dict, List, Optional, Tuple

import torch

from . import _lib
from ._lib import BF16, F32, F64, U8, LOSS_GRPO, LOSS_GSPO

# Scratch memory a backward call may take when the caller names neither a chunk nor a workspace: the
# token chunk is halved until the plan fits (8192 tokens of a 152k vocabulary need 6.5 GB: d(logits) in
# both orientations, hidden^T, W^T, split-K partials).
DEFAULT_BWD_WORKSPACE_BYTES = 8 << 30


def _dtype_enum(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return BF16
    if t.dtype == torch.float32:
        return F32
    if t.dtype == torch.float64:
        return F64
    raise TypeError(f"unsupported dtype {t.dtype}")


def _dev(t: torch.Tensor, name: str, dtype=None) -> torch.Tensor:
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on the GPU (got {t.device}); this package has no CPU path")
    if dtype is not None and t.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
    return t if t.is_contiguous() else t.contiguous()


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _stream(t: torch.Tensor):
    return torch.cuda.current_stream(t.device).cuda_stream


# --------------------------------------------------------------------------- fused lm_head

def _round_up(x: int, m: int) -> int:
    return (x + m - 1) // m * m


def saved_logits_ld(V: int) -> int:
    """Elements per row of a kept-logits buffer for a vocabulary of V entries."""
    return int(_lib.lib().clgrpo_saved_logits_ld(V))


def saved_logits_buffer(T: int, V: int, dtype, device) -> torch.Tensor:
    """An (uninitialised) buffer the forward can keep raw logits in for the backward: T rows rounded
    up to whole blocks of 256 by the padded vocabulary extent, elements of the size of ``dtype``.  Its
    contents are opaque (``saved_logits_rowmajor`` decodes them): the forward stores the logits in the
    order of its accumulators, 16-bit inputs as IEEE half; the backward overwrites the buffer with
    d(logits) in the layout of its GEMM operands."""
    return torch.empty(_round_up(max(T, 1), 256), _lib.lib().clgrpo_saved_logits_ld(V), dtype=dtype, device=device)


def _unblock(buf: torch.Tensor, rows: int, cols: int) -> torch.Tensor:
    """[rows, cols] row-major copy of a K-blocked buffer: blocks of 256 rows, each block holding its
    128-byte K slabs one after another (slab = 256 rows x 128 bytes)."""
    e = 128 // buf.element_size()
    nb, ld = buf.shape[0] // 256, buf.shape[1]
    return buf.reshape(nb, ld // e, 256, e).permute(0, 2, 1, 3).reshape(nb * 256, ld)[:rows, :cols]


def saved_logits_rowmajor(buf: torch.Tensor, rows: int, V: int) -> torch.Tensor:
    """The first ``rows`` kept rows as an ordinary fp32 [rows, V] tensor (a copy; for inspection and tests).
    Decodes the forward's layout: 32 KB units of 256 rows x one 128-byte slab of vocabulary; inside a unit
    sub-blocks of 32 rows x 32 entries, each stored as [16-byte piece][lane half][row][values] where value
    r of lane half h is vocabulary entry 8 * (r // 4) + 4 * h + r % 4 of the sub-block."""
    es = buf.element_size()
    z = buf.view(torch.float16) if es == 2 else buf
    e = 128 // es                       # vocabulary entries per unit
    vsub, pieces = e // 32, es          # sub-blocks along the vocabulary, 16-byte pieces per lane
    per = 16 // pieces                  # values per piece
    nb, ld = buf.shape[0] // 256, buf.shape[1]
    z = z.reshape(nb, ld // e, 8, vsub, pieces, 2, 32, per)           # unit: [rs][vs][piece j][h][t32][value]
    z = z.permute(0, 2, 6, 1, 3, 4, 7, 5)                             # [nb][rs][t32][ks][vs][j][value][h]
    z = z.reshape(nb, 8, 32, ld // e, vsub, pieces * per // 4, 4, 2)  # register r = 4 * q + i -> [q][i][h]
    z = z.permute(0, 1, 2, 3, 4, 5, 7, 6)                             # entry = 8 * q + 4 * h + i
    return z.reshape(nb * 256, ld)[:rows, :V].float()


def weight_t_buffer(weight: torch.Tensor) -> torch.Tensor:
    """An (uninitialised) buffer for W^T (K-blocked, H rounded up to 256 rows) that ``lmhead_backward``
    can fill once and reuse."""
    V, H = weight.shape
    return torch.empty(_round_up(H, 256), _lib.lib().clgrpo_saved_logits_ld(V), dtype=weight.dtype, device=weight.device)


def weight_t_rowmajor(weight_t: torch.Tensor, H: int, V: int) -> torch.Tensor:
    """W^T as an ordinary [H, V] tensor (a copy; for inspection and tests)."""
    return _unblock(weight_t, H, V)


def lmhead_forward(hidden: torch.Tensor, weight: torch.Tensor, labels: Optional[torch.Tensor],
                   temperature: float = 1.0, need_entropy: bool = True,
                   saved_logits: Optional[torch.Tensor] = None, saved_row_map: Optional[torch.Tensor] = None,
                   _shard_begin: Optional[int] = None, workspace: Optional[torch.Tensor] = None
                   ) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor], torch.Tensor, torch.Tensor]:
    """(logprob, entropy, rowmax, lse), each fp32 [T].  Logits are not materialised unless the caller
    hands in ``saved_logits`` (from ``saved_logits_buffer``) for these T rows, which a following
    ``lmhead_backward`` of the same rows consumes instead of recomputing them.  ``saved_row_map``
    (int32 [T]) sends token t's logits to row ``map[t]`` of the buffer, or nowhere if negative; without
    a map token t goes to row t, and tokens past the buffer's rows are not kept."""
    hidden = _dev(hidden, "hidden")
    weight = _dev(weight, "weight", hidden.dtype)
    if hidden.dim() != 2 or weight.dim() != 2 or hidden.shape[1] != weight.shape[1]:
        raise ValueError(f"hidden [T,H] / weight [V,H] expected, got {tuple(hidden.shape)} / {tuple(weight.shape)}")
    T, H = hidden.shape
    V = weight.shape[0]
    if labels is not None:
        labels = _dev(labels, "labels", torch.int64)
        if labels.numel() != T:
            raise ValueError(f"labels must have {T} elements, got {labels.numel()}")
    dt = _dtype_enum(hidden)
    f = dict(dtype=torch.float32, device=hidden.device)
    if _shard_begin is not None:
        record = torch.empty(T, 4, **f)
        lse = rowmax = logprob = entropy = None
        if T == 0:
            return record
    else:
        lse = torch.empty(T, **f)
        rowmax = torch.empty(T, **f)
        logprob = torch.empty(T, **f) if labels is not None else None
        entropy = torch.empty(T, **f) if need_entropy else None
        if T == 0:
            return logprob, entropy, rowmax, lse
    ws_bytes = _lib.lib().clgrpo_lmhead_fwd_workspace_bytes(T, H, V, dt)
    ws = workspace if (workspace is not None and workspace.numel() >= ws_bytes) else \
        torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=hidden.device)
    ld_saved = 0
    if saved_logits is not None:
        saved_logits = _dev(saved_logits, "saved_logits", hidden.dtype)
        if saved_logits.dim() != 2 or not saved_logits.is_contiguous():
            raise ValueError("saved_logits must be a contiguous [rows, ld] tensor")
        if saved_logits.shape[0] % 256 != 0:
            raise ValueError("saved_logits must come from saved_logits_buffer (whole blocks of 256 rows)")
        ld_saved = saved_logits.shape[1]
        if saved_row_map is not None:
            saved_row_map = _dev(saved_row_map, "saved_row_map", torch.int32)
            if saved_row_map.numel() != T:
                raise ValueError("saved_row_map must have T elements")
    a = _lib.LmheadFwdArgs(_ptr(hidden), _ptr(weight), _ptr(labels), T, H, V, dt, 1.0 / float(temperature),
                           _ptr(logprob), _ptr(entropy), _ptr(rowmax), _ptr(lse), _ptr(ws), ws.numel(),
                           _ptr(saved_logits), ld_saved, _ptr(saved_row_map) if saved_logits is not None else None,
                           saved_logits.shape[0] if saved_logits is not None else 0)
    if _shard_begin is not None:
        _lib.check(_lib.lib().clgrpo_lmhead_fwd_shard(_lib.C.byref(a), int(_shard_begin), _ptr(record),
                                                      _lib.vp(_stream(hidden) or 0)))
        return record
    _lib.call("clgrpo_lmhead_fwd", a, _stream(hidden))
    return logprob, entropy, rowmax, lse


def lmhead_forward_launch_plan(T: int, V: int, cus: int = 0) -> Tuple[int, int, int]:
    """(blocks of 256 tokens, vocabulary splits, vocabulary tiles per workgroup) of the forward launch for T
    tokens on a device with ``cus`` compute units (0: 256)."""
    out = (C.c_int32 * 3)()
    _lib.check(_lib.lib().clgrpo_lmhead_fwd_launch_plan(int(T), int(V), int(cus), C.cast(out, C.c_void_p)))
    return int(out[0]), int(out[1]), int(out[2])


def dhidden_launch_plan(rows: int, H: int, V: int, dtype, cus: int = 0) -> Tuple[int, int]:
    """(256-token tiles of a first launch without a K split or 0, K ranges of the remaining launch) for the
    dhidden contraction of ``rows`` tokens."""
    out = (C.c_int32 * 2)()
    _lib.check(_lib.lib().clgrpo_lmhead_bwd_dhidden_plan(int(rows), int(H), int(V), BF16 if dtype == torch.bfloat16 else F32,
                                                         int(cus), C.cast(out, C.c_void_p)))
    return int(out[0]), int(out[1])


def dweight_launch_plan(rows: int, H: int, V: int, dtype, cus: int = 0) -> Tuple[int, int, int]:
    """(walks or 0, vocabulary tiles of a first launch of equally long walks or 0, K ranges of the launch over the
    remaining vocabulary tiles) for the dW contraction over a chunk of ``rows`` tokens."""
    out = (C.c_int32 * 3)()
    _lib.check(_lib.lib().clgrpo_lmhead_bwd_dweight_plan(int(rows), int(H), int(V), BF16 if dtype == torch.bfloat16 else F32,
                                                         int(cus), C.cast(out, C.c_void_p)))
    return int(out[0]), int(out[1]), int(out[2])


def lmhead_forward_workspace_bytes(T: int, H: int, V: int, dtype) -> int:
    """Bytes of scratch one ``lmhead_forward`` call of T tokens needs."""
    return int(_lib.lib().clgrpo_lmhead_fwd_workspace_bytes(T, H, V, BF16 if dtype == torch.bfloat16 else F32))


def lmhead_backward_workspace_bytes(T: int, H: int, V: int, dtype, with_saved_logits: bool,
                                    caller_keeps_weight_t: bool = False) -> int:
    """Bytes of scratch one unchunked ``lmhead_backward`` call of T tokens needs."""
    flags = (1 if with_saved_logits else 0) | (2 if caller_keeps_weight_t else 0)
    return int(_lib.lib().clgrpo_lmhead_bwd_workspace_bytes(T, H, V, BF16 if dtype == torch.bfloat16 else F32, T, flags))


def lmhead_forward_shard(hidden: torch.Tensor, weight_shard: torch.Tensor, labels: Optional[torch.Tensor],
                         vocab_begin: int, temperature: float = 1.0,
                         saved_logits: Optional[torch.Tensor] = None,
                         saved_row_map: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One vocabulary shard of the head: ``weight_shard`` holds rows ``[vocab_begin, vocab_begin + Vs)``
    of the full matrix, ``labels`` are global ids.  Returns the per-token record fp32 [T, 4] =
    (max raw logit, sum 2^((z-max)c), sum 2^((z-max)c)*z, target logit or 0) that
    ``lmhead_merge_shards`` combines across shards."""
    return lmhead_forward(hidden, weight_shard, labels, temperature, True, saved_logits, saved_row_map,
                          _shard_begin=int(vocab_begin))


def lmhead_merge_shards(records: torch.Tensor, labels: Optional[torch.Tensor], vocab_size: int,
                        temperature: float = 1.0, need_entropy: bool = True):
    """Merge the records of all vocabulary shards ([n_shards, T, 4], e.g. after an all-gather over
    the tensor-parallel group) into (logprob, entropy, rowmax, lse), each fp32 [T]."""
    records = _dev(records, "records", torch.float32)
    if records.dim() != 3 or records.shape[2] != 4:
        raise ValueError(f"records must be [n_shards, T, 4], got {tuple(records.shape)}")
    n, T = records.shape[0], records.shape[1]
    if labels is not None:
        labels = _dev(labels, "labels", torch.int64)
        if labels.numel() != T:
            raise ValueError(f"labels must have {T} elements, got {labels.numel()}")
    f = dict(dtype=torch.float32, device=records.device)
    lse, rowmax = torch.empty(T, **f), torch.empty(T, **f)
    logprob = torch.empty(T, **f) if labels is not None else None
    entropy = torch.empty(T, **f) if need_entropy else None
    if T == 0:
        return logprob, entropy, rowmax, lse
    if n == 0:
        raise ValueError("at least one shard is needed")
    _lib.check(_lib.lib().clgrpo_lmhead_merge_shards(_ptr(records), n, T, _ptr(labels), int(vocab_size),
                                                     1.0 / float(temperature), _ptr(logprob), _ptr(entropy),
                                                     _ptr(rowmax), _ptr(lse), _lib.vp(_stream(records) or 0)))
    return logprob, entropy, rowmax, lse


def lmhead_backward(hidden, weight, labels, lse, entropy, g_logprob, g_entropy=None, temperature=1.0,
                    need_dhidden=True, need_dweight=True, dweight: Optional[torch.Tensor] = None,
                    accumulate_dweight=False, chunk_tokens: Optional[int] = None,
                    max_workspace_bytes: int = DEFAULT_BWD_WORKSPACE_BYTES,
                    saved_logits: Optional[torch.Tensor] = None, weight_t: Optional[torch.Tensor] = None,
                    weight_t_ready: bool = False, vocab_begin: int = 0, workspace: Optional[torch.Tensor] = None):
    """(dhidden [T,H] in hidden's dtype, dweight [V,H] fp32).  ``dweight`` may be a caller
    buffer (e.g. the fp32 main-grad) that is overwritten or, with ``accumulate_dweight``, added to.
    ``saved_logits``: the buffer the forward of these rows filled; it is overwritten with d(logits).
    ``weight_t`` (from ``weight_t_buffer``) keeps W^T between calls that share the weight; pass
    ``weight_t_ready=True`` once a call has filled it.  ``vocab_begin`` > 0 (or a weight that is a
    vocabulary shard starting at 0): ``weight`` holds rows ``[vocab_begin, vocab_begin + V)`` of the full
    matrix, ``labels`` are global ids, ``lse`` / ``entropy`` the merged ones of all shards; ``dweight`` is
    then this shard's rows and ``dhidden`` its partial sum."""
    hidden = _dev(hidden, "hidden")
    weight = _dev(weight, "weight", hidden.dtype)
    labels = _dev(labels, "labels", torch.int64)
    lse = _dev(lse, "lse", torch.float32)
    g_logprob = _dev(g_logprob, "g_logprob", torch.float32)
    T, H = hidden.shape
    V = weight.shape[0]
    for name, t in (("labels", labels), ("lse", lse), ("g_logprob", g_logprob)):
        if t.numel() != T:
            raise ValueError(f"{name} must have {T} elements, got {t.numel()}")
    if g_entropy is not None:
        g_entropy = _dev(g_entropy, "g_entropy", torch.float32)
        entropy = _dev(entropy, "entropy", torch.float32)
        if g_entropy.numel() != T or entropy.numel() != T:
            raise ValueError("g_entropy / entropy must have T elements")
    dt = _dtype_enum(hidden)
    dhidden = torch.empty_like(hidden) if need_dhidden else None
    if need_dweight:
        if dweight is None:
            dweight = torch.empty(V, H, dtype=torch.float32, device=hidden.device)
            accumulate_dweight = False
        else:
            dweight = _dev(dweight, "dweight", torch.float32)
            if tuple(dweight.shape) != (V, H) or not dweight.is_contiguous():
                raise ValueError("dweight must be a contiguous fp32 [V,H] tensor")
    else:
        dweight = None
    if T == 0:
        if dweight is not None and not accumulate_dweight:
            dweight.zero_()
        return dhidden, dweight
    L = _lib.lib()
    ld_saved, has_saved = 0, 0
    if saved_logits is not None:
        saved_logits = _dev(saved_logits, "saved_logits", hidden.dtype)
        if saved_logits.dim() != 2 or saved_logits.shape[0] < T or saved_logits.shape[0] % 256 != 0 \
                or not saved_logits.is_contiguous():
            raise ValueError("saved_logits must come from saved_logits_buffer with at least T rows")
        ld_saved, has_saved = saved_logits.shape[1], 1
    if weight_t is not None:
        weight_t = _dev(weight_t, "weight_t", hidden.dtype)
        if tuple(weight_t.shape) != (_round_up(H, 256), L.clgrpo_saved_logits_ld(V)) or not weight_t.is_contiguous():
            raise ValueError("weight_t must come from weight_t_buffer(weight)")
    plan_flags = has_saved | (2 if weight_t is not None else 0)
    if chunk_tokens is None:
        chunk_tokens = T
        while chunk_tokens > 256 and \
                L.clgrpo_lmhead_bwd_workspace_bytes(T, H, V, dt, chunk_tokens, plan_flags) > max_workspace_bytes:
            chunk_tokens = max(256, (chunk_tokens // 2 + 255) // 256 * 256)
    ws_bytes = L.clgrpo_lmhead_bwd_workspace_bytes(T, H, V, dt, chunk_tokens, plan_flags)
    ws = workspace if (workspace is not None and workspace.numel() >= ws_bytes) else \
        torch.empty(ws_bytes, dtype=torch.uint8, device=hidden.device)
    a = _lib.LmheadBwdArgs(_ptr(hidden), _ptr(weight), _ptr(labels), _ptr(lse), _ptr(entropy), _ptr(g_logprob),
                           _ptr(g_entropy), T, H, V, dt, 1.0 / float(temperature), _ptr(dhidden), _ptr(dweight),
                           1 if accumulate_dweight else 0, _ptr(ws), ws.numel(), _ptr(saved_logits), ld_saved,
                           _ptr(weight_t), 1 if (weight_t is not None and weight_t_ready) else 0,
                           saved_logits.shape[0] if saved_logits is not None else 0)
    if vocab_begin:
        _lib.check(L.clgrpo_lmhead_bwd_shard(_lib.C.byref(a), int(vocab_begin), _lib.vp(_stream(hidden) or 0)))
    else:
        _lib.call("clgrpo_lmhead_bwd", a, _stream(hidden))
    return dhidden, dweight


# --------------------------------------------------------------------------- stats from logits

def softmax_stats(logits2d: torch.Tensor, labels: Optional[torch.Tensor], need_entropy=True, need_logprob=True):
    """(logprob, entropy, lse) fp32 [R] from materialised [R,V] logits (last dim contiguous)."""
    if logits2d.dim() != 2:
        raise ValueError("logits2d must be [R,V]")
    if not logits2d.is_cuda:
        raise RuntimeError("logits must live on the GPU; this package has no CPU path")
    if logits2d.stride(1) != 1:
        logits2d = logits2d.contiguous()
    R, V = logits2d.shape
    ld = logits2d.stride(0) if R > 1 else V
    dt = _dtype_enum(logits2d)
    f = dict(dtype=torch.float32, device=logits2d.device)
    need_logprob = need_logprob and labels is not None
    if need_logprob:
        labels = _dev(labels, "labels", torch.int64)
    lp = torch.empty(R, **f) if need_logprob else None
    ent = torch.empty(R, **f) if need_entropy else None
    lse = torch.empty(R, **f)
    a = _lib.SoftmaxStatsArgs(_ptr(logits2d), _ptr(labels) if need_logprob else None, R, V, ld, dt,
                              _ptr(lp), _ptr(ent), _ptr(lse))
    _lib.call("clgrpo_softmax_stats", a, _stream(logits2d))
    return lp, ent, lse


def softmax_stats_backward(logits2d, labels, g_logprob, g_entropy, lse=None, entropy=None):
    """d(logits) [R,V] in the logits' dtype.  ``lse`` (and ``entropy`` when ``g_entropy`` is given) from the
    forward let the kernel read each row once; without them it rebuilds them with one more pass."""
    if not logits2d.is_cuda:
        raise RuntimeError("logits must live on the GPU; this package has no CPU path")
    if logits2d.stride(1) != 1:
        logits2d = logits2d.contiguous()
    R, V = logits2d.shape
    ld = logits2d.stride(0) if R > 1 else V
    out = torch.empty(R, V, dtype=logits2d.dtype, device=logits2d.device)
    if g_logprob is not None:
        g_logprob = _dev(g_logprob, "g_logprob", torch.float32)
        labels = _dev(labels, "labels", torch.int64)
    if g_entropy is not None:
        g_entropy = _dev(g_entropy, "g_entropy", torch.float32)
    if lse is not None:
        lse = _dev(lse, "lse", torch.float32)
    if entropy is not None:
        entropy = _dev(entropy, "entropy", torch.float32)
    a = _lib.SoftmaxStatsBwdArgs(_ptr(logits2d), _ptr(labels) if g_logprob is not None else None, _ptr(g_logprob),
                                 _ptr(g_entropy), R, V, ld, _dtype_enum(logits2d), _ptr(out), _ptr(lse), _ptr(entropy))
    _lib.call("clgrpo_softmax_stats_bwd", a, _stream(logits2d))
    return out


# --------------------------------------------------------------------------- policy loss

class PolicyLossResult:
    """Outputs of one clgrpo_policy_loss launch (device tensors; ``sums``/``flags`` not yet synced)."""
    __slots__ = ("loss", "dloss", "kl", "is_positive_clipped", "is_negative_clipped", "is_clipped",
                 "g_logprob", "g_entropy", "sums", "flags")

    def raise_on_flags(self):
        """Same assertions, same messages, as the reference raises (one host sync)."""
        fl = int(self.flags.item())
        assert not fl & 1, "pg loss is nan"
        assert not fl & 2, "kl loss ratio has inf values"
        assert not fl & 4, "kl loss ratio has nan values"


def policy_loss(logprob, old_logprob, advantages, *, mode=LOSS_GRPO, cu_seqlens=None, ref_logprob=None,
                entropy=None, loss_mask=None, diff_clip_ratio=10, pos_clip_ratio=0.2, neg_clip_ratio=0.2,
                final_clip_ratio=3.0, kl_coef=0.0, entropy_coef=0.0, grad_scale=1.0, want_dloss=True,
                want_kl=None, want_flags3=False, want_upstream=False, token_offset=0) -> PolicyLossResult:
    """logprob/old/ref/entropy fp32, either [B,S] (padded) or flat [n] with ``cu_seqlens`` int32 [B+1];
    ``advantages`` a device tensor [B], fp32 or fp64 (sets the dtype of the loss)."""
    logprob = _dev(logprob, "logprob", torch.float32)
    old_logprob = _dev(old_logprob, "old_logprob", torch.float32)
    advantages = _dev(advantages, "advantages")
    cdt = _dtype_enum(advantages)
    if cdt not in (F32, F64):
        raise TypeError("advantages must be fp32 or fp64")
    n = logprob.numel()
    if old_logprob.numel() != n:
        raise ValueError("old_logprob and logprob differ in size")
    if cu_seqlens is not None:
        cu_seqlens = _dev(cu_seqlens, "cu_seqlens", torch.int32)
        B, S = cu_seqlens.numel() - 1, 0
    else:
        if logprob.dim() != 2:
            raise ValueError("padded layout needs [B,S] tensors (or pass cu_seqlens)")
        B, S = logprob.shape
    if advantages.numel() != B:
        raise ValueError(f"advantages must have {B} elements, got {advantages.numel()}")
    dev = logprob.device

    def opt(t, name, dtype):
        if t is None:
            return None
        t = _dev(t, name, dtype)
        if t.numel() != n:
            raise ValueError(f"{name} must have {n} elements")
        return t

    ref_logprob = opt(ref_logprob, "ref_logprob", torch.float32)
    entropy = opt(entropy, "entropy", torch.float32)
    if loss_mask is not None and loss_mask.dtype != torch.int32:
        loss_mask = loss_mask.to(torch.int32)
    loss_mask = opt(loss_mask, "loss_mask", torch.int32)
    if want_kl is None:
        want_kl = ref_logprob is not None
    r = PolicyLossResult()
    r.loss = torch.empty(logprob.shape, dtype=advantages.dtype, device=dev)
    r.dloss = torch.empty(logprob.shape, dtype=advantages.dtype, device=dev) if want_dloss else None
    r.kl = torch.empty(logprob.shape, dtype=torch.float32, device=dev) if want_kl else None
    mk = lambda: torch.empty(logprob.shape, dtype=torch.bool, device=dev)
    r.is_positive_clipped, r.is_negative_clipped, r.is_clipped = (mk(), mk(), mk()) if want_flags3 else (None, None, None)
    r.g_logprob = torch.empty(logprob.shape, dtype=torch.float32, device=dev) if want_upstream else None
    r.g_entropy = (torch.empty(logprob.shape, dtype=torch.float32, device=dev)
                   if (want_upstream and entropy_coef > 0) else None)
    r.sums = torch.empty(8, dtype=torch.float64, device=dev)
    r.flags = torch.empty(1, dtype=torch.int32, device=dev)
    if n == 0:
        r.sums.zero_()
        r.flags.zero_()
        return r
    ws_bytes = _lib.lib().clgrpo_policy_loss_workspace_bytes(n, B)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    a = _lib.PolicyLossArgs(mode, cdt, n, B, S, _ptr(cu_seqlens), _ptr(logprob), _ptr(old_logprob), _ptr(ref_logprob),
                            _ptr(entropy), _ptr(loss_mask), _ptr(advantages), float(diff_clip_ratio),
                            float(pos_clip_ratio), float(neg_clip_ratio), float(final_clip_ratio), float(kl_coef),
                            float(entropy_coef), float(grad_scale), _ptr(r.loss), _ptr(r.dloss), _ptr(r.kl),
                            _ptr(r.is_positive_clipped), _ptr(r.is_negative_clipped), _ptr(r.is_clipped),
                            _ptr(r.g_logprob), _ptr(r.g_entropy), _ptr(r.sums), _ptr(r.flags), _ptr(ws), ws.numel(),
                            int(token_offset))
    _lib.call("clgrpo_policy_loss", a, _stream(logprob))
    return r


def masked_sums(tensors, mask: torch.Tensor, averaged):
    """(sums fp32 [k], count int32 [1]): sums[j] = sum(float(tensors[j]) * mask), divided by
    (1e-5 + sum(mask)) where ``averaged[j]``; count = sum(mask).  Tensors are fp32, fp64 or bool and
    have the mask's number of elements; the mask holds zeros and ones.  One launch for all of them."""
    tensors = list(tensors)
    k = len(tensors)
    if not 1 <= k <= 16:
        raise ValueError(f"between 1 and 16 tensors expected, got {k}")
    if mask.dtype != torch.int32:
        mask = mask.to(torch.int32)
    mask = _dev(mask, "mask", torch.int32)
    n = mask.numel()
    if n == 0:
        return (torch.zeros(k, dtype=torch.float32, device=mask.device),
                torch.zeros(1, dtype=torch.int32, device=mask.device))
    a = _lib.MaskedSumsArgs()
    a.n, a.k = n, k
    keep = []
    for j, t in enumerate(tensors):
        t = _dev(t.detach(), f"tensors[{j}]")
        if t.numel() != n:
            raise ValueError(f"tensors[{j}] must have {n} elements, got {t.numel()}")
        if t.dtype == torch.bool:
            code = U8
        elif t.dtype in (torch.float32, torch.float64):
            code = _dtype_enum(t)
        else:
            t, code = t.float(), F32
        keep.append(t)
        a.src[j], a.dtype[j], a.average[j] = t.data_ptr(), code, 1 if averaged[j] else 0
    sums = torch.empty(k, dtype=torch.float32, device=mask.device)
    count = torch.empty(1, dtype=torch.int32, device=mask.device)
    a.mask, a.out, a.count = mask.data_ptr(), sums.data_ptr(), count.data_ptr()
    _lib.call("clgrpo_masked_sums", a, _stream(mask))
    return sums, count


def masked_sums_backward(g: torch.Tensor, mask: torch.Tensor, dtype, shape) -> torch.Tensor:
    """g[0] * mask as a tensor of ``dtype`` (fp32 / fp64) and ``shape``; ``g`` a one-element fp32 device tensor."""
    if mask.dtype != torch.int32:
        mask = mask.to(torch.int32)
    mask = _dev(mask, "mask", torch.int32)
    g = _dev(g, "g", torch.float32)
    if dtype not in (torch.float32, torch.float64):
        raise TypeError(f"gradient dtype must be fp32 or fp64, got {dtype}")
    out = torch.empty(shape, dtype=dtype, device=mask.device)
    _lib.check(_lib.lib().clgrpo_masked_sums_bwd(mask.numel(), _ptr(g), _ptr(mask), _ptr(out),
                                                 F32 if dtype == torch.float32 else F64, _lib.vp(_stream(mask) or 0)))
    return out


# --------------------------------------------------------------------------- advantages

def group_advantage(rewards, group_of, pool, pool_offsets, eps=1e-5):
    """adv fp64 [n], all_zeros bool [n], all_ones bool [n]; all arguments device tensors."""
    rewards = _dev(rewards, "rewards", torch.float64)
    group_of = _dev(group_of, "group_of", torch.int32)
    pool = _dev(pool, "pool", torch.float64)
    pool_offsets = _dev(pool_offsets, "pool_offsets", torch.int32)
    n = rewards.numel()
    dev = rewards.device
    adv = torch.empty(n, dtype=torch.float64, device=dev)
    z = torch.empty(n, dtype=torch.bool, device=dev)
    o = torch.empty(n, dtype=torch.bool, device=dev)
    a = _lib.GroupAdvantageArgs(n, pool_offsets.numel() - 1, _ptr(rewards), _ptr(group_of), _ptr(pool),
                                _ptr(pool_offsets), float(eps), _ptr(adv), _ptr(z), _ptr(o))
    _lib.call("clgrpo_group_advantage", a, _stream(rewards))
    return adv, z, o


# --------------------------------------------------------------------------- masks / indices

def build_masks(prompt_len: torch.Tensor, response_len: torch.Tensor, S: int, want_position_ids=True):
    prompt_len = _dev(prompt_len, "prompt_len", torch.int32)
    response_len = _dev(response_len, "response_len", torch.int32)
    B = prompt_len.numel()
    dev = prompt_len.device
    attn = torch.empty(B, S, dtype=torch.int32, device=dev)
    loss = torch.empty(B, S, dtype=torch.int32, device=dev)
    pos = torch.empty(B, S, dtype=torch.int64, device=dev) if want_position_ids else None
    a = _lib.BuildMasksArgs(B, S, _ptr(prompt_len), _ptr(response_len), _ptr(attn), _ptr(loss), _ptr(pos))
    _lib.call("clgrpo_build_masks", a, _stream(prompt_len))
    return attn, loss, pos


def shift_labels(tokens: Optional[torch.Tensor], loss_mask: Optional[torch.Tensor], zero_last: bool):
    ref = tokens if tokens is not None else loss_mask
    B, S = ref.shape
    labels = shifted = None
    if tokens is not None:
        tokens = _dev(tokens, "tokens", torch.int64)
        labels = torch.empty_like(tokens)
    if loss_mask is not None:
        loss_mask = _dev(loss_mask, "loss_mask", torch.int32)
        shifted = torch.empty_like(loss_mask)
    a = _lib.ShiftLabelsArgs(B, S, _ptr(tokens), _ptr(loss_mask), _ptr(labels), _ptr(shifted), 1 if zero_last else 0)
    _lib.call("clgrpo_shift_labels", a, _stream(ref))
    return labels, shifted


def unpad_indices(attn_mask: torch.Tensor):
    """(indices int64 [T], cu_seqlens int32 [B+1], seqlens int32 [B], max_seqlen int) - one host sync."""
    if attn_mask.dtype != torch.int32:
        attn_mask = attn_mask.to(torch.int32)
    attn_mask = _dev(attn_mask, "attention_mask", torch.int32)
    B, S = attn_mask.shape
    dev = attn_mask.device
    indices = torch.empty(B * S, dtype=torch.int64, device=dev)
    cu = torch.empty(B + 1, dtype=torch.int32, device=dev)
    seqlens = torch.empty(B, dtype=torch.int32, device=dev)
    total = torch.empty(2, dtype=torch.int32, device=dev)
    row_off = torch.empty(B + 1, dtype=torch.int32, device=dev)
    a = _lib.UnpadIndicesArgs(B, S, _ptr(attn_mask), _ptr(indices), _ptr(cu), _ptr(seqlens), _ptr(total), _ptr(row_off))
    _lib.call("clgrpo_unpad_indices", a, _stream(attn_mask))
    n_idx, max_len = total.tolist()
    return indices[:n_idx], cu, seqlens, max_len


def thd_pack(tokens: torch.Tensor, prompt_len, response_len, align: int, pad_token: int, cp_size: int = 1,
             cp_rank: int = 0, want_loss_mask: bool = True, want_position_ids: bool = False,
             verify_on_device: bool = True) -> Dict[str, object]:
    """Packed (THD) micro-batch from per-sample lengths, in one device pass.

    ``tokens`` int64 [B, S] on the device; ``prompt_len`` / ``response_len`` host sequences (or CPU
    tensors) of B ints, from which the padded sizes are computed on the host, so no device value is
    read back to size the outputs.  Every sequence is padded with ``pad_token`` to a multiple of
    ``align``.  Returns a dict: ``cu_seqlens_padded`` int32 [B+1], ``seqlens`` / ``seqlens_padded`` int32
    [B], ``indices`` int64 [total] (positions in the padded [B, max padded length] layout),
    ``seq_indices`` / ``tokens`` / ``labels`` (/ ``position_ids``) int64 [total / cp_size] and ``loss_mask`` int32
    for this context-parallel rank, ``num_loss_tokens`` (device int32 scalar), ``total_padded`` and
    ``max_seqlen_padded`` (host ints).  The lengths are checked on the host; with ``verify_on_device`` the
    device's own consistency word is read back as well (one host round trip)."""
    tokens = _dev(tokens, "tokens", torch.int64)
    if tokens.dim() != 2:
        raise ValueError("tokens must be [B, S]")
    B, S = tokens.shape
    pl = [int(x) for x in (prompt_len.tolist() if isinstance(prompt_len, torch.Tensor) else prompt_len)]
    rl = [int(x) for x in (response_len.tolist() if isinstance(response_len, torch.Tensor) else response_len)]
    if len(pl) != B or len(rl) != B:
        raise ValueError(f"prompt_len / response_len must have {B} entries")
    align, cp_size, cp_rank = int(align), int(cp_size), int(cp_rank)
    if align <= 0 or cp_size <= 0:
        raise ValueError("align and cp_size must be positive")
    if any(p < 0 or r < 0 or p + r > S for p, r in zip(pl, rl)):
        raise ValueError("thd_pack: a sequence is longer than S (or a length is negative)")
    padded = [(p + r + align - 1) // align * align for p, r in zip(pl, rl)]
    if any(x % (2 * cp_size) for x in padded) and cp_size > 1:
        raise ValueError("thd_pack: a padded length is not a multiple of 2*cp_size")
    total, max_padded = sum(padded), max(padded)
    dev = tokens.device
    i32 = dict(dtype=torch.int32, device=dev)
    lens = torch.tensor([pl, rl], dtype=torch.int32).to(dev)
    cu, seqlens, seqlens_padded = torch.empty(B + 1, **i32), torch.empty(B, **i32), torch.empty(B, **i32)
    stats, status = torch.empty(3, **i32), torch.empty(1, **i32)
    per_rank = total // cp_size
    i64o = dict(dtype=torch.int64, device=dev)
    indices, seq_indices = torch.empty(total, **i64o), torch.empty(per_rank, **i64o)
    out_tokens, out_labels = torch.empty(per_rank, **i64o), torch.empty(per_rank, **i64o)
    out_mask = torch.empty(per_rank, **i32) if want_loss_mask else None
    out_pos = torch.empty(per_rank, **i64o) if want_position_ids else None
    a = _lib.ThdPackArgs(B, S, _ptr(tokens), _ptr(lens[0]), _ptr(lens[1]), align, cp_size, cp_rank, int(pad_token), total,
                         _ptr(cu), _ptr(seqlens), _ptr(seqlens_padded), _ptr(stats), _ptr(status), _ptr(indices),
                         _ptr(seq_indices), _ptr(out_tokens), _ptr(out_labels), _ptr(out_mask), _ptr(out_pos))
    _lib.call("clgrpo_thd_pack", a, _stream(tokens))
    # the device recomputes the sizes from the same lengths; reading its result back costs a host round trip
    bad = int(status.item()) if verify_on_device else 0
    if bad:
        why = [m for bit, m in ((1, "padded total differs from the host's"), (2, "a sequence is longer than S"),
                                (4, "a padded length is not a multiple of 2*cp_size")) if bad & bit]
        raise ValueError("thd_pack: " + "; ".join(why))
    return {"cu_seqlens_padded": cu, "seqlens": seqlens, "seqlens_padded": seqlens_padded, "indices": indices,
            "seq_indices": seq_indices, "tokens": out_tokens, "labels": out_labels, "loss_mask": out_mask,
            "position_ids": out_pos,
            "num_loss_tokens": stats[2], "total_padded": total, "max_seqlen_padded": max_padded}


def gather_rows(src: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
    """src [N, ...] -> [len(indices), ...]"""
    src = _dev(src, "src")
    indices = _dev(indices, "indices", torch.int64)
    row_shape = src.shape[1:]
    row_bytes = src.element_size() * int(torch.Size(row_shape).numel())
    out = torch.empty((indices.numel(),) + tuple(row_shape), dtype=src.dtype, device=src.device)
    a = _lib.RowsArgs(_ptr(src), _ptr(out), _ptr(indices), indices.numel(), row_bytes, src.shape[0])
    _lib.call("clgrpo_gather_rows", a, _stream(src))
    return out


def scatter_rows(src: torch.Tensor, indices: torch.Tensor, n_rows: int) -> torch.Tensor:
    """zeros [n_rows, ...] with out[indices[i]] = src[i]"""
    src = _dev(src, "src")
    indices = _dev(indices, "indices", torch.int64)
    row_shape = src.shape[1:]
    row_bytes = src.element_size() * int(torch.Size(row_shape).numel())
    out = torch.empty((n_rows,) + tuple(row_shape), dtype=src.dtype, device=src.device)
    a = _lib.RowsArgs(_ptr(src), _ptr(out), _ptr(indices), indices.numel(), row_bytes, n_rows)
    _lib.call("clgrpo_scatter_rows", a, _stream(src))
    return out


# --------------------------------------------------------------------------- host bin packing

def _unflatten(order, offsets, n_bins) -> List[List[int]]:
    return [list(order[offsets[b]:offsets[b + 1]]) for b in range(n_bins)]


def bin_packing_ids(seq_len_list, max_train_token) -> List[List[int]]:
    n = len(seq_len_list)
    lens = (C.c_int64 * max(n, 1))(*[int(x) for x in seq_len_list])
    order = (C.c_int64 * max(n, 1))()
    offsets = (C.c_int64 * (n + 1))()
    nb = C.c_int64(0)
    _lib.check(_lib.lib().clgrpo_bin_packing(lens, n, int(max_train_token), order, offsets, C.byref(nb)))
    return _unflatten(order, offsets, nb.value)


def bin_packing_fix_bin_ids(seq_len_list, bin_size) -> List[List[int]]:
    n = len(seq_len_list)
    lens = (C.c_int64 * max(n, 1))(*[int(x) for x in seq_len_list])
    order = (C.c_int64 * max(n, 1))()
    offsets = (C.c_int64 * (int(bin_size) + 1))()
    _lib.check(_lib.lib().clgrpo_bin_packing_fix_bin(lens, n, int(bin_size), order, offsets))
    return _unflatten(order, offsets, int(bin_size))
