"""The seam the reference lacks: logprob / entropy straight from the final hidden
states and lm_head.weight, without the [T, V] logits tensor.

``fused_linear_logprob_entropy`` stands where the reference runs
``self.model(...).logits`` followed by ``logprobs_from_logits`` and
``entropy_from_logits_with_chunking`` (policy_trainer.py:216-228); it is
autograd-aware, so ``total_loss.backward()`` (policy_trainer.py:286) reaches
``hidden`` and ``weight`` through the fused backward kernels.

``grpo_head_step`` does a whole micro-batch of the head - fused forward, fused
loss (+ upstream gradients), fused backward - for callers that own the training
loop; it walks the micro-batch in token chunks and lets the backward reuse the
chunk's logits instead of recomputing them.
"""
import bisect
from typing import Optional

import numpy as np
import torch

from . import ops
from ._lib import LOSS_GRPO, LOSS_GSPO


DEFAULT_KEEP_LOGITS_TOKENS = 8192   # tokens whose logits one chunk keeps for its backward (2.5 GB at a 152k vocabulary)


def _nonzero_rows(mask: torch.Tensor) -> torch.Tensor:
    """Ascending positions of the nonzero entries of a flat int32 device mask (one host round trip for
    their count).  The index kernels use one workgroup per row of a [B, S] mask, so the flat mask is
    presented as rows of 64 entries, zero-padded at the end (the flat positions are the same)."""
    n = mask.numel()
    if n == 0:
        return torch.empty(0, dtype=torch.int64, device=mask.device)
    if n % 64:
        mask = torch.nn.functional.pad(mask, (0, 64 - n % 64))
    live, _, _, _ = ops.unpad_indices(mask.reshape(-1, 64))
    return live


class _PinnedStaging:
    """Host-side staging for small index arrays that go to the device without stalling the host: two pinned
    buffers used in turn, each guarded by an event so that it is not rewritten while its copy is in flight."""

    def __init__(self):
        self.slots = [None, None]
        self.events = [None, None]
        self.turn = 0

    def upload(self, host: torch.Tensor, device) -> torch.Tensor:
        i = self.turn
        self.turn ^= 1
        nbytes = host.numel() * host.element_size()
        if self.events[i] is not None:
            self.events[i].synchronize()
        if self.slots[i] is None or self.slots[i].numel() < nbytes:
            self.slots[i] = torch.empty(max(nbytes, 1 << 16), dtype=torch.uint8, pin_memory=True)
        stage = self.slots[i][:nbytes].view(host.dtype)
        stage.copy_(host.reshape(-1))
        out = stage.to(device, non_blocking=True)
        self.events[i] = torch.cuda.Event()
        self.events[i].record()
        return out.reshape(host.shape)


_staging = {}


def _upload(host: torch.Tensor, device) -> torch.Tensor:
    key = (torch.device(device).index or 0, host.dtype)
    return _staging.setdefault(key, _PinnedStaging()).upload(host, device)


def _live_rows_from_host_mask(mask_host: torch.Tensor, chunks, device):
    """Per token chunk: (positions of the unmasked rows inside the chunk, int64; row map int32 with the
    rank of each unmasked row or -1), built on the host from a host copy of the loss mask and sent
    over in two asynchronous copies, so that no device value has to be read back.  The index work is
    numpy's (single-threaded): a few microseconds, and no thread pool to wake on the step's critical path."""
    flat = mask_host.reshape(-1).numpy() != 0
    live_all = np.flatnonzero(flat).astype(np.int64)
    bounds = np.searchsorted(live_all, [lo for lo, _ in chunks] + [chunks[-1][1]])
    local = live_all.copy()
    row_map = np.full(flat.shape[0], -1, dtype=np.int32)
    counts = []
    for k, (lo, hi) in enumerate(chunks):
        a, b = int(bounds[k]), int(bounds[k + 1])
        local[a:b] -= lo
        row_map[live_all[a:b]] = np.arange(b - a, dtype=np.int32)
        counts.append((a, b))
    local_d = _upload(torch.from_numpy(local), device) if local.size else torch.empty(0, dtype=torch.int64, device=device)
    map_d = _upload(torch.from_numpy(row_map), device)
    return [(local_d[a:b], map_d[lo:hi]) for (a, b), (lo, hi) in zip(counts, chunks)]


class _FusedHead(torch.autograd.Function):
    @staticmethod
    def forward(ctx, hidden, weight, labels, temperature, need_entropy, dweight_buffer, keep_rows, row_mask):
        T = hidden.shape[0]
        zbuf = live = row_map = None
        if keep_rows is not None and T > 0:
            if row_mask is not None:
                # rows outside the mask get a zero upstream gradient whatever their logits are:
                # keep logits only for the others and run the backward on that compact set
                live = _nonzero_rows(row_mask)
            rows = T if live is None else int(live.numel())
            if rows > keep_rows:
                live = None                  # more rows than may be kept: the backward recomputes its logit tiles
            elif rows > 0:
                zbuf = ops.saved_logits_buffer(rows, weight.shape[0], hidden.dtype, hidden.device)
                if live is not None:
                    row_map = torch.full((T,), -1, dtype=torch.int32, device=hidden.device)
                    row_map[live] = torch.arange(live.numel(), dtype=torch.int32, device=hidden.device)
        lp, ent, _, lse = ops.lmhead_forward(hidden, weight, labels, temperature, need_entropy,
                                             saved_logits=zbuf, saved_row_map=row_map if zbuf is not None else None)
        ctx.save_for_backward(hidden, weight, labels, lse, ent if ent is not None else lse)
        ctx.set_materialize_grads(False)
        ctx.temperature = temperature
        ctx.has_entropy = ent is not None
        ctx.dweight_buffer = dweight_buffer
        ctx.zbuf, ctx.live = zbuf, live
        if ent is None:
            ent = torch.zeros(0, device=hidden.device)
            ctx.mark_non_differentiable(ent)
        return lp, ent

    @staticmethod
    def backward(ctx, g_lp, g_ent):
        hidden, weight, labels, lse, ent = ctx.saved_tensors
        need_h, need_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        zbuf, live = ctx.zbuf, ctx.live
        ctx.zbuf = None                      # the buffer is consumed (overwritten) by this backward
        none = (None,) * 8
        if g_lp is None and g_ent is None:
            return none
        if g_lp is None:
            g_lp = torch.zeros_like(lse)
        use_ent = ctx.has_entropy and g_ent is not None
        g_lp = g_lp.float().contiguous()
        g_ent = g_ent.float().contiguous() if use_ent else None
        ent = ent if use_ent else None
        T = hidden.shape[0]
        kw = dict(need_dhidden=need_h, need_dweight=need_w, dweight=ctx.dweight_buffer,
                  accumulate_dweight=ctx.dweight_buffer is not None)
        if live is None:
            dh, dw = ops.lmhead_backward(hidden, weight, labels, lse, ent, g_lp, g_ent, ctx.temperature,
                                         saved_logits=zbuf, **kw)
        elif live.numel() == 0:
            dh = torch.zeros_like(hidden) if need_h else None
            dw = None
            if need_w and ctx.dweight_buffer is None:
                dw = torch.zeros(weight.shape, dtype=torch.float32, device=hidden.device)
        else:
            pick = lambda x: None if x is None else ops.gather_rows(x.reshape(T, -1), live).reshape(-1)
            dh_c, dw = ops.lmhead_backward(ops.gather_rows(hidden, live), weight, pick(labels), pick(lse), pick(ent),
                                           pick(g_lp), pick(g_ent), ctx.temperature, saved_logits=zbuf, **kw)
            dh = ops.scatter_rows(dh_c, live, T) if need_h else None
        if dw is not None:
            # A caller-supplied fp32 main-grad buffer was accumulated in place; autograd gets no copy.
            dw = None if ctx.dweight_buffer is not None else dw.to(weight.dtype)
        return (dh, dw) + (None,) * 6


def fused_linear_logprob_entropy(hidden: torch.Tensor, weight: torch.Tensor, labels: torch.Tensor, *,
                                 temperature: float = 1.0, need_entropy: bool = True,
                                 dweight_buffer: Optional[torch.Tensor] = None,
                                 keep_logits_rows: Optional[int] = DEFAULT_KEEP_LOGITS_TOKENS, loss_mask: Optional[torch.Tensor] = None):
    """(logprob fp32 [T], entropy fp32 [T]) of ``labels`` under softmax(hidden @ weight.T / temperature).

    hidden [T,H] and weight [V,H] share a dtype (bf16 or fp32), labels int64 [T].
    ``dweight_buffer``: optional fp32 [V,H] tensor that receives ``+= dW`` in the
    backward (the fp32 gradient accumulation FSDP2 does with ``reduce_dtype=fp32``);
    without it ``weight.grad`` gets dW cast to the weight dtype, as torch would.
    Leading dimensions of hidden/labels are flattened and restored.

    ``keep_logits_rows``: when a gradient is needed and there are at most this many rows (with
    ``loss_mask``: unmasked rows), the forward keeps their raw logits (one 16-bit copy for 16-bit inputs, released by the backward) so that the
    backward does not recompute them; ``None`` or more rows: recompute.  The default bounds the kept
    logits at 2.5 GB for a 152k vocabulary; a caller that wants the fast path for a larger micro-batch
    either raises it or runs the head chunk by chunk (forward, loss, backward per chunk), which is what
    ``grpo_head_step`` does.  ``loss_mask`` (same shape as
    ``labels``) is a promise that rows where it is zero receive a zero upstream gradient - true
    of the reference's loss, which multiplies by this mask (policy_trainer.py:259-283): their
    logits are then not kept and the backward runs on the other rows only.
    """
    lead = labels.shape
    h2 = hidden.reshape(-1, hidden.shape[-1])
    T = h2.shape[0]
    needs_grad = torch.is_grad_enabled() and (hidden.requires_grad or weight.requires_grad)
    keep = keep_logits_rows if needs_grad else None      # rows whose logits may be kept; None: keep nothing
    mask = None
    if keep is not None and loss_mask is not None:
        mask = loss_mask.reshape(-1).to(torch.int32)
    lp, ent = _FusedHead.apply(h2, weight, labels.reshape(-1), float(temperature), bool(need_entropy), dweight_buffer,
                               keep, mask)
    lp = lp.reshape(lead)
    ent = ent.reshape(lead) if need_entropy else None
    return lp, ent


def _token_chunks(T, chunk_rows, seq_bounds, live_cum=None):
    """[lo, hi) token ranges holding at most ``chunk_rows`` rows each: as few ranges as that allows, and
    of about equal length in tokens (the forward runs on every token of a range; a short last range would
    run all kernels at poor efficiency).  A token counts as a row, unless ``live_cum`` is given (a numpy
    array, live_cum[i] = rows among tokens [0, i) whose logits are kept, i.e. the unmasked ones): then the
    bound is on those.  With ``seq_bounds`` (the host copy of cu_seqlens) every range ends on a sequence
    boundary (a range exceeds ``chunk_rows`` only where a single sequence is larger than it), otherwise
    on a multiple of 256 tokens where the bound leaves room for that."""
    total = T if live_cum is None else int(live_cum[T])
    if chunk_rows is None or chunk_rows >= total or T == 0:
        return [(0, T)]
    wt = (lambda pos: pos) if live_cum is None else (lambda pos: int(live_cum[pos]))

    def first_with(rows):       # smallest position with at least `rows` rows before it
        return min(T, rows) if live_cum is None else min(T, int(live_cum.searchsorted(rows, side="left")))

    def last_with(rows):        # largest position with at most `rows` rows before it
        return min(T, rows) if live_cum is None else min(T, int(live_cum.searchsorted(rows, side="right")) - 1)

    cuts = wcuts = None
    if seq_bounds is not None:
        cuts = sorted(set(int(x) for x in seq_bounds if 0 < int(x) < T)) + [T]
        wcuts = [wt(c) for c in cuts]

    def choose(lo, need, target):
        """End of the range that starts at lo: within the bound, leaving at most `total - need` rows behind
        where possible, and as near to token `target` as those two allow."""
        limit = wt(lo) + chunk_rows
        if cuts is None:
            hi_max = max(lo + 1, last_with(limit))
            hi_min = min(hi_max, max(lo + 1, first_with(need)))
            hi = min(max(target, hi_min), hi_max)
            for r in sorted({hi // 256 * 256, (hi + 255) // 256 * 256}, key=lambda r: abs(r - hi)):
                if hi_min <= r <= hi_max and r < T:
                    return r
            return hi
        a = bisect.bisect_right(cuts, lo)
        b = max(a + 1, bisect.bisect_right(wcuts, limit))          # a single longer sequence gets a range of its own
        a2 = min(max(bisect.bisect_left(wcuts, need, a, b), a), b - 1)
        return min(cuts[a2:b], key=lambda c: (abs(c - target), c))

    # number of ranges: fill each to the bound
    n, lo = 0, 0
    while lo < T:
        lo = choose(lo, total, T)
        if wt(lo) == total:
            lo = T                                                 # a tail without rows rides along
        n += 1
    out, lo = [], 0
    while lo < T:
        left = n - len(out)
        if left <= 1 and total - wt(lo) <= chunk_rows:
            hi = T
        else:
            left = max(left, 2)
            hi = choose(lo, total - (left - 1) * chunk_rows, lo + -(-(T - lo) // left))
            if wt(hi) == total:
                hi = T
        out.append((lo, hi))
        lo = hi
    return out


def head_step_chunks(T, keep_logits_chunk, sequence_level, cu_seqlens, loss_mask_host=None):
    """The token ranges ``grpo_head_step`` walks: at most ``keep_logits_chunk`` kept rows each.  Only
    unmasked rows keep their logits, so with the mask known on the host (``loss_mask_host``, given when
    masked rows are skipped) the bound counts those; the sequence-level loss needs ranges that end on
    sequence boundaries (``cu_seqlens``: host list or device tensor, read only when a split is needed)."""
    live_cum = None
    if loss_mask_host is not None and T > 0:
        live_cum = np.concatenate([[0], np.cumsum(loss_mask_host.reshape(-1).numpy() != 0, dtype=np.int64)])
    rows_total = T if live_cum is None else int(live_cum[T])
    bounds = None
    if keep_logits_chunk is not None and keep_logits_chunk < rows_total and sequence_level:
        bounds = cu_seqlens.tolist() if isinstance(cu_seqlens, torch.Tensor) else list(cu_seqlens)
    return _token_chunks(T, keep_logits_chunk, bounds, live_cum)


def grpo_head_step(hidden, weight, labels, old_logprob, ref_logprob, advantages, cu_seqlens, loss_mask, *,
                   n_tokens_total: float, fsdp_size: int = 1, use_group_sequence_policy=False,
                   pos_clip_ratio=0.2, neg_clip_ratio=0.2, diff_clip_ratio=10, final_clip_ratio=3,
                   kl_coef=0.0, entropy_coef=0.0, temperature=1.0, dweight: Optional[torch.Tensor] = None,
                   accumulate_dweight=False, need_dhidden=True, check_flags=True,
                   keep_logits_chunk: Optional[int] = DEFAULT_KEEP_LOGITS_TOKENS, cu_seqlens_host=None,
                   skip_masked_rows=True, skip_masked_forward=False, weight_t_cache: Optional[dict] = None,
                   stage_hook=None, loss_mask_host: Optional[torch.Tensor] = None,
                   workspace_cache: Optional[dict] = None):
    """Forward + loss + backward of the head for one packed micro-batch, no autograd graph.

    Mirrors policy_trainer.py:216-286 on packed rows: returns a dict with the
    per-token ``logprob``/``entropy``, the loss scalars ``pg_loss_mean``,
    ``kl_loss_mean``, ``entropy_loss_mean``, ``total_loss`` (device fp64 scalars),
    ``dhidden`` and ``dweight``.  ``advantages`` is a device tensor [B].

    ``keep_logits_chunk``: the micro-batch is walked in token chunks that keep the raw logits of at most
    this many rows (one [chunk, V] buffer of 16-bit or fp32 elements, reused chunk after chunk) so that
    the backward does not recompute them.  Every token counts as a row, except that with
    ``skip_masked_rows`` and ``loss_mask_host`` only the unmasked tokens do (only they are kept).  ``None`` keeps nothing: the
    backward then recomputes the logit tiles from ``hidden`` and ``weight``.  The sequence-level
    loss needs chunks that end on sequence boundaries, so it reads ``cu_seqlens_host`` (or copies
    ``cu_seqlens`` to the host once).

    ``skip_masked_rows`` (only with kept logits and a loss mask): rows whose mask is zero have an
    exactly zero upstream gradient, so the backward runs on the compacted set of the other rows
    (their dhidden rows are zero); ``rows_projected_bwd`` in the result counts the rows it ran on.

    ``skip_masked_forward`` (off by default, needs ``skip_masked_rows``): also leave those rows out of
    the forward.  The loss, its sums and every gradient are unchanged (masked rows enter none of
    them), but the returned per-token ``logprob`` / ``entropy`` / ``lse`` are zero at masked rows
    instead of the values the reference computes and then ignores; ``rows_projected_fwd`` counts
    the rows the forward ran on.

    ``loss_mask_host``: a host copy of ``loss_mask`` (the trainer builds the mask on the host anyway).  With
    it the unmasked rows of every chunk are found on the host and sent over asynchronously; without it
    they are found on the device, which costs one host round trip per chunk for their count.

    ``weight_t_cache``: a dict the caller keeps while ``weight`` does not change (the micro-batches
    of one optimizer step).  The first backward leaves the transposed weight in it and later calls
    reuse it instead of transposing again; the caller clears it after updating the weight.

    ``workspace_cache``: a dict the caller keeps between calls.  The kept-logits buffer and the forward /
    backward scratch memory (a few GB, sized by the chunk, not by T) then live in it and are reused by every
    later call they are large enough for, instead of being allocated and released per call: micro-batches of
    varying length otherwise ask the framework's allocator for differently sized multi-GB blocks each time,
    which now and then costs a device-wide stall for a fresh allocation.

    ``stage_hook(name)`` is called on the host at "forward", "loss", "backward", "end" boundaries
    of every chunk (a benchmark records stream events there).
    """
    hook = stage_hook or (lambda name: None)
    T = hidden.shape[0]
    V = weight.shape[0]
    scale = float(fsdp_size) / float(n_tokens_total)
    mode = LOSS_GSPO if use_group_sequence_policy else LOSS_GRPO
    skip = keep_logits_chunk is not None and loss_mask is not None and skip_masked_rows
    chunks = head_step_chunks(T, keep_logits_chunk, use_group_sequence_policy,
                              cu_seqlens_host if cu_seqlens_host is not None else cu_seqlens,
                              loss_mask_host if skip else None)
    zbuf = None
    rows_of = None
    if skip and loss_mask_host is not None and T > 0:
        rows_of = _live_rows_from_host_mask(loss_mask_host, chunks, hidden.device)
    longest = max(hi - lo for lo, hi in chunks)
    cache = workspace_cache if workspace_cache is not None else {}

    def scratch(name, nbytes):
        buf = cache.get(name)
        if buf is None or buf.numel() < nbytes or buf.device != hidden.device:
            buf = cache[name] = torch.empty(nbytes, dtype=torch.uint8, device=hidden.device)
        return buf

    if keep_logits_chunk is not None and T > 0:
        kept = longest if rows_of is None else max(int(live.numel()) for live, _ in rows_of)
        zbuf = cache.get("kept_logits")
        if zbuf is None or zbuf.shape[0] < kept or zbuf.dtype != hidden.dtype or zbuf.device != hidden.device \
                or zbuf.shape[1] != ops.saved_logits_ld(V):
            zbuf = cache["kept_logits"] = ops.saved_logits_buffer(kept, V, hidden.dtype, hidden.device)
    # scratch memory of the forward and the backward, shared by all chunks of this call
    H = hidden.shape[1]
    fwd_ws = scratch("forward", max(ops.lmhead_forward_workspace_bytes(longest, H, V, hidden.dtype), 16)) if T > 0 else None
    bwd_rows = longest if zbuf is None else min(longest, zbuf.shape[0])
    bwd_ws = None
    f = dict(dtype=torch.float32, device=hidden.device)
    lp_all, ent_all, lse_all, glp_all = (torch.empty(T, **f) for _ in range(4))
    loss_all = torch.empty(T, dtype=advantages.dtype, device=hidden.device)
    kl_all = torch.empty(T, **f) if ref_logprob is not None else None
    dh_all = torch.empty_like(hidden) if need_dhidden else None
    sums = torch.zeros(8, dtype=torch.float64, device=hidden.device)
    flags = torch.zeros(1, dtype=torch.int32, device=hidden.device)
    dw = dweight
    acc_dw = accumulate_dweight
    rows_projected_bwd = 0
    rows_projected_fwd = 0
    wt, wt_ready = None, False
    if need_dhidden and weight_t_cache is not None:
        wt, wt_ready = weight_t_cache.get("weight_t"), weight_t_cache.get("weight_t") is not None
    if need_dhidden and wt is None and (len(chunks) > 1 or weight_t_cache is not None):
        wt = ops.weight_t_buffer(weight)
    if zbuf is not None:
        bwd_ws = scratch("backward", ops.lmhead_backward_workspace_bytes(bwd_rows, H, V, hidden.dtype, True, wt is not None))
    kl_c = kl_coef if kl_coef > 0 else 0.0
    en_c = entropy_coef if entropy_coef > 0 else 0.0
    for k, (lo, hi) in enumerate(chunks):
        sl = slice(lo, hi)
        n = hi - lo
        live = row_map = None
        if skip and n > 0:
            # Rows whose loss mask is zero get a zero upstream gradient whatever the logits are:
            # keep logits only for the others and run the backward on that compact set of rows.
            if rows_of is not None:
                live, row_map = rows_of[k]
            else:
                live = _nonzero_rows(loss_mask[sl])
                row_map = torch.full((n,), -1, dtype=torch.int32, device=hidden.device)
                row_map[live] = torch.arange(live.numel(), dtype=torch.int32, device=hidden.device)
        hook("forward")
        h_c = lab_c = None
        if live is not None and skip_masked_forward and live.numel() > 0:
            # forward on the compact set of unmasked rows; results scattered back, zeros elsewhere
            h_c, lab_c = ops.gather_rows(hidden[sl], live), ops.gather_rows(labels[sl].reshape(n, 1), live).reshape(-1)
            lp_c, ent_c, _, lse_c = ops.lmhead_forward(h_c, weight, lab_c, temperature, need_entropy=True,
                                                       saved_logits=zbuf, workspace=fwd_ws)
            spread = lambda x: ops.scatter_rows(x.reshape(-1, 1), live, n).reshape(-1)
            lp, ent, lse = spread(lp_c), spread(ent_c), spread(lse_c)
            rows_projected_fwd += int(live.numel())
        else:
            lp, ent, _, lse = ops.lmhead_forward(hidden[sl], weight, labels[sl], temperature, need_entropy=True,
                                                 saved_logits=zbuf, saved_row_map=row_map, workspace=fwd_ws)
            rows_projected_fwd += n
        hook("loss")
        res = ops.policy_loss(
            lp, old_logprob[sl], advantages, mode=mode, cu_seqlens=cu_seqlens,
            ref_logprob=None if ref_logprob is None else ref_logprob[sl], entropy=ent,
            loss_mask=None if loss_mask is None else loss_mask[sl], diff_clip_ratio=diff_clip_ratio,
            pos_clip_ratio=pos_clip_ratio, neg_clip_ratio=neg_clip_ratio, final_clip_ratio=final_clip_ratio,
            kl_coef=kl_c, entropy_coef=en_c, grad_scale=scale, want_dloss=False, want_upstream=True,
            token_offset=lo)
        hook("backward")
        if live is None:
            dh, dw = ops.lmhead_backward(hidden[sl], weight, labels[sl], lse, ent, res.g_logprob, res.g_entropy,
                                         temperature, need_dhidden=need_dhidden, need_dweight=True, dweight=dw,
                                         accumulate_dweight=acc_dw, saved_logits=zbuf, weight_t=wt,
                                         weight_t_ready=wt_ready, workspace=bwd_ws)
            wt_ready = True
        elif live.numel() == 0:
            dh = torch.zeros_like(hidden[sl]) if need_dhidden else None
            if not acc_dw:
                dw = torch.zeros(V, hidden.shape[1], dtype=torch.float32, device=hidden.device) if dw is None \
                    else dw.zero_()
            rows_projected_bwd -= n
        else:
            pick = lambda x: None if x is None else ops.gather_rows(x.reshape(n, -1), live).reshape(-1)
            if h_c is None:
                h_c, lab_c = ops.gather_rows(hidden[sl], live), pick(labels[sl])
            dh_c, dw = ops.lmhead_backward(
                h_c, weight, lab_c, pick(lse), pick(ent),
                pick(res.g_logprob), pick(res.g_entropy), temperature, need_dhidden=need_dhidden,
                need_dweight=True, dweight=dw, accumulate_dweight=acc_dw, saved_logits=zbuf, weight_t=wt,
                weight_t_ready=wt_ready, workspace=bwd_ws)
            wt_ready = True
            dh = ops.scatter_rows(dh_c, live, n) if need_dhidden else None
            rows_projected_bwd += int(live.numel()) - n
        rows_projected_bwd += n
        hook("end")
        acc_dw = True
        if weight_t_cache is not None and wt_ready:
            weight_t_cache["weight_t"] = wt
        lp_all[sl], ent_all[sl], lse_all[sl], glp_all[sl], loss_all[sl] = lp, ent, lse, res.g_logprob, res.loss
        if kl_all is not None:
            kl_all[sl] = res.kl
        if need_dhidden:
            dh_all[sl] = dh
        sums += res.sums
        flags |= res.flags
    if check_flags:
        fl = int(flags.item())
        assert not fl & 1, "pg loss is nan"
        assert not fl & 2, "kl loss ratio has inf values"
        assert not fl & 4, "kl loss ratio has nan values"
    pg = sums[0] * scale
    kl = sums[1] * scale
    en = sums[2] * scale
    total = pg
    if entropy_coef > 0:
        total = total - entropy_coef * en
    if kl_coef > 0:
        total = total + kl_coef * kl
    return {"logprob": lp_all, "entropy": ent_all, "lse": lse_all, "pg_loss_mean": pg, "kl_loss_mean": kl,
            "entropy_loss_mean": en, "total_loss": total, "num_masked": sums[3],
            "per_token_loss": loss_all, "per_token_kl": kl_all, "dhidden": dh_all, "dweight": dw,
            "g_logprob": glp_all, "rows_projected_bwd": rows_projected_bwd,
            "rows_projected_fwd": rows_projected_fwd, "sums": sums, "token_chunks": chunks,
            # device memory this call held beyond its inputs and outputs: kept logits (they become d(logits) in
            # place), the backward's operands (d(logits)^T, hidden^T, W^T unless the caller's cache holds it,
            # split-K partials) and the forward's per-split records
            "scratch_bytes": sum(t.numel() * t.element_size() for t in (zbuf, fwd_ws, bwd_ws) if t is not None)
                             + (wt.numel() * wt.element_size() if wt is not None else 0)
                             + (0 if (zbuf is not None or T == 0) else min(
                                 ops.lmhead_backward_workspace_bytes(longest, H, V, hidden.dtype, False, wt is not None),
                                 ops.DEFAULT_BWD_WORKSPACE_BYTES))}
