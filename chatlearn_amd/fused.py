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


# Memory one chunk's kept logits may take (they are turned into d(logits) in place; the backward's transposed
# copy takes as much again).  The bound is on bytes, whatever the hidden size: 35328 rows of a 152k
# vocabulary, 41472 rows of a 129k one, in 16-bit elements - a 32768-token micro-batch in one chunk.  Only
# what a micro-batch needs is allocated.
DEFAULT_KEEP_LOGITS_BYTES = 10 << 30
AUTO = "auto"


def default_keep_rows(V: int, dtype) -> int:
    """Rows whose logits fit DEFAULT_KEEP_LOGITS_BYTES: a multiple of 256 (the kept-logits buffer is cut
    into blocks of 256 rows), at least 256."""
    es = torch.empty(0, dtype=dtype).element_size()
    rows = DEFAULT_KEEP_LOGITS_BYTES // (ops.saved_logits_ld(V) * es)
    return max(256, rows // 256 * 256)


def _resolve_keep(keep, V, dtype):
    return default_keep_rows(V, dtype) if isinstance(keep, str) and keep == AUTO else keep


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


def _host_live_rows(mask_host, T):
    """Ascending positions of the nonzero entries of a host copy of the loss mask (numpy int64)."""
    if not isinstance(mask_host, torch.Tensor) or mask_host.is_cuda:
        raise TypeError("loss_mask_host must be a CPU tensor")
    if mask_host.numel() != T:
        raise ValueError(f"loss_mask_host has {mask_host.numel()} entries for {T} tokens")
    return np.flatnonzero(mask_host.reshape(-1).numpy() != 0).astype(np.int64)


class _FusedHead(torch.autograd.Function):
    """Rows that carry a gradient ("live": all rows, or the unmasked ones when the caller hands in the loss
    mask) are split in two: the first ``keep_rows`` of them keep their logits in the forward, and their
    backward runs from those; the others are recomputed in the backward.  Both parts add into one dW."""

    @staticmethod
    def forward(ctx, hidden, weight, labels, temperature, need_entropy, dweight_buffer, keep_rows, row_mask, mask_host):
        T = hidden.shape[0]
        dev = hidden.device
        zbuf = row_map = None
        live = None            # device int64 positions of the live rows; None: every row
        n_live = T
        if T > 0:
            if mask_host is not None:
                live_h = _host_live_rows(mask_host, T)          # no device value is read back
                n_live = int(live_h.size)
                live = _upload(torch.from_numpy(live_h), dev) if n_live else torch.empty(0, dtype=torch.int64, device=dev)
            elif row_mask is not None:
                live = _nonzero_rows(row_mask)                  # one host round trip for the count
                n_live = int(live.numel())
        n_kept = 0 if keep_rows is None else min(int(keep_rows), n_live)
        if n_kept > 0:
            zbuf = ops.saved_logits_buffer(n_kept, weight.shape[0], hidden.dtype, dev)
            if live is not None:
                row_map = torch.full((T,), -1, dtype=torch.int32, device=dev)
                row_map[live[:n_kept]] = torch.arange(n_kept, dtype=torch.int32, device=dev)
        lp, ent, _, lse = ops.lmhead_forward(hidden, weight, labels, temperature, need_entropy,
                                             saved_logits=zbuf, saved_row_map=row_map)
        ctx.save_for_backward(hidden, weight, labels, lse, ent if ent is not None else lse)
        ctx.set_materialize_grads(False)
        ctx.temperature = temperature
        ctx.has_entropy = ent is not None
        ctx.dweight_buffer = dweight_buffer
        ctx.zbuf, ctx.live, ctx.n_live, ctx.n_kept = zbuf, live, n_live, n_kept
        if ent is None:
            ent = torch.zeros(0, device=dev)
            ctx.mark_non_differentiable(ent)
        return lp, ent

    @staticmethod
    def backward(ctx, g_lp, g_ent):
        hidden, weight, labels, lse, ent = ctx.saved_tensors
        need_h, need_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        zbuf, live, n_live, n_kept = ctx.zbuf, ctx.live, ctx.n_live, ctx.n_kept
        ctx.zbuf = None                      # the buffer is consumed (overwritten) by this backward
        if zbuf is None:
            n_kept = 0                       # a second backward through a retained graph recomputes
        none = (None,) * 9
        if g_lp is None and g_ent is None:
            return none
        if g_lp is None:
            g_lp = torch.zeros_like(lse)
        use_ent = ctx.has_entropy and g_ent is not None
        g_lp = g_lp.float().contiguous()
        g_ent = g_ent.float().contiguous() if use_ent else None
        ent = ent if use_ent else None
        T = hidden.shape[0]
        dw_buf = ctx.dweight_buffer
        if n_live == 0:
            dh = torch.zeros_like(hidden) if need_h else None
            dw = torch.zeros(weight.shape, dtype=weight.dtype, device=hidden.device) if (need_w and dw_buf is None) else None
            return (dh, dw) + (None,) * 7

        def part(lo, hi, saved, dweight, accumulate):
            """Backward of live rows [lo, hi) (in live order): from kept logits, or recomputing them."""
            if live is None:
                pick = lambda x: None if x is None else x[lo:hi]
            else:
                idx = live[lo:hi]
                pick = lambda x: None if x is None else ops.gather_rows(x.reshape(T, -1), idx).reshape((hi - lo,) + x.shape[1:])
            return ops.lmhead_backward(pick(hidden), weight, pick(labels), pick(lse), pick(ent), pick(g_lp), pick(g_ent),
                                       ctx.temperature, need_dhidden=need_h, need_dweight=need_w, dweight=dweight,
                                       accumulate_dweight=accumulate, saved_logits=saved)

        dw, acc = dw_buf, dw_buf is not None
        pieces = []
        for lo, hi, saved in ((0, n_kept, zbuf), (n_kept, n_live, None)):
            if hi > lo:
                dh_p, dw = part(lo, hi, saved, dw, acc)
                acc = True
                pieces.append(dh_p)
        dh = None
        if need_h:
            dh_c = pieces[0] if len(pieces) == 1 else torch.cat(pieces, 0)
            dh = dh_c if live is None else ops.scatter_rows(dh_c, live, T)
        if dw is not None:
            # A caller-supplied fp32 main-grad buffer was accumulated in place; autograd gets no copy.
            dw = None if dw_buf is not None else dw.to(weight.dtype)
        return (dh, dw) + (None,) * 7


def fused_linear_logprob_entropy(hidden: torch.Tensor, weight: torch.Tensor, labels: torch.Tensor, *,
                                 temperature: float = 1.0, need_entropy: bool = True,
                                 dweight_buffer: Optional[torch.Tensor] = None,
                                 keep_logits_rows=AUTO, loss_mask: Optional[torch.Tensor] = None,
                                 loss_mask_host: Optional[torch.Tensor] = None):
    """(logprob fp32 [T], entropy fp32 [T]) of ``labels`` under softmax(hidden @ weight.T / temperature).

    hidden [T,H] and weight [V,H] share a dtype (bf16 or fp32), labels int64 [T].
    ``dweight_buffer``: optional fp32 [V,H] tensor that receives ``+= dW`` in the
    backward (the fp32 gradient accumulation FSDP2 does with ``reduce_dtype=fp32``);
    without it ``weight.grad`` gets dW cast to the weight dtype, as torch would.
    Leading dimensions of hidden/labels are flattened and restored.

    ``keep_logits_rows``: when a gradient is needed, the forward keeps the raw logits of up to this many
    rows (one 16-bit copy for 16-bit inputs, released by the backward) so that the backward does not
    recompute them; rows beyond the bound are recomputed in the backward, tile by tile, and both parts
    add into one dW.  ``"auto"`` (the default) bounds the kept logits at ``DEFAULT_KEEP_LOGITS_BYTES``;
    ``None`` keeps nothing.  A caller that owns the training loop can instead run the head chunk by
    chunk (forward, loss, backward per chunk), which is what ``grpo_head_step`` does.

    ``loss_mask`` (same shape as ``labels``) is a promise that rows where it is zero receive a zero
    upstream gradient - true of the reference's loss, which multiplies by this mask
    (policy_trainer.py:259-283): their logits are then not kept and the backward runs on the other
    rows only.  ``loss_mask_host`` is a CPU copy of the same mask (the trainer builds the mask on the
    host anyway): with it the unmasked rows are found on the host and nothing is read back from the
    device; with the device mask alone, their count costs one host round trip.
    """
    lead = labels.shape
    h2 = hidden.reshape(-1, hidden.shape[-1])
    needs_grad = torch.is_grad_enabled() and (hidden.requires_grad or weight.requires_grad)
    keep = _resolve_keep(keep_logits_rows, weight.shape[0], hidden.dtype) if needs_grad else None
    mask = host = None
    if needs_grad:                 # the masks only matter to the backward (and to which rows keep their logits)
        host = loss_mask_host
        if loss_mask is not None and host is None:
            mask = loss_mask.reshape(-1).to(torch.int32)
    lp, ent = _FusedHead.apply(h2, weight, labels.reshape(-1), float(temperature), bool(need_entropy), dweight_buffer,
                               keep, mask, host)
    lp = lp.reshape(lead)
    ent = ent.reshape(lead) if need_entropy else None
    return lp, ent


def _token_chunks(T, chunk_rows, seq_bounds, live_cum=None, n_ranges=None):
    """[lo, hi) token ranges holding at most ``chunk_rows`` rows each: as few ranges as that allows, and
    of about equal length in tokens (the forward runs on every token of a range; a short last range would
    run all kernels at poor efficiency).  A token counts as a row, unless ``live_cum`` is given (a numpy
    array, live_cum[i] = rows among tokens [0, i) whose logits are kept, i.e. the unmasked ones): then the
    bound is on those.  With ``seq_bounds`` (the host copy of cu_seqlens) every range ends on a sequence
    boundary (a range exceeds ``chunk_rows`` only where a single sequence is larger than it), otherwise
    on a multiple of 256 tokens where the bound leaves room for that.  ``n_ranges`` asks for that many
    ranges instead of the fewest (it is raised to the fewest when smaller)."""
    total = T if live_cum is None else int(live_cum[T])
    if T == 0 or ((chunk_rows is None or chunk_rows >= total) and (n_ranges is None or n_ranges <= 1)):
        return [(0, T)]
    if chunk_rows is None or chunk_rows > total:
        chunk_rows = max(total, 1)                                 # no bound on the rows: only the number of ranges is asked for
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
    if n_ranges is not None:
        n = max(n, int(n_ranges))
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


def _launch_cost(chunks, live_cum, H, V, dtype=torch.bfloat16, cus=256):
    """Relative time of the three GEMM-shaped passes of every chunk, in units of one 256 x 256 tile over one
    K element on one CU: a launch of n work items takes ceil(n / cus) rounds.  Asks the library for its
    launch plans (vocabulary splits of the forward, bulk / K-split launches of the dhidden and dW GEMMs);
    the passes that do not depend on the cuts (d(logits), transposes) are left out, the read of dW's previous contents by every chunk after the first is counted."""
    n_vt = -(-V // 256)
    n_ht = -(-H // 256)
    cost = 0.0
    for k, (lo, hi) in enumerate(chunks):
        rows = (hi - lo) if live_cum is None else int(live_cum[hi] - live_cum[lo])
        n_tb, _, tps = ops.lmhead_forward_launch_plan(hi - lo, V, cus)
        cost += -(-(n_tb * -(-n_vt // tps)) // cus) * tps * H
        if rows == 0:
            continue
        bulk_nt, ks = ops.dhidden_launch_plan(rows, H, V, dtype, cus)
        n_rt = -(-rows // 256)
        if bulk_nt:
            cost += -(-(bulk_nt * n_ht) // cus) * V
        cost += -(-((n_rt - bulk_nt) * n_ht * ks) // cus) * (V / ks)
        n_walk, bulk_vt, ks_w = ops.dweight_launch_plan(rows, H, V, dtype, cus)   # dW: walks over vocabulary tiles, K-split tail
        if bulk_vt:
            cost += (bulk_vt // n_walk) * rows + -(-((n_vt - bulk_vt) * n_ht * ks_w) // cus) * (rows / ks_w)
        else:
            cost += (-(-n_vt // n_walk) if n_walk else -(-(n_vt * n_ht) // cus)) * rows
        if k > 0:
            cost += 0.15 * n_vt * n_ht / cus * 2048            # re-reading dW [V,H] fp32: HBM time in the same unit
    return cost


def head_step_chunks(T, keep_logits_chunk, sequence_level, cu_seqlens, loss_mask_host=None, shape=None,
                     dtype=torch.bfloat16, chunk_hidden_bytes=None):
    """The token ranges ``grpo_head_step`` walks: at most ``keep_logits_chunk`` kept rows each.  Only
    unmasked rows keep their logits, so with the mask known on the host (``loss_mask_host``, given when
    masked rows are skipped) the bound counts those; the sequence-level loss needs ranges that end on
    sequence boundaries (``cu_seqlens``: host list or device tensor, read only when a split is needed).
    With ``shape`` = (H, V) the number of ranges is the fewest the bound allows or up to two more,
    whichever fills the CUs best over the forward and the two backward GEMMs (a launch takes whole
    rounds of one workgroup per CU; ragged sequence-aligned ranges can leave a round nearly empty).
    ``chunk_hidden_bytes`` (with ``shape``) also bounds the hidden states of a range."""
    live_cum = None
    if loss_mask_host is not None and T > 0:
        live_cum = np.concatenate([[0], np.cumsum(loss_mask_host.reshape(-1).numpy() != 0, dtype=np.int64)])
    rows_total = T if live_cum is None else int(live_cum[T])
    min_ranges = 1
    if chunk_hidden_bytes and shape is not None and T > 0:
        row_bytes = shape[0] * (2 if dtype != torch.float32 else 4)
        min_ranges = max(1, -(-(T * row_bytes) // int(chunk_hidden_bytes)))
    split = (keep_logits_chunk is not None and keep_logits_chunk < rows_total) or min_ranges > 1
    bounds = None
    if split and sequence_level:
        bounds = cu_seqlens.tolist() if isinstance(cu_seqlens, torch.Tensor) else list(cu_seqlens)
    fewest = _token_chunks(T, keep_logits_chunk, bounds, live_cum, n_ranges=min_ranges if min_ranges > 1 else None)
    if shape is None or len(fewest) == 1:
        return fewest
    H, V = shape
    best, best_cost = fewest, _launch_cost(fewest, live_cum, H, V, dtype)
    for extra in (1, 2):
        cand = _token_chunks(T, keep_logits_chunk, bounds, live_cum, n_ranges=len(fewest) + extra)
        if len(cand) != len(fewest) + extra:
            continue
        c = _launch_cost(cand, live_cum, H, V, dtype)
        if c < 0.98 * best_cost:                                # more ranges must buy more than 2 %
            best, best_cost = cand, c
    return best


def grpo_head_step(hidden, weight, labels, old_logprob, ref_logprob, advantages, cu_seqlens, loss_mask, *,
                   n_tokens_total: float, fsdp_size: int = 1, use_group_sequence_policy=False,
                   pos_clip_ratio=0.2, neg_clip_ratio=0.2, diff_clip_ratio=10, final_clip_ratio=3,
                   kl_coef=0.0, entropy_coef=0.0, temperature=1.0, dweight: Optional[torch.Tensor] = None,
                   accumulate_dweight=False, need_dhidden=True, check_flags=True,
                   keep_logits_chunk=AUTO, cu_seqlens_host=None,
                   skip_masked_rows=True, skip_masked_forward=False, weight_t_cache: Optional[dict] = None,
                   stage_hook=None, loss_mask_host: Optional[torch.Tensor] = None,
                   workspace_cache: Optional[dict] = None, chunk_hidden_bytes: Optional[int] = None):
    """Forward + loss + backward of the head for one packed micro-batch, no autograd graph.

    Mirrors policy_trainer.py:216-286 on packed rows: returns a dict with the
    per-token ``logprob``/``entropy``, the loss scalars ``pg_loss_mean``,
    ``kl_loss_mean``, ``entropy_loss_mean``, ``total_loss`` (device fp64 scalars),
    ``dhidden`` and ``dweight``.  ``advantages`` is a device tensor [B].

    ``keep_logits_chunk``: the micro-batch is walked in token chunks that keep the raw logits of at most
    this many rows (one [chunk, V] buffer of 16-bit or fp32 elements, reused chunk after chunk) so that
    the backward does not recompute them; ``"auto"`` (the default) bounds that buffer at
    ``DEFAULT_KEEP_LOGITS_BYTES``.  Every token counts as a row, except that with
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

    ``chunk_hidden_bytes``: a chunk's hidden states are also kept below this many bytes (``None``, the
    default: no such bound).  It paid at H = 7168 (two chunks of 16384 tokens against one of 32768) only while
    the forward's workgroups of different XCDs worked on vocabulary ranges far apart.

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
    keep_logits_chunk = _resolve_keep(keep_logits_chunk, V, hidden.dtype)
    scale = float(fsdp_size) / float(n_tokens_total)
    mode = LOSS_GSPO if use_group_sequence_policy else LOSS_GRPO
    skip = keep_logits_chunk is not None and loss_mask is not None and skip_masked_rows
    if loss_mask_host is not None and (loss_mask_host.is_cuda or loss_mask_host.numel() != T):
        raise ValueError(f"loss_mask_host must be a CPU copy of loss_mask with {T} entries")
    chunks = head_step_chunks(T, keep_logits_chunk, use_group_sequence_policy,
                              cu_seqlens_host if cu_seqlens_host is not None else cu_seqlens,
                              loss_mask_host if skip else None, shape=(hidden.shape[1], V), dtype=hidden.dtype,
                              chunk_hidden_bytes=chunk_hidden_bytes if keep_logits_chunk is not None else None)
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
        # one read-back for the reference's three assertions and the host mask's consistency
        fl, n_masked = (int(x) for x in torch.stack([flags[0].double(), sums[3]]).tolist())
        assert not fl & 1, "pg loss is nan"
        assert not fl & 2, "kl loss ratio has inf values"
        assert not fl & 4, "kl loss ratio has nan values"
        if rows_of is not None and loss_mask is not None:
            n_host = int(loss_mask_host.sum())
            if n_host != n_masked:
                raise ValueError(f"loss_mask_host sums to {n_host}, the device loss_mask to {n_masked}: "
                                 "the host copy is stale or laid out differently")
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
