#!/usr/bin/env python3
"""Benchmark of the fused logprob + GRPO loss head path (forward + backward).

One step = one packed micro-batch through: fused lm_head forward (logprob, entropy, lse), the
policy-loss kernel (loss sums + per-token upstream grads) and the fused backward (dhidden bf16,
dW fp32), walked in token chunks so that only one chunk's logits are ever kept.  Default workload:
the Qwen3-8B head (H=4096, V=151936, bf16) on a 16384-token micro-batch, inputs resident in HBM.

Prints ONE JSON line:  metric/value/unit per the driver contract, plus
  roofline        - the forward kernel against the bf16 MFMA peak (HIP-event timed, live)
  gemm_kernels    - forward / dhidden / dW, each against the peak on the rows it actually ran
  step_mfma_frac_executed - flops the step executed (forward rows + 2 x backward rows) / time / peak
  loss_stage      - bytes, GB/s and launches of the loss stage
  variants        - the same step with other chunk sizes, without row skipping, with recomputation
  sweep           - all micro-batches of the configuration, built by the library's bin packing
  other_configs   - the other benchmark configurations, compactly
  cpu_baseline    - the torch oracle (reference op order) timed on the host cores on a row sample
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from chatlearn_amd import _lib, ops, synthetic  # noqa: E402
from chatlearn_amd._lib import LOSS_GRPO, LOSS_GSPO  # noqa: E402
from chatlearn_amd.fused import default_keep_rows, grpo_head_step, head_step_chunks  # noqa: E402

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_F32_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0

# HBM-side bytes per forward launch are read from this summary of two rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE,
# copy-calibrated); its line "bench.roofline.traffic {json}" maps "<config>:<tokens per launch>:<logits kept 0|1>" to bytes.
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "lmhead_fwd_c2_pmc_fetch_write.txt")


def measured_traffic(cfg_name, tokens_per_launch, kept):
    try:
        with open(TRAFFIC_SUMMARY) as f:
            for line in f:
                if "bench.roofline.traffic" in line:
                    table = json.loads(line.split("bench.roofline.traffic", 1)[1])
                    return table.get(f"{cfg_name}:{tokens_per_launch}:{int(bool(kept))}")
    except (OSError, ValueError):
        pass
    return None


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def peak_of(cfg):
    return PEAK_BF16_TFLOPS if cfg.dtype == torch.bfloat16 else PEAK_F32_TFLOPS


class Workload:
    """One packed micro-batch of a configuration, resident on the device."""

    def __init__(self, cfg, device, samples=None):
        self.cfg = cfg
        gen = synthetic.generator_for(cfg)
        if samples is None:
            samples = synthetic.fill_microbatch(cfg, synthetic.sample_population(cfg, gen))
        self.samples = samples
        cu, mask = synthetic.packed_layout(samples)
        self.T = int(cu[-1])
        self.mask_host = mask
        self.cu, self.mask = cu.to(device), mask.to(device)
        self.cu_host = cu.tolist()
        self.n_tok = float(mask.sum().item())
        self.device = device
        self.hidden = self.weight = self.labels = self.adv = self.old = self.ref = None

    def tensors(self):
        self.hidden, self.weight, self.labels = synthetic.make_head_tensors(
            self.cfg, self.T, synthetic.generator_for(self.cfg), device=self.device, device_generate=True)
        return self

    def finish(self):
        """Advantages through the library's AdvantageComputer mirror; old / ref logprobs around the model's own."""
        if self.adv is None:
            self.adv = advantages_for(self.samples, self.device)
        lp0, *_ = ops.lmhead_forward(self.hidden, self.weight, self.labels, self.cfg.temperature, need_entropy=False)
        self.old, self.ref = synthetic.noisy_logprobs(lp0, synthetic.generator_for(self.cfg))
        return self


def advantages_for(samples, device, group=1 << 30):
    """Group mean/std advantages through the library's AdvantageComputer mirror."""
    from chatlearn_amd.algorithm.grpo_utils.advantage_compute import AdvantageComputer

    class _Buf:
        def __init__(self, b):
            self.buffer = b
    pop = [dict(s) for s in samples]
    AdvantageComputer(num_inference_per_prompt=group)([_Buf(pop)])
    return torch.tensor([float(s["advantages"]) for s in pop], dtype=torch.float32, device=device)


def head_step(w, keep, dweight, *, skip_masked=True, skip_masked_forward=False, hook=None, accumulate=False,
              weight_t_cache=None, n_tok=None, workspace_cache=None, check_flags=True):
    cfg = w.cfg
    return grpo_head_step(w.hidden, w.weight, w.labels, w.old, w.ref, w.adv, w.cu, w.mask,
                          n_tokens_total=n_tok or w.n_tok, use_group_sequence_policy=(cfg.loss == "gspo"),
                          pos_clip_ratio=cfg.pos_clip_ratio, neg_clip_ratio=cfg.neg_clip_ratio,
                          diff_clip_ratio=cfg.diff_clip_ratio, final_clip_ratio=cfg.final_clip_ratio, kl_coef=cfg.kl_coef,
                          entropy_coef=cfg.entropy_coef, temperature=cfg.temperature, dweight=dweight,
                          accumulate_dweight=accumulate, keep_logits_chunk=keep, cu_seqlens_host=w.cu_host,
                          skip_masked_rows=skip_masked, skip_masked_forward=skip_masked_forward, stage_hook=hook,
                          loss_mask_host=w.mask_host, weight_t_cache=weight_t_cache, check_flags=check_flags,
                          workspace_cache=workspace_cache)


def time_step(w, keep, dweight, steps, warmup, **kw):
    """(seconds per step, per-stage ms from stream events, last result).  Training configurations: per token
    chunk, fused forward (keeping the chunk's logits), loss + upstream gradients, fused backward (dhidden, dW
    accumulated).  The no-grad configuration: fused forward only."""
    cfg = w.cfg
    marks = []
    ws_cache = {}     # kept logits and scratch memory stay allocated between the steps, as a trainer's loop keeps them

    def once(record):
        if cfg.loss is None:
            e = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
            e[0].record()
            ops.lmhead_forward(w.hidden, w.weight, w.labels, cfg.temperature, need_entropy=True)
            e[1].record()
            if record:
                marks.append([("forward", e[0]), ("end", e[1])])
            return None
        cur = []

        def hook(name):
            ev = torch.cuda.Event(enable_timing=True)
            ev.record()
            cur.append((name, ev))
        out = head_step(w, keep, dweight, hook=hook if record else None, workspace_cache=ws_cache, **kw)
        if record:
            marks.append(cur)
        return out

    last = None
    for _ in range(warmup):
        last = once(False)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        last = once(True)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps

    def stage(name):
        tot = 0.0
        for cur in marks:
            for (a, ea), (_, eb) in zip(cur[:-1], cur[1:]):
                if a == name:
                    tot += ea.elapsed_time(eb)
        return tot / len(marks)
    return dt, {"forward": stage("forward"), "loss": stage("loss"), "backward": stage("backward")}, last


def step_record(w, keep, dt, stages, out):
    """Figures of one timed variant of the step."""
    cfg = w.cfg
    train = cfg.loss is not None
    T = w.T
    chunks = out["token_chunks"] if train else [(0, T)]
    rows_fwd = out["rows_projected_fwd"] if train else T
    rows_bwd = out["rows_projected_bwd"] if train else 0
    hv = float(cfg.H) * cfg.V
    executed = 2.0 * hv * (rows_fwd + 2.0 * rows_bwd)
    rec = {"tokens_per_s": T / dt, "ms_per_step": dt * 1e3, "token_chunks": [hi - lo for lo, hi in chunks],
           "T_projected_forward": rows_fwd, "T_projected_backward": rows_bwd,
           "step_mfma_frac_executed": executed / dt / 1e12 / peak_of(cfg),
           "stage_ms": {k: round(v, 3) for k, v in stages.items()}}
    if train:
        rec["scratch_bytes"] = int(out["scratch_bytes"])
    return rec


def cpu_baseline(cfg, rows, threads):
    """The oracle (torch, reference op order: linear -> log_softmax+gather -> chunked entropy ->
    GRPO/GSPO loss -> masked sums -> backward) on the host cores, fp32, on `rows` packed tokens."""
    from oracle import losses as ol
    from oracle import softmax_stats as osm
    torch.set_num_threads(threads)
    g = torch.Generator().manual_seed(cfg.seed)
    hidden = torch.randn(rows, cfg.H, generator=g).requires_grad_(cfg.loss is not None)
    weight = (torch.randn(cfg.V, cfg.H, generator=g) * cfg.w_std).requires_grad_(cfg.loss is not None)
    labels = torch.randint(0, cfg.V, (1, rows), generator=g)
    old = torch.full((1, rows), -12.0)
    ref = torch.full((1, rows), -12.0)
    mask = torch.ones(1, rows, dtype=torch.int32)

    def step():
        logits = torch.nn.functional.linear(hidden, weight).unsqueeze(0) / cfg.temperature
        lp = osm.logprobs_from_logits(logits, labels)
        if cfg.loss is None:
            with torch.no_grad():
                osm.entropy_from_logits_with_chunking(logits)
            return
        ctx = torch.enable_grad() if cfg.entropy_coef > 0 else torch.no_grad()
        with ctx:
            ent = osm.entropy_from_logits_with_chunking(logits)
        total, _ = ol.fsdp_policy_loss(lp, ent, old, ref, [0.5], mask, float(rows), entropy_coef=cfg.entropy_coef,
                                       kl_coef=cfg.kl_coef, pos_clip_ratio=cfg.pos_clip_ratio,
                                       neg_clip_ratio=cfg.neg_clip_ratio, final_clip_ratio=cfg.final_clip_ratio,
                                       use_group_sequence_policy=(cfg.loss == "gspo"))
        total.backward()
        hidden.grad = None
        weight.grad = None

    ctx = torch.no_grad() if cfg.loss is None else torch.enable_grad()
    with ctx:
        step()  # warm-up
        t0 = time.perf_counter()
        reps = 0
        while reps < 2 or time.perf_counter() - t0 < 10.0:
            step()
            reps += 1
            if time.perf_counter() - t0 > 30.0:
                break
        dt = (time.perf_counter() - t0) / reps
    return rows / dt, reps


def unfused_gpu(w, steps):
    """What the reference's FSDP trainer does today, on the same GPU in bf16: materialised logits,
    log_softmax + gather, chunked entropy, re-padding to [B,S], torch loss ops, autograd backward
    (policy_trainer.py:216-286)."""
    from oracle import indexing as oi
    from oracle import losses as ol
    from oracle import softmax_stats as osm
    cfg = w.cfg
    h = w.hidden.detach().clone().requires_grad_(True)
    wt = w.weight.detach().clone().requires_grad_(True)
    lab = w.labels.view(1, -1)
    lens = (w.cu[1:] - w.cu[:-1]).long()
    B, S = lens.numel(), int(lens.max())
    ar = torch.arange(S, device=h.device)
    attn = (ar.unsqueeze(0) < lens.unsqueeze(1))
    indices = torch.nonzero(attn.flatten(), as_tuple=False).flatten()
    pad = lambda x: oi.pad_input(x.unsqueeze(-1), indices, B, S).squeeze(-1)
    old_p, ref_p, mask_p = pad(w.old), pad(w.ref), pad(w.mask)
    adv_list = w.adv.tolist()

    def step():
        logits = torch.nn.functional.linear(h, wt).unsqueeze(0)
        if cfg.temperature != 1.0:
            logits = logits / cfg.temperature
        lp = osm.logprobs_from_logits(logits, lab)
        with (torch.enable_grad() if cfg.entropy_coef > 0 else torch.no_grad()):
            ent = osm.entropy_from_logits_with_chunking(logits)
        total, _ = ol.fsdp_policy_loss(pad(lp[0].float()), pad(ent[0]), old_p, ref_p, adv_list, mask_p, w.n_tok,
                                       entropy_coef=cfg.entropy_coef, kl_coef=cfg.kl_coef,
                                       pos_clip_ratio=cfg.pos_clip_ratio, neg_clip_ratio=cfg.neg_clip_ratio,
                                       diff_clip_ratio=cfg.diff_clip_ratio, final_clip_ratio=cfg.final_clip_ratio,
                                       use_group_sequence_policy=(cfg.loss == "gspo"))
        total.backward()
        h.grad = None
        wt.grad = None

    step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def library_gemms(hidden, weight, reps=5):
    """Plain library GEMMs (no softmax, logits materialised) at the head shape: the practical
    ceiling of this GPU's matrix cores under sustained load, for context next to the fused kernels."""
    T, H = hidden.shape
    V = weight.shape[0]
    flops = 2.0 * T * H * V

    def timed(fn):
        fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return flops / (e0.elapsed_time(e1) / reps * 1e-3) / 1e12
    z = torch.nn.functional.linear(hidden, weight)
    return {"unit": "TFLOP/s", "logits = hidden @ W^T": timed(lambda: torch.nn.functional.linear(hidden, weight)),
            "dhidden = dlogits @ W": timed(lambda: z @ weight), "dW = dlogits^T @ hidden": timed(lambda: z.t() @ hidden)}


def _events(fn, reps, setup=None):
    """Average milliseconds of fn() between stream events; setup() runs untimed before every repetition."""
    tot = 0.0
    for _ in range(reps):
        if setup:
            setup()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        torch.cuda.synchronize()
        tot += e0.elapsed_time(e1)
    return tot / reps


def gemm_kernels(w, keep, reps=3):
    """The three GEMM-shaped kernels on the largest token chunk of the step, each against the matrix-core peak
    on the rows it ran: the forward launch timed directly; dhidden and dW as the differences between the
    whole backward of the chunk and the backward without that output (what remains in either is the
    d(logits) pass and a transpose)."""
    cfg = w.cfg
    chunks = head_step_chunks(w.T, keep, cfg.loss == "gspo", w.cu_host, w.mask_host, shape=(cfg.H, cfg.V), dtype=cfg.dtype)
    lo, hi = max(chunks, key=lambda c: c[1] - c[0])
    n = hi - lo
    dev = w.device
    live = torch.nonzero(w.mask_host[lo:hi]).flatten().to(dev)
    rows = int(live.numel())
    row_map = torch.full((n,), -1, dtype=torch.int32, device=dev)
    row_map[live] = torch.arange(rows, dtype=torch.int32, device=dev)
    zbuf = ops.saved_logits_buffer(rows, cfg.V, cfg.dtype, dev)
    wt = ops.weight_t_buffer(w.weight)
    hidden, labels = w.hidden[lo:hi], w.labels[lo:hi]
    state = {}

    def fwd():
        state["out"] = ops.lmhead_forward(hidden, w.weight, labels, cfg.temperature, saved_logits=zbuf, saved_row_map=row_map)

    def fwd_and_pick():       # untimed set-up of a backward: refill the kept logits, compact the per-token vectors
        fwd()
        _, ent, _, lse = state["out"]
        state.update(lse=lse[live].contiguous(), ent=ent[live].contiguous())
    fwd_and_pick()
    h_c, lab_c = hidden[live].contiguous(), labels[live].contiguous()
    g_lp = torch.randn(rows, device=dev) / max(w.n_tok, 1.0)
    g_en = g_lp * 1e-3 if cfg.entropy_coef > 0 else None
    dwbuf = torch.zeros(cfg.V, cfg.H, dtype=torch.float32, device=dev)

    def bwd(need_h, need_w):
        ops.lmhead_backward(h_c, w.weight, lab_c, state["lse"], state["ent"] if g_en is not None else None, g_lp, g_en,
                            cfg.temperature, need_dhidden=need_h, need_dweight=need_w, dweight=dwbuf if need_w else None,
                            accumulate_dweight=False, saved_logits=zbuf, weight_t=wt, weight_t_ready=True)
    ops.lmhead_backward(h_c, w.weight, lab_c, state["lse"], None, g_lp, None, cfg.temperature, need_dweight=False,
                        saved_logits=zbuf, weight_t=wt, weight_t_ready=False)          # fills W^T once
    t_fwd = _events(fwd, reps)
    t_both = _events(lambda: bwd(True, True), reps, setup=fwd_and_pick)
    t_dh_only = _events(lambda: bwd(True, False), reps, setup=fwd_and_pick)
    t_dw_only = _events(lambda: bwd(False, True), reps, setup=fwd_and_pick)
    hv = 2.0 * cfg.H * cfg.V
    peak = peak_of(cfg)

    def rec(kernel, r, ms):
        tf = hv * r / (ms * 1e-3) / 1e12
        return {"kernel": kernel, "rows": r, "ms": round(ms, 3), "achieved": round(tf, 1), "peak": peak, "unit": "TFLOP/s",
                "frac": round(tf / peak, 4)}
    return {"chunk_tokens": n,
            "forward": rec("lmhead_fwd_kernel (+ finalize)", n, t_fwd),
            "dhidden": rec("gemm_nt_kernel<16-bit out> (+ split-K reduce)", rows, t_both - t_dw_only),
            "dweight": rec("gemm_nt_kernel<fp32 out>", rows, t_both - t_dh_only),
            "rest_of_backward_ms": round(t_dh_only + t_dw_only - t_both, 3)}


def glue_stages(cfg, samples, device, reps=20):
    """The loss / advantage / index kernels of one micro-batch at this workload's shapes: average
    time per call (events around `reps` back-to-back calls), bytes each call touches by construction,
    and launches per call.  They move a few MB at most, so launch latency is what they cost."""
    from chatlearn_amd.algorithm.grpo_utils.advantage_compute import AdvantageComputer
    p = [s["prompt_token_length"] for s in samples]
    r = [s["response_token_length"] for s in samples]
    B, S = len(samples), max(a + b for a, b in zip(p, r))
    T = sum(p) + sum(r)
    gen = torch.Generator(device=device).manual_seed(7)
    tokens = torch.randint(0, cfg.V, (B, S), generator=gen, device=device)
    plen = torch.tensor(p, dtype=torch.int32, device=device)
    rlen = torch.tensor(r, dtype=torch.int32, device=device)
    cu, mask = synthetic.packed_layout(samples)
    cu, mask = cu.to(device), mask.to(device)
    lp = -torch.rand(T, generator=gen, device=device)
    old = lp + 0.01 * torch.randn(T, generator=gen, device=device)
    ent = torch.rand(T, generator=gen, device=device)
    adv = torch.randn(B, generator=gen, device=device)
    attn, lmask, _ = ops.build_masks(plen, rlen, S)
    idx, *_ = ops.unpad_indices(attn)
    vec = torch.randn(T, 1, generator=gen, device=device)

    class _Buf:
        def __init__(self, b):
            self.buffer = b
    pop = synthetic.sample_population(cfg, synthetic.generator_for(cfg))

    def advantages():
        AdvantageComputer(num_inference_per_prompt=cfg.group)([_Buf([dict(x) for x in pop])])
    stages = {
        # name: (callable, bytes touched, launches)
        "build_masks [B,S]": (lambda: ops.build_masks(plen, rlen, S), B * S * 16 + B * 8, 1),
        "shift_labels [B,S]": (lambda: ops.shift_labels(tokens, lmask, zero_last=True), B * S * 24, 1),
        "thd_pack (align 1)": (lambda: ops.thd_pack(tokens, p, r, align=1, pad_token=0, want_position_ids=True,
                                                    verify_on_device=False), T * 44 + B * 20, 2),
        "pad_input (scatter rows) [T]->[B,S]": (lambda: ops.scatter_rows(vec, idx, B * S), T * 12 + B * S * 4, 2),
        "policy_loss grpo, upstream grads": (
            lambda: ops.policy_loss(lp, old, adv, mode=0, cu_seqlens=cu, ref_logprob=old, entropy=ent, loss_mask=mask,
                                    kl_coef=1e-3, entropy_coef=1e-3, grad_scale=1.0 / T, want_dloss=False,
                                    want_upstream=True), T * 44, _lib.lib().clgrpo_policy_loss_launches(T, 0)),
        "group advantages (whole episode, host grouping + kernel)": (advantages, len(pop) * 24, 1),
    }
    # The statistics kernels for callers that already hold logits (the reference's logprobs_from_logits /
    # entropy_from_logits mirrors): HBM-bound, so their GB/s is against the 8 TB/s peak.  2048 rows of the
    # full vocabulary in the workload's dtype.
    R = 2048
    logits = torch.randn(R, cfg.V, generator=gen, device=device, dtype=torch.float32).to(cfg.dtype)
    lab = torch.randint(0, cfg.V, (R,), generator=gen, device=device)
    es = logits.element_size()
    s_lp, s_ent, s_lse = ops.softmax_stats(logits, lab)
    g1 = torch.randn(R, generator=gen, device=device)
    stages["softmax_stats (logprob + entropy from logits) [2048,V]"] = (
        lambda: ops.softmax_stats(logits, lab), R * cfg.V * es, 1)
    stages["softmax_stats_backward (d logits, statistics from the forward) [2048,V]"] = (
        lambda: ops.softmax_stats_backward(logits, lab, g1, g1, lse=s_lse, entropy=s_ent), 2 * R * cfg.V * es, 1)
    out = {}
    for name, (fn, nbytes, launches) in stages.items():
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) / reps
        out[name] = {"us_per_call_device_span": e0.elapsed_time(e1) * 1e3 / reps, "us_per_call_wall": wall * 1e6,
                     "bytes": nbytes, "launches": launches,
                     "GB_per_s_vs_8000": nbytes / max(e0.elapsed_time(e1) * 1e-3 / reps, 1e-9) / 1e9}
    return {"B": B, "S": S, "T": T, "episode_samples": len(pop), "stages": out}


def loss_stage(w, reps=50):
    """The loss stage alone at the step's shapes: one clgrpo_policy_loss call over the micro-batch's tokens
    (what it reads and writes by construction: logprob, old, ref, entropy, mask in; loss, kl, g_logprob,
    g_entropy out), timed between stream events over back-to-back calls."""
    cfg = w.cfg
    T = w.T
    lp, ent, _, _ = ops.lmhead_forward(w.hidden, w.weight, w.labels, cfg.temperature)
    mode = LOSS_GSPO if cfg.loss == "gspo" else LOSS_GRPO
    call = lambda: ops.policy_loss(lp, w.old, w.adv, mode=mode, cu_seqlens=w.cu, ref_logprob=w.ref, entropy=ent,
                                   loss_mask=w.mask, kl_coef=cfg.kl_coef, entropy_coef=cfg.entropy_coef,
                                   pos_clip_ratio=cfg.pos_clip_ratio, neg_clip_ratio=cfg.neg_clip_ratio,
                                   grad_scale=1.0 / w.n_tok, want_dloss=False, want_upstream=True)
    for _ in range(3):
        call()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        call()
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / reps
    nbytes = T * (4 * 5 + 4 + 4 + 4 + (4 if cfg.entropy_coef > 0 else 0)) + len(w.samples) * 8
    return {"bytes": nbytes, "us_per_call": round(us, 2), "GB_per_s": round(nbytes / (us * 1e-6) / 1e9, 1),
            "frac_of_hbm_peak": round(nbytes / (us * 1e-6) / 1e9 / PEAK_HBM_GBS, 4),
            "launches": int(_lib.lib().clgrpo_policy_loss_launches(T, mode)),
            "note": "a few hundred KB per call: launch latency, not bandwidth, is what it costs"}


def operand_activity(w, reps=6):
    """The same forward launch (all tokens, nothing kept) on the workload's random operands and on all-zero
    operands: identical instruction stream and memory traffic, different switching activity in the
    matrix cores.  The gap between the two is what the power limit costs; the vendor library's plain
    GEMM of the same shape is given the same two inputs for comparison."""
    cfg = w.cfg
    flops = 2.0 * w.T * cfg.H * cfg.V
    zero_h, zero_w = torch.zeros_like(w.hidden), torch.zeros_like(w.weight)

    def rate(fn):
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        ms = _events(fn, reps)
        return {"ms": round(ms, 3), "TFLOP_per_s": round(flops / ms / 1e9, 1), "frac_of_peak": round(flops / ms / 1e9 / peak_of(cfg), 4)}
    fused = lambda h, wt: (lambda: ops.lmhead_forward(h, wt, w.labels, cfg.temperature))
    plain = lambda h, wt: (lambda: torch.nn.functional.linear(h, wt))
    return {"lmhead_fwd_kernel, random operands": rate(fused(w.hidden, w.weight)),
            "lmhead_fwd_kernel, zero operands": rate(fused(zero_h, zero_w)),
            "vendor GEMM hidden @ W^T, random operands": rate(plain(w.hidden, w.weight)),
            "vendor GEMM hidden @ W^T, zero operands": rate(plain(zero_h, zero_w)),
            "lmhead_fwd_kernel, random operands again": rate(fused(w.hidden, w.weight))}


def autograd_seam(w, steps):
    """The drop-in seam through torch autograd at this workload's shapes: forward, a linear stand-in
    for the loss, ``.backward()`` into ``hidden.grad`` and an fp32 main-grad buffer."""
    from chatlearn_amd import fused_linear_logprob_entropy
    cfg, T = w.cfg, w.T
    coef = torch.randn(T, device=w.device) * w.mask
    main_grad = torch.zeros(cfg.V, cfg.H, dtype=torch.float32, device=w.device)

    def step(**kw):
        h = w.hidden.detach().requires_grad_(True)
        wt = w.weight.detach().requires_grad_(True)
        lp, _ = fused_linear_logprob_entropy(h, wt, w.labels, temperature=cfg.temperature, dweight_buffer=main_grad, **kw)
        ((lp * coef).sum() / T).backward()
    out = {}
    plan = (("default_arguments", {}),
            ("default_with_loss_mask", dict(loss_mask=w.mask)),
            ("default_with_host_loss_mask", dict(loss_mask_host=w.mask_host)),
            ("keep_8192_rows_recompute_the_rest_host_loss_mask", dict(keep_logits_rows=8192, loss_mask_host=w.mask_host)),
            ("recompute_everything", dict(keep_logits_rows=None)))
    for name, kw in plan:
        torch.cuda.empty_cache()
        for _ in range(2):
            step(**kw)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step(**kw)
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / steps
        out[name] = {"ms_per_step": round(dt * 1e3, 3), "tokens_per_s": round(T / dt, 1)}
    return out


def sweep(cfg, device, weight, keep):
    """Every micro-batch of the configuration's mini-batch: the sample population regrouped by the library's
    bin packing (split_microbatch with packing, rows 6-8 of the path) into micro-batches of at most cfg.T
    tokens, each run through the head step; dW accumulates across them and W^T is built once."""
    from chatlearn_amd.algorithm.grpo_utils.trainer_utils import split_microbatch
    pop = synthetic.sample_population(cfg, synthetic.generator_for(cfg))
    adv_all = advantages_for(pop, device, group=cfg.group)
    for i, s in enumerate(pop):
        s["sample_index"] = i
    t0 = time.perf_counter()
    groups = split_microbatch(data_list=[dict(s) for s in pop], max_train_token=cfg.T, packing=True)
    packing_ms = (time.perf_counter() - t0) * 1e3
    # the two library calls behind it alone (lengths in, bins out), without the Python that moves the sample dicts
    lens = [s["prompt_token_length"] + s["response_token_length"] for s in pop]
    t0 = time.perf_counter()
    n_bins = len(ops.bin_packing_ids(lens, cfg.T))
    ops.bin_packing_fix_bin_ids(lens, n_bins)
    packing_calls_ms = (time.perf_counter() - t0) * 1e3
    n_tok_total = float(sum(s["response_token_length"] for s in pop))
    works = []
    for mb in groups:
        w = Workload(cfg, device, samples=mb)
        w.weight = weight
        g = torch.Generator(device=device).manual_seed(cfg.seed + 17 * len(works))
        w.hidden = torch.randn(w.T, cfg.H, generator=g, device=device, dtype=torch.float32).to(cfg.dtype)
        w.labels = torch.randint(0, cfg.V, (w.T,), generator=g, device=device)
        w.adv = adv_all[torch.tensor([s["sample_index"] for s in mb], device=device)]
        works.append(w.finish())
    dweight = torch.zeros(cfg.V, cfg.H, dtype=torch.float32, device=device)
    cache, ws_cache = {}, {}
    for w in works[:2]:                                    # warm-up
        head_step(w, keep, dweight, accumulate=True, weight_t_cache=cache, n_tok=n_tok_total, workspace_cache=ws_cache)
    cache.clear()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    rows_bwd = launches = 0
    for i, w in enumerate(works):
        o = head_step(w, keep, dweight, accumulate=i > 0, weight_t_cache=cache, n_tok=n_tok_total, workspace_cache=ws_cache)
        rows_bwd += o["rows_projected_bwd"]
        launches += len(o["token_chunks"])
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    tokens = sum(w.T for w in works)
    hv = float(cfg.H) * cfg.V
    return {"micro_batches": len(works), "tokens": tokens, "T_projected_backward": rows_bwd, "token_chunks_total": launches,
            "step_mfma_frac_executed": 2.0 * hv * (tokens + 2.0 * rows_bwd) / dt / 1e12 / peak_of(cfg),
            "tokens_per_micro_batch_min_max": [min(w.T for w in works), max(w.T for w in works)],
            "ms_total": dt * 1e3, "tokens_per_s": tokens / dt, "host_bin_packing_ms": round(packing_ms, 2),
            "host_bin_packing_library_calls_ms": round(packing_calls_ms, 3),
            "note": "bin-packed micro-batches of the whole mini-batch, dW accumulated, W^T built once"}


def other_config(name, device, steps, warmup):
    cfg = synthetic.CONFIGS[name]
    w = Workload(cfg, device).tensors().finish()
    train = cfg.loss is not None
    keep = default_keep_rows(cfg.V, cfg.dtype) if train else None
    dweight = torch.zeros(cfg.V, cfg.H, dtype=torch.float32, device=device) if train else None
    dt, stages, out = time_step(w, keep, dweight, steps, warmup)
    rec = step_record(w, keep, dt, stages, out)
    rows_fwd = rec["T_projected_forward"]
    fwd_tf = 2.0 * rows_fwd * cfg.H * cfg.V / (stages["forward"] * 1e-3) / 1e12
    rec.update({"workload": f"H={cfg.H} V={cfg.V} T={w.T} {cfg.loss or 'no-grad logprob+entropy'} "
                            f"{'bf16' if cfg.dtype == torch.bfloat16 else 'fp32'}"
                            f"{' temperature ' + str(cfg.temperature) if cfg.temperature != 1.0 else ''}",
                "forward_kernel_frac_of_peak": round(fwd_tf / peak_of(cfg), 4),
                "forward_launches": len(rec["token_chunks"]),
                "forward_traffic_bytes_per_launch": measured_traffic(cfg.name, max(rec["token_chunks"]), keep)})
    rec["tokens_per_s"] = round(rec["tokens_per_s"], 1)
    rec["ms_per_step"] = round(rec["ms_per_step"], 3)
    rec["step_mfma_frac_executed"] = round(rec["step_mfma_frac_executed"], 4)
    if train:
        del out, dweight
        torch.cuda.empty_cache()
        rec["gemm_kernels"] = gemm_kernels(w, keep, reps=2)
    return rec


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="c2", choices=sorted(synthetic.CONFIGS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-unfused", action="store_true")
    ap.add_argument("--no-variants", action="store_true", help="skip the variants / gemm_kernels / loss_stage records")
    ap.add_argument("--no-sweep", action="store_true", help="skip the whole-mini-batch sweep")
    ap.add_argument("--no-other-configs", action="store_true", help="skip the compact records of the other configurations")
    ap.add_argument("--lean", action="store_true", help="only the headline step (for profiling runs)")
    ap.add_argument("--cpu-rows", type=int, default=256)
    ap.add_argument("--gemm-reference", action="store_true",
                    help="also time the vendor library's plain GEMMs (torch.matmul) at this head shape, for context")
    ap.add_argument("--operand-activity", action="store_true",
                    help="also time the forward launch and the vendor GEMM on random and on all-zero operands "
                         "(same instructions and traffic, different switching activity: what the power limit costs)")
    ap.add_argument("--glue", action="store_true",
                    help="also time the loss / advantage / index kernels at this workload's shapes")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three plain 1 GiB device copies (a kernel of known HBM traffic, for scaling "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    ap.add_argument("--skip-masked-forward", action="store_true",
                    help="also leave rows whose loss mask is zero out of the forward (their per-token outputs become zero)")
    ap.add_argument("--no-skip-masked", action="store_true",
                    help="run the backward on every row, also those whose loss mask is zero")
    ap.add_argument("--keep-logits-chunk", type=int, default=-1,
                    help="rows per chunk whose logits the forward keeps for the backward (0: recompute; "
                         "-1: the library's default, a bound in bytes)")
    args = ap.parse_args()
    if args.lean:
        args.no_cpu_baseline = args.no_unfused = args.no_variants = args.no_sweep = args.no_other_configs = True
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives are built); use --gpus 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    cfg = synthetic.CONFIGS[args.config]
    w = Workload(cfg, dev).tensors().finish()
    T = w.T
    train = cfg.loss is not None
    dweight = torch.zeros(cfg.V, cfg.H, dtype=torch.float32, device=dev) if train else None
    if args.keep_logits_chunk < 0:
        args.keep_logits_chunk = default_keep_rows(cfg.V, cfg.dtype)
    keep = args.keep_logits_chunk if (train and args.keep_logits_chunk > 0) else None

    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    dt, stages, out_last = time_step(w, keep, dweight, args.steps, args.warmup, skip_masked=not args.no_skip_masked,
                                     skip_masked_forward=args.skip_masked_forward)
    head = step_record(w, keep, dt, stages, out_last)
    fwd_ms = stages["forward"]
    n_fwd_launch = len(head["token_chunks"])
    rows_fwd = head["T_projected_forward"]
    peak = peak_of(cfg)
    # the kernel's rate counts the rows its launches projected (all T unless --skip-masked-forward)
    fwd_flops = 2.0 * float(rows_fwd) * cfg.H * cfg.V
    fwd_tflops = fwd_flops / (fwd_ms * 1e-3) / 1e12          # all forward launches of a step together
    out = {
        "metric": "packed tokens/sec, fused logprob+GRPO loss fwd+bwd (Qwen3-8B head); % MFMA peak",
        "value": T / dt,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": dt * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if cfg.dtype == torch.bfloat16 else "f32",
        "data": "synthetic",
        "config": {"workload": f"{cfg.name}: H={cfg.H} V={cfg.V} T={T} packed tokens in {len(w.samples)} sequences, "
                               f"{cfg.loss or 'no-grad logprob+entropy'}"
                               f"{' fwd+bwd (dhidden ' + str(cfg.dtype).split('.')[-1] + ', dW fp32)' if train else ''}",
                   "temperature": cfg.temperature, "kl_coef": cfg.kl_coef, "entropy_coef": cfg.entropy_coef,
                   "token_chunks": head["token_chunks"], "logits_kept_per_chunk": bool(keep),
                   "T_projected_forward": rows_fwd, "T_projected_backward": head["T_projected_backward"],
                   "scratch_bytes": head.get("scratch_bytes")},
        "roofline": {"bound": "mfma", "kernel": "lmhead_fwd_kernel", "achieved": fwd_tflops, "peak": peak,
                     "unit": "TFLOP/s", "frac": fwd_tflops / peak,
                     "traffic": measured_traffic(cfg.name, max(head["token_chunks"]), keep),
                     "algorithmic_flops_per_launch": fwd_flops / n_fwd_launch,
                     "avg_launch_ms": fwd_ms / n_fwd_launch, "launches_per_step": n_fwd_launch},
        # flops the step executed on the matrix cores for its results: forward on T_projected_forward rows,
        # the two backward contractions on T_projected_backward rows (rows outside the loss mask have an exactly
        # zero gradient and are skipped); and the same step priced at the 6*T*H*V convention of the metric
        "step_mfma_frac_executed": head["step_mfma_frac_executed"],
        "step_mfma_frac_6THV_convention": 6.0 * T * cfg.H * cfg.V / dt / 1e12 / peak if train else None,
        "stage_ms": stages,
    }
    if train and not args.no_variants:
        out["gemm_kernels"] = gemm_kernels(w, keep)
        out["loss_stage"] = loss_stage(w)
        torch.cuda.empty_cache()
        variants = {}
        plan = [("no_flag_readback", dict(keep=keep, check_flags=False)),
                ("chunk_8192_rows", dict(keep=8192)), ("chunk_4096_rows", dict(keep=4096)),
                ("recompute_no_logits_kept", dict(keep=None)),
                ("no_row_skipping", dict(keep=keep, skip_masked=False)),
                ("skip_masked_rows_in_forward_too", dict(keep=keep, skip_masked_forward=True))]
        for name, kw in plan:
            k = kw.pop("keep")
            torch.cuda.empty_cache()     # each variant sizes its scratch differently: start from an unfragmented pool
            v_dt, v_st, v_out = time_step(w, k, dweight, max(3, args.steps // 2), 3, **kw)
            variants[name] = step_record(w, k, v_dt, v_st, v_out)
        variants["autograd_seam"] = autograd_seam(w, max(3, args.steps // 2))
        variants["note"] = ("same micro-batch; the headline reads the loss flags back once per step as the reference's assertions do, "
                            "no_flag_readback leaves that out; chunk_8192_rows / chunk_4096_rows: smaller bounds on the kept logits; "
                            "recompute: nothing kept, logit tiles recomputed in the backward; no_row_skipping: backward on all T rows; "
                            "skip_masked_rows_in_forward_too: per-token outputs of masked rows become zero (not the headline); "
                            "autograd_seam: fused_linear_logprob_entropy through torch autograd (forward, a linear stand-in for the "
                            "loss, backward into hidden.grad and an fp32 main-grad buffer)")
        out["variants"] = variants
    if not args.no_unfused and train:
        try:
            u_dt = unfused_gpu(w, max(2, args.steps // 3))
            out["unfused_torch_gpu"] = {"tokens_per_s": T / u_dt, "ms_per_step": u_dt * 1e3,
                                        "speedup_fused": u_dt / dt}
        except Exception as e:  # the unfused path can run out of memory on large configs
            out["unfused_torch_gpu"] = {"error": str(e)[:200]}
    if args.gemm_reference:
        out["library_gemm_reference"] = library_gemms(w.hidden, w.weight)
    if args.operand_activity:
        out["operand_activity"] = operand_activity(w)
    if args.glue:
        out["glue_stages"] = glue_stages(cfg, w.samples, dev)
    if train and not args.no_sweep:
        torch.cuda.empty_cache()
        out["sweep"] = sweep(cfg, dev, w.weight, keep)
    if not args.no_other_configs:
        del w, dweight, out_last
        torch.cuda.empty_cache()
        others = {}
        for name in sorted(synthetic.CONFIGS):
            if name == cfg.name:
                continue
            try:
                others[name] = other_config(name, dev, 3, 2)
            except Exception as e:
                others[name] = {"error": str(e)[:200]}
            torch.cuda.empty_cache()
        out["other_configs"] = others
    if not args.no_cpu_baseline:
        threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or min(16, os.cpu_count() or 1)
        tps, reps = cpu_baseline(cfg, args.cpu_rows, threads)
        out["cpu_baseline"] = {"value": tps, "unit": "tokens/s", "cores": threads, "cpu_model": cpu_model(), "kind": "port",
                               "sample": f"{args.cpu_rows} packed rows at full H and V, fp32, fwd"
                                         f"{'+bwd' if train else ''}, {reps} timed repetitions"}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
