#!/usr/bin/env python3
"""Benchmark of the fused logprob + GRPO loss head path (forward + backward).

One step = one packed micro-batch through: fused lm_head forward (logprob,
entropy, lse), the policy-loss kernel (loss sums + per-token upstream grads) and
the fused backward (dhidden bf16, dW fp32).  Default workload: the Qwen3-8B head
(H=4096, V=151936, bf16) on a 16384-token micro-batch, inputs resident in HBM.

Prints ONE JSON line:  metric/value/unit per the driver contract, plus
  roofline     - the forward kernel against the bf16 MFMA peak (HIP-event timed, live)
  cpu_baseline - the torch oracle (reference op order) timed on the host cores on a row sample
and some extra, clearly named fields (per-stage times, the unfused torch-on-GPU path).
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from chatlearn_amd import ops, synthetic  # noqa: E402
from chatlearn_amd._lib import LOSS_GRPO, LOSS_GSPO  # noqa: E402

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_F32_TFLOPS = 157.3

# HBM-side bytes (L2 <-> fabric, read + written) of ONE forward launch, from two rocprofv3 --pmc runs
# (FETCH_SIZE scaled by 2.00, WRITE_SIZE by 1.00 after a plain 1 GiB copy calibration; the summary is
# kept with the other profiles).  Key: (config, tokens per launch, chunk logits kept).  Other
# workloads have not been measured and report null.
MEASURED_FWD_TRAFFIC_BYTES = {("c2", 16384, True): 43.10e9}


def build_workload(cfg, device):
    gen = synthetic.generator_for(cfg)
    samples = synthetic.fill_microbatch(cfg, synthetic.sample_population(cfg, gen))
    cu, mask = synthetic.packed_layout(samples)
    T = int(cu[-1])
    hidden, weight, labels = synthetic.make_head_tensors(cfg, T, gen, device=device, device_generate=True)
    return samples, cu.to(device), mask.to(device), T, hidden, weight, labels, mask


def advantages_for(samples, device):
    """Group mean/std advantages through the library's AdvantageComputer mirror."""
    from chatlearn_amd.algorithm.grpo_utils.advantage_compute import AdvantageComputer

    class _Buf:
        def __init__(self, b):
            self.buffer = b
    pop = [dict(s) for s in samples]
    AdvantageComputer(num_inference_per_prompt=1 << 30)([_Buf(pop)])
    return torch.tensor([float(s["advantages"]) for s in pop], dtype=torch.float32, device=device)


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


def unfused_gpu(cfg, hidden, weight, labels, old, ref, adv, cu, mask, n_tok, steps):
    """What the reference's FSDP trainer does today, on the same GPU in bf16: materialised logits,
    log_softmax + gather, chunked entropy, re-padding to [B,S], torch loss ops, autograd backward
    (policy_trainer.py:216-286)."""
    from oracle import indexing as oi
    from oracle import losses as ol
    from oracle import softmax_stats as osm
    h = hidden.detach().clone().requires_grad_(True)
    w = weight.detach().clone().requires_grad_(True)
    lab = labels.view(1, -1)
    lens = (cu[1:] - cu[:-1]).long()
    B, S = lens.numel(), int(lens.max())
    ar = torch.arange(S, device=hidden.device)
    attn = (ar.unsqueeze(0) < lens.unsqueeze(1))
    indices = torch.nonzero(attn.flatten(), as_tuple=False).flatten()
    pad = lambda x: oi.pad_input(x.unsqueeze(-1), indices, B, S).squeeze(-1)
    old_p, ref_p, mask_p = pad(old), pad(ref), pad(mask)
    adv_list = adv.tolist()

    def step():
        logits = torch.nn.functional.linear(h, w).unsqueeze(0)
        if cfg.temperature != 1.0:
            logits = logits / cfg.temperature
        lp = osm.logprobs_from_logits(logits, lab)
        with (torch.enable_grad() if cfg.entropy_coef > 0 else torch.no_grad()):
            ent = osm.entropy_from_logits_with_chunking(logits)
        total, _ = ol.fsdp_policy_loss(pad(lp[0].float()), pad(ent[0]), old_p, ref_p, adv_list, mask_p, n_tok,
                                       entropy_coef=cfg.entropy_coef, kl_coef=cfg.kl_coef,
                                       pos_clip_ratio=cfg.pos_clip_ratio, neg_clip_ratio=cfg.neg_clip_ratio,
                                       diff_clip_ratio=cfg.diff_clip_ratio, final_clip_ratio=cfg.final_clip_ratio,
                                       use_group_sequence_policy=(cfg.loss == "gspo"))
        total.backward()
        h.grad = None
        w.grad = None

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


def glue_stages(cfg, samples, device, reps=20):
    """The loss / advantage / index kernels of one micro-batch at this workload's shapes: average
    time per call (events around `reps` back-to-back calls), bytes each call touches by construction,
    and launches per call.  They move a few MB at most, so launch latency is what they cost."""
    from chatlearn_amd.algorithm.grpo_utils.advantage_compute import AdvantageComputer
    from chatlearn_amd.algorithm.grpo_utils.megatron_utils.train_helper import get_batch_packed
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
                                    want_upstream=True), T * 44, 3),
        "group advantages (whole episode, host grouping + kernel)": (advantages, len(pop) * 24, 1),
    }
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


def autograd_seam(cfg, hidden, weight, labels, mask, steps):
    """The drop-in seam through torch autograd at this workload's shapes: forward, a linear stand-in
    for the loss, ``.backward()`` into ``hidden.grad`` and an fp32 main-grad buffer; with the logits
    recomputed in the backward, kept, and kept with the loss mask as a hint."""
    from chatlearn_amd import fused_linear_logprob_entropy
    T = hidden.shape[0]
    coef = torch.randn(T, device=hidden.device) * mask
    main_grad = torch.zeros(cfg.V, cfg.H, dtype=torch.float32, device=hidden.device)

    def step(**kw):
        h = hidden.detach().requires_grad_(True)
        w = weight.detach().requires_grad_(True)
        lp, _ = fused_linear_logprob_entropy(h, w, labels, temperature=cfg.temperature, dweight_buffer=main_grad, **kw)
        ((lp * coef).sum() / T).backward()
    out = {}
    for name, kw in (("recompute", dict(keep_logits_rows=None)), ("kept_logits", {}),
                     ("kept_logits_mask_hint", dict(loss_mask=mask))):
        for _ in range(2):
            step(**kw)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step(**kw)
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / steps
        out[name] = {"ms_per_step": dt * 1e3, "tokens_per_s": T / dt}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="c2", choices=sorted(synthetic.CONFIGS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-unfused", action="store_true")
    ap.add_argument("--cpu-rows", type=int, default=256)
    ap.add_argument("--gemm-reference", action="store_true",
                    help="also time the vendor library's plain GEMMs (torch.matmul) at this head shape, for context")
    ap.add_argument("--autograd-seam", action="store_true",
                    help="also time fused_linear_logprob_entropy through torch autograd (<= 16384 tokens)")
    ap.add_argument("--glue", action="store_true",
                    help="also time the loss / advantage / index kernels at this workload's shapes")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three plain 1 GiB device copies (a kernel of known HBM traffic, for scaling "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    ap.add_argument("--skip-masked-forward", action="store_true",
                    help="also leave rows whose loss mask is zero out of the forward (their per-token outputs become zero)")
    ap.add_argument("--no-skip-masked", action="store_true",
                    help="run the backward on every row, also those whose loss mask is zero")
    ap.add_argument("--keep-logits-chunk", type=int, default=16384,
                    help="tokens per chunk whose logits the forward keeps for the backward (0: recompute)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives are built); use --gpus 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    cfg = synthetic.CONFIGS[args.config]
    samples, cu, mask, T, hidden, weight, labels, mask_host = build_workload(cfg, dev)
    train = cfg.loss is not None
    n_tok = float(mask.sum().item())
    adv = advantages_for(samples, dev)

    # old / ref logprobs around the model's own logprob, as the recipe says
    lp0, *_ = ops.lmhead_forward(hidden, weight, labels, cfg.temperature, need_entropy=False)
    old, ref = synthetic.noisy_logprobs(lp0, synthetic.generator_for(cfg))
    dweight = torch.zeros(cfg.V, cfg.H, dtype=torch.float32, device=dev) if train else None

    from chatlearn_amd.fused import grpo_head_step, _token_chunks
    keep = args.keep_logits_chunk if (train and args.keep_logits_chunk > 0) else None
    cu_host = cu.tolist()
    chunks = _token_chunks(T, keep, cu_host if (keep and cfg.loss == "gspo") else None)
    marks = []

    def step(record=False):
        """One pass of the head over the micro-batch.  Training configurations: per token chunk,
        fused forward (keeping the chunk's logits), loss + upstream gradients, fused backward
        (dhidden, dW accumulated).  The no-grad configuration: fused forward only."""
        if not train:
            if record:
                e = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
                e[0].record()
            ops.lmhead_forward(hidden, weight, labels, cfg.temperature, need_entropy=True)
            if record:
                e[1].record()
                marks.append([("forward", e[0]), ("end", e[1])])
            return None
        cur = []

        def hook(name):
            ev = torch.cuda.Event(enable_timing=True)
            ev.record()
            cur.append((name, ev))
        out = grpo_head_step(hidden, weight, labels, old, ref, adv, cu, mask, n_tokens_total=n_tok,
                             use_group_sequence_policy=(cfg.loss == "gspo"), pos_clip_ratio=cfg.pos_clip_ratio,
                             neg_clip_ratio=cfg.neg_clip_ratio, diff_clip_ratio=cfg.diff_clip_ratio,
                             final_clip_ratio=cfg.final_clip_ratio, kl_coef=cfg.kl_coef,
                             entropy_coef=cfg.entropy_coef, temperature=cfg.temperature, dweight=dweight,
                             accumulate_dweight=False, keep_logits_chunk=keep, cu_seqlens_host=cu_host,
                             skip_masked_rows=not args.no_skip_masked, skip_masked_forward=args.skip_masked_forward,
                             stage_hook=hook if record else None, loss_mask_host=mask_host,
                             check_flags=False)
        if record:
            marks.append(cur)
        return out

    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    out_last = None
    for _ in range(args.warmup):
        out_last = step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out_last = step(record=True)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps

    def stage_ms(name):
        tot = 0.0
        for cur in marks:
            for (a, ea), (_, eb) in zip(cur[:-1], cur[1:]):
                if a == name:
                    tot += ea.elapsed_time(eb)
        return tot / len(marks)
    fwd_ms, loss_ms, bwd_ms = stage_ms("forward"), stage_ms("loss"), stage_ms("backward")
    n_fwd_launch = len(chunks) if train else 1
    rows_bwd = out_last["rows_projected_bwd"] if train else 0
    rows_fwd = out_last["rows_projected_fwd"] if train else T

    thv = float(T) * cfg.H * cfg.V
    peak = PEAK_BF16_TFLOPS if cfg.dtype == torch.bfloat16 else PEAK_F32_TFLOPS
    # the kernel's rate counts the rows its launches projected (all T unless --skip-masked-forward)
    fwd_flops = 2.0 * float(rows_fwd) * cfg.H * cfg.V
    fwd_tflops = fwd_flops / (fwd_ms * 1e-3) / 1e12          # all forward launches of a step together
    step_flops = (6.0 if train else 2.0) * thv
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
        "config": {"workload": f"{cfg.name}: H={cfg.H} V={cfg.V} T={T} packed tokens in {len(samples)} sequences, "
                               f"{cfg.loss or 'no-grad logprob+entropy'}"
                               f"{' fwd+bwd (dhidden ' + str(cfg.dtype).split('.')[-1] + ', dW fp32)' if train else ''}",
                   "temperature": cfg.temperature, "kl_coef": cfg.kl_coef, "entropy_coef": cfg.entropy_coef,
                   "token_chunks": [hi - lo for lo, hi in chunks], "logits_kept_per_chunk": bool(keep),
                   "T_projected_forward": rows_fwd, "T_projected_backward": rows_bwd},
        "roofline": {"bound": "mfma", "kernel": "lmhead_fwd_kernel", "achieved": fwd_tflops, "peak": peak,
                     "unit": "TFLOP/s", "frac": fwd_tflops / peak,
                     "traffic": MEASURED_FWD_TRAFFIC_BYTES.get((cfg.name, max(hi - lo for lo, hi in chunks), bool(keep))),
                     "algorithmic_flops_per_launch": fwd_flops / n_fwd_launch,
                     "avg_launch_ms": fwd_ms / n_fwd_launch, "launches_per_step": n_fwd_launch},
        "step_mfma_frac": step_flops / dt / 1e12 / peak,
        "stage_ms": {"forward": fwd_ms, "loss": loss_ms, "backward": bwd_ms},
    }
    if train and mask is not None and not args.skip_masked_forward and not args.no_skip_masked:
        # Reported beside the headline, never as `value`: the same step with the rows outside the loss
        # mask also left out of the forward (their per-token outputs become zero, loss and gradients
        # are unchanged).
        args.skip_masked_forward = True
        for _ in range(max(1, args.warmup // 2)):
            lean = step()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for _ in range(args.steps):
            lean = step()
        torch.cuda.synchronize()
        l_dt = (time.perf_counter() - t1) / args.steps
        args.skip_masked_forward = False
        out["variant_skip_masked_forward"] = {"tokens_per_s": T / l_dt, "ms_per_step": l_dt * 1e3,
                                              "T_projected_forward": lean["rows_projected_fwd"],
                                              "T_projected_backward": lean["rows_projected_bwd"]}
    if not args.no_unfused and train:
        try:
            u_dt = unfused_gpu(cfg, hidden, weight, labels, old, ref, adv, cu, mask, n_tok, max(2, args.steps // 3))
            out["unfused_torch_gpu"] = {"tokens_per_s": T / u_dt, "ms_per_step": u_dt * 1e3,
                                        "speedup_fused": u_dt / dt}
        except Exception as e:  # the unfused path can run out of memory on large configs
            out["unfused_torch_gpu"] = {"error": str(e)[:200]}
    if args.gemm_reference:
        out["library_gemm_reference"] = library_gemms(hidden, weight)
    if args.glue:
        out["glue_stages"] = glue_stages(cfg, samples, dev)
    if args.autograd_seam and train:
        out["autograd_seam"] = autograd_seam(cfg, hidden, weight, labels, mask, max(2, args.steps // 2))
    if not args.no_cpu_baseline:
        threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or min(16, os.cpu_count() or 1)
        tps, reps = cpu_baseline(cfg, args.cpu_rows, threads)
        out["cpu_baseline"] = {"value": tps, "unit": "tokens/s", "cores": threads, "kind": "port",
                               "sample": f"{args.cpu_rows} packed rows at full H and V, fp32, fwd"
                                         f"{'+bwd' if train else ''}, {reps} timed repetitions"}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
