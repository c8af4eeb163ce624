"""Seeded synthetic inputs for the five benchmark configurations of the head path.

Only shapes and distributions matter (no checkpoints or datasets are involved):
hidden ~ N(0,1) standing for the output of the final RMSNorm, lm_head weight
~ N(0, w_std), uniform labels, response / prompt lengths uniform in a range,
rewards Bernoulli or uniform per response.  Tensors are drawn with a CPU
``torch.Generator`` (then moved) unless ``device_generate`` is set, so the CPU
checker and the GPU kernels can be handed identical bits.

Nothing here computes on the hot path; it only builds inputs.
"""
from dataclasses import dataclass, replace
from typing import Dict, List, Optional, Tuple

import torch

BASE_SEED = 1234  # the reference's default seed (configs/base/base_model_config.py:64)


@dataclass(frozen=True)
class HeadConfig:
    name: str
    dtype: torch.dtype
    H: int
    V: int
    T: int                      # token cap of one packed micro-batch
    n_prompts: int
    group: int                  # responses per prompt
    prompt_range: Tuple[int, int]
    response_range: Tuple[int, int]
    w_std: float
    reward: str                 # "bernoulli:<p>" or "uniform"
    loss: Optional[str]         # "grpo", "gspo" or None (no-grad logprob recompute)
    pos_clip_ratio: float = 0.2
    neg_clip_ratio: float = 0.2
    diff_clip_ratio: float = 10
    final_clip_ratio: float = 3
    kl_coef: float = 0.0
    entropy_coef: float = 0.0
    temperature: float = 1.0
    seed: int = BASE_SEED


CONFIGS: Dict[str, HeadConfig] = {
    # plumbing run, fp32, Qwen3-0.6B head
    "c1": HeadConfig("c1", torch.float32, 1024, 151936, 2048, 4, 8, (0, 0), (32, 64), 0.02,
                     "bernoulli:0.5", "grpo", kl_coef=1e-3, seed=BASE_SEED + 1),
    # headline: Qwen3-8B head, GRPO fwd+bwd
    "c2": HeadConfig("c2", torch.bfloat16, 4096, 151936, 16384, 64, 8, (128, 512), (256, 2048), 0.02,
                     "bernoulli:0.3", "grpo", seed=BASE_SEED + 2),
    # GSPO, Qwen3-30B-A3B head
    "c3": HeadConfig("c3", torch.bfloat16, 2048, 151936, 32768, 32, 16, (0, 0), (512, 8192), 0.02,
                     "uniform", "gspo", pos_clip_ratio=4e-4, neg_clip_ratio=3e-4, seed=BASE_SEED + 3),
    # no-grad logprob + entropy recompute, Qwen3-235B-A22B head
    "c4": HeadConfig("c4", torch.bfloat16, 4096, 151936, 65536, 128, 16, (0, 0), (256, 4096), 0.02,
                     "bernoulli:0.5", None, seed=BASE_SEED + 4),
    # long-context MLA head (DeepSeek-V3 / Moonlight shape), temperature 0.7
    "c5": HeadConfig("c5", torch.bfloat16, 7168, 129280, 32768, 1, 8, (0, 0), (2048, 8192), 0.006,
                     "bernoulli:0.5", "grpo", kl_coef=1e-3, entropy_coef=1e-3, temperature=0.7,
                     seed=BASE_SEED + 5),
}


def scaled(cfg: HeadConfig, **kw) -> HeadConfig:
    """Same recipe at other sizes (for parity cases the CPU checker finishes in seconds)."""
    return replace(cfg, **kw)


def _randint(gen, lo, hi, n):
    if hi <= lo:
        return [lo] * n
    return torch.randint(lo, hi + 1, (n,), generator=gen).tolist()


def sample_population(cfg: HeadConfig, gen: torch.Generator) -> List[dict]:
    """The whole mini-batch of samples (n_prompts * group), in rollout order, as the
    per-sample dicts the trainers exchange (only the fields the head path reads)."""
    n = cfg.n_prompts * cfg.group
    p = _randint(gen, cfg.prompt_range[0], cfg.prompt_range[1], n)
    r = _randint(gen, cfg.response_range[0], cfg.response_range[1], n)
    if cfg.reward.startswith("bernoulli"):
        prob = float(cfg.reward.split(":")[1])
        rew = (torch.rand(n, generator=gen) < prob).to(torch.float64).tolist()
    else:
        rew = torch.rand(n, generator=gen, dtype=torch.float64).tolist()
    return [{"prompt_uid": f"0_{i // cfg.group}", "prompt_token_length": p[i], "response_token_length": r[i],
             "rule_reward": rew[i]} for i in range(n)]


def fill_microbatch(cfg: HeadConfig, samples: List[dict], T: Optional[int] = None) -> List[dict]:
    """Samples taken in order until the token cap is reached; the last one is cut (response
    first) so the packed row has exactly T tokens when enough samples exist."""
    T = T or cfg.T
    out, used = [], 0
    for s in samples:
        need = s["prompt_token_length"] + s["response_token_length"]
        if used + need <= T:
            out.append(dict(s))
            used += need
        else:
            room = T - used
            if room >= 2:
                c = dict(s)
                c["prompt_token_length"] = min(c["prompt_token_length"], room // 2)
                c["response_token_length"] = room - c["prompt_token_length"]
                out.append(c)
                used = T
            break
    return out


def make_head_tensors(cfg: HeadConfig, T: int, gen: torch.Generator, device="cpu", device_generate=False):
    """hidden [T,H], weight [V,H] in cfg.dtype and labels int64 [T]."""
    if device_generate:
        dgen = torch.Generator(device=device)
        dgen.manual_seed(cfg.seed)
        hidden = torch.randn(T, cfg.H, generator=dgen, device=device, dtype=torch.float32).to(cfg.dtype)
        weight = (torch.randn(cfg.V, cfg.H, generator=dgen, device=device, dtype=torch.float32) * cfg.w_std).to(cfg.dtype)
        labels = torch.randint(0, cfg.V, (T,), generator=dgen, device=device, dtype=torch.int64)
        return hidden, weight, labels
    hidden = torch.randn(T, cfg.H, generator=gen, dtype=torch.float32).to(cfg.dtype).to(device)
    weight = (torch.randn(cfg.V, cfg.H, generator=gen, dtype=torch.float32) * cfg.w_std).to(cfg.dtype).to(device)
    labels = torch.randint(0, cfg.V, (T,), generator=gen, dtype=torch.int64).to(device)
    return hidden, weight, labels


def packed_layout(samples: List[dict]):
    """cu_seqlens int32 [B+1] and the training loss mask int32 [T] of a packed row: response
    positions, shifted left by one so position t scores token t+1, last position of the row
    zeroed (policy_trainer.py:160-162)."""
    lens = [s["prompt_token_length"] + s["response_token_length"] for s in samples]
    cu = torch.zeros(len(lens) + 1, dtype=torch.int32)
    cu[1:] = torch.cumsum(torch.tensor(lens, dtype=torch.int64), 0).to(torch.int32)
    T = int(cu[-1])
    mask = torch.zeros(T, dtype=torch.int32)
    for b, s in enumerate(samples):
        lo = int(cu[b]) + s["prompt_token_length"]
        mask[lo:lo + s["response_token_length"]] = 1
    mask = torch.roll(mask, -1)
    mask[-1] = 0
    return cu, mask


def noisy_logprobs(lp_center: torch.Tensor, gen: torch.Generator, old_std=0.05, ref_std=0.1):
    """old = center + N(0, old_std), ref = center + N(0, ref_std), fp32, drawn on the CPU."""
    c = lp_center.detach().float().cpu()
    old = c + torch.randn(c.shape, generator=gen) * old_std
    ref = c + torch.randn(c.shape, generator=gen) * ref_std
    return old.to(lp_center.device), ref.to(lp_center.device)


def generator_for(cfg: HeadConfig) -> torch.Generator:
    g = torch.Generator()
    g.manual_seed(cfg.seed)
    return g
