"""PolicyStep (the reference trainer's micro-batch loops on the fused head) against the
oracle's restatement of those loops with materialised logits."""
import copy

import numpy as np
import pytest
import torch

from oracle import policy_loop as opl
from tests.util import assert_close_rel

pytestmark = pytest.mark.gpu

VOCAB, H, MAXLEN = 3000, 128, 96


def _samples(n, seed, with_train_fields):
    g = torch.Generator().manual_seed(seed)
    out = []
    for i in range(n):
        p = int(torch.randint(4, 20, (1,), generator=g))
        r = int(torch.randint(8, 60, (1,), generator=g))
        s = {"all_tokens": torch.randint(0, VOCAB, (p + r,), generator=g), "prompt_token_length": p,
             "response_token_length": r, "prompt_uid": f"0_{i // 4}"}
        if with_train_fields:
            s["old_logprobs"] = -8.0 + torch.randn(p + r, generator=g) * 0.05
            s["ref_logprobs"] = -8.0 + torch.randn(p + r, generator=g) * 0.1
            s["advantages"] = np.float64(torch.randn(1, generator=g).item())
        out.append(s)
    return out


class _Backbone(torch.nn.Module):
    def __init__(self, dtype, seed=0):
        super().__init__()
        g = torch.Generator().manual_seed(seed)
        self.tok = torch.nn.Parameter(torch.randn(VOCAB, H, generator=g).to(dtype))
        self.pos = torch.nn.Parameter((torch.randn(MAXLEN * 8, H, generator=g) * 0.1).to(dtype))

    def forward(self, input_ids, position_ids):
        return self.tok[input_ids] + self.pos[position_ids]


def _oracle_model(bb, weight):
    tok = bb.tok.detach().double().cpu().requires_grad_(True)
    pos = bb.pos.detach().double().cpu().requires_grad_(True)
    w = weight.detach().double().cpu().requires_grad_(True)
    model = lambda ids, p: torch.nn.functional.linear(tok[ids] + pos[p], w)
    return model, tok, pos, w


@pytest.mark.parametrize("packing", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_train_step_matches_reference_loop(dev, packing, dtype):
    from chatlearn_amd.algorithm.grpo_utils.policy_step import PolicyStep
    data = _samples(13, 3, True)
    # make the old / ref logprobs meaningful: centre them on the model's own logprobs
    bb = _Backbone(dtype).to(dev)
    g = torch.Generator().manual_seed(9)
    weight = (torch.randn(VOCAB, H, generator=g) * 0.05).to(dtype).to(dev).requires_grad_(True)
    model, tok, pos, w = _oracle_model(bb, weight)
    args = {"entropy_coef": 0.01, "kl_coef": 0.05, "pos_clip_ratio": 0.2, "neg_clip_ratio": 0.2}
    kw = dict(max_token_in_seq=200, train_micro_batch_size=4)
    centred = opl.forward_step(model, copy.deepcopy(data), packing=packing, trainable=True, **kw)
    for s, c in zip(data, centred):
        s["old_logprobs"] = (c["old_logprobs"] + (s["old_logprobs"] + 8.0)).float()
        s["ref_logprobs"] = (c["old_logprobs"] + (s["ref_logprobs"] + 8.0)).float()
    want_stats, _ = opl.train_step(model, copy.deepcopy(data), packing=packing, module_args=args, **kw)

    step = PolicyStep(bb, weight, module_args=args, packing=packing, keep_logits_chunk=64, **kw)
    got_stats = step.train_step(copy.deepcopy(data))
    rt = 1e-5 if dtype == torch.float32 else 1e-2
    for k in ("pg_loss", "kl_loss", "entropy_loss"):
        assert got_stats[k] == pytest.approx(want_stats[k], rel=rt, abs=rt * 1e-2), k
    assert_close_rel(bb.tok.grad, tok.grad, rt, "token-embedding grad")
    assert_close_rel(bb.pos.grad, pos.grad, rt, "position-embedding grad")
    assert_close_rel(weight.grad, w.grad, rt, "lm_head grad")
    name, metrics = step.get_and_clear_metrics()
    assert name == "policy_trainer" and metrics == [got_stats]


@pytest.mark.parametrize("packing", [False, True])
def test_forward_step_records_match(dev, packing):
    from chatlearn_amd.algorithm.grpo_utils.policy_step import PolicyStep
    data = _samples(9, 5, False)
    bb = _Backbone(torch.float32).to(dev)
    weight = (torch.randn(VOCAB, H, generator=torch.Generator().manual_seed(1)) * 0.05).to(dev)
    model, *_ = _oracle_model(bb, weight)
    kw = dict(max_token_in_seq=150, generate_micro_batch_size=4)
    want = opl.forward_step(model, copy.deepcopy(data), packing=packing, trainable=False, **kw)
    got = PolicyStep(bb, weight, packing=packing, trainable=False, **kw).forward_step(copy.deepcopy(data))
    for a, b, s in zip(got, want, data):
        n = s["prompt_token_length"] + s["response_token_length"]
        assert a["ref_logprobs"].shape == (n,) and "old_logprobs" not in a
        assert a["id_in_list"] == b["id_in_list"]
        # the last position of a sample predicts the next sample's first token (packing) or wraps:
        # the reference keeps that value too, so it is compared as well
        assert_close_rel(a["ref_logprobs"], b["ref_logprobs"], 1e-5, "per-sample logprobs")
