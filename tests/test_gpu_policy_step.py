"""PolicyStep (the reference trainer's micro-batch loops on the fused head) against the
oracle's restatement of those loops with materialised logits."""
import copy
import math

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


@pytest.mark.parametrize("packing", [False, True])
def test_train_step_sequence_level_policy_matches_reference_loop(dev, packing):
    """GSPO through PolicyStep.train_step against the oracle loop (fp32, so that both sides see the same
    sequence ratios; the case checks in float64 that no ratio sits near a clip bound)."""
    from chatlearn_amd.algorithm.grpo_utils.policy_step import PolicyStep
    data = _samples(11, 17, True)
    bb = _Backbone(torch.float32).to(dev)
    weight = (torch.randn(VOCAB, H, generator=torch.Generator().manual_seed(4)) * 0.05).to(dev).requires_grad_(True)
    model, tok, pos, w = _oracle_model(bb, weight)
    args = {"entropy_coef": 0.0, "kl_coef": 0.02, "pos_clip_ratio": 4e-3, "neg_clip_ratio": 3e-3,
            "use_group_sequence_policy": True}
    kw = dict(max_token_in_seq=200, train_micro_batch_size=4)
    centred = opl.forward_step(model, copy.deepcopy(data), packing=packing, trainable=True, **kw)
    g = torch.Generator().manual_seed(2)
    clipped = 0
    for s, c in zip(data, centred):
        n = s["prompt_token_length"] + s["response_token_length"]
        shift = float(torch.randn(1, generator=g)) * 0.01                  # the sequence's mean log-ratio, about +-1 %
        s["old_logprobs"] = (c["old_logprobs"] - shift + torch.randn(n, generator=g) * 1e-4).float()
        s["ref_logprobs"] = (c["old_logprobs"] + torch.randn(n, generator=g) * 0.1).float()
        # the ratio the loss will form: mean over the shifted response mask (positions p-1 .. p+r-2)
        p, r = s["prompt_token_length"], s["response_token_length"]
        delta = (c["old_logprobs"].double() - s["old_logprobs"].double())[p - 1:p + r - 1]
        ratio = math.exp(float(delta.mean()))
        assert min(abs(ratio - 1.004), abs(ratio - 0.997)) > 1e-5
        clipped += (ratio > 1.004) or (ratio < 0.997)
    assert 0 < clipped < len(data)                                          # both branches occur
    want_stats, _ = opl.train_step(model, copy.deepcopy(data), packing=packing, module_args=args, **kw)
    step = PolicyStep(bb, weight, module_args=args, packing=packing, keep_logits_chunk=64, **kw)
    got_stats = step.train_step(copy.deepcopy(data))
    for k in ("pg_loss", "kl_loss", "entropy_loss"):
        assert got_stats[k] == pytest.approx(want_stats[k], rel=1e-5, abs=1e-7), k
    assert_close_rel(bb.tok.grad, tok.grad, 1e-5, "token-embedding grad")
    assert_close_rel(weight.grad, w.grad, 1e-5, "lm_head grad")


@pytest.mark.parametrize("packing", [False, True])
def test_host_copy_of_the_training_mask_equals_the_device_mask(dev, packing):
    """preprocess_data_list builds the shifted training mask twice: on the device (what the loss reads) and
    on the host, flattened the way the head step sees the tokens (what finds the rows that carry a gradient).
    The two must be the same mask."""
    from chatlearn_amd.algorithm.grpo_utils.policy_step import PolicyStep
    data = _samples(10, 23, True)
    data[3]["loss_mask"] = (torch.rand(data[3]["all_tokens"].numel(), generator=torch.Generator().manual_seed(1)) < 0.5).int()
    for s in data:
        s.setdefault("loss_mask", torch.cat([torch.zeros(s["prompt_token_length"], dtype=torch.int32),
                                             torch.ones(s["response_token_length"], dtype=torch.int32)]))
    bb = _Backbone(torch.float32).to(dev)
    weight = torch.zeros(VOCAB, H, device=dev)
    step = PolicyStep(bb, weight, packing=packing, max_token_in_seq=200, train_micro_batch_size=4)
    _, mbs = step.preprocess_data_list(copy.deepcopy(data), training=True)
    assert len(mbs) > 1
    for inputs in mbs:
        inputs = step._to_device(inputs)
        hidden = bb(inputs["all_tokens"], inputs["position_ids"])
        _, _, pick = step._flat_view(inputs, hidden)
        assert torch.equal(pick(inputs["loss_mask"]).cpu(), inputs["loss_mask_host"])


def test_stale_host_mask_is_refused(dev):
    """A host mask that does not match the device mask would silently drop gradients: the head step
    compares the two sums in the read-back it does anyway for the reference's assertions."""
    from chatlearn_amd import grpo_head_step
    T, Hd, V = 300, 64, 500
    g = torch.Generator().manual_seed(0)
    hidden, weight = torch.randn(T, Hd, generator=g).to(dev), (torch.randn(V, Hd, generator=g) * 0.1).to(dev)
    labels = torch.randint(0, V, (T,), generator=g).to(dev)
    mask = (torch.rand(T, generator=g) < 0.5).int()
    cu = torch.tensor([0, 100, 300], dtype=torch.int32, device=dev)
    lp = torch.full((T,), -6.0, device=dev)
    call = lambda host: grpo_head_step(hidden, weight, labels, lp, lp, torch.tensor([1.0, -1.0], device=dev), cu,
                                       mask.to(dev), n_tokens_total=float(mask.sum()), loss_mask_host=host)
    call(mask)
    stale = mask.clone()
    stale[int(torch.nonzero(mask)[0])] = 0
    with pytest.raises(ValueError, match="stale"):
        call(stale)
    with pytest.raises(ValueError, match="CPU copy"):
        call(mask[:-1])


def test_episode_through_records_advantages_and_train_steps(dev):
    """An episode as the trainer sees it: rollout records -> AdvantageComputer (group kernel) over the whole
    episode -> mini-batches in the replay buffer's fixed order -> PolicyStep.train_step per mini-batch, against
    the oracle's advantage restatement and loop on literally sliced mini-batches.  13 samples, one data-parallel
    rank, 3 mini-batches: even_slice(13, 3) = [0, 5, 9, 13] (utils/utils.py:320-327: 13 = 3 * 4 + 1, the first
    slice is one longer); with two ranks, each rank's share is cut on its own: [0, 7, 13] -> [0, 4, 7, 10, 13]
    (data/data.py:160-167)."""
    from oracle import advantage as oadv
    from chatlearn_amd import records
    from chatlearn_amd.algorithm.grpo_utils.advantage_compute import AdvantageComputer
    from chatlearn_amd.algorithm.grpo_utils.policy_step import PolicyStep
    g = torch.Generator().manual_seed(41)
    episode = []
    for i in range(13):
        p, r = int(torch.randint(3, 10, (1,), generator=g)), int(torch.randint(5, 40, (1,), generator=g))
        prompt = {"prompt_uid": f"0_{i // 4}", "data_source": "toy", "rollout_round": 0}
        rec = records.rollout_record(prompt, torch.randint(0, VOCAB, (p,), generator=g).tolist(),
                                     torch.randint(0, VOCAB, (r,), generator=g).tolist(), "text")
        rec["rule_reward"] = float(torch.rand(1, generator=g) < 0.5)
        episode.append(rec)

    class _Buf:
        def __init__(self, b):
            self.buffer = b
    bb = _Backbone(torch.float32).to(dev)
    weight = (torch.randn(VOCAB, H, generator=g) * 0.05).to(dev).requires_grad_(True)
    model, tok, pos, w = _oracle_model(bb, weight)
    kw = dict(max_token_in_seq=120, train_micro_batch_size=4)
    args = {"entropy_coef": 0.0, "kl_coef": 0.01}
    # old / reference logprobs of every sample: the no-grad pass of the same loop
    step = PolicyStep(bb, weight, module_args=args, packing=True, **kw)
    got_ep = step.forward_step(copy.deepcopy(episode))
    for s in got_ep:
        s["ref_logprobs"] = s["old_logprobs"] - 0.05
    want_ep = opl.forward_step(model, copy.deepcopy(episode), packing=True, trainable=True, **kw)
    for s, mine in zip(want_ep, got_ep):
        assert_close_rel(mine["old_logprobs"], s["old_logprobs"], 1e-5, "per-sample old logprobs")
        # from here on both sides train on the same records (the kernel's), as a trainer would
        s["old_logprobs"], s["ref_logprobs"] = mine["old_logprobs"].cpu(), mine["ref_logprobs"].cpu()
    # advantages over the whole episode (the last group of 13 = 3 * 4 + 1 samples is incomplete and stays pooled)
    comp = AdvantageComputer(num_inference_per_prompt=4, device=dev)
    got_ep = comp([_Buf(got_ep)])
    ocomp = oadv.AdvantageComputer(4)
    want_ep = ocomp([oadv._Buffer(want_ep)])
    assert [float(s["advantages"]) for s in got_ep] == [float(s["advantages"]) for s in want_ep]
    assert dict(comp.rule_reward_buffer) == dict(ocomp.rule_reward_buffer) and list(comp.rule_reward_buffer) == ["0_3"]
    for s in got_ep:
        records.check_train_record(s, training=True)
    assert records.minibatch_slice_index(13, 2, 2) == [0, 4, 7, 10, 13]
    got_batches = list(records.iter_fixed_order(got_ep, dp_size=1, num_minibsz=3))
    assert [len(b) for b in got_batches] == [5, 4, 4]
    want_batches = [want_ep[0:5], want_ep[5:9], want_ep[9:13]]
    for mine, theirs in zip(got_batches, want_batches):
        assert [s["prompt_uid"] for s in mine] == [s["prompt_uid"] for s in theirs]
        bb.zero_grad()
        weight.grad = None
        tok.grad = pos.grad = w.grad = None
        got_stats = step.train_step(copy.deepcopy(mine))
        want_stats, _ = opl.train_step(model, copy.deepcopy(theirs), packing=True, module_args=args, **kw)
        for k in ("pg_loss", "kl_loss", "entropy_loss"):
            assert got_stats[k] == pytest.approx(want_stats[k], rel=1e-5, abs=1e-7), k
        assert_close_rel(bb.tok.grad, tok.grad, 1e-5, "token-embedding grad")
        assert_close_rel(weight.grad, w.grad, 1e-5, "lm_head grad")


class _VLBackbone(torch.nn.Module):
    """Stand-in for a vision-language decoder: token embedding + one embedding per position channel + a
    projection of the micro-batch's image patches (their mean), so that every carried input reaches the
    hidden states."""

    def __init__(self, dtype, seed=0):
        super().__init__()
        g = torch.Generator().manual_seed(seed)
        self.tok = torch.nn.Parameter(torch.randn(VOCAB, H, generator=g).to(dtype))
        self.pos = torch.nn.Parameter((torch.randn(4, MAXLEN * 2, H, generator=g) * 0.1).to(dtype))
        self.vis = torch.nn.Parameter((torch.randn(6, H, generator=g) * 0.1).to(dtype))

    def forward(self, input_ids, position_ids, pixel_values=None, image_grid_thw=None):
        h = self.tok[input_ids]
        for ch in range(position_ids.shape[0]):
            h = h + self.pos[ch][position_ids[ch]]
        scale = image_grid_thw.to(h.dtype).prod(dim=1).sum() * 0.01
        return h + (pixel_values.to(h.dtype).mean(dim=0) @ self.vis) * scale


@pytest.mark.parametrize("packing", [False, True])
@pytest.mark.parametrize("prepend", [False, True])
def test_vision_language_inputs_reach_the_backbone_and_train(dev, packing, prepend):
    """model_type = 'vlm': the three position channels, pixel_values and image_grid_thw are carried to the
    backbone as the reference carries them to the model (policy_trainer.py:104-152,206-214), on the 4-D
    unpad_input branch when packing; train_step against the oracle loop."""
    from chatlearn_amd.algorithm.grpo_utils.policy_step import PolicyStep
    g = torch.Generator().manual_seed(77)
    data = _samples(7, 29, True)
    for s in data:
        p = s["prompt_token_length"]
        s["position_ids"] = [sorted(torch.randint(0, p, (p,), generator=g).tolist()) for _ in range(3)]
        n_patch = int(torch.randint(1, 5, (1,), generator=g))
        s["pixel_values"] = torch.randn(n_patch, 6, generator=g)
        s["image_grid_thw"] = torch.tensor([[1, 1, n_patch]])
    bb = _VLBackbone(torch.float32).to(dev)
    weight = (torch.randn(VOCAB, H, generator=g) * 0.05).to(dev).requires_grad_(True)
    tok, pos, vis = (x.detach().double().cpu().requires_grad_(True) for x in (bb.tok, bb.pos, bb.vis))
    w = weight.detach().double().cpu().requires_grad_(True)

    def model(ids, position_ids, pixel_values=None, image_grid_thw=None):
        h = tok[ids]
        for ch in range(position_ids.shape[0]):
            h = h + pos[ch][position_ids[ch]]
        scale = image_grid_thw.double().prod(dim=1).sum() * 0.01
        return torch.nn.functional.linear(h + (pixel_values.double().mean(dim=0) @ vis) * scale, w)
    args = {"entropy_coef": 0.0, "kl_coef": 0.02}
    kw = dict(max_token_in_seq=200, train_micro_batch_size=3)
    okw = dict(model_type="vlm", prepend_text_position_channel=prepend, **kw)
    centred = opl.forward_step(model, copy.deepcopy(data), packing=packing, trainable=True, **okw)
    for s, c in zip(data, centred):
        s["old_logprobs"] = (c["old_logprobs"] + (s["old_logprobs"] + 8.0)).float()
        s["ref_logprobs"] = (c["old_logprobs"] + (s["ref_logprobs"] + 8.0)).float()
    want_stats, _ = opl.train_step(model, copy.deepcopy(data), packing=packing, module_args=args, **okw)
    step = PolicyStep(bb, weight, module_args=args, packing=packing, model_type="vlm",
                      prepend_text_position_channel=prepend, **kw)
    # what the backbone receives, against the oracle's pre-processing, bit for bit
    _, got_mbs = step.preprocess_data_list(copy.deepcopy(data), training=True)
    _, want_mbs = opl.preprocess_data_list(copy.deepcopy(data), True, packing=packing, **okw)
    assert len(got_mbs) == len(want_mbs)
    for a, b in zip(got_mbs, want_mbs):
        assert torch.equal(a["position_ids"].cpu(), b["position_ids"])
        assert a["position_ids"].shape[0] == (4 if (packing and prepend) else 3)
        assert torch.equal(a["all_tokens"].cpu(), b["all_tokens"]) and torch.equal(a["labels"].cpu(), b["labels"])
        assert torch.equal(a["pixel_values"], b["pixel_values"]) and torch.equal(a["image_grid_thw"], b["image_grid_thw"])
    got_stats = step.train_step(copy.deepcopy(data))
    for k in ("pg_loss", "kl_loss", "entropy_loss"):
        assert got_stats[k] == pytest.approx(want_stats[k], rel=1e-5, abs=1e-7), k
    assert_close_rel(bb.tok.grad, tok.grad, 1e-5, "token-embedding grad")
    assert_close_rel(bb.pos.grad, pos.grad, 1e-5, "position-channel grad")
    assert_close_rel(bb.vis.grad, vis.grad, 1e-5, "vision-projection grad")
    assert_close_rel(weight.grad, w.grad, 1e-5, "lm_head grad")
    # the no-grad pass carries them too
    recs = step.forward_step(copy.deepcopy(data))
    for a, b in zip(recs, centred):
        assert_close_rel(a["old_logprobs"], b["old_logprobs"], 1e-5, "per-sample logprobs (vlm)")
