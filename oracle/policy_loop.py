"""Oracle: the FSDP policy trainer's micro-batch loops on one rank, text models.

Test infrastructure only; never imported by the product package.

Reference semantics restated here (sp_size = 1, fsdp_size = 1; vision-language inputs are carried
through as the reference carries them, model_type = 'vlm'):
  * preprocess_data_list      policy_trainer.py:80-172
  * train_step loop           policy_trainer.py:203-311   (without optimizer / grad clipping)
  * forward_step loop         policy_trainer.py:316-365

``model(input_ids, position_ids)`` stands for ``self.model(...).logits``: it returns
logits [b, s, V]; a vision-language model is called as
``model(input_ids, position_ids, pixel_values=..., image_grid_thw=...)`` (policy_trainer.py:206-214).  Everything runs on the CPU with the other oracle modules.

Pinned by tests/test_policy_loop_cpu.py: a three-sample case worked by hand from the
reference lines above (micro-batch order with a tie on the bin totals, packed token row,
indices, position ids, labels that roll across sequence boundaries, shifted training mask,
N, per-sample record lengths and values, train_stats) with literal expected tables, and the
sequence-level (GSPO) variant of the loss by hand-worked sequence ratios on the same case.
"""
import torch
import torch.nn.functional as F

from . import indexing as oi
from . import losses as ol
from . import packing as opk
from . import softmax_stats as osm


def preprocess_data_list(data_list, training, *, packing, max_token_in_seq=None, train_micro_batch_size=1,
                         generate_micro_batch_size=1, model_type="llm", prepend_text_position_channel=False):
    total_resp = torch.tensor(sum(d["response_token_length"] for d in data_list)) / 1   # / sp_size, all-reduce = identity
    if packing:
        mbs = opk.split_microbatch(data_list=data_list, max_train_token=max_token_in_seq, packing=True)
    else:
        size = train_micro_batch_size if training else generate_micro_batch_size
        mbs = opk.split_microbatch(data_list=data_list, micro_batch_size=size, packing=False)
    batches = [opk.batching(mb) for mb in mbs]
    out = []
    for b in batches:
        tokens_ = b["all_tokens"].long()
        p_len, r_len = b["prompt_token_length"], b["response_token_length"]
        ori_bs, ori_len = tokens_.size()
        attn, loss_mask, pos = oi.generate_loss_mask_position_ids(tokens_, p_len, r_len, b.get("position_ids", None))
        if "loss_mask" in b:
            loss_mask = b["loss_mask"]
        indices = None
        if packing:
            tokens_, indices, *_ = oi.unpad_input(tokens_.unsqueeze(-1), attn)
            tokens_ = tokens_.permute(1, 0)
            pos, *_ = oi.unpad_input(pos.unsqueeze(-1), attn)
            if model_type == "vlm":
                pos = pos.permute(0, 2, 1)                       # [3, 1, T]   (policy_trainer.py:121-123)
                if prepend_text_position_channel:                # transformers >= 4.55 (policy_trainer.py:124-125)
                    pos = torch.cat([pos[0:1], pos], dim=0)
            else:
                pos = pos.permute(1, 0)
        tokens = tokens_
        labels = oi.shift_labels(tokens)
        obj = {"all_tokens": tokens, "position_ids": pos, "labels": labels, "ori_seq_len": ori_len,
               "indices": indices, "ori_batch_size": ori_bs, "sample_ids": b["id_in_list"],
               "attention_mask": attn, "pad_size": 0}
        if model_type == "vlm":
            obj.update({"pixel_values": b.get("pixel_values", None), "image_grid_thw": b.get("image_grid_thw", None)})
        if training:
            obj.update({"loss_mask": oi.shift_loss_mask_fsdp(loss_mask), "old_logprobs": b["old_logprobs"], "ref_logprobs": b["ref_logprobs"],
                        "advantages": b["advantages"]})
        out.append(obj)
    return total_resp, out


def _repad(x, inputs, packing):
    if packing:
        return oi.pad_input(x[0, :x.shape[1] - inputs["pad_size"]].unsqueeze(-1), inputs["indices"],
                            inputs["ori_batch_size"], inputs["ori_seq_len"]).squeeze(-1)
    return F.pad(x, (0, inputs["ori_seq_len"] - x.shape[1]), mode="constant", value=0)


def _call_model(model, inputs, model_type):
    if model_type == "vlm":
        return model(inputs["all_tokens"], inputs["position_ids"], pixel_values=inputs["pixel_values"],
                     image_grid_thw=inputs["image_grid_thw"])
    return model(inputs["all_tokens"], inputs["position_ids"])


def train_step(model, data_list, *, packing, module_args, **prep):
    """Returns (train_stats, per-micro-batch totals); gradients accumulate in the model's parameters."""
    n_tok, mbs = preprocess_data_list(data_list, True, packing=packing, **prep)
    model_type = prep.get("model_type", "llm")
    pg_l, en_l, kl_l, totals = [], [], [], []
    for inputs in mbs:
        logits = _call_model(model, inputs, model_type)
        logprobs = osm.logprobs_from_logits(logits, inputs["labels"])
        ctx = torch.enable_grad() if module_args["entropy_coef"] > 0 else torch.no_grad()
        with ctx:
            entropy = osm.entropy_from_logits_with_chunking(logits)
        logprobs, entropy = _repad(logprobs, inputs, packing), _repad(entropy, inputs, packing)
        total, parts = ol.fsdp_policy_loss(
            logprobs, entropy, inputs["old_logprobs"], inputs["ref_logprobs"], inputs["advantages"],
            inputs["loss_mask"], n_tok, entropy_coef=module_args["entropy_coef"], kl_coef=module_args["kl_coef"],
            pos_clip_ratio=module_args.get("pos_clip_ratio", 0.2), neg_clip_ratio=module_args.get("neg_clip_ratio", 0.2),
            diff_clip_ratio=module_args.get("diff_clip_ratio", 10), final_clip_ratio=module_args.get("final_clip_ratio", 3),
            # the reference wires the sequence-level surrogate into its Megatron trainer only
            # (train_helper.py:491-506); on this loop it is the same arithmetic on the same padded rows
            use_group_sequence_policy=module_args.get("use_group_sequence_policy", False))
        total.backward()
        totals.append(total.detach())
        pg_l.append(parts["pg_loss"]); en_l.append(parts["entropy_loss"]); kl_l.append(parts["kl_loss"])
    return ol.fsdp_train_metrics(pg_l, en_l, kl_l, n_tok), totals


def forward_step(model, data, *, packing, trainable, **prep):
    _, mbs = preprocess_data_list(data, False, packing=packing, **prep)
    tag = "old_logprobs" if trainable else "ref_logprobs"
    for inputs in mbs:
        with torch.no_grad():
            logits = _call_model(model, inputs, prep.get("model_type", "llm"))
            logprobs = _repad(osm.logprobs_from_logits(logits, inputs["labels"]), inputs, packing)
        for sid, lp in zip(inputs["sample_ids"], oi.split_and_unpadding(logprobs, inputs["attention_mask"])):
            data[sid].update({tag: lp})
    return data
