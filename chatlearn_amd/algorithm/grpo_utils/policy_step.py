"""The micro-batch loops of the reference's FSDP policy trainer, for the head path only.

``PolicyStep`` mirrors ``PolicyTrainer.preprocess_data_list`` / ``train_step`` /
``forward_step`` (policy_trainer.py:80-172, 187-311, 313-365) on one rank (sp_size = 1), for
text models and - carrying the three-channel position ids, ``pixel_values`` and
``image_grid_thw`` through as the reference does - for vision-language ones: same
per-sample dict fields in, same ``train_stats`` keys and the same per-sample
``old_logprobs`` / ``ref_logprobs`` records out.  What differs is the
seam: instead of ``self.model(...).logits`` the caller supplies a ``backbone`` that
returns the final hidden states, and the lm_head weight; logits are never
materialised beyond one bounded chunk.  FSDP wrapping, the optimizer step and
gradient clipping stay with the caller.
"""
from typing import Any, Callable, Dict, List, Optional

import torch

from ... import ops
from ...fused import AUTO, grpo_head_step
from .trainer_utils import (batching, generate_loss_mask_position_ids, split_and_unpadding, split_microbatch,
                            unpad_input)

_DEFAULT_ARGS = {"entropy_coef": 0.0, "kl_coef": 0.0, "pos_clip_ratio": 0.2, "neg_clip_ratio": 0.2,
                 "diff_clip_ratio": 10, "final_clip_ratio": 3, "use_group_sequence_policy": False}


class PolicyStep:
    """policy trainer loops on top of the fused head"""

    def __init__(self, backbone: Callable[[torch.Tensor, torch.Tensor], torch.Tensor], lm_head_weight: torch.Tensor, *,
                 module_args: Optional[Dict[str, Any]] = None, packing: bool = False, max_token_in_seq: int = 32768,
                 train_micro_batch_size: int = 1, generate_micro_batch_size: int = 1, trainable: bool = True,
                 fsdp_size: int = 1, temperature: float = 1.0, dweight_buffer: Optional[torch.Tensor] = None,
                 keep_logits_chunk=AUTO, model_type: str = "llm",
                 prepend_text_position_channel: Optional[bool] = None):
        """``backbone(input_ids, position_ids)`` returns the final hidden states ``[b, s, H]``; with
        ``model_type='vlm'`` it is called as ``backbone(input_ids, position_ids, pixel_values=...,
        image_grid_thw=...)`` (policy_trainer.py:206-214).  ``prepend_text_position_channel``: packed
        vision-language position ids get the first channel repeated in front, which the reference does for
        transformers >= 4.55 (policy_trainer.py:124-125); ``None`` decides the same way from the installed
        transformers, if there is one."""
        self.backbone = backbone
        self.weight = lm_head_weight
        self.module_args = dict(_DEFAULT_ARGS)
        self.module_args.update(module_args or {})
        self.packing = packing
        self.max_token_in_seq = max_token_in_seq
        self.train_micro_batch_size = train_micro_batch_size
        self.generate_micro_batch_size = generate_micro_batch_size
        self.trainable = trainable
        self.fsdp_size = fsdp_size
        self.temperature = temperature
        self.dweight_buffer = dweight_buffer
        self.keep_logits_chunk = keep_logits_chunk
        self.model_type = model_type
        if prepend_text_position_channel is None and model_type == "vlm":
            try:
                import transformers
                from packaging.version import Version
                prepend_text_position_channel = Version(transformers.__version__) >= Version("4.55.0")
            except ImportError:
                prepend_text_position_channel = False
        self.prepend_text_position_channel = bool(prepend_text_position_channel)
        self._metric_prefix = "policy_trainer"
        self._metric_list = []
        self.device = lm_head_weight.device

    # ------------------------------------------------------------------ preprocessing
    def preprocess_data_list(self, data_list: List[Dict[str, Any]], training: bool):
        """Split into micro-batches, batch, build masks / position ids / labels, pack when asked
        (policy_trainer.py:80-172).  The all-reduce of the response-token count is the identity here."""
        response_token_length_total = torch.tensor(
            sum(data["response_token_length"] for data in data_list), device=self.device) / 1
        if self.packing:
            microbatch_list = split_microbatch(data_list=data_list, max_train_token=self.max_token_in_seq,
                                               packing=self.packing)
        else:
            size = self.train_micro_batch_size if training else self.generate_micro_batch_size
            microbatch_list = split_microbatch(data_list=data_list, micro_batch_size=size, packing=self.packing)
        data_after_process = []
        for data_b in (batching(mb) for mb in microbatch_list):
            tokens_ = data_b["all_tokens"].long()
            ori_batch_size, ori_seq_len = tokens_.size()
            # vision-language samples carry their prompt's three position channels and the image tensors
            attn_mask, loss_mask, position_ids = generate_loss_mask_position_ids(
                tokens_, data_b["prompt_token_length"], data_b["response_token_length"], data_b.get("position_ids", None))
            if 'loss_mask' in data_b:
                loss_mask = data_b['loss_mask']
            indices = cu_seqlens = None
            if self.packing and 'position_ids' not in data_b and self.model_type != "vlm":
                # unpad_input of tokens and position ids plus the label roll (policy_trainer.py:143-162) in
                # one device pass driven by the length lists; no device value is read back
                packed = ops.thd_pack(tokens_.to(self.device), data_b["prompt_token_length"],
                                      data_b["response_token_length"], align=1, pad_token=0,
                                      want_loss_mask=False, want_position_ids=True, verify_on_device=False)
                tokens = packed["tokens"].unsqueeze(0)
                position_ids = packed["position_ids"].unsqueeze(0)
                labels = packed["labels"].unsqueeze(0)
                indices, cu_seqlens = packed["indices"], packed["cu_seqlens_padded"]
                width = packed["max_seqlen_padded"]
                if width != ori_seq_len:      # the batch is padded wider than its longest sample
                    indices = (indices // width) * ori_seq_len + indices % width
            else:
                if self.packing:
                    tokens_, indices, cu_seqlens, _ = unpad_input(tokens_.unsqueeze(-1).to(self.device),
                                                                  attn_mask.to(self.device))
                    tokens_ = tokens_.permute(1, 0)
                    position_ids, *_ = unpad_input(position_ids.unsqueeze(-1).to(self.device),
                                                   attn_mask.to(self.device))
                    if self.model_type == "vlm":
                        position_ids = position_ids.permute(0, 2, 1)        # [3, 1, T] (policy_trainer.py:121-123)
                        if self.prepend_text_position_channel:
                            position_ids = torch.cat([position_ids[0:1], position_ids], dim=0)
                    else:
                        position_ids = position_ids.permute(1, 0)
                tokens = tokens_
                # labels roll along the (packed or padded) token row (policy_trainer.py:135,160)
                labels, _ = ops.shift_labels(tokens.to(self.device).contiguous(), None, zero_last=False)
            # the training mask rolls along the padded rows and loses its last column (policy_trainer.py:161-162)
            shifted = shifted_host = None
            if training:
                _, shifted = ops.shift_labels(None, loss_mask.to(self.device).to(torch.int32).contiguous(),
                                              zero_last=True)
                # the same shift on the host copy, flattened the way the kernels see the tokens: it tells the
                # head step which rows carry a gradient without reading anything back from the device
                shifted_host = torch.roll(loss_mask.cpu().to(torch.int32), shifts=-1, dims=1)
                shifted_host[:, -1] = 0
                if self.packing:
                    lens = [p + r for p, r in zip(data_b["prompt_token_length"], data_b["response_token_length"])]
                    shifted_host = torch.cat([shifted_host[i, :n] for i, n in enumerate(lens)])
                else:
                    shifted_host = shifted_host.reshape(-1)
            data_obj = {"all_tokens": tokens, "position_ids": position_ids, "labels": labels,
                        "ori_seq_len": ori_seq_len, "indices": indices, "cu_seqlens": cu_seqlens,
                        "ori_batch_size": ori_batch_size, "sample_ids": data_b["id_in_list"],
                        "attention_mask": attn_mask, "pad_size": 0}
            if self.model_type == "vlm":
                data_obj.update({"pixel_values": data_b.get("pixel_values", None),
                                 "image_grid_thw": data_b.get("image_grid_thw", None)})
            if training:
                data_obj.update({"loss_mask": shifted, "loss_mask_host": shifted_host,
                                 "old_logprobs": data_b["old_logprobs"],
                                 "ref_logprobs": data_b["ref_logprobs"], "advantages": data_b["advantages"]})
            data_after_process.append(data_obj)
        return response_token_length_total, data_after_process

    def _to_device(self, inputs):
        return {k: (v.to(self.device) if isinstance(v, torch.Tensor) and not k.endswith("_host") else v)
                for k, v in inputs.items()}

    def _backbone(self, inputs):
        if self.model_type == "vlm":
            return self.backbone(inputs["all_tokens"], inputs["position_ids"], pixel_values=inputs["pixel_values"],
                                 image_grid_thw=inputs["image_grid_thw"])
        return self.backbone(inputs["all_tokens"], inputs["position_ids"])

    def _flat_view(self, inputs, hidden):
        """hidden as [T, H] plus the per-token views of the padded [B, S] side inputs."""
        H = hidden.shape[-1]
        if self.packing:
            idx = inputs["indices"]
            pick = lambda x: ops.gather_rows(x.reshape(-1, 1).contiguous(), idx).reshape(-1)
            return hidden.reshape(-1, H), inputs["cu_seqlens"], pick
        B, S = inputs["ori_batch_size"], inputs["ori_seq_len"]
        cu = torch.arange(0, (B + 1) * S, S, dtype=torch.int32, device=self.device)
        return hidden.reshape(-1, H), cu, (lambda x: x.reshape(-1))

    # ------------------------------------------------------------------ training
    def train_step(self, data_list: List[Dict[str, Any]], **kwargs):  # pylint: disable=unused-argument
        """Forward, loss and backward over all micro-batches (policy_trainer.py:187-311 without the
        optimizer).  Gradients reach the backbone through ``hidden.backward`` and the lm_head weight
        through ``dweight_buffer`` (fp32, accumulated) or ``lm_head_weight.grad``."""
        args = self.module_args
        n_tok, data_list = self.preprocess_data_list(data_list=data_list, training=True)
        n_tok_f = float(n_tok.item())
        sums = torch.zeros(8, dtype=torch.float64, device=self.device)
        dw = self.dweight_buffer
        accumulate = dw is not None
        wt_cache = {}   # the weight does not change between the micro-batches of this step
        ws_cache = {}   # kept logits and head scratch memory, shared by the micro-batches of this step
        for inputs in data_list:
            inputs = self._to_device(inputs)
            hidden = self._backbone(inputs)
            flat, cu, pick = self._flat_view(inputs, hidden)
            adv = torch.tensor(inputs["advantages"]).to(self.device)
            out = grpo_head_step(
                flat.detach(), self.weight.detach(), inputs["labels"].reshape(-1), pick(inputs["old_logprobs"].float()),
                pick(inputs["ref_logprobs"].float()), adv, cu, pick(inputs["loss_mask"]), n_tokens_total=n_tok_f,
                fsdp_size=self.fsdp_size, use_group_sequence_policy=args["use_group_sequence_policy"],
                pos_clip_ratio=args["pos_clip_ratio"], neg_clip_ratio=args["neg_clip_ratio"],
                diff_clip_ratio=args["diff_clip_ratio"], final_clip_ratio=args["final_clip_ratio"],
                kl_coef=args["kl_coef"], entropy_coef=args["entropy_coef"], temperature=self.temperature, dweight=dw,
                accumulate_dweight=accumulate, need_dhidden=flat.requires_grad,
                keep_logits_chunk=self.keep_logits_chunk,
                # only masked sums leave this method, so rows outside the loss mask need no forward either
                skip_masked_forward=True, weight_t_cache=wt_cache, loss_mask_host=inputs["loss_mask_host"],
                workspace_cache=ws_cache)
            dw, accumulate = out["dweight"], True
            if flat.requires_grad:
                hidden.backward(out["dhidden"].reshape(hidden.shape))
            sums += out["sums"]
        if self.dweight_buffer is None and dw is not None and self.weight.requires_grad:
            g = dw.to(self.weight.dtype)
            self.weight.grad = g if self.weight.grad is None else self.weight.grad + g
        pg_sum, kl_sum, en_sum, cnt = sums[:4].tolist()
        train_stats = {
            "pg_loss": pg_sum / n_tok_f * self.fsdp_size,        # sum over N  (policy_trainer.py:301)
            "kl_loss": kl_sum / cnt if cnt else float("nan"),    # plain means over the masked tokens (:302-303)
            "entropy_loss": en_sum / cnt if cnt else float("nan"),
        }
        self._metric_list.append(train_stats)
        return train_stats

    # ------------------------------------------------------------------ no-grad logprob recompute
    def forward_step(self, data: List[Dict[str, Any]], **kwargs) -> List[Dict[str, Any]]:  # pylint: disable=unused-argument
        """Per-sample logprobs of the old / reference policy (policy_trainer.py:313-365); each sample gets a
        1-D tensor of length prompt + response under ``old_logprobs`` (trainable) or ``ref_logprobs``."""
        _, data_list = self.preprocess_data_list(data_list=data, training=False)
        tag = "old_logprobs" if self.trainable else "ref_logprobs"
        for inputs in data_list:
            inputs = self._to_device(inputs)
            with torch.no_grad():
                hidden = self._backbone(inputs)
                lp, *_ = ops.lmhead_forward(hidden.reshape(-1, hidden.shape[-1]), self.weight,
                                            inputs["labels"].reshape(-1), self.temperature, need_entropy=False)
                B, S = inputs["ori_batch_size"], inputs["ori_seq_len"]
                if self.packing:
                    lp = ops.scatter_rows(lp.reshape(-1, 1), inputs["indices"], B * S).reshape(B, S)
                else:
                    lp = lp.reshape(B, S)
            for sample_id, logprob in zip(inputs['sample_ids'], split_and_unpadding(lp, inputs['attention_mask'])):
                data[sample_id].update({tag: logprob})
        return data

    def get_and_clear_metrics(self):
        out, self._metric_list = self._metric_list, []
        return self._metric_prefix, out
