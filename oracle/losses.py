"""Oracle: GRPO / GSPO clipped-ratio surrogate, k3 KL and loss assembly.

Test infrastructure only; never imported by the product package.

Reference semantics restated here:
  * token-level GRPO surrogate                    loss_gallery.py:6-33
  * sequence-level GSPO surrogate + clip flags    loss_gallery.py:35-74
  * FSDP loss assembly (masked sums / N, k3 KL,
    entropy bonus, total)                         policy_trainer.py:263-286
  * FSDP metrics                                  policy_trainer.py:301-311
  * Megatron loss dict and loss_func reduction    train_helper.py:426-547
"""
import torch


def _adv_column(advantages, like):
    """torch.tensor(list) on the device of ``like``, one value per row
    (loss_gallery.py:19,53).  A list of numpy float64 becomes a float64
    tensor, a list of Python floats float32: exactly torch's rule."""
    return torch.tensor(advantages).to(like.device).unsqueeze(-1)


def _clipped_surrogate(ratio, adv, pos_clip_ratio, neg_clip_ratio, final_clip_ratio):
    unclipped = -adv * ratio
    clipped = -adv * torch.clamp(ratio, 1 - neg_clip_ratio, 1 + pos_clip_ratio)
    worst = torch.max(unclipped, clipped)
    cap = torch.ones_like(unclipped) * final_clip_ratio
    return torch.min(worst, cap), unclipped, clipped


def calculate_grpo_loss(log_probs, old_log_probs, advantages, diff_clip_ratio=10,
                        pos_clip_ratio=0.2, neg_clip_ratio=0.2, final_clip_ratio=3.0):
    """loss_gallery.py:6-33."""
    delta = torch.clamp(log_probs - old_log_probs, max=diff_clip_ratio)
    ratio = torch.exp(delta)
    adv = _adv_column(advantages, delta)
    loss, _, _ = _clipped_surrogate(ratio, adv, pos_clip_ratio, neg_clip_ratio, final_clip_ratio)
    assert not torch.isnan(loss).any(), "pg loss is nan"
    return loss.contiguous()


def calculate_gspo_loss(log_probs, old_log_probs, advantages, diff_clip_ratio=10,
                        pos_clip_ratio=1e-3, neg_clip_ratio=1e-3, final_clip_ratio=0.01,
                        loss_mask=None):
    """loss_gallery.py:35-74.  The per-row mean of (lp - old) over masked
    positions is a constant (detached); the gradient reaches lp only through
    ``lp - lp.detach()``, so d(seq ratio)/d lp_t carries no 1/|y| factor."""
    delta = log_probs - old_log_probs
    kept = torch.where(loss_mask.bool(), delta.detach(), 0.0)
    row_mean = (kept * loss_mask).sum(axis=1) / (loss_mask.sum(axis=1) + 1e-8)
    seq_delta = log_probs - log_probs.detach() + row_mean.unsqueeze(1)
    ratio = torch.exp(torch.clamp(seq_delta, max=diff_clip_ratio))
    adv = _adv_column(advantages, ratio)
    is_pos = (ratio > (1 + pos_clip_ratio)) * (adv > 0)
    is_neg = (ratio < (1 - neg_clip_ratio)) * (adv < 0)
    loss, unclipped, clipped = _clipped_surrogate(ratio, adv, pos_clip_ratio, neg_clip_ratio,
                                                  final_clip_ratio)
    is_clipped = clipped > unclipped
    assert not torch.isnan(loss).any(), "pg loss is nan"
    return loss.contiguous(), is_pos, is_neg, is_clipped


def k3_kl(ref_logprobs, logprobs):
    """k = ref - lp; kl = clamp(exp(k) - k - 1, -10, 10) (policy_trainer.py:269-276)."""
    k = ref_logprobs - logprobs
    ratio = torch.exp(k)
    assert not torch.isinf(ratio).any(), "kl loss ratio has inf values"
    assert not torch.isnan(ratio).any(), "kl loss ratio has nan values"
    return torch.clamp(ratio - k - 1, min=-10, max=10)


def fsdp_policy_loss(logprobs, entropy, old_logprobs, ref_logprobs, advantages, loss_mask,
                     response_token_length_total, *, entropy_coef=0.0, kl_coef=0.0,
                     pos_clip_ratio=0.2, neg_clip_ratio=0.2, diff_clip_ratio=10,
                     final_clip_ratio=3, fsdp_size=1, use_group_sequence_policy=False):
    """One micro-batch of policy_trainer.py:253-286 on padded [B, S] tensors.

    Returns (total_loss, dict of the detached masked per-token vectors and the
    three means).  ``use_group_sequence_policy`` swaps in the GSPO surrogate on
    this call path; the reference only wires GSPO into its Megatron trainer
    (train_helper.py:491-506), the arithmetic is the same.
    """
    if use_group_sequence_policy:
        loss, *_ = calculate_gspo_loss(logprobs, old_logprobs, advantages, diff_clip_ratio,
                                       pos_clip_ratio, neg_clip_ratio, final_clip_ratio, loss_mask)
    else:
        loss = calculate_grpo_loss(logprobs, old_logprobs, advantages, diff_clip_ratio,
                                   pos_clip_ratio, neg_clip_ratio, final_clip_ratio)
    keep = loss_mask.bool()
    n_tok = response_token_length_total
    pg = torch.masked_select(loss, keep)
    ent = torch.masked_select(entropy, keep)
    ent_mean = ent.sum() / n_tok * fsdp_size
    k = torch.masked_select(ref_logprobs - logprobs, keep)
    ratio = torch.exp(k)
    assert not torch.isinf(ratio).any(), "kl loss ratio has inf values"
    assert not torch.isnan(ratio).any(), "kl loss ratio has nan values"
    kl = torch.clamp((ratio - k - 1).contiguous(), min=-10, max=10)
    kl_mean = kl.sum() / n_tok * fsdp_size
    pg_mean = pg.sum() / n_tok * fsdp_size
    total = pg_mean
    if entropy_coef > 0:
        total = total - entropy_coef * ent_mean
    if kl_coef > 0:
        total = total + kl_coef * kl_mean
    parts = {"pg_loss": pg.detach(), "entropy_loss": ent.detach(), "kl_loss": kl.detach(),
             "pg_loss_mean": pg_mean.detach(), "entropy_loss_mean": ent_mean.detach(),
             "kl_loss_mean": kl_mean.detach()}
    return total, parts


def fsdp_train_metrics(pg_list, ent_list, kl_list, response_token_length_total, fsdp_size=1):
    """policy_trainer.py:301-303: pg is a sum over N, the other two plain means."""
    return {
        "pg_loss": (torch.cat(pg_list).sum() / response_token_length_total * fsdp_size).item(),
        "kl_loss": torch.cat(kl_list).mean().item(),
        "entropy_loss": torch.cat(ent_list).mean().item(),
    }


def megatron_all_losses(logprobs, entropy, old_logprobs, ref_logprobs, advantages, loss_mask, *,
                        use_group_sequence_policy=False, pos_clip_ratio=0.2, neg_clip_ratio=0.2,
                        diff_clip_ratio=10, final_clip_ratio=3):
    """train_helper.py:465-547 after the logprob/entropy have been formed."""
    if use_group_sequence_policy:
        pg, is_pos, is_neg, is_clip = calculate_gspo_loss(
            logprobs, old_logprobs, advantages, diff_clip_ratio, pos_clip_ratio, neg_clip_ratio,
            final_clip_ratio, loss_mask)
    else:
        pg = calculate_grpo_loss(logprobs, old_logprobs, advantages, diff_clip_ratio,
                                 pos_clip_ratio, neg_clip_ratio, final_clip_ratio)
    k = ref_logprobs - logprobs
    ratio = torch.exp(k)
    ratio[~loss_mask.bool()] = 1
    assert not torch.isinf(ratio).any(), "kl loss ratio has inf values"
    assert not torch.isnan(ratio).any(), "kl loss ratio has nan values"
    kl = torch.clamp((ratio - k - 1).contiguous(), min=-10, max=10)
    out = {"pg_loss": pg, "entropy_loss": entropy, "kl_loss": kl}
    if use_group_sequence_policy:
        out.update({"is_positive_clipped": is_pos, "is_negative_clipped": is_neg,
                    "is_clipped": is_clip, "is_positive_clipped_sample_average": is_pos,
                    "is_negative_clipped_sample_average": is_neg,
                    "is_clipped_sample_average": is_clip})
    return out


def megatron_loss_func(loss_mask, losses):
    """train_helper.py:426-463: masked sums (or masked means for *_sample_average);
    only ``pg_loss`` is back-propagated; returns (loss, num_tokens, report)."""
    m = loss_mask.float()
    total = 0
    report = {}
    for key, val in losses.items():
        if key != "pg_loss":
            val = val.detach()
        if key.endswith("_sample_average"):
            red = (val.float() * m).sum() / (1e-5 + m.sum())
        else:
            red = (val.float() * m).sum()
        if key == "pg_loss":
            total = total + red
        report[key] = red.detach().clone().to(torch.float)
    n = m.sum().clone().detach().to(torch.int)
    report["num_tokens"] = n
    report["num_samples"] = torch.ones_like(n)
    return total, n, report
