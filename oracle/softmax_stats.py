"""Oracle: lm_head projection, per-token logprob, entropy, and their backward.

Test infrastructure only; never imported by the product package.

Reference semantics restated here:
  * lm_head logits ``z = hidden @ W^T``          policy_trainer.py:216-221
    (HF ``nn.Linear(H, V, bias=False)``; under FSDP2 the module runs in bf16,
    fsdp_module.py:357, so the reference's logits are bf16-rounded).
  * ``logprobs_from_logits``                       trainer_utils.py:46-52
  * ``entropy_from_logits``                        trainer_utils.py:27-31
  * ``entropy_from_logits_with_chunking``          trainer_utils.py:33-44
  * vocab-parallel entropy at tp=1                 train_helper.py:605-627
  * backward through the three of them (autograd at policy_trainer.py:286).

Temperature (``z / tau`` before the softmax) is not in the reference; it is the
closed-form extension asked for by the long-context benchmark configuration.
"""
import torch
import torch.nn.functional as F


def lm_head_logits(hidden, weight, temperature=1.0, compute_dtype=None, round_logits_to=None):
    """z[t, v] = sum_h hidden[t, h] * W[v, h] / tau.

    ``compute_dtype`` picks the accumulation type (float64 gives the "truth"
    used to judge both the reference-like and the fused result);
    ``round_logits_to`` reproduces the reference's bf16 rounding of the logits.
    """
    cd = compute_dtype or hidden.dtype
    z = F.linear(hidden.to(cd), weight.to(cd))
    if round_logits_to is not None:
        z = z.to(round_logits_to).to(cd)
    if temperature != 1.0:
        z = z / temperature
    return z


def logprobs_from_logits(logits, labels):
    """log_softmax over the last dim, then gather the label column (trainer_utils.py:46-52)."""
    lsm = F.log_softmax(logits, dim=-1)
    return lsm.gather(-1, labels.unsqueeze(-1)).squeeze(-1)


def entropy_from_logits(logits):
    """H = logsumexp(z) - sum softmax(z) * z (trainer_utils.py:27-31)."""
    p = torch.softmax(logits, dim=-1)
    return torch.logsumexp(logits, dim=-1) - (p * logits).sum(-1)


def entropy_from_logits_with_chunking(logits, chunk_size=512):
    """Same value as entropy_from_logits, walked in chunks along dim 1; the
    result buffer is default-dtype (fp32) zeros (trainer_utils.py:33-44)."""
    out = torch.zeros(logits.shape[:-1], device=logits.device)
    for lo in range(0, logits.shape[1], chunk_size):
        sl = logits[:, lo:lo + chunk_size]
        out[:, lo:lo + chunk_size] = entropy_from_logits(sl)
    return out


def vocab_parallel_entropy_tp1(logits):
    """train_helper.py:605-627 with a tensor-parallel group of one rank:
    fp32 forced, max-shifted exponentials, product with the UNshifted logits."""
    z = logits.float()
    m = z.max(-1).values
    e = (z - m.unsqueeze(-1)).exp()
    s = e.sum(-1)
    u = (e / s.unsqueeze(-1) * z).sum(-1)
    return m + s.log() - u


def fused_head_forward(hidden, weight, labels, temperature=1.0, compute_dtype=torch.float64,
                       round_logits_to=None):
    """(logprob, entropy, rowmax, lse) per packed token, via the full [T, V] logits."""
    z = lm_head_logits(hidden, weight, temperature, compute_dtype, round_logits_to)
    lse = torch.logsumexp(z, -1)
    lp = z.gather(-1, labels.unsqueeze(-1)).squeeze(-1) - lse
    ent = entropy_from_logits(z)
    return lp, ent, z.max(-1).values, lse


def fused_head_backward_closed_form(hidden, weight, labels, g_lp, g_ent, temperature=1.0,
                                    compute_dtype=torch.float64):
    """dz = g_lp (onehot - p) - g_ent p (log p + H); dhidden = dz W / tau; dW = dz^T hidden / tau.

    Written from the calculus, not from autograd, so that the autograd result
    of the restated forward and this closed form check each other.
    """
    cd = compute_dtype
    z = lm_head_logits(hidden, weight, temperature, cd)
    logp = F.log_softmax(z, -1)
    p = logp.exp()
    ent = -(p * logp).sum(-1)
    onehot = torch.zeros_like(p)
    onehot.scatter_(-1, labels.unsqueeze(-1), 1.0)
    dz = g_lp.to(cd).unsqueeze(-1) * (onehot - p)
    if g_ent is not None:
        dz = dz - g_ent.to(cd).unsqueeze(-1) * p * (logp + ent.unsqueeze(-1))
    dz = dz / temperature
    return dz @ weight.to(cd), dz.t() @ hidden.to(cd)


def fused_head_backward_autograd(hidden, weight, labels, g_lp, g_ent, temperature=1.0,
                                 compute_dtype=torch.float64):
    """Same gradients through torch autograd of the restated forward."""
    h = hidden.to(compute_dtype).detach().requires_grad_(True)
    w = weight.to(compute_dtype).detach().requires_grad_(True)
    z = F.linear(h, w) / temperature
    lp = logprobs_from_logits(z, labels)
    obj = (lp * g_lp.to(compute_dtype)).sum()
    if g_ent is not None:
        obj = obj + (entropy_from_logits(z) * g_ent.to(compute_dtype)).sum()
    obj.backward()
    return h.grad, w.grad
