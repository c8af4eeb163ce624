"""Mirror of the three ``flash_attn.bert_padding`` helpers the reference imports
(trainer_utils.py:22, policy_trainer.py:24, train_helper.py:25): a row gather,
its inverse scatter into zeros, both differentiable, on the HIP row kernels."""
import torch

from . import ops


class _IndexFirstAxis(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, indices):
        ctx.save_for_backward(indices)
        ctx.n_rows = x.shape[0]
        return ops.gather_rows(x, indices)

    @staticmethod
    def backward(ctx, g):
        (indices,) = ctx.saved_tensors
        return ops.scatter_rows(g.contiguous(), indices, ctx.n_rows), None


class _IndexPutFirstAxis(torch.autograd.Function):
    @staticmethod
    def forward(ctx, values, indices, n_rows):
        ctx.save_for_backward(indices)
        return ops.scatter_rows(values, indices, n_rows)

    @staticmethod
    def backward(ctx, g):
        (indices,) = ctx.saved_tensors
        return ops.gather_rows(g.contiguous(), indices), None, None


def index_first_axis(x, indices):
    """x [N, ...] -> x[indices]"""
    return _IndexFirstAxis.apply(x, indices)


def index_put_first_axis(values, indices, first_axis_dim):
    return _IndexPutFirstAxis.apply(values, indices, first_axis_dim)


def pad_input(hidden_states, indices, batch, seqlen):
    """(total_nnz, ...) -> (batch, seqlen, ...): zeros with the rows written back at ``indices``."""
    out = index_put_first_axis(hidden_states, indices, batch * seqlen)
    return out.reshape(batch, seqlen, *hidden_states.shape[1:])
