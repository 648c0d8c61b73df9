"""Packing of padded batches into the variable-length layout the attention kernels consume, and back.
Same names and semantics as the reference's flash_attn/bert_padding.py (:9-95): `unpad_input` gathers the valid
tokens of a (batch, seqlen, ...) tensor into (total, ...) rows and returns the cumulative sequence lengths;
`pad_input` scatters rows back into a zero-filled padded tensor.  Both are differentiable.
"""
import torch
import torch.nn.functional as F


class IndexFirstAxis(torch.autograd.Function):
    """rows = input[indices] for a 2-D input, with a scatter as backward."""

    @staticmethod
    def forward(ctx, input, indices):
        assert input.ndim == 2
        ctx.save_for_backward(indices)
        ctx.first_axis_dim = input.shape[0]
        return input.index_select(0, indices)

    @staticmethod
    def backward(ctx, grad_output):
        (indices,) = ctx.saved_tensors
        grad_input = grad_output.new_zeros((ctx.first_axis_dim,) + tuple(grad_output.shape[1:]))
        grad_input.index_copy_(0, indices, grad_output)
        return grad_input, None


index_first_axis = IndexFirstAxis.apply


class IndexPutFirstAxis(torch.autograd.Function):
    """output = zeros(first_axis_dim, dim); output[indices] = values, with a gather as backward."""

    @staticmethod
    def forward(ctx, values, indices, first_axis_dim):
        assert indices.ndim == 1
        assert values.ndim == 2
        ctx.save_for_backward(indices)
        output = values.new_zeros((first_axis_dim, values.shape[1]))
        output.index_copy_(0, indices, values)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        (indices,) = ctx.saved_tensors
        return grad_output.index_select(0, indices), None, None


index_put_first_axis = IndexPutFirstAxis.apply


def unpad_input(hidden_states, attention_mask):
    """
    Arguments:
        hidden_states: (batch, seqlen, dim)
        attention_mask: (batch, seqlen), bool / int, nonzero = valid token.
    Return:
        hidden_states: (total_nnz, dim), the valid tokens in batch-major order.
        indices: (total_nnz,), positions of those tokens in the flattened (batch * seqlen) axis.
        cu_seqlens: (batch + 1,) int32 cumulative sequence lengths.
        max_seqlen_in_batch: int
    """
    seqlens = attention_mask.sum(dim=-1, dtype=torch.int32)
    indices = torch.nonzero(attention_mask.flatten(), as_tuple=False).flatten()
    max_seqlen_in_batch = int(seqlens.max().item())
    cu_seqlens = F.pad(torch.cumsum(seqlens, dim=0, dtype=torch.int32), (1, 0))
    flat = hidden_states.reshape(hidden_states.shape[0] * hidden_states.shape[1], -1)
    return index_first_axis(flat, indices), indices, cu_seqlens, max_seqlen_in_batch


def pad_input(hidden_states, indices, batch, seqlen):
    """
    Arguments:
        hidden_states: (total_nnz, dim)
        indices: (total_nnz,)
    Return:
        hidden_states: (batch, seqlen, dim), zero where no token was scattered.
    """
    output = index_put_first_axis(hidden_states, indices, batch * seqlen)
    return output.reshape(batch, seqlen, hidden_states.shape[-1])
