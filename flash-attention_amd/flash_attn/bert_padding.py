"""Packing of padded batches into the variable-length layout the attention kernels consume, and back.
Same names and semantics as the reference's flash_attn/bert_padding.py (:9-95): `unpad_input` gathers the valid
tokens of a (batch, seqlen, ...) tensor into (total, ...) rows and returns the cumulative sequence lengths;
`pad_input` scatters rows back into a zero-filled padded tensor.  Both are differentiable.

For GPU tensors the row gather / scatter run as HIP kernels of the attention library (fa_gather_rows /
fa_scatter_rows; the scatter writes the padded tensor in one pass, without a zero fill); host tensors use the
equivalent torch indexing, which is what the reference does on every device.
"""
import torch
import torch.nn.functional as F

from . import flash_attn_gfx950 as _backend


# The device of the INPUT decides, never the availability of the library: a GPU tensor always goes to the HIP kernels
# (and raises if the library is not built); only tensors that live in host memory, which no GPU kernel could read,
# are indexed by torch.
def _gather(input, indices):
    if input.is_cuda:
        return _backend.gather_rows(input, indices)
    return input.index_select(0, indices)


def _scatter(values, indices, first_axis_dim):
    if values.is_cuda:
        return _backend.scatter_rows(values, indices, first_axis_dim)
    out = values.new_zeros((first_axis_dim,) + tuple(values.shape[1:]))
    out.index_copy_(0, indices, values)
    return out


class IndexFirstAxis(torch.autograd.Function):
    """rows = input[indices] for a 2-D input, with a scatter as backward."""

    @staticmethod
    def forward(ctx, input, indices):
        assert input.ndim == 2
        ctx.save_for_backward(indices)
        ctx.first_axis_dim = input.shape[0]
        return _gather(input if input.stride(-1) == 1 else input.contiguous(), indices)

    @staticmethod
    def backward(ctx, grad_output):
        (indices,) = ctx.saved_tensors
        return _scatter(grad_output if grad_output.stride(-1) == 1 else grad_output.contiguous(), indices,
                        ctx.first_axis_dim), None


index_first_axis = IndexFirstAxis.apply


class IndexPutFirstAxis(torch.autograd.Function):
    """output = zeros(first_axis_dim, dim); output[indices] = values, with a gather as backward."""

    @staticmethod
    def forward(ctx, values, indices, first_axis_dim):
        assert indices.ndim == 1
        assert values.ndim == 2
        ctx.save_for_backward(indices)
        return _scatter(values if values.stride(-1) == 1 else values.contiguous(), indices, first_axis_dim)

    @staticmethod
    def backward(ctx, grad_output):
        (indices,) = ctx.saved_tensors
        return _gather(grad_output if grad_output.stride(-1) == 1 else grad_output.contiguous(), indices), None, None


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
