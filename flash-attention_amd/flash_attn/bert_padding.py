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


def _rows(t):
    """the kernels move rows whose elements are contiguous"""
    return t if t.stride(-1) == 1 else t.contiguous()


class _MoveRows(torch.autograd.Function):
    """One differentiable row move in either direction: gather=True picks rows `indices` of a 2-D tensor, gather=False
    places the rows of a 2-D tensor at `indices` of a zero tensor with n_rows rows.  Each is the other's backward."""

    @staticmethod
    def forward(ctx, src, indices, n_rows, gather):
        assert src.ndim == 2 and indices.ndim == 1
        ctx.save_for_backward(indices)
        ctx.gather = gather
        ctx.n_src = src.shape[0]
        return _gather(_rows(src), indices) if gather else _scatter(_rows(src), indices, n_rows)

    @staticmethod
    def backward(ctx, grad):
        (indices,) = ctx.saved_tensors
        g = _scatter(_rows(grad), indices, ctx.n_src) if ctx.gather else _gather(_rows(grad), indices)
        return g, None, None, None


def index_first_axis(input, indices):
    """input[indices] for a 2-D input (what the reference's IndexFirstAxis.apply computes, :9-33)."""
    return _MoveRows.apply(input, indices, indices.shape[0], True)


def index_put_first_axis(values, indices, first_axis_dim):
    """zeros(first_axis_dim, dim) with values written at rows `indices` (the reference's IndexPutFirstAxis.apply, :36-57)."""
    return _MoveRows.apply(values, indices, first_axis_dim, False)


class IndexFirstAxis:
    """kept for callers that spell it IndexFirstAxis.apply(input, indices)"""
    apply = staticmethod(index_first_axis)


class IndexPutFirstAxis:
    """kept for callers that spell it IndexPutFirstAxis.apply(values, indices, first_axis_dim)"""
    apply = staticmethod(index_put_first_axis)


def unpad_input(hidden_states, attention_mask):
    """Drop the padding: hidden_states (batch, seqlen, dim) and a (batch, seqlen) mask whose nonzero entries mark real
    tokens give
        the real tokens as (total, dim) rows, batch-major,
        their positions in the flattened batch * seqlen axis (int64, what pad_input takes back),
        cu_seqlens (batch + 1,) int32, the running sum of the sequence lengths starting at 0,
        the longest sequence length as a Python int."""
    lengths = attention_mask.sum(dim=-1, dtype=torch.int32)
    positions = torch.nonzero(attention_mask.flatten(), as_tuple=False).flatten()
    cu_seqlens = F.pad(torch.cumsum(lengths, dim=0, dtype=torch.int32), (1, 0))
    tokens = hidden_states.reshape(hidden_states.shape[0] * hidden_states.shape[1], -1)
    return index_first_axis(tokens, positions), positions, cu_seqlens, int(lengths.max().item())


def pad_input(hidden_states, indices, batch, seqlen):
    """Inverse of unpad_input: rows (total, dim) go back to their positions `indices` of a (batch, seqlen, dim) tensor
    that is zero everywhere else."""
    padded = index_put_first_axis(hidden_states, indices, batch * seqlen)
    return padded.reshape(batch, seqlen, hidden_states.shape[-1])
