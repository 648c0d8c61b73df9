"""Block-sparse attention, signature-compatible with the reference's flash_attn/flash_blocksparse_attn_interface.py.

The sparsity layout has one entry per 16-row x 256-key block of the score matrix.  `convert_blockmask` turns a 0/1
layout into the per-column block lists the native entry points take (the reference's own format, :8-40).  The
reference's Python at this commit calls its extension with an argument list its C++ no longer accepts
(:45-47,56-58 vs fmha_api.cpp:451-464,575-594); here the public signature is kept and the native call uses the
C++ argument order.
"""
import torch

from . import flash_attn_gfx950 as _backend
from .flash_attn_interface import bias_grad_in_shape, new_bias_grad


def convert_blockmask(blockmask, causal):
    """0/1 layout (row, col) -> int32 (col, row).  Row c of the result lists the nonzero row-block indices of column
    c in ascending order, padded with -1.  Each index is multiplied by 4; bit 0 marks the first nonzero of its
    layout row, bit 1 the last nonzero of its layout row.

    causal=True (the reference asserts against it, :21; the kernels here apply the element-wise causal mask on top of the
    block list): blocks that lie wholly above the diagonal are dropped from the lists first, so that the first/last
    marks describe the blocks that are actually computed."""
    nz = blockmask != 0
    nrow, ncol = nz.shape
    dev = nz.device
    cols = torch.arange(ncol, device=dev)
    if causal:  # block (r, c) holds a key <= query iff its first key 256 c is <= its last row 16 r + 15
        nz = nz & (256 * cols[None, :] <= 16 * torch.arange(nrow, device=dev)[:, None] + 15)
    big = ncol + 1
    first_col = torch.where(nz, cols, torch.full_like(cols, big)).min(dim=1).values   # (nrow,)
    last_col = torch.where(nz, cols, torch.full_like(cols, -1)).max(dim=1).values
    rows = torch.arange(nrow, device=dev)[:, None]
    code = 4 * rows + (cols[None, :] == first_col[:, None]).long() + 2 * (cols[None, :] == last_col[:, None]).long()
    code = torch.where(nz, code, torch.full_like(code, -1))                           # (nrow, ncol)
    # per column: active rows first (ascending), then the -1 padding
    order = torch.sort((~nz).to(torch.int64) * (nrow + 1) + rows, dim=0).indices      # (nrow, ncol)
    return torch.gather(code, 0, order).T.contiguous().to(torch.int32)


_ROW_ORDERS = {}  # converted blockmask (address, shape, version) -> row order


def _row_order(blockmask, causal):
    """The order of the 16-row blocks the kernels' workgroups take them in (flash_attn_gfx950.blockmask_row_order), worked
    out once per converted blockmask (the first call reads the blockmask back to the host).  Any order gives the same
    results; a cache entry that outlived its tensor costs speed at worst."""
    if causal:
        return None
    key = (blockmask.data_ptr(), tuple(blockmask.shape), blockmask._version, str(blockmask.device))
    order = _ROW_ORDERS.get(key)
    if order is None:
        conv = blockmask.cpu()
        ncol, nrow = conv.shape
        layout = torch.zeros(nrow, ncol, dtype=torch.bool)
        cols = torch.arange(ncol)[:, None].expand(ncol, nrow)
        live = (conv >= 0) & ((conv >> 2) < nrow)
        layout[(conv >> 2)[live].long(), cols[live]] = True
        order = _backend.blockmask_row_order(layout).to(blockmask.device)
        if len(_ROW_ORDERS) >= 64:
            _ROW_ORDERS.clear()
        _ROW_ORDERS[key] = order
    return order


def _flash_blocksparse_attn_forward(qkv, cu_seqlens, blockmask, dropout_p, max_s, softmax_scale, causal,
                                    return_softmax, alibi_slopes=None, attn_bias=None):
    res = _backend.fwd_block(qkv[:, 0], qkv[:, 1], qkv[:, 2], cu_seqlens, cu_seqlens, blockmask, max_s, max_s,
                             dropout_p, softmax_scale, causal, return_softmax, None, row_order=_row_order(blockmask, causal),
                             alibi_slopes=alibi_slopes, attn_bias=attn_bias)
    return res[0], res[1], (res[2] if return_softmax else None)


def _flash_blocksparse_attn_backward(dout, qkv, out, S_dmask, softmax_lse, cu_seqlens, blockmask, dropout_p, max_s,
                                     softmax_scale, causal, alibi_slopes=None, attn_bias=None, dbias=None):
    dqkv = torch.empty_like(qkv)
    _backend.bwd_block(dout.contiguous(), qkv[:, 0], qkv[:, 1], qkv[:, 2], out, softmax_lse, dqkv[:, 0], dqkv[:, 1],
                       dqkv[:, 2], cu_seqlens, cu_seqlens, blockmask, max_s, max_s, dropout_p, softmax_scale, causal,
                       None, row_order=_row_order(blockmask, causal), alibi_slopes=alibi_slopes, attn_bias=attn_bias,
                       dbias=dbias)
    return dqkv


def _fwd_common(ctx, qkv, cu_seqlens, blockmask, dropout_p, max_s, softmax_scale, causal, return_softmax, alibi_slopes,
                attn_bias):
    rng_state = torch.cuda.get_rng_state(qkv.device) if dropout_p > 0 else None
    if softmax_scale is None:
        softmax_scale = qkv.shape[-1] ** (-0.5)
    # the bias in the form the kernels read (the caller's tensor itself if its layout allows, else a padded copy)
    bias_t = None
    if attn_bias is not None:
        bias_t = _backend.prepare_attn_bias(attn_bias.detach(), qkv[:, 0], cu_seqlens.numel() - 1, qkv.shape[2], int(max_s),
                                            int(max_s))
    context, softmax_lse, S_dmask = _flash_blocksparse_attn_forward(
        qkv, cu_seqlens, blockmask, dropout_p, max_s, softmax_scale, causal, return_softmax, alibi_slopes, bias_t)
    ctx.save_for_backward(qkv, context, softmax_lse, cu_seqlens, blockmask, rng_state, bias_t)
    ctx.dropout_p = dropout_p
    ctx.max_s = max_s
    ctx.softmax_scale = softmax_scale
    ctx.causal = causal
    ctx.alibi_slopes = alibi_slopes  # fixed slopes, not differentiated
    ctx.bias_shape = tuple(attn_bias.shape) if attn_bias is not None else None
    ctx.bias_needs_grad = attn_bias is not None and attn_bias.requires_grad
    return context, S_dmask, softmax_lse


def _bwd_common(ctx, dout):
    """(dqkv, gradient of attn_bias or None)"""
    qkv, context, softmax_lse, cu_seqlens, blockmask, rng_state, bias_t = ctx.saved_tensors
    dev = qkv.device
    if rng_state is not None:
        cur_rng_state = torch.cuda.get_rng_state(dev)
        torch.cuda.set_rng_state(rng_state, dev)
    dbias = None
    if ctx.bias_needs_grad:
        dbias = new_bias_grad(qkv[:, 0], cu_seqlens.numel() - 1, ctx.max_s, ctx.max_s)
    dqkv = _flash_blocksparse_attn_backward(dout, qkv, context, None, softmax_lse, cu_seqlens, blockmask,
                                            ctx.dropout_p, ctx.max_s, ctx.softmax_scale, ctx.causal, ctx.alibi_slopes,
                                            bias_t, dbias)
    if rng_state is not None:
        torch.cuda.set_rng_state(cur_rng_state, dev)
    return dqkv, (bias_grad_in_shape(dbias, ctx.bias_shape, ctx.max_s, ctx.max_s) if dbias is not None else None)


class FlashBlocksparseAttnFun(torch.autograd.Function):
    """apply(qkv, cu_seqlens, blockmask_converted, dropout_p, max_s, softmax_scale, causal, alibi_slopes, attn_bias)
    -> context"""

    @staticmethod
    def forward(ctx, qkv, cu_seqlens, blockmask, dropout_p, max_s, softmax_scale, causal, alibi_slopes=None, attn_bias=None):
        return _fwd_common(ctx, qkv, cu_seqlens, blockmask, dropout_p, max_s, softmax_scale, causal, False, alibi_slopes,
                           attn_bias)[0]

    @staticmethod
    def backward(ctx, dout):
        dqkv, dbias = _bwd_common(ctx, dout)
        return dqkv, None, None, None, None, None, None, None, dbias


class FlashBlocksparseAttnFunWithS(torch.autograd.Function):
    """Same, returning (context, S_dmask, softmax_lse) for tests."""

    @staticmethod
    def forward(ctx, qkv, cu_seqlens, blockmask, dropout_p, max_s, softmax_scale, causal, alibi_slopes=None, attn_bias=None):
        context, S_dmask, softmax_lse = _fwd_common(ctx, qkv, cu_seqlens, blockmask, dropout_p, max_s, softmax_scale,
                                                    causal, True, alibi_slopes, attn_bias)
        ctx.mark_non_differentiable(S_dmask, softmax_lse)
        return context, S_dmask, softmax_lse

    @staticmethod
    def backward(ctx, dout, _dS_dmask_ignored, _dsoftmax_sum_ignored):
        dqkv, dbias = _bwd_common(ctx, dout)
        return dqkv, None, None, None, None, None, None, None, dbias


def flash_blocksparse_attn_func(qkv, cu_seqlens, blockmask, dropout_p, max_s, softmax_scale=None,
                                causal=False, return_attn_probs=False, convert_mask=True, alibi_slopes=None, attn_bias=None):
    """Self-attention on packed qkv (total, 3, nheads, headdim) restricted to the active blocks of `blockmask`
    ((seqlen rounded to 16) / 16 rows by (seqlen rounded to 256) / 256 columns of 0/1, or already converted when
    convert_mask=False).  Query rows whose blocks are all inactive produce zeros.  dropout_p must be 0.0 at
    evaluation time.  With return_attn_probs=True returns (context, S_dmask, softmax_lse).
    alibi_slopes, attn_bias (extensions, as in flash_attn_unpadded_qkvpacked_func): a score bias inside the active
    blocks; attn_bias is differentiable."""
    func = FlashBlocksparseAttnFun if not return_attn_probs else FlashBlocksparseAttnFunWithS
    if convert_mask:
        blockmask = convert_blockmask(blockmask, causal=causal)
    return func.apply(qkv, cu_seqlens, blockmask, dropout_p, max_s, softmax_scale, causal, alibi_slopes, attn_bias)
