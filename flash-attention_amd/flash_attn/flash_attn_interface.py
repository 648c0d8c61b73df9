"""Functional API of the fused attention path, signature-compatible with the reference's
flash_attn/flash_attn_interface.py (:151-252).  All three packings (qkv packed, kv packed, separate q/k/v) share one
implementation; the packed variants hand strided views of the packed tensor to the kernels and let the backward write
straight into views of one packed gradient buffer, as the reference does (:58-72, :96-111).
"""
import torch

from . import flash_attn_gfx950 as _backend


def _get_block_size(device, head_dim, is_dropout):
    """Width of the key blocks that fix the rounded length of S_dmask (the reference keeps the same helper, :7-14;
    on this device the answer follows fmha_api.cpp:232 for a non-sm80 part)."""
    assert head_dim in [16, 32, 64, 128]
    return 128 if head_dim == 128 else 256


def _flash_attn_forward(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, dropout_p,
                        softmax_scale, causal, return_softmax, alibi_slopes=None, keep_words=None, attn_bias=None,
                        rotary=None, q_rot=None):
    res = _backend.fwd(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, dropout_p, softmax_scale,
                       False, causal, return_softmax, None, alibi_slopes, keep_words, attn_bias, rotary=rotary, q_rot=q_rot)
    return res[0], res[1], (res[2] if return_softmax else None)


def _flash_attn_backward(dout, q, k, v, out, softmax_lse, dq, dk, dv, cu_seqlens_q, cu_seqlens_k,
                         max_seqlen_q, max_seqlen_k, dropout_p, softmax_scale, causal, alibi_slopes=None,
                         keep_words=None, attn_bias=None, dbias=None, rotary=None):
    _, _, _, softmax_d = _backend.bwd(dout, q, k, v, out, softmax_lse, dq, dk, dv, cu_seqlens_q, cu_seqlens_k,
                                      max_seqlen_q, max_seqlen_k, dropout_p, softmax_scale, False, causal, None,
                                      alibi_slopes=alibi_slopes, keep_words=keep_words, attn_bias=attn_bias, dbias=dbias,
                                      rotary=rotary)
    return dq, dk, dv, softmax_d


def _rotated_keys(qkv, cu_seqlens, max_seqlen, cos_half, sin_half):
    """(total, 2, nheads, headdim) buffer whose part 1 holds the rotated keys of a packed qkv (part 0 is left for the
    rotated queries, which the attention kernel writes): one pass of the rotary kernel over the k third only."""
    total, _, nheads, headdim = qkv.shape
    batch = cu_seqlens.numel() - 1
    rot = torch.empty((total, 2, nheads, headdim), dtype=qkv.dtype, device=qkv.device)
    positions = None
    if total != batch * max_seqlen:  # ragged: every row's position inside its sequence
        lens = (cu_seqlens[1:] - cu_seqlens[:-1]).long()
        positions = (torch.arange(total, device=qkv.device, dtype=torch.int32)
                     - torch.repeat_interleave(cu_seqlens[:-1], lens, output_size=total))
        src, dst = qkv[None, :, 1:2], rot[None, :, 1:2]
    else:
        src = qkv.reshape(batch, max_seqlen, 3, nheads, headdim)[:, :, 1:2]
        dst = rot.view(batch, max_seqlen, 2, nheads, headdim)[:, :, 1:2]
    _backend.rotary(src, dst, cos_half, sin_half, n_rotated=1, positions=positions)
    return rot


def _split(packing, tensors):
    """q, k, v views of the user's tensors for a given packing."""
    if packing == "qkv":
        (qkv,) = tensors
        return qkv[:, 0], qkv[:, 1], qkv[:, 2]
    if packing == "kv":
        q, kv = tensors
        return q, kv[:, 0], kv[:, 1]
    return tensors


def _forward(ctx, packing, tensors, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, dropout_p,
             softmax_scale, causal, return_softmax, alibi_slopes=None, attn_bias=None, rotary=None):
    q, k, v = _split(packing, tensors)
    # rotary embedding inside the kernels (packed qkv only): the keys are rotated into a side buffer by the rotary kernel,
    # the queries by the attention kernel as it loads them, which also leaves them in the side buffer for the backward
    rot = q_rot = None
    if rotary is not None:
        rot = _rotated_keys(tensors[0], cu_seqlens_q, int(max_seqlen_q), *rotary)
        q_rot, k = rot[:, 0], rot[:, 1]
    # the dropout mask is a function of the generator state at this point; the backward rewinds to it
    rng_state = torch.cuda.get_rng_state(q.device) if dropout_p > 0 else None
    if softmax_scale is None:
        softmax_scale = q.shape[-1] ** (-0.5)
    # with a backward to come, the forward leaves its dropout decisions (one bit per score) for it to read instead of
    # drawing them twice more; None (no dropout, no gradient wanted, or larger than _backend.KEEP_WORDS_MAX_BYTES or than the
    # inputs themselves) = redraw
    keep_words = None
    if dropout_p > 0 and any(ctx.needs_input_grad):
        keep_words = _backend.new_keep_words(q, cu_seqlens_q, max_seqlen_q, max_seqlen_k, dropout_p, total_k=k.shape[0])
    # the bias in the form the kernels read (the caller's tensor itself if its layout allows, else a padded copy)
    bias_t = None
    if attn_bias is not None:
        bias_t = _backend.prepare_attn_bias(attn_bias.detach(), q, cu_seqlens_q.numel() - 1, q.shape[1], int(max_seqlen_q),
                                            int(max_seqlen_k))
    out, softmax_lse, S_dmask = _flash_attn_forward(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
                                                    dropout_p, softmax_scale, causal, return_softmax, alibi_slopes,
                                                    keep_words, bias_t, rotary, q_rot)
    ctx.save_for_backward(*tensors, out, softmax_lse, cu_seqlens_q, cu_seqlens_k, rng_state, bias_t, rot)
    ctx.rotary = rotary  # constant tables, not differentiated
    ctx.bias_shape = tuple(attn_bias.shape) if attn_bias is not None else None
    ctx.bias_needs_grad = attn_bias is not None and attn_bias.requires_grad
    ctx.keep_words = keep_words
    ctx.alibi_slopes = alibi_slopes  # fixed slopes, not differentiated
    ctx.packing = packing
    ctx.n_in = len(tensors)
    ctx.dropout_p = dropout_p
    ctx.max_seqlen_q, ctx.max_seqlen_k = max_seqlen_q, max_seqlen_k
    ctx.softmax_scale = softmax_scale
    ctx.causal = causal
    return out if not return_softmax else (out, softmax_lse, S_dmask)


def _backward(ctx, dout):
    saved = ctx.saved_tensors
    tensors = saved[:ctx.n_in]
    out, softmax_lse, cu_seqlens_q, cu_seqlens_k, rng_state, bias_t, rot = saved[ctx.n_in:]
    q, k, v = _split(ctx.packing, tensors)
    if rot is not None:  # the kernels take the rotated q and k and turn dq and dk back themselves
        q, k = rot[:, 0], rot[:, 1]
    grads = tuple(torch.empty_like(t) for t in tensors)
    dq, dk, dv = _split(ctx.packing, grads)
    dev = q.device
    dbias = new_bias_grad(q, cu_seqlens_q.numel() - 1, ctx.max_seqlen_q, ctx.max_seqlen_k) if ctx.bias_needs_grad else None
    if rng_state is not None:
        cur_rng_state = torch.cuda.get_rng_state(dev)
        torch.cuda.set_rng_state(rng_state, dev)
    _flash_attn_backward(dout.contiguous(), q, k, v, out, softmax_lse, dq, dk, dv, cu_seqlens_q, cu_seqlens_k,
                         ctx.max_seqlen_q, ctx.max_seqlen_k, ctx.dropout_p, ctx.softmax_scale, ctx.causal,
                         ctx.alibi_slopes, ctx.keep_words, bias_t, dbias, ctx.rotary)
    if rng_state is not None:
        torch.cuda.set_rng_state(cur_rng_state, dev)
    ctx.dbias = bias_grad_in_shape(dbias, ctx.bias_shape, ctx.max_seqlen_q, ctx.max_seqlen_k) if dbias is not None else None
    return grads


def new_bias_grad(q, batch, max_seqlen_q, max_seqlen_k):
    """The tensor the backward kernels leave the bias gradient in: per (batch, head), rows padded to 8 keys, cleared (only
    the tiles the kernels visit are written)."""
    return torch.zeros((batch, q.shape[1], max_seqlen_q, (max_seqlen_k + 7) // 8 * 8), dtype=q.dtype, device=q.device)


def bias_grad_in_shape(dbias, shape, max_seqlen_q, max_seqlen_k):
    """The gradient of an attn_bias of `shape` from the per-(batch, head) tensor of new_bias_grad(): summed over the batch
    entries / heads that shared the bias (one pass, fp32 sums, one rounding); rows / keys beyond max_seqlen get none."""
    full = torch.zeros(shape, dtype=dbias.dtype, device=dbias.device)
    view = full[:, :, :max_seqlen_q, :max_seqlen_k]
    sum_batch, sum_heads = shape[0] == 1 and dbias.shape[0] > 1, shape[1] == 1 and dbias.shape[1] > 1
    if sum_batch or sum_heads:
        _backend.reduce_bias_grad(dbias, view, sum_batch, sum_heads)
    else:
        view.copy_(dbias[:, :, :, :max_seqlen_k])
    return full


def _extra_grads(ctx, grads):
    """grads of the tensors, then None for every other argument - but the bias gradient for attn_bias, the last one."""
    extra = [None] * ctx.n_extra
    if ctx.dbias is not None:
        extra[-1] = ctx.dbias
    return grads + tuple(extra)


class FlashAttnQKVPackedFunc(torch.autograd.Function):
    """apply(qkv, cu_seqlens, max_seqlen, dropout_p, softmax_scale, causal, return_softmax[, alibi_slopes[, attn_bias]])"""

    @staticmethod
    def forward(ctx, qkv, cu_seqlens, max_seqlen, dropout_p, softmax_scale, causal, return_softmax, *bias):
        ctx.n_extra = 6 + len(bias)  # the reference's six non-tensor arguments (:72), plus the optional alibi_slopes, attn_bias
        return _forward(ctx, "qkv", (qkv,), cu_seqlens, cu_seqlens, max_seqlen, max_seqlen, dropout_p, softmax_scale,
                        causal, return_softmax, *bias)

    @staticmethod
    def backward(ctx, dout, *args):
        return _extra_grads(ctx, _backward(ctx, dout))


class FlashAttnRotaryQKVPackedFunc(torch.autograd.Function):
    """apply(qkv, cos_half, sin_half, cu_seqlens, max_seqlen, dropout_p, softmax_scale, causal): self-attention on a
    packed qkv whose q and k get the rotary embedding inside the kernels (no counterpart in the reference, whose FlashMHA
    rotates them with elementwise ops first, flash_attention.py:109-113).  qkv itself is left as it is."""

    @staticmethod
    def forward(ctx, qkv, cos_half, sin_half, cu_seqlens, max_seqlen, dropout_p, softmax_scale, causal):
        ctx.n_extra = 7
        return _forward(ctx, "qkv", (qkv,), cu_seqlens, cu_seqlens, max_seqlen, max_seqlen, dropout_p, softmax_scale,
                        causal, False, rotary=(cos_half, sin_half))

    @staticmethod
    def backward(ctx, dout, *args):
        return _extra_grads(ctx, _backward(ctx, dout))


class FlashAttnKVPackedFunc(torch.autograd.Function):
    """apply(q, kv, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, dropout_p, softmax_scale, causal,
    return_softmax)"""

    @staticmethod
    def forward(ctx, q, kv, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, dropout_p, softmax_scale, causal,
                return_softmax, *bias):
        ctx.n_extra = 8 + len(bias)  # :111
        return _forward(ctx, "kv", (q, kv), cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, dropout_p,
                        softmax_scale, causal, return_softmax, *bias)

    @staticmethod
    def backward(ctx, dout, *args):
        return _extra_grads(ctx, _backward(ctx, dout))


class FlashAttnFunc(torch.autograd.Function):
    """apply(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, dropout_p, softmax_scale, causal,
    return_softmax)"""

    @staticmethod
    def forward(ctx, q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, dropout_p, softmax_scale, causal,
                return_softmax, *bias):
        ctx.n_extra = 8 + len(bias)  # :148
        return _forward(ctx, "sep", (q, k, v), cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, dropout_p,
                        softmax_scale, causal, return_softmax, *bias)

    @staticmethod
    def backward(ctx, dout, *args):
        return _extra_grads(ctx, _backward(ctx, dout))


_COMMON_DOC = """
    dropout_p must be 0.0 at evaluation time.

    Common arguments
        cu_seqlens*: (batch_size + 1,) int32, cumulative sequence lengths; sequence b occupies rows
            cu_seqlens[b]:cu_seqlens[b+1] of the packed token dimension.
        max_seqlen*: int, an upper bound on the longest sequence in the batch.
        dropout_p: float, probability of dropping an attention weight.
        softmax_scale: float, multiplies Q K^T before the softmax; defaults to headdim ** -0.5.
        causal: bool, query i of a sequence attends only to keys j <= i of that sequence.
        return_attn_probs: bool, testing aid.
        alibi_slopes: None, or (nheads,) fp32 on the GPU.  Not in the reference (its README lists attention bias as
            planned): the score of query i and key j, positions counted inside their sequences, becomes
            softmax_scale * q_i.k_j - alibi_slopes[head] * |i - j|.  The slopes are constants (no gradient).
        attn_bias: None, or (1 or batch_size, 1 or nheads, max_seqlen_q, max_seqlen_k) in the inputs' dtype (not in the
            reference either): the score becomes softmax_scale * q_i.k_j + attn_bias[b, head, i, j]; -inf entries mask.
            Differentiable (a shared bias gets the sum over the batch entries / heads that share it).  Not together
            with alibi_slopes.
    Returns
        out: (total_q, nheads, headdim).
        With return_attn_probs=True additionally
        softmax_lse: (batch_size, nheads, seqlen_q rounded up to 16), fp32 log-sum-exp of each scaled score row.
        S_dmask: (batch_size, nheads, seqlen_q rounded, seqlen_k rounded), softmax probabilities in the input dtype
            with the dropout pattern in the sign bit: sign set = dropped, clear = kept.
"""


def flash_attn_unpadded_qkvpacked_func(qkv, cu_seqlens, max_seqlen, dropout_p, softmax_scale=None,
                                       causal=False, return_attn_probs=False, alibi_slopes=None, attn_bias=None):
    """Self-attention on a packed (total, 3, nheads, headdim) tensor of variable-length sequences."""
    return FlashAttnQKVPackedFunc.apply(qkv, cu_seqlens, max_seqlen, dropout_p, softmax_scale, causal,
                                        return_attn_probs, alibi_slopes, attn_bias)


def flash_attn_unpadded_qkvpacked_rotary_func(qkv, cos_half, sin_half, cu_seqlens, max_seqlen, dropout_p,
                                              softmax_scale=None, causal=False):
    """flash_attn_unpadded_qkvpacked_func on a qkv whose q and k are first turned by the rotary position embedding
    (not in the reference's functional API; its FlashMHA does apply_rotary_pos_emb to q and k and then calls the function
    above).  cos_half, sin_half: (>= max_seqlen, headdim / 2) tables in qkv's dtype, one entry per rotated pair
    (RotaryEmbedding.half_tables); the token at position i of its sequence is turned by row i.  Same result as
    apply_rotary_emb_qkv_ followed by flash_attn_unpadded_qkvpacked_func, bit for bit in the forward; the gradient is
    rounded once instead of twice.  The rotation of q and of the gradients happens inside the attention kernels; only k
    takes a pass of its own.  Differentiable with respect to qkv."""
    return FlashAttnRotaryQKVPackedFunc.apply(qkv, cos_half, sin_half, cu_seqlens, max_seqlen, dropout_p, softmax_scale,
                                              causal)


def flash_attn_unpadded_kvpacked_func(q, kv, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
                                      dropout_p, softmax_scale=None, causal=False,
                                      return_attn_probs=False, alibi_slopes=None, attn_bias=None):
    """Attention of q (total_q, nheads, headdim) over packed keys/values kv (total_k, 2, nheads, headdim)."""
    return FlashAttnKVPackedFunc.apply(q, kv, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, dropout_p,
                                       softmax_scale, causal, return_attn_probs, alibi_slopes, attn_bias)


def flash_attn_unpadded_func(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
                             dropout_p, softmax_scale=None, causal=False, return_attn_probs=False, alibi_slopes=None,
                             attn_bias=None):
    """Attention of q (total_q, nheads, headdim) over k, v (total_k, nheads, headdim)."""
    return FlashAttnFunc.apply(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, dropout_p,
                               softmax_scale, causal, return_attn_probs, alibi_slopes, attn_bias)


def flash_attn_func(qkv, cu_seqlens, dropout_p, max_s, softmax_scale=None, causal=False,
                    return_attn_probs=False):
    """Older argument order of flash_attn_unpadded_qkvpacked_func, kept for callers that still use it."""
    return flash_attn_unpadded_qkvpacked_func(qkv, cu_seqlens, max_s, dropout_p, softmax_scale, causal,
                                              return_attn_probs)


for _f in (flash_attn_unpadded_qkvpacked_func, flash_attn_unpadded_kvpacked_func, flash_attn_unpadded_func):
    _f.__doc__ += _COMMON_DOC
