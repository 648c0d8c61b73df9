"""Rotary position embeddings used by FlashMHA(use_rotary_emb=...), interface-compatible with the reference's
flash_attn/rotary.py (:22-135).  The general functions are PyTorch elementwise ops as in the reference; for the case
the attention modules use, q and k of a packed (batch, seqlen, 3, nheads, headdim) GPU tensor, `apply_rotary_emb_qkv_`
rotates both in place in one pass of a HIP kernel (fa_rotary), with a matching backward.

Convention (rotary.py:22-42,66-87): channel pairs are interleaved, (x[2i], x[2i+1]) is rotated by angle
pos * 10000^(-2i/dim):   x'[2i] = x[2i] cos - x[2i+1] sin,   x'[2i+1] = x[2i+1] cos + x[2i] sin.
The cos/sin tables are rounded to the input dtype before use, as the reference does.
"""
import math
from typing import Tuple

import torch


def rotate_half(x):
    """(x0, x1, x2, x3, ...) -> (-x1, x0, -x3, x2, ...)"""
    pairs = x.reshape(*x.shape[:-1], -1, 2)
    return torch.stack((-pairs[..., 1], pairs[..., 0]), dim=-1).reshape(x.shape)


def apply_rotary_pos_emb(x, cos, sin, seq_dimension: int = -2):
    """x: (..., s, d) if seq_dimension == -2, (..., s, h, d) if -3.  cos, sin: (>= s, d)."""
    n = x.shape[seq_dimension]
    cos, sin = cos[:n], sin[:n]
    if seq_dimension == -3:
        cos, sin = cos[:, None, :], sin[:, None, :]
    return x * cos + rotate_half(x) * sin


class _ApplyRotaryQKV(torch.autograd.Function):
    """In-place rotation of the q and k parts of a packed qkv; the backward rotates the incoming gradient by the
    opposite angle (the transpose of a rotation) and passes the v part through."""

    @staticmethod
    def forward(ctx, qkv, cos_half, sin_half):
        from . import flash_attn_gfx950 as backend
        ctx.save_for_backward(cos_half, sin_half)
        backend.rotary(qkv, qkv, cos_half, sin_half, n_rotated=2)
        ctx.mark_dirty(qkv)
        return qkv

    @staticmethod
    def backward(ctx, grad):
        from . import flash_attn_gfx950 as backend
        cos_half, sin_half = ctx.saved_tensors
        grad = grad.contiguous()
        return backend.rotary(grad, torch.empty_like(grad), cos_half, sin_half, n_rotated=2, conjugate=True), None, None


def apply_rotary_emb_qkv_(qkv, cos_half, sin_half):
    """Rotates q = qkv[:, :, 0] and k = qkv[:, :, 1] of a packed (batch, seqlen, 3, nheads, headdim) fp16 / bf16 GPU
    tensor IN PLACE by the angles whose cosines / sines are cos_half / sin_half ((>= seqlen, headdim / 2), same dtype):
    the same map as apply_rotary_pos_emb(q, ...), apply_rotary_pos_emb(k, ...) with seq_dimension=-3, products formed in
    fp32 and rounded once.  Differentiable."""
    return _ApplyRotaryQKV.apply(qkv, cos_half, sin_half)


class RotaryEmbedding(torch.nn.Module):
    """Rotary embedding of RoFormer (Su et al., arXiv:2104.09864) for queries and keys."""

    def __init__(self, dim_model: int, *_, **__):
        super().__init__()
        exponent = torch.arange(0, dim_model, 2).float() / dim_model
        self.register_buffer("inv_freq", 1.0 / (10000 ** exponent))
        self._seq_len_cached = None
        self._cos_cached = None
        self._sin_cached = None

    def _update_cos_sin_tables(self, x, seq_dimension=-2):
        seq_len = x.shape[seq_dimension]
        stale = (seq_len != self._seq_len_cached or self._cos_cached.device != x.device
                 or self._cos_cached.dtype != x.dtype)
        if stale:
            self._seq_len_cached = seq_len
            pos = torch.arange(seq_len, device=x.device, dtype=self.inv_freq.dtype)
            angles = torch.outer(pos, self.inv_freq.to(x.device))  # fp32 (seq, dim/2)
            self._cos_cached = torch.cos(angles).to(x.dtype).repeat_interleave(2, dim=-1)
            self._sin_cached = torch.sin(angles).to(x.dtype).repeat_interleave(2, dim=-1)
        return self._cos_cached, self._sin_cached

    def half_tables(self, qkv):
        """(cos, sin) of shape (seqlen, headdim / 2) for a (batch, seqlen, 3, nheads, headdim) tensor: one entry per rotated
        pair, the form the HIP kernels read.  Same values as forward()'s tables; kept until those change."""
        cos, sin = self._update_cos_sin_tables(qkv[:, :, 0], seq_dimension=-3)
        if getattr(self, "_half_of", None) is not cos:
            self._half = (cos[:, ::2].contiguous(), sin[:, ::2].contiguous())
            self._half_of = cos
        return self._half

    def rotate_qkv_(self, qkv):
        """q and k of a packed (batch, seqlen, 3, nheads, headdim) GPU tensor rotated in place (one HIP kernel); returns
        qkv.  Same tables as forward()."""
        return apply_rotary_emb_qkv_(qkv, *self.half_tables(qkv))

    def forward(self, q: torch.Tensor, k: torch.Tensor, seq_dimension=-2) -> Tuple[torch.Tensor, torch.Tensor]:
        assert seq_dimension in [-2, -3]  # (bs, h, s, d) or (bs, s, h, d)
        cos, sin = self._update_cos_sin_tables(k, seq_dimension=seq_dimension)
        return (apply_rotary_pos_emb(q, cos, sin, seq_dimension), apply_rotary_pos_emb(k, cos, sin, seq_dimension))


class _ApplyRotaryQKV2D(torch.autograd.Function):
    """In-place 2-D rotation of q and k of a packed qkv: channels [0, d/2) by the token's column, [d/2, d) by its row
    (two passes of the same kernel over the two half-channel views, the position of every token given explicitly).  The
    backward applies the opposite rotations to the incoming gradient."""

    @staticmethod
    def _rotate(t, cos_half, sin_half, col_pos, row_pos, conjugate):
        from . import flash_attn_gfx950 as backend
        half = t.shape[-1] // 2
        lo, hi = t[..., :half], t[..., half:]
        backend.rotary(lo, lo, cos_half, sin_half, n_rotated=2, conjugate=conjugate, positions=col_pos)
        backend.rotary(hi, hi, cos_half, sin_half, n_rotated=2, conjugate=conjugate, positions=row_pos)

    @staticmethod
    def forward(ctx, qkv, cos_half, sin_half, col_pos, row_pos):
        ctx.save_for_backward(cos_half, sin_half, col_pos, row_pos)
        _ApplyRotaryQKV2D._rotate(qkv, cos_half, sin_half, col_pos, row_pos, False)
        ctx.mark_dirty(qkv)
        return qkv

    @staticmethod
    def backward(ctx, grad):
        cos_half, sin_half, col_pos, row_pos = ctx.saved_tensors
        grad = grad.clone(memory_format=torch.contiguous_format)
        _ApplyRotaryQKV2D._rotate(grad, cos_half, sin_half, col_pos, row_pos, True)
        return grad, None, None, None, None


class RotaryEmbedding2D(torch.nn.Module):
    """Rotary embedding for a square grid of tokens (seqlen = side * side): the first half of the channels is
    rotated by the column index, the second half by the row index."""

    def __init__(self, dim: int):
        super().__init__()
        assert dim % 4 == 0
        self.rotary_emb1d = RotaryEmbedding(dim // 2)
        self._pos_cached = None

    def rotate_qkv_(self, qkv):
        """q and k of a packed (batch, side * side, 3, nheads, headdim) fp16 / bf16 GPU tensor rotated in place by the HIP
        kernel (headdim a multiple of 16); returns qkv.  Same map as forward() on q and k, products in fp32, one rounding."""
        b, seqlen = qkv.shape[0], qkv.shape[1]
        side = int(math.sqrt(seqlen))
        assert seqlen == side * side
        grid = qkv[:, :side, 0, :, :qkv.shape[-1] // 2]  # (b, side, nheads, headdim / 2): `side` positions per axis
        cos, sin = self.rotary_emb1d._update_cos_sin_tables(grid, seq_dimension=-3)
        key = (b, side, qkv.device)
        if self._pos_cached is None or self._pos_cached[0] != key:
            tok = torch.arange(seqlen, device=qkv.device, dtype=torch.int32)
            col = (tok % side).repeat(b).contiguous()
            row = torch.div(tok, side, rounding_mode="floor").to(torch.int32).repeat(b).contiguous()
            self._pos_cached = (key, col, row)
        _, col, row = self._pos_cached
        return _ApplyRotaryQKV2D.apply(qkv, cos[:, ::2].contiguous(), sin[:, ::2].contiguous(), col, row)

    def forward(self, q: torch.Tensor, k: torch.Tensor, seq_dimension=-2):
        assert seq_dimension in [-2, -3]
        seqlen = q.shape[seq_dimension]
        side = int(math.sqrt(seqlen))
        assert seqlen == side * side
        if seq_dimension == -3:  # (bs, s, h, d) -> (bs, h, s, d)
            q, k = q.transpose(1, 2), k.transpose(1, 2)
        half = q.shape[-1] // 2

        def grid(t):  # (b, nheads, side*side, c) -> (b, nheads, side, side, c)
            return t.reshape(t.shape[0], t.shape[1], side, side, t.shape[-1])

        # first half: position = column (inner grid axis); second half: position = row (outer grid axis)
        q0, k0 = self.rotary_emb1d(grid(q[..., :half]), grid(k[..., :half]), seq_dimension=-2)
        q1, k1 = self.rotary_emb1d(grid(q[..., half:]), grid(k[..., half:]), seq_dimension=-3)
        q_emb = torch.cat([q0.reshape(*q.shape[:-1], half), q1.reshape(*q.shape[:-1], half)], dim=-1)
        k_emb = torch.cat([k0.reshape(*k.shape[:-1], half), k1.reshape(*k.shape[:-1], half)], dim=-1)
        if seq_dimension == -3:
            q_emb, k_emb = q_emb.transpose(1, 2), k_emb.transpose(1, 2)
        return q_emb, k_emb
