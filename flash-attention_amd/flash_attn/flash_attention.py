"""nn.Module front ends of the fused attention path, interface-compatible with the reference's
flash_attn/flash_attention.py (:12-118)."""
import torch
import torch.nn as nn

from .bert_padding import pad_input, unpad_input
from .flash_attn_interface import flash_attn_unpadded_qkvpacked_func, flash_attn_unpadded_qkvpacked_rotary_func


class FlashAttention(nn.Module):
    """Scaled dot-product softmax attention on packed qkv.

    Arguments
    ---------
        softmax_scale: temperature of the softmax (default: 1/sqrt(head_dim), taken at run time)
        attention_dropout: dropout probability applied to the attention weights while training (default 0.0)
    """

    def __init__(self, softmax_scale=None, attention_dropout=0.0, device=None, dtype=None):
        super().__init__()
        self.softmax_scale = softmax_scale
        self.dropout_p = attention_dropout

    def forward(self, qkv, attn_mask=None, key_padding_mask=None, causal=False, cu_seqlens=None, max_s=None,
                need_weights=False, alibi_slopes=None, attn_bias=None, rotary=None):
        """qkv is (B, S, 3, H, D) when cu_seqlens is None, else already packed (nnz, 3, H, D) with cu_seqlens / max_s.
        key_padding_mask, if given, is an object whose `.bool_matrix` is a (B, S) bool tensor, True = keep.
        alibi_slopes (not in the reference): (H,) fp32 slopes of the in-kernel attention bias -slope * |i - j|.
        attn_bias (not in the reference): (1 or B, 1 or H, S, S) in qkv's dtype, added to the scaled scores; positions are
        counted inside each sequence (so with a key_padding_mask, among the tokens that are kept); differentiable.
        rotary (not in the reference): (cos_half, sin_half) tables of RotaryEmbedding.half_tables: q and k are turned by
        their position inside their sequence within the attention kernels (not with key_padding_mask, alibi_slopes or
        attn_bias).
        Returns (output, None); output has the layout of the input's token dimensions."""
        assert not need_weights
        assert attn_mask is None
        assert qkv.dtype == torch.float16  # the reference's module restriction (:41); the functional API takes bf16 too
        assert qkv.is_cuda
        p = self.dropout_p if self.training else 0.0

        if rotary is not None:
            assert key_padding_mask is None and alibi_slopes is None and attn_bias is None
            if cu_seqlens is not None:
                assert max_s is not None
                return flash_attn_unpadded_qkvpacked_rotary_func(qkv, *rotary, cu_seqlens, max_s, p,
                                                                 softmax_scale=self.softmax_scale, causal=causal), None
            batch, seqlen = qkv.shape[0], qkv.shape[1]
            packed = qkv.reshape(batch * seqlen, *qkv.shape[2:])
            cu = torch.arange(0, (batch + 1) * seqlen, step=seqlen, dtype=torch.int32, device=qkv.device)
            out = flash_attn_unpadded_qkvpacked_rotary_func(packed, *rotary, cu, seqlen, p,
                                                            softmax_scale=self.softmax_scale, causal=causal)
            return out.reshape(batch, seqlen, *out.shape[1:]), None

        if cu_seqlens is not None:
            assert max_s is not None
            out = flash_attn_unpadded_qkvpacked_func(qkv, cu_seqlens, max_s, p, softmax_scale=self.softmax_scale,
                                                     causal=causal, alibi_slopes=alibi_slopes, attn_bias=attn_bias)
            return out, None

        batch, seqlen = qkv.shape[0], qkv.shape[1]
        if key_padding_mask is None:
            packed = qkv.reshape(batch * seqlen, *qkv.shape[2:])
            cu = torch.arange(0, (batch + 1) * seqlen, step=seqlen, dtype=torch.int32, device=qkv.device)
            out = flash_attn_unpadded_qkvpacked_func(packed, cu, seqlen, p, softmax_scale=self.softmax_scale,
                                                     causal=causal, alibi_slopes=alibi_slopes, attn_bias=attn_bias)
            return out.reshape(batch, seqlen, *out.shape[1:]), None

        nheads, headdim = qkv.shape[-2], qkv.shape[-1]
        x = qkv.reshape(batch, seqlen, 3 * nheads * headdim)
        x_unpad, indices, cu, max_len = unpad_input(x, key_padding_mask.bool_matrix)
        out_unpad = flash_attn_unpadded_qkvpacked_func(x_unpad.reshape(-1, 3, nheads, headdim), cu, max_len, p,
                                                       softmax_scale=self.softmax_scale, causal=causal,
                                                       alibi_slopes=alibi_slopes, attn_bias=attn_bias)
        out = pad_input(out_unpad.reshape(-1, nheads * headdim), indices, batch, seqlen)
        return out.reshape(batch, seqlen, nheads, headdim), None


class FlashMHA(nn.Module):
    """Multi-head self-attention block: fused QKV projection, FlashAttention, output projection."""

    def __init__(self, embed_dim, num_heads, bias=True, batch_first=True, attention_dropout=0.0, causal=False,
                 use_rotary_emb=None, device=None, dtype=None, **kwargs) -> None:
        assert batch_first
        factory_kwargs = {"device": device, "dtype": dtype}
        super().__init__()
        self.embed_dim = embed_dim
        self.causal = causal
        self.num_heads = num_heads
        assert self.embed_dim % num_heads == 0, "self.kdim must be divisible by num_heads"
        self.head_dim = self.embed_dim // num_heads
        assert self.head_dim in [16, 32, 64], "Only support head_dim == 16, 32, or 64"
        assert use_rotary_emb in [None, "1d", "2d"]
        self.use_rotary_emb = use_rotary_emb
        if use_rotary_emb is not None:
            from .rotary import RotaryEmbedding, RotaryEmbedding2D
            self.rotary_emb = RotaryEmbedding(self.head_dim) if use_rotary_emb == "1d" else RotaryEmbedding2D(self.head_dim)
        self.Wqkv = nn.Linear(embed_dim, 3 * embed_dim, bias=bias, **factory_kwargs)
        self.inner_attn = FlashAttention(attention_dropout=attention_dropout, **factory_kwargs)
        self.out_proj = nn.Linear(embed_dim, embed_dim, bias=bias, **factory_kwargs)

    def forward(self, x, x_ignored_, x_ignored_1_, attn_mask=None, key_padding_mask=None, need_weights=False):
        b, s = x.shape[0], x.shape[1]
        qkv = self.Wqkv(x).reshape(b, s, 3, self.num_heads, self.head_dim)
        if (self.use_rotary_emb == "1d" and key_padding_mask is None and qkv.is_cuda and qkv.dtype == torch.float16):
            # the rotation happens inside the attention kernels (q as it is loaded, dq and dk as they are stored)
            context, attn_weights = self.inner_attn(qkv, need_weights=need_weights, causal=self.causal,
                                                    rotary=self.rotary_emb.half_tables(qkv))
            return self.out_proj(context.reshape(b, s, self.embed_dim)), attn_weights
        if self.use_rotary_emb and qkv.is_cuda and qkv.dtype in (torch.float16, torch.bfloat16) and (
                self.use_rotary_emb == "1d" or self.head_dim % 16 == 0):
            qkv = self.rotary_emb.rotate_qkv_(qkv)  # q and k rotated in place by the HIP kernel (one pass; "2d": two)
        elif self.use_rotary_emb:  # other devices / dtypes: the reference's elementwise formulation
            query, key, value = qkv.unbind(dim=2)
            query, key = self.rotary_emb(query, key, seq_dimension=-3)
            qkv = torch.stack([query, key, value], dim=2)
        context, attn_weights = self.inner_attn(qkv, key_padding_mask=key_padding_mask, need_weights=need_weights,
                                                causal=self.causal)
        return self.out_proj(context.reshape(b, s, self.embed_dim)), attn_weights
