"""nn.Module front ends of block-sparse attention, interface-compatible with the reference's
flash_attn/flash_blocksparse_attention.py (:14-136).

The reference builds its sparsity pattern with `hydra.utils.instantiate(sparsity_config)` and calls
`make_layout(max_seq_length)` on the result (:27-33).  Here `sparsity_config` may be any of
  * a 0/1 layout tensor of shape (max_seq_length / 16, max_seq_length / 256) (16-row by 256-column blocks),
  * an object with a `make_layout(seqlen)` method returning such a tensor,
  * a hydra-style mapping with a `_target_` key (instantiated through hydra, which must then be installed),
so the modules work without hydra.
"""
import torch
import torch.nn as nn

from .bert_padding import pad_input, unpad_input
from .flash_blocksparse_attn_interface import convert_blockmask, flash_blocksparse_attn_func


def _round256(n):
    return ((n + 255) // 256) * 256


def _layout_from_config(sparsity_config, max_seq_length):
    if torch.is_tensor(sparsity_config):
        layout = sparsity_config
    else:
        if not hasattr(sparsity_config, "make_layout"):
            if hasattr(sparsity_config, "keys") and "_target_" in sparsity_config.keys():
                try:
                    import hydra
                except ImportError as e:
                    raise RuntimeError("sparsity_config is a hydra mapping but hydra is not installed; pass a layout "
                                       "tensor or an object with make_layout(seqlen) instead") from e
                sparsity_config = hydra.utils.instantiate(sparsity_config)
            else:
                raise TypeError("sparsity_config must be a layout tensor, an object with make_layout(seqlen), or a "
                                "hydra mapping with a _target_")
        layout = sparsity_config.make_layout(max_seq_length)
    if layout.ndim != 2 or layout.shape[0] < max_seq_length // 16 or layout.shape[1] < max_seq_length // 256:
        raise ValueError("layout must cover (%d, %d) blocks of 16 x 256, got %s"
                         % (max_seq_length // 16, max_seq_length // 256, tuple(layout.shape)))
    return layout


class FlashBlocksparseAttention(nn.Module):
    """Scaled dot-product softmax attention restricted to the active 16 x 256 blocks of a fixed layout.

    Arguments
    ---------
        sparsity_config: see the module docstring
        softmax_temp: temperature of the softmax (default: 1/sqrt(head_dim), taken at run time)
        attention_dropout: dropout probability applied while training (default 0.0)
        max_seq_length: longest sequence the layout must cover (rounded up to a multiple of 256)
    """

    def __init__(self, sparsity_config, softmax_temp=None, attention_dropout=0.0, max_seq_length=2048, device=None,
                 dtype=None):
        super().__init__()
        self.softmax_temp = softmax_temp
        self.dropout_p = attention_dropout
        max_seq_length = _round256(max_seq_length)
        layout = _layout_from_config(sparsity_config, max_seq_length)
        if device is not None:
            layout = layout.to(device)
        # the layout and its converted form for the full length live with the module (:31-36)
        self.register_buffer("layout", layout)
        self.register_buffer("blockmask_converted", convert_blockmask(self.layout, causal=False))

    def _blockmask(self, seqlen):
        """The corner of the layout that a call with max_seqlen = seqlen reads: ceil(seqlen / 16) row blocks by
        ceil(seqlen / 256) column blocks (the shape the native entry point checks, fmha_api.cpp:509-515)."""
        nrow, ncol = (seqlen + 15) // 16, _round256(seqlen) // 256
        assert nrow <= self.layout.shape[0] and ncol <= self.layout.shape[1], \
            "sequence length %d exceeds the module's max_seq_length" % seqlen
        return self.layout[:nrow, :ncol]

    def forward(self, qkv, attn_mask=None, key_padding_mask=None, causal=False, cu_seqlens=None, max_s=None,
                need_weights=False, convert_mask=True):
        """qkv is (B, S, 3, H, D) when cu_seqlens is None, else packed (nnz, 3, H, D) with cu_seqlens / max_s.
        key_padding_mask, if given, is a (B, S) bool tensor or an object whose `.bool_matrix` is one, True = keep.
        With convert_mask=False (packed input only) the converted full-length mask stored in the module is used as is.
        Returns (output, None)."""
        assert not need_weights
        assert attn_mask is None
        assert qkv.dtype == torch.float16  # the reference's restriction (:54)
        assert qkv.is_cuda
        p = self.dropout_p if self.training else 0.0

        if cu_seqlens is not None:
            assert max_s is not None
            if convert_mask:
                out = flash_blocksparse_attn_func(qkv, cu_seqlens, self._blockmask(max_s), p, max_s,
                                                  softmax_scale=self.softmax_temp, causal=causal)
            else:
                out = flash_blocksparse_attn_func(qkv, cu_seqlens, self.blockmask_converted, p, max_s,
                                                  softmax_scale=self.softmax_temp, causal=causal, convert_mask=False)
            return out, None

        batch, seqlen = qkv.shape[0], qkv.shape[1]
        blockmask = self._blockmask(seqlen)
        if key_padding_mask is None:
            packed = qkv.reshape(batch * seqlen, *qkv.shape[2:])
            cu = torch.arange(0, (batch + 1) * seqlen, step=seqlen, dtype=torch.int32, device=qkv.device)
            out = flash_blocksparse_attn_func(packed, cu, blockmask, p, seqlen, softmax_scale=self.softmax_temp,
                                              causal=causal)
            return out.reshape(batch, seqlen, *out.shape[1:]), None

        keep = key_padding_mask.bool_matrix if hasattr(key_padding_mask, "bool_matrix") else key_padding_mask
        nheads, headdim = qkv.shape[-2], qkv.shape[-1]
        x = qkv.reshape(batch, seqlen, 3 * nheads * headdim)
        x_unpad, indices, cu, max_len = unpad_input(x, keep)
        # the layout is cut for the longest sequence of the batch: the corner of what the reference cuts for the padded
        # length (:60-63); block (i, j) keeps meaning rows 16i.. of a sequence against its keys 256j..
        out_unpad = flash_blocksparse_attn_func(x_unpad.reshape(-1, 3, nheads, headdim), cu, self._blockmask(max_len), p,
                                                max_len, softmax_scale=self.softmax_temp, causal=causal)
        out = pad_input(out_unpad.reshape(-1, nheads * headdim), indices, batch, seqlen)
        return out.reshape(batch, seqlen, nheads, headdim), None


class FlashBlocksparseMHA(nn.Module):
    """Multi-head self-attention block: fused QKV projection, block-sparse attention, output projection (:104-136)."""

    def __init__(self, embed_dim, num_heads, sparsity_config, bias=True, batch_first=True, attention_dropout=0.0,
                 causal=False, max_seq_length=2048, device=None, dtype=None, **kwargs):
        assert batch_first
        factory_kwargs = {"device": device, "dtype": dtype}
        super().__init__()
        self.embed_dim = embed_dim
        self.causal = causal
        self.num_heads = num_heads
        assert embed_dim % num_heads == 0, "embed_dim must be divisible by num_heads"
        self.head_dim = embed_dim // num_heads
        assert self.head_dim in (16, 32, 64, 128), "head_dim must be 16, 32, 64 or 128"
        self.Wqkv = nn.Linear(embed_dim, 3 * embed_dim, bias=bias, **factory_kwargs)
        self.inner_attn = FlashBlocksparseAttention(sparsity_config, attention_dropout=attention_dropout,
                                                    max_seq_length=max_seq_length, **factory_kwargs)
        self.out_proj = nn.Linear(embed_dim, embed_dim, bias=bias, **factory_kwargs)

    def forward(self, x, x_ignored_, x_ignored_1_, attn_mask=None, key_padding_mask=None, need_weights=False):
        qkv = self.Wqkv(x)
        qkv = qkv.reshape(x.shape[0], x.shape[1], 3, self.num_heads, self.head_dim)
        context, attn_weights = self.inner_attn(qkv, key_padding_mask=key_padding_mask, need_weights=need_weights,
                                                causal=self.causal)
        return self.out_proj(context.reshape(x.shape[0], x.shape[1], self.embed_dim)), attn_weights
