"""CPU-side tests: the C-ABI library loads and exports what include/flash_attn_gfx950.h declares, argument
validation returns errors instead of aborting, the seqlen rounding follows fmha_api.cpp, and the pure-host helpers
(bert_padding, convert_blockmask, rotary) match their specifications.  Nothing here launches a kernel."""
import ctypes
import inspect
import os
import re

import numpy as np
import pytest
import torch

from oracle import attention_oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol(lib):
    header = open(os.path.join(ROOT, "include", "flash_attn_gfx950.h")).read()
    declared = set(re.findall(r"^\s*(?:int|size_t|void|uint64_t|const char\*)\s+(fa_\w+)\s*\(", header, re.M))
    from flash_attn import flash_attn_gfx950 as be
    assert declared == set(be.EXPORTED_SYMBOLS)
    # the instrumentation entry point of bench.py has a header of its own and is not part of the drop-in boundary
    bench = open(os.path.join(ROOT, "include", "flash_attn_gfx950_bench.h")).read()
    declared_bench = set(re.findall(r"^\s*(?:int|size_t|void)\s+(fa_\w+)\s*\(", bench, re.M))
    assert declared_bench == set(be.BENCH_SYMBOLS) and not (declared & declared_bench)
    for name in declared | declared_bench:
        assert hasattr(lib, name), name
    assert lib.fa_abi_version() == be.FA_ABI_VERSION == 5


def test_struct_layout_matches_library(lib):
    """a wrong struct size is reported as an ABI mismatch; the right size passes that check"""
    from flash_attn import flash_attn_gfx950 as be
    a = be.FwdArgs()
    a.struct_bytes = ctypes.sizeof(a) - 8
    assert lib.fa_fwd(ctypes.byref(a)) == -1 and b"ABI mismatch" in lib.fa_last_error()
    a.struct_bytes = ctypes.sizeof(a)
    a.dtype = 7
    assert lib.fa_fwd(ctypes.byref(a)) == -1 and b"dtype" in lib.fa_last_error()
    g = be.BwdArgs()
    g.struct_bytes = ctypes.sizeof(g)
    g.dtype = 7
    assert lib.fa_bwd(ctypes.byref(g)) == -1 and b"dtype" in lib.fa_last_error()


def _valid_fwd_args(be):
    a = be.FwdArgs()
    a.struct_bytes = ctypes.sizeof(a)
    a.dtype = be.FA_FP16
    a.batch, a.nheads, a.head_dim = 1, 1, 64
    a.total_q = a.total_k = 16
    a.max_seqlen_q = a.max_seqlen_k = 16
    a.p_dropout, a.softmax_scale = 0.0, 0.125
    for f in ("q_row_stride", "k_row_stride", "v_row_stride", "o_row_stride"):
        setattr(a, f, 64)
    for f in ("q_head_stride", "k_head_stride", "v_head_stride", "o_head_stride"):
        setattr(a, f, 64)
    return a


@pytest.mark.parametrize("field,value,needle", [
    ("batch", 0, b"batch_size"),                 # fmha_api.cpp:223
    ("head_dim", 48, b"head_size"),              # :224
    ("p_dropout", 1.0, b"p_dropout"),            # :113
    ("p_dropout", -0.1, b"p_dropout"),
    ("softmax_scale", 0.0, b"softmax_scale"),
    ("max_seqlen_q", 0, b"max_seqlen"),
])
def test_forward_argument_checks(lib, field, value, needle):
    from flash_attn import flash_attn_gfx950 as be
    a = _valid_fwd_args(be)
    setattr(a, field, value)
    rc = lib.fa_fwd(ctypes.byref(a))
    assert rc == -1 and needle in lib.fa_last_error(), lib.fa_last_error()


def test_null_pointers_and_alignment_are_errors_not_crashes(lib):
    from flash_attn import flash_attn_gfx950 as be
    a = _valid_fwd_args(be)
    assert lib.fa_fwd(ctypes.byref(a)) == -1 and b"NULL" in lib.fa_last_error()
    for f in ("q", "k", "v", "o", "softmax_lse", "cu_seqlens_q", "cu_seqlens_k"):
        setattr(a, f, 0x1000)
    a.q = 0x1008
    assert lib.fa_fwd(ctypes.byref(a)) == -1 and b"aligned" in lib.fa_last_error()
    a.q = 0x1000
    a.k_row_stride = 70
    assert lib.fa_fwd(ctypes.byref(a)) == -1 and b"strides" in lib.fa_last_error()
    a.k_row_stride = 64
    a.blockmask = 0x1000  # dense entry point refuses a blockmask, block entry point refuses its absence
    assert lib.fa_fwd(ctypes.byref(a)) == -1 and b"blockmask" in lib.fa_last_error()
    a.blockmask = None
    assert lib.fa_fwd_block(ctypes.byref(a)) == -1 and b"blockmask" in lib.fa_last_error()
    assert lib.fa_fwd(None) == -1


def test_block_sparse_needs_workspace_also_when_causal(lib):
    from flash_attn import flash_attn_gfx950 as be
    a = _valid_fwd_args(be)
    for f in ("q", "k", "v", "o", "softmax_lse", "cu_seqlens_q", "cu_seqlens_k", "blockmask"):
        setattr(a, f, 0x1000)
    assert lib.fa_fwd_workspace_bytes(ctypes.byref(a)) > 0
    assert lib.fa_fwd_block(ctypes.byref(a)) == -2 and b"workspace" in lib.fa_last_error()
    a.is_causal = 1  # accepted together with a blockmask: the same workspace rule applies
    assert lib.fa_fwd_workspace_bytes(ctypes.byref(a)) > 0
    assert lib.fa_fwd_block(ctypes.byref(a)) == -2 and b"workspace" in lib.fa_last_error()


def test_workspace_sizes(lib):
    from flash_attn import flash_attn_gfx950 as be
    a = _valid_fwd_args(be)
    assert lib.fa_fwd_workspace_bytes(ctypes.byref(a)) == 0  # the dense forward needs no scratch (no o_tmp)
    g = be.BwdArgs()
    g.struct_bytes = ctypes.sizeof(g)
    g.batch, g.nheads, g.head_dim, g.total_q, g.total_k = 2, 3, 64, 100, 100
    g.max_seqlen_q = g.max_seqlen_k = 64
    assert lib.fa_bwd_workspace_bytes(ctypes.byref(g)) == 0  # nor the dense backward (no fp32 dq_tmp)
    g.blockmask = 0x1000
    assert lib.fa_bwd_workspace_bytes(ctypes.byref(g)) > 0   # block-sparse: room for the block activity maps
    # dropout keep words: one bit per (batch, head, query, key), both lengths rounded up to 128
    assert lib.fa_keep_words_bytes(8, 12, 512, 512) == 8 * 12 * 512 * 512 // 8
    assert lib.fa_keep_words_bytes(1, 1, 100, 300) == 128 * 384 // 8
    assert lib.fa_keep_words_bytes(2, 3, 129, 1) == 2 * 3 * 256 * 128 // 8
    assert lib.fa_keep_words_bytes(0, 3, 129, 1) == 0 and lib.fa_keep_words_bytes(2, 3, 0, 1) == 0


@pytest.mark.parametrize("d,sq,sk,sparse,want", [
    (64, 1, 1, False, (16, 128)),          # fmha_api.cpp:235-236
    (64, 128, 129, False, (128, 256)),     # :237-238
    (64, 500, 500, False, (512, 512)),     # :234 with blocksize_c = 256
    (64, 513, 513, False, (528, 768)),
    (128, 300, 300, False, (304, 384)),    # blocksize_c = 128 for head_size 128 off sm80 (:232)
    (32, 100, 100, True, (112, 256)),      # :509-513
    (64, 4096, 4096, True, (4096, 4096)),
    (64, 4097, 4097, True, (4112, 4352)),
])
def test_round_seqlens(lib, d, sq, sk, sparse, want):
    from flash_attn import flash_attn_gfx950 as be
    assert be.round_seqlens(d, sq, sk, sparse) == want


def test_python_checks_raise_runtime_error():
    """the binding's own checks mirror TORCH_CHECK -> RuntimeError before anything touches a GPU"""
    from flash_attn import flash_attn_gfx950 as be
    q = torch.zeros(16, 1, 64, dtype=torch.float32)
    cu = torch.tensor([0, 16], dtype=torch.int32)
    with pytest.raises(RuntimeError, match="fp16 or bf16"):
        be.fwd(q, q, q, cu, cu, 16, 16, 0.0, 0.125, False, False, False, None)
    h = q.half()
    with pytest.raises(RuntimeError, match="GPU"):
        be.fwd(h, h, h, cu, cu, 16, 16, 0.0, 0.125, False, False, False, None)
    with pytest.raises(RuntimeError, match="head_size"):
        be.fwd(h[..., :48], h[..., :48], h[..., :48], cu, cu, 16, 16, 0.0, 0.125, False, False, False, None)


def test_public_signatures_match_the_reference():
    """names, order and defaults of flash_attn_interface.py:151-252 and flash_blocksparse_attn_interface.py:135-137"""
    from flash_attn import flash_attn_interface as fi
    from flash_attn import flash_blocksparse_attn_interface as bi
    from flash_attn import bert_padding as bp

    def sig(f):
        return [(n, p.default if p.default is not inspect.Parameter.empty else "<req>")
                for n, p in inspect.signature(f).parameters.items()]

    # the functions that reach the kernels take the reference's parameters followed by two extensions,
    # alibi_slopes=None and attn_bias=None (attention bias: planned in the reference's README, absent from its API)
    ext = [("alibi_slopes", None), ("attn_bias", None)]
    assert sig(fi.flash_attn_unpadded_qkvpacked_func) == [
        ("qkv", "<req>"), ("cu_seqlens", "<req>"), ("max_seqlen", "<req>"), ("dropout_p", "<req>"),
        ("softmax_scale", None), ("causal", False), ("return_attn_probs", False)] + ext
    assert sig(fi.flash_attn_unpadded_kvpacked_func) == [
        ("q", "<req>"), ("kv", "<req>"), ("cu_seqlens_q", "<req>"), ("cu_seqlens_k", "<req>"),
        ("max_seqlen_q", "<req>"), ("max_seqlen_k", "<req>"), ("dropout_p", "<req>"), ("softmax_scale", None),
        ("causal", False), ("return_attn_probs", False)] + ext
    assert sig(fi.flash_attn_unpadded_func) == [
        ("q", "<req>"), ("k", "<req>"), ("v", "<req>"), ("cu_seqlens_q", "<req>"), ("cu_seqlens_k", "<req>"),
        ("max_seqlen_q", "<req>"), ("max_seqlen_k", "<req>"), ("dropout_p", "<req>"), ("softmax_scale", None),
        ("causal", False), ("return_attn_probs", False)] + ext
    assert sig(fi.flash_attn_func) == [
        ("qkv", "<req>"), ("cu_seqlens", "<req>"), ("dropout_p", "<req>"), ("max_s", "<req>"),
        ("softmax_scale", None), ("causal", False), ("return_attn_probs", False)]
    assert sig(bi.flash_blocksparse_attn_func) == [
        ("qkv", "<req>"), ("cu_seqlens", "<req>"), ("blockmask", "<req>"), ("dropout_p", "<req>"), ("max_s", "<req>"),
        ("softmax_scale", None), ("causal", False), ("return_attn_probs", False), ("convert_mask", True)] + ext
    assert [n for n, _ in sig(bp.unpad_input)] == ["hidden_states", "attention_mask"]
    assert [n for n, _ in sig(bp.pad_input)] == ["hidden_states", "indices", "batch", "seqlen"]
    for cls in ("FlashAttnQKVPackedFunc", "FlashAttnKVPackedFunc", "FlashAttnFunc"):
        assert issubclass(getattr(fi, cls), torch.autograd.Function)
    from flash_attn import flash_attn_gfx950 as be
    assert list(inspect.signature(be.fwd).parameters) == [
        "q", "k", "v", "cu_seqlens_q", "cu_seqlens_k", "max_seqlen_q", "max_seqlen_k", "p_dropout", "softmax_scale",
        "zero_tensors", "is_causal", "return_softmax", "gen", "alibi_slopes", "keep_words", "attn_bias", "rotary",
        "q_rot"]  # fmha_api.cpp:173-186 + extensions
    assert sig(fi.flash_attn_unpadded_qkvpacked_rotary_func) == [
        ("qkv", "<req>"), ("cos_half", "<req>"), ("sin_half", "<req>"), ("cu_seqlens", "<req>"), ("max_seqlen", "<req>"),
        ("dropout_p", "<req>"), ("softmax_scale", None), ("causal", False)]  # extension: rotary embedding inside the kernels
    assert list(inspect.signature(be.bwd_block).parameters) == [
        "dout", "q", "k", "v", "out", "softmax_lse", "dq", "dk", "dv", "cu_seqlens_q", "cu_seqlens_k", "blockmask",
        "max_seqlen_q", "max_seqlen_k", "p_dropout", "softmax_scale", "is_causal", "gen", "row_order", "alibi_slopes",
        "attn_bias", "dbias"]  # fmha_api.cpp:575-594 + extensions


def test_blockmask_row_order_is_a_permutation_that_groups_similar_rows():
    """fa_blocksparse_row_order (host code of the library) lists every row block once, is deterministic, never stages more
    key blocks than the plain order, saves a third of the staged blocks and a fifth of the waves' work on independently drawn
    16 x 256 blocks, handles more than 64 key blocks and ragged ends, and leaves layouts made of whole 128-row tiles alone"""
    from flash_attn import flash_attn_gfx950 as be
    g = torch.Generator().manual_seed(0)

    def staged(m, order):  # key blocks a workgroup (eight consecutive entries) has to stage, summed
        return sum(int(m[order[i:i + 8]].any(0).sum()) for i in range(0, len(order), 8))

    def computed(m, order):  # key blocks a wave (two consecutive entries) has to compute on, summed
        return sum(int(m[order[i:i + 2]].any(0).sum()) for i in range(0, len(order), 2))

    for nrow, ncol, dens in ((256, 16, 0.25), (19, 2, 0.5), (64, 4, 0.1), (8, 1, 1.0), (1, 1, 0.0), (100, 70, 0.2)):
        m = torch.rand(nrow, ncol, generator=g) < dens
        order = be.blockmask_row_order(m)
        assert order.dtype == torch.int32 and sorted(order.tolist()) == list(range(nrow))
        assert torch.equal(order, be.blockmask_row_order(m))
        ident = torch.arange(nrow)
        assert staged(m, order.long()) <= staged(m, ident)
        if nrow == 256:
            assert staged(m, order.long()) < 0.7 * staged(m, ident)
            assert computed(m, order.long()) < 0.82 * computed(m, ident)
    tiles = (torch.rand(16, 16, generator=g) < 0.3).repeat_interleave(16, 0)  # 256 x 256 blocks
    assert be.blockmask_row_order(tiles).tolist() == list(range(256))
    lib = be.load_library()
    assert lib.fa_blocksparse_row_order(None, 4, 4, None) == -1


# ---------------------------------------------------------------- host helpers
def test_convert_blockmask_matches_spec():
    from flash_attn.flash_blocksparse_attn_interface import convert_blockmask
    g = torch.Generator().manual_seed(0)
    for shape in ((1, 1), (3, 2), (7, 5), (16, 4), (256, 16)):
        for dens in (0.0, 0.2, 0.6, 1.0):
            m = torch.rand(shape, generator=g) < dens
            got = convert_blockmask(m, causal=False)
            assert got.dtype == torch.int32 and tuple(got.shape) == (shape[1], shape[0])
            assert np.array_equal(got.numpy(), orc.convert_blockmask_ref(m.numpy()))
    # causal (the reference asserts against it, flash_blocksparse_attn_interface.py:21): the list of the layout with
    # the blocks that hold no key <= query taken out, found here element by element
    for shape in ((3, 2), (16, 1), (40, 3), (64, 4)):
        m = torch.rand(shape, generator=g) < 0.7
        seen = np.zeros(shape, dtype=bool)
        for r in range(shape[0]):
            for c in range(shape[1]):
                seen[r, c] = any(k <= q for q in range(16 * r, 16 * r + 16) for k in (256 * c, 256 * c + 255))
        want = orc.convert_blockmask_ref(m.numpy() & seen)
        assert np.array_equal(convert_blockmask(m, causal=True).numpy(), want)


def test_unpad_pad_match_spec_and_backprop():
    from flash_attn.bert_padding import pad_input, unpad_input
    g = torch.Generator().manual_seed(1)
    x = torch.randn(3, 9, 6, generator=g, dtype=torch.float64, requires_grad=True)
    lens = torch.tensor([9, 4, 1])
    mask = torch.arange(9)[None, :] < lens[:, None]
    rows, idx, cu, mx = unpad_input(x, mask)
    r_rows, r_idx, r_cu, r_mx = orc.unpad_ref(x.detach().numpy(), mask.numpy())
    assert np.array_equal(rows.detach().numpy(), r_rows) and np.array_equal(idx.numpy(), r_idx)
    assert cu.dtype == torch.int32 and cu.tolist() == r_cu.tolist() and mx == r_mx
    back = pad_input(rows, idx, 3, 9)
    assert np.array_equal(back.detach().numpy(), orc.pad_ref(r_rows, r_idx, 3, 9))
    assert torch.equal(back.detach(), x.detach() * mask[..., None])  # pad(unpad(x)) == x o mask
    w = torch.randn(3, 9, 6, generator=g, dtype=torch.float64)
    (back * w).sum().backward()
    assert torch.equal(x.grad, w * mask[..., None])


def test_rotary_is_a_rotation_by_position_times_frequency():
    """closed form of rotary.py:22-42,66-87: pair i at position t is rotated by t * 10000^(-2i/dim)."""
    from flash_attn.rotary import RotaryEmbedding, RotaryEmbedding2D
    dim, S = 8, 5
    rot = RotaryEmbedding(dim)
    g = torch.Generator().manual_seed(2)
    q = torch.randn(2, 3, S, dim, generator=g, dtype=torch.float64)
    k = torch.randn(2, 3, S, dim, generator=g, dtype=torch.float64)
    rq, rk = rot(q, k)
    t = torch.arange(S, dtype=torch.float64)[:, None]
    ang = t * (10000.0 ** (-torch.arange(0, dim, 2, dtype=torch.float64) / dim))[None, :]
    zq = torch.view_as_complex(q.reshape(2, 3, S, dim // 2, 2).contiguous()) * torch.polar(torch.ones_like(ang), ang)
    assert torch.allclose(torch.view_as_real(zq).reshape(2, 3, S, dim), rq, atol=1e-6)
    # norms are preserved and q.k depends only on relative position
    assert torch.allclose(rq.norm(dim=-1), q.norm(dim=-1), atol=1e-6)
    q1 = torch.randn(dim, generator=g, dtype=torch.float64).expand(1, 1, S, dim).contiguous()
    k1 = torch.randn(dim, generator=g, dtype=torch.float64).expand(1, 1, S, dim).contiguous()
    a, b = RotaryEmbedding(dim)(q1, k1)
    dots = a[0, 0] @ b[0, 0].T
    assert torch.allclose(dots[1, 0], dots[3, 2], atol=1e-6) and torch.allclose(dots[0, 2], dots[2, 4], atol=1e-6)
    # layout (b, s, h, d) gives the same numbers as (b, h, s, d)
    rq2, _ = RotaryEmbedding(dim)(q.transpose(1, 2), k.transpose(1, 2), seq_dimension=-3)
    assert torch.allclose(rq2.transpose(1, 2), rq, atol=1e-12)
    # 2-D: first half of the channels rotates with the column index, second half with the row index
    side = 3
    x = torch.randn(1, 2, side * side, 8, generator=g, dtype=torch.float64)
    r2, _ = RotaryEmbedding2D(8)(x, x)
    one = RotaryEmbedding(4)
    grid = x.reshape(1, 2, side, side, 8)
    cols, _ = one(grid[..., :4], grid[..., :4], seq_dimension=-2)
    rows, _ = RotaryEmbedding(4)(grid[..., 4:].transpose(2, 3), grid[..., 4:].transpose(2, 3), seq_dimension=-2)
    want = torch.cat([cols, rows.transpose(2, 3)], dim=-1).reshape(1, 2, side * side, 8)
    assert torch.allclose(r2, want, atol=1e-12)


def test_blocksparse_module_layout_handling_on_host():
    """FlashBlocksparseAttention keeps the layout and its converted form as buffers (flash_blocksparse_attention.py:31-36)
    and accepts a tensor, a make_layout() object or, only with hydra installed, a _target_ mapping."""
    import importlib.util
    from flash_attn.flash_blocksparse_attention import FlashBlocksparseAttention
    layout = (torch.arange(48 * 3).reshape(48, 3) % 4 != 1).to(torch.int32)

    class Cfg:
        def make_layout(self, seqlen):
            assert seqlen == 768  # 700 rounded up to a multiple of 256
            return layout

    m = FlashBlocksparseAttention(Cfg(), max_seq_length=700)
    assert set(dict(m.named_buffers())) == {"layout", "blockmask_converted"}
    assert torch.equal(m.blockmask_converted, torch.tensor(orc.convert_blockmask_ref(layout.numpy())))
    assert tuple(m._blockmask(300).shape) == (19, 2) and tuple(m._blockmask(768).shape) == (48, 3)
    with pytest.raises(AssertionError):
        m._blockmask(769)
    with pytest.raises(ValueError):
        FlashBlocksparseAttention(layout[:10], max_seq_length=700)
    with pytest.raises(TypeError):
        FlashBlocksparseAttention("not a layout")
    if importlib.util.find_spec("hydra") is None:
        with pytest.raises(RuntimeError, match="hydra"):
            FlashBlocksparseAttention({"_target_": "some.module.Config"})


def test_dbias_layout_is_validated_before_anything_is_launched(lib):
    """every (batch, head) must have its own slice of dbias: overlapping slices would be written by several workgroups"""
    from flash_attn import flash_attn_gfx950 as be
    a = be.BwdArgs()
    a.struct_bytes = ctypes.sizeof(a)
    a.dtype = be.FA_FP16
    a.batch, a.nheads, a.head_dim = 2, 3, 64
    a.total_q = a.total_k = 64
    a.max_seqlen_q = a.max_seqlen_k = 32
    a.lse_seq_stride = 32
    a.p_dropout, a.softmax_scale = 0.0, 0.125
    fake = 0x10000  # never dereferenced: the checks below fail before any launch
    for f in ("dout", "q", "k", "v", "out", "softmax_lse", "dq", "dk", "dv", "softmax_d", "cu_seqlens_q", "cu_seqlens_k"):
        setattr(a, f, fake)
    for t in ("do", "q", "k", "v", "o", "dq", "dk", "dv"):
        setattr(a, t + "_row_stride", 192)
        setattr(a, t + "_head_stride", 64)
    a.attn_bias, a.bias_row_stride, a.bias_head_stride, a.bias_batch_stride = fake, 32, 32 * 32, 3 * 32 * 32
    a.dbias = fake
    good = dict(dbias_row_stride=32, dbias_head_stride=32 * 32, dbias_batch_stride=3 * 32 * 32)
    for field, value in (("dbias_row_stride", 24), ("dbias_head_stride", 31 * 32), ("dbias_head_stride", 0),
                         ("dbias_batch_stride", 2 * 32 * 32), ("dbias_batch_stride", 0)):
        for k, v in good.items():
            setattr(a, k, v)
        setattr(a, field, value)
        assert lib.fa_bwd(ctypes.byref(a)) == -1 and b"dbias needs its own slice" in lib.fa_last_error(), (field, value)
    for k, v in good.items():
        setattr(a, k, v)
    a.dbias = fake + 1
    assert lib.fa_bwd(ctypes.byref(a)) == -1 and b"2-byte alignment" in lib.fa_last_error()
    a.dbias, a.attn_bias = fake, None
    assert lib.fa_bwd(ctypes.byref(a)) == -1 and b"dbias without attn_bias" in lib.fa_last_error()


def test_in_kernel_rotary_arguments_are_validated_before_anything_is_launched(lib):
    """tables come in pairs, aligned, with a row for every position; not together with the probability dump"""
    from flash_attn import flash_attn_gfx950 as be
    fake = 0x10000  # never dereferenced: the checks below fail before any launch
    f = be.FwdArgs()
    f.struct_bytes = ctypes.sizeof(f)
    f.dtype = be.FA_FP16
    f.batch, f.nheads, f.head_dim = 2, 3, 64
    f.total_q = f.total_k = 64
    f.max_seqlen_q = f.max_seqlen_k = 32
    f.p_dropout, f.softmax_scale = 0.0, 0.125
    for name in ("q", "k", "v", "o", "softmax_lse", "cu_seqlens_q", "cu_seqlens_k"):
        setattr(f, name, fake)
    for t in ("q", "k", "v", "o"):
        setattr(f, t + "_row_stride", 192)
        setattr(f, t + "_head_stride", 64)
    f.rotary_cos, f.rotary_table_rows = fake, 32
    assert lib.fa_fwd(ctypes.byref(f)) == -1 and b"come together" in lib.fa_last_error()
    f.rotary_sin = fake + 8
    assert lib.fa_fwd(ctypes.byref(f)) == -1 and b"16-byte aligned" in lib.fa_last_error()
    f.rotary_sin, f.rotary_table_rows = fake, 31
    assert lib.fa_fwd(ctypes.byref(f)) == -1 and b"a row for every query position" in lib.fa_last_error()
    f.rotary_table_rows, f.s_dmask = 32, fake
    assert lib.fa_fwd(ctypes.byref(f)) == -4 and b"rotate with fa_rotary first" in lib.fa_last_error()
    f.s_dmask, f.q_rot, f.q_rot_row_stride, f.q_rot_head_stride = None, fake, 100, 64
    assert lib.fa_fwd(ctypes.byref(f)) == -1 and b"q_rot must be" in lib.fa_last_error()

    a = be.BwdArgs()
    a.struct_bytes = ctypes.sizeof(a)
    a.dtype = be.FA_FP16
    a.batch, a.nheads, a.head_dim = 2, 3, 64
    a.total_q = a.total_k = 64
    a.max_seqlen_q, a.max_seqlen_k = 32, 40
    a.lse_seq_stride = 32
    a.p_dropout, a.softmax_scale = 0.0, 0.125
    for name in ("dout", "q", "k", "v", "out", "softmax_lse", "dq", "dk", "dv", "softmax_d", "cu_seqlens_q", "cu_seqlens_k"):
        setattr(a, name, fake)
    for t in ("do", "q", "k", "v", "o", "dq", "dk", "dv"):
        setattr(a, t + "_row_stride", 192)
        setattr(a, t + "_head_stride", 64)
    a.rotary_sin, a.rotary_table_rows = fake, 40
    assert lib.fa_bwd(ctypes.byref(a)) == -1 and b"come together" in lib.fa_last_error()
    a.rotary_cos, a.rotary_table_rows = fake, 39
    assert lib.fa_bwd(ctypes.byref(a)) == -1 and b"a row for every query and key position" in lib.fa_last_error()


def test_launch_policy_values_and_one_kernel_backward_scratch(lib):
    """fa_set_launch_policy: tile shape in the low bits, backward plan in 0x30; the one-kernel backward asks for scratch only
    where it exists (head dim 64, dense, no mask, dropout or bias, at most 32 key tiles)"""
    from flash_attn import flash_attn_gfx950 as be
    for ok in (0, 1, 2, 0x10, 0x11, 0x12, 0x20, 0x21, 0x22, 0x40, 0x52):
        assert lib.fa_set_launch_policy(ok) == 0
    for bad in (3, 0x30, 0x80, 0x43, -1, 0x100):
        assert lib.fa_set_launch_policy(bad) == -1 and b"launch policy" in lib.fa_last_error()
    a = be.BwdArgs()
    a.struct_bytes = ctypes.sizeof(a)
    a.batch, a.nheads, a.head_dim = 8, 12, 64
    a.max_seqlen_q = a.max_seqlen_k = 2048
    try:
        lib.fa_set_launch_policy(0)
        assert lib.fa_bwd_workspace_bytes(ctypes.byref(a)) == 0      # the two-kernel backward needs no scratch
        lib.fa_set_launch_policy(0x20)
        want = 8 * 12 * 64 * (32 * 64 * 4 + 16)                      # fp32 running sums and four counters per 32-row tile
        assert lib.fa_bwd_workspace_bytes(ctypes.byref(a)) == want
        for field, value in (("head_dim", 128), ("is_causal", 1), ("p_dropout", 0.1), ("max_seqlen_k", 4097)):
            b = be.BwdArgs.from_buffer_copy(a)
            setattr(b, field, value)
            assert lib.fa_bwd_workspace_bytes(ctypes.byref(b)) == 0, field
    finally:
        lib.fa_set_launch_policy(0)


def test_key_split_workspace_plan(lib):
    """fa_fwd_workspace_bytes asks for scratch only for dense, non-causal forwards with one query tile, few
    (batch, head) pairs and many keys; the size is n_splits * (fp32 partial outputs + partial lse)."""
    from flash_attn import flash_attn_gfx950 as be
    a = _valid_fwd_args(be)
    a.batch, a.nheads, a.head_dim = 8, 12, 64
    a.total_q, a.total_k, a.max_seqlen_q, a.max_seqlen_k = 8, 8 * 2048, 1, 2048
    need = lib.fa_fwd_workspace_bytes(ctypes.byref(a))
    # 96 workgroups -> 8 splits of 4 key tiles; partial o: 8 x 8 x 12 x 64 fp32, partial lse: 8 x 8 x 12 x 16 fp32
    assert need == 8 * 8 * 12 * 64 * 4 + 8 * 8 * 12 * 16 * 4
    a.is_causal = 1
    assert lib.fa_fwd_workspace_bytes(ctypes.byref(a)) == 0
    a.is_causal = 0
    a.max_seqlen_q, a.total_q = 129, 8 * 129                   # more than one query tile per sequence
    assert lib.fa_fwd_workspace_bytes(ctypes.byref(a)) == 0
    a.max_seqlen_q, a.total_q, a.max_seqlen_k = 1, 8, 300      # too few keys to share
    assert lib.fa_fwd_workspace_bytes(ctypes.byref(a)) == 0
    a.max_seqlen_k, a.batch, a.total_q = 2048, 64, 64          # enough (batch, head) pairs to fill the chip
    assert lib.fa_fwd_workspace_bytes(ctypes.byref(a)) == 0
    # the backward asks for the fp32 partial dQ of the same plan (8 splits x 8 rows x 12 heads x 64), and for nothing
    # where the forward asks for nothing
    g = be.BwdArgs()
    g.struct_bytes = ctypes.sizeof(g)
    g.batch, g.nheads, g.head_dim = 8, 12, 64
    g.total_q, g.total_k, g.max_seqlen_q, g.max_seqlen_k = 8, 8 * 2048, 1, 2048
    assert lib.fa_bwd_workspace_bytes(ctypes.byref(g)) == 8 * 8 * 12 * 64 * 4
    g.is_causal = 1
    assert lib.fa_bwd_workspace_bytes(ctypes.byref(g)) == 0
    g.is_causal, g.max_seqlen_q, g.total_q = 0, 2048, 8 * 2048
    assert lib.fa_bwd_workspace_bytes(ctypes.byref(g)) == 0


def test_rows_and_rotary_argument_checks(lib):
    """the byte-movement entry points reject bad arguments before any launch (CPU only: nothing valid is executed)"""
    from flash_attn import flash_attn_gfx950 as be
    assert lib.fa_scatter_rows_workspace_bytes(1000) == 4000 and lib.fa_scatter_rows_workspace_bytes(0) == 0
    assert lib.fa_gather_rows(0x1000, 0x2000, 0x3000, 4, 4, 64, 32, 64, None) == -1      # row stride < row width
    assert b"stride" in lib.fa_last_error()
    assert lib.fa_gather_rows(None, 0x2000, 0x3000, 4, 4, 64, 64, 64, None) == -1        # null source
    assert lib.fa_gather_rows(None, None, None, 0, 0, 64, 64, 64, None) == 0             # nothing to do
    assert lib.fa_scatter_rows(0x1000, 0x2000, 0x3000, 4, 8, 64, 64, 64, None, 0, None) == -2
    assert b"workspace" in lib.fa_last_error()
    assert lib.fa_scatter_rows(0x1000, 0x2000, 0x3000, 4, -1, 64, 64, 64, 0x4000, 64, None) == -1
    r = be.RotaryArgs()
    r.struct_bytes = ctypes.sizeof(r) - 4
    assert lib.fa_rotary(ctypes.byref(r)) == -1 and b"struct size" in lib.fa_last_error()
    r.struct_bytes = ctypes.sizeof(r)
    r.dtype, r.n_rows, r.n_parts, r.n_rotated, r.n_heads, r.head_dim = 0, 4, 3, 2, 2, 12
    assert lib.fa_rotary(ctypes.byref(r)) == -1 and b"multiple of 8" in lib.fa_last_error()
    r.head_dim, r.n_rotated = 64, 4
    assert lib.fa_rotary(ctypes.byref(r)) == -1 and b"sizes" in lib.fa_last_error()
    r.n_rotated = 2
    assert lib.fa_rotary(ctypes.byref(r)) == -1 and b"null" in lib.fa_last_error()
    r.n_rows = 0
    assert lib.fa_rotary(ctypes.byref(r)) == 0


def test_bias_grad_reduce_argument_checks(lib):
    """fa_bias_grad_reduce rejects bad arguments before any launch (CPU only: nothing valid is executed)"""
    ok_in = (2, 3, 16, 20, 3 * 16 * 24, 16 * 24, 24)   # batch, heads, rows, cols, dbias strides (rows padded to 24 columns)
    ok_out = (1, 0, 3 * 16 * 20, 16 * 20, 20)          # sum_batch, sum_heads, out strides
    call = lambda dbias, out, dtype, i, o: lib.fa_bias_grad_reduce(dbias, out, dtype, *i, *o, None)
    assert call(0x1000, 0x2000, 2, ok_in, ok_out) == -1 and b"dtype" in lib.fa_last_error()
    assert call(None, 0x2000, 0, ok_in, ok_out) == -1 and b"null" in lib.fa_last_error()
    assert call(0x1008, 0x2000, 0, ok_in, ok_out) == -1 and b"aligned" in lib.fa_last_error()            # 8-byte aligned only
    assert call(0x1000, 0x2000, 0, (2, 3, 16, 20, 3 * 16 * 20, 16 * 20, 20), ok_out) == -1               # rows not padded to 8
    assert call(0x1000, 0x2000, 0, ok_in, (1, 0, 3 * 16 * 20, 16 * 20, 19)) == -1 and b"out row" in lib.fa_last_error()
    assert call(0x1000, 0x2000, 0, (70000, 3, 16, 20, 3 * 16 * 24, 16 * 24, 24), ok_out) == -1
    assert call(None, None, 1, (0, 3, 16, 20, 0, 0, 24), ok_out) == 0                                    # nothing to do
    assert call(None, None, 1, (2, 3, 16, 0, 0, 0, 0), ok_out) == 0


def test_header_is_plain_c(tmp_path):
    """include/flash_attn_gfx950.h must be usable from C (the boundary a cgo / JNI / ctypes binding sees): it compiles as
    C99 with warnings as errors, and every declared entry point can be named."""
    import subprocess
    from flash_attn import flash_attn_gfx950 as be
    src = tmp_path / "use_header.c"
    names = [n for n in be.EXPORTED_SYMBOLS]
    src.write_text('#include "flash_attn_gfx950.h"\n'
                   "typedef void (*entry_t)(void);\n"
                   "entry_t entry_points[] = {" + ", ".join("(entry_t)%s" % n for n in names) + "};\n"
                   "int sizes[] = {(int)sizeof(fa_fwd_args), (int)sizeof(fa_bwd_args), (int)sizeof(fa_rotary_args)};\n")
    r = subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-fsyntax-only",
                        "-I", os.path.join(ROOT, "include"), str(src)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, r.stdout



def test_prepare_attn_bias_layout_rules():
    """prepare_attn_bias hands the caller's tensor through when the kernels can read it as it is (keys contiguous, rows a
    multiple of 8 elements, 16-byte aligned) and pads a copy otherwise; shape, dtype and device are checked."""
    from flash_attn import flash_attn_gfx950 as be
    q = torch.zeros(10, 3, 64, dtype=torch.float16)
    good = torch.randn(1, 3, 40, 48).half()
    assert be.prepare_attn_bias(good, q, 2, 3, 40, 48) is good
    assert be.prepare_attn_bias(good, q, 2, 3, 33, 41) is good                       # larger than needed is fine
    odd = torch.randn(2, 1, 40, 45).half()
    p = be.prepare_attn_bias(odd, q, 2, 3, 40, 45)
    assert p is not odd and tuple(p.shape) == (2, 1, 40, 48) and p.stride(2) % 8 == 0 and p.stride(3) == 1
    assert torch.equal(p[..., :45], odd) and torch.equal(p[..., 45:], torch.zeros(2, 1, 40, 3).half())
    view = torch.randn(1, 3, 40, 96).half()[..., ::2]                                  # keys not contiguous
    p = be.prepare_attn_bias(view, q, 2, 3, 40, 48)
    assert p.stride(3) == 1 and torch.equal(p, view)
    for bad, msg in ((torch.zeros(3, 3, 40, 48).half(), "attn_bias must be"),           # batch neither 1 nor 2
                     (torch.zeros(1, 2, 40, 48).half(), "attn_bias must be"),           # heads neither 1 nor 3
                     (torch.zeros(1, 3, 39, 48).half(), "attn_bias must be"),           # too few rows
                     (torch.zeros(1, 3, 40, 47).half(), "attn_bias must be"),           # too few keys
                     (torch.zeros(3, 40, 48).half(), "attn_bias must be"),              # not 4-D
                     (torch.zeros(1, 3, 40, 48), "dtype and device")):                  # fp32 for fp16 inputs
        with pytest.raises(RuntimeError, match=msg):
            be.prepare_attn_bias(bad, q, 2, 3, 40, 48)
