"""fa_fwd_block_noalloc (the block-sparse forward whose activity maps live in a device array inside the library, for
callers that cannot allocate) against fa_fwd_block with caller scratch: same kernels, so outputs must agree bit for bit.
Two calls in a row through the raw C ABI, the second on a smaller input: the built-in array keeps the first call's maps
and every call must rebuild what it reads."""
import ctypes
import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "flash-attention_amd"))
sys.path.insert(0, ROOT)

def _args(be, q, k, v, o, lse, cu, bm, max_s, causal):
    a = be.FwdArgs()
    a.struct_bytes = ctypes.sizeof(be.FwdArgs)
    a.dtype = be.FA_FP16 if q.dtype == torch.float16 else be.FA_BF16
    a.q, a.k, a.v, a.o = q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr()
    a.softmax_lse = lse.data_ptr()
    a.cu_seqlens_q = a.cu_seqlens_k = cu.data_ptr()
    a.blockmask = bm.data_ptr()
    a.q_row_stride, a.q_head_stride = q.stride(0), q.stride(1)
    a.k_row_stride, a.k_head_stride = k.stride(0), k.stride(1)
    a.v_row_stride, a.v_head_stride = v.stride(0), v.stride(1)
    a.o_row_stride, a.o_head_stride = o.stride(0), o.stride(1)
    a.batch, a.nheads, a.head_dim = cu.numel() - 1, q.shape[1], q.shape[2]
    a.total_q = a.total_k = q.shape[0]
    a.max_seqlen_q = a.max_seqlen_k = max_s
    a.p_dropout, a.softmax_scale = 0.0, q.shape[2] ** -0.5
    a.is_causal = int(causal)
    a.stream = torch.cuda.current_stream().cuda_stream
    return a


def _run_case(be, lib, lens, H, D, dtype, density, causal, seed):
    from flash_attn.flash_blocksparse_attn_interface import convert_blockmask
    g = torch.Generator().manual_seed(seed)
    total, max_s = sum(lens), max(lens)
    qkv = torch.randn(total, 3, H, D, generator=g).to(dtype).cuda()
    q, k, v = qkv[:, 0], qkv[:, 1], qkv[:, 2]
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32).cuda()
    sq_r, sk_r = be.round_seqlens(D, max_s, max_s, True)
    layout = torch.rand(sq_r // 16, sk_r // 256, generator=g) < density
    layout[1] = False  # a row block without keys
    bm = convert_blockmask(layout.cuda(), causal=causal)
    outs = []
    for entry in ("fa_fwd_block", "fa_fwd_block_noalloc"):
        o = torch.full((total, H, D), 7.0, dtype=dtype, device="cuda")
        lse = torch.full((len(lens), H, sq_r), 7.0, dtype=torch.float32, device="cuda")
        a = _args(be, q, k, v, o, lse, cu, bm, max_s, causal)
        ws = None
        if entry == "fa_fwd_block":
            n = lib.fa_fwd_workspace_bytes(ctypes.byref(a))
            assert n > 0
            ws = torch.empty(n, dtype=torch.uint8, device="cuda")
            a.workspace, a.workspace_bytes = ws.data_ptr(), n
        rc = getattr(lib, entry)(ctypes.byref(a))
        assert rc == 0, lib.fa_last_error()
        torch.cuda.synchronize()
        outs.append((o, lse))
    (o0, l0), (o1, l1) = outs
    assert torch.equal(o0, o1), "o differs: max %g" % (o0.float() - o1.float()).abs().max().item()
    for b, L in enumerate(lens):
        assert torch.equal(l0[b, :, :L], l1[b, :, :L])
    assert torch.isfinite(o1.float()).all() and o1.float().abs().max() > 0


@pytest.mark.gpu
def test_noalloc_matches_fwd_block_on_two_calls_in_a_row():
    from flash_attn import flash_attn_gfx950 as be
    lib = be.load_library()
    print("case 1: lens [1500, 1100] H=3 d=64 fp16", flush=True)
    _run_case(be, lib, [1500, 1100], 3, 64, torch.float16, 0.35, False, 1)
    print("case 2 (smaller): lens [300, 77] H=2 d=32 bf16 causal", flush=True)
    _run_case(be, lib, [300, 77], 2, 32, torch.bfloat16, 0.6, True, 2)


def test_noalloc_refuses_layouts_beyond_its_scratch():
    # host-side check only: runs without a GPU
    from flash_attn import flash_attn_gfx950 as be
    lib = be.load_library()
    a = be.FwdArgs()
    a.struct_bytes = ctypes.sizeof(be.FwdArgs)
    a.head_dim, a.max_seqlen_q, a.max_seqlen_k = 64, 40000, 40000
    a.blockmask = 256  # never read: the size check comes first
    assert lib.fa_fwd_block_noalloc(ctypes.byref(a)) == -2
    assert b"built-in scratch" in lib.fa_last_error()
