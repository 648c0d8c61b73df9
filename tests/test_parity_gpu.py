"""GPU parity tests: the HIP kernels (called through the ctypes binding of the C ABI) against the CPU oracle on the
same seeded inputs.

Tolerance (stated by the build's target): for every output X in {out, dq, dk, dv}
    max|X_ours - X_ref32| <= 2 * max|X_half - X_ref32| + floor
where X_ref32 is the fp32 closed form (oracle), X_half the same closed form evaluated by PyTorch in the input dtype
(fp16/bf16) on the GPU, and floor = 2e-4 (fp16) / 2e-3 (bf16), or half an ulp of the largest |X_ref32| if that is more
(two correct roundings of the same sum differ by that much), absorbs outputs that are exactly representable in the half
evaluation.  Every comparison is recorded (error, yardstick, their ratio, how much of the floor was used) and, if the
environment variable FA_PARITY_RATIOS_DIR names a directory, the list is written to parity_error_ratios.json there at the
end of the session.
softmax_lse is fp32 on both sides and is held to two bounds: the same yardstick - the logsumexp PyTorch computes from
half-precision scores - and an absolute cap |lse_ours - lse_ref32| <= LSE_TOL = 1e-3 (fp16) / 4.5e-3 (bf16).
The inputs are exact; the forward kernel sums the probabilities after they have been rounded to the tensor dtype (the
values the P V product consumes), so a row dominated by one key carries that one rounding: at most 2^-11 (fp16) or
2^-8 (bf16) relative in the row sum, i.e. 4.9e-4 / 3.9e-3 absolute in its logarithm.  Dropout masks are compared bit for
bit.
"""
import ctypes
import math
import os

import numpy as np
import pytest
import torch

from oracle import attention_oracle as orc

pytestmark = pytest.mark.gpu

FLOOR = {torch.float16: 2e-4, torch.bfloat16: 2e-3}
LSE_TOL = {torch.float16: 1e-3, torch.bfloat16: 4.5e-3}
HALF_ULP = {torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.fixture(scope="module", autouse=True)
def _need_gpu(lib):
    assert torch.cuda.is_available(), "these tests need the MI355X"


@pytest.fixture(params=[1, 2], ids=["full-size tiles", "half-size tiles"])
def tile_shape(request):
    """Runs a test with both tile shapes of the dense kernels (the library picks per launch by default; the half-size
    variants exist for head dims up to 64): fa_set_launch_policy."""
    from flash_attn import flash_attn_gfx950 as be
    be.set_launch_policy(request.param)
    yield request.param
    be.set_launch_policy(0)


@pytest.fixture
def full_size_tiles():
    """Bitwise comparisons between launches of different sizes hold for one tile shape, not across the automatic choice."""
    from flash_attn import flash_attn_gfx950 as be
    be.set_launch_policy(1)
    yield
    be.set_launch_policy(0)


@pytest.fixture(params=[1 << 30, 0], ids=["keep words", "redrawn"])
def dropout_path(request):
    """Runs a dropout test both ways: the forward leaves its keep decisions for the backward to read (the default when
    the buffer is small enough), or every kernel draws them again (flash_attn_gfx950.KEEP_WORDS_MAX_BYTES = 0)."""
    from flash_attn import flash_attn_gfx950 as be
    old = be.KEEP_WORDS_MAX_BYTES, be.KEEP_WORDS_MAX_INPUT_RATIO
    be.KEEP_WORDS_MAX_BYTES, be.KEEP_WORDS_MAX_INPUT_RATIO = request.param, None  # (no cap relative to the inputs' size either)
    yield request.param
    be.KEEP_WORDS_MAX_BYTES, be.KEEP_WORDS_MAX_INPUT_RATIO = old


def _cu(lens, device="cuda"):
    return torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32, device=device)


def _inputs(lens_q, lens_k, H, D, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    tq, tk = sum(lens_q), sum(lens_k)
    mk = lambda n: torch.randn(n, H, D, generator=g).to(dtype)
    return mk(tq), mk(tk), mk(tk), mk(tq)


def half_attention(q, k, v, cu_q, cu_k, scale, causal, keep_mask=None, p=0.0, layout=None, dout=None, alibi_slopes=None,
                   attn_bias=None):
    """the closed form evaluated in the tensors' own half dtype by PyTorch (the error yardstick)"""
    q, k, v = (x.detach().clone().requires_grad_(dout is not None) for x in (q, k, v))
    bias = attn_bias.detach().clone().requires_grad_(dout is not None) if attn_bias is not None else None
    outs, lses = [], []
    for b in range(len(cu_q) - 1):
        qb = q[cu_q[b]:cu_q[b + 1]].transpose(0, 1)
        kb = k[cu_k[b]:cu_k[b + 1]].transpose(0, 1)
        vb = v[cu_k[b]:cu_k[b + 1]].transpose(0, 1)
        s = torch.matmul(qb, kb.transpose(1, 2)) * scale
        if alibi_slopes is not None:
            s = s + orc.alibi_bias(alibi_slopes, qb.shape[1], kb.shape[1], q.device).to(s.dtype)
        if bias is not None:
            s = s + bias[b if bias.shape[0] > 1 else 0, :, :qb.shape[1], :kb.shape[1]]
        valid = orc._score_mask(qb.shape[1], kb.shape[1], causal, layout, q.device)
        s = s.masked_fill(~valid[None], float("-inf"))
        empty = ~valid.any(-1)
        s = s.masked_fill(empty[None, :, None], 0.0)
        pr = torch.softmax(s, dim=-1)
        lses.append(torch.logsumexp(s, dim=-1).masked_fill(empty[None], float("-inf")).detach())
        pr = pr.masked_fill(~valid[None], 0.0)
        if keep_mask is not None:
            pr = pr * keep_mask[b].to(device=q.device, dtype=pr.dtype) / (1.0 - p)
        outs.append(torch.matmul(pr, vb).transpose(0, 1))
    out = torch.cat(outs, 0)
    res = {"out": out.detach(), "lse": lses}
    if dout is not None:
        out.backward(dout)
        res.update(dq=q.grad, dk=k.grad, dv=v.grad)
        if bias is not None:
            res["dbias"] = bias.grad
    return res


def _maxerr(a, b):
    return (a.float().cpu() - b.float().cpu()).abs().max().item()


RATIOS = []  # one record per comparison against the oracle, written out by _write_ratios at the end of the session


@pytest.fixture(scope="module", autouse=True)
def _write_ratios():
    yield
    out_dir = os.environ.get("FA_PARITY_RATIOS_DIR", "")
    if RATIOS and out_dir and os.path.isdir(out_dir):
        import json
        with open(os.path.join(out_dir, "parity_error_ratios.json"), "w") as f:
            json.dump(RATIOS, f, indent=0)


def check_against_oracle(ours, ref, half, dtype, names=("out", "dq", "dk", "dv"), what=""):
    for n in names:
        e_ours, e_half = _maxerr(ours[n], ref[n]), _maxerr(half[n], ref[n])
        # the floor is at least half an ulp of the largest output (gradients of a few tens are stored with a spacing of
        # 0.016 in fp16: two correct roundings of the same sum can differ by that much from the fp32 value)
        floor = max(FLOOR[dtype], HALF_ULP[dtype] * ref[n].float().abs().max().item())
        RATIOS.append({"case": what, "output": n, "dtype": str(dtype)[6:], "err": e_ours, "err_half_precision_pytorch": e_half,
                       "ratio": e_ours / e_half if e_half > 0 else None, "floor": floor,
                       "floor_used": max(0.0, e_ours - 2 * e_half) / floor})
        assert e_ours <= 2 * e_half + floor, "%s %s: ours %.3e vs half-precision PyTorch %.3e" % (what, n, e_ours, e_half)


def check_lse(got, want, half_lse, dtype, what=""):
    """got, want, half_lse: (H, L) for one sequence; want fp32 oracle, half_lse PyTorch's logsumexp of half-precision scores"""
    fin = torch.isfinite(want)
    assert torch.equal(torch.isfinite(got), fin), what
    if not fin.any():
        return
    e_ours = (got[fin] - want[fin]).abs().max().item()
    e_half = (half_lse.float().cpu()[fin] - want[fin]).abs().max().item()
    RATIOS.append({"case": what, "output": "lse", "dtype": str(dtype)[6:], "err": e_ours, "err_half_precision_pytorch": e_half,
                   "ratio": e_ours / e_half if e_half > 0 else None, "floor": 1e-4, "floor_used": max(0.0, e_ours - 2 * e_half) / 1e-4})
    assert e_ours <= 2 * e_half + 1e-4 and e_ours <= LSE_TOL[dtype], "%s lse: ours %.3e vs half-precision PyTorch %.3e" % (what, e_ours, e_half)


def run_ours(q, k, v, do, cu_q, cu_k, max_q, max_k, p, scale, causal, packing="sep", probs=False, alibi_slopes=None,
             attn_bias=None):
    from flash_attn import flash_attn_interface as fi
    dev = "cuda"
    cu_q, cu_k = cu_q.to(dev), cu_k.to(dev)
    bias_kw = {}
    if attn_bias is not None:
        bias_g = attn_bias.to(dev).requires_grad_()
        bias_kw = {"attn_bias": bias_g}
    if packing == "qkv":
        qkv = torch.stack([q, k, v], 1).to(dev).requires_grad_()
        res = fi.flash_attn_unpadded_qkvpacked_func(qkv, cu_q, max_q, p, scale, causal, probs, alibi_slopes=alibi_slopes,
                                                    **bias_kw)
    elif packing == "kv":
        qg = q.to(dev).requires_grad_()
        kv = torch.stack([k, v], 1).to(dev).requires_grad_()
        res = fi.flash_attn_unpadded_kvpacked_func(qg, kv, cu_q, cu_k, max_q, max_k, p, scale, causal, probs,
                                                   alibi_slopes=alibi_slopes, **bias_kw)
    else:
        qg, kg, vg = (x.to(dev).requires_grad_() for x in (q, k, v))
        res = fi.flash_attn_unpadded_func(qg, kg, vg, cu_q, cu_k, max_q, max_k, p, scale, causal, probs,
                                          alibi_slopes=alibi_slopes, **bias_kw)
    out = res[0] if probs else res
    out.backward(do.to(dev))
    torch.cuda.synchronize()
    if packing == "qkv":
        dq, dk, dv = qkv.grad[:, 0], qkv.grad[:, 1], qkv.grad[:, 2]
    elif packing == "kv":
        dq, dk, dv = qg.grad, kv.grad[:, 0], kv.grad[:, 1]
    else:
        dq, dk, dv = qg.grad, kg.grad, vg.grad
    r = {"out": out.detach(), "dq": dq, "dk": dk, "dv": dv}
    if attn_bias is not None:
        r["dbias"] = bias_g.grad
    if probs:
        r["lse"], r["S_dmask"] = res[1], res[2]
    return r


def _parity_case(lens_q, lens_k, H, D, dtype, causal, packing="sep", seed=0, scale=None, max_pad=0):
    q, k, v, do = _inputs(lens_q, lens_k, H, D, dtype, seed)
    cu_q, cu_k = _cu(lens_q, "cpu"), _cu(lens_k, "cpu")
    sc = D ** -0.5 if scale is None else scale
    ours = run_ours(q, k, v, do, cu_q, cu_k, max(lens_q) + max_pad, max(lens_k) + max_pad, 0.0, scale, causal, packing,
                    probs=True)
    ref = orc.varlen_attention(q, k, v, cu_q, cu_k, sc, causal, dout=do)
    half = half_attention(q.cuda(), k.cuda(), v.cuda(), cu_q.tolist(), cu_k.tolist(), sc, causal, dout=do.cuda())
    what = "q%s k%s H%d D%d %s causal=%s %s" % (lens_q, lens_k, H, D, dtype, causal, packing)
    check_against_oracle(ours, ref, half, dtype, what=what)
    for b, L in enumerate(lens_q):  # lse: only rows < seqlen_q are defined
        check_lse(ours["lse"][b, :, :L].cpu(), ref["lse"][b], half["lse"][b], dtype, what)
    return ours, ref


# ------------------------------------------------------------------------------------------------
# seeded parity at oracle-friendly sizes: every head dim, both dtypes, causal, ragged lengths, packings
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("D", [16, 32, 64, 128])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("causal", [False, True])
def test_parity_head_dims(D, dtype, causal, tile_shape):
    _parity_case([113, 256, 37], [113, 256, 37], 3, D, dtype, causal, packing="qkv", seed=D)


@pytest.mark.parametrize("lens_q,lens_k", [
    ([1], [1]),                      # single token
    ([1, 1, 1], [300, 1, 17]),       # decode-like: one query per sequence
    ([15, 17, 16], [15, 17, 16]),    # around the 16-row granularity
    ([128, 129, 127], [128, 129, 127]),
    ([64, 200], [300, 65]),          # seqlen_q != seqlen_k
    ([257], [513]),
    ([5, 0, 9], [5, 0, 9]),          # an empty sequence in the batch
])
@pytest.mark.parametrize("causal", [False, True])
def test_parity_ragged_shapes(lens_q, lens_k, causal, tile_shape):
    _parity_case(lens_q, lens_k, 2, 64, torch.float16, causal, packing="kv", seed=len(lens_q))


def test_parity_separate_qkv_and_scale():
    _parity_case([100, 140], [90, 260], 4, 32, torch.bfloat16, False, packing="sep", seed=5, scale=0.3)
    _parity_case([100, 140], [100, 140], 4, 32, torch.float16, True, packing="sep", seed=6, scale=0.05)


def test_max_seqlen_may_exceed_the_longest_sequence(tile_shape):
    _parity_case([70, 33], [70, 33], 2, 64, torch.float16, False, packing="qkv", seed=7, max_pad=200)


def test_cpu_reference_config():
    """BASELINE config 1 (the reference's CPU-runnable case): B=2, H=12, d=64, N=128, packed qkv, non-causal, p=0."""
    _parity_case([128, 128], [128, 128], 12, 64, torch.float16, False, packing="qkv", seed=0)


def test_golden_fixture():
    z = np.load(os.path.join(GOLDEN, "attention_small.npz"))
    lens = z["lens"].tolist()
    cu = torch.tensor(z["cu_seqlens"])
    for dtype in (torch.float16, torch.bfloat16):
        q, k, v, do = (torch.tensor(z[n]).to(dtype) for n in ("q", "k", "v", "dout"))  # exact in both dtypes
        for causal, tag in ((False, "dense"), (True, "causal")):
            ours = run_ours(q, k, v, do, cu, cu, max(lens), max(lens), 0.0, None, causal, "sep", probs=True)
            ref = {n: torch.tensor(z["%s_%s" % (tag, n)]) for n in ("out", "dq", "dk", "dv")}
            half = half_attention(q.cuda(), k.cuda(), v.cuda(), cu.tolist(), cu.tolist(), 16 ** -0.5, causal, dout=do.cuda())
            check_against_oracle(ours, ref, half, dtype, what="golden " + tag)
            for b in range(2):
                assert (ours["lse"][b, :, :lens[b]].cpu() - torch.tensor(z["%s_lse%d" % (tag, b)])).abs().max() < 2e-3


def test_softmax_d_and_raw_c_abi():
    """calls fa_fwd / fa_bwd with raw pointers (no interface layer) and checks softmax_d = rowsum(dO o O)."""
    from flash_attn import flash_attn_gfx950 as be
    lens = [50, 77]
    q, k, v, do = (x.cuda() for x in _inputs(lens, lens, 2, 64, torch.float16, 11))
    cu = _cu(lens)
    o, lse = be.fwd(q, k, v, cu, cu, 77, 77, 0.0, 0.125, False, False, False, None)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    _, _, _, sd = be.bwd(do, q, k, v, o, lse, dq, dk, dv, cu, cu, 77, 77, 0.0, 0.125, False, False, None)
    torch.cuda.synchronize()
    assert tuple(lse.shape) == (2, 2, 80) and tuple(sd.shape) == (2, 2, 80)
    ref = orc.varlen_attention(q.cpu(), k.cpu(), v.cpu(), cu.tolist(), cu.tolist(), 0.125, False, dout=do.cpu())
    for b, L in enumerate(lens):
        assert (sd[b, :, :L].cpu() - ref["softmax_d"][b]).abs().max() < 2e-2
    assert _maxerr(dq, ref["dq"]) < 5e-3 and _maxerr(o, ref["out"]) < 2e-3
    # zero_tensors pre-fills what the kernels do not write (fmha_api.cpp:256-260): lse padding becomes -inf
    o2, lse2 = be.fwd(q, k, v, cu, cu, 77, 77, 0.0, 0.125, True, False, False, None)
    torch.cuda.synchronize()
    assert torch.equal(o2, o) and torch.isinf(lse2[0, :, 50:]).all() and torch.equal(lse2[1, :, :77], lse[1, :, :77])


def test_strided_views_and_noncontiguous_grads(tile_shape):
    """q, k, v as views of a packed tensor with extra padding between rows (row stride != 3*H*D)."""
    from flash_attn import flash_attn_gfx950 as be
    lens = [40, 90]
    H, D = 2, 64
    tot = sum(lens)
    g = torch.Generator().manual_seed(3)
    big = torch.randn(tot, 4, H, D + 8, generator=g).half().cuda()
    q, k, v = big[:, 0, :, :D], big[:, 1, :, :D], big[:, 3, :, :D]
    cu = _cu(lens)
    o, lse = be.fwd(q, k, v, cu, cu, 90, 90, 0.0, 0.125, False, True, False, None)
    o_c, _ = be.fwd(q.contiguous(), k.contiguous(), v.contiguous(), cu, cu, 90, 90, 0.0, 0.125, False, True, False, None)
    torch.cuda.synchronize()
    assert torch.equal(o, o_c)
    do = torch.randn(tot, H, D, generator=g).half().cuda()
    dbig = torch.zeros_like(big)
    be.bwd(do, q, k, v, o, lse, dbig[:, 0, :, :D], dbig[:, 1, :, :D], dbig[:, 3, :, :D], cu, cu, 90, 90, 0.0, 0.125,
           False, True, None)
    dq, dk, dv = (torch.empty(tot, H, D, dtype=torch.half, device="cuda") for _ in range(3))
    be.bwd(do, q.contiguous(), k.contiguous(), v.contiguous(), o, lse, dq, dk, dv, cu, cu, 90, 90, 0.0, 0.125, False,
           True, None)
    torch.cuda.synchronize()
    assert torch.equal(dbig[:, 1, :, :D], dk) and torch.equal(dbig[:, 3, :, :D], dv)
    assert torch.equal(dbig[:, 0, :, :D], dq)  # no atomics anywhere: results are bitwise reproducible
    assert dbig[:, 2].abs().max() == 0 and dbig[..., D:].abs().max() == 0  # nothing written outside the views


def test_error_behaviour_on_device():
    from flash_attn import flash_attn_gfx950 as be
    q = torch.zeros(16, 1, 64, dtype=torch.half, device="cuda")
    cu = torch.tensor([0, 16], dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError, match="p_dropout"):
        be.fwd(q, q, q, cu, cu, 16, 16, 1.0, 0.125, False, False, False, None)          # fmha_api.cpp:113
    with pytest.raises(RuntimeError, match="int32"):
        be.fwd(q, q, q, cu.long(), cu, 16, 16, 0.0, 0.125, False, False, False, None)   # :201
    with pytest.raises(RuntimeError, match="contiguous last"):
        qt = torch.zeros(16, 1, 128, dtype=torch.half, device="cuda")[..., ::2]
        be.fwd(qt, qt, qt, cu, cu, 16, 16, 0.0, 0.125, False, False, False, None)       # :210
    with pytest.raises(RuntimeError, match="shape"):
        be.fwd(q, q[:8], q, cu, cu, 16, 16, 0.0, 0.125, False, False, False, None)      # CHECK_SHAPE :227
    # an empty sequence in the batch is skipped, not an error
    cu2 = torch.tensor([0, 0, 16], dtype=torch.int32, device="cuda")
    o, lse = be.fwd(q, q, q, cu2, cu2, 16, 16, 0.0, 0.125, False, False, False, None)
    torch.cuda.synchronize()
    assert torch.isfinite(o).all()


def test_zero_tensors_prefills_what_the_kernels_do_not_write():
    """zero_tensors = True (fmha_api.cpp:256-260, 406-411): rows of the packed tensors that belong to no sequence
    (cu_seqlens[-1] < total) and the padding of lse / softmax_d / S_dmask come out as 0 / -inf instead of whatever the
    buffers held; the rows of real sequences are what a call without the flag computes."""
    from flash_attn import flash_attn_gfx950 as be
    H, D, lens, extra = 2, 32, [40, 23], 9
    total = sum(lens) + extra
    g = torch.Generator().manual_seed(11)
    q, k, v, do = (torch.randn(total, H, D, generator=g).half().cuda() for _ in range(4))
    cu = _cu(lens)
    used = sum(lens)
    o, lse, S = be.fwd(q, k, v, cu, cu, max(lens), max(lens), 0.0, D ** -0.5, True, False, True, None)
    o0, lse0 = be.fwd(q, k, v, cu, cu, max(lens), max(lens), 0.0, D ** -0.5, False, False, False, None)
    torch.cuda.synchronize()
    assert torch.equal(o[:used], o0[:used]) and o[used:].abs().max() == 0
    assert torch.equal(lse[0, :, :40], lse0[0, :, :40]) and torch.isinf(lse[0, :, 40:]).all() and torch.isinf(lse[1, :, 23:]).all()
    assert S[1, :, 23:].abs().max() == 0 and S[1, :, :, 23:].abs().max() == 0 and S[0, :, :40, :40].abs().max() > 0
    grads = [torch.full((total, H, D), 7.0, dtype=torch.half, device="cuda") for _ in range(3)]
    dq, dk, dv, sd = be.bwd(do, q, k, v, o, lse, grads[0], grads[1], grads[2], cu, cu, max(lens), max(lens), 0.0, D ** -0.5,
                            True, False, None)
    ref_g = [torch.full((total, H, D), 7.0, dtype=torch.half, device="cuda") for _ in range(3)]
    _, _, _, sd0 = be.bwd(do, q, k, v, o0, lse0, ref_g[0], ref_g[1], ref_g[2], cu, cu, max(lens), max(lens), 0.0, D ** -0.5,
                          False, False, None)
    torch.cuda.synchronize()
    for got, want in zip((dq, dk, dv), ref_g):
        assert torch.equal(got[:used], want[:used]) and got[used:].abs().max() == 0 and (want[used:] == 7).all()
    assert torch.equal(sd[0, :, :40], sd0[0, :, :40]) and sd[0, :, 40:].abs().max() == 0 and sd[1, :, 23:].abs().max() == 0
    want_sd = (do[:40].float() * o[:40].float()).sum(-1).transpose(0, 1)  # p_dropout = 0: rowsum(dout * out)
    assert (sd[0, :, :40] - want_sd).abs().max() < 2e-3
    # written tensors may not overlap: a zero head stride of the output is refused before anything is launched
    with pytest.raises(RuntimeError, match="may not overlap"):
        bad = torch.empty(total, 1, D, dtype=torch.half, device="cuda").expand(total, H, D)
        be.bwd(do, q, k, v, o, lse, bad, grads[1], grads[2], cu, cu, max(lens), max(lens), 0.0, D ** -0.5, False, False, None)


# ------------------------------------------------------------------------------------------------
# dropout: exact mask, exact algebra with that mask, keep rate, RNG semantics
# ------------------------------------------------------------------------------------------------
def _gen_state():
    torch.cuda.init()  # the default generators only exist once the runtime is up
    g = torch.cuda.default_generators[torch.cuda.current_device()]
    return g.initial_seed(), g.get_offset()


@pytest.mark.parametrize("D,dtype,causal", [(64, torch.float16, False), (32, torch.bfloat16, True), (128, torch.float16, False)])
def test_dropout_mask_is_the_defined_one_and_is_applied(D, dtype, causal, tile_shape, dropout_path):
    p = 0.17
    lens_q, lens_k, H = [70, 130], [70, 130], 3
    q, k, v, do = _inputs(lens_q, lens_k, H, D, dtype, 21)
    cu = _cu(lens_q, "cpu")
    torch.manual_seed(1234)
    seed, offset = _gen_state()
    ours = run_ours(q, k, v, do, cu, cu, 130, 130, p, None, causal, "qkv", probs=True)
    S = ours["S_dmask"].cpu()
    sq_r, sk_r = S.shape[2], S.shape[3]
    assert (sq_r, sk_r) == (144, 256)
    masks = []
    ref_plain = orc.varlen_attention(q, k, v, cu, cu, None, causal)
    for b, L in enumerate(lens_q):
        mb = np.stack([orc.dropout_keep_mask(seed, offset, b * H + h, L, L, p) for h in range(H)])
        masks.append(torch.tensor(mb))
        dropped = torch.signbit(S[b, :, :L, :L])
        valid = orc._score_mask(L, L, causal, None)
        assert torch.equal(dropped[:, valid], ~masks[b][:, valid]), "mask differs from its definition"
        assert (S[b, :, :L, :L].abs().float() - ref_plain["probs"][b]).abs().max() < (3e-3 if dtype == torch.float16 else 1.6e-2)
        assert S[b, :, L:, :].abs().max() == 0 and S[b, :, :, L:].abs().max() == 0  # padding region is zero
    # o and the gradients equal the closed form with exactly that mask
    ref = orc.varlen_attention(q, k, v, cu, cu, None, causal, p_dropout=p, keep_mask=masks, dout=do)
    half = half_attention(q.cuda(), k.cuda(), v.cuda(), cu.tolist(), cu.tolist(), D ** -0.5, causal, masks, p, dout=do.cuda())
    check_against_oracle(ours, ref, half, dtype, what="dropout D%d" % D)


def test_dropout_random_shapes_sweep(tile_shape, dropout_path):
    """Eight seeded random dropout cases (rates, head dims, ragged self- and cross-attention lengths, packings): the
    returned mask equals its definition bit for bit and out / gradients equal the closed form with that mask."""
    rng = np.random.default_rng(77)
    for case in range(8):
        D = int(rng.choice([16, 32, 64, 128]))
        dtype = torch.float16 if rng.integers(2) else torch.bfloat16
        B, H = int(rng.integers(1, 4)), int(rng.integers(1, 3))
        causal = bool(rng.integers(2))
        cross = bool(rng.integers(2)) and not causal
        lens_q = [int(x) for x in rng.integers(1, 200, B)]
        lens_k = [int(x) for x in rng.integers(1, 200, B)] if cross else list(lens_q)
        p = float(rng.choice([0.05, 0.1, 0.3, 0.5]))
        packing = "kv" if cross else str(rng.choice(["qkv", "sep"]))
        print("case %d: D=%d %s B=%d H=%d causal=%s q=%s k=%s p=%.2f %s" % (case, D, dtype, B, H, causal, lens_q, lens_k, p,
                                                                          packing), flush=True)
        q, k, v, do = _inputs(lens_q, lens_k, H, D, dtype, 300 + case)
        cu_q, cu_k = _cu(lens_q, "cpu"), _cu(lens_k, "cpu")
        torch.manual_seed(500 + case)
        seed, offset = _gen_state()
        ours = run_ours(q, k, v, do, cu_q, cu_k, max(lens_q), max(lens_k), p, None, causal, packing, probs=True)
        S = ours["S_dmask"].cpu()
        masks = []
        for b, (Lq, Lk) in enumerate(zip(lens_q, lens_k)):
            mb = np.stack([orc.dropout_keep_mask(seed, offset, b * H + h, Lq, Lk, p) for h in range(H)])
            masks.append(torch.tensor(mb))
            valid = orc._score_mask(Lq, Lk, causal, None)
            assert torch.equal(torch.signbit(S[b, :, :Lq, :Lk])[:, valid], ~masks[b][:, valid]), "mask differs from its definition"
        ref = orc.varlen_attention(q, k, v, cu_q, cu_k, None, causal, p_dropout=p, keep_mask=masks, dout=do)
        half = half_attention(q.cuda(), k.cuda(), v.cuda(), cu_q.tolist(), cu_k.tolist(), D ** -0.5, causal, masks, p,
                              dout=do.cuda())
        check_against_oracle(ours, ref, half, dtype, what="dropout sweep case %d" % case)


def test_dropout_keep_rate_and_rng_semantics():
    from flash_attn import flash_attn_interface as fi
    p, N, H, D = 0.1, 512, 4, 64
    qkv = torch.randn(2 * N, 3, H, D, device="cuda", dtype=torch.float16)
    cu = _cu([N, N])
    torch.manual_seed(7)
    _, _, S1 = fi.flash_attn_unpadded_qkvpacked_func(qkv, cu, N, p, None, False, True)
    _, _, S2 = fi.flash_attn_unpadded_qkvpacked_func(qkv, cu, N, p, None, False, True)
    torch.manual_seed(7)
    _, _, S3 = fi.flash_attn_unpadded_qkvpacked_func(qkv, cu, N, p, None, False, True)
    k1, k2, k3 = (~torch.signbit(s) for s in (S1, S2, S3))
    assert torch.equal(k1, k3), "same seed must give the same mask"
    assert not torch.equal(k1, k2), "successive calls must draw different masks"
    n = k1.numel()
    kp = orc.keep_probability(p)
    z = (k1.sum().item() - n * kp) / math.sqrt(n * kp * (1 - kp))
    assert abs(z) < 4.5, "keep rate off: z = %.2f" % z
    per_head = k1.float().mean(dim=(2, 3))
    assert (per_head - kp).abs().max() < 5e-3


def test_dropout_backward_reuses_the_forward_mask_without_probs(dropout_path):
    """production path (no S_dmask): gradients must match the closed form under the mask defined by the state the
    generator had when the forward ran, even after other draws moved the generator on."""
    p, lens, H, D = 0.25, [96, 200], 2, 64
    q, k, v, do = _inputs(lens, lens, H, D, torch.float16, 31)
    cu = _cu(lens, "cpu")
    from flash_attn import flash_attn_interface as fi
    torch.manual_seed(99)
    seed, offset = _gen_state()
    qkv = torch.stack([q, k, v], 1).cuda().requires_grad_()
    out = fi.flash_attn_unpadded_qkvpacked_func(qkv, cu.cuda(), 200, p)
    torch.rand(1000, device="cuda")  # advances the generator between forward and backward
    after = _gen_state()
    out.backward(do.cuda())
    assert _gen_state() == after, "backward must leave the generator where it found it"
    masks = [torch.tensor(np.stack([orc.dropout_keep_mask(seed, offset, b * H + h, L, L, p) for h in range(H)]))
             for b, L in enumerate(lens)]
    ref = orc.varlen_attention(q, k, v, cu, cu, None, False, p_dropout=p, keep_mask=masks, dout=do)
    half = half_attention(q.cuda(), k.cuda(), v.cuda(), cu.tolist(), cu.tolist(), D ** -0.5, False, masks, p, dout=do.cuda())
    ours = {"out": out.detach(), "dq": qkv.grad[:, 0], "dk": qkv.grad[:, 1], "dv": qkv.grad[:, 2]}
    check_against_oracle(ours, ref, half, torch.float16, what="dropout production path")


@pytest.mark.parametrize("D,dtype,causal,lens_q,lens_k,alibi", [
    (64, torch.float16, False, [300, 129, 512, 77], None, False),
    (64, torch.bfloat16, True, [405, 435, 303, 318], None, False),
    (32, torch.float16, True, [300, 129, 512, 77], None, False),
    (16, torch.bfloat16, False, [200, 100], [333, 1000], False),
    (128, torch.float16, False, [300, 129, 512], None, False),
    (128, torch.bfloat16, True, [1024, 77], None, False),
    (64, torch.float16, False, [64, 100], [2048, 1500], False),   # short query side: the key-split dQ
    (64, torch.float16, True, [300, 129], None, True),
])
def test_keep_words_hold_the_defined_mask_and_give_the_same_results(D, dtype, causal, lens_q, lens_k, alibi, tile_shape,
                                                                   monkeypatch):
    """The forward's keep words (one bit per score) equal the oracle's mask bit for bit in their documented layout, the
    forward's outputs do not depend on whether it leaves them, and the backward that reads them gives the gradients of the
    backward that draws the decisions again: bit for bit (at head dim 128 dq within one rounding: there the two dQ variants
    subtract Dk from dP at different points)."""
    from flash_attn import flash_attn_gfx950 as be
    monkeypatch.setattr(be, "KEEP_WORDS_MAX_INPUT_RATIO", None)  # small head dims: the words outweigh the inputs early
    lens_k = lens_k or lens_q
    p, H = 0.17, 3
    q, k, v, do = (x.cuda() for x in _inputs(lens_q, lens_k, H, D, dtype, 77))
    cq, ck = _cu(lens_q), _cu(lens_k)
    mq, mk = max(lens_q), max(lens_k)
    sl = (torch.rand(H, device="cuda") * 0.3) if alibi else None
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    st = g.get_state()
    seed, offset = g.initial_seed(), g.get_offset()
    o0, lse0 = be.fwd(q, k, v, cq, ck, mq, mk, p, D ** -0.5, False, causal, False, g, alibi_slopes=sl)
    g.set_state(st)
    kw = be.new_keep_words(q, cq, mq, mk, p)
    assert kw is not None and kw.numel() == len(lens_q) * H * ((mq + 127) // 128 * 128) * ((mk + 127) // 128 * 128) // 8
    kw.fill_(0xA5)
    o1, lse1 = be.fwd(q, k, v, cq, ck, mq, mk, p, D ** -0.5, False, causal, False, g, alibi_slopes=sl, keep_words=kw)
    assert torch.equal(o0, o1)
    for b, L in enumerate(lens_q):
        assert torch.equal(lse0[b, :, :L], lse1[b, :, :L])
    # layout: word [(b H + h) * key_blocks + key / 32][slot(q)], bit key % 32; slot swaps q's bits so that rows q and q + 4 are neighbours
    q_ext, kbs = (mq + 127) // 128 * 128, (mk + 127) // 128 * 128 // 32
    words = kw.view(torch.int32).view(len(lens_q) * H, kbs, q_ext).cpu().numpy().astype(np.uint32)
    for b, (Lq, Lk) in enumerate(zip(lens_q, lens_k)):
        for h in range(H):
            want = orc.dropout_keep_mask(seed, offset, b * H + h, Lq, Lk, p)          # [Lq, Lk] bool
            qs = np.arange(Lq)
            slot = (qs & ~31) | (qs & 24) | ((qs & 3) << 1) | ((qs >> 2) & 1)
            keys = np.arange(Lk)
            got = (words[b * H + h][keys[None, :] // 32, slot[:, None]] >> (keys[None, :] % 32).astype(np.uint32)) & 1
            valid = orc._score_mask(Lq, Lk, causal, None).numpy()
            assert np.array_equal(got.astype(bool)[valid], want[valid]), "keep words differ from the mask's definition"
    grads = []
    for words_arg in (None, kw):
        g.set_state(st)
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        be.bwd(do, q, k, v, o1, lse1, dq, dk, dv, cq, ck, mq, mk, p, D ** -0.5, False, causal, g, alibi_slopes=sl,
               keep_words=words_arg)
        grads.append((dq, dk, dv))
    torch.cuda.synchronize()
    assert torch.equal(grads[0][1], grads[1][1]) and torch.equal(grads[0][2], grads[1][2])
    if D <= 64:
        assert torch.equal(grads[0][0], grads[1][0])
    else:
        a, b_ = grads[0][0].float(), grads[1][0].float()
        assert (a - b_).abs().max() <= 2.0 ** (-10 if dtype == torch.float16 else -7) * a.abs().max()


def test_keep_words_argument_checks():
    from flash_attn import flash_attn_gfx950 as be
    lens, H, D, p = [100, 60], 2, 64, 0.1
    q, k, v, do = (x.cuda() for x in _inputs(lens, lens, H, D, torch.float16, 3))
    cu = _cu(lens)
    need = be.load_library().fa_keep_words_bytes(2, H, 100, 100)
    assert need == 2 * H * (128 // 32) * 128 * 4
    small = torch.empty(need - 16, dtype=torch.uint8, device="cuda")
    with pytest.raises(RuntimeError, match="keep_words of"):
        be.fwd(q, k, v, cu, cu, 100, 100, p, D ** -0.5, False, False, False, None, keep_words=small)
    odd = torch.empty(need + 16, dtype=torch.uint8, device="cuda")[4:]
    with pytest.raises(RuntimeError, match="16-byte aligned"):
        be.fwd(q, k, v, cu, cu, 100, 100, p, D ** -0.5, False, False, False, None, keep_words=odd)
    with pytest.raises(RuntimeError, match="uint8"):
        be.fwd(q, k, v, cu, cu, 100, 100, p, D ** -0.5, False, False, False, None, keep_words=small.view(torch.int16))
    # without dropout the buffer is ignored, whatever its size
    be.fwd(q, k, v, cu, cu, 100, 100, 0.0, D ** -0.5, False, False, False, None, keep_words=small)
    old = be.KEEP_WORDS_MAX_BYTES
    try:
        be.KEEP_WORDS_MAX_BYTES = need - 1
        assert be.new_keep_words(q, cu, 100, 100, p) is None
        be.KEEP_WORDS_MAX_BYTES = need
        assert be.new_keep_words(q, cu, 100, 100, p).numel() == need
        assert be.new_keep_words(q, cu, 100, 100, 0.0) is None
        # ... and not when it would outweigh q, k and v (here 8192 bytes against 3 * 160 * 2 * 64 * 2)
        ratio = be.KEEP_WORDS_MAX_INPUT_RATIO
        be.KEEP_WORDS_MAX_INPUT_RATIO = 8191.0 / (3 * 160 * 2 * 64 * 2)
        assert be.new_keep_words(q, cu, 100, 100, p) is None
        be.KEEP_WORDS_MAX_INPUT_RATIO = ratio
        assert ratio == 1.0 and be.new_keep_words(q, cu, 100, 100, p) is not None
    finally:
        be.KEEP_WORDS_MAX_BYTES = old
    torch.cuda.synchronize()


def test_element_offsets_beyond_int32():
    """A packed qkv tensor of 2.2e9 elements (4.4 GB): the last sequences live at element offsets above 2^31, which the
    kernels must address with 64-bit arithmetic.  Forward and backward of the first and the last sequence are compared
    with the oracle; the others only have to be finite."""
    H, D, N, B = 16, 128, 1024, 350
    assert B * N * 3 * H * D > 2 ** 31
    g = torch.Generator(device="cuda").manual_seed(5)
    qkv = torch.randn(B * N, 3, H, D, device="cuda", dtype=torch.float16, generator=g).requires_grad_()
    do = torch.randn(B * N, H, D, device="cuda", dtype=torch.float16, generator=g)
    cu = torch.arange(0, (B + 1) * N, N, dtype=torch.int32, device="cuda")
    from flash_attn import flash_attn_interface as fi
    out = fi.flash_attn_unpadded_qkvpacked_func(qkv, cu, N, 0.0, None, True)
    out.backward(do)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out).all()) and bool(torch.isfinite(qkv.grad).all())
    cu1 = _cu([N], "cpu")
    for b in (0, B - 1):
        sl = slice(b * N, (b + 1) * N)
        q, k, v = (qkv[sl, i].detach().cpu() for i in range(3))
        ref = orc.varlen_attention(q, k, v, cu1, cu1, None, True, dout=do[sl].cpu())
        half = half_attention(q.cuda(), k.cuda(), v.cuda(), [0, N], [0, N], D ** -0.5, True, dout=do[sl])
        ours = {"out": out[sl].detach(), "dq": qkv.grad[sl, 0], "dk": qkv.grad[sl, 1], "dv": qkv.grad[sl, 2]}
        check_against_oracle(ours, ref, half, torch.float16, what="sequence %d of %d" % (b, B))


@pytest.mark.parametrize("causal", [False, True])
def test_sequence_of_64k_tokens(causal):
    """One sequence of 65536 tokens (the longest the reference advertises, README.md:68): 512 query tiles and 1024 key
    tiles per head, far more than any other test walks.  The N x N closed form does not fit the oracle's way of working,
    so it is evaluated in fp32 on the GPU in row chunks (exact lse and out for every row), and the gradients are checked
    on sampled rows (dq) and sampled key columns (dk, dv) from the explicit formulas dV = P^T dO, dS = P o (dP - D),
    dQ = scale dS K, dK = scale dS^T Q.  Tolerances: a few fp16 roundings of values of order one."""
    from flash_attn import flash_attn_gfx950 as be
    N, H, D = 65536, 2, 64
    scale = D ** -0.5
    g = torch.Generator(device="cuda").manual_seed(11)
    qkv = torch.randn(N, 3, H, D, device="cuda", dtype=torch.float16, generator=g)
    do = torch.randn(N, H, D, device="cuda", dtype=torch.float16, generator=g)
    cu = torch.tensor([0, N], dtype=torch.int32, device="cuda")
    out, lse = be.fwd(qkv[:, 0], qkv[:, 1], qkv[:, 2], cu, cu, N, N, 0.0, scale, False, causal, False, None)
    grad = torch.empty_like(qkv)
    be.bwd(do, qkv[:, 0], qkv[:, 1], qkv[:, 2], out, lse, grad[:, 0], grad[:, 1], grad[:, 2], cu, cu, N, N, 0.0, scale,
           False, causal, None)
    torch.cuda.synchronize()
    q, k, v = (qkv[:, i].float().transpose(0, 1) for i in range(3))             # (H, N, D)
    dof = do.float().transpose(0, 1)
    pos = torch.arange(N, device="cuda")
    lse_ref = torch.empty(H, N, device="cuda")
    out_ref = torch.empty(H, N, D, device="cuda")
    for r0 in range(0, N, 4096):
        sc = torch.einsum("hqd,hkd->hqk", q[:, r0:r0 + 4096], k) * scale
        if causal:
            sc = sc.masked_fill(pos[None, None, :] > pos[None, r0:r0 + 4096, None], float("-inf"))
        lse_ref[:, r0:r0 + 4096] = torch.logsumexp(sc, -1)
        out_ref[:, r0:r0 + 4096] = torch.einsum("hqk,hkd->hqd", torch.exp(sc - lse_ref[:, r0:r0 + 4096, None]), v)
        del sc
    assert (lse[0, :, :N] - lse_ref).abs().max() < 1e-3
    assert (out.float().transpose(0, 1) - out_ref).abs().max() < 2e-3
    dsum = (dof * out_ref).sum(-1)                                             # D_i = rowsum(dO o O)
    gsel = torch.Generator().manual_seed(3)
    rows = torch.cat([torch.tensor([0, 1, 127, 128, N - 1]), torch.randint(0, N, (251,), generator=gsel)]).cuda()
    cols = torch.cat([torch.tensor([0, 63, 64, N - 2, N - 1]), torch.randint(0, N, (251,), generator=gsel)]).cuda()
    # sampled query rows against every key
    sc = torch.einsum("hqd,hkd->hqk", q[:, rows], k) * scale
    if causal:
        sc = sc.masked_fill(pos[None, None, :] > rows[None, :, None], float("-inf"))
    pr = torch.exp(sc - lse_ref[:, rows, None])
    ds = pr * (torch.einsum("hqd,hkd->hqk", dof[:, rows], v) - dsum[:, rows, None])
    dq_ref = scale * torch.einsum("hqk,hkd->hqd", ds, k)
    assert (grad[rows, 0].float().transpose(0, 1) - dq_ref).abs().max() < 4e-3
    del sc, pr, ds
    # every query row against sampled key columns
    sc = torch.einsum("hqd,hkd->hqk", q, k[:, cols]) * scale
    if causal:
        sc = sc.masked_fill(cols[None, None, :] > pos[None, :, None], float("-inf"))
    pr = torch.exp(sc - lse_ref[:, :, None])
    dv_ref = torch.einsum("hqk,hqd->hkd", pr, dof)
    ds = pr * (torch.einsum("hqd,hkd->hqk", dof, v[:, cols]) - dsum[:, :, None])
    dk_ref = scale * torch.einsum("hqk,hqd->hkd", ds, q)
    tol = lambda ref: 4e-3 + 2.0 ** -10 * ref.abs().max().item()
    assert (grad[cols, 2].float().transpose(0, 1) - dv_ref).abs().max() < tol(dv_ref)
    assert (grad[cols, 1].float().transpose(0, 1) - dk_ref).abs().max() < tol(dk_ref)


def test_parity_random_shapes_sweep(tile_shape):
    """Twenty-four seeded random cases over what the parametrised tests hold fixed: batch size, ragged query and key
    lengths (self- and cross-attention, empty key sides excluded), heads, head dim, dtype, causal, packing, scale."""
    rng = np.random.default_rng(2024)
    for case in range(24):
        D = int(rng.choice([16, 32, 64, 128]))
        dtype = torch.float16 if rng.integers(2) else torch.bfloat16
        B, H = int(rng.integers(1, 5)), int(rng.integers(1, 4))
        causal = bool(rng.integers(2))
        cross = bool(rng.integers(2)) and not causal
        top = int(rng.choice([40, 150, 300, 520]))
        lens_q = [int(x) for x in rng.integers(1, top + 1, B)]
        lens_k = [int(x) for x in rng.integers(1, top + 1, B)] if cross else list(lens_q)
        packing = "kv" if cross else str(rng.choice(["qkv", "kv", "sep"]))
        scale = None if rng.integers(2) else float(rng.uniform(0.05, 0.5))
        print("case %d: D=%d %s B=%d H=%d causal=%s q=%s k=%s %s scale=%s" % (case, D, dtype, B, H, causal, lens_q, lens_k,
                                                                            packing, scale), flush=True)
        _parity_case(lens_q, lens_k, H, D, dtype, causal, packing=packing, seed=100 + case, scale=scale)


# ------------------------------------------------------------------------------------------------
# attention bias: ALiBi slopes (an extension; the reference's README lists attention bias as planned)
# ------------------------------------------------------------------------------------------------
def _alibi_slopes(H):
    """the geometric sequence of the ALiBi paper for a power-of-two head count, cut to H heads"""
    n = 1 << max(1, (H - 1).bit_length())
    return torch.tensor([2.0 ** (-8.0 * (i + 1) / n) for i in range(H)], dtype=torch.float32)


def test_alibi_random_shapes_sweep():
    """Sixteen seeded cases with per-head ALiBi slopes: every head dim, both dtypes, causal and not, ragged self- and
    cross-attention lengths, all packings, with and without dropout; out, lse, dq, dk, dv and the returned probabilities
    against the closed form with the bias added to the scaled scores."""
    rng = np.random.default_rng(909)
    for case in range(16):
        D = int(rng.choice([16, 32, 64, 128]))
        dtype = torch.float16 if rng.integers(2) else torch.bfloat16
        B, H = int(rng.integers(1, 4)), int(rng.integers(1, 5))
        causal = bool(rng.integers(2))
        cross = bool(rng.integers(2)) and not causal
        top = int(rng.choice([40, 150, 300, 520]))
        lens_q = [int(x) for x in rng.integers(1, top + 1, B)]
        lens_k = [int(x) for x in rng.integers(1, top + 1, B)] if cross else list(lens_q)
        packing = "kv" if cross else str(rng.choice(["qkv", "kv", "sep"]))
        p = float(rng.choice([0.0, 0.0, 0.15]))
        slopes = _alibi_slopes(H) * float(rng.choice([1.0, 4.0]))
        what = "case %d: D=%d %s B=%d H=%d causal=%s q=%s k=%s %s p=%.2f" % (case, D, dtype, B, H, causal, lens_q, lens_k,
                                                                          packing, p)
        print(what, flush=True)
        q, k, v, do = _inputs(lens_q, lens_k, H, D, dtype, 700 + case)
        cu_q, cu_k = _cu(lens_q, "cpu"), _cu(lens_k, "cpu")
        sc = D ** -0.5
        torch.manual_seed(case)
        seed, offset = _gen_state()
        ours = run_ours(q, k, v, do, cu_q, cu_k, max(lens_q), max(lens_k), p, None, causal, packing, probs=True,
                        alibi_slopes=slopes.cuda())
        masks = None
        if p > 0:
            masks = [torch.tensor(np.stack([orc.dropout_keep_mask(seed, offset, b * H + h, lens_q[b], lens_k[b], p)
                                            for h in range(H)])) for b in range(B)]
        ref = orc.varlen_attention(q, k, v, cu_q, cu_k, sc, causal, p_dropout=p, keep_mask=masks, dout=do,
                                   alibi_slopes=slopes)
        half = half_attention(q.cuda(), k.cuda(), v.cuda(), cu_q.tolist(), cu_k.tolist(), sc, causal, masks, p, dout=do.cuda(),
                              alibi_slopes=slopes)
        check_against_oracle(ours, ref, half, dtype, what=what)
        for b in range(B):
            Lq, Lk = lens_q[b], lens_k[b]
            check_lse(ours["lse"][b, :, :Lq].cpu(), ref["lse"][b], half["lse"][b], dtype, what)
            probs = ours["S_dmask"][b, :, :Lq, :Lk].float().cpu()
            assert (probs.abs() - ref["probs"][b]).abs().max().item() < (2e-3 if dtype == torch.float16 else 1e-2), what


def test_alibi_decode_shape_with_key_split():
    """A few query rows against thousands of keys with ALiBi slopes: the key-split forward and the key-split dQ kernel
    (partial results per key range, merged by a second launch) see the bias through the same scores."""
    lens_q, lens_k, H, D = [3, 1], [4100, 2900], 4, 64
    slopes = _alibi_slopes(H) * 0.25
    q, k, v, do = _inputs(lens_q, lens_k, H, D, torch.float16, 77)
    cu_q, cu_k = _cu(lens_q, "cpu"), _cu(lens_k, "cpu")
    ours = run_ours(q, k, v, do, cu_q, cu_k, max(lens_q), max(lens_k), 0.0, None, False, "kv", probs=True,
                    alibi_slopes=slopes.cuda())
    ref = orc.varlen_attention(q, k, v, cu_q, cu_k, None, False, dout=do, alibi_slopes=slopes)
    half = half_attention(q.cuda(), k.cuda(), v.cuda(), cu_q.tolist(), cu_k.tolist(), D ** -0.5, False, dout=do.cuda(),
                          alibi_slopes=slopes)
    check_against_oracle(ours, ref, half, torch.float16, what="alibi decode shape")
    for b, L in enumerate(lens_q):
        assert (ours["lse"][b, :, :L].cpu() - ref["lse"][b]).abs().max() <= LSE_TOL[torch.float16]
    # the bias matters here: without it the result is visibly different
    plain = orc.varlen_attention(q, k, v, cu_q, cu_k, None, False)
    assert (plain["out"] - ref["out"]).abs().max() > 0.05


def test_alibi_headline_shape_and_errors():
    """ALiBi at the headline shape (all tiles full, no masking code in the way) against the fp32 closed form on the GPU
    for one (batch, head) pair, slope 0 == no bias bit for bit, the refusals (slopes of the wrong shape / dtype / device),
    and the same slopes under a block layout that lists every block."""
    from flash_attn import flash_attn_interface as fi
    from flash_attn.flash_blocksparse_attn_interface import convert_blockmask
    from flash_attn import flash_attn_gfx950 as be
    B, H, D, N = 2, 4, 64, 2048
    g = torch.Generator(device="cuda").manual_seed(2)
    qkv = torch.randn(B * N, 3, H, D, device="cuda", dtype=torch.float16, generator=g).requires_grad_()
    do = torch.randn(B * N, H, D, device="cuda", dtype=torch.float16, generator=g)
    cu = _cu([N] * B)
    slopes = _alibi_slopes(H).cuda()
    out = fi.flash_attn_unpadded_qkvpacked_func(qkv, cu, N, 0.0, causal=True, alibi_slopes=slopes)
    out.backward(do)
    torch.cuda.synchronize()
    b, h = 1, 2
    sl = slice(b * N, (b + 1) * N)
    q, k, v = (qkv[sl, i, h].detach().float()[:, None] for i in range(3))
    ref = orc.varlen_attention(q, k, v, [0, N], [0, N], None, True, dout=do[sl, h].float()[:, None],
                               alibi_slopes=slopes[h:h + 1].cpu())
    assert (out[sl, h].detach().float() - ref["out"][:, 0]).abs().max() < 2e-3
    for i, name in enumerate(("dq", "dk", "dv")):
        assert (qkv.grad[sl, i, h].float() - ref[name][:, 0]).abs().max() < 4e-3, name
    plain = fi.flash_attn_unpadded_qkvpacked_func(qkv.detach(), cu, N, 0.0, causal=True)
    zero = fi.flash_attn_unpadded_qkvpacked_func(qkv.detach(), cu, N, 0.0, causal=True, alibi_slopes=torch.zeros_like(slopes))
    assert (zero.float() - plain.float()).abs().max() < 1e-3  # different kernel variants, same mathematics
    for bad in (slopes[:3], slopes.double(), slopes.cpu(), slopes[None]):
        with pytest.raises(RuntimeError):
            fi.flash_attn_unpadded_qkvpacked_func(qkv.detach(), cu, N, 0.0, alibi_slopes=bad)
    # with a block layout that lists every block the slopes give what the dense kernels give (other tile shapes: within rounding)
    sq_r, sk_r = be.round_seqlens(D, N, N, True)
    bm = convert_blockmask(torch.ones(sq_r // 16, sk_r // 256, device="cuda"), causal=True)
    q3 = qkv.detach()
    o_sparse = be.fwd_block(q3[:, 0], q3[:, 1], q3[:, 2], cu, cu, bm, N, N, 0.0, D ** -0.5, True, False, alibi_slopes=slopes)[0]
    assert (o_sparse.float() - out.detach().float()).abs().max() < 1e-3


# ------------------------------------------------------------------------------------------------
# attention bias as a tensor (extension: the reference only plans it, README.md:50)
# ------------------------------------------------------------------------------------------------
def _random_bias(rng, shape, dtype, minus_inf=0.0):
    g = torch.Generator().manual_seed(int(rng.integers(1 << 30)))
    bias = (torch.randn(shape, generator=g) * 1.5).to(dtype)
    if minus_inf > 0:  # masked entries, never a whole row (key 0 stays)
        drop = torch.rand(shape, generator=g) < minus_inf
        drop[..., 0] = False
        bias = bias.masked_fill(drop, float("-inf"))
    return bias


def test_attn_bias_random_shapes_sweep():
    """Sixteen seeded random cases with a bias tensor added to the scaled scores: head dims, dtypes, ragged self- and
    cross-attention, causal or not, the bias per (batch, head), shared over the batch or over everything, with and
    without -inf entries, key extents that are and are not multiples of 8 (the latter make the binding pad a copy):
    out, lse, dq, dk, dv and the bias gradient against the oracle (closed form + autograd, itself pinned against
    torch's scaled_dot_product_attention with the same tensor as float mask)."""
    rng = np.random.default_rng(4242)
    for case in range(16):
        D = int(rng.choice([16, 32, 64, 128]))
        dtype = torch.float16 if rng.integers(2) else torch.bfloat16
        B, H = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        causal = bool(rng.integers(2))
        cross = bool(rng.integers(2)) and not causal
        top = int(rng.choice([40, 150, 330]))
        lens_q = [int(x) for x in rng.integers(1, top + 1, B)]
        lens_k = [int(x) for x in rng.integers(1, top + 1, B)] if cross else list(lens_q)
        mq, mk = max(lens_q), max(lens_k)
        if rng.integers(2):
            mk8 = (mk + 7) // 8 * 8   # a bias whose rows the kernels can read as they are
        else:
            mk8 = mk
        bshape = ((B, H), (1, H), (1, 1), (B, 1))[int(rng.integers(4))] + (mq, mk8)
        bias = _random_bias(rng, bshape, dtype, minus_inf=float(rng.choice([0.0, 0.2])))
        packing = "kv" if cross else str(rng.choice(["qkv", "sep"]))
        print("case %d: D=%d %s B=%d H=%d causal=%s q=%s k=%s bias%s %s" % (case, D, dtype, B, H, causal, lens_q, lens_k,
                                                                            tuple(bshape), packing), flush=True)
        q, k, v, do = _inputs(lens_q, lens_k, H, D, dtype, 900 + case)
        cu_q, cu_k = _cu(lens_q, "cpu"), _cu(lens_k, "cpu")
        ours = run_ours(q, k, v, do, cu_q, cu_k, mq, mk, 0.0, None, causal, packing, probs=True, attn_bias=bias)
        ref = orc.varlen_attention(q, k, v, cu_q, cu_k, None, causal, dout=do, attn_bias=bias)
        half = half_attention(q.cuda(), k.cuda(), v.cuda(), cu_q.tolist(), cu_k.tolist(), D ** -0.5, causal, dout=do.cuda(),
                              attn_bias=bias.cuda())
        what = "attn_bias sweep case %d" % case
        check_against_oracle(ours, ref, half, dtype, names=("out", "dq", "dk", "dv", "dbias"), what=what)
        for b, L in enumerate(lens_q):
            check_lse(ours["lse"][b, :, :L].cpu(), ref["lse"][b], half["lse"][b], dtype, what)
        # the probabilities returned for testing carry the bias too
        S = ours["S_dmask"].float().cpu()
        for b, (Lq, Lk) in enumerate(zip(lens_q, lens_k)):
            assert (S[b, :, :Lq, :Lk] - ref["probs"][b]).abs().max() < (2e-3 if dtype == torch.float16 else 1.6e-2)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_bias_grad_reduce_sums_in_fp32_and_rounds_once(dtype):
    """fa_bias_grad_reduce against float64 sums of the same slices: over the batch, over the heads, over both; key extents
    that are and are not multiples of 8, an output whose rows are not 16-byte aligned (scalar stores), a view into a larger
    tensor whose surroundings must stay untouched.  The fp32 running sum and the one rounding bound the error; two calls
    give the same bits."""
    from flash_attn import flash_attn_gfx950 as be
    g = torch.Generator(device="cuda").manual_seed(5)
    eps = 2.0 ** -11 if dtype == torch.float16 else 2.0 ** -8
    for B, H, rows, cols, out_cols in ((5, 3, 37, 64, 64), (2, 4, 16, 45, 53), (9, 1, 130, 200, 200), (1, 6, 8, 7, 7)):
        cols8 = (cols + 7) // 8 * 8
        dbias = (torch.randn(B, H, rows, cols8, device="cuda", generator=g) * 3).to(dtype)
        for sum_batch, sum_heads in ((True, False), (False, True), (True, True)):
            ob, oh = (1 if sum_batch else B), (1 if sum_heads else H)
            full = torch.full((ob, oh, rows + 3, out_cols + 2), 7.0, device="cuda", dtype=dtype)
            view = full[:, :, :rows, :cols]
            be.reduce_bias_grad(dbias, view, sum_batch, sum_heads)
            ref = dbias[..., :cols].double()
            mag = dbias[..., :cols].double().abs()
            if sum_batch:
                ref, mag = ref.sum(0, keepdim=True), mag.sum(0, keepdim=True)
            if sum_heads:
                ref, mag = ref.sum(1, keepdim=True), mag.sum(1, keepdim=True)
            err = (view.double() - ref).abs()
            assert bool((err <= eps * ref.abs() * 1.001 + 2.0 ** -22 * mag).all()), (B, H, rows, cols, sum_batch, sum_heads)
            assert bool((full[:, :, rows:] == 7).all()) and bool((full[:, :, :, cols:] == 7).all())
            again = torch.empty_like(full)[:, :, :rows, :cols]
            be.reduce_bias_grad(dbias, again, sum_batch, sum_heads)
            assert torch.equal(again, view)
    with pytest.raises(RuntimeError):
        be.reduce_bias_grad(dbias, torch.empty(2, 6, 8, 7, device="cuda", dtype=dtype), True, False)  # wrong batch extent


@pytest.mark.parametrize("D,dtype,causal", [(64, torch.float16, False), (128, torch.bfloat16, True), (32, torch.float16, True)])
def test_attn_bias_with_dropout(D, dtype, causal, dropout_path):
    """bias and dropout together (the backward reading the forward's keep words, or drawing again): the mask is the defined
    one, out / gradients / bias gradient equal the closed form with that mask."""
    lens, H, p = [150, 77, 200], 2, 0.2
    rng = np.random.default_rng(7)
    bias = _random_bias(rng, (1, H, max(lens), max(lens)), dtype)
    q, k, v, do = _inputs(lens, lens, H, D, dtype, 31)
    cu = _cu(lens, "cpu")
    torch.manual_seed(123)
    seed, offset = _gen_state()
    ours = run_ours(q, k, v, do, cu, cu, max(lens), max(lens), p, None, causal, "qkv", probs=True, attn_bias=bias)
    S = ours["S_dmask"].cpu()
    masks = []
    for b, L in enumerate(lens):
        mb = np.stack([orc.dropout_keep_mask(seed, offset, b * H + h, L, L, p) for h in range(H)])
        masks.append(torch.tensor(mb))
        valid = orc._score_mask(L, L, causal, None)
        assert torch.equal(torch.signbit(S[b, :, :L, :L])[:, valid], ~masks[b][:, valid])
    ref = orc.varlen_attention(q, k, v, cu, cu, None, causal, p_dropout=p, keep_mask=masks, dout=do, attn_bias=bias)
    half = half_attention(q.cuda(), k.cuda(), v.cuda(), cu.tolist(), cu.tolist(), D ** -0.5, causal, masks, p, dout=do.cuda(),
                          attn_bias=bias.cuda())
    check_against_oracle(ours, ref, half, dtype, names=("out", "dq", "dk", "dv", "dbias"), what="attn_bias + dropout D=%d" % D)


def test_attn_bias_special_cases_and_errors():
    """A bias of zeros changes nothing (bit for bit against the kernels without bias at d = 128, where both run the same
    tile shapes; within rounding elsewhere); 0 / -inf above the diagonal is the causal mask; a row whose bias is -inf
    everywhere gives out = 0 and lse = -inf; the slopes' bias as a tensor equals alibi_slopes; argument errors."""
    from flash_attn import flash_attn_interface as fi
    B, H, D, N = 2, 3, 64, 200
    torch.manual_seed(5)
    qkv = torch.randn(B * N, 3, H, D, device="cuda", dtype=torch.float16)
    cu = torch.arange(0, (B + 1) * N, N, dtype=torch.int32, device="cuda")
    plain = fi.flash_attn_unpadded_qkvpacked_func(qkv, cu, N, 0.0)
    zero = fi.flash_attn_unpadded_qkvpacked_func(qkv, cu, N, 0.0, attn_bias=torch.zeros(1, 1, N, N, device="cuda", dtype=torch.float16))
    assert (plain.float() - zero.float()).abs().max() < 2e-3
    tri = torch.zeros(1, 1, N, N, device="cuda", dtype=torch.float16).masked_fill(
        torch.triu(torch.ones(N, N, dtype=torch.bool, device="cuda"), 1), float("-inf"))
    a = fi.flash_attn_unpadded_qkvpacked_func(qkv, cu, N, 0.0, attn_bias=tri)
    c = fi.flash_attn_unpadded_qkvpacked_func(qkv, cu, N, 0.0, causal=True)
    assert (a.float() - c.float()).abs().max() < 2e-3
    # a fully masked row
    dead = torch.zeros(1, 1, N, N, device="cuda", dtype=torch.float16)
    dead[0, 0, 17, :] = float("-inf")
    out, lse, _ = fi.flash_attn_unpadded_qkvpacked_func(qkv, cu, N, 0.0, return_attn_probs=True, attn_bias=dead)
    assert torch.equal(out[17], torch.zeros_like(out[17])) and torch.isinf(lse[0, :, 17]).all() and (lse[0, :, 17] < 0).all()
    assert torch.isfinite(out).all()
    # ALiBi written out as a tensor
    slopes = _alibi_slopes(H).cuda()
    al = fi.flash_attn_unpadded_qkvpacked_func(qkv, cu, N, 0.0, alibi_slopes=slopes)
    tb = orc.alibi_bias(slopes.cpu(), N, N)[None].to(torch.float16).cuda()
    at = fi.flash_attn_unpadded_qkvpacked_func(qkv, cu, N, 0.0, attn_bias=tb)
    assert (al.float() - at.float()).abs().max() < 4e-3   # the tensor's entries are rounded to fp16, the slopes' are not
    # errors
    with pytest.raises(RuntimeError, match="attn_bias"):
        fi.flash_attn_unpadded_qkvpacked_func(qkv, cu, N, 0.0, attn_bias=torch.zeros(1, 1, N, N - 1, device="cuda", dtype=torch.float16))
    with pytest.raises(RuntimeError, match="attn_bias"):
        fi.flash_attn_unpadded_qkvpacked_func(qkv, cu, N, 0.0, attn_bias=torch.zeros(1, 1, N, N, device="cuda", dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="together"):
        fi.flash_attn_unpadded_qkvpacked_func(qkv, cu, N, 0.0, alibi_slopes=slopes,
                                              attn_bias=torch.zeros(1, 1, N, N, device="cuda", dtype=torch.float16))


def test_attn_bias_full_size_against_pytorch_and_decode_shape():
    """Headline-sized check (B=2, H=12, d=64, N=2048, a bias per head shared over the batch) against PyTorch's
    scaled_dot_product_attention in fp32 with the same tensor as mask, forward and backward, and a decode-shaped call
    (one query row per sequence over thousands of keys: the key-split kernels) against the oracle."""
    B, H, D, N = 2, 12, 64, 2048
    torch.manual_seed(9)
    qkv = torch.randn(B * N, 3, H, D, device="cuda", dtype=torch.float16, requires_grad=True)
    bias = (torch.randn(1, H, N, N, device="cuda") * 1.5).to(torch.float16).requires_grad_()
    cu = torch.arange(0, (B + 1) * N, N, dtype=torch.int32, device="cuda")
    from flash_attn import flash_attn_interface as fi
    out = fi.flash_attn_unpadded_qkvpacked_func(qkv, cu, N, 0.0, attn_bias=bias)
    do = torch.randn_like(out)
    out.backward(do)
    q32 = qkv.detach().float().view(B, N, 3, H, D).permute(2, 0, 3, 1, 4).clone().requires_grad_()
    b32 = bias.detach().float().clone().requires_grad_()
    ref = torch.nn.functional.scaled_dot_product_attention(q32[0], q32[1], q32[2], attn_mask=b32)
    ref.backward(do.float().view(B, N, H, D).permute(0, 2, 1, 3))
    assert (out.float().view(B, N, H, D).permute(0, 2, 1, 3) - ref).abs().max() < 4e-3
    g = qkv.grad.float().view(B, N, 3, H, D).permute(2, 0, 3, 1, 4)
    assert (g - q32.grad).abs().max() < 8e-3
    assert (bias.grad.float() - b32.grad).abs().max() < 8e-3
    # decode shape
    lens_q, lens_k = [1, 1], [3000, 1777]
    q, k, v, do = _inputs(lens_q, lens_k, 4, 64, torch.float16, 77)
    rng = np.random.default_rng(3)
    db = _random_bias(rng, (2, 4, 1, 3000), torch.float16)
    cu_q, cu_k = _cu(lens_q, "cpu"), _cu(lens_k, "cpu")
    ours = run_ours(q, k, v, do, cu_q, cu_k, 1, 3000, 0.0, None, False, "kv", attn_bias=db)
    ref = orc.varlen_attention(q, k, v, cu_q, cu_k, None, False, dout=do, attn_bias=db)
    half = half_attention(q.cuda(), k.cuda(), v.cuda(), cu_q.tolist(), cu_k.tolist(), 64 ** -0.5, False, dout=do.cuda(),
                          attn_bias=db.cuda())
    check_against_oracle(ours, ref, half, torch.float16, names=("out", "dq", "dk", "dv", "dbias"), what="attn_bias decode shape")


# ------------------------------------------------------------------------------------------------
# block-sparse
# ------------------------------------------------------------------------------------------------
def _layout(nrow, ncol, density, seed):
    g = torch.Generator().manual_seed(seed)
    band = (torch.arange(nrow)[:, None] // 16 - torch.arange(ncol)[None, :]).abs() <= 0
    return (band | (torch.rand(nrow, ncol, generator=g) < density))


@pytest.mark.parametrize("D,N,p", [(64, 512, 0.0), (32, 700, 0.0), (16, 300, 0.0), (64, 512, 0.2)])
def test_blocksparse_parity(D, N, p):
    from flash_attn.flash_blocksparse_attn_interface import flash_blocksparse_attn_func
    from flash_attn import flash_attn_gfx950 as be
    H, lens = 2, [N, N - 37]
    sq_r, sk_r = be.round_seqlens(D, N, N, True)
    layout = _layout(sq_r // 16, sk_r // 256, 0.3, N)
    layout[3] = False  # a row block with no active tile: its rows must come out as zeros
    q, k, v, do = _inputs(lens, lens, H, D, torch.float16, N)
    cu = _cu(lens, "cpu")
    qkv = torch.stack([q, k, v], 1).cuda().requires_grad_()
    torch.manual_seed(5)
    seed, offset = _gen_state()
    ctx, S, lse = flash_blocksparse_attn_func(qkv, cu.cuda(), layout.cuda(), p, N, None, False, True)
    ctx.backward(do.cuda())
    torch.cuda.synchronize()
    masks = None
    if p > 0:
        masks = [torch.tensor(np.stack([orc.dropout_keep_mask(seed, offset, b * H + h, L, L, p) for h in range(H)]))
                 for b, L in enumerate(lens)]
    ref = orc.varlen_attention(q, k, v, cu, cu, None, False, p_dropout=p, keep_mask=masks, layout=layout.numpy(), dout=do)
    half = half_attention(q.cuda(), k.cuda(), v.cuda(), cu.tolist(), cu.tolist(), D ** -0.5, False, masks, p,
                          layout=layout.numpy(), dout=do.cuda())
    ours = {"out": ctx.detach(), "dq": qkv.grad[:, 0], "dk": qkv.grad[:, 1], "dv": qkv.grad[:, 2]}
    check_against_oracle(ours, ref, half, torch.float16, what="blocksparse D%d N%d" % (D, N))
    assert ctx[48:64].abs().max() == 0 and torch.isinf(lse[0, :, 48:64]).all()
    assert qkv.grad[48:64, 0].abs().max() == 0
    # probabilities are zero on inactive blocks
    full = orc.expand_block_layout(layout.numpy(), lens[0], lens[0])
    assert S[0, :, :lens[0], :lens[0]].cpu()[:, ~full].abs().max() == 0


def test_blocksparse_more_than_64_key_blocks():
    """The kernels keep the activity bits of 64 key blocks (16384 keys) in registers and reload them beyond: a key side of
    66 blocks with active blocks on both sides of the boundary, through the raw entry points (separate q and k lengths)."""
    from flash_attn import flash_attn_gfx950 as be
    from flash_attn.flash_blocksparse_attn_interface import convert_blockmask
    H, D, lens_q, lens_k = 2, 32, [200, 120], [16700, 16500]
    sq_r, sk_r = be.round_seqlens(D, max(lens_q), max(lens_k), True)
    layout = torch.rand(sq_r // 16, sk_r // 256, generator=torch.Generator().manual_seed(3)) < 0.1
    layout[:, 63:66] = torch.rand(sq_r // 16, 3, generator=torch.Generator().manual_seed(4)) < 0.5
    layout[5] = False
    layout[5, 65] = True        # a row block whose only keys lie beyond the boundary
    q, k, v, do = _inputs(lens_q, lens_k, H, D, torch.float16, 9)
    cu_q, cu_k = _cu(lens_q, "cpu"), _cu(lens_k, "cpu")
    qc, kc, vc, doc = (x.cuda() for x in (q, k, v, do))
    bm = convert_blockmask(layout.cuda(), causal=False)
    out, lse = be.fwd_block(qc, kc, vc, cu_q.cuda(), cu_k.cuda(), bm, max(lens_q), max(lens_k), 0.0, D ** -0.5, False, False, None)
    dq, dk, dv = torch.empty_like(qc), torch.empty_like(kc), torch.empty_like(vc)
    be.bwd_block(doc, qc, kc, vc, out, lse, dq, dk, dv, cu_q.cuda(), cu_k.cuda(), bm, max(lens_q), max(lens_k), 0.0, D ** -0.5,
                 False, None)
    torch.cuda.synchronize()
    ref = orc.varlen_attention(q, k, v, cu_q, cu_k, None, False, layout=layout.numpy(), dout=do)
    half = half_attention(qc, kc, vc, cu_q.tolist(), cu_k.tolist(), D ** -0.5, False, layout=layout.numpy(), dout=doc)
    check_against_oracle({"out": out, "dq": dq, "dk": dk, "dv": dv}, ref, half, torch.float16, what="blocksparse 66 key blocks")


def test_blocksparse_random_layouts_sweep():
    """Ten seeded random block-sparse cases: densities from 5 % to 90 % (with and without the diagonal band), ragged
    lengths up to 2100 (several activity words per key block on the backward side), every head dim, both dtypes, dropout."""
    from flash_attn.flash_blocksparse_attn_interface import flash_blocksparse_attn_func
    from flash_attn import flash_attn_gfx950 as be
    rng = np.random.default_rng(31)
    for case in range(10):
        D = int(rng.choice([16, 32, 64, 128]))
        dtype = torch.float16 if rng.integers(2) else torch.bfloat16
        B, H = int(rng.integers(1, 4)), int(rng.integers(1, 3))
        N = int(rng.choice([100, 300, 520, 1100, 2100]))
        lens = [N] + [int(x) for x in rng.integers(max(1, N // 3), N + 1, B - 1)]
        dens = float(rng.choice([0.05, 0.2, 0.5, 0.9]))
        p = float(rng.choice([0.0, 0.0, 0.2]))
        sq_r, sk_r = be.round_seqlens(D, N, N, True)
        layout = torch.rand(sq_r // 16, sk_r // 256, generator=torch.Generator().manual_seed(case)) < dens
        if rng.integers(2):
            layout |= (torch.arange(sq_r // 16)[:, None] // 16) == torch.arange(sk_r // 256)[None, :]
        what = "case %d: D=%d %s B=%d H=%d lens=%s density %.2f p=%.1f" % (case, D, dtype, B, H, lens, dens, p)
        print(what, flush=True)
        q, k, v, do = _inputs(lens, lens, H, D, dtype, 3000 + case)
        cu = _cu(lens, "cpu")
        qkv = torch.stack([q, k, v], 1).cuda().requires_grad_()
        torch.manual_seed(case)
        seed, offset = _gen_state()
        ctx = flash_blocksparse_attn_func(qkv, cu.cuda(), layout.cuda(), p, N)
        ctx.backward(do.cuda())
        torch.cuda.synchronize()
        masks = None
        if p > 0:
            masks = [torch.tensor(np.stack([orc.dropout_keep_mask(seed, offset, b * H + h, L, L, p) for h in range(H)]))
                     for b, L in enumerate(lens)]
        ref = orc.varlen_attention(q, k, v, cu, cu, None, False, p_dropout=p, keep_mask=masks, layout=layout.numpy(), dout=do)
        half = half_attention(q.cuda(), k.cuda(), v.cuda(), cu.tolist(), cu.tolist(), D ** -0.5, False, masks, p,
                              layout=layout.numpy(), dout=do.cuda())
        ours = {"out": ctx.detach(), "dq": qkv.grad[:, 0], "dk": qkv.grad[:, 1], "dv": qkv.grad[:, 2]}
        check_against_oracle(ours, ref, half, dtype, what=what)


def _blocksparse_bias_case(case, D, dtype, H, lens, dens, p, causal, slopes, bias, what):
    """one block-sparse case with ALiBi slopes or a bias tensor through flash_blocksparse_attn_func, against the oracle"""
    from flash_attn.flash_blocksparse_attn_interface import flash_blocksparse_attn_func
    from flash_attn import flash_attn_gfx950 as be
    N = max(lens)
    sq_r, sk_r = be.round_seqlens(D, N, N, True)
    layout = torch.rand(sq_r // 16, sk_r // 256, generator=torch.Generator().manual_seed(100 + case)) < dens
    layout |= (torch.arange(sq_r // 16)[:, None] // 16) == torch.arange(sk_r // 256)[None, :]  # the diagonal band
    print(what, flush=True)
    q, k, v, do = _inputs(lens, lens, H, D, dtype, 5000 + case)
    cu = _cu(lens, "cpu")
    qkv = torch.stack([q, k, v], 1).cuda().requires_grad_()
    bias_g = bias.cuda().requires_grad_() if bias is not None else None
    torch.manual_seed(case)
    seed, offset = _gen_state()
    ctx = flash_blocksparse_attn_func(qkv, cu.cuda(), layout.cuda(), p, N, causal=causal,
                                      alibi_slopes=slopes.cuda() if slopes is not None else None, attn_bias=bias_g)
    ctx.backward(do.cuda())
    torch.cuda.synchronize()
    masks = None
    if p > 0:
        masks = [torch.tensor(np.stack([orc.dropout_keep_mask(seed, offset, b * H + h, L, L, p) for h in range(H)]))
                 for b, L in enumerate(lens)]
    ref = orc.varlen_attention(q, k, v, cu, cu, None, causal, p_dropout=p, keep_mask=masks, layout=layout.numpy(), dout=do,
                               alibi_slopes=slopes, attn_bias=bias)
    half = half_attention(q.cuda(), k.cuda(), v.cuda(), cu.tolist(), cu.tolist(), D ** -0.5, causal, masks, p,
                          layout=layout.numpy(), dout=do.cuda(), alibi_slopes=slopes,
                          attn_bias=bias.cuda() if bias is not None else None)
    ours = {"out": ctx.detach(), "dq": qkv.grad[:, 0], "dk": qkv.grad[:, 1], "dv": qkv.grad[:, 2]}
    names = ("out", "dq", "dk", "dv")
    if bias is not None:
        ours["dbias"] = bias_g.grad
        names += ("dbias",)
        # blocks the layout leaves out take no gradient
        dead = ~orc.expand_block_layout(layout.numpy(), N, N)
        assert bool((bias_g.grad[..., :N, :N].cpu()[..., dead] == 0).all()), what
    check_against_oracle(ours, ref, half, dtype, names=names, what=what)


def test_blocksparse_with_score_bias_sweep():
    """Twelve seeded random block-sparse cases with a score bias inside the active blocks: ALiBi slopes or a bias tensor
    (per (batch, head), shared over the batch, over everything; with -inf entries), every head dim, both dtypes, causal or
    not (causal: no row order, the packed tiles of the backward straddle the diagonal), ragged lengths, dropout - out, dq,
    dk, dv and the bias gradient against the oracle's closed form with the layout, the bias and the drawn mask."""
    rng = np.random.default_rng(77)
    for case in range(12):
        D = int(rng.choice([16, 32, 64, 128]))
        dtype = torch.float16 if rng.integers(2) else torch.bfloat16
        B, H = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        N = int(rng.choice([100, 300, 520, 1100]))
        lens = [N] + [int(x) for x in rng.integers(max(1, N // 3), N + 1, B - 1)]
        dens = float(rng.choice([0.1, 0.3, 0.6]))
        p = float(rng.choice([0.0, 0.0, 0.2]))
        causal = bool(rng.integers(2))
        kind = ("alibi", "tensor", "tensor")[int(rng.integers(3))]
        slopes = bias = None
        if kind == "alibi":
            slopes = _alibi_slopes(H) * 0.5
        else:
            bshape = ((B, H), (1, H), (1, 1))[int(rng.integers(3))] + (N, N if rng.integers(2) else (N + 7) // 8 * 8)
            bias = _random_bias(rng, bshape, dtype, minus_inf=float(rng.choice([0.0, 0.15])))
        what = "case %d: D=%d %s B=%d H=%d lens=%s density %.1f p=%.1f causal=%s %s%s" % (
            case, D, dtype, B, H, lens, dens, p, causal, kind, tuple(bias.shape) if bias is not None else "")
        _blocksparse_bias_case(case, D, dtype, H, lens, dens, p, causal, slopes, bias, what)


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("kind", ["alibi", "tensor"])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("p", [0.0, 0.2])
def test_blocksparse_with_score_bias_variants(D, kind, causal, p):
    """every block-sparse kernel variant with a score bias at the two large head dims: (ALiBi, tensor) x (causal or not) x
    (dropout or not), ragged batch of two, a bias shared over the batch (its gradient is the sum of both entries')"""
    H, lens, dtype = 2, [520, 300], torch.float16
    slopes = bias = None
    if kind == "alibi":
        slopes = _alibi_slopes(H) * 0.5
    else:
        bias = _random_bias(np.random.default_rng(D + 3), (1, H, 520, 520), dtype)
    what = "variant D=%d %s causal=%s p=%.1f" % (D, kind, causal, p)
    _blocksparse_bias_case(D + 2 * causal + (p > 0), D, dtype, H, lens, 0.3, p, causal, slopes, bias, what)


@pytest.mark.parametrize("D,N,dtype", [(64, 1280, torch.float16), (32, 300, torch.bfloat16), (128, 700, torch.float16)])
def test_blocksparse_row_order(D, N, dtype):
    """the 16-row blocks a workgroup owns may be any eight of a caller's order: no order, the greedy grouping the autograd
    functions use, and a random permutation give the same results within rounding, each within the parity bar"""
    from flash_attn import flash_attn_gfx950 as be
    from flash_attn.flash_blocksparse_attn_interface import convert_blockmask
    H, lens = 2, [N, N - 150, 20]
    sq_r, sk_r = be.round_seqlens(D, N, N, True)
    layout = _layout(sq_r // 16, sk_r // 256, 0.25, N + D)
    layout[5] = False
    q, k, v, do = _inputs(lens, lens, H, D, dtype, N)
    cu = _cu(lens, "cpu")
    conv = convert_blockmask(layout.cuda(), causal=False)
    nrb = sq_r // 16
    greedy = be.blockmask_row_order(layout.cuda())
    assert sorted(greedy.tolist()) == list(range(nrb))
    rand = torch.randperm(nrb, generator=torch.Generator().manual_seed(3)).to(torch.int32).cuda()
    ref = orc.varlen_attention(q, k, v, cu, cu, None, False, layout=layout.numpy(), dout=do)
    half = half_attention(q.cuda(), k.cuda(), v.cuda(), cu.tolist(), cu.tolist(), D ** -0.5, False, layout=layout.numpy(),
                          dout=do.cuda())
    qg, kg, vg, dog, cug = q.cuda(), k.cuda(), v.cuda(), do.cuda(), cu.cuda()
    res = []
    for order in (None, greedy, rand):
        o, lse = be.fwd_block(qg, kg, vg, cug, cug, conv, N, N, 0.0, D ** -0.5, False, False, None, row_order=order)
        dq, dk, dv = (torch.full_like(x, float("nan")) for x in (qg, kg, vg))
        be.bwd_block(dog, qg, kg, vg, o, lse, dq, dk, dv, cug, cug, conv, N, N, 0.0, D ** -0.5, False, None, row_order=order)
        torch.cuda.synchronize()
        ours = {"out": o, "dq": dq, "dk": dk, "dv": dv}
        check_against_oracle(ours, ref, half, dtype, what="blocksparse row order D%d N%d" % (D, N))
        assert o[80:96].abs().max() == 0 and dq[80:96].abs().max() == 0  # the row block without an active tile
        res.append(ours)
    for other in res[1:]:
        for n in ("out", "dq", "dk", "dv"):
            assert _maxerr(res[0][n], other[n]) <= 4 * HALF_ULP[dtype] * max(1.0, res[0][n].float().abs().max().item()), n
    bad = torch.zeros(nrb - 1, dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError, match="row_order"):
        be.fwd_block(qg, kg, vg, cug, cug, conv, N, N, 0.0, D ** -0.5, False, False, None, row_order=bad)


def test_blocksparse_full_layout_equals_dense(full_size_tiles):
    from flash_attn.flash_blocksparse_attn_interface import flash_blocksparse_attn_func
    from flash_attn.flash_attn_interface import flash_attn_unpadded_qkvpacked_func
    N, H, D = 600, 2, 64
    qkv = torch.randn(2 * N, 3, H, D, device="cuda", dtype=torch.float16)
    cu = _cu([N, N])
    layout = torch.ones(608 // 16, 768 // 256, device="cuda")
    a = flash_blocksparse_attn_func(qkv, cu, layout, 0.0, N)
    b = flash_attn_unpadded_qkvpacked_func(qkv, cu, N, 0.0)
    torch.cuda.synchronize()
    assert torch.equal(a, b)
    a = flash_blocksparse_attn_func(qkv, cu, layout, 0.0, N, causal=True)
    b = flash_attn_unpadded_qkvpacked_func(qkv, cu, N, 0.0, causal=True)
    torch.cuda.synchronize()
    assert torch.equal(a, b)


def test_blocksparse_causal_sweep():
    """Causal on top of a block layout (the reference's Python refuses the pair, flash_blocksparse_attn_interface.py:21;
    its kernels take both): a score counts iff its block is listed and key <= query.  Eight seeded cases over head dim,
    dtype, ragged lengths, density and dropout; rows whose listed blocks all lie above the diagonal give zeros; the
    returned probabilities vanish above the diagonal and outside the layout."""
    from flash_attn.flash_blocksparse_attn_interface import flash_blocksparse_attn_func
    from flash_attn import flash_attn_gfx950 as be
    rng = np.random.default_rng(77)
    for case in range(8):
        D = int(rng.choice([16, 32, 64, 128]))
        dtype = torch.float16 if rng.integers(2) else torch.bfloat16
        B, H = int(rng.integers(1, 4)), int(rng.integers(1, 3))
        N = int(rng.choice([100, 300, 520, 1100, 2100]))
        lens = [N] + [int(x) for x in rng.integers(max(1, N // 3), N + 1, B - 1)]
        dens = float(rng.choice([0.1, 0.3, 0.6, 1.0]))
        p = float(rng.choice([0.0, 0.0, 0.2]))
        sq_r, sk_r = be.round_seqlens(D, N, N, True)
        layout = torch.rand(sq_r // 16, sk_r // 256, generator=torch.Generator().manual_seed(50 + case)) < dens
        if rng.integers(2):
            layout |= (torch.arange(sq_r // 16)[:, None] // 16) == torch.arange(sk_r // 256)[None, :]
        if sk_r > 256 and sq_r // 16 > 2:
            layout[2] = False
            layout[2, 1] = True     # rows 32..47 list only keys 256..511: nothing visible under the causal mask
        what = "case %d: D=%d %s B=%d H=%d lens=%s density %.2f p=%.1f" % (case, D, dtype, B, H, lens, dens, p)
        print(what, flush=True)
        q, k, v, do = _inputs(lens, lens, H, D, dtype, 4000 + case)
        cu = _cu(lens, "cpu")
        qkv = torch.stack([q, k, v], 1).cuda().requires_grad_()
        torch.manual_seed(case)
        seed, offset = _gen_state()
        ctx, S, lse = flash_blocksparse_attn_func(qkv, cu.cuda(), layout.cuda(), p, N, None, True, True)
        ctx.backward(do.cuda())
        torch.cuda.synchronize()
        masks = None
        if p > 0:
            masks = [torch.tensor(np.stack([orc.dropout_keep_mask(seed, offset, b * H + h, L, L, p) for h in range(H)]))
                     for b, L in enumerate(lens)]
        ref = orc.varlen_attention(q, k, v, cu, cu, None, True, p_dropout=p, keep_mask=masks, layout=layout.numpy(), dout=do)
        half = half_attention(q.cuda(), k.cuda(), v.cuda(), cu.tolist(), cu.tolist(), D ** -0.5, True, masks, p,
                              layout=layout.numpy(), dout=do.cuda())
        ours = {"out": ctx.detach(), "dq": qkv.grad[:, 0], "dk": qkv.grad[:, 1], "dv": qkv.grad[:, 2]}
        check_against_oracle(ours, ref, half, dtype, what=what)
        seen = orc.expand_block_layout(layout.numpy(), N, N) & (torch.arange(N)[None, :] <= torch.arange(N)[:, None])
        assert S[0, :, :N, :N].cpu()[:, ~seen].abs().max() == 0, what
        if sk_r > 256 and sq_r // 16 > 2:
            assert ctx[32:48].abs().max() == 0 and torch.isinf(lse[0, :, 32:48]).all(), what
            assert qkv.grad[32:48, 0].abs().max() == 0, what


# ------------------------------------------------------------------------------------------------
# modules
# ------------------------------------------------------------------------------------------------
def test_flash_attention_module_three_input_modes():
    from flash_attn.flash_attention import FlashAttention
    B, S, H, D = 3, 96, 2, 64
    g = torch.Generator().manual_seed(8)
    qkv = torch.randn(B, S, 3, H, D, generator=g).half()
    lens = torch.tensor([96, 40, 7])
    mask = torch.arange(S)[None, :] < lens[:, None]
    m = FlashAttention().eval()

    class KPM:
        bool_matrix = mask.cuda()

    # ALiBi slopes through the module (padded input with a key padding mask)
    slopes = _alibi_slopes(H)
    out_al, _ = m(qkv.cuda(), key_padding_mask=KPM(), causal=True, alibi_slopes=slopes.cuda())
    for b in range(B):
        L = int(lens[b])
        r = orc.varlen_attention(qkv[b, :L, 0], qkv[b, :L, 1], qkv[b, :L, 2], [0, L], [0, L], None, True, alibi_slopes=slopes)
        assert (out_al[b, :L].float().cpu() - r["out"]).abs().max() < 2e-3
    # a bias tensor through the module (shared over the batch, per head; padded input: positions inside each sequence)
    tb = (torch.randn(1, H, S, S, generator=g) * 1.5).half()
    out_tb, _ = m(qkv.cuda(), key_padding_mask=KPM(), attn_bias=tb.cuda())
    for b in range(B):
        L = int(lens[b])
        r = orc.varlen_attention(qkv[b, :L, 0], qkv[b, :L, 1], qkv[b, :L, 2], [0, L], [0, L], None, False, attn_bias=tb)
        assert (out_tb[b, :L].float().cpu() - r["out"]).abs().max() < 2e-3
    ref = orc.attention_ref(qkv, mask, 0.0, upcast=True, causal=True).float()
    out_pad, _ = m(qkv.cuda(), key_padding_mask=KPM(), causal=True)
    assert tuple(out_pad.shape) == (B, S, H, D)
    assert (out_pad.cpu().float() - ref)[mask].abs().max() < 2e-3
    assert out_pad.cpu()[~mask].abs().max() == 0
    full = torch.ones(B, S, dtype=torch.bool)
    out_full, _ = m(qkv.cuda(), causal=False)
    assert (out_full.cpu().float() - orc.attention_ref(qkv, full, 0.0, upcast=True).float()).abs().max() < 2e-3
    packed = torch.cat([qkv[b, :lens[b]] for b in range(B)], 0).cuda()
    out_packed, _ = m(packed, cu_seqlens=_cu(lens.tolist()), max_s=96, causal=True)
    assert torch.equal(out_packed, out_pad[mask.cuda()])


def test_flash_mha_matches_torch_multihead_attention():
    from flash_attn.flash_attention import FlashMHA
    torch.manual_seed(0)
    E, H, B, S = 128, 4, 2, 50
    mha = FlashMHA(E, H, device="cuda", dtype=torch.float16).eval()
    ref = torch.nn.MultiheadAttention(E, H, batch_first=True, device="cuda", dtype=torch.float32)
    with torch.no_grad():
        ref.in_proj_weight.copy_(mha.Wqkv.weight.float())
        ref.in_proj_bias.copy_(mha.Wqkv.bias.float())
        ref.out_proj.weight.copy_(mha.out_proj.weight.float())
        ref.out_proj.bias.copy_(mha.out_proj.bias.float())
    x = torch.randn(B, S, E, device="cuda", dtype=torch.float16)
    y, _ = mha(x, None, None)
    y_ref, _ = ref(x.float(), x.float(), x.float(), need_weights=False)
    assert (y.float() - y_ref).abs().max() < 1e-2
    y.sum().backward()
    assert mha.Wqkv.weight.grad is not None and torch.isfinite(mha.Wqkv.weight.grad).all()
    rot = FlashMHA(E, H, use_rotary_emb="1d", causal=True, device="cuda", dtype=torch.float16).eval()
    y2, _ = rot(x, None, None)
    assert tuple(y2.shape) == (B, S, E) and torch.isfinite(y2).all()


# ------------------------------------------------------------------------------------------------
# BASELINE configurations at full size: fp32 PyTorch on the GPU as the reference, plus size-independent properties
# ------------------------------------------------------------------------------------------------
# ------------------------------------------------------------------------------------------------
# the one-kernel backward (launch policy 0x20: head dim 64, dense, no mask / dropout / bias)
# ------------------------------------------------------------------------------------------------
@pytest.fixture
def one_kernel_backward():
    from flash_attn import flash_attn_gfx950 as be
    be.set_launch_policy(0x20)
    yield
    be.set_launch_policy(0)


@pytest.mark.parametrize("lens_q,lens_k,dtype,packing", [
    ([256, 256], [256, 256], torch.float16, "qkv"),
    ([300, 77], [300, 77], torch.float16, "qkv"),
    ([1024, 130, 640], [1024, 130, 640], torch.bfloat16, "qkv"),
    ([200, 31, 512], [640, 129, 96], torch.float16, "kv"),     # more key tiles than query tiles and the reverse
    ([33], [1500], torch.bfloat16, "sep"),                     # two query tiles, twelve key tiles
    ([700, 5], [1, 260], torch.float16, "sep"),
])
def test_one_kernel_backward_parity(lens_q, lens_k, dtype, packing, one_kernel_backward):
    """the same parity bar as the two-kernel backward, on shapes that wrap the ring of query tiles in every way"""
    from flash_attn import flash_attn_gfx950 as be
    a = be.BwdArgs()
    a.struct_bytes = ctypes.sizeof(a)
    a.batch, a.nheads, a.head_dim = len(lens_q), 3, 64
    a.max_seqlen_q, a.max_seqlen_k = max(lens_q), max(lens_k)
    assert be.load_library().fa_bwd_workspace_bytes(ctypes.byref(a)) > 0  # the path under test is the one that runs
    _parity_case(lens_q, lens_k, 3, 64, dtype, False, packing, seed=11)


def test_one_kernel_backward_headline_and_determinism(one_kernel_backward):
    """the headline shape: parity, bitwise equal results from run to run (one owner at a time, fixed order), and agreement
    with the two-kernel backward within the rounding of the 16-bit results"""
    from flash_attn import flash_attn_gfx950 as be
    q, k, v, do, cu, ours = _full_size_check([2048] * 8, 12, 64, torch.float16, False, seed=1)
    again = run_ours(q, k, v, do, cu, cu, 2048, 2048, 0.0, None, False, "qkv")
    for n in ("dq", "dk", "dv"):
        assert torch.equal(ours[n], again[n]), n
    be.set_launch_policy(0x10)
    two = run_ours(q, k, v, do, cu, cu, 2048, 2048, 0.0, None, False, "qkv")
    for n in ("dq", "dk", "dv"):
        assert _maxerr(ours[n], two[n]) <= 4 * HALF_ULP[torch.float16] * two[n].float().abs().max().item(), n


def test_one_kernel_backward_batch_entries_without_keys_or_queries(one_kernel_backward):
    """a batch entry without keys has no key tile: its dq rows are zero; one without queries leaves dk = dv = 0"""
    from flash_attn import flash_attn_gfx950 as be
    lens_q, lens_k, H, D = [100, 64, 0], [90, 0, 70], 2, 64
    q, k, v, do = (x.cuda() for x in _inputs(lens_q, lens_k, H, D, torch.float16, 5))
    cu_q, cu_k = _cu(lens_q), _cu(lens_k)
    o, lse = be.fwd(q, k, v, cu_q, cu_k, 100, 90, 0.0, 0.125, False, False, False, None)
    dq, dk, dv = (torch.full_like(x, float("nan")) for x in (q, k, v))
    be.bwd(do, q, k, v, o, lse, dq, dk, dv, cu_q, cu_k, 100, 90, 0.0, 0.125, False, False, None)
    torch.cuda.synchronize()
    be.set_launch_policy(0x10)
    dq2, dk2, dv2 = (torch.full_like(x, float("nan")) for x in (q, k, v))
    be.bwd(do, q, k, v, o, lse, dq2, dk2, dv2, cu_q, cu_k, 100, 90, 0.0, 0.125, False, False, None)
    torch.cuda.synchronize()
    assert not torch.isnan(dq).any() and not torch.isnan(dk).any() and not torch.isnan(dv).any()
    assert torch.equal(dq[100:164], torch.zeros_like(dq[100:164])) and torch.equal(dk[90:], torch.zeros_like(dk[90:]))
    for a_, b_ in ((dq, dq2), (dk, dk2), (dv, dv2)):
        assert _maxerr(a_, b_) <= 4 * HALF_ULP[torch.float16] * max(1.0, b_.float().abs().max().item())


def _full_size_check(lens, H, D, dtype, causal, p=0.0, seed=0):
    q, k, v, do = (x.cuda() for x in _inputs(lens, lens, H, D, dtype, seed))
    cu = _cu(lens, "cpu")
    torch.manual_seed(seed)
    seed_, offset = _gen_state()
    ours = run_ours(q, k, v, do, cu, cu, max(lens), max(lens), p, None, causal, "qkv", probs=False)
    masks = None
    if p > 0:
        masks = [torch.tensor(np.stack([orc.dropout_keep_mask(seed_, offset, b * H + h, L, L, p) for h in range(H)]))
                 for b, L in enumerate(lens)]
    ref = orc.varlen_attention(q, k, v, cu, cu, None, causal, p_dropout=p, keep_mask=masks, dout=do)  # fp32 on the GPU
    half = half_attention(q, k, v, cu.tolist(), cu.tolist(), D ** -0.5, causal, masks, p, dout=do)
    check_against_oracle(ours, ref, half, dtype, what="full size %s" % ((len(lens), H, D, max(lens), causal, p),))
    return q, k, v, do, cu, ours


def test_config_bert_varlen_dropout(tile_shape, dropout_path):
    """BASELINE config 2: fp16, B=8, H=12, d=64, lengths uniform in [256, 512], p=0.1."""
    g = torch.Generator().manual_seed(0)
    lens = torch.randint(256, 513, (8,), generator=g).tolist()
    _full_size_check(lens, 12, 64, torch.float16, False, p=0.1, seed=2)


@pytest.mark.parametrize("N", [1024, 2048, 4096])
def test_config_gpt2_causal_bf16(N):
    """BASELINE config 3: bf16, B=8, H=12, d=64, causal."""
    q, k, v, do, cu, ours = _full_size_check([N] * 8, 12, 64, torch.bfloat16, True, seed=N)
    # causal first row of every sequence attends to key 0 only: o = v0 exactly
    first = torch.arange(0, 8 * N, N, device="cuda")
    assert torch.equal(ours["out"][first], v[first])


def test_headline_config_fp16():
    """the configuration the metric is quoted on: fp16, B=8, H=12, d=64, N=2048, non-causal, p=0."""
    _full_size_check([2048] * 8, 12, 64, torch.float16, False, seed=1)


@pytest.mark.parametrize("causal", [False, True])
def test_config_head_dim_128(causal):
    """BASELINE config 4: fp16, B=16, H=12, d=128, N=2048."""
    _full_size_check([2048] * 16, 12, 128, torch.float16, causal, seed=4)


def test_config_blocksparse_long_sequence():
    """BASELINE config 5: fp16, B=4, H=16, d=64, N=4096, ~25% density band + random blocks."""
    from flash_attn.flash_blocksparse_attn_interface import flash_blocksparse_attn_func
    B, H, D, N = 4, 16, 64, 4096
    g = torch.Generator().manual_seed(0)
    nrow, ncol = N // 16, N // 256
    band = (torch.arange(nrow)[:, None] // 16 - torch.arange(ncol)[None, :]).abs() <= 1
    layout = band | (torch.rand(nrow, ncol, generator=g) < 0.08)
    assert 0.2 < layout.float().mean() < 0.3
    lens = [N] * B
    q, k, v, do = (x.cuda() for x in _inputs(lens, lens, H, D, torch.float16, 5))
    cu = _cu(lens, "cpu")
    qkv = torch.stack([q, k, v], 1).requires_grad_()
    out = flash_blocksparse_attn_func(qkv, cu.cuda(), layout.cuda(), 0.0, N)
    out.backward(do)
    torch.cuda.synchronize()
    ours = {"out": out.detach(), "dq": qkv.grad[:, 0], "dk": qkv.grad[:, 1], "dv": qkv.grad[:, 2]}
    ref = orc.varlen_attention(q, k, v, cu, cu, None, False, layout=layout.numpy(), dout=do)
    half = half_attention(q, k, v, cu.tolist(), cu.tolist(), D ** -0.5, False, layout=layout.numpy(), dout=do)
    check_against_oracle(ours, ref, half, torch.float16, what="blocksparse N4096")


def test_size_independent_properties_at_full_size(full_size_tiles):
    """varlen == per-sequence dense; batch permutation; linearity in V; uniform attention for q = 0."""
    from flash_attn.flash_attn_interface import flash_attn_unpadded_func
    H, D = 12, 64
    g = torch.Generator().manual_seed(3)
    lens = torch.randint(256, 2049, (8,), generator=g).tolist()
    q, k, v, do = (x.cuda() for x in _inputs(lens, lens, H, D, torch.float16, 9))
    cu = _cu(lens)
    mx = max(lens)
    out = flash_attn_unpadded_func(q, k, v, cu, cu, mx, mx, 0.0, None, True)
    offs = [0] + list(np.cumsum(lens))
    # (1) packed result == each sequence run alone (bitwise: same tiles, same order)
    for b in (0, 3, 7):
        sl = slice(offs[b], offs[b + 1])
        one = flash_attn_unpadded_func(q[sl], k[sl], v[sl], _cu([lens[b]]), _cu([lens[b]]), lens[b], lens[b], 0.0, None, True)
        assert torch.equal(one, out[sl])
    # (2) permuting the batch permutes the result
    perm = [5, 2, 7, 0, 1, 6, 3, 4]
    pq, pk, pv = (torch.cat([x[offs[b]:offs[b + 1]] for b in perm]) for x in (q, k, v))
    pout = flash_attn_unpadded_func(pq, pk, pv, _cu([lens[b] for b in perm]), _cu([lens[b] for b in perm]), mx, mx, 0.0, None, True)
    assert torch.equal(pout, torch.cat([out[offs[b]:offs[b + 1]] for b in perm]))
    # (3) linear in V (up to rounding of the half outputs): f(v1 + v2) = f(v1) + f(v2)
    v2 = torch.randn_like(v)
    o1 = flash_attn_unpadded_func(q, k, v, cu, cu, mx, mx, 0.0).float()
    o2 = flash_attn_unpadded_func(q, k, v2, cu, cu, mx, mx, 0.0).float()
    o12 = flash_attn_unpadded_func(q, k, (v.float() + v2.float()).half(), cu, cu, mx, mx, 0.0).float()
    assert (o12 - (o1 + o2)).abs().max() < 4e-3
    # (4) q = 0: uniform weights, o = running/whole mean of v, lse = log(#visible keys)
    z = torch.zeros_like(q)
    oz, lse, _ = flash_attn_unpadded_func(z, k, v, cu, cu, mx, mx, 0.0, None, False, True)
    for b in (1, 4):
        sl = slice(offs[b], offs[b + 1])
        assert (oz[sl].float() - v[sl].float().mean(0, keepdim=True)).abs().max() < 2e-3
        assert (lse[b, :, :lens[b]] - math.log(lens[b])).abs().max() < 1e-4


# ------------------------------------------------------------------------------------------------
# unpad / pad: byte movement, compared bit for bit with the oracle (bert_padding.py:9-95)
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype,dim", [(torch.float16, 768), (torch.bfloat16, 40), (torch.float32, 5), (torch.float16, 3),
                                       (torch.float16, 1024)])
def test_unpad_pad_rows_bit_exact(dtype, dim):
    """unpad_input / pad_input on the GPU run fa_gather_rows / fa_scatter_rows; rows of 6 .. 2048 bytes exercise every
    chunk width.  Forward results and both backward directions equal the oracle's index arithmetic exactly."""
    from flash_attn.bert_padding import pad_input, unpad_input
    g = torch.Generator().manual_seed(dim)
    B, S = 5, 37
    lens = [37, 0, 1, 20, 36]
    mask = torch.zeros(B, S, dtype=torch.bool)
    for b, L in enumerate(lens):
        mask[b, :L] = True
    mask[3, 5] = False  # a hole in the middle: indices need not be a prefix per row
    x = torch.randn(B, S, dim, generator=g).to(dtype)
    xg = x.cuda().requires_grad_(True)
    rows, idx, cu, mx = unpad_input(xg, mask.cuda())
    r_rows, r_idx, r_cu, r_mx = orc.unpad_ref(x.view(torch.int16 if x.element_size() == 2 else torch.int32).numpy(), mask.numpy())
    as_int = lambda t: t.detach().cpu().view(torch.int16 if t.element_size() == 2 else torch.int32).numpy()
    assert np.array_equal(as_int(rows), r_rows)
    assert np.array_equal(idx.cpu().numpy(), r_idx) and np.array_equal(cu.cpu().numpy(), r_cu) and mx == r_mx
    # backward of the gather = scatter into zeros
    gr = torch.randn(rows.shape, generator=g).to(dtype)
    rows.backward(gr.cuda())
    assert np.array_equal(as_int(xg.grad), orc.pad_ref(as_int(gr), r_idx, B, S).reshape(B, S, dim))
    # pad_input and its backward (a gather)
    vg = gr.cuda().requires_grad_(True)
    padded = pad_input(vg, idx, B, S)
    assert np.array_equal(as_int(padded), orc.pad_ref(as_int(gr), r_idx, B, S))
    gp = torch.randn(B, S, dim, generator=g).to(dtype)
    padded.backward(gp.cuda())
    assert np.array_equal(as_int(vg.grad), as_int(gp).reshape(B * S, dim)[r_idx])


def test_rows_raw_c_abi_unsorted_strided_and_errors():
    """fa_gather_rows / fa_scatter_rows called directly: unsorted unique indices, strided rows, out-of-range indices,
    empty inputs, missing workspace."""
    import ctypes
    from flash_attn import flash_attn_gfx950 as be
    lib = be.load_library()
    g = torch.Generator().manual_seed(3)
    n_src, dim = 50, 24
    base = torch.randn(n_src, 2 * dim, generator=g).half().cuda()
    src = base[:, :dim]                                  # row stride 96 bytes, row width 48 bytes
    perm = torch.randperm(n_src, generator=g)[:31]
    idx = perm.clone()
    idx[4] = n_src + 7                                   # out of range: zero row
    idx[9] = -1
    idx_d = idx.cuda()
    dst = torch.full((31, dim), 7.0, dtype=torch.float16, device="cuda")
    rc = lib.fa_gather_rows(src.data_ptr(), dst.data_ptr(), idx_d.data_ptr(), 31, n_src, dim * 2, src.stride(0) * 2,
                            dim * 2, None)
    assert rc == 0, lib.fa_last_error()
    want = src.cpu()[perm]
    want[4] = 0
    want[9] = 0
    assert torch.equal(dst.cpu(), want)
    # scatter with unsorted indices into a strided destination; rows that receive nothing become zero
    n_dst = 64
    out_base = torch.full((n_dst, 2 * dim), 5.0, dtype=torch.float16, device="cuda")
    out = out_base[:, dim:]
    vals = torch.randn(31, dim, generator=g).half().cuda()
    sidx = torch.randperm(n_dst, generator=g)[:31]
    sidx_bad = sidx.clone()
    sidx_bad[0] = n_dst                                   # ignored
    want = torch.zeros(n_dst, dim, dtype=torch.float16)
    want[sidx[1:]] = vals.cpu()[1:]
    # the workspace arrives with whatever the last user left in it: plausible source rows, the entries of an earlier
    # call with other indices, values far out of range
    stale = [torch.arange(n_dst) % 31, torch.randperm(n_dst, generator=g) % 31, torch.full((n_dst,), 2 ** 31 - 1),
             torch.full((n_dst,), -2 ** 31), torch.zeros(n_dst)]
    for fill in stale:
        ws = fill.to(torch.int32).cuda()
        out.fill_(5.0)
        rc = lib.fa_scatter_rows(vals.data_ptr(), out.data_ptr(), sidx_bad.cuda().data_ptr(), 31, n_dst, dim * 2, dim * 2,
                                 out.stride(0) * 2, ws.data_ptr(), n_dst * 4, None)
        assert rc == 0, lib.fa_last_error()
        torch.cuda.synchronize()
        assert torch.equal(out.cpu(), want)
    assert torch.equal(out_base[:, :dim].cpu(), torch.full((n_dst, dim), 5.0, dtype=torch.float16))  # neighbours untouched
    # empty and error cases
    assert lib.fa_gather_rows(None, None, None, 0, 0, 16, 16, 16, None) == 0
    assert lib.fa_scatter_rows(None, out.data_ptr(), None, 0, n_dst, dim * 2, dim * 2, out.stride(0) * 2, ws.data_ptr(),
                               n_dst * 4, None) == 0
    torch.cuda.synchronize()
    assert not out.cpu().any()
    assert lib.fa_scatter_rows(vals.data_ptr(), out.data_ptr(), sidx.cuda().data_ptr(), 31, n_dst, dim * 2, dim * 2,
                               out.stride(0) * 2, None, 0, None) == -2
    assert b"workspace" in lib.fa_last_error()
    assert lib.fa_gather_rows(src.data_ptr(), dst.data_ptr(), idx_d.data_ptr(), 31, n_src, dim * 2, 8, dim * 2, None) == -1


def test_blocksparse_modules_layout_sources_and_padding():
    """FlashBlocksparseAttention / FlashBlocksparseMHA (flash_blocksparse_attention.py:14-136) built from a layout
    tensor and from an object with make_layout(); padded, packed and key_padding_mask inputs agree with the oracle on
    the expanded layout."""
    from flash_attn.flash_blocksparse_attention import FlashBlocksparseAttention, FlashBlocksparseMHA
    torch.manual_seed(0)
    S, H, D, B = 512, 2, 64, 2
    g = torch.Generator().manual_seed(1)
    layout = (torch.rand(S // 16, S // 256, generator=g) < 0.5).to(torch.int32)
    layout[:, 0] |= (torch.arange(S // 16) % 3 != 0).to(torch.int32)

    class Cfg:
        def make_layout(self, seqlen):
            assert seqlen == S
            return layout

    m_t = FlashBlocksparseAttention(layout, max_seq_length=S).cuda().eval()
    m_o = FlashBlocksparseAttention(Cfg(), max_seq_length=S - 100).cuda().eval()   # rounded up to 512
    assert torch.equal(m_t.layout.cpu(), layout) and torch.equal(m_o.blockmask_converted, m_t.blockmask_converted)
    qkv = torch.randn(B, S, 3, H, D, generator=g).half()
    out, w = m_t(qkv.cuda())
    assert w is None
    sc = D ** -0.5
    for b in range(B):
        ref = orc.varlen_attention(qkv[b, :, 0], qkv[b, :, 1], qkv[b, :, 2], _cu([S], "cpu"), _cu([S], "cpu"), sc, False,
                                   layout=layout.numpy())
        assert (out[b].float().cpu() - ref["out"]).abs().max() < 2e-3
    # packed input with and without mask conversion
    cu = _cu([S] * B, "cuda")
    packed = qkv.reshape(B * S, 3, H, D).cuda()
    o1, _ = m_o(packed, cu_seqlens=cu, max_s=S)
    o2, _ = m_o(packed, cu_seqlens=cu, max_s=S, convert_mask=False)
    assert torch.equal(o1, out.reshape(B * S, H, D)) and torch.equal(o2, o1)
    # key padding mask (tensor and .bool_matrix object): shorter sequences use the corner of the layout
    lens = [300, 512]
    keep = torch.zeros(B, S, dtype=torch.bool)
    for b, L in enumerate(lens):
        keep[b, :L] = True

    class Mask:
        bool_matrix = keep.cuda()

    o3, _ = m_t(qkv.cuda(), key_padding_mask=keep.cuda())
    o4, _ = m_t(qkv.cuda(), key_padding_mask=Mask())
    assert torch.equal(o3, o4)
    for b, L in enumerate(lens):
        ref = orc.varlen_attention(qkv[b, :L, 0], qkv[b, :L, 1], qkv[b, :L, 2], _cu([L], "cpu"), _cu([L], "cpu"), sc, False,
                                   layout=layout[:(L + 15) // 16, :(L + 255) // 256].numpy())
        assert (o3[b, :L].float().cpu() - ref["out"]).abs().max() < 2e-3
        assert not o3[b, L:].any()
    # causal=True through the module: padded, and packed with the module's stored (non-causal) conversion
    oc, _ = m_t(qkv.cuda(), causal=True)
    oc2, _ = m_o(packed, cu_seqlens=cu, max_s=S, causal=True, convert_mask=False)
    assert torch.equal(oc2, oc.reshape(B * S, H, D))
    ref = orc.varlen_attention(qkv[0, :, 0], qkv[0, :, 1], qkv[0, :, 2], _cu([S], "cpu"), _cu([S], "cpu"), sc, True,
                               layout=layout.numpy())
    assert (oc[0].float().cpu() - ref["out"]).abs().max() < 2e-3
    # MHA block: gradient flows to the projections
    mha = FlashBlocksparseMHA(H * D, H, layout, max_seq_length=S, device="cuda", dtype=torch.float16)
    x = torch.randn(B, S, H * D, device="cuda", dtype=torch.float16, requires_grad=True)
    y, _ = mha(x, None, None)
    y.float().pow(2).mean().backward()
    assert y.shape == x.shape and torch.isfinite(x.grad).all() and mha.Wqkv.weight.grad.abs().sum() > 0
    with pytest.raises(TypeError):
        FlashBlocksparseAttention(object())


# ------------------------------------------------------------------------------------------------
# short launches: dQ and dK/dV in one launch (fa_bwd_merged_kernel; the default where the dQ kernel takes half-size tiles)
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("lens,dtype,causal,p", [
    ([405, 435, 303, 318, 325, 368, 319, 504], torch.float16, False, 0.1),   # the BERT batch
    ([405, 435, 303, 318, 325, 368, 319, 504], torch.bfloat16, True, 0.0),
    ([512] * 8, torch.float16, True, 0.1),
    ([300, 1, 77, 512, 129], torch.bfloat16, False, 0.2),
    ([300, 0, 77, 512, 129, 200], torch.float16, False, 0.1),                # a batch entry without tokens
    ([300, 0, 77, 512, 129, 200], torch.bfloat16, True, 0.0),
])
def test_merged_backward_equals_the_two_kernel_backward(lens, dtype, causal, p):
    """Shapes whose backward runs as one launch by default (12 heads: 256 to 511 full-size dQ workgroups, dropout or a causal
    mask): dq, dk, dv and softmax_d are bit for bit those of the two-kernel plan (launch policy 0x10; the dK/dV part sums its
    own Dk in the dQ kernel's order), with the forward's keep words and without dropout; parity with the oracle is what
    test_config_bert_varlen_dropout and the sweeps check."""
    from flash_attn import flash_attn_gfx950 as be
    torch.manual_seed(len(lens))
    H, D = 12, 64
    total, max_s = sum(lens), max(lens)
    cu = _cu(lens)
    qkv = torch.randn(total, 3, H, D, device="cuda").to(dtype)
    do = torch.randn(total, H, D, device="cuda").to(dtype)
    q, k, v = qkv[:, 0], qkv[:, 1], qkv[:, 2]
    g = torch.Generator(device="cuda")
    g.manual_seed(3)
    st = g.get_state()
    kw = be.new_keep_words(q, cu, max_s, max_s, p)
    o, lse = be.fwd(q, k, v, cu, cu, max_s, max_s, p, D ** -0.5, False, causal, False, g, keep_words=kw)
    res = []
    try:
        for policy in (0, 0x10, 0):
            be.set_launch_policy(policy)
            g.set_state(st)
            grads = torch.full_like(qkv, float("nan"))
            out = be.bwd(do, q, k, v, o, lse, grads[:, 0], grads[:, 1], grads[:, 2], cu, cu, max_s, max_s, p, D ** -0.5, False,
                         causal, g, keep_words=kw)
            res.append((grads, out[3]))
    finally:
        be.set_launch_policy(0)
    torch.cuda.synchronize()
    assert torch.isfinite(res[0][0].float()).all()
    for a, b in ((res[0], res[1]), (res[0], res[2])):
        assert torch.equal(a[0], b[0])
        for bi, L in enumerate(lens):
            assert torch.equal(a[1][bi, :, :L], b[1][bi, :, :L])


# ------------------------------------------------------------------------------------------------
# head dim 128: the dK/dV kernel of wave pairs (launch policy 0x40)
# ------------------------------------------------------------------------------------------------
@pytest.fixture
def d128_wave_pairs():
    from flash_attn import flash_attn_gfx950 as be
    be.set_launch_policy(0x40)
    yield
    be.set_launch_policy(0)


@pytest.mark.parametrize("lens_q,lens_k,dtype,causal,packing", [
    ([256, 256], [256, 256], torch.float16, False, "qkv"),
    ([300, 77, 1], [300, 77, 1], torch.bfloat16, True, "qkv"),
    ([1024, 130], [1024, 130], torch.float16, True, "qkv"),
    ([200, 31, 512], [640, 129, 96], torch.float16, False, "kv"),
    ([33], [1500], torch.bfloat16, False, "sep"),
    ([700, 5], [1, 260], torch.float16, False, "sep"),
])
def test_d128_wave_pair_dkdv_parity(lens_q, lens_k, dtype, causal, packing, d128_wave_pairs):
    """the parity bar of the default kernels, on shapes with ragged ends, single rows, more keys than queries and the reverse"""
    _parity_case(lens_q, lens_k, 3, 128, dtype, causal, packing=packing, seed=7)


def test_d128_wave_pair_dkdv_full_size_and_rotary(d128_wave_pairs):
    """B=16 H=12 N=2048 against the default kernels (same arithmetic, P handed to the partner wave rounded: dK within a
    rounding of the default's, dV bit for bit), twice (reproducible), and with the rotation inside the kernels"""
    from flash_attn import flash_attn_gfx950 as be
    from flash_attn.rotary import RotaryEmbedding
    torch.manual_seed(1)
    B, H, D, N = 16, 12, 128, 2048
    qkv = torch.randn(B * N, 3, H, D, device="cuda").half()
    do = torch.randn(B * N, H, D, device="cuda").half()
    cu = _cu([N] * B)
    q, k, v = qkv[:, 0], qkv[:, 1], qkv[:, 2]
    cos_h, sin_h = RotaryEmbedding(D).half_tables(torch.empty(1, N, 3, H, D, device="cuda", dtype=torch.float16))
    for causal, rotary in ((False, None), (True, None), (False, (cos_h, sin_h))):
        o, lse = be.fwd(q, k, v, cu, cu, N, N, 0.0, D ** -0.5, False, causal, False)
        grads = []
        for policy in (0, 0x40, 0x40):
            be.set_launch_policy(policy)
            g = torch.empty_like(qkv)
            be.bwd(do, q, k, v, o, lse, g[:, 0], g[:, 1], g[:, 2], cu, cu, N, N, 0.0, D ** -0.5, False, causal, rotary=rotary)
            grads.append(g)
        assert torch.equal(grads[1], grads[2])
        assert torch.equal(grads[0][:, 0], grads[1][:, 0]) and torch.equal(grads[0][:, 2], grads[1][:, 2])
        assert _maxerr(grads[0][:, 1], grads[1][:, 1]) <= 2.0 ** -9 * float(grads[0][:, 1].abs().max())


# ------------------------------------------------------------------------------------------------
# rotary embedding kernel (fa_rotary) against the oracle; tolerance: one rounding of the result (the reference's
# elementwise fp16 ops round three times, rotary.py:32-42)
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D", [16, 64, 128])
def test_rotary_kernel_matches_oracle(dtype, D):
    from flash_attn import flash_attn_gfx950 as be
    from flash_attn.rotary import RotaryEmbedding, apply_rotary_pos_emb, apply_rotary_emb_qkv_
    g = torch.Generator().manual_seed(D)
    B, S, H = 3, 50, 2
    qkv = torch.randn(B, S, 3, H, D, generator=g).to(dtype)
    emb = RotaryEmbedding(D)
    cos_full, sin_full = emb._update_cos_sin_tables(qkv[:, :, 0].cuda(), seq_dimension=-3)   # (S, D) in dtype
    cos_h, sin_h = cos_full[:, ::2].contiguous(), sin_full[:, ::2].contiguous()
    ulp = 2.0 ** (-10 if dtype == torch.float16 else -7)
    pos = np.tile(np.arange(S), B)

    def close(got, want64):  # one rounding to the 16-bit type
        got = got.double().cpu().numpy()
        assert np.all(np.abs(got - want64) <= ulp * np.abs(want64) * 0.51 + 1e-7), np.abs(got - want64).max()

    out = be.rotary(qkv.cuda(), torch.empty_like(qkv).cuda(), cos_h, sin_h, n_rotated=2)
    for part in range(2):
        want = orc.rotary_ref(qkv[:, :, part].reshape(B * S, H, D).double().numpy(), cos_h.double().cpu().numpy(),
                              sin_h.double().cpu().numpy(), pos)
        close(out[:, :, part].reshape(B * S, H, D), want)
    assert torch.equal(out[:, :, 2].cpu(), qkv[:, :, 2])                                   # v copied untouched
    # the reference's elementwise formulation agrees within its own three roundings
    q_t = apply_rotary_pos_emb(qkv[:, :, 0].cuda(), cos_full, sin_full, seq_dimension=-3)
    assert (q_t.float() - out[:, :, 0].float()).abs().max() <= 3 * ulp * qkv.abs().max() * 1.5
    # explicit positions, conjugate = inverse, in-place autograd wrapper
    p32 = torch.randint(0, S, (B * S,), generator=g, dtype=torch.int32)
    outp = be.rotary(qkv.cuda(), torch.empty_like(qkv).cuda(), cos_h, sin_h, n_rotated=1, positions=p32.cuda())
    close(outp[:, :, 0].reshape(B * S, H, D), orc.rotary_ref(qkv[:, :, 0].reshape(B * S, H, D).double().numpy(),
                                                            cos_h.double().cpu().numpy(), sin_h.double().cpu().numpy(), p32.numpy()))
    assert torch.equal(outp[:, :, 1:].cpu(), qkv[:, :, 1:])
    back = be.rotary(out, torch.empty_like(out), cos_h, sin_h, n_rotated=2, conjugate=True)
    assert (back.float().cpu() - qkv.float()).abs().max() <= 4 * ulp * qkv.abs().max()
    x = qkv.cuda().clone().requires_grad_(True)
    y = apply_rotary_emb_qkv_(x * 1.0, cos_h, sin_h)
    assert torch.equal(y, out)
    go = torch.randn(B, S, 3, H, D, generator=g).to(dtype)
    y.backward(go.cuda())
    for part in range(2):
        want = orc.rotary_ref(go[:, :, part].reshape(B * S, H, D).double().numpy(), cos_h.double().cpu().numpy(),
                              sin_h.double().cpu().numpy(), pos, conjugate=True)
        close(x.grad[:, :, part].reshape(B * S, H, D), want)
    assert torch.equal(x.grad[:, :, 2].cpu(), go[:, :, 2])


# ------------------------------------------------------------------------------------------------
# rotary embedding inside the attention kernels (fa_fwd_args.rotary_cos / fa_bwd_args.rotary_cos): the forward must give
# the bits of fa_rotary followed by fa_fwd; the gradients, rounded once instead of twice, must be at least as close to an
# fp32 PyTorch evaluation of rotation + attention as those of the separate passes are
# ------------------------------------------------------------------------------------------------
def _rotary_attention_fp32(qkv, cos_h, sin_h, lens, scale, causal, dout):
    """d(out . dout)/d(qkv) of attention over rotated q, k, in fp32 PyTorch (tables as rounded to the tensors' dtype)"""
    x = qkv.float().detach().requires_grad_(True)
    outs, start = [], 0
    for L in lens:
        c = cos_h[:L].float()[:, None, :].repeat_interleave(2, -1)
        s_ = sin_h[:L].float()[:, None, :].repeat_interleave(2, -1)

        def rot(t):
            pairs = t.reshape(*t.shape[:-1], -1, 2)
            half_turn = torch.stack((-pairs[..., 1], pairs[..., 0]), -1).reshape(t.shape)
            return t * c + half_turn * s_
        q, k, v = rot(x[start:start + L, 0]), rot(x[start:start + L, 1]), x[start:start + L, 2]
        sc = torch.einsum("ihd,jhd->hij", q, k) * scale
        if causal:
            sc = sc.masked_fill(torch.ones(L, L, dtype=torch.bool, device=x.device).triu(1), float("-inf"))
        outs.append(torch.einsum("hij,jhd->ihd", torch.softmax(sc, -1), v))
        start += L
    out = torch.cat(outs)
    out.backward(dout.float())
    return out.detach(), x.grad


@pytest.mark.parametrize("D,dtype,causal,lens", [
    (64, torch.float16, False, [256, 256]),
    (64, torch.float16, True, [200, 37, 129]),
    (128, torch.bfloat16, False, [150, 300]),
    (32, torch.bfloat16, True, [128, 128, 128]),
    (16, torch.float16, False, [65, 500]),
    (64, torch.bfloat16, False, [1024]),
])
def test_in_kernel_rotary_equals_the_separate_passes(D, dtype, causal, lens, tile_shape):
    from flash_attn import flash_attn_gfx950 as be
    from flash_attn import flash_attn_interface as fi
    from flash_attn.rotary import RotaryEmbedding
    torch.manual_seed(D + len(lens))
    H, total, max_s = 3, sum(lens), max(lens)
    cu = _cu(lens)
    qkv = torch.randn(total, 3, H, D, device="cuda").to(dtype)
    dout = torch.randn(total, H, D, device="cuda").to(dtype)
    emb = RotaryEmbedding(D)
    cos_h, sin_h = emb.half_tables(torch.empty(1, max_s + 3, 3, H, D, device="cuda", dtype=dtype))   # (max_s + 3, D / 2)
    scale = D ** -0.5
    positions = torch.cat([torch.arange(L, dtype=torch.int32) for L in lens]).cuda()

    # separate passes: rotate q and k, attention, rotate the gradients back
    a = qkv.clone()
    be.rotary(a[None], a[None], cos_h, sin_h, n_rotated=2, positions=positions)
    a.requires_grad_(True)
    out_a = fi.flash_attn_unpadded_qkvpacked_func(a, cu, max_s, 0.0, causal=causal)
    out_a.backward(dout)
    g = a.grad.contiguous()
    grad_a = be.rotary(g[None], torch.empty_like(g)[None], cos_h, sin_h, n_rotated=2, conjugate=True, positions=positions)[0]

    b = qkv.clone().requires_grad_(True)
    out_b = fi.flash_attn_unpadded_qkvpacked_rotary_func(b, cos_h, sin_h, cu, max_s, 0.0, causal=causal)
    out_b.backward(dout)
    assert torch.equal(b.detach(), qkv)                               # the caller's tensor is left as it is
    assert torch.equal(out_b, out_a)                                  # same bits
    assert torch.equal(b.grad[:, 2], grad_a[:, 2])                    # dv: same kernel on the same bits
    out_ref, grad_ref = _rotary_attention_fp32(qkv, cos_h, sin_h, lens, scale, causal, dout)
    # both paths round the same fp32 sums: the separate passes twice (rotating in between), the kernels once; the largest
    # errors may sit on different elements, so one path's may exceed the other's by the three roundings (half a unit in the
    # last place of the largest value each), and must not by more
    ulp = 2.0 ** (-10 if dtype == torch.float16 else -7)
    for part, name in ((0, "dq"), (1, "dk")):
        top = float(grad_ref[:, part].abs().max())
        err_a = _maxerr(grad_a[:, part], grad_ref[:, part])
        err_b = _maxerr(b.grad[:, part], grad_ref[:, part])
        assert err_b <= err_a + 2 * ulp * top, (name, err_b, err_a)
        assert err_a < 0.05 * top, (name, err_a)   # the yardstick itself is sound
        # and element by element they differ by those roundings only
        assert _maxerr(b.grad[:, part], grad_a[:, part]) <= 2 * ulp * max(top, float(grad_a[:, part].abs().max()))


def test_in_kernel_rotary_with_dropout_short_queries_and_the_module():
    """dropout (the keep words ride along), a decode-like shape whose keys are split over workgroups, and FlashMHA, whose
    "1d" rotary path goes through the kernels when no padding mask is given and through the separate pass otherwise"""
    from flash_attn import flash_attn_gfx950 as be
    from flash_attn import flash_attn_interface as fi
    from flash_attn.flash_attention import FlashMHA
    from flash_attn.rotary import RotaryEmbedding
    D, H, dtype = 64, 4, torch.float16
    for lens, p in (([300, 212], 0.17), ([2048] * 2, 0.0)):
        torch.manual_seed(5)
        total, max_s = sum(lens), max(lens)
        cu = _cu(lens)
        qkv = torch.randn(total, 3, H, D, device="cuda").to(dtype)
        dout = torch.randn(total, H, D, device="cuda").to(dtype)
        cos_h, sin_h = RotaryEmbedding(D).half_tables(torch.empty(1, max_s, 3, H, D, device="cuda", dtype=dtype))
        positions = torch.cat([torch.arange(L, dtype=torch.int32) for L in lens]).cuda()
        a = qkv.clone()
        be.rotary(a[None], a[None], cos_h, sin_h, n_rotated=2, positions=positions)
        a.requires_grad_(True)
        torch.manual_seed(11)
        out_a = fi.flash_attn_unpadded_qkvpacked_func(a, cu, max_s, p)
        out_a.backward(dout)
        g = a.grad.contiguous()
        grad_a = be.rotary(g[None], torch.empty_like(g)[None], cos_h, sin_h, n_rotated=2, conjugate=True, positions=positions)[0]
        b = qkv.clone().requires_grad_(True)
        torch.manual_seed(11)
        out_b = fi.flash_attn_unpadded_qkvpacked_rotary_func(b, cos_h, sin_h, cu, max_s, p)
        out_b.backward(dout)
        assert torch.equal(out_b, out_a) and torch.equal(b.grad[:, 2], grad_a[:, 2])
        for part in range(2):  # two roundings against one: a few units in the last place of the larger of a pair
            assert _maxerr(b.grad[:, part], grad_a[:, part]) <= 2.0 ** -8 * float(grad_a[:, part].abs().max())

    # few queries, many keys: the forward and the dQ kernel split the keys (their partial sums take the rotation too)
    torch.manual_seed(3)
    Lq, Lk, Hs = 16, 8192, 2
    q = torch.randn(Lq, Hs, D, device="cuda").to(dtype)
    k = torch.randn(Lk, Hs, D, device="cuda").to(dtype)
    v = torch.randn(Lk, Hs, D, device="cuda").to(dtype)
    do = torch.randn(Lq, Hs, D, device="cuda").to(dtype)
    cos_h, sin_h = RotaryEmbedding(D).half_tables(torch.empty(1, Lk, 3, Hs, D, device="cuda", dtype=dtype))
    cu_q, cu_k = _cu([Lq]), _cu([Lk])
    q_r = be.rotary(q[None, :, None], torch.empty_like(q)[None, :, None], cos_h, sin_h, n_rotated=1)[0, :, 0]
    k_r = be.rotary(k[None, :, None], torch.empty_like(k)[None, :, None], cos_h, sin_h, n_rotated=1)[0, :, 0]
    o_a, lse_a = be.fwd(q_r, k_r, v, cu_q, cu_k, Lq, Lk, 0.0, D ** -0.5, False, False, False)
    q_rot = torch.empty_like(q)
    o_b, lse_b = be.fwd(q, k_r, v, cu_q, cu_k, Lq, Lk, 0.0, D ** -0.5, False, False, False, rotary=(cos_h, sin_h), q_rot=q_rot)
    assert torch.equal(o_a, o_b) and torch.equal(lse_a, lse_b) and torch.equal(q_rot, q_r)
    ga = [torch.empty_like(t) for t in (q, k, v)]
    gb = [torch.empty_like(t) for t in (q, k, v)]
    be.bwd(do, q_r, k_r, v, o_a, lse_a, *ga, cu_q, cu_k, Lq, Lk, 0.0, D ** -0.5, False, False)
    be.bwd(do, q_rot, k_r, v, o_b, lse_b, *gb, cu_q, cu_k, Lq, Lk, 0.0, D ** -0.5, False, False, rotary=(cos_h, sin_h))
    dq_a = be.rotary(ga[0][None, :, None], torch.empty_like(q)[None, :, None], cos_h, sin_h, n_rotated=1, conjugate=True)[0, :, 0]
    dk_a = be.rotary(ga[1][None, :, None], torch.empty_like(k)[None, :, None], cos_h, sin_h, n_rotated=1, conjugate=True)[0, :, 0]
    assert torch.equal(ga[2], gb[2])
    assert _maxerr(gb[0], dq_a) <= 2.0 ** -8 * float(dq_a.abs().max())
    assert _maxerr(gb[1], dk_a) <= 2.0 ** -8 * float(dk_a.abs().max())

    torch.manual_seed(0)
    E, Hm, B, S = 256, 4, 2, 100
    mha = FlashMHA(E, Hm, use_rotary_emb="1d", causal=True, device="cuda", dtype=torch.float16).eval()
    x = torch.randn(B, S, E, device="cuda", dtype=torch.float16)

    class AllKept:
        bool_matrix = torch.ones(B, S, dtype=torch.bool, device="cuda")
    y_fused, _ = mha(x, None, None)
    y_fused.float().square().sum().backward()
    g_fused = mha.Wqkv.weight.grad.clone()
    mha.zero_grad()
    y_sep, _ = mha(x, None, None, key_padding_mask=AllKept)
    y_sep.float().square().sum().backward()
    assert torch.equal(y_fused, y_sep)
    assert _maxerr(g_fused, mha.Wqkv.weight.grad) <= 2.0 ** -7 * float(g_fused.abs().max())


@pytest.mark.parametrize("dtype,D", [(torch.float16, 64), (torch.bfloat16, 32), (torch.float16, 16)])
def test_rotary_2d_kernel_path_matches_oracle(dtype, D):
    """RotaryEmbedding2D.rotate_qkv_ (flash_attn/rotary.py:103-135 done by two passes of fa_rotary over the half-channel
    views, positions = column / row of the token in its square grid): against the fp64 rotation of each half, against
    the module's own elementwise forward(), and its backward against the opposite rotation."""
    from flash_attn.rotary import RotaryEmbedding2D
    g = torch.Generator().manual_seed(D + 1)
    B, side, H = 2, 7, 3
    S, half = side * side, D // 2
    qkv = torch.randn(B, S, 3, H, D, generator=g).to(dtype)
    emb = RotaryEmbedding2D(D).cuda()
    x = qkv.cuda().clone().requires_grad_(True)
    y = emb.rotate_qkv_(x * 1.0)
    cos, sin = emb.rotary_emb1d._cos_cached[:, ::2].double().cpu().numpy(), emb.rotary_emb1d._sin_cached[:, ::2].double().cpu().numpy()
    tok = np.tile(np.arange(S), B)
    col, row = tok % side, tok // side
    ulp = 2.0 ** (-10 if dtype == torch.float16 else -7)

    def close(got, want64):
        got = got.detach().double().cpu().numpy()
        assert np.all(np.abs(got - want64) <= ulp * np.abs(want64) * 0.51 + 1e-7), np.abs(got - want64).max()

    for part in range(2):
        src = qkv[:, :, part].reshape(B * S, H, D).double().numpy()
        close(y[:, :, part, :, :half].reshape(B * S, H, half), orc.rotary_ref(src[..., :half], cos, sin, col))
        close(y[:, :, part, :, half:].reshape(B * S, H, half), orc.rotary_ref(src[..., half:], cos, sin, row))
    y_d = y.detach()
    assert torch.equal(y_d[:, :, 2].cpu(), qkv[:, :, 2])
    q_t, k_t = emb(qkv[:, :, 0].cuda(), qkv[:, :, 1].cuda(), seq_dimension=-3)  # elementwise formulation, three roundings
    assert (q_t.float() - y_d[:, :, 0].float()).abs().max() <= 4.5 * ulp * qkv.abs().max()
    assert (k_t.float() - y_d[:, :, 1].float()).abs().max() <= 4.5 * ulp * qkv.abs().max()
    go = torch.randn(B, S, 3, H, D, generator=g).to(dtype)
    y.backward(go.cuda())
    for part in range(2):
        src = go[:, :, part].reshape(B * S, H, D).double().numpy()
        close(x.grad[:, :, part, :, :half].reshape(B * S, H, half), orc.rotary_ref(src[..., :half], cos, sin, col, conjugate=True))
        close(x.grad[:, :, part, :, half:].reshape(B * S, H, half), orc.rotary_ref(src[..., half:], cos, sin, row, conjugate=True))
    assert torch.equal(x.grad[:, :, 2].cpu(), go[:, :, 2])


# ------------------------------------------------------------------------------------------------
# key-split forward (short query side, long key side: decode / cross-attention shapes)
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("lens_q,lens_k,D,p", [
    ([1, 1], [2048, 1500], 64, 0.0),        # one query per sequence
    ([16, 5, 128], [1024, 4000, 513], 64, 0.0),
    ([100], [3000], 128, 0.0),
    ([3, 40], [1300, 2100], 32, 0.15),
])
def test_key_split_forward(lens_q, lens_k, D, p):
    """fa_fwd with the scratch fa_fwd_workspace_bytes() asks for takes the key-split path; results must match the
    oracle, the single-pass kernel (same call without workspace) and, with dropout, use the same mask."""
    from flash_attn import flash_attn_gfx950 as be
    lib = be.load_library()
    H, dtype = 3, torch.float16
    q, k, v, do = _inputs(lens_q, lens_k, H, D, dtype, seed=sum(lens_k))
    cu_q, cu_k = _cu(lens_q, "cuda"), _cu(lens_k, "cuda")
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    sq_r, _ = be.round_seqlens(D, max(lens_q), max(lens_k))

    def call(with_ws):
        o = torch.zeros_like(qd)
        lse = torch.full((len(lens_q), H, sq_r), float("nan"), device="cuda")
        a = be.FwdArgs()
        a.struct_bytes = ctypes.sizeof(a)
        a.dtype = 0
        a.q, a.k, a.v, a.o, a.softmax_lse = qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), o.data_ptr(), lse.data_ptr()
        a.cu_seqlens_q, a.cu_seqlens_k = cu_q.data_ptr(), cu_k.data_ptr()
        a.q_row_stride = a.k_row_stride = a.v_row_stride = a.o_row_stride = H * D
        a.q_head_stride = a.k_head_stride = a.v_head_stride = a.o_head_stride = D
        a.batch, a.nheads, a.head_dim = len(lens_q), H, D
        a.total_q, a.total_k, a.max_seqlen_q, a.max_seqlen_k = sum(lens_q), sum(lens_k), max(lens_q), max(lens_k)
        a.p_dropout, a.softmax_scale = p, D ** -0.5
        a.philox_seed, a.philox_offset = 1234, 8
        need = lib.fa_fwd_workspace_bytes(ctypes.byref(a))
        assert need > 0
        ws = torch.empty(need, dtype=torch.uint8, device="cuda") if with_ws else None
        a.workspace, a.workspace_bytes = (ws.data_ptr(), need) if with_ws else (None, 0)
        assert lib.fa_fwd(ctypes.byref(a)) == 0, lib.fa_last_error()
        torch.cuda.synchronize()
        return o.cpu(), lse.cpu()

    o_split, lse_split = call(True)
    o_single, lse_single = call(False)
    masks = None
    if p > 0:
        masks = [torch.tensor(np.stack([orc.dropout_keep_mask(1234, 8, b * H + h, lq, lk, p) for h in range(H)]))
                 for b, (lq, lk) in enumerate(zip(lens_q, lens_k))]
    ref = orc.varlen_attention(q, k, v, cu_q.cpu(), cu_k.cpu(), D ** -0.5, False, p_dropout=p, keep_mask=masks)
    tol = 2e-3
    assert (o_split.float() - ref["out"]).abs().max() < tol and (o_single.float() - ref["out"]).abs().max() < tol
    assert (o_split.float() - o_single.float()).abs().max() < 1e-3
    for b, L in enumerate(lens_q):
        assert (lse_split[b, :, :L] - ref["lse"][b]).abs().max() < 2e-3
        assert (lse_split[b, :, :L] - lse_single[b, :, :L]).abs().max() < 1e-4
    # the interface layer allocates the scratch itself and backpropagates through the result
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    from flash_attn.flash_attn_interface import flash_attn_unpadded_func
    out = flash_attn_unpadded_func(qg, kg, vg, cu_q, cu_k, max(lens_q), max(lens_k), 0.0)
    assert (out.float().cpu() - orc.varlen_attention(q, k, v, cu_q.cpu(), cu_k.cpu(), D ** -0.5, False)["out"]).abs().max() < tol
    out.backward(do.cuda())
    refb = orc.varlen_attention(q, k, v, cu_q.cpu(), cu_k.cpu(), D ** -0.5, False, dout=do)
    for name, g in (("dq", qg.grad), ("dk", kg.grad), ("dv", vg.grad)):
        assert (g.float().cpu() - refb[name]).abs().max() < 5e-3, name


def test_forward_and_backward_replay_from_a_hip_graph():
    """The C ABI neither allocates nor synchronises, so a forward + backward pair can be captured in a HIP graph.
    Every replay (with new inputs copied into the captured buffers and eager work in between) must equal the eager
    result bit for bit."""
    from flash_attn import flash_attn_gfx950 as be
    lens, H, D = [200, 131], 3, 64
    total = sum(lens)
    cu = _cu(lens, "cuda")
    g = torch.Generator(device="cuda").manual_seed(11)
    qkv = torch.randn(total, 3, H, D, device="cuda", generator=g).half()
    do = torch.randn(total, H, D, device="cuda", generator=g).half()
    dqkv = torch.empty_like(qkv)

    def step():
        o, lse = be.fwd(qkv[:, 0], qkv[:, 1], qkv[:, 2], cu, cu, max(lens), max(lens), 0.0, D ** -0.5, False, True, False, None)
        be.bwd(do, qkv[:, 0], qkv[:, 1], qkv[:, 2], o, lse, dqkv[:, 0], dqkv[:, 1], dqkv[:, 2], cu, cu, max(lens), max(lens),
               0.0, D ** -0.5, False, True, None)
        return o, lse

    step()  # warm-up outside the capture (library load, lazy initialisation)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            o_g, lse_g = step()
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(3):
        qkv.copy_(torch.randn(total, 3, H, D, device="cuda", generator=g).half())
        do.copy_(torch.randn(total, H, D, device="cuda", generator=g).half())
        graph.replay()
        torch.cuda.synchronize()
        got = (o_g.clone(), lse_g.clone(), dqkv.clone())
        dqkv.zero_()
        o_e, lse_e = step()                      # eager work between the replays, on the same buffers
        torch.cuda.synchronize()
        assert torch.equal(got[0], o_e) and torch.equal(got[1][:, :, :1], lse_e[:, :, :1]), rep
        for b, L in enumerate(lens):
            assert torch.equal(got[1][b, :, :L], lse_e[b, :, :L]), rep
        assert torch.equal(got[2], dqkv), rep


def test_c_abi_caller_without_python_or_torch():
    """examples/c_abi_caller.cpp (built by build.py): hipMalloc'ed buffers, the header's structs, one forward and backward of
    a ragged causal batch, checked inside the program against the closed form in double precision."""
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = os.path.join(root, "flash-attention_amd", "build", "c_abi_caller")
    assert os.path.exists(exe), "run `python flash-attention_amd/build.py` first"
    r = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    print(r.stdout)
    assert r.returncode == 0 and "PASS" in r.stdout, r.stdout



@pytest.mark.parametrize("lens_q,lens_k,D,p", [
    ([1, 1], [2048, 1500], 64, 0.0),
    ([16, 5, 128], [1024, 4000, 513], 64, 0.0),
    ([100], [3000], 128, 0.0),
    ([3, 40], [1300, 2100], 32, 0.15),
])
def test_key_split_backward(lens_q, lens_k, D, p):
    """fa_bwd with the scratch fa_bwd_workspace_bytes() asks for splits the keys of the dQ kernel's lone query tile over
    several workgroups (fp32 partial dQ, summed by a second launch); dq must match the oracle and the unsplit kernel
    (same call without workspace), dk and dv must be bitwise those of the unsplit call."""
    from flash_attn import flash_attn_gfx950 as be
    lib = be.load_library()
    H, dtype = 3, torch.float16
    q, k, v, do = _inputs(lens_q, lens_k, H, D, dtype, seed=sum(lens_k) + 1)
    cu_q, cu_k = _cu(lens_q, "cuda"), _cu(lens_k, "cuda")
    qd, kd, vd, dod = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    torch.manual_seed(99)
    seed, offset = _gen_state()  # the pair the forward below reads from the default generator (and then advances)
    out, lse = be.fwd(qd, kd, vd, cu_q, cu_k, max(lens_q), max(lens_k), p, D ** -0.5, False, False, False, None)
    sq_r, _ = be.round_seqlens(D, max(lens_q), max(lens_k))

    def call(with_ws):
        dq, dk, dv = torch.zeros_like(qd), torch.zeros_like(kd), torch.zeros_like(vd)
        sd = torch.zeros(len(lens_q), H, sq_r, device="cuda")
        a = be.BwdArgs()
        a.struct_bytes = ctypes.sizeof(a)
        a.dtype = 0
        a.dout, a.q, a.k, a.v, a.out, a.softmax_lse = (dod.data_ptr(), qd.data_ptr(), kd.data_ptr(), vd.data_ptr(),
                                                       out.data_ptr(), lse.data_ptr())
        a.dq, a.dk, a.dv, a.softmax_d = dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), sd.data_ptr()
        a.cu_seqlens_q, a.cu_seqlens_k = cu_q.data_ptr(), cu_k.data_ptr()
        for name in ("do", "q", "k", "v", "o", "dq", "dk", "dv"):
            setattr(a, name + "_row_stride", H * D)
            setattr(a, name + "_head_stride", D)
        a.lse_seq_stride = lse.shape[2]
        a.batch, a.nheads, a.head_dim = len(lens_q), H, D
        a.total_q, a.total_k, a.max_seqlen_q, a.max_seqlen_k = sum(lens_q), sum(lens_k), max(lens_q), max(lens_k)
        a.p_dropout, a.softmax_scale = p, D ** -0.5
        a.philox_seed, a.philox_offset = seed, offset
        need = lib.fa_bwd_workspace_bytes(ctypes.byref(a))
        assert need > 0
        ws = torch.empty(need, dtype=torch.uint8, device="cuda") if with_ws else None
        a.workspace, a.workspace_bytes = (ws.data_ptr(), need) if with_ws else (None, 0)
        assert lib.fa_bwd(ctypes.byref(a)) == 0, lib.fa_last_error()
        torch.cuda.synchronize()
        return dq.cpu(), dk.cpu(), dv.cpu(), sd.cpu()

    dq_s, dk_s, dv_s, sd_s = call(True)
    dq_1, dk_1, dv_1, sd_1 = call(False)
    assert torch.equal(dk_s, dk_1) and torch.equal(dv_s, dv_1) and torch.equal(sd_s, sd_1)
    masks = None
    if p > 0:
        masks = [torch.tensor(np.stack([orc.dropout_keep_mask(seed, offset, b * H + h, lq, lk, p) for h in range(H)]))
                 for b, (lq, lk) in enumerate(zip(lens_q, lens_k))]
    ref = orc.varlen_attention(q, k, v, cu_q.cpu(), cu_k.cpu(), D ** -0.5, False, p_dropout=p, keep_mask=masks, dout=do)
    half = half_attention(qd, kd, vd, cu_q.tolist(), cu_k.tolist(), D ** -0.5, False, masks, p, dout=dod)
    for got in (dq_s, dq_1):
        check_against_oracle({"dq": got}, ref, half, dtype, names=("dq",), what="key-split backward")
    assert (dq_s.float() - dq_1.float()).abs().max() <= 2.0 ** -10 * max(1.0, ref["dq"].abs().max().item())
