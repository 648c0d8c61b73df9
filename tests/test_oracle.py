"""Pins the CPU oracle (oracle/attention_oracle.py) without the reference: library routines, closed forms,
special cases, finite differences, published known-answer vectors and brute force.  The reference repository has
no tests or golden vectors of its own for this path."""
import itertools
import json
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import attention_oracle as orc

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _rand(shape, seed, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g, dtype=dtype)


# ---------------------------------------------------------------- forward
@pytest.mark.parametrize("causal", [False, True])
def test_attention_ref_matches_sdpa(causal):
    B, S, H, D = 2, 33, 3, 16
    qkv = _rand((B, S, 3, H, D), 0, torch.float32)
    mask = torch.ones(B, S, dtype=torch.bool)
    got = orc.attention_ref(qkv, mask, 0.0, upcast=True, causal=causal)
    q, k, v = (qkv[:, :, i].transpose(1, 2) for i in range(3))
    want = F.scaled_dot_product_attention(q, k, v, is_causal=causal).transpose(1, 2)
    assert torch.allclose(got, want, atol=2e-6, rtol=1e-5)


def test_attention_ref_key_padding_matches_sdpa():
    B, S, H, D = 2, 40, 2, 8
    qkv = _rand((B, S, 3, H, D), 1, torch.float32)
    lens = torch.tensor([40, 23])
    mask = torch.arange(S)[None, :] < lens[:, None]
    got = orc.attention_ref(qkv, mask, 0.0, upcast=True)
    q, k, v = (qkv[:, :, i].transpose(1, 2) for i in range(3))
    want = F.scaled_dot_product_attention(q, k, v, attn_mask=mask[:, None, None, :]).transpose(1, 2)
    assert torch.allclose(got, want, atol=2e-6, rtol=1e-5)


@pytest.mark.parametrize("causal", [False, True])
def test_varlen_equals_attention_ref_per_sequence(causal):
    """packed result == padded standard attention on each sequence (varlen invariant)."""
    H, D = 2, 16
    lens = [5, 17, 32]
    S = max(lens)
    cu = [0] + list(np.cumsum(lens))
    qkv_pad = _rand((3, S, 3, H, D), 2)
    packed = torch.cat([qkv_pad[b, :lens[b]] for b in range(3)], 0)
    r = orc.varlen_attention(packed[:, 0], packed[:, 1], packed[:, 2], cu, cu, None, causal, dtype=torch.float64)
    mask = torch.arange(S)[None, :] < torch.tensor(lens)[:, None]
    ref = orc.attention_ref(qkv_pad, mask, 0.0, causal=causal)
    for b in range(3):
        assert torch.allclose(r["out"][cu[b]:cu[b + 1]], ref[b, :lens[b]], atol=1e-12)


def test_forward_special_cases():
    H, D = 1, 8
    q, k, v = _rand((6, H, D), 3), _rand((6, H, D), 4), _rand((6, H, D), 5)
    # one key: o = v
    r = orc.varlen_attention(q, k[:1], v[:1], [0, 6], [0, 1])
    assert torch.allclose(r["out"], v[:1].float().expand(6, H, D), atol=1e-6)
    assert torch.allclose(r["lse"][0][0], (q[:, 0] @ k[0, 0]).float() * D ** -0.5, atol=1e-5)
    # causal: first row sees key 0 only
    r = orc.varlen_attention(q, k, v, [0, 6], [0, 6], causal=True, dtype=torch.float64)
    assert torch.allclose(r["out"][0], v[0], atol=1e-12)
    # zero queries: uniform weights, o = mean(v), lse = log(n)
    r = orc.varlen_attention(torch.zeros_like(q), k, v, [0, 6], [0, 6], dtype=torch.float64)
    assert torch.allclose(r["out"], v.mean(0, keepdim=True).expand(6, H, D), atol=1e-12)
    assert torch.allclose(r["lse"][0], torch.full((1, 6), math.log(6.0), dtype=torch.float64), atol=1e-12)
    # probabilities: rows of exp(scale*S - lse) sum to one
    r = orc.varlen_attention(q, k, v, [0, 6], [0, 6], dtype=torch.float64)
    assert torch.allclose(r["probs"][0].sum(-1), torch.ones(1, 6, dtype=torch.float64), atol=1e-12)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("block_n", [16, 128, 256, 1000])
def test_tiled_recurrence_is_tile_size_independent(causal, block_n):
    """the reference's (lse, normalised O) carry over key blocks reproduces the closed form for any block width;
    block_n >= Lk reduces to a plain softmax."""
    Lq, Lk, D = 70, 300, 16
    q, k, v = _rand((Lq, D), 6).numpy(), _rand((Lk, D), 7).numpy(), _rand((Lk, D), 8).numpy()
    o, lse = orc.tiled_forward(q, k, v, D ** -0.5, block_n, causal)
    r = orc.varlen_attention(torch.tensor(q)[:, None], torch.tensor(k)[:, None], torch.tensor(v)[:, None], [0, Lq],
                             [0, Lk], None, causal, dtype=torch.float64)
    assert np.allclose(o, r["out"][:, 0].numpy(), atol=1e-11)
    assert np.allclose(lse, r["lse"][0][0].numpy(), atol=1e-11)


def test_block_layout_semantics():
    """masked 16x256 tiles are -inf; rows with no active tile give o = 0, lse = -inf; a full layout is dense."""
    Lq, Lk, D = 48, 512, 8
    q, k, v = _rand((Lq, 1, D), 9), _rand((Lk, 1, D), 10), _rand((Lk, 1, D), 11)
    layout = np.array([[1, 0], [0, 0], [1, 1]])
    r = orc.varlen_attention(q, k, v, [0, Lq], [0, Lk], layout=layout, dtype=torch.float64)
    assert torch.all(r["out"][16:32] == 0) and torch.all(torch.isinf(r["lse"][0][0, 16:32]))
    first = orc.varlen_attention(q[:16], k[:256], v[:256], [0, 16], [0, 256], dtype=torch.float64)
    assert torch.allclose(r["out"][:16], first["out"], atol=1e-12)
    dense = orc.varlen_attention(q, k, v, [0, Lq], [0, Lk], dtype=torch.float64)
    full = orc.varlen_attention(q, k, v, [0, Lq], [0, Lk], layout=np.ones((3, 2)), dtype=torch.float64)
    assert torch.allclose(full["out"], dense["out"], atol=1e-12)
    assert torch.allclose(r["out"][32:], dense["out"][32:], atol=1e-12)


# ---------------------------------------------------------------- backward
@pytest.mark.parametrize("causal", [False, True])
def test_backward_matches_explicit_formulas(causal):
    Lq, Lk, D = 9, 13, 8
    q, k, v, do = _rand((Lq, D), 12), _rand((Lk, D), 13), _rand((Lk, D), 14), _rand((Lq, D), 15)
    e = orc.explicit_backward(q, k, v, do, D ** -0.5, causal)
    r = orc.varlen_attention(q[:, None], k[:, None], v[:, None], [0, Lq], [0, Lk], None, causal, dout=do[:, None],
                             dtype=torch.float64)
    for name in ("dq", "dk", "dv", "out"):
        assert np.allclose(r[name][:, 0].numpy(), e[name], atol=1e-11), name
    assert np.allclose(r["softmax_d"][0][0].numpy(), e["softmax_d"], atol=1e-11)
    assert np.allclose(r["lse"][0][0].numpy(), e["lse"], atol=1e-11)


def test_backward_matches_finite_differences():
    Lq, Lk, D = 4, 5, 4
    q, k, v, do = _rand((Lq, 1, D), 16), _rand((Lk, 1, D), 17), _rand((Lk, 1, D), 18), _rand((Lq, 1, D), 19)
    r = orc.varlen_attention(q, k, v, [0, Lq], [0, Lk], None, True, dout=do, dtype=torch.float64)

    def loss(q_, k_, v_):
        return float((orc.varlen_attention(q_, k_, v_, [0, Lq], [0, Lk], None, True, dtype=torch.float64)["out"] * do).sum())

    eps = 1e-6
    for name, t in (("dq", q), ("dk", k), ("dv", v)):
        num = torch.zeros_like(t)
        for idx in itertools.product(*[range(n) for n in t.shape]):
            tp, tm = t.clone(), t.clone()
            tp[idx] += eps
            tm[idx] -= eps
            args_p = [tp if x is t else x for x in (q, k, v)]
            args_m = [tm if x is t else x for x in (q, k, v)]
            num[idx] = (loss(*args_p) - loss(*args_m)) / (2 * eps)
        assert torch.allclose(r[name], num, atol=1e-7), name


def test_dropout_backward_with_given_mask():
    """with a keep mask M: O = (P o M / keep) V, so dV = (P o M / keep)^T dO and softmax_d = keep * rowsum(dO o O)."""
    Lq, Lk, D, p = 8, 12, 4, 0.25
    q, k, v, do = _rand((Lq, 1, D), 20), _rand((Lk, 1, D), 21), _rand((Lk, 1, D), 22), _rand((Lq, 1, D), 23)
    M = torch.rand(1, Lq, Lk, generator=torch.Generator().manual_seed(5)) > p
    r = orc.varlen_attention(q, k, v, [0, Lq], [0, Lk], p_dropout=p, keep_mask=[M], dout=do, dtype=torch.float64)
    P = r["probs"][0][0]
    pd = P * M[0] / (1 - p)
    assert torch.allclose(r["out"][:, 0], pd @ v[:, 0], atol=1e-12)
    assert torch.allclose(r["dv"][:, 0], pd.T @ do[:, 0], atol=1e-12)
    assert torch.allclose(r["softmax_d"][0][0], (1 - p) * (do[:, 0] * r["out"][:, 0]).sum(-1), atol=1e-12)


def test_golden_fixture_is_current():
    z = np.load(os.path.join(GOLDEN, "attention_small.npz"))
    q, k, v, do = (torch.tensor(z[n]).double() for n in ("q", "k", "v", "dout"))
    cu = z["cu_seqlens"].tolist()
    for causal, tag in ((False, "dense"), (True, "causal")):
        r = orc.varlen_attention(q, k, v, cu, cu, None, causal, dout=do, dtype=torch.float64)
        for name in ("out", "dq", "dk", "dv"):
            assert np.allclose(r[name].numpy(), z["%s_%s" % (tag, name)], atol=2e-6, rtol=1e-6)
        for b in range(2):
            assert np.allclose(r["lse"][b].numpy(), z["%s_lse%d" % (tag, b)], atol=2e-6)


# ---------------------------------------------------------------- Philox / dropout mask
def test_philox_known_answers():
    kat = json.load(open(os.path.join(GOLDEN, "philox_kat.json")))
    assert {v["rounds"] for v in kat["vectors"]} == {7, 10}
    for v in kat["vectors"]:
        got = orc.philox4x32([int(x, 16) for x in v["counter"]], [int(x, 16) for x in v["key"]], v["rounds"])
        assert ["%08x" % int(x) for x in got] == v["expect"]


def test_philox_vectorised_equals_scalar():
    c0 = np.arange(5, dtype=np.uint32)
    vec = orc.philox4x32((c0, 7, 9, 11), (123, 456), 7)
    for i in range(5):
        one = orc.philox4x32((int(c0[i]), 7, 9, 11), (123, 456), 7)
        assert [int(x[i]) for x in vec] == [int(x) for x in one]


def test_keep_threshold_and_rate():
    # fmha_api.cpp:110 computes floor(p_keep * 65535) for the uint16 comparison: values worked out by hand / exact
    # binary fractions (0.5 * 65535 = 32767.5, 0.75 * 65535 = 49151.25, 0.9 * 65535 = 58981.5)
    assert [orc.keep_threshold(x) for x in (0.0, 0.5, 0.25, 0.1)] == [65535, 32767, 49151, 58981]
    assert orc.keep_probability(0.0) == 1.0 and orc.keep_probability(0.5) == 0.5 and orc.keep_probability(0.25) == 0.75
    p = 0.17
    m = orc.dropout_keep_mask(seed=42, offset=8, bh=3, Lq=256, Lk=512, p_dropout=p)
    n = m.size
    kp = orc.keep_probability(p)
    z = (m.sum() - n * kp) / math.sqrt(n * kp * (1 - kp))
    assert abs(z) < 4.5, z
    # rows and columns individually look Bernoulli too (no stuck fields)
    assert abs(m.mean(0) - kp).max() < 0.12 and abs(m.mean(1) - kp).max() < 0.09


def test_dropout_mask_definition_scalar():
    """element-by-element evaluation of the definition in the docstring, independent of the vectorised code."""
    seed, offset, bh, p = (0x1234567 << 32) | 0x89ABCDEF, (5 << 32) | 12, 7, 0.3
    m = orc.dropout_keep_mask(seed, offset, bh, 11, 13, p)
    thr = orc.keep_threshold(p)
    key = (seed & 0xFFFFFFFF, ((seed >> 32) ^ (offset >> 32)) & 0xFFFFFFFF)
    for qi in range(11):
        for ki in range(13):
            f = 4 * (qi % 4) + ki % 4
            r = orc.philox4x32((2 * (ki // 4) + f // 8, qi // 4, bh, offset & 0xFFFFFFFF), key, 7)
            word = int(r[(f // 2) % 4])
            field = (word >> (16 * (f % 2))) & 0xFFFF
            assert bool(m[qi, ki]) == (field <= thr)


def test_dropout_mask_depends_on_all_inputs():
    base = orc.dropout_keep_mask(1, 0, 0, 64, 64, 0.5)
    assert (base != orc.dropout_keep_mask(2, 0, 0, 64, 64, 0.5)).any()
    assert (base != orc.dropout_keep_mask(1, 4, 0, 64, 64, 0.5)).any()
    assert (base != orc.dropout_keep_mask(1, 0, 1, 64, 64, 0.5)).any()
    assert (base != orc.dropout_keep_mask(1 + (1 << 32), 0, 0, 64, 64, 0.5)).any()
    assert (base == orc.dropout_keep_mask(1, 0, 0, 64, 64, 0.5)).all()
    assert (base[:32, :48] == orc.dropout_keep_mask(1, 0, 0, 32, 48, 0.5)).all()  # independent of the extent


# ---------------------------------------------------------------- block mask conversion, padding
def test_convert_blockmask_bruteforce():
    """every 3x3 and a sample of 4x4 masks against a per-element definition written independently."""
    def spec(m):
        nrow, ncol = m.shape
        out = -np.ones((ncol, nrow), dtype=np.int64)
        for c in range(ncol):
            rows = [r for r in range(nrow) if m[r, c]]
            for i, r in enumerate(rows):
                nz = [cc for cc in range(ncol) if m[r, cc]]
                out[c, i] = 4 * r + (nz[0] == c) + 2 * (nz[-1] == c)
        return out
    for bits in range(1 << 9):
        m = np.array([(bits >> i) & 1 for i in range(9)]).reshape(3, 3)
        assert (orc.convert_blockmask_ref(m) == spec(m)).all()
    rng = np.random.default_rng(0)
    for _ in range(200):
        m = rng.integers(0, 2, (4, 4))
        assert (orc.convert_blockmask_ref(m) == spec(m)).all()
    # worked example: rows 0..2, cols 0..1
    m = np.array([[1, 1], [0, 1], [1, 0]])
    assert orc.convert_blockmask_ref(m).tolist() == [[0 * 4 + 1, 2 * 4 + 3, -1], [0 * 4 + 2, 1 * 4 + 3, -1]]


def test_unpad_pad_roundtrip():
    rng = np.random.default_rng(1)
    x = rng.standard_normal((3, 7, 4))
    mask = np.array([[1, 1, 1, 0, 0, 0, 0], [1, 1, 1, 1, 1, 1, 1], [1, 0, 0, 0, 0, 0, 0]])
    rows, idx, cu, mx = orc.unpad_ref(x, mask)
    assert cu.tolist() == [0, 3, 10, 11] and mx == 7 and rows.shape == (11, 4)
    assert np.array_equal(orc.pad_ref(rows, idx, 3, 7), x * mask[..., None])


def test_rotary_ref_is_a_rotation_and_matches_the_elementwise_definition():
    """rotary_ref against the definition it cites evaluated literally (x * cos + rotate_half(x) * sin with repeated
    tables), norm preservation of every pair, angle addition (rotating by t1 then t2 = rotating by t1 + t2), and the
    conjugate being the inverse."""
    rng = np.random.default_rng(0)
    rows, H, dim = 7, 2, 8
    x = rng.standard_normal((rows, H, dim))
    inv_freq = 1.0 / (10000 ** (np.arange(0, dim, 2) / dim))
    ang = np.outer(np.arange(20), inv_freq)
    cos_h, sin_h = np.cos(ang), np.sin(ang)
    pos = np.array([0, 3, 5, 1, 19, 7, 2])
    got = orc.rotary_ref(x, cos_h, sin_h, pos)
    cos_f, sin_f = np.repeat(cos_h, 2, -1)[pos][:, None], np.repeat(sin_h, 2, -1)[pos][:, None]
    rot_half = np.stack([-x[..., 1::2], x[..., 0::2]], -1).reshape(x.shape)
    assert np.allclose(got, x * cos_f + rot_half * sin_f, atol=1e-14)
    assert np.allclose(got[..., 0::2] ** 2 + got[..., 1::2] ** 2, x[..., 0::2] ** 2 + x[..., 1::2] ** 2)
    assert np.allclose(orc.rotary_ref(got, cos_h, sin_h, pos, conjugate=True), x, atol=1e-14)
    twice = orc.rotary_ref(orc.rotary_ref(x, cos_h, sin_h, np.full(rows, 4)), cos_h, sin_h, np.full(rows, 9))
    assert np.allclose(twice, orc.rotary_ref(x, cos_h, sin_h, np.full(rows, 13)), atol=1e-13)
    assert np.allclose(orc.rotary_ref(x, cos_h, sin_h, np.zeros(rows, dtype=int)), x)


def test_alibi_bias_against_sdpa_float_mask():
    """varlen_attention with alibi_slopes against torch's scaled_dot_product_attention given the same bias as a float
    attn_mask (library routine), with and without a causal mask; slope 0 is no bias; gradients flow the same way."""
    g = torch.Generator().manual_seed(21)
    H, D, Lq, Lk = 3, 16, 37, 37
    q, k, v, do = (torch.randn(L, H, D, generator=g, dtype=torch.float64) for L in (Lq, Lk, Lk, Lq))
    slopes = torch.tensor([0.5, 0.0625, 0.0])
    cu = [0, Lq]
    for causal in (False, True):
        res = orc.varlen_attention(q, k, v, cu, cu, None, causal, dout=do, dtype=torch.float64, alibi_slopes=slopes)
        bias = orc.alibi_bias(slopes, Lq, Lk, dtype=torch.float64)
        if causal:
            bias = bias.masked_fill(torch.triu(torch.ones(Lq, Lk, dtype=torch.bool), 1), float("-inf"))
        qq, kk, vv = (x.transpose(0, 1).clone().requires_grad_() for x in (q, k, v))
        ref = torch.nn.functional.scaled_dot_product_attention(qq[None], kk[None], vv[None], attn_mask=bias[None])[0]
        ref.backward(do.transpose(0, 1))
        assert torch.allclose(res["out"].transpose(0, 1), ref, atol=1e-12)
        for name, t in (("dq", qq), ("dk", kk), ("dv", vv)):
            assert torch.allclose(res[name].transpose(0, 1), t.grad, atol=1e-11), name
        plain = orc.varlen_attention(q, k, v, cu, cu, None, causal, dtype=torch.float64)
        assert torch.equal(res["out"][:, 2], plain["out"][:, 2])          # head with slope 0
        assert not torch.allclose(res["out"][:, 0], plain["out"][:, 0], atol=1e-3)


def test_attn_bias_against_sdpa_float_mask_and_finite_differences():
    """varlen_attention with a bias tensor against torch's scaled_dot_product_attention given the same tensor as a float
    attn_mask (library routine): forward, and through its autograd dq, dk, dv and dbias; two ragged sequences share one
    (1, H, S, S) bias, whose gradient is then the sum over the batch; -inf entries spell a causal mask."""
    g = torch.Generator().manual_seed(33)
    H, D = 2, 8
    lens = [7, 5]
    S = max(lens)
    cu = [0, 7, 12]
    q, k, v, do = (torch.randn(sum(lens), H, D, generator=g, dtype=torch.float64) for _ in range(4))
    bias = torch.randn(1, H, S, S, generator=g, dtype=torch.float64)
    res = orc.varlen_attention(q, k, v, cu, cu, None, False, dout=do, dtype=torch.float64, attn_bias=bias)
    bb = bias.clone().requires_grad_()
    grads = {n: torch.zeros_like(q) for n in ("dq", "dk", "dv")}
    for b, L in enumerate(lens):
        sl = slice(cu[b], cu[b + 1])
        qq, kk, vv = (x[sl].transpose(0, 1).clone().requires_grad_() for x in (q, k, v))
        ref = torch.nn.functional.scaled_dot_product_attention(qq[None], kk[None], vv[None], attn_mask=bb[:, :, :L, :L])[0]
        ref.backward(do[sl].transpose(0, 1))
        assert torch.allclose(res["out"][sl].transpose(0, 1), ref, atol=1e-12)
        for n, t in (("dq", qq), ("dk", kk), ("dv", vv)):
            assert torch.allclose(res[n][sl].transpose(0, 1), t.grad, atol=1e-11), n
    assert torch.allclose(res["dbias"], bb.grad, atol=1e-11)           # summed over the two sequences that share it
    assert res["dbias"][0, :, 5:, :].abs().max() > 0 and torch.equal(res["dbias"][0, :, 7:, :], torch.zeros(H, 0, S, dtype=torch.float64))
    # a bias of 0 / -inf above the diagonal is the causal mask
    tri = torch.zeros(1, 1, S, S, dtype=torch.float64).masked_fill(torch.triu(torch.ones(S, S, dtype=torch.bool), 1), float("-inf"))
    a = orc.varlen_attention(q, k, v, cu, cu, None, False, dout=do, dtype=torch.float64, attn_bias=tri)
    c = orc.varlen_attention(q, k, v, cu, cu, None, True, dout=do, dtype=torch.float64)
    for n in ("out", "dq", "dk", "dv"):
        assert torch.allclose(a[n], c[n], atol=1e-12), n
    # dbias by central differences of sum(out * dout) on a few entries
    eps = 1e-6
    for (h, i, j) in ((0, 0, 0), (1, 3, 4), (0, 6, 2)):
        bp, bm = bias.clone(), bias.clone()
        bp[0, h, i, j] += eps
        bm[0, h, i, j] -= eps
        fp = (orc.varlen_attention(q, k, v, cu, cu, None, False, dtype=torch.float64, attn_bias=bp)["out"] * do).sum()
        fm = (orc.varlen_attention(q, k, v, cu, cu, None, False, dtype=torch.float64, attn_bias=bm)["out"] * do).sum()
        assert abs((fp - fm) / (2 * eps) - res["dbias"][0, h, i, j]) < 1e-7
