"""CPU oracle for the fused attention path.  TEST INFRASTRUCTURE ONLY: imported by tests/, by
__graft_entry__.smoke() and by bench.py's cpu_baseline leg as the checker / baseline, never by the product.

It restates, in plain fp32/fp64 PyTorch and NumPy on the host, the algorithm of the reference's attention path:

  attention_ref            benchmarks/benchmark_flash_attention.py:14-36  (the reference's own standard attention)
  varlen_attention         closed form of mha_fwd/mha_bwd for packed variable-length batches
                           (csrc/flash_attn/fmha_api.cpp:173-449; maths of fmha_fprop_kernel_1xN.h:365-638 and
                           fmha_dgrad_kernel_1xN_loop.h:304-661): out, softmax_lse, dq, dk, dv, softmax_d
  tiled_forward            the column-block recurrence of fmha_fprop_kernel_1xN.h:408-422,560-625 with a running
                           (lse, normalised O) carry
  philox4x32               round function / constants of csrc/flash_attn/src/philox.cuh:35-42,121-135
  dropout_keep_mask        this engine's mapping from (seed, offset, b, h, q, key) to keep/drop
  convert_blockmask_ref    specification of flash_attn/flash_blocksparse_attn_interface.py:8-40
  unpad_ref / pad_ref      specification of flash_attn/bert_padding.py:60-95
  rotary_ref               rotation of flash_attn/rotary.py:22-42 (x * cos + rotate_half(x) * sin) in fp64
  alibi_bias               -slope * |i - j| score bias of the engine's alibi_slopes extension (no reference counterpart)

How each function is pinned (the reference has no tests, golden vectors or fixtures of its own):
  attention_ref / varlen_attention forward: against torch.nn.functional.scaled_dot_product_attention (library
      routine), against hand-computable special cases (one key => o = v; causal first row => o = v0; uniform scores
      => mean of v) and against tiled_forward for several block widths;  lse: rows of exp(scale*S - lse) sum to 1.
  varlen_attention backward: autograd of the closed form, cross-checked with fp64 finite differences and with the
      explicit formulas dV = P^T dO, dS = P o (dP - D), dQ = scale dS K, dK = scale dS^T Q.
  philox4x32: the published Random123 known-answer vectors for philox4x32 with 10 rounds and with the 7 rounds
      the reference uses (tests/golden/philox_kat.json).
  dropout_keep_mask: it is the definition; tests compare the kernels' S_dmask signs to it bit for bit.
  convert_blockmask_ref: brute force over all small masks against an independent per-element definition.
  alibi_bias (inside varlen_attention): torch's scaled_dot_product_attention with the same bias as a float attn_mask;
      slope 0 is no bias; a bias that is constant along a row changes nothing.
  attn_bias (inside varlen_attention; the engine's tensor-bias extension): the same library routine with the tensor as float
      attn_mask, forward and - through its autograd - dq, dk, dv and dbias; -inf entries equal the causal mask they spell; a
      shared bias gets the sum of the per-(batch, head) gradients; fp64 finite differences on a tiny case.
  unpad_ref / pad_ref: round trip pad(unpad(x)) == x * mask, cu_seqlens against the cumulative sum of the lengths.
  rotary_ref: the cited definition evaluated literally; it is a rotation (norm kept, conjugate inverts it, angles add,
      position 0 is the identity).
PARITY UNPINNED (only running the CUDA reference could pin them; nothing in this pipeline can): the reference's
  fragment-permuted S_dmask layout and running-max scaling (gmem_tile.h:289-405), its thread-indexed Philox stream
  assignment (so masks are compared with this engine's own definition, not NVIDIA's), and bit-level fp16 rounding /
  ex2.approx behaviour of its kernels.
"""
import math

import numpy as np
import torch


# --------------------------------------------------------------------------------------------------
# Standard attention: benchmarks/benchmark_flash_attention.py:14-36
# --------------------------------------------------------------------------------------------------
def attention_ref(qkv, attn_mask, dropout_p, upcast=False, causal=False, keep_mask=None):
    """qkv (B, S, 3, H, D); attn_mask (B, S) bool, True = valid key.  Returns (B, S, H, D) in qkv's dtype.
    With keep_mask (B, H, S, S) bool the dropout pattern is given instead of drawn."""
    x = qkv.float() if upcast else qkv
    q, k, v = x.unbind(dim=2)
    S, d = qkv.shape[1], qkv.shape[-1]
    scores = torch.einsum("bthd,bshd->bhts", q, k / math.sqrt(d))
    scores = scores.masked_fill(~attn_mask[:, None, None, :], float("-inf"))
    if causal:
        scores = scores.masked_fill(torch.triu(torch.ones(S, S, dtype=torch.bool, device=qkv.device), 1), float("-inf"))
    attention = torch.softmax(scores, dim=-1)
    if keep_mask is not None:
        attention = attention * keep_mask.to(attention.dtype) / (1.0 - dropout_p)
    elif dropout_p > 0:
        attention = torch.nn.functional.dropout(attention, dropout_p)
    out = torch.einsum("bhts,bshd->bthd", attention, v)
    return out.to(dtype=qkv.dtype)


# --------------------------------------------------------------------------------------------------
# Closed form on packed variable-length batches
# --------------------------------------------------------------------------------------------------
def expand_block_layout(layout, Lq, Lk, device="cpu"):
    """bool (Lq, Lk) mask from a 0/1 layout of 16-row x 256-key blocks (fmha_api.cpp:509-515)."""
    m = torch.as_tensor(layout).bool().to(device)
    full = m.repeat_interleave(16, 0).repeat_interleave(256, 1)
    return full[:Lq, :Lk]


def _score_mask(Lq, Lk, causal, layout, device="cpu"):
    valid = torch.ones(Lq, Lk, dtype=torch.bool, device=device)
    if causal:  # query i sees keys j <= i, both counted from the start of the sequence (mask.h:69)
        valid &= torch.arange(Lk, device=device)[None, :] <= torch.arange(Lq, device=device)[:, None]
    if layout is not None:
        valid &= expand_block_layout(layout, Lq, Lk, device)
    return valid


def alibi_bias(slopes, Lq, Lk, device="cpu", dtype=torch.float32):
    """(H, Lq, Lk) additive score bias -slope[h] * |i - j| (ALiBi, Press et al. 2021, mirrored for keys after the
    query).  The reference has no attention bias (its README lists it as planned, README.md:49-50); this is the
    definition the engine's alibi_slopes extension follows."""
    sl = torch.as_tensor(slopes, dtype=dtype, device=device)
    dist = (torch.arange(Lq, device=device)[:, None] - torch.arange(Lk, device=device)[None, :]).abs().to(dtype)
    return -sl[:, None, None] * dist[None]


def varlen_attention(q, k, v, cu_q, cu_k, softmax_scale=None, causal=False, p_dropout=0.0, keep_mask=None,
                     layout=None, dout=None, dtype=torch.float32, alibi_slopes=None, attn_bias=None):
    """Closed-form attention forward (+ backward if dout is given) on packed tensors.

    q (total_q, H, D), k, v (total_k, H, D) any float dtype (upcast to `dtype`); cu_q, cu_k int sequences of length
    B+1; keep_mask: list of B bool tensors (H, Lq_b, Lk_b) or None; layout: 0/1 (rows/16, keys/256) block layout.
    Returns dict(out, lse [list of (H, Lq_b)], dq, dk, dv, softmax_d [list of (H, Lq_b)], probs [list]).
    Rows with no visible key give out = 0, lse = -inf (fmha_fprop_kernel_1xN.h:575,606; fmha_api.cpp:519).
    softmax_d is keep * rowsum(dO o O) (fmha_dgrad_kernel_1xN_loop.h:15-30,226).
    attn_bias (the engine's extension, no reference counterpart): (1 or B, 1 or H, >= Lq, >= Lk), added to the scaled scores
    at positions counted inside each sequence; with dout the result also holds dbias, in attn_bias's shape.
    """
    cu_q = [int(x) for x in cu_q]
    cu_k = [int(x) for x in cu_k]
    B = len(cu_q) - 1
    D = q.shape[-1]
    scale = D ** -0.5 if softmax_scale is None else float(softmax_scale)
    keep = 1.0 - p_dropout
    qf = q.detach().to(dtype).requires_grad_(dout is not None)
    kf = k.detach().to(dtype).requires_grad_(dout is not None)
    vf = v.detach().to(dtype).requires_grad_(dout is not None)
    bf = attn_bias.detach().to(dtype).requires_grad_(dout is not None) if attn_bias is not None else None
    outs, lses, probs = [], [], []
    for b in range(B):
        qb = qf[cu_q[b]:cu_q[b + 1]].transpose(0, 1)  # (H, Lq, D)
        kb = kf[cu_k[b]:cu_k[b + 1]].transpose(0, 1)
        vb = vf[cu_k[b]:cu_k[b + 1]].transpose(0, 1)
        Lq, Lk = qb.shape[1], kb.shape[1]
        s = torch.einsum("hqd,hkd->hqk", qb, kb) * scale
        if alibi_slopes is not None:
            s = s + alibi_bias(alibi_slopes, Lq, Lk, qf.device, dtype)
        if bf is not None:
            s = s + bf[b if bf.shape[0] > 1 else 0, :, :Lq, :Lk]
        valid = _score_mask(Lq, Lk, causal, layout, qf.device)
        s = s.masked_fill(~valid[None], float("-inf"))
        lse = torch.logsumexp(s, dim=-1)  # -inf for empty rows
        p = torch.exp(s - torch.where(torch.isinf(lse), torch.zeros_like(lse), lse)[..., None])
        p = torch.where(valid[None], p, torch.zeros_like(p))
        pd = p
        if keep_mask is not None:
            pd = p * keep_mask[b].to(device=qf.device, dtype=dtype) / keep
        ob = torch.einsum("hqk,hkd->hqd", pd, vb)
        outs.append(ob.transpose(0, 1))
        lses.append(lse.detach())
        probs.append(p.detach())
    out = torch.cat(outs, dim=0) if outs else qf.new_zeros(q.shape)
    res = {"out": out.detach(), "lse": lses, "probs": probs}
    if dout is not None:
        do = dout.detach().to(dtype)
        out.backward(do)
        res["dq"], res["dk"], res["dv"] = qf.grad, kf.grad, vf.grad
        if bf is not None:
            res["dbias"] = bf.grad if bf.grad is not None else torch.zeros_like(bf)
        dsum = (do * out.detach()).sum(-1) * keep  # (total_q, H)
        res["softmax_d"] = [dsum[cu_q[b]:cu_q[b + 1]].transpose(0, 1) for b in range(B)]
    return res


def explicit_backward(q, k, v, dout, scale, causal=False):
    """Single sequence, single head, no dropout: the backward written out term by term
    (fmha_dgrad_kernel_1xN_loop.h:333-560 without tiling).  q (Lq, D), k, v (Lk, D), float64 arrays."""
    q, k, v, dout = (np.asarray(x, dtype=np.float64) for x in (q, k, v, dout))
    s = q @ k.T * scale
    if causal:
        s = np.where(np.arange(k.shape[0])[None, :] <= np.arange(q.shape[0])[:, None], s, -np.inf)
    m = s.max(-1, keepdims=True)
    e = np.exp(s - m)
    lse = m[:, 0] + np.log(e.sum(-1))
    p = np.exp(s - lse[:, None])
    o = p @ v
    dv = p.T @ dout
    dp = dout @ v.T
    dsum = (dout * o).sum(-1, keepdims=True)
    ds = p * (dp - dsum)
    return {"out": o, "lse": lse, "dq": ds @ k * scale, "dk": ds.T @ q * scale, "dv": dv, "softmax_d": dsum[:, 0]}


def tiled_forward(q, k, v, scale, block_n, causal=False, block_m=16):
    """The reference's loop nest for one (batch, head): key blocks of width block_n outside, 16-row query blocks
    inside, carrying (lse, normalised O) between key blocks (fmha_fprop_kernel_1xN.h:255,270,408-422,560-625).
    q (Lq, D), k, v (Lk, D) float64.  Returns (o, lse)."""
    q, k, v = (np.asarray(x, dtype=np.float64) for x in (q, k, v))
    Lq, Lk, D = q.shape[0], k.shape[0], q.shape[1]
    o = np.zeros((Lq, D))
    lse = np.full((Lq,), -np.inf)
    for c0 in range(0, Lk, block_n):
        kc, vc = k[c0:c0 + block_n], v[c0:c0 + block_n]
        for r0 in range(0, Lq, block_m):
            r1 = min(r0 + block_m, Lq)
            if causal and r1 - 1 < c0:  # whole row block above the diagonal of this key block
                continue
            s = q[r0:r1] @ kc.T
            if causal:
                cols = c0 + np.arange(kc.shape[0])[None, :]
                rows = np.arange(r0, r1)[:, None]
                s = np.where(cols <= rows, s, -np.inf)
            m = np.maximum(s.max(-1) * scale, lse[r0:r1])      # running max includes the previous lse
            m_safe = np.where(np.isinf(m), 0.0, m)
            p = np.exp(s * scale - m_safe[:, None])
            w = np.exp(lse[r0:r1] - m_safe)                      # weight of the carried, normalised O
            l_new = p.sum(-1) + w
            acc = p @ vc
            with np.errstate(divide="ignore", invalid="ignore"):
                o[r0:r1] = np.where(l_new[:, None] > 0, (o[r0:r1] * w[:, None] + acc) / l_new[:, None], 0.0)
                lse[r0:r1] = np.where(l_new > 0, m_safe + np.log(l_new), -np.inf)
    return o, lse


# --------------------------------------------------------------------------------------------------
# Philox-4x32 (philox.cuh:35-42,121-135) and the dropout mask definition
# --------------------------------------------------------------------------------------------------
_PHILOX_M0 = np.uint64(0xD2511F53)
_PHILOX_M1 = np.uint64(0xCD9E8D57)
_PHILOX_W0 = 0x9E3779B9
_PHILOX_W1 = 0xBB67AE85
_MASK32 = np.uint64(0xFFFFFFFF)


def philox4x32(counter, key, rounds):
    """counter: 4 arrays (or ints) of uint32, key: 2 ints; returns 4 uint32 arrays.  Vectorised over the counter."""
    c = [np.asarray(x, dtype=np.uint64) & _MASK32 for x in counter]
    c = list(np.broadcast_arrays(*c))
    k0, k1 = int(key[0]) & 0xFFFFFFFF, int(key[1]) & 0xFFFFFFFF
    for _ in range(rounds):
        p0 = _PHILOX_M0 * c[0]
        p1 = _PHILOX_M1 * c[2]
        n0 = ((p1 >> np.uint64(32)) ^ c[1] ^ np.uint64(k0)) & _MASK32
        n1 = p1 & _MASK32
        n2 = ((p0 >> np.uint64(32)) ^ c[3] ^ np.uint64(k1)) & _MASK32
        n3 = p0 & _MASK32
        c = [n0, n1, n2, n3]
        k0 = (k0 + _PHILOX_W0) & 0xFFFFFFFF
        k1 = (k1 + _PHILOX_W1) & 0xFFFFFFFF
    return [x.astype(np.uint32) for x in c]


def keep_threshold(p_dropout):
    """uint16 threshold of fmha_api.cpp:110; an element is kept iff its 16-bit random field <= threshold."""
    return int(math.floor((1.0 - p_dropout) * 65535.0))


def keep_probability(p_dropout):
    return (keep_threshold(p_dropout) + 1) / 65536.0


def dropout_keep_mask(seed, offset, bh, Lq, Lk, p_dropout):
    """bool (Lq, Lk): keep decision of score element (q, key) of flattened (batch*H + head) index bh.

    Definition (shared by the forward, the backward and the S_dmask dump of the HIP engine): the 4x4 micro-block
    (Q4, K4) = (q // 4, key // 4) draws Philox-4x32-7 twice, with counter (2*K4 + call, Q4, bh, offset_lo) and key
    (seed_lo, seed_hi ^ offset_hi); call = (q % 4) // 2.  Element (q % 4, key % 4) takes 16-bit field
    f = 4*(q % 4) + key % 4 of the 16 fields of the two calls: bits 16*(f % 2).. of word (f // 2) % 4 of call f // 8.
    """
    thr = keep_threshold(p_dropout)
    qi = np.arange(Lq, dtype=np.int64)[:, None]
    ki = np.arange(Lk, dtype=np.int64)[None, :]
    f = 4 * (qi % 4) + (ki % 4)
    call = f // 8
    word = (f // 2) % 4
    half = f % 2
    c0 = 2 * (ki // 4) + call
    c1 = np.broadcast_to(qi // 4, c0.shape)
    key = (seed & 0xFFFFFFFF, ((seed >> 32) ^ (offset >> 32)) & 0xFFFFFFFF)
    r = philox4x32((c0, c1, np.full(c0.shape, bh), np.full(c0.shape, offset & 0xFFFFFFFF)), key, 7)
    words = np.stack(r, axis=0)  # (4, Lq, Lk)
    w = np.take_along_axis(words, word[None].astype(np.int64), axis=0)[0]
    field = (w >> (16 * half).astype(np.uint32)) & np.uint32(0xFFFF)
    return field <= thr


# --------------------------------------------------------------------------------------------------
# Block-sparse mask conversion: flash_blocksparse_attn_interface.py:8-40
# --------------------------------------------------------------------------------------------------
def convert_blockmask_ref(blockmask):
    """(nrow, ncol) 0/1 -> int32 (ncol, nrow).  Row c of the result lists, in ascending order, the rows r with
    blockmask[r, c] != 0 as 4*r + 1*[c is the first nonzero column of row r] + 2*[c is the last nonzero column of
    row r], padded with -1."""
    m = np.asarray(blockmask) != 0
    nrow, ncol = m.shape
    out = np.full((ncol, nrow), -1, dtype=np.int32)
    for c in range(ncol):
        n = 0
        for r in range(nrow):
            if m[r, c]:
                cols = np.nonzero(m[r])[0]
                out[c, n] = 4 * r + (1 if cols[0] == c else 0) + (2 if cols[-1] == c else 0)
                n += 1
    return out


# --------------------------------------------------------------------------------------------------
# Padding helpers: bert_padding.py:60-95
# --------------------------------------------------------------------------------------------------
def unpad_ref(hidden, mask):
    """hidden (B, S, dim), mask (B, S) 0/1 -> (rows of valid tokens, flat indices, cu_seqlens int32, max_len)."""
    hidden = np.asarray(hidden)
    mask = np.asarray(mask) != 0
    B, S = mask.shape
    idx = np.array([b * S + s for b in range(B) for s in range(S) if mask[b, s]], dtype=np.int64)
    lens = mask.sum(-1)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    return hidden.reshape(B * S, -1)[idx], idx, cu, int(lens.max()) if B else 0


def pad_ref(rows, idx, B, S):
    rows = np.asarray(rows)
    out = np.zeros((B * S, rows.shape[-1]), dtype=rows.dtype)
    out[np.asarray(idx)] = rows
    return out.reshape(B, S, -1)


# --------------------------------------------------------------------------------------------------
# Rotary position embedding (flash_attn/rotary.py:22-42,66-87)
# --------------------------------------------------------------------------------------------------
def rotary_ref(x, cos_half, sin_half, positions, conjugate=False):
    """x (rows, nheads, dim) float array; cos_half, sin_half (table_rows, dim / 2); positions (rows,) ints.
    Pair (x[2i], x[2i+1]) of row r becomes (x[2i] c - x[2i+1] s, x[2i+1] c + x[2i] s), c = cos_half[positions[r], i]:
    x * cos + rotate_half(x) * sin with rotate_half(x) = (-x1, x0, -x3, x2, ...) and each table entry repeated twice
    (rotary.py:22-42, 84-85).  Evaluated in float64."""
    x = np.asarray(x, dtype=np.float64)
    c = np.asarray(cos_half, dtype=np.float64)[np.asarray(positions)][:, None, :]
    s = np.asarray(sin_half, dtype=np.float64)[np.asarray(positions)][:, None, :]
    if conjugate:
        s = -s
    a, b = x[..., 0::2], x[..., 1::2]
    out = np.empty_like(x)
    out[..., 0::2] = a * c - b * s
    out[..., 1::2] = b * c + a * s
    return out
