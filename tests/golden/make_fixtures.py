"""Writes tests/golden/attention_small.npz from the oracle (float64).  Run from the repository root:
    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle.attention_oracle import varlen_attention  # noqa: E402


def main():
    g = torch.Generator().manual_seed(1234)
    lens = [13, 20]
    cu = [0, 13, 33]
    H, D = 2, 16
    # values are multiples of 1/8 so that they are exact in fp16 and bf16
    q = torch.randint(-16, 17, (33, H, D), generator=g).double() / 8
    k = torch.randint(-16, 17, (33, H, D), generator=g).double() / 8
    v = torch.randint(-16, 17, (33, H, D), generator=g).double() / 8
    do = torch.randint(-16, 17, (33, H, D), generator=g).double() / 8
    out = {"q": q.numpy().astype(np.float32), "k": k.numpy().astype(np.float32), "v": v.numpy().astype(np.float32),
           "dout": do.numpy().astype(np.float32), "cu_seqlens": np.array(cu, np.int32),
           "lens": np.array(lens, np.int32)}
    for causal in (False, True):
        r = varlen_attention(q, k, v, cu, cu, None, causal, dout=do, dtype=torch.float64)
        tag = "causal" if causal else "dense"
        f32 = lambda t: t.numpy().astype(np.float32)  # expected values are kept in float32 to keep the file small
        out[tag + "_out"] = f32(r["out"])
        out[tag + "_dq"], out[tag + "_dk"], out[tag + "_dv"] = f32(r["dq"]), f32(r["dk"]), f32(r["dv"])
        for b in range(2):
            out["%s_lse%d" % (tag, b)] = f32(r["lse"][b])
            out["%s_softmax_d%d" % (tag, b)] = f32(r["softmax_d"][b])
    np.savez_compressed(os.path.join(HERE, "attention_small.npz"), **out)
    print("wrote", os.path.join(HERE, "attention_small.npz"))


if __name__ == "__main__":
    main()
