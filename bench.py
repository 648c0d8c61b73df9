#!/usr/bin/env python3
"""Benchmark of the fused attention path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--all] [--no-cpu] [--no-configs] [--backward PLAN]

One step = one forward + one backward pass of the headline workload (fp16, B=8, H=12, d=64, N=2048, packed qkv,
non-causal, dropout 0, synthetic N(0,1) data resident in HBM), called through the C ABI.  Prints ONE JSON line:
whole-job fwd+bwd TFLOP/s (4*B*H*N^2*d forward, 2.5x that backward), the roofline position of the dominant kernel
(the backward dK/dV kernel, timed with HIP events recorded around it on its stream) and the CPU baseline (the
oracle's standard attention, fp32 PyTorch on the host cores, timed on a bounded sample of the same workload).
The line also carries `configs` (the other BASELINE configurations: TFLOP/s, share of the MFMA peak and the HBM GB/s of
their algorithmic bytes; --no-configs skips them) and `sustained_mfma` (what a library fp16 GEMM reaches on this GPU in
the same process: the matrix cores' rate under their power limit, to read the attention figures against).
--all additionally prints the configurations as a table to stderr, with PyTorch standard attention timed beside each,
and the unpad / pad / rotary kernels.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "flash-attention_amd"))
sys.path.insert(0, ROOT)

MFMA_PEAK_TFLOPS = 2500.0  # MI355X dense fp16 / bf16
HBM_PEAK_GBS = 8000.0


def attention_flops(B, H, N, D, causal=False):
    f = 4.0 * B * H * N * N * D
    return f * (0.5 if causal else 1.0)


def sparse_layout(torch, N, density=0.25, seed=0, rows_per_draw=1):
    """Block mask at the interface's granularity (rows of 16 queries, columns of 256 keys): the diagonal band of
    256 x 256 blocks plus seeded random blocks, `density` of all blocks active in expectation.  One random draw decides
    rows_per_draw consecutive mask rows (16: the random blocks are 256 x 256 like the band's)."""
    nrow, ncol = N // 16, N // 256
    band = (torch.arange(nrow)[:, None] // 16) == torch.arange(ncol)[None, :]
    extra = (density - 1.0 / ncol) / (1.0 - 1.0 / ncol)
    draws = torch.rand(nrow // rows_per_draw, ncol, generator=torch.Generator().manual_seed(seed)) < extra
    return band | draws.repeat_interleave(rows_per_draw, 0)


class Workload:
    def __init__(self, torch, B, H, D, N, dtype, causal=False, p=0.0, lens=None, seed=0, blockmask=None, alibi=False):
        self.B, self.H, self.D, self.N, self.dtype, self.causal, self.p = B, H, D, N, dtype, causal, p
        # ALiBi slopes 2^(-8 (h + 1) / H), one per head (the engine's attention-bias extension)
        self.alibi = torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)], dtype=torch.float32, device="cuda") \
            if alibi else None
        self.blockmask = blockmask  # (N/16, N/256) bool: the block-sparse entry points are timed instead
        g = torch.Generator(device="cuda").manual_seed(seed)
        lens = lens or [N] * B
        self.lens = lens
        total = sum(lens)
        self.qkv = torch.randn(total, 3, H, D, device="cuda", dtype=torch.float32, generator=g).to(dtype)
        self.dout = torch.randn(total, H, D, device="cuda", dtype=torch.float32, generator=g).to(dtype)
        cu = [0]
        for L in lens:
            cu.append(cu[-1] + L)
        self.cu = torch.tensor(cu, dtype=torch.int32, device="cuda")
        self.max_s = max(lens)
        self.dqkv = torch.empty_like(self.qkv)
        # the views a step passes in are made once (a view costs the host more than a microsecond, six of them are a
        # tenth of a short-sequence step)
        self.q, self.k, self.v = self.qkv[:, 0], self.qkv[:, 1], self.qkv[:, 2]
        self.dq, self.dk, self.dv = self.dqkv[:, 0], self.dqkv[:, 1], self.dqkv[:, 2]
        self.scale = D ** -0.5
        self.fwd_flops = sum(4.0 * H * L * L * D for L in lens) * (0.5 if causal else 1.0)
        if blockmask is not None:  # only the active 16 x 256 blocks are counted
            self.fwd_flops = 4.0 * B * H * D * 16 * 256 * float(blockmask.sum())
            from flash_attn.flash_blocksparse_attn_interface import convert_blockmask
            self.blockmask = convert_blockmask(blockmask.cuda(), causal=False)  # the entry points' own column-major form
            # the order the workgroups take the 16-row blocks in, worked out once per layout (as the autograd functions do)
            from flash_attn import flash_attn_gfx950 as be
            self.row_order = be.blockmask_row_order(blockmask.cuda()) if os.environ.get("FA_BENCH_ROW_ORDER", "1") != "0" else None
        self.bytes_fwd = 4 * total * H * D * 2 + 4 * B * H * self.max_s          # q,k,v read + o written, lse
        self.bytes_bwd = 8 * total * H * D * 2 + 2 * 4 * B * H * self.max_s      # q,k,v,o,do read + dq,dk,dv written
        # dropout (dense): the forward leaves its keep decisions, one bit per score, for the backward's two kernels, as
        # the autograd functions do (flash_attn_interface.py); the buffer is made once, like the tensors
        self.keep_words = None
        if p > 0 and blockmask is None:
            from flash_attn import flash_attn_gfx950 as be
            self.keep_words = be.new_keep_words(self.q, self.cu, self.max_s, self.max_s, p)
            if self.keep_words is not None:
                bits = sum(H * L * L for L in lens) / 8
                self.bytes_fwd += bits
                self.bytes_bwd += 2 * bits

    def forward(self, be):
        q, k, v = self.q, self.k, self.v
        if self.blockmask is not None:
            self.out, self.lse = be.fwd_block(q, k, v, self.cu, self.cu, self.blockmask, self.max_s, self.max_s, self.p,
                                              self.scale, self.causal, False, None, row_order=self.row_order)
            return
        self.out, self.lse = be.fwd(q, k, v, self.cu, self.cu, self.max_s, self.max_s, self.p, self.scale, False,
                                    self.causal, False, None, self.alibi, self.keep_words)

    def backward(self, be, events=None):
        q, k, v = self.q, self.k, self.v
        dq, dk, dv = self.dq, self.dk, self.dv
        if self.blockmask is not None:
            if events is not None:
                events[0].record()
            be.bwd_block(self.dout, q, k, v, self.out, self.lse, dq, dk, dv, self.cu, self.cu, self.blockmask, self.max_s,
                         self.max_s, self.p, self.scale, self.causal, None, row_order=self.row_order)
            if events is not None:
                events[1].record()  # whole backward: the sparse entry point has no per-kernel hook
            return
        be.bwd(self.dout, q, k, v, self.out, self.lse, dq, dk, dv, self.cu, self.cu, self.max_s, self.max_s, self.p,
               self.scale, False, self.causal, None, main_kernel_events=events, alibi_slopes=self.alibi,
               keep_words=self.keep_words)


def time_steps(torch, be, w, steps, warmup, settle_s=0.2):
    # The clock governor needs some tens of milliseconds of load before the frequency (and so a step's duration)
    # stops moving: run untimed steps for settle_s seconds first, then the requested warm-up and timed steps.
    t_end = time.perf_counter() + settle_s
    while time.perf_counter() < t_end:
        for _ in range(10):
            w.forward(be)
            w.backward(be)
        torch.cuda.synchronize()
    for _ in range(warmup):
        w.forward(be)
        w.backward(be)
    torch.cuda.synchronize()
    ev = lambda: torch.cuda.Event(enable_timing=True)
    # HIP events around the dK/dV kernel on every 4th step of the timed region (an event record costs the stream a few
    # microseconds, so not on every step)
    kern = [(ev(), ev()) if i % 4 == 0 else None for i in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        w.forward(be)
        w.backward(be, kern[i])
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ks = [k for k in kern if k is not None]
    bwd_main_ms = sum(a.elapsed_time(b) for a, b in ks) / len(ks)
    # forward / backward split: a separate, shorter pass with events between the two halves of a step
    n2 = max(10, steps // 4)
    marks = [(ev(), ev(), ev()) for _ in range(n2)]
    for i in range(n2):
        marks[i][0].record()
        w.forward(be)
        marks[i][1].record()
        w.backward(be)
        marks[i][2].record()
    torch.cuda.synchronize()
    fwd_ms = sum(a.elapsed_time(b) for a, b, _ in marks) / n2
    bwd_ms = sum(b.elapsed_time(c) for _, b, c in marks) / n2
    return {"wall_ms": wall_ms, "ms_per_step": wall_ms / steps, "fwd_ms": fwd_ms, "bwd_ms": bwd_ms,
            "bwd_main_kernel_ms": bwd_main_ms}


def torch_attention_ms(torch, w, iters=8, want_memory=False):
    """Forward + backward of standard attention written with PyTorch ops in the workload's own dtype on the GPU - the
    comparison point of every speed-up the reference publishes (attention_ref, benchmarks/benchmark_flash_attention.py:
    14-36, 60-66: scores, key-padding and causal masks as -inf, softmax, dropout, attn @ v on a padded batch)."""
    B, H, D, N = w.B, w.H, w.D, w.max_s
    qkv = torch.zeros(B, N, 3, H, D, device="cuda", dtype=w.dtype)
    dout = torch.zeros(B, N, H, D, device="cuda", dtype=w.dtype)
    keep = torch.zeros(B, N, dtype=torch.bool, device="cuda")
    cu = w.cu.tolist()
    for b, L in enumerate(w.lens):
        qkv[b, :L] = w.qkv[cu[b]:cu[b + 1]]
        dout[b, :L] = w.dout[cu[b]:cu[b + 1]]
        keep[b, :L] = True
    qkv.requires_grad_()
    ragged = min(w.lens) < N
    causal_mask = torch.triu(torch.ones(N, N, dtype=torch.bool, device="cuda"), 1) if w.causal else None
    bias = None
    if w.alibi is not None:  # (H, N, N) additive bias, as a model without a fused kernel would hold it
        pos = torch.arange(N, device="cuda")
        bias = (-w.alibi[:, None, None] * (pos[:, None] - pos[None, :]).abs()[None]).to(w.dtype)

    def step():
        q, k, v = qkv.unbind(dim=2)
        scores = torch.einsum("bthd,bshd->bhts", q * w.scale, k)
        if bias is not None:
            scores = scores + bias[None]
        if ragged:
            scores = scores.masked_fill(~keep[:, None, None, :], float("-inf"))
        if causal_mask is not None:
            scores = scores.masked_fill(causal_mask, float("-inf"))
        attn = torch.nn.functional.dropout(torch.softmax(scores, dim=-1), w.p)
        out = torch.einsum("bhts,bshd->bthd", attn, v)
        qkv.grad = None
        out.backward(dout)

    for _ in range(3):
        step()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        step()
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / iters
    if not want_memory:
        return ms
    # peak device memory of one step beyond what is allocated before it (inputs, dout, the previous gradient)
    qkv.grad = None
    torch.cuda.synchronize()
    base = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    step()
    torch.cuda.synchronize()
    return ms, torch.cuda.max_memory_allocated() - base


def fused_step_memory(torch, w):
    """Peak device memory of one forward + backward through the public autograd function beyond what is allocated
    before it (out, softmax_lse, dqkv; no N x N tensor)."""
    from flash_attn.flash_attn_interface import flash_attn_unpadded_qkvpacked_func
    qkv = w.qkv.detach().clone().requires_grad_()

    def step():
        qkv.grad = None
        out = flash_attn_unpadded_qkvpacked_func(qkv, w.cu, w.max_s, w.p, causal=w.causal)
        out.backward(w.dout)

    step()
    qkv.grad = None
    torch.cuda.synchronize()
    base = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    step()
    torch.cuda.synchronize()
    return torch.cuda.max_memory_allocated() - base


def cpu_baseline(torch, B, H, D, N, budget_s=20.0):
    """The oracle's standard attention (attention_ref: fp32, PyTorch ops on the host cores), forward + backward through
    autograd, on a bounded sample of the headline workload: whole batches of (B, N) are repeated until about
    `budget_s` seconds of CPU work have been spent (at least one repetition)."""
    from oracle.attention_oracle import attention_ref
    torch.manual_seed(0)
    qkv = torch.randn(B, N, 3, H, D, dtype=torch.float32, requires_grad=True)
    dout = torch.randn(B, N, H, D, dtype=torch.float32)
    mask = torch.ones(B, N, dtype=torch.bool)
    reps, spent = 0, 0.0
    while reps < 1 or (spent < budget_s and spent + spent / reps < 1.5 * budget_s):
        t0 = time.perf_counter()
        out = attention_ref(qkv, mask, 0.0, upcast=True)
        out.backward(dout)
        qkv.grad = None
        spent += time.perf_counter() - t0
        reps += 1
    flops = 3.5 * attention_flops(B, H, N, D) * reps
    return {"value": round(flops / spent / 1e12, 4), "unit": "TFLOP/s", "cores": torch.get_num_threads(),
            "kind": "port", "ms_per_step": round(spent / reps * 1e3, 1),
            "sample": "%d repetition(s) of the full B=%d H=%d d=%d N=%d fp32 batch, fwd+bwd via autograd, %.1f s of host time"
                      % (reps, B, H, D, N, spent)}


def device_peak(torch):
    """Dense fp16 MFMA rate from what the device reports: compute units x 4096 flop/clock x the maximum shader clock
    (v_mfma_f32_32x32x16_f16 = 32768 flop in 32 cycles on each of a compute unit's 4 SIMDs)."""
    import ctypes
    props = torch.cuda.get_device_properties(0)
    cus = int(props.multi_processor_count)
    mhz = 0.0
    try:  # hipDeviceAttributeClockRate = 5: peak clock in kHz (torch's device properties do not carry it)
        khz = ctypes.c_int(0)
        if ctypes.CDLL("libamdhip64.so").hipDeviceGetAttribute(ctypes.byref(khz), 5, 0) == 0:
            mhz = khz.value / 1e3
    except OSError:
        pass
    return {"name": props.name, "compute_units": cus, "max_clock_mhz": round(mhz, 1),
            "tflops": round(cus * 4096 * mhz * 1e6 / 1e12, 1) if mhz else None}


def sustained_mfma(torch, n=8192, iters=20):
    """fp16 and bf16 torch.matmul (hipBLASLt / rocBLAS) on random n x n operands, timed after a settle phase: a library
    routine's answer to what the matrix cores sustain on this GPU (they are power limited on operands that toggle)."""
    out = {"what": "torch.matmul %d^3, random N(0,1) operands, after 0.3 s of the same GEMM" % n}
    for name, dt in (("fp16_tflops", torch.float16), ("bf16_tflops", torch.bfloat16)):
        a = torch.randn(n, n, device="cuda", dtype=dt)
        b = torch.randn(n, n, device="cuda", dtype=dt)
        t_end = time.perf_counter() + 0.3
        while time.perf_counter() < t_end:
            for _ in range(5):
                a @ b
            torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            a @ b
        e1.record()
        torch.cuda.synchronize()
        out[name] = round(2.0 * n ** 3 / (e0.elapsed_time(e1) / iters * 1e-3) / 1e12, 1)
        del a, b
    return out


def graph_replay_ms(torch, fn, calls=20, replays=5):
    """Milliseconds per call of fn, with `calls` of them captured in a HIP graph and the replays timed: for kernels that
    run shorter than their Python call takes (argument checks, ctypes), a loop of calls would time the host.  The C ABI
    neither allocates nor synchronises, so its calls can be captured."""
    for _ in range(5):
        fn()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            for _ in range(calls):
                fn()
    torch.cuda.current_stream().wait_stream(side)
    graph.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(replays):
        graph.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / (calls * replays)


TRAFFIC_PROFILE = os.path.join("profiles", "headline_fp16_b8_h12_d64_n2048_hbm_traffic.md")


def measured_traffic():
    """HBM bytes per launch of the dominant kernel, from the committed rocprofv3 FETCH_SIZE / WRITE_SIZE summary (the line
    `traffic_bytes_per_launch(<kernel>): <bytes>` there); None if the file does not carry it."""
    try:
        for line in open(os.path.join(ROOT, TRAFFIC_PROFILE)):
            if line.startswith("traffic_bytes_per_launch(fa_bwd_dkdv_kernel"):
                return float(line.split(":")[1])
    except OSError:
        pass
    return None


def config_list(torch):
    return [
        ("BERT varlen p=0.1 fp16", dict(B=8, H=12, D=64, N=512, dtype=torch.float16, p=0.1,
                                        lens=torch.randint(256, 513, (8,), generator=torch.Generator().manual_seed(0)).tolist())),
        # the configuration of the reference's own script (benchmarks/benchmark_flash_attention.py:39-70)
        ("reference script B64 H16 p=0.1", dict(B=64, H=16, D=64, N=1024, dtype=torch.float16, p=0.1,
                                                lens=torch.randint(1004, 1024, (64,), generator=torch.Generator().manual_seed(0)).tolist())),
        ("GPT2 causal bf16 N=1024", dict(B=8, H=12, D=64, N=1024, dtype=torch.bfloat16, causal=True)),
        ("GPT2 causal bf16 N=2048", dict(B=8, H=12, D=64, N=2048, dtype=torch.bfloat16, causal=True)),
        ("GPT2 causal bf16 N=4096", dict(B=8, H=12, D=64, N=4096, dtype=torch.bfloat16, causal=True)),
        ("  + ALiBi slopes, N=2048", dict(B=8, H=12, D=64, N=2048, dtype=torch.bfloat16, causal=True, alibi=True)),
        ("d128 fp16 N=2048", dict(B=16, H=12, D=128, N=2048, dtype=torch.float16)),
        ("d128 fp16 N=2048 causal", dict(B=16, H=12, D=128, N=2048, dtype=torch.float16, causal=True)),
        ("blocksparse 25% 16x256", dict(B=4, H=16, D=64, N=4096, dtype=torch.float16, blockmask=sparse_layout(torch, 4096))),
        ("blocksparse 25% 256x256", dict(B=4, H=16, D=64, N=4096, dtype=torch.float16,
                                         blockmask=sparse_layout(torch, 4096, rows_per_draw=16))),
    ]


def tile_sweep(torch, be, steps, warmup):
    """Full-size (128 query rows / keys per workgroup) against half-size tiles (64 rows, wave pairs split the keys) of the
    forward and the dQ kernel on launches of growing size: the table small_launch() (csrc/fa_params.h) takes its threshold
    from.  The dK/dV kernel has one shape, so the backward column moves with the dQ kernel alone."""
    g = torch.Generator().manual_seed(0)
    bert = torch.randint(256, 513, (8,), generator=g).tolist()
    bert16 = torch.randint(256, 513, (16,), generator=g).tolist()
    shapes = [("BERT varlen p=0.1", dict(B=8, H=12, D=64, N=512, dtype=torch.float16, p=0.1, lens=bert)),
              ("BERT varlen p=0.1, B=4", dict(B=4, H=12, D=64, N=512, dtype=torch.float16, p=0.1, lens=bert[:4])),
              ("BERT varlen p=0.1, B=16", dict(B=16, H=12, D=64, N=512, dtype=torch.float16, p=0.1, lens=bert16)),
              ("BERT varlen p=0, B=8", dict(B=8, H=12, D=64, N=512, dtype=torch.float16, lens=bert))]
    for B, N in ((8, 512), (12, 512), (16, 512), (4, 1024), (8, 1024), (4, 2048)):
        shapes.append(("fp16 p=0.1 B=%d N=%d" % (B, N), dict(B=B, H=12, D=64, N=N, dtype=torch.float16, p=0.1)))
    for B, N in ((16, 128), (32, 128), (64, 128), (8, 256), (16, 256), (24, 256), (32, 256), (64, 256), (4, 512), (8, 512), (12, 512),
                 (16, 512), (32, 512), (2, 1024), (4, 1024), (6, 1024), (8, 1024), (16, 1024), (1, 2048), (2, 2048), (3, 2048),
                 (4, 2048), (6, 2048), (8, 2048), (12, 2048), (1, 4096), (2, 4096), (4, 4096)):
        shapes.append(("fp16 B=%d N=%d" % (B, N), dict(B=B, H=12, D=64, N=N, dtype=torch.float16)))
    for B, N in ((8, 256), (16, 256), (8, 512), (12, 512), (16, 512), (4, 1024), (6, 1024), (8, 1024), (16, 1024), (2, 2048), (3, 2048),
                 (4, 2048), (8, 2048), (2, 4096), (4, 4096)):
        shapes.append(("bf16 causal B=%d N=%d" % (B, N), dict(B=B, H=12, D=64, N=N, dtype=torch.bfloat16, causal=True)))
    for B, N in ((8, 512), (16, 512), (8, 1024)):
        shapes.append(("fp16 d=32 B=%d N=%d" % (B, N), dict(B=B, H=12, D=32, N=N, dtype=torch.float16)))
    print("| launch | workgroups of 128 rows per compute unit | fwd full / half (us) | bwd full / half (us) | half wins fwd / bwd |",
          file=sys.stderr)
    print("|---|---|---|---|---|", file=sys.stderr)
    for name, kw in shapes:
        wl = Workload(torch, **kw)
        wgs = wl.B * wl.H * ((wl.max_s + 127) // 128) / 256.0
        t = {}
        for pol in (1, 2):
            be.set_launch_policy(pol)
            t[pol] = time_steps(torch, be, wl, steps, warmup, 0.1)
        be.set_launch_policy(0)
        print("| %s | %.2f | %.1f / %.1f | %.1f / %.1f | %s / %s |" % (
            name, wgs, t[1]["fwd_ms"] * 1e3, t[2]["fwd_ms"] * 1e3, t[1]["bwd_ms"] * 1e3, t[2]["bwd_ms"] * 1e3,
            "yes" if t[2]["fwd_ms"] < t[1]["fwd_ms"] else "no", "yes" if t[2]["bwd_ms"] < t[1]["bwd_ms"] else "no"), file=sys.stderr)
        del wl
        torch.cuda.empty_cache()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=300)
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--all", action="store_true", help="also time the other BASELINE configurations (stderr table)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-configs", action="store_true", help="skip the other BASELINE configurations (`configs` in the JSON line)")
    ap.add_argument("--cpu-budget", type=float, default=20.0)
    ap.add_argument("--settle", type=float, default=0.2,
                    help="seconds of untimed steps before the warm-up (0 for counter-collection runs)")
    ap.add_argument("--redraw-dropout", action="store_true",
                    help="dropout configurations: every kernel draws its keep decisions with Philox (the reference's scheme) "
                         "instead of the backward reading those the forward left (flash_attn_gfx950.KEEP_WORDS_MAX_BYTES = 0)")
    ap.add_argument("--only", default=None, metavar="TEXT",
                    help="time only the BASELINE configurations whose name contains TEXT and print their table rows "
                         "(no JSON line): for collecting rocprofv3 counters of one configuration")
    ap.add_argument("--backward", choices=("auto", "two-kernel", "one-kernel"), default="auto",
                    help="backward plan (fa_set_launch_policy 0x10 / 0x20): the dQ + dK/dV kernel pair, or the one-kernel "
                         "backward where it exists (head dim 64, dense, no mask, dropout or bias)")
    ap.add_argument("--d128-wave-pairs", action="store_true",
                    help="launch policy 0x40: the head-dim-128 dK/dV kernel as wave pairs (64 keys per workgroup)")
    ap.add_argument("--tile-sweep", action="store_true",
                    help="time full-size against half-size tiles on launches of growing size (markdown table on stderr, no JSON line)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 256 MiB device copy (for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (every (batch, head, tile) is independent; there is no "
                 "multi-GPU path to measure). Run with --gpus 1.")
    import torch
    from flash_attn import flash_attn_gfx950 as be
    be.load_library()  # fails loudly if the HIP library is not built
    if a.redraw_dropout:
        be.KEEP_WORDS_MAX_BYTES = 0
    be.set_launch_policy({"auto": 0, "two-kernel": 0x10, "one-kernel": 0x20}[a.backward] | (0x40 if a.d128_wave_pairs else 0))
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")

    if a.calibrate_copy:  # a kernel whose HBM traffic is known: reads 256 MiB, writes 256 MiB
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").random_(0, 255)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    if a.tile_sweep:
        tile_sweep(torch, be, max(20, a.steps // 5), 5)
        return

    if a.only is not None:
        for name, kw in config_list(torch):
            if a.only.lower() not in name.lower():
                continue
            wl = Workload(torch, **kw)
            tt = time_steps(torch, be, wl, a.steps, a.warmup, a.settle)
            fb = 3.5 * wl.fwd_flops / ((tt["fwd_ms"] + tt["bwd_ms"]) * 1e-3) / 1e12
            gbs = (wl.bytes_fwd + wl.bytes_bwd) / ((tt["fwd_ms"] + tt["bwd_ms"]) * 1e-3) / 1e9
            print("%-31s fwd %.4f ms  bwd %.4f ms  fwd+bwd %.1f TFLOP/s (%.2f %% of MFMA peak)  %.1f GB/s of algorithmic bytes "
                  "(fwd %.1f MB, bwd %.1f MB)  [step %.4f ms by the host clock over %d steps]"
                  % (name.strip(), tt["fwd_ms"], tt["bwd_ms"], fb, 100 * fb / MFMA_PEAK_TFLOPS, gbs,
                     wl.bytes_fwd / 1e6, wl.bytes_bwd / 1e6, tt["ms_per_step"], a.steps), file=sys.stderr)
            del wl
            torch.cuda.empty_cache()
        return

    B, H, D, N = 8, 12, 64, 2048
    w = Workload(torch, B, H, D, N, torch.float16)
    t = time_steps(torch, be, w, a.steps, a.warmup, a.settle)
    fwd_flops = attention_flops(B, H, N, D)
    step_flops = 3.5 * fwd_flops
    value = step_flops / (t["ms_per_step"] * 1e-3) / 1e12
    # the dK/dV kernel performs 4 of the backward's 5 algorithmic GEMMs (S, dP, dV, dK): 8*B*H*N^2*d flops per launch
    bwd_kernel_tflops = 2.0 * fwd_flops / (t["bwd_main_kernel_ms"] * 1e-3) / 1e12
    res = {
        "metric": "fwd+bwd TFLOPS, fp16 B8 H12 d64 N=2K (4*B*H*N^2*d fwd, 2.5x bwd)",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(t["ms_per_step"], 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic N(0,1) q,k,v,dout resident in HBM",
        "settle": "%.1f s of untimed steps before the warm-up steps (clock governor)" % a.settle,
        "config": {"workload": "headline: fp16 packed qkv [16384,3,12,64], B=8 H=12 d=64 N=2048 equal lengths, "
                               "non-causal, dropout 0, fwd+bwd with dout~N(0,1)"},
        "pct_of_mfma_peak": round(100.0 * value / MFMA_PEAK_TFLOPS, 2),
        "device_peak": device_peak(torch),
        "fwd_ms": round(t["fwd_ms"], 4), "bwd_ms": round(t["bwd_ms"], 4),
        "fwd_tflops": round(fwd_flops / (t["fwd_ms"] * 1e-3) / 1e12, 1),
        "bwd_tflops": round(2.5 * fwd_flops / (t["bwd_ms"] * 1e-3) / 1e12, 1),
        "roofline": {"kernel": "fa_bwd_dkdv_kernel<f16, d64> (S, dP, dV, dK GEMMs: 8*B*H*N^2*d flops per launch)", "bound": "mfma",
                     "achieved": round(bwd_kernel_tflops, 1), "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(bwd_kernel_tflops / MFMA_PEAK_TFLOPS, 4),
                     "avg_launch_ms": round(t["bwd_main_kernel_ms"], 4),
                     # HBM bytes per launch from the committed rocprofv3 FETCH_SIZE / WRITE_SIZE summary
                     "traffic": measured_traffic(), "traffic_source": TRAFFIC_PROFILE},
    }
    res["sustained_mfma"] = sustained_mfma(torch)
    # the boxes of a pool differ by a few per cent in what their matrix cores sustain; this ratio does not
    res["sustained_mfma"]["value_over_fp16_gemm"] = round(value / res["sustained_mfma"]["fp16_tflops"], 3)
    pt_ms, pt_mem = torch_attention_ms(torch, w, want_memory=True)
    our_mem = fused_step_memory(torch, w)
    res["pytorch_attention_same_gpu"] = {
        "ms_per_step": round(pt_ms, 3), "speedup": round(pt_ms / (t["fwd_ms"] + t["bwd_ms"]), 2),
        "step_memory_mb": round(pt_mem / 2 ** 20, 1), "fused_step_memory_mb": round(our_mem / 2 ** 20, 1),
        "memory_reduction": round(pt_mem / our_mem, 1),
        "what": "standard attention with PyTorch fp16 ops, fwd+bwd, same inputs, same GPU: the comparison point of the "
                "reference's published speed-ups (about 2x on A100 for this shape without mask or dropout) and memory "
                "savings (about 10x at N=2048); step memory = peak device memory of one fwd+bwd beyond its inputs"}
    # with dropout the autograd function also holds the keep words (one bit per score) from forward to backward, when they
    # are no larger than q, k and v together
    wd = Workload(torch, B, H, D, N, torch.float16, p=0.1)
    res["pytorch_attention_same_gpu"]["fused_step_memory_mb_dropout"] = round(fused_step_memory(torch, wd) / 2 ** 20, 1)
    res["pytorch_attention_same_gpu"]["keep_words_mb"] = round(wd.keep_words.numel() / 2 ** 20, 1) if wd.keep_words is not None else 0.0
    del wd
    if not a.no_cpu:
        res["cpu_baseline"] = cpu_baseline(torch, B, H, D, N, a.cpu_budget)
    else:
        res["cpu_baseline"] = None

    if not a.no_configs or a.all:
        if a.all:
            print("%-31s %9s %9s %9s %9s %8s %10s %11s %8s" % ("config", "fwd ms", "bwd ms", "fwd TF", "f+b TF", "% peak", "f+b GB/s",
                                                              "PyTorch ms", "speedup"), file=sys.stderr)
        res["configs"] = []
        for name, kw in config_list(torch):
            wl = Workload(torch, **kw)
            tt = time_steps(torch, be, wl, max(10, a.steps // 2), 5, a.settle)
            fb = 3.5 * wl.fwd_flops / ((tt["fwd_ms"] + tt["bwd_ms"]) * 1e-3) / 1e12
            gbs = (wl.bytes_fwd + wl.bytes_bwd) / ((tt["fwd_ms"] + tt["bwd_ms"]) * 1e-3) / 1e9
            row = {"config": name.strip(), "fwd_ms": round(tt["fwd_ms"], 4), "bwd_ms": round(tt["bwd_ms"], 4),
                   "fwd_tflops": round(wl.fwd_flops / (tt["fwd_ms"] * 1e-3) / 1e12, 1), "fwd_bwd_tflops": round(fb, 1),
                   "pct_of_mfma_peak": round(100 * fb / MFMA_PEAK_TFLOPS, 2), "hbm_gbs": round(gbs, 1),
                   "pct_of_hbm_peak": round(100 * gbs / HBM_PEAK_GBS, 2)}
            if a.all:
                # PyTorch standard attention on the same GPU (no counterpart for a block layout)
                pt = torch_attention_ms(torch, wl, 4) if wl.blockmask is None else None
                if pt:
                    row["pytorch_ms"] = round(pt, 3)
                print("%-31s %9.4f %9.4f %9.1f %9.1f %8.2f %10.1f %11s %8s" % (
                    name, tt["fwd_ms"], tt["bwd_ms"], wl.fwd_flops / (tt["fwd_ms"] * 1e-3) / 1e12, fb,
                    100 * fb / MFMA_PEAK_TFLOPS, gbs, "%.3f" % pt if pt else "-",
                    "%.1fx" % (pt / (tt["fwd_ms"] + tt["bwd_ms"])) if pt else "-"), file=sys.stderr)
            res["configs"].append(row)
            del wl
            torch.cuda.empty_cache()
    if a.all:
        # unpad / pad (row gather and scatter, HBM-bound): BERT-large-like padded batch, 75 % of the tokens valid
        from flash_attn.bert_padding import unpad_input
        Bp, Sp, dim = 64, 512, 1024
        gen = torch.Generator().manual_seed(0)
        lens_p = torch.randint(Sp // 2, Sp + 1, (Bp,), generator=gen)
        mask = (torch.arange(Sp)[None, :] < lens_p[:, None]).cuda()
        hidden = torch.randn(Bp, Sp, dim, device="cuda", dtype=torch.float16)
        rows, idx, _, _ = unpad_input(hidden, mask)
        nnz = rows.shape[0]
        for name, fn, nbytes in (
                ("unpad_input (gather)", lambda: be.gather_rows(hidden.view(Bp * Sp, dim), idx), 2 * nnz * dim * 2 + nnz * 8),
                ("pad_input (scatter)", lambda: be.scatter_rows(rows, idx, Bp * Sp), (nnz + Bp * Sp) * dim * 2 + nnz * 8)):
            ms = graph_replay_ms(torch, fn)
            print("%-28s %9.4f ms  %8.1f GB/s of %d (%.1f %% of HBM peak)  [B=%d S=%d dim=%d fp16, %d of %d tokens valid]"
                  % (name, ms, nbytes / ms / 1e6, HBM_PEAK_GBS, 100 * nbytes / ms / 1e6 / HBM_PEAK_GBS, Bp, Sp, dim, nnz, Bp * Sp),
                  file=sys.stderr)
        # rotary embedding of q and k of a packed qkv, in place (HBM-bound: 2/3 of the tensor read and written)
        Br, Sr, Hr, Dr = 8, 2048, 12, 64
        qkv_r = torch.randn(Br, Sr, 3, Hr, Dr, device="cuda", dtype=torch.float16)
        ang = torch.outer(torch.arange(Sr, device="cuda", dtype=torch.float32),
                          1.0 / (10000 ** (torch.arange(0, Dr, 2, device="cuda").float() / Dr)))
        cos_h, sin_h = torch.cos(ang).half().contiguous(), torch.sin(ang).half().contiguous()
        ms = graph_replay_ms(torch, lambda: be.rotary(qkv_r, qkv_r, cos_h, sin_h, n_rotated=2))
        nbytes = 2 * 2 * Br * Sr * Hr * Dr * 2   # q and k read and written; v is not touched in place
        print("%-28s %9.4f ms  %8.1f GB/s of %d (%.1f %% of HBM peak)  [B=%d S=%d H=%d d=%d fp16 packed qkv, in place]"
              % ("rotary q,k (fa_rotary)", ms, nbytes / ms / 1e6, HBM_PEAK_GBS, 100 * nbytes / ms / 1e6 / HBM_PEAK_GBS,
                 Br, Sr, Hr, Dr), file=sys.stderr)
        # the same embedding around one attention step (fwd + bwd), as FlashMHA(use_rotary_emb="1d") runs it: q and k rotated
        # by a pass before the forward and dq, dk by a pass after the backward, against the rotation inside the attention
        # kernels (only k takes a pass)
        packed = qkv_r.view(Br * Sr, 3, Hr, Dr)
        do_r = torch.randn(Br * Sr, Hr, Dr, device="cuda", dtype=torch.float16)
        cu_r = torch.arange(0, (Br + 1) * Sr, Sr, dtype=torch.int32, device="cuda")
        dqkv_r, rot_r = torch.empty_like(packed), torch.empty(Br * Sr, 2, Hr, Dr, device="cuda", dtype=torch.float16)
        scale_r = Dr ** -0.5

        def step_separate():
            be.rotary(qkv_r, qkv_r, cos_h, sin_h, n_rotated=2)
            o, lse = be.fwd(packed[:, 0], packed[:, 1], packed[:, 2], cu_r, cu_r, Sr, Sr, 0.0, scale_r, False, False, False)
            be.bwd(do_r, packed[:, 0], packed[:, 1], packed[:, 2], o, lse, dqkv_r[:, 0], dqkv_r[:, 1], dqkv_r[:, 2], cu_r, cu_r,
                   Sr, Sr, 0.0, scale_r, False, False)
            g5 = dqkv_r.view(Br, Sr, 3, Hr, Dr)
            be.rotary(g5, torch.empty_like(g5), cos_h, sin_h, n_rotated=2, conjugate=True)

        def step_in_kernel():
            be.rotary(qkv_r[:, :, 1:2], rot_r.view(Br, Sr, 2, Hr, Dr)[:, :, 1:2], cos_h, sin_h, n_rotated=1)
            o, lse = be.fwd(packed[:, 0], rot_r[:, 1], packed[:, 2], cu_r, cu_r, Sr, Sr, 0.0, scale_r, False, False, False,
                            rotary=(cos_h, sin_h), q_rot=rot_r[:, 0])
            be.bwd(do_r, rot_r[:, 0], rot_r[:, 1], packed[:, 2], o, lse, dqkv_r[:, 0], dqkv_r[:, 1], dqkv_r[:, 2], cu_r, cu_r,
                   Sr, Sr, 0.0, scale_r, False, False, rotary=(cos_h, sin_h))
        ms_sep, ms_in = graph_replay_ms(torch, step_separate), graph_replay_ms(torch, step_in_kernel)
        print("%-28s %9.4f ms with separate passes, %.4f ms inside the kernels (%.1f %% less)  [same shape, fwd + bwd, no "
              "dropout]" % ("rotary + attention step", ms_sep, ms_in, 100 * (1 - ms_in / ms_sep)), file=sys.stderr)
        # gradient of a bias shared over the batch: the per-(batch, head) slices the dK/dV kernel wrote, summed in one pass
        # (fp32 sums, one rounding) against the same sum with torch ops (a float copy, a sum, a cast)
        del qkv_r, packed, do_r, dqkv_r, rot_r
        torch.cuda.empty_cache()
        Bb, Hb, Nb = 8, 12, 2048
        db = torch.randn(Bb, Hb, Nb, Nb, device="cuda", dtype=torch.float16)
        red = torch.empty(1, Hb, Nb, Nb, device="cuda", dtype=torch.float16)
        ms_lib = graph_replay_ms(torch, lambda: be.reduce_bias_grad(db, red, True, False), calls=5)
        ms_torch = graph_replay_ms(torch, lambda: db.float().sum(0, keepdim=True).to(torch.float16), calls=5)
        nbytes = (Bb + 1) * Hb * Nb * Nb * 2
        print("%-28s %9.4f ms  %8.1f GB/s of %d (%.1f %% of HBM peak); with torch ops %.4f ms  [B=%d H=%d N=%d fp16 -> (1, H, "
              "N, N)]" % ("bias gradient over batch", ms_lib, nbytes / ms_lib / 1e6, HBM_PEAK_GBS,
                          100 * nbytes / ms_lib / 1e6 / HBM_PEAK_GBS, ms_torch, Bb, Hb, Nb), file=sys.stderr)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
