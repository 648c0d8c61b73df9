"""Binding of libflash_attn_gfx950.so: the module that stands where the reference's pybind11 extension
``flash_attn_cuda`` stood (csrc/flash_attn/fmha_api.cpp:721-727).

``fwd``, ``bwd``, ``fwd_block`` and ``bwd_block`` take the same arguments, in the same order, as
mha_fwd / mha_bwd / mha_fwd_block / mha_bwd_block (fmha_api.cpp:173-186, 302-321, 451-464, 575-594) and return the
same lists of tensors.  Torch is used only to own device memory, the current stream and the Philox
(seed, offset) of the device's default generator; all computation happens behind the C ABI declared in
include/flash_attn_gfx950.h.  There is no fallback: if the shared library is missing, importing the
functions works but the first call raises.
"""
import ctypes
import functools
import os
import threading

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libflash_attn_gfx950.so"
LIB_PATH = os.path.join(_HERE, LIB_NAME)

FA_FP16, FA_BF16 = 0, 1
FA_ABI_VERSION = 5

_c_i32p = ctypes.c_void_p

# Dropout keep words: the forward can leave its keep decisions (one bit per score) in a buffer from which the backward's two
# kernels read them instead of drawing them again with Philox; results are the same bit for bit.  new_keep_words() makes
# that buffer unless it would be larger than this many bytes (0: never) or larger than q, k and v together (one bit per score
# grows with the square of the sequence length: from about 3 * 16 * head_dim tokens on it would outweigh the inputs), in which
# case every kernel draws its own decisions, as the reference's do, and no memory beyond O(seqlen) is held between forward
# and backward.
KEEP_WORDS_MAX_BYTES = 1 << 30
# ... and at most this multiple of the bytes of q, k and v (None: no such limit)
KEEP_WORDS_MAX_INPUT_RATIO = 1.0


class FwdArgs(ctypes.Structure):
    """struct fa_fwd_args of include/flash_attn_gfx950.h"""
    _fields_ = [
        ("struct_bytes", ctypes.c_uint32), ("dtype", ctypes.c_int32),
        ("q", ctypes.c_void_p), ("k", ctypes.c_void_p), ("v", ctypes.c_void_p), ("o", ctypes.c_void_p),
        ("softmax_lse", ctypes.c_void_p), ("s_dmask", ctypes.c_void_p),
        ("cu_seqlens_q", _c_i32p), ("cu_seqlens_k", _c_i32p), ("blockmask", _c_i32p),
        ("q_row_stride", ctypes.c_int64), ("q_head_stride", ctypes.c_int64),
        ("k_row_stride", ctypes.c_int64), ("k_head_stride", ctypes.c_int64),
        ("v_row_stride", ctypes.c_int64), ("v_head_stride", ctypes.c_int64),
        ("o_row_stride", ctypes.c_int64), ("o_head_stride", ctypes.c_int64),
        ("batch", ctypes.c_int32), ("nheads", ctypes.c_int32), ("head_dim", ctypes.c_int32),
        ("total_q", ctypes.c_int32), ("total_k", ctypes.c_int32),
        ("max_seqlen_q", ctypes.c_int32), ("max_seqlen_k", ctypes.c_int32),
        ("p_dropout", ctypes.c_float), ("softmax_scale", ctypes.c_float),
        ("zero_tensors", ctypes.c_int32), ("is_causal", ctypes.c_int32),
        ("philox_seed", ctypes.c_uint64), ("philox_offset", ctypes.c_uint64),
        ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_size_t),
        ("stream", ctypes.c_void_p),
        ("alibi_slopes", ctypes.c_void_p),
        ("keep_words", ctypes.c_void_p), ("keep_words_bytes", ctypes.c_size_t),
        ("attn_bias", ctypes.c_void_p), ("bias_batch_stride", ctypes.c_int64), ("bias_head_stride", ctypes.c_int64),
        ("bias_row_stride", ctypes.c_int64),
        ("row_order", ctypes.c_void_p),
        ("rotary_cos", ctypes.c_void_p), ("rotary_sin", ctypes.c_void_p),
        ("rotary_table_rows", ctypes.c_int32), ("reserved0", ctypes.c_int32),
        ("q_rot", ctypes.c_void_p), ("q_rot_row_stride", ctypes.c_int64), ("q_rot_head_stride", ctypes.c_int64),
    ]


class BwdArgs(ctypes.Structure):
    """struct fa_bwd_args of include/flash_attn_gfx950.h"""
    _fields_ = [
        ("struct_bytes", ctypes.c_uint32), ("dtype", ctypes.c_int32),
        ("dout", ctypes.c_void_p), ("q", ctypes.c_void_p), ("k", ctypes.c_void_p), ("v", ctypes.c_void_p),
        ("out", ctypes.c_void_p), ("softmax_lse", ctypes.c_void_p),
        ("dq", ctypes.c_void_p), ("dk", ctypes.c_void_p), ("dv", ctypes.c_void_p), ("softmax_d", ctypes.c_void_p),
        ("cu_seqlens_q", _c_i32p), ("cu_seqlens_k", _c_i32p), ("blockmask", _c_i32p),
        ("do_row_stride", ctypes.c_int64), ("do_head_stride", ctypes.c_int64),
        ("q_row_stride", ctypes.c_int64), ("q_head_stride", ctypes.c_int64),
        ("k_row_stride", ctypes.c_int64), ("k_head_stride", ctypes.c_int64),
        ("v_row_stride", ctypes.c_int64), ("v_head_stride", ctypes.c_int64),
        ("o_row_stride", ctypes.c_int64), ("o_head_stride", ctypes.c_int64),
        ("dq_row_stride", ctypes.c_int64), ("dq_head_stride", ctypes.c_int64),
        ("dk_row_stride", ctypes.c_int64), ("dk_head_stride", ctypes.c_int64),
        ("dv_row_stride", ctypes.c_int64), ("dv_head_stride", ctypes.c_int64),
        ("lse_seq_stride", ctypes.c_int32),
        ("batch", ctypes.c_int32), ("nheads", ctypes.c_int32), ("head_dim", ctypes.c_int32),
        ("total_q", ctypes.c_int32), ("total_k", ctypes.c_int32),
        ("max_seqlen_q", ctypes.c_int32), ("max_seqlen_k", ctypes.c_int32),
        ("p_dropout", ctypes.c_float), ("softmax_scale", ctypes.c_float),
        ("zero_tensors", ctypes.c_int32), ("is_causal", ctypes.c_int32),
        ("philox_seed", ctypes.c_uint64), ("philox_offset", ctypes.c_uint64),
        ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_size_t),
        ("stream", ctypes.c_void_p),
        ("alibi_slopes", ctypes.c_void_p),
        ("keep_words", ctypes.c_void_p), ("keep_words_bytes", ctypes.c_size_t),
        ("attn_bias", ctypes.c_void_p), ("bias_batch_stride", ctypes.c_int64), ("bias_head_stride", ctypes.c_int64),
        ("bias_row_stride", ctypes.c_int64),
        ("dbias", ctypes.c_void_p), ("dbias_batch_stride", ctypes.c_int64), ("dbias_head_stride", ctypes.c_int64),
        ("dbias_row_stride", ctypes.c_int64),
        ("row_order", ctypes.c_void_p),
        ("rotary_cos", ctypes.c_void_p), ("rotary_sin", ctypes.c_void_p),
        ("rotary_table_rows", ctypes.c_int32), ("reserved0", ctypes.c_int32),
    ]


class RotaryArgs(ctypes.Structure):
    """struct fa_rotary_args, field for field."""
    _fields_ = [
        ("struct_bytes", ctypes.c_uint32), ("dtype", ctypes.c_int32),
        ("src", ctypes.c_void_p), ("dst", ctypes.c_void_p), ("cos_table", ctypes.c_void_p), ("sin_table", ctypes.c_void_p),
        ("positions", ctypes.c_void_p), ("n_rows", ctypes.c_int64),
        ("src_row_stride", ctypes.c_int64), ("src_part_stride", ctypes.c_int64), ("src_head_stride", ctypes.c_int64),
        ("dst_row_stride", ctypes.c_int64), ("dst_part_stride", ctypes.c_int64), ("dst_head_stride", ctypes.c_int64),
        ("n_parts", ctypes.c_int32), ("n_rotated", ctypes.c_int32), ("n_heads", ctypes.c_int32), ("head_dim", ctypes.c_int32),
        ("seqlen", ctypes.c_int32), ("table_rows", ctypes.c_int32), ("conjugate", ctypes.c_int32),
        ("stream", ctypes.c_void_p),
    ]


EXPORTED_SYMBOLS = (
    "fa_fwd", "fa_bwd", "fa_fwd_block", "fa_bwd_block", "fa_fwd_block_noalloc", "fa_fwd_workspace_bytes", "fa_bwd_workspace_bytes",
    "fa_round_seqlens", "fa_philox_offset_increment", "fa_last_error", "fa_abi_version",
    "fa_gather_rows", "fa_scatter_rows", "fa_scatter_rows_workspace_bytes", "fa_rotary", "fa_set_launch_policy",
    "fa_keep_words_bytes", "fa_blocksparse_row_order", "fa_bias_grad_reduce",
)
# declared in include/flash_attn_gfx950_bench.h: instrumentation for bench.py, not part of the drop-in boundary
BENCH_SYMBOLS = ("fa_bwd_profiled",)

_lib = None
_lib_lock = threading.Lock()


def load_library():
    """dlopen the shared library once and declare the prototypes.  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lib_lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "%s is not built (expected at %s); run `python flash-attention_amd/build.py`. "
                "There is no non-HIP fallback." % (LIB_NAME, LIB_PATH))
        lib = ctypes.CDLL(LIB_PATH)
        for name in ("fa_fwd", "fa_fwd_block", "fa_fwd_block_noalloc"):
            fn = getattr(lib, name)
            fn.argtypes = [ctypes.POINTER(FwdArgs)]
            fn.restype = ctypes.c_int
        for name in ("fa_bwd", "fa_bwd_block"):
            fn = getattr(lib, name)
            fn.argtypes = [ctypes.POINTER(BwdArgs)]
            fn.restype = ctypes.c_int
        lib.fa_bwd_profiled.argtypes = [ctypes.POINTER(BwdArgs), ctypes.c_void_p, ctypes.c_void_p]
        lib.fa_bwd_profiled.restype = ctypes.c_int
        lib.fa_fwd_workspace_bytes.argtypes = [ctypes.POINTER(FwdArgs)]
        lib.fa_fwd_workspace_bytes.restype = ctypes.c_size_t
        lib.fa_bwd_workspace_bytes.argtypes = [ctypes.POINTER(BwdArgs)]
        lib.fa_bwd_workspace_bytes.restype = ctypes.c_size_t
        lib.fa_keep_words_bytes.argtypes = [ctypes.c_int32] * 4
        lib.fa_keep_words_bytes.restype = ctypes.c_size_t
        lib.fa_round_seqlens.argtypes = [ctypes.c_int32] * 4 + [ctypes.POINTER(ctypes.c_int32)] * 2
        lib.fa_round_seqlens.restype = None
        lib.fa_philox_offset_increment.argtypes = []
        lib.fa_philox_offset_increment.restype = ctypes.c_uint64
        lib.fa_last_error.argtypes = []
        lib.fa_last_error.restype = ctypes.c_char_p
        lib.fa_abi_version.argtypes = []
        lib.fa_abi_version.restype = ctypes.c_int
        lib.fa_gather_rows.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_int64] * 5 + [ctypes.c_void_p]
        lib.fa_gather_rows.restype = ctypes.c_int
        lib.fa_scatter_rows.argtypes = ([ctypes.c_void_p] * 3 + [ctypes.c_int64] * 5 +
                                        [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p])
        lib.fa_scatter_rows.restype = ctypes.c_int
        lib.fa_bias_grad_reduce.argtypes = ([ctypes.c_void_p] * 2 + [ctypes.c_int32] * 5 + [ctypes.c_int64] * 3 +
                                            [ctypes.c_int32] * 2 + [ctypes.c_int64] * 3 + [ctypes.c_void_p])
        lib.fa_bias_grad_reduce.restype = ctypes.c_int
        lib.fa_scatter_rows_workspace_bytes.argtypes = [ctypes.c_int64]
        lib.fa_scatter_rows_workspace_bytes.restype = ctypes.c_size_t
        lib.fa_rotary.argtypes = [ctypes.POINTER(RotaryArgs)]
        lib.fa_rotary.restype = ctypes.c_int
        lib.fa_blocksparse_row_order.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p]
        lib.fa_blocksparse_row_order.restype = ctypes.c_int
        lib.fa_set_launch_policy.argtypes = [ctypes.c_int]
        lib.fa_set_launch_policy.restype = ctypes.c_int
        if lib.fa_abi_version() != FA_ABI_VERSION:
            raise RuntimeError("%s has ABI version %d, binding expects %d" % (LIB_NAME, lib.fa_abi_version(), FA_ABI_VERSION))
        _lib = lib
    return _lib


def set_launch_policy(policy):
    """Tile shape: 0 chosen per launch (default), 1 always the full-size tiles, 2 the half-size tiles wherever they exist;
    plus the backward plan: 0x10 the dQ + dK/dV kernel pair (also the default), 0x20 the one-kernel backward where it
    exists; plus 0x40: the head-dim-128 dK/dV kernel as wave pairs where it exists (fa_set_launch_policy)."""
    global _policy_epoch
    lib = load_library()
    rc = lib.fa_set_launch_policy(int(policy))
    if rc != 0:
        _raise(rc, lib)
    _policy_epoch += 1


@functools.lru_cache(maxsize=256)
def round_seqlens(head_dim, max_seqlen_q, max_seqlen_k, blocksparse=False):
    """(max_seqlen_q_rounded, max_seqlen_k_rounded) as the library shapes softmax_lse / S_dmask
    (fmha_api.cpp:232-241 and :509-514)."""
    sq, sk = ctypes.c_int32(), ctypes.c_int32()
    load_library().fa_round_seqlens(head_dim, max_seqlen_q, max_seqlen_k, int(blocksparse), ctypes.byref(sq), ctypes.byref(sk))
    return sq.value, sk.value


def _check(cond, msg):
    # the reference's TORCH_CHECK failures surface in Python as RuntimeError
    if not cond:
        raise RuntimeError(msg)


def _dtype_code(t):
    _check(t.dtype in (torch.float16, torch.bfloat16), "q, k, v must be fp16 or bf16")  # fmha_api.cpp:198
    return FA_FP16 if t.dtype == torch.float16 else FA_BF16


def _check_qkv(name, t, dtype, total, nheads, head_dim):
    if t.is_cuda and t.dtype == dtype and t.shape == (total, nheads, head_dim) and t.stride(-1) == 1:
        return  # the common case in one test; the individual checks below only produce the message
    _check(t.is_cuda, "%s must be on the GPU" % name)                                    # fmha_api.cpp:204-208
    _check(t.dtype == dtype, "%s has dtype %s, expected %s" % (name, t.dtype, dtype))    # :199-200
    _check(t.dim() == 3 and tuple(t.shape) == (total, nheads, head_dim),
           "%s has shape %s, expected %s" % (name, tuple(t.shape), (total, nheads, head_dim)))  # CHECK_SHAPE :226-228
    _check(t.stride(-1) == 1, "%s must have a contiguous last dimension" % name)         # :210-212


def _check_cu(name, t, batch):
    if t.is_cuda and t.dtype == torch.int32 and t.dim() == 1 and t.numel() == batch + 1 and t.is_contiguous():
        return
    _check(t.is_cuda, "%s must be on the GPU" % name)
    _check(t.dtype == torch.int32, "%s must be int32" % name)                            # :201-202
    _check(t.is_contiguous(), "%s must be contiguous" % name)                            # :213-214
    _check(t.dim() == 1 and t.numel() == batch + 1, "%s must have shape (batch + 1,)" % name)  # :229-230


def _philox_state(device, p_dropout, gen):
    """(seed, offset) of the device's generator, advanced the way philox_cuda_state(counter_offset) does
    (fmha_api.cpp:288-292).  Restoring the generator state reproduces the pair, which is how the backward
    regenerates the forward's mask (flash_attn_interface.py:43,61-63)."""
    if not p_dropout > 0.0:
        return 0, 0
    if gen is None:
        idx = device.index if device.index is not None else torch.cuda.current_device()
        gen = torch.cuda.default_generators[idx]
    seed = gen.initial_seed()
    offset = gen.get_offset()
    gen.set_offset(offset + int(load_library().fa_philox_offset_increment()))
    return seed & 0xFFFFFFFFFFFFFFFF, offset & 0xFFFFFFFFFFFFFFFF


# torch's current stream as a raw hipStream_t: the public route (torch.cuda.current_stream(device).cuda_stream) builds a
# Stream object per call and costs 4 us, a fifth of a whole call here; the accessor below is what it wraps
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream_handle(device):
    """hipStream_t of torch's current stream on `device`, as an integer."""
    if _raw_stream is not None:
        return _raw_stream(device.index if device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(device).cuda_stream


# Argument structs are kept per thread and per call signature (shapes, strides, flags): a call then only writes what changes
# from call to call - pointers, dropout state, stream - instead of allocating and filling forty fields, and does not ask the
# library for the workspace size again.  set_launch_policy() empties the cache (the workspace size depends on the policy).
_args_tls = threading.local()
_policy_epoch = 0


def _cached_args(key, cls, fill):
    """(struct, workspace bytes) for a call signature; fill(struct) -> workspace bytes runs on a miss."""
    cache = getattr(_args_tls, "cache", None)
    if cache is None or getattr(_args_tls, "epoch", -1) != _policy_epoch:
        cache = _args_tls.cache = {}
        _args_tls.epoch = _policy_epoch
    ent = cache.get(key)
    if ent is None:
        if len(cache) >= 512:
            cache.clear()
        a = cls()
        a.struct_bytes = ctypes.sizeof(cls)
        ent = cache[key] = (a, fill(a))
    return ent


class _OnDevice:
    """`with torch.cuda.device(dev)` without its cost when dev already is the current device."""

    def __init__(self, device):
        self._ctx = None
        if device.index is not None and device.index != torch.cuda.current_device():
            self._ctx = torch.cuda.device(device)

    def __enter__(self):
        if self._ctx is not None:
            self._ctx.__enter__()

    def __exit__(self, *exc):
        if self._ctx is not None:
            return self._ctx.__exit__(*exc)
        return False


def _raise(rc, lib):
    msg = lib.fa_last_error().decode("utf-8", "replace")
    raise RuntimeError("flash_attn_gfx950 error %d: %s" % (rc, msg))


def _check_alibi(alibi_slopes, nheads, device, sparse):
    """alibi_slopes: None or nheads fp32 slopes on the tensors' device (an extension: the reference has no attention bias)."""
    if alibi_slopes is None:
        return None
    _check(alibi_slopes.device == device and alibi_slopes.dtype == torch.float32 and alibi_slopes.is_contiguous() and
           tuple(alibi_slopes.shape) == (nheads,), "alibi_slopes must be a contiguous fp32 tensor of nheads slopes on the GPU")
    return alibi_slopes.data_ptr()


def prepare_attn_bias(attn_bias, q, batch, nheads, max_seqlen_q, max_seqlen_k):
    """The tensor the kernels read for attn_bias (an extension: the reference only plans attention bias, README.md:50):
    attn_bias itself if it already is what they need - 4-D, (1 or batch, 1 or nheads, >= max_seqlen_q, >= max_seqlen_k) in
    q's dtype on q's device, keys contiguous, 16-byte aligned, row stride a multiple of 8 - else a copy with padded rows."""
    _check(attn_bias.dim() == 4 and attn_bias.shape[0] in (1, batch) and attn_bias.shape[1] in (1, nheads) and
           attn_bias.shape[2] >= max_seqlen_q and attn_bias.shape[3] >= max_seqlen_k,
           "attn_bias must be (1 or batch, 1 or nheads, >= max_seqlen_q, >= max_seqlen_k), got %s" % (tuple(attn_bias.shape),))
    _check(attn_bias.device == q.device and attn_bias.dtype == q.dtype, "attn_bias must have q's dtype and device")
    ok = (attn_bias.stride(3) == 1 and attn_bias.stride(2) % 8 == 0 and attn_bias.stride(2) >= max_seqlen_k and
          attn_bias.data_ptr() % 16 == 0 and all(attn_bias.stride(i) % 8 == 0 for i in (0, 1)))
    if not ok:
        sk8 = (attn_bias.shape[3] + 7) // 8 * 8
        padded = torch.zeros(attn_bias.shape[:3] + (sk8,), dtype=attn_bias.dtype, device=attn_bias.device)
        padded[..., :attn_bias.shape[3]] = attn_bias
        attn_bias = padded
    return attn_bias


def _bias_arg(a, attn_bias, q, batch, nheads, max_seqlen_q, max_seqlen_k, sparse):
    """Fills the attn_bias fields of a FwdArgs / BwdArgs; returns the tensor they point into (to be kept alive)."""
    if attn_bias is None:
        return None
    t = prepare_attn_bias(attn_bias, q, batch, nheads, int(max_seqlen_q), int(max_seqlen_k))
    a.attn_bias = t.data_ptr()
    a.bias_batch_stride = 0 if t.shape[0] == 1 else t.stride(0)
    a.bias_head_stride = 0 if t.shape[1] == 1 else t.stride(1)
    a.bias_row_stride = t.stride(2)
    return t


def new_keep_words(q, cu_seqlens_q, max_seqlen_q, max_seqlen_k, p_dropout, total_k=None):
    """Buffer for the dropout keep words of one forward call (argument keep_words of fwd and bwd), or None if there is no
    dropout or the buffer would exceed KEEP_WORDS_MAX_BYTES or KEEP_WORDS_MAX_INPUT_RATIO times the bytes of q, k and v
    (total_k: rows of k and v; default: those of q)."""
    if not p_dropout > 0:
        return None
    n = load_library().fa_keep_words_bytes(cu_seqlens_q.numel() - 1, q.shape[1], int(max_seqlen_q), int(max_seqlen_k))
    inputs = (q.shape[0] + 2 * (q.shape[0] if total_k is None else int(total_k))) * q.shape[1] * q.shape[2] * q.element_size()
    if n == 0 or n > KEEP_WORDS_MAX_BYTES or (KEEP_WORDS_MAX_INPUT_RATIO is not None and n > KEEP_WORDS_MAX_INPUT_RATIO * inputs):
        return None
    return torch.empty((n,), dtype=torch.uint8, device=q.device)


def _keep_words_arg(a, keep_words, dev, sparse):
    if keep_words is None or sparse:
        return
    _check(keep_words.device == dev and keep_words.dtype == torch.uint8 and keep_words.is_contiguous(),
           "keep_words must be a contiguous uint8 tensor on the tensors' device (see new_keep_words)")
    a.keep_words, a.keep_words_bytes = keep_words.data_ptr(), keep_words.numel()


def _row_order_arg(a, row_order, sq_r, dev):
    if row_order is None:
        return
    _check(row_order.device == dev and row_order.dtype == torch.int32 and row_order.is_contiguous() and
           row_order.numel() == sq_r // 16, "row_order must be a contiguous int32 tensor of max_seqlen_q_rounded / 16 row blocks "
                                            "on the tensors' device (see blockmask_row_order)")
    a.row_order = row_order.data_ptr()


def blockmask_row_order(layout):
    """An order of the 16-row blocks of a block-sparse layout ((rows / 16, keys / 256) of 0 / 1) for the `row_order` argument
    of fwd_block / bwd_block.  A workgroup of the forward and of the dQ kernel owns eight consecutive entries and stages every
    key tile that any of the eight lists; each of its waves owns two consecutive entries and computes on every tile that
    either of the two lists.  fa_blocksparse_row_order (host code of the library) groups row blocks with similar lists: a
    greedy grouping, then exchanges that lower the staged and computed tiles; the plain order 0, 1, 2, ... if that saves
    less than 5 % of the staged tiles (layouts made of whole 128-row tiles).  int32 tensor on the layout's device."""
    import numpy as np
    m = np.ascontiguousarray((layout != 0).cpu().numpy().astype(np.uint8))
    _check(m.ndim == 2, "layout must be (rows / 16, keys / 256)")
    order = np.empty(m.shape[0], dtype=np.int32)
    lib = load_library()
    rc = lib.fa_blocksparse_row_order(m.ctypes.data, m.shape[0], m.shape[1], order.ctypes.data)
    if rc != 0:
        _raise(rc, lib)
    return torch.from_numpy(order).to(layout.device)


def _rotary_arg(a, rotary, q, rows_needed):
    """(cos, sin) tables of the in-kernel rotary embedding into an argument struct."""
    if rotary is None:
        return
    cos, sin = rotary
    _check(cos.shape == sin.shape and cos.ndim == 2 and cos.shape[1] == q.shape[-1] // 2 and cos.dtype == q.dtype
           and sin.dtype == q.dtype and cos.is_contiguous() and sin.is_contiguous() and cos.device == q.device
           and sin.device == q.device, "rotary: cos / sin must be contiguous (rows, headdim / 2) tables in q's dtype")
    _check(cos.shape[0] >= rows_needed, "rotary: the tables have fewer rows than the sequences have positions")
    a.rotary_cos, a.rotary_sin, a.rotary_table_rows = cos.data_ptr(), sin.data_ptr(), cos.shape[0]


def _fwd_impl(q, k, v, cu_seqlens_q, cu_seqlens_k, blockmask, max_seqlen_q, max_seqlen_k, p_dropout, softmax_scale,
              zero_tensors, is_causal, return_softmax, gen, alibi_slopes=None, keep_words=None, attn_bias=None,
              row_order=None, rotary=None, q_rot=None):
    lib = load_library()
    code = _dtype_code(q)
    _check(q.dim() == 3, "q must be (total_q, nheads, head_size)")
    total_q, nheads, head_dim = q.shape
    total_k = k.shape[0]
    batch = cu_seqlens_q.numel() - 1
    _check(batch > 0, "batch size must be positive")                                     # :223
    _check(head_dim in (16, 32, 64, 128), "head_size must be 16, 32, 64 or 128")         # :224
    _check_qkv("q", q, q.dtype, total_q, nheads, head_dim)
    _check_qkv("k", k, q.dtype, total_k, nheads, head_dim)
    _check_qkv("v", v, q.dtype, total_k, nheads, head_dim)
    _check_cu("cu_seqlens_q", cu_seqlens_q, batch)
    _check_cu("cu_seqlens_k", cu_seqlens_k, batch)
    sparse = blockmask is not None
    sq_r, sk_r = round_seqlens(head_dim, max_seqlen_q, max_seqlen_k, sparse)
    if sparse:
        _check(blockmask.is_cuda and blockmask.dtype == torch.int32 and blockmask.is_contiguous(),
               "blockmask must be a contiguous int32 GPU tensor")                         # :477,484,491
        _check(tuple(blockmask.shape) == (sk_r // 256, sq_r // 16),
               "blockmask has shape %s, expected %s" % (tuple(blockmask.shape), (sk_r // 256, sq_r // 16)))  # :515

    dev = q.device
    with _OnDevice(dev):
        o = torch.empty((total_q, nheads, head_dim), dtype=q.dtype, device=dev)
        lse = torch.empty((batch, nheads, sq_r), dtype=torch.float32, device=dev)
        s = torch.empty((batch, nheads, sq_r, sk_r), dtype=q.dtype, device=dev) if return_softmax else None
        seed, offset = _philox_state(dev, p_dropout, gen)
        qs, ks, vs = q.stride(), k.stride(), v.stride()
        mq, mk = int(max_seqlen_q), int(max_seqlen_k)
        dropout = p_dropout > 0

        def fill(a):  # everything a call signature fixes; returns the workspace size of such calls
            a.dtype = code
            a.q_row_stride, a.q_head_stride = qs[0], qs[1]
            a.k_row_stride, a.k_head_stride = ks[0], ks[1]
            a.v_row_stride, a.v_head_stride = vs[0], vs[1]
            a.o_row_stride, a.o_head_stride = nheads * head_dim, head_dim
            a.batch, a.nheads, a.head_dim = batch, nheads, head_dim
            a.total_q, a.total_k = total_q, total_k
            a.max_seqlen_q, a.max_seqlen_k = mq, mk
            a.zero_tensors, a.is_causal = int(bool(zero_tensors)), int(bool(is_causal))
            # (the size query reads shapes, is_causal, p_dropout > 0 and which optional pointers are set)
            a.p_dropout = float(p_dropout)
            a.blockmask = 16 if sparse else None
            a.alibi_slopes = 16 if alibi_slopes is not None else None
            a.attn_bias = 16 if attn_bias is not None else None
            return lib.fa_fwd_workspace_bytes(ctypes.byref(a))

        a, ws_bytes = _cached_args(("fwd", code, qs, ks, vs, batch, nheads, head_dim, total_q, total_k, mq, mk,
                                    bool(zero_tensors), bool(is_causal), dropout, sparse, alibi_slopes is not None,
                                    attn_bias is not None), FwdArgs, fill)
        a.q, a.k, a.v, a.o = q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr()
        a.softmax_lse = lse.data_ptr()
        a.s_dmask = s.data_ptr() if s is not None else None
        a.cu_seqlens_q, a.cu_seqlens_k = cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr()
        a.blockmask = blockmask.data_ptr() if sparse else None
        a.p_dropout, a.softmax_scale = float(p_dropout), float(softmax_scale)
        a.philox_seed, a.philox_offset = seed, offset
        ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=dev) if ws_bytes else None
        a.workspace = ws.data_ptr() if ws is not None else None
        a.workspace_bytes = ws_bytes
        # (the struct is reused: the optional fields are cleared before the helpers below set the ones that are given)
        a.keep_words, a.keep_words_bytes, a.attn_bias, a.row_order = None, 0, None, None
        a.rotary_cos, a.rotary_sin, a.q_rot = None, None, None
        a.stream = _stream_handle(dev)
        a.alibi_slopes = _check_alibi(alibi_slopes, nheads, dev, sparse)
        _keep_words_arg(a, keep_words, dev, sparse)
        bias_t = _bias_arg(a, attn_bias, q, batch, nheads, max_seqlen_q, max_seqlen_k, sparse)  # noqa: F841 (kept alive)
        if sparse:
            _row_order_arg(a, row_order, sq_r, dev)
        _rotary_arg(a, rotary, q, int(max_seqlen_q))
        if q_rot is not None:
            _check(rotary is not None, "q_rot without rotary tables")
            _check_qkv("q_rot", q_rot, q.dtype, total_q, nheads, head_dim)
            a.q_rot, a.q_rot_row_stride, a.q_rot_head_stride = q_rot.data_ptr(), q_rot.stride(0), q_rot.stride(1)
        rc = (lib.fa_fwd_block if sparse else lib.fa_fwd)(ctypes.byref(a))
        if rc != 0:
            _raise(rc, lib)
    return [o, lse, s] if return_softmax else [o, lse]


def _bwd_impl(dout, q, k, v, out, softmax_lse, dq, dk, dv, cu_seqlens_q, cu_seqlens_k, blockmask, max_seqlen_q,
              max_seqlen_k, p_dropout, softmax_scale, zero_tensors, is_causal, gen, main_kernel_events=None,
              alibi_slopes=None, keep_words=None, attn_bias=None, dbias=None, row_order=None, rotary=None):
    lib = load_library()
    code = _dtype_code(q)
    _check(q.dim() == 3, "q must be (total_q, nheads, head_size)")
    total_q, nheads, head_dim = q.shape
    total_k = k.shape[0]
    batch = cu_seqlens_q.numel() - 1
    _check(batch > 0, "batch size must be positive")                                     # :371
    _check(head_dim in (16, 32, 64, 128), "head_size must be 16, 32, 64 or 128")         # :372
    for name, t, tot in (("q", q, total_q), ("k", k, total_k), ("v", v, total_k), ("out", out, total_q),
                         ("dout", dout, total_q), ("dq", dq, total_q), ("dk", dk, total_k), ("dv", dv, total_k)):
        _check_qkv(name, t, q.dtype, tot, nheads, head_dim)                              # :332-386
    _check(out.is_contiguous() and dout.is_contiguous(), "out and dout must be contiguous")  # :355-356
    _check_cu("cu_seqlens_q", cu_seqlens_q, batch)
    _check_cu("cu_seqlens_k", cu_seqlens_k, batch)
    _check(softmax_lse.is_cuda and softmax_lse.dtype == torch.float32 and softmax_lse.dim() == 3 and
           softmax_lse.shape[0] == batch and softmax_lse.shape[1] == nheads, "softmax_lse must be fp32 (batch, nheads, seqlen)")
    sparse = blockmask is not None
    sq_r, sk_r = round_seqlens(head_dim, max_seqlen_q, max_seqlen_k, sparse)
    if sparse:
        _check(blockmask.is_cuda and blockmask.dtype == torch.int32 and blockmask.is_contiguous(),
               "blockmask must be a contiguous int32 GPU tensor")
        _check(tuple(blockmask.shape) == (sk_r // 256, sq_r // 16),
               "blockmask has shape %s, expected %s" % (tuple(blockmask.shape), (sk_r // 256, sq_r // 16)))
    softmax_lse = softmax_lse.contiguous()

    dev = q.device
    with _OnDevice(dev):
        softmax_d = torch.empty((batch, nheads, sq_r), dtype=torch.float32, device=dev)
        seed, offset = _philox_state(dev, p_dropout, gen)
        strides = (dout.stride(), q.stride(), k.stride(), v.stride(), out.stride(), dq.stride(), dk.stride(), dv.stride())
        mq, mk = int(max_seqlen_q), int(max_seqlen_k)
        lse_stride = softmax_lse.shape[2]

        def fill(a):  # everything a call signature fixes; returns the workspace size of such calls
            a.dtype = code
            for name, st in zip(("do", "q", "k", "v", "o", "dq", "dk", "dv"), strides):
                setattr(a, name + "_row_stride", st[0])
                setattr(a, name + "_head_stride", st[1])
            a.lse_seq_stride = lse_stride
            a.batch, a.nheads, a.head_dim = batch, nheads, head_dim
            a.total_q, a.total_k = total_q, total_k
            a.max_seqlen_q, a.max_seqlen_k = mq, mk
            a.zero_tensors, a.is_causal = int(bool(zero_tensors)), int(bool(is_causal))
            # (the size query reads shapes, is_causal, p_dropout > 0 and which optional pointers are set)
            a.p_dropout = float(p_dropout)
            a.blockmask = 16 if sparse else None
            a.alibi_slopes = 16 if alibi_slopes is not None else None
            a.attn_bias = 16 if attn_bias is not None else None
            a.rotary_cos = 16 if rotary is not None else None
            return lib.fa_bwd_workspace_bytes(ctypes.byref(a))

        a, ws_bytes = _cached_args(("bwd", code, strides, lse_stride, batch, nheads, head_dim, total_q, total_k, mq, mk,
                                    bool(zero_tensors), bool(is_causal), p_dropout > 0, sparse, alibi_slopes is not None,
                                    attn_bias is not None, rotary is not None), BwdArgs, fill)
        a.dout, a.q, a.k, a.v, a.out = dout.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr()
        a.softmax_lse = softmax_lse.data_ptr()
        a.dq, a.dk, a.dv = dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
        a.softmax_d = softmax_d.data_ptr()
        a.cu_seqlens_q, a.cu_seqlens_k = cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr()
        a.blockmask = blockmask.data_ptr() if sparse else None
        a.p_dropout, a.softmax_scale = float(p_dropout), float(softmax_scale)
        a.philox_seed, a.philox_offset = seed, offset
        ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=dev) if ws_bytes else None
        a.workspace = ws.data_ptr() if ws is not None else None
        a.workspace_bytes = ws_bytes
        # (the struct is reused: the optional fields are cleared before the helpers below set the ones that are given)
        a.keep_words, a.keep_words_bytes, a.attn_bias, a.dbias, a.row_order = None, 0, None, None, None
        a.rotary_cos, a.rotary_sin = None, None
        a.stream = _stream_handle(dev)
        a.alibi_slopes = _check_alibi(alibi_slopes, nheads, dev, sparse)
        _keep_words_arg(a, keep_words, dev, sparse)
        bias_t = _bias_arg(a, attn_bias, q, batch, nheads, max_seqlen_q, max_seqlen_k, sparse)  # noqa: F841 (kept alive)
        if dbias is not None:
            _check(attn_bias is not None, "dbias without attn_bias")
            _check(dbias.dim() == 4 and tuple(dbias.shape[:2]) == (batch, nheads) and dbias.shape[2] >= max_seqlen_q and
                   dbias.shape[3] >= max_seqlen_k and dbias.stride(3) == 1 and dbias.dtype == q.dtype and dbias.device == dev,
                   "dbias must be (batch, nheads, >= max_seqlen_q, >= max_seqlen_k) in q's dtype, keys contiguous")
            a.dbias = dbias.data_ptr()
            a.dbias_batch_stride, a.dbias_head_stride, a.dbias_row_stride = dbias.stride(0), dbias.stride(1), dbias.stride(2)
        if sparse:
            _row_order_arg(a, row_order, sq_r, dev)
        _rotary_arg(a, rotary, q, max(int(max_seqlen_q), int(max_seqlen_k)))
        if main_kernel_events is not None and not sparse:  # (start, stop) torch.cuda.Event created with enable_timing=True
            for ev in main_kernel_events:
                if not ev.cuda_event:  # torch creates the HIP event lazily, on first record
                    ev.record()
            rc = lib.fa_bwd_profiled(ctypes.byref(a), main_kernel_events[0].cuda_event, main_kernel_events[1].cuda_event)
        else:
            rc = (lib.fa_bwd_block if sparse else lib.fa_bwd)(ctypes.byref(a))
        if rc != 0:
            _raise(rc, lib)
    return [dq, dk, dv, softmax_d]


def fwd(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, p_dropout, softmax_scale, zero_tensors,
        is_causal, return_softmax, gen=None, alibi_slopes=None, keep_words=None, attn_bias=None, rotary=None, q_rot=None):
    """mha_fwd (fmha_api.cpp:173-299): returns [o, softmax_lse] or [o, softmax_lse, s].
    alibi_slopes (extension, not in the reference): nheads fp32 slopes; scores get -slope * |i - j| added.
    keep_words (extension): a buffer from new_keep_words() in which the dropout keep decisions are left for bwd.
    attn_bias (extension): (1 or batch, 1 or nheads, max_seqlen_q, max_seqlen_k) in q's dtype, added to the scaled scores
    (positions counted inside the sequences; -inf masks); see prepare_attn_bias.
    rotary (extension): None, or (cos, sin) tables as for rotary(): q is turned by its position inside its sequence as the
    kernel loads it (k must come in rotated; not with return_softmax); q_rot: a (total_q, nheads, head_size) tensor that
    receives the rotated q, which bwd wants."""
    return _fwd_impl(q, k, v, cu_seqlens_q, cu_seqlens_k, None, max_seqlen_q, max_seqlen_k, p_dropout, softmax_scale,
                     zero_tensors, is_causal, return_softmax, gen, alibi_slopes, keep_words, attn_bias, rotary=rotary,
                     q_rot=q_rot)


def bwd(dout, q, k, v, out, softmax_lse, dq, dk, dv, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
        p_dropout, softmax_scale, zero_tensors, is_causal, gen=None, main_kernel_events=None, alibi_slopes=None,
        keep_words=None, attn_bias=None, dbias=None, rotary=None):
    """mha_bwd (fmha_api.cpp:302-449): fills dq, dk, dv in place, returns [dq, dk, dv, softmax_d].
    attn_bias: the bias the forward was given; dbias: None, or a zero-filled (batch, nheads, max_seqlen_q, max_seqlen_k)
    tensor of q's dtype in which the gradient of the bias is left (per batch entry and head: sum for a shared bias).
    main_kernel_events: optional (start, stop) timing events recorded around the dq/dk/dv kernel alone.
    alibi_slopes: the slopes the forward was given (extension, not in the reference).
    keep_words (extension): the buffer the forward of this call filled; the kernels then read the dropout decisions.
    rotary (extension): the tables the forward was given; q and k are then the rotated tensors and dq, dk come out as
    gradients with respect to the unrotated ones."""
    return _bwd_impl(dout, q, k, v, out, softmax_lse, dq, dk, dv, cu_seqlens_q, cu_seqlens_k, None, max_seqlen_q,
                     max_seqlen_k, p_dropout, softmax_scale, zero_tensors, is_causal, gen, main_kernel_events, alibi_slopes,
                     keep_words, attn_bias, dbias, rotary=rotary)


def fwd_block(q, k, v, cu_seqlens_q, cu_seqlens_k, blockmask, max_seqlen_q, max_seqlen_k, p_dropout, softmax_scale,
              is_causal, return_softmax, gen=None, row_order=None, alibi_slopes=None, attn_bias=None):
    """mha_fwd_block (fmha_api.cpp:451-573).  row_order (extension): None, or the int32 order of the 16-row blocks from
    blockmask_row_order() of the layout: the kernels' workgroups then own row blocks with similar key-block lists.
    alibi_slopes, attn_bias (extensions): as in fwd."""
    _check(blockmask is not None, "blockmask is required")
    return _fwd_impl(q, k, v, cu_seqlens_q, cu_seqlens_k, blockmask, max_seqlen_q, max_seqlen_k, p_dropout,
                     softmax_scale, False, is_causal, return_softmax, gen, alibi_slopes=alibi_slopes, attn_bias=attn_bias,
                     row_order=row_order)


def bwd_block(dout, q, k, v, out, softmax_lse, dq, dk, dv, cu_seqlens_q, cu_seqlens_k, blockmask, max_seqlen_q,
              max_seqlen_k, p_dropout, softmax_scale, is_causal, gen=None, row_order=None, alibi_slopes=None,
              attn_bias=None, dbias=None):
    """mha_bwd_block (fmha_api.cpp:575-718).  row_order: as in fwd_block; alibi_slopes, attn_bias, dbias: as in bwd."""
    _check(blockmask is not None, "blockmask is required")
    return _bwd_impl(dout, q, k, v, out, softmax_lse, dq, dk, dv, cu_seqlens_q, cu_seqlens_k, blockmask, max_seqlen_q,
                     max_seqlen_k, p_dropout, softmax_scale, False, is_causal, gen, alibi_slopes=alibi_slopes,
                     attn_bias=attn_bias, dbias=dbias, row_order=row_order)


def _check_rows(name, t):
    _check(t.is_cuda, "%s must be on the GPU" % name)
    _check(t.ndim == 2 and (t.shape[1] == 0 or t.stride(1) == 1), "%s must be 2-D with a contiguous last dimension" % name)


def _index_i64(indices, device):
    _check(indices.ndim == 1 and indices.device == device, "indices must be 1-D and on the same device")
    _check(indices.dtype in (torch.int64, torch.int32), "indices must be int64 or int32")
    return indices.to(torch.int64).contiguous()


def gather_rows(input, indices):
    """input[indices] for a 2-D GPU tensor: the gather of IndexFirstAxis.forward / IndexPutFirstAxis.backward
    (flash_attn/bert_padding.py:12-19, 51-57), done by fa_gather_rows."""
    _check_rows("input", input)
    if input.stride(0) < input.shape[1]:  # broadcast rows
        input = input.contiguous()
    idx = _index_i64(indices, input.device)
    lib = load_library()
    out = torch.empty((idx.numel(), input.shape[1]), dtype=input.dtype, device=input.device)
    es = input.element_size()
    with _OnDevice(input.device):
        rc = lib.fa_gather_rows(input.data_ptr(), out.data_ptr(), idx.data_ptr(), idx.numel(), input.shape[0],
                                input.shape[1] * es, input.stride(0) * es, out.stride(0) * es,
                                _stream_handle(input.device))
    if rc != 0:
        _raise(rc, lib)
    return out


def reduce_bias_grad(dbias, out, sum_batch, sum_heads):
    """out[...] = sum of the per-(batch, head) bias gradient `dbias` (batch, nheads, rows, cols padded to 8) over the
    batch entries (sum_batch) and / or heads (sum_heads), added in fp32 and rounded once, by fa_bias_grad_reduce.
    out: a (1 or batch, 1 or nheads, rows, cols) view in dbias's dtype, cols <= dbias.shape[3], innermost stride 1."""
    _check(dbias.dim() == 4 and out.dim() == 4 and dbias.is_cuda and out.device == dbias.device and out.dtype == dbias.dtype,
           "dbias and out must be 4-D tensors of one dtype on one GPU")
    batch, nheads, rows, _ = dbias.shape
    _check(tuple(out.shape[:3]) == (1 if sum_batch else batch, 1 if sum_heads else nheads, rows) and
           out.shape[3] <= dbias.shape[3] and dbias.stride(3) == 1 and (out.stride(3) == 1 or out.shape[3] <= 1),
           "out must be (1 or batch, 1 or nheads, rows, cols <= dbias's) with contiguous keys")
    lib = load_library()
    with _OnDevice(dbias.device):
        rc = lib.fa_bias_grad_reduce(dbias.data_ptr(), out.data_ptr(), _dtype_code(dbias), batch, nheads, rows, out.shape[3],
                                     dbias.stride(0), dbias.stride(1), dbias.stride(2), int(bool(sum_batch)),
                                     int(bool(sum_heads)), out.stride(0), out.stride(1), out.stride(2),
                                     _stream_handle(dbias.device))
    if rc != 0:
        _raise(rc, lib)
    return out


def scatter_rows(values, indices, first_axis_dim):
    """zeros(first_axis_dim, dim) with rows `indices` set to `values`: the scatter of IndexPutFirstAxis.forward /
    IndexFirstAxis.backward (flash_attn/bert_padding.py:21-30, 38-48), done in one pass by fa_scatter_rows (the output is
    not zero-filled first).  `indices` must be unique."""
    _check_rows("values", values)
    if values.stride(0) < values.shape[1]:
        values = values.contiguous()
    idx = _index_i64(indices, values.device)
    _check(idx.numel() == values.shape[0], "one index per row of values")
    lib = load_library()
    out = torch.empty((first_axis_dim, values.shape[1]), dtype=values.dtype, device=values.device)
    ws_bytes = lib.fa_scatter_rows_workspace_bytes(first_axis_dim)
    ws = torch.empty(max(ws_bytes // 4, 1), dtype=torch.int32, device=values.device)
    es = values.element_size()
    with _OnDevice(values.device):
        rc = lib.fa_scatter_rows(values.data_ptr(), out.data_ptr(), idx.data_ptr(), idx.numel(), first_axis_dim,
                                 values.shape[1] * es, values.stride(0) * es, out.stride(0) * es,
                                 ws.data_ptr(), ws_bytes, _stream_handle(values.device))
    if rc != 0:
        _raise(rc, lib)
    return out


def rotary(src, dst, cos, sin, n_rotated, conjugate=False, positions=None):
    """Rotary embedding of the first `n_rotated` parts of src (batch, seqlen, parts, nheads, headdim) into dst (same
    shape; may be src), remaining parts copied: the arithmetic of apply_rotary_pos_emb (flash_attn/rotary.py:32-42) for
    q and k of a packed qkv in one pass (fa_rotary).  cos, sin: (>= seqlen, headdim / 2) tables in src's dtype.
    positions: optional int32 (batch * seqlen,) table rows to use instead of the position inside the sequence."""
    _check(src.is_cuda and dst.is_cuda and src.ndim == 5 and src.shape == dst.shape and src.dtype == dst.dtype,
           "src and dst must be GPU tensors of the same (batch, seqlen, parts, nheads, headdim) shape and dtype")
    B, S, P, H, D = src.shape
    for t, name in ((src, "src"), (dst, "dst")):
        _check(t.stride(4) == 1 and (B <= 1 or t.stride(0) == S * t.stride(1)), "%s rows must be evenly strided" % name)
    _check(cos.shape == sin.shape and cos.ndim == 2 and cos.shape[1] == D // 2 and cos.dtype == src.dtype
           and cos.is_contiguous() and sin.is_contiguous() and cos.device == src.device,
           "cos / sin must be contiguous (rows, headdim / 2) tables in the tensor's dtype")
    if positions is not None:
        _check(positions.dtype == torch.int32 and positions.numel() == B * S and positions.is_contiguous()
               and positions.device == src.device, "positions must be a contiguous int32 tensor with one entry per row")
    else:
        _check(cos.shape[0] >= S, "the tables have fewer rows than the sequence has positions")
    lib = load_library()
    a = RotaryArgs()
    a.struct_bytes = ctypes.sizeof(a)
    a.dtype = _dtype_code(src)
    a.src, a.dst, a.cos_table, a.sin_table = src.data_ptr(), dst.data_ptr(), cos.data_ptr(), sin.data_ptr()
    a.positions = positions.data_ptr() if positions is not None else None
    a.n_rows = B * S
    a.src_row_stride, a.src_part_stride, a.src_head_stride = src.stride(1), src.stride(2), src.stride(3)
    a.dst_row_stride, a.dst_part_stride, a.dst_head_stride = dst.stride(1), dst.stride(2), dst.stride(3)
    in_place = src.data_ptr() == dst.data_ptr() and src.stride() == dst.stride()
    a.n_parts, a.n_rotated, a.n_heads, a.head_dim = (n_rotated if in_place else P), n_rotated, H, D  # in place: no copy
    a.seqlen, a.table_rows, a.conjugate = S, cos.shape[0], int(bool(conjugate))
    a.stream = _stream_handle(src.device)
    with _OnDevice(src.device):
        rc = lib.fa_rotary(ctypes.byref(a))
    if rc != 0:
        _raise(rc, lib)
    return dst
