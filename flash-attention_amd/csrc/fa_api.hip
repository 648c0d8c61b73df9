// C-ABI front end: argument validation, seqlen rounding, workspace layout and kernel dispatch.
// Host-side counterpart of mha_fwd / mha_bwd / mha_fwd_block / mha_bwd_block
// (csrc/flash_attn/fmha_api.cpp:173-718).  Every failed check returns a negative status and leaves a
// message for fa_last_error(); nothing here synchronises the device or terminates the process.
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <atomic>
#include <mutex>

#include "../../include/flash_attn_gfx950_bench.h"
#include "fa_params.h"

// ---- fa_fwd_block_noalloc: the block activity maps live in this file-scope device array instead of caller scratch.
// Every GPU the library runs on holds its own copy at its own address until the process ends; `scratch` itself is only
// a host-side handle, so the device address is looked up once per device (with that device current) and used from then on.
constexpr size_t kNoAllocScratchBytes = FA_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];

namespace {
std::atomic<int> g_launch_policy{0};
}
namespace fa {
int launch_policy() { return g_launch_policy.load(std::memory_order_relaxed); }
}  // namespace fa

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

#define FA_REQUIRE(cond, ...) \
  do {                        \
    if (!(cond)) return fail(FA_ERR_INVALID_ARGUMENT, __VA_ARGS__); \
  } while (0)

#define FA_LAUNCH(expr)                                                                              \
  do {                                                                                               \
    hipError_t e_ = (expr);                                                                          \
    if (e_ != hipSuccess) return fail(FA_ERR_LAUNCH, "%s failed: %s", #expr, hipGetErrorString(e_)); \
  } while (0)

inline size_t align16(size_t x) { return (x + 15) & ~(size_t)15; }
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
// strides are in elements: multiples of 8 (16-byte vectors), non-negative, and below 2^24 so that the kernels' 32-bit
// per-lane byte offsets inside a tile (up to 63 rows) cannot overflow
inline bool stride_ok(int64_t s) { return s % 8 == 0 && s >= 0 && s < ((int64_t)1 << 24); }
// tensors that are written: rows and heads must not overlap (a zero or short stride would make several workgroups write
// the same bytes)
inline bool out_stride_ok(int64_t s, int head_dim) { return stride_ok(s) && s >= head_dim; }

struct Rounded {
  int sq_r, sk_r;
};

// fmha_api.cpp:232-241 (dense; blocksize_c taken for a device that is not sm80) and :509-514 (block-sparse)
Rounded round_seqlens(int head_dim, int max_sq, int max_sk, bool blocksparse) {
  Rounded r;
  if (blocksparse) {
    r.sk_r = ((max_sk + 255) / 256) * 256;
    if (r.sk_r <= 256) r.sk_r = 256;
  } else {
    const int blocksize_c = head_dim == 128 ? 128 : 256;
    r.sk_r = ((max_sk + blocksize_c - 1) / blocksize_c) * blocksize_c;
    if (max_sk <= 128) r.sk_r = 128;
    else if (max_sk <= 256) r.sk_r = 256;
  }
  r.sq_r = ((max_sq + 15) / 16) * 16;
  return r;
}

struct SparseLayout {
  int nrb, ncb, nqt, ncw, nrw;
  size_t offr, offq, offc, offi, bytes;
};

SparseLayout sparse_layout(const Rounded& r) {
  SparseLayout s;
  s.nrb = r.sq_r / 16;
  s.ncb = r.sk_r / 256;
  s.nqt = (r.sq_r + fa::kFwdBM - 1) / fa::kFwdBM;
  s.ncw = (s.ncb + 63) / 64;
  s.nrw = (s.nrb + 63) / 64;
  s.offr = 0;
  s.offq = s.offr + align16((size_t)s.nrb * s.ncw * 8);
  s.offc = s.offq + align16((size_t)s.nqt * s.ncw * 8);
  s.offi = s.offc + align16((size_t)s.ncb * s.nrw * 8);  // inverse of the row order
  s.bytes = s.offi + align16((size_t)s.nrb * 4);
  return s;
}

// Key-split forward: worth it when the query tiles alone cannot fill the chip and there are many key tiles to share.
// Returns the number of splits (1 = single pass) and the scratch the partial results need.
struct SplitPlan {
  int n_splits;
  size_t o_bytes, bytes;
};
SplitPlan split_plan(int batch, int nheads, int head_dim, int total_q, int max_sq, int max_sk, int sq_r, bool causal,
                     bool sparse) {
  SplitPlan sp{1, 0, 0};
  if (causal || sparse || max_sq <= 0 || max_sq > fa::kFwdBM) return sp;  // one query tile per (batch, head) only
  const int64_t blocks = (int64_t)batch * nheads * ((max_sq + fa::kFwdBM - 1) / fa::kFwdBM);
  const int key_tiles = (max_sk + 63) / 64;
  if (blocks >= 128 || key_tiles < 8) return sp;
  int64_t n = (768 + blocks - 1) / blocks;  // about three workgroups per compute unit
  if (n > key_tiles / 4) n = key_tiles / 4; // at least four key tiles per split
  if (n > 64) n = 64;
  if (n < 2) return sp;
  sp.n_splits = (int)n;
  sp.o_bytes = align16((size_t)n * total_q * nheads * head_dim * 4);
  sp.bytes = sp.o_bytes + align16((size_t)n * batch * nheads * sq_r * 4);
  return sp;
}

int build_maps(const int32_t* blockmask, const int32_t* row_order, unsigned char* ws, const SparseLayout& sl,
               fa::SparseMaps* out, hipStream_t stream) {
  FA_LAUNCH(fa::launch_fill_f32(reinterpret_cast<float*>(ws), sl.bytes / 4, 0.f, stream));
  FA_LAUNCH(fa::launch_build_sparse_maps(blockmask, reinterpret_cast<uint64_t*>(ws + sl.offr),
                                         reinterpret_cast<uint64_t*>(ws + sl.offq),
                                         reinterpret_cast<uint64_t*>(ws + sl.offc), sl.nrb, sl.ncb, fa::kFwdBM, sl.nqt,
                                         sl.ncw, sl.nrw, row_order, reinterpret_cast<int32_t*>(ws + sl.offi), stream));
  out->order = row_order;
  out->rbits = reinterpret_cast<const uint64_t*>(ws + sl.offr);
  out->qbits = reinterpret_cast<const uint64_t*>(ws + sl.offq);
  out->cbits = reinterpret_cast<const uint64_t*>(ws + sl.offc);
  out->nrb = sl.nrb;
  out->ncb = sl.ncb;
  out->nqt = sl.nqt;
  out->ncw = sl.ncw;
  out->nrw = sl.nrw;
  return FA_OK;
}

// Causal launches (fa_params.h, map_tile): how many (batch, head) pairs of an XCD are in flight together.  All of them while
// their K and V stay within about twice an XCD's 4 MB of L2 (dearest-first over everything balances best, and what the L2
// misses then costs nothing measurable); beyond that as many as hold 6 MB of K and V, and at least four (fewer cost more in
// balance than their traffic saves).  Measured: profiles/causal_tile_order_hbm_traffic.md.
int causal_tile_group(int batch, int nheads, int head_dim, int max_seqlen_k) {
  const int64_t pairs = ((int64_t)batch * nheads + 7) / 8;
  const int64_t kv_bytes = (int64_t)max_seqlen_k * head_dim * 2 * 2;
  if (pairs * kv_bytes <= ((int64_t)8 << 20)) return 0;
  const int64_t g = ((int64_t)6 << 20) / kv_bytes;
  return (int)(g < 4 ? 4 : g);
}

fa::PhiloxKey make_key(uint64_t seed, uint64_t offset) {
  fa::PhiloxKey k;
  k.k0 = (uint32_t)seed;
  k.k1 = (uint32_t)(seed >> 32) ^ (uint32_t)(offset >> 32);
  k.c3 = (uint32_t)offset;
  return k;
}

int check_common(uint32_t struct_bytes, size_t expect, int dtype, int batch, int nheads, int head_dim, int total_q,
                 int total_k, int max_sq, int max_sk, float p_dropout, float scale) {
  FA_REQUIRE(struct_bytes == expect, "struct_bytes is %u, this library expects %zu (ABI mismatch)", struct_bytes, expect);
  FA_REQUIRE(dtype == FA_FP16 || dtype == FA_BF16, "dtype must be fp16 or bf16");                  // fmha_api.cpp:198
  FA_REQUIRE(batch > 0, "batch_size must be positive");                                            // :223
  FA_REQUIRE(nheads > 0, "nheads must be positive");
  FA_REQUIRE(head_dim == 16 || head_dim == 32 || head_dim == 64 || head_dim == 128,
             "head_size must be 16, 32, 64 or 128 (got %d)", head_dim);                            // :224
  FA_REQUIRE(total_q >= 0 && total_k >= 0, "negative token count");
  FA_REQUIRE(max_sq > 0 && max_sk > 0, "max_seqlen must be positive");
  FA_REQUIRE(p_dropout >= 0.f && p_dropout < 1.f, "p_dropout must be in [0, 1) (got %g)", p_dropout);  // :113
  FA_REQUIRE(std::isfinite(scale) && scale > 0.f, "softmax_scale must be finite and positive (got %g)", scale);
  return FA_OK;
}

int fwd_impl(const fa_fwd_args* a, bool want_block) {
  if (!a) return fail(FA_ERR_INVALID_ARGUMENT, "args is NULL");
  int rc = check_common(a->struct_bytes, sizeof(fa_fwd_args), a->dtype, a->batch, a->nheads, a->head_dim, a->total_q,
                        a->total_k, a->max_seqlen_q, a->max_seqlen_k, a->p_dropout, a->softmax_scale);
  if (rc) return rc;
  const bool sparse = a->blockmask != nullptr;
  FA_REQUIRE(sparse == want_block, want_block ? "fa_fwd_block needs a blockmask" : "fa_fwd takes no blockmask; call fa_fwd_block");
  FA_REQUIRE(a->q && a->k && a->v && a->o && a->softmax_lse && a->cu_seqlens_q && a->cu_seqlens_k, "NULL tensor pointer");
  FA_REQUIRE(aligned16(a->q) && aligned16(a->k) && aligned16(a->v) && aligned16(a->o),
             "q, k, v, o must be 16-byte aligned");
  FA_REQUIRE(stride_ok(a->q_row_stride) && stride_ok(a->q_head_stride) && stride_ok(a->k_row_stride) &&
                 stride_ok(a->k_head_stride) && stride_ok(a->v_row_stride) && stride_ok(a->v_head_stride) &&
                 stride_ok(a->o_row_stride) && stride_ok(a->o_head_stride),
             "row and head strides must be multiples of 8 elements in [0, 2^24)");
  FA_REQUIRE(out_stride_ok(a->o_row_stride, a->head_dim) && out_stride_ok(a->o_head_stride, a->head_dim),
             "row and head strides of o must be at least head_dim (the output's rows and heads may not overlap)");

  if (a->alibi_slopes && a->attn_bias) return fail(FA_ERR_UNSUPPORTED, "alibi_slopes and attn_bias are not supported together");

  const Rounded r = round_seqlens(a->head_dim, a->max_seqlen_q, a->max_seqlen_k, sparse);
  // the probability dump puts the rounded query length and batch * heads into grid dimensions: refuse what does not fit
  // before anything is enqueued
  if (a->s_dmask && (r.sq_r > 65535 || (int64_t)a->batch * a->nheads > 65535))
    return fail(FA_ERR_UNSUPPORTED, "s_dmask is limited to max_seqlen_q <= 65535 and batch * nheads <= 65535");
  hipStream_t stream = reinterpret_cast<hipStream_t>(a->stream);
  const bool dropout = a->p_dropout > 0.f;
  const float p_keep = 1.f - a->p_dropout;

  fa::FwdParams p;
  memset(&p, 0, sizeof(p));
  if (sparse) {
    const SparseLayout sl = sparse_layout(r);
    if (!a->workspace || a->workspace_bytes < sl.bytes)
      return fail(FA_ERR_WORKSPACE, "workspace of %zu bytes needed, %zu given", sl.bytes, a->workspace_bytes);
    FA_REQUIRE(aligned16(a->workspace), "workspace must be 16-byte aligned");
    FA_REQUIRE(!a->row_order || (reinterpret_cast<uintptr_t>(a->row_order) & 3) == 0, "row_order must be 4-byte aligned");
    rc = build_maps(a->blockmask, a->is_causal ? nullptr : a->row_order, reinterpret_cast<unsigned char*>(a->workspace), sl,
                    &p.sp, stream);
    if (rc) return rc;
  }
  if (a->zero_tensors) {  // fmha_api.cpp:256-260
    FA_LAUNCH(fa::launch_zero_rows(a->o, a->o_row_stride, a->o_head_stride, a->total_q, a->nheads, a->head_dim, stream));
    FA_LAUNCH(fa::launch_fill_f32(a->softmax_lse, (size_t)a->batch * a->nheads * r.sq_r, -INFINITY, stream));
    if (a->s_dmask)  // 16-bit elements, an even number of them (the rounded key length is a multiple of 128)
      FA_LAUNCH(fa::launch_fill_f32(reinterpret_cast<float*>(a->s_dmask),
                                    (size_t)a->batch * a->nheads * r.sq_r * r.sk_r / 2, 0.f, stream));
  }

  p.q = a->q; p.k = a->k; p.v = a->v; p.o = a->o; p.lse = a->softmax_lse;
  p.cu_q = a->cu_seqlens_q; p.cu_k = a->cu_seqlens_k;
  p.q_rs = a->q_row_stride; p.q_hs = a->q_head_stride;
  p.k_rs = a->k_row_stride; p.k_hs = a->k_head_stride;
  p.v_rs = a->v_row_stride; p.v_hs = a->v_head_stride;
  p.o_rs = a->o_row_stride; p.o_hs = a->o_head_stride;
  p.B = a->batch; p.H = a->nheads;
  p.total_q = a->total_q; p.total_k = a->total_k;
  p.max_sq = a->max_seqlen_q; p.max_sk = a->max_seqlen_k;
  p.sq_r = r.sq_r;
  p.nq_tiles = (a->max_seqlen_q + fa::kFwdBM - 1) / fa::kFwdBM;
  p.tile_group = a->is_causal ? causal_tile_group(a->batch, a->nheads, a->head_dim, a->max_seqlen_k) : 0;
  p.scale = a->softmax_scale;
  p.scale_log2 = a->softmax_scale * fa::kLog2e;
  p.rp_keep = 1.f / p_keep;
  p.keep_thr = (uint32_t)std::floor(p_keep * 65535.0);  // fmha_api.cpp:110
  p.pk = make_key(a->philox_seed, a->philox_offset);
  p.alibi = a->alibi_slopes;
  if (a->attn_bias) {
    FA_REQUIRE(aligned16(a->attn_bias) && a->bias_row_stride % 8 == 0 && a->bias_row_stride >= a->max_seqlen_k &&
                   a->bias_batch_stride >= 0 && a->bias_head_stride >= 0,
               "attn_bias must be 16-byte aligned with a row stride that is a multiple of 8 and at least max_seqlen_k");
    if ((int64_t)a->max_seqlen_q * a->bias_row_stride >= ((int64_t)1 << 31))
      return fail(FA_ERR_UNSUPPORTED, "attn_bias: a (batch, head) slice is limited to 2^31 elements");
    p.bias = a->attn_bias;
    p.bias_bs = a->bias_batch_stride; p.bias_hs = a->bias_head_stride; p.bias_rs = a->bias_row_stride;
  }
  if (a->rotary_cos || a->rotary_sin) {
    FA_REQUIRE(a->rotary_cos && a->rotary_sin && aligned16(a->rotary_cos) && aligned16(a->rotary_sin),
               "rotary_cos and rotary_sin come together, 16-byte aligned");
    FA_REQUIRE(a->rotary_table_rows >= a->max_seqlen_q, "the rotary tables must have a row for every query position");
    if (sparse || a->alibi_slopes || a->attn_bias)
      return fail(FA_ERR_UNSUPPORTED, "rotary_cos with a blockmask, alibi_slopes or attn_bias: rotate with fa_rotary first");
    if (a->s_dmask) return fail(FA_ERR_UNSUPPORTED, "rotary_cos with s_dmask: rotate with fa_rotary first");
    p.rot_cos = a->rotary_cos; p.rot_sin = a->rotary_sin; p.rot_rows = a->rotary_table_rows;
    if (a->q_rot) {
      FA_REQUIRE(aligned16(a->q_rot) && a->q_rot_row_stride % 8 == 0 && a->q_rot_head_stride % 8 == 0 &&
                     a->q_rot_head_stride >= a->head_dim && a->q_rot_row_stride >= a->head_dim,
                 "q_rot must be 16-byte aligned with strides that are multiples of 8 and at least head_dim");
      p.q_rot = a->q_rot; p.qr_rs = a->q_rot_row_stride; p.qr_hs = a->q_rot_head_stride;
    }
  }
  if (a->keep_words && dropout && !sparse) {
    FA_REQUIRE(aligned16(a->keep_words), "keep_words must be 16-byte aligned");
    const size_t kw_need = fa_keep_words_bytes(a->batch, a->nheads, a->max_seqlen_q, a->max_seqlen_k);
    if (a->keep_words_bytes < kw_need)
      return fail(FA_ERR_WORKSPACE, "keep_words of %zu bytes needed, %zu given", kw_need, a->keep_words_bytes);
    p.keep_words = reinterpret_cast<uint32_t*>(a->keep_words);
    p.kw_q = (int)fa::keep_words_q_extent(a->max_seqlen_q);
    p.kw_kb = (int)fa::keep_words_key_blocks(a->max_seqlen_k);
  }
  // short query side, long key side: split the keys over several workgroups if the caller brought the scratch for it
  const SplitPlan sp = split_plan(a->batch, a->nheads, a->head_dim, a->total_q, a->max_seqlen_q, a->max_seqlen_k, r.sq_r,
                                  a->is_causal != 0, sparse);
  const bool split = sp.n_splits > 1 && a->workspace && a->workspace_bytes >= sp.bytes && aligned16(a->workspace);
  if (split) {
    p.n_splits = sp.n_splits;
    p.o_part = reinterpret_cast<float*>(a->workspace);
    p.lse_part = reinterpret_cast<float*>(reinterpret_cast<unsigned char*>(a->workspace) + sp.o_bytes);
  }
  FA_LAUNCH(fa::launch_fwd(p, a->dtype, a->head_dim, a->is_causal != 0, dropout, sparse, stream));
  if (split) FA_LAUNCH(fa::launch_fwd_combine(p, a->dtype, a->head_dim, stream));

  if (a->s_dmask) {
    fa::DumpParams d;
    memset(&d, 0, sizeof(d));
    d.q = a->q; d.k = a->k; d.lse = a->softmax_lse; d.s = a->s_dmask;
    d.cu_q = a->cu_seqlens_q; d.cu_k = a->cu_seqlens_k;
    d.q_rs = a->q_row_stride; d.q_hs = a->q_head_stride; d.k_rs = a->k_row_stride; d.k_hs = a->k_head_stride;
    d.B = a->batch; d.H = a->nheads; d.D = a->head_dim;
    d.total_q = a->total_q; d.total_k = a->total_k;
    d.max_sq = a->max_seqlen_q; d.max_sk = a->max_seqlen_k;
    d.sq_r = r.sq_r; d.sk_r = r.sk_r;
    d.scale = a->softmax_scale;
    d.causal = a->is_causal != 0; d.dropout = dropout; d.sparse = sparse;
    d.keep_thr = p.keep_thr; d.pk = p.pk; d.sp = p.sp; d.alibi = p.alibi;
    d.bias = p.bias; d.bias_bs = p.bias_bs; d.bias_hs = p.bias_hs; d.bias_rs = p.bias_rs;
    FA_LAUNCH(fa::launch_dump_probs(d, a->dtype, stream));
  }
  return FA_OK;
}

// Scratch of the one-kernel backward (fa_bwd_fused_kernel.h) where it applies, else 0: an fp32 dQ and its hand-over counters.
// It applies to head_dim 64 without mask, dropout, bias or block layout, when the launch policy asks for it, and only when
// all key tiles of a (batch, head) fit one XCD at once with room to spare (they wait for each other).
size_t fused_bwd_bytes(const fa_bwd_args* a) {
  if ((fa::launch_policy() & 0x30) != 0x20) return 0;
  if (a->head_dim != 64 || a->blockmask || a->p_dropout > 0.f || a->alibi_slopes || a->attn_bias || a->is_causal ||
      a->rotary_cos)
    return 0;
  if (a->batch <= 0 || a->nheads <= 0 || a->max_seqlen_q <= 0 || a->max_seqlen_k <= 0) return 0;
  if ((a->max_seqlen_k + fa::kBwdBN - 1) / fa::kBwdBN > 32) return 0;
  const size_t nqt = ((size_t)a->max_seqlen_q + fa::kFusedBM - 1) / fa::kFusedBM;
  return (size_t)a->batch * a->nheads * nqt * (fa::kFusedBM * 64 * 4 + 4 * 4);
}

int bwd_impl(const fa_bwd_args* a, bool want_block, void* ev_main_start = nullptr, void* ev_main_stop = nullptr) {
  if (!a) return fail(FA_ERR_INVALID_ARGUMENT, "args is NULL");
  int rc = check_common(a->struct_bytes, sizeof(fa_bwd_args), a->dtype, a->batch, a->nheads, a->head_dim, a->total_q,
                        a->total_k, a->max_seqlen_q, a->max_seqlen_k, a->p_dropout, a->softmax_scale);
  if (rc) return rc;
  const bool sparse = a->blockmask != nullptr;
  FA_REQUIRE(sparse == want_block, want_block ? "fa_bwd_block needs a blockmask" : "fa_bwd takes no blockmask; call fa_bwd_block");
  if (a->alibi_slopes && a->attn_bias) return fail(FA_ERR_UNSUPPORTED, "alibi_slopes and attn_bias are not supported together");
  FA_REQUIRE(a->dout && a->q && a->k && a->v && a->out && a->softmax_lse && a->dq && a->dk && a->dv && a->softmax_d &&
                 a->cu_seqlens_q && a->cu_seqlens_k, "NULL tensor pointer");
  FA_REQUIRE(aligned16(a->dout) && aligned16(a->q) && aligned16(a->k) && aligned16(a->v) && aligned16(a->out) &&
                 aligned16(a->dq) && aligned16(a->dk) && aligned16(a->dv), "tensors must be 16-byte aligned");
  const int64_t strides[] = {a->do_row_stride, a->do_head_stride, a->q_row_stride,  a->q_head_stride,  a->k_row_stride,
                             a->k_head_stride, a->v_row_stride,  a->v_head_stride, a->o_row_stride,  a->o_head_stride,
                             a->dq_row_stride, a->dq_head_stride, a->dk_row_stride, a->dk_head_stride, a->dv_row_stride,
                             a->dv_head_stride};
  for (int64_t s : strides) FA_REQUIRE(stride_ok(s), "row and head strides must be multiples of 8 elements in [0, 2^24)");
  for (int i = 10; i < 16; i++)
    FA_REQUIRE(out_stride_ok(strides[i], a->head_dim),
               "row and head strides of dq, dk, dv must be at least head_dim (the gradients' rows and heads may not overlap)");

  const Rounded r = round_seqlens(a->head_dim, a->max_seqlen_q, a->max_seqlen_k, sparse);
  FA_REQUIRE(a->lse_seq_stride >= a->max_seqlen_q, "softmax_lse is shorter than max_seqlen_q");
  hipStream_t stream = reinterpret_cast<hipStream_t>(a->stream);
  const bool dropout = a->p_dropout > 0.f;
  const float p_keep = 1.f - a->p_dropout;

  const SparseLayout sl = sparse_layout(r);
  // the dense backward needs no scratch: no dq_tmp (fmha_api.cpp:403-404); it uses some, if offered, to split the keys of
  // a lone query tile over several workgroups (see below)
  const size_t need = sparse ? sl.bytes : 0;
  if (need > 0 && (!a->workspace || a->workspace_bytes < need))
    return fail(FA_ERR_WORKSPACE, "workspace of %zu bytes needed, %zu given", need, a->workspace_bytes);
  FA_REQUIRE(need == 0 || aligned16(a->workspace), "workspace must be 16-byte aligned");
  unsigned char* ws = reinterpret_cast<unsigned char*>(a->workspace);

  fa::BwdParams p;
  memset(&p, 0, sizeof(p));
  if (sparse) {
    FA_REQUIRE(!a->row_order || (reinterpret_cast<uintptr_t>(a->row_order) & 3) == 0, "row_order must be 4-byte aligned");
    rc = build_maps(a->blockmask, a->is_causal ? nullptr : a->row_order, ws, sl, &p.sp, stream);
    if (rc) return rc;
  }
  if (a->zero_tensors) {  // fmha_api.cpp:406-411
    FA_LAUNCH(fa::launch_zero_rows(a->dq, a->dq_row_stride, a->dq_head_stride, a->total_q, a->nheads, a->head_dim, stream));
    FA_LAUNCH(fa::launch_zero_rows(a->dk, a->dk_row_stride, a->dk_head_stride, a->total_k, a->nheads, a->head_dim, stream));
    FA_LAUNCH(fa::launch_zero_rows(a->dv, a->dv_row_stride, a->dv_head_stride, a->total_k, a->nheads, a->head_dim, stream));
    FA_LAUNCH(fa::launch_fill_f32(a->softmax_d, (size_t)a->batch * a->nheads * r.sq_r, 0.f, stream));
  }
  p.dout = a->dout; p.q = a->q; p.k = a->k; p.v = a->v; p.out = a->out; p.lse = a->softmax_lse;
  p.dsoftmax = a->softmax_d;
  p.dq = a->dq; p.dk = a->dk; p.dv = a->dv;
  p.cu_q = a->cu_seqlens_q; p.cu_k = a->cu_seqlens_k;
  p.do_rs = a->do_row_stride; p.do_hs = a->do_head_stride;
  p.q_rs = a->q_row_stride; p.q_hs = a->q_head_stride;
  p.k_rs = a->k_row_stride; p.k_hs = a->k_head_stride;
  p.v_rs = a->v_row_stride; p.v_hs = a->v_head_stride;
  p.o_rs = a->o_row_stride; p.o_hs = a->o_head_stride;
  p.dq_rs = a->dq_row_stride; p.dq_hs = a->dq_head_stride;
  p.dk_rs = a->dk_row_stride; p.dk_hs = a->dk_head_stride;
  p.dv_rs = a->dv_row_stride; p.dv_hs = a->dv_head_stride;
  p.B = a->batch; p.H = a->nheads;
  p.total_q = a->total_q; p.total_k = a->total_k;
  p.max_sq = a->max_seqlen_q; p.max_sk = a->max_seqlen_k;
  p.sq_r = r.sq_r; p.lse_stride = a->lse_seq_stride;
  p.nk_tiles = (a->max_seqlen_k + fa::kBwdBN - 1) / fa::kBwdBN;
  p.nq_tiles = (a->max_seqlen_q + fa::kFwdBM - 1) / fa::kFwdBM;
  p.tile_group = a->is_causal ? causal_tile_group(a->batch, a->nheads, a->head_dim, a->max_seqlen_k) : 0;
  p.scale = a->softmax_scale;
  p.scale_log2 = a->softmax_scale * fa::kLog2e;
  p.p_keep = p_keep;
  p.rp_keep = 1.f / p_keep;
  p.keep_thr = (uint32_t)std::floor(p_keep * 65535.0);
  p.pk = make_key(a->philox_seed, a->philox_offset);
  p.alibi = a->alibi_slopes;
  if (a->attn_bias) {
    FA_REQUIRE(aligned16(a->attn_bias) && a->bias_row_stride % 8 == 0 && a->bias_row_stride >= a->max_seqlen_k &&
                   a->bias_batch_stride >= 0 && a->bias_head_stride >= 0,
               "attn_bias must be 16-byte aligned with a row stride that is a multiple of 8 and at least max_seqlen_k");
    if ((int64_t)a->max_seqlen_q * a->bias_row_stride >= ((int64_t)1 << 31))
      return fail(FA_ERR_UNSUPPORTED, "attn_bias: a (batch, head) slice is limited to 2^31 elements");
    p.bias = a->attn_bias;
    p.bias_bs = a->bias_batch_stride; p.bias_hs = a->bias_head_stride; p.bias_rs = a->bias_row_stride;
  }
  if (a->dbias) {
    FA_REQUIRE(a->attn_bias, "dbias without attn_bias");
    FA_REQUIRE(a->dbias_row_stride >= a->max_seqlen_k &&
                   a->dbias_head_stride >= (int64_t)a->max_seqlen_q * a->dbias_row_stride &&
                   (a->batch == 1 || a->dbias_batch_stride >= (int64_t)a->nheads * a->dbias_head_stride) &&
                   (reinterpret_cast<uintptr_t>(a->dbias) & 1) == 0,
               "dbias needs its own slice for every (batch, head) - rows of at least max_seqlen_k elements, head stride of at least "
               "max_seqlen_q rows, batch stride of at least nheads head strides - and 2-byte alignment");
    if ((int64_t)a->max_seqlen_q * a->dbias_row_stride >= ((int64_t)1 << 31))
      return fail(FA_ERR_UNSUPPORTED, "dbias: a (batch, head) slice is limited to 2^31 elements");
    p.dbias = a->dbias;
    p.dbias_bs = a->dbias_batch_stride; p.dbias_hs = a->dbias_head_stride; p.dbias_rs = a->dbias_row_stride;
  }
  if (a->rotary_cos || a->rotary_sin) {
    FA_REQUIRE(a->rotary_cos && a->rotary_sin && (reinterpret_cast<uintptr_t>(a->rotary_cos) & 3) == 0 &&
                   (reinterpret_cast<uintptr_t>(a->rotary_sin) & 3) == 0,
               "rotary_cos and rotary_sin come together, 4-byte aligned");
    FA_REQUIRE(a->rotary_table_rows >= a->max_seqlen_q && a->rotary_table_rows >= a->max_seqlen_k,
               "the rotary tables must have a row for every query and key position");
    if (sparse || a->alibi_slopes || a->attn_bias)
      return fail(FA_ERR_UNSUPPORTED, "rotary_cos with a blockmask, alibi_slopes or attn_bias: rotate with fa_rotary first");
    p.rot_cos = a->rotary_cos; p.rot_sin = a->rotary_sin; p.rot_rows = a->rotary_table_rows;
  }
  if (a->keep_words && dropout && !sparse) {
    FA_REQUIRE(aligned16(a->keep_words), "keep_words must be 16-byte aligned");
    const size_t kw_need = fa_keep_words_bytes(a->batch, a->nheads, a->max_seqlen_q, a->max_seqlen_k);
    if (a->keep_words_bytes < kw_need)
      return fail(FA_ERR_WORKSPACE, "keep_words of %zu bytes needed, %zu given", kw_need, a->keep_words_bytes);
    p.keep_words = reinterpret_cast<const uint32_t*>(a->keep_words);
    p.kw_q = (int)fa::keep_words_q_extent(a->max_seqlen_q);
    p.kw_kb = (int)fa::keep_words_key_blocks(a->max_seqlen_k);
  }

  // the whole backward in one kernel, if the caller brought the scratch for it
  const size_t fused_need = fused_bwd_bytes(a);
  if (fused_need > 0 && !a->dbias && a->workspace && a->workspace_bytes >= fused_need && aligned16(a->workspace)) {
    p.nqt_ring = (a->max_seqlen_q + fa::kFusedBM - 1) / fa::kFusedBM;
    p.dq_acc = reinterpret_cast<float*>(a->workspace);
    p.dq_flags = reinterpret_cast<int*>(ws + (size_t)a->batch * a->nheads * p.nqt_ring * fa::kFusedBM * a->head_dim * 4);
    FA_LAUNCH(fa::launch_bwd_fused(p, a->dtype, stream, reinterpret_cast<hipEvent_t>(ev_main_start),
                                   reinterpret_cast<hipEvent_t>(ev_main_stop)));
    return FA_OK;
  }
  // short query side, long key side: the dQ kernel would walk all keys with one workgroup per (batch, head)
  const SplitPlan sp = split_plan(a->batch, a->nheads, a->head_dim, a->total_q, a->max_seqlen_q, a->max_seqlen_k, r.sq_r,
                                  a->is_causal != 0, sparse);
  const bool split = sp.n_splits > 1 && a->workspace && a->workspace_bytes >= sp.o_bytes && aligned16(a->workspace);
  if (split) {
    p.n_splits = sp.n_splits;
    p.dq_part = reinterpret_cast<float*>(a->workspace);
  }
  if (!split && fa::merged_backward_launch(a->head_dim, a->batch * a->nheads, a->max_seqlen_q, a->is_causal != 0, dropout,
                                           p.keep_words != nullptr, sparse, p.alibi != nullptr || p.bias != nullptr,
                                           p.rot_cos != nullptr, sp.n_splits)) {
    if (ev_main_start) FA_LAUNCH(hipEventRecord(reinterpret_cast<hipEvent_t>(ev_main_start), stream));
    FA_LAUNCH(fa::launch_bwd(p, 2, a->dtype, a->head_dim, a->is_causal != 0, dropout, sparse, stream));  // both in one launch
    if (ev_main_stop) FA_LAUNCH(hipEventRecord(reinterpret_cast<hipEvent_t>(ev_main_stop), stream));
    return FA_OK;
  }
  FA_LAUNCH(fa::launch_bwd(p, 0, a->dtype, a->head_dim, a->is_causal != 0, dropout, sparse, stream));  // dQ, softmax_d
  if (split) FA_LAUNCH(fa::launch_dq_combine(p, a->dtype, a->head_dim, stream));
  if (ev_main_start) FA_LAUNCH(hipEventRecord(reinterpret_cast<hipEvent_t>(ev_main_start), stream));
  FA_LAUNCH(fa::launch_bwd(p, 1, a->dtype, a->head_dim, a->is_causal != 0, dropout, sparse, stream));  // dK, dV
  if (ev_main_stop) FA_LAUNCH(hipEventRecord(reinterpret_cast<hipEvent_t>(ev_main_stop), stream));
  return FA_OK;
}

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

int noalloc_scratch(void** out) {
  int dev = -1;
  FA_LAUNCH(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return fail(FA_ERR_UNSUPPORTED, "device ordinal %d out of range", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    FA_LAUNCH(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (!ptr) return fail(FA_ERR_LAUNCH, "hipGetSymbolAddress returned a null address");
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return FA_OK;
}

}  // namespace

extern "C" {

int fa_fwd_block_noalloc(const fa_fwd_args* args) {
  if (!args) return fail(FA_ERR_INVALID_ARGUMENT, "args is NULL");
  if (args->struct_bytes != sizeof(fa_fwd_args))
    return fail(FA_ERR_INVALID_ARGUMENT, "struct_bytes is %u, this library expects %zu (ABI mismatch)", args->struct_bytes,
                sizeof(fa_fwd_args));
  if (!args->blockmask) return fail(FA_ERR_INVALID_ARGUMENT, "fa_fwd_block_noalloc needs a blockmask");
  if (args->max_seqlen_q <= 0 || args->max_seqlen_k <= 0) return fail(FA_ERR_INVALID_ARGUMENT, "max_seqlen must be positive");
  const size_t need = sparse_layout(round_seqlens(args->head_dim, args->max_seqlen_q, args->max_seqlen_k, true)).bytes;
  if (need > kNoAllocScratchBytes)
    return fail(FA_ERR_WORKSPACE,
                "fa_fwd_block_noalloc: this block layout needs %zu bytes of activity maps, the built-in scratch holds %zu "
                "(use fa_fwd_block with caller scratch)", need, kNoAllocScratchBytes);
  void* ptr = nullptr;
  const int rc = noalloc_scratch(&ptr);
  if (rc) return rc;
  fa_fwd_args a = *args;
  a.workspace = ptr;  // the device address, never the symbol
  a.workspace_bytes = kNoAllocScratchBytes;
  return fwd_impl(&a, true);
}

int fa_fwd(const fa_fwd_args* args) { return fwd_impl(args, false); }
int fa_fwd_block(const fa_fwd_args* args) { return fwd_impl(args, true); }
int fa_bwd(const fa_bwd_args* args) { return bwd_impl(args, false); }
int fa_bwd_profiled(const fa_bwd_args* args, void* ev_main_start, void* ev_main_stop) {
  return bwd_impl(args, false, ev_main_start, ev_main_stop);
}
int fa_bwd_block(const fa_bwd_args* args) { return bwd_impl(args, true); }

size_t fa_fwd_workspace_bytes(const fa_fwd_args* a) {
  if (!a) return 0;
  if (a->blockmask) return sparse_layout(round_seqlens(a->head_dim, a->max_seqlen_q, a->max_seqlen_k, true)).bytes;
  const Rounded r = round_seqlens(a->head_dim, a->max_seqlen_q, a->max_seqlen_k, false);
  return split_plan(a->batch, a->nheads, a->head_dim, a->total_q, a->max_seqlen_q, a->max_seqlen_k, r.sq_r,
                    a->is_causal != 0, false).bytes;
}

size_t fa_bwd_workspace_bytes(const fa_bwd_args* a) {
  if (!a) return 0;
  if (a->blockmask) return sparse_layout(round_seqlens(a->head_dim, a->max_seqlen_q, a->max_seqlen_k, true)).bytes;
  // optional: the fp32 dQ and counters of the one-kernel backward, or the partial dQ of the key-split dQ kernel (same plan as
  // the forward's; o_bytes is n_splits fp32 copies of dq)
  const size_t fused = fused_bwd_bytes(a);
  if (fused > 0) return fused;
  const Rounded r = round_seqlens(a->head_dim, a->max_seqlen_q, a->max_seqlen_k, false);
  return split_plan(a->batch, a->nheads, a->head_dim, a->total_q, a->max_seqlen_q, a->max_seqlen_k, r.sq_r,
                    a->is_causal != 0, false).o_bytes;
}

size_t fa_keep_words_bytes(int32_t batch, int32_t nheads, int32_t max_seqlen_q, int32_t max_seqlen_k) {
  if (batch <= 0 || nheads <= 0 || max_seqlen_q <= 0 || max_seqlen_k <= 0) return 0;
  return (size_t)batch * nheads * fa::keep_words_key_blocks(max_seqlen_k) * fa::keep_words_q_extent(max_seqlen_q) * 4;
}

void fa_round_seqlens(int32_t head_dim, int32_t max_seqlen_q, int32_t max_seqlen_k, int32_t blocksparse,
                      int32_t* max_seqlen_q_rounded, int32_t* max_seqlen_k_rounded) {
  const Rounded r = round_seqlens(head_dim, max_seqlen_q, max_seqlen_k, blocksparse != 0);
  if (max_seqlen_q_rounded) *max_seqlen_q_rounded = r.sq_r;
  if (max_seqlen_k_rounded) *max_seqlen_k_rounded = r.sk_r;
}

uint64_t fa_philox_offset_increment(void) { return 4; }

namespace {
// widest chunk (bytes, power of two <= 16) that divides the row width and every address involved
int row_vector_bytes(const void* a, const void* b, int64_t row_bytes, int64_t sa, int64_t sb) {
  uint64_t m = (uint64_t)reinterpret_cast<uintptr_t>(a) | (uint64_t)reinterpret_cast<uintptr_t>(b) | (uint64_t)row_bytes |
               (uint64_t)sa | (uint64_t)sb | 16u;
  return (int)(m & (~m + 1));  // lowest set bit
}
}  // namespace

int fa_gather_rows(const void* src, void* dst, const int64_t* indices, int64_t n_indices, int64_t n_src_rows,
                   int64_t row_bytes, int64_t src_row_stride, int64_t dst_row_stride, void* stream) {
  FA_REQUIRE(n_indices >= 0 && n_src_rows >= 0 && row_bytes >= 0, "fa_gather_rows: negative size");
  FA_REQUIRE(src_row_stride >= row_bytes && dst_row_stride >= row_bytes, "fa_gather_rows: row stride smaller than row");
  if (n_indices == 0 || row_bytes == 0) return FA_OK;
  FA_REQUIRE(src && dst && indices, "fa_gather_rows: null pointer");
  const int vec = row_vector_bytes(src, dst, row_bytes, src_row_stride, dst_row_stride);
  FA_LAUNCH(fa::launch_gather_rows(src, dst, indices, n_indices, n_src_rows, row_bytes, src_row_stride, dst_row_stride, vec,
                                   reinterpret_cast<hipStream_t>(stream)));
  return FA_OK;
}

size_t fa_scatter_rows_workspace_bytes(int64_t n_dst_rows) { return n_dst_rows > 0 ? (size_t)n_dst_rows * 4 : 0; }

int fa_scatter_rows(const void* src, void* dst, const int64_t* indices, int64_t n_indices, int64_t n_dst_rows,
                    int64_t row_bytes, int64_t src_row_stride, int64_t dst_row_stride, void* workspace,
                    size_t workspace_bytes, void* stream) {
  FA_REQUIRE(n_indices >= 0 && n_dst_rows >= 0 && row_bytes >= 0, "fa_scatter_rows: negative size");
  FA_REQUIRE(n_dst_rows < ((int64_t)1 << 31) && n_indices < ((int64_t)1 << 31), "fa_scatter_rows: more than 2^31 rows");
  FA_REQUIRE(src_row_stride >= row_bytes && dst_row_stride >= row_bytes, "fa_scatter_rows: row stride smaller than row");
  if (n_dst_rows == 0 || row_bytes == 0) return FA_OK;
  FA_REQUIRE(dst && (n_indices == 0 || (src && indices)), "fa_scatter_rows: null pointer");
  if (!workspace || workspace_bytes < fa_scatter_rows_workspace_bytes(n_dst_rows) ||
      (reinterpret_cast<uintptr_t>(workspace) & 3))
    return fail(FA_ERR_WORKSPACE, "fa_scatter_rows: needs %zu bytes of 4-byte aligned workspace",
                fa_scatter_rows_workspace_bytes(n_dst_rows));
  const int vec = row_vector_bytes(n_indices ? src : dst, dst, row_bytes, src_row_stride, dst_row_stride);
  FA_LAUNCH(fa::launch_scatter_rows(src, dst, indices, n_indices, n_dst_rows, row_bytes, src_row_stride, dst_row_stride,
                                    vec, reinterpret_cast<int32_t*>(workspace), reinterpret_cast<hipStream_t>(stream)));
  return FA_OK;
}

int fa_bias_grad_reduce(const void* dbias, void* out, int32_t dtype, int32_t batch, int32_t heads, int32_t rows,
                        int32_t cols, int64_t dbias_batch_stride, int64_t dbias_head_stride, int64_t dbias_row_stride,
                        int32_t sum_batch, int32_t sum_heads, int64_t out_batch_stride, int64_t out_head_stride,
                        int64_t out_row_stride, void* stream) {
  FA_REQUIRE(dtype == 0 || dtype == 1, "fa_bias_grad_reduce: dtype must be 0 (fp16) or 1 (bf16)");
  FA_REQUIRE(batch >= 0 && heads >= 0 && rows >= 0 && cols >= 0, "fa_bias_grad_reduce: negative size");
  FA_REQUIRE(batch <= 65535 && heads <= 65535, "fa_bias_grad_reduce: more than 65535 batch entries or heads");
  if (batch == 0 || heads == 0 || rows == 0 || cols == 0) return FA_OK;
  FA_REQUIRE(dbias && out, "fa_bias_grad_reduce: null pointer");
  const int64_t cols8 = ((int64_t)cols + 7) / 8 * 8;
  FA_REQUIRE((reinterpret_cast<uintptr_t>(dbias) & 15) == 0 && dbias_batch_stride % 8 == 0 && dbias_head_stride % 8 == 0 &&
                 dbias_row_stride % 8 == 0 && dbias_row_stride >= cols8,
             "fa_bias_grad_reduce: dbias must be 16-byte aligned, its strides multiples of 8 and its rows padded to a "
             "multiple of 8 columns");
  FA_REQUIRE(out_row_stride >= cols, "fa_bias_grad_reduce: out row stride smaller than a row");
  const bool vec_store = (reinterpret_cast<uintptr_t>(out) & 15) == 0 && out_batch_stride % 8 == 0 &&
                         out_head_stride % 8 == 0 && out_row_stride % 8 == 0;
  FA_LAUNCH(fa::launch_bias_grad_reduce(dbias, out, dtype, batch, heads, rows, cols, dbias_batch_stride, dbias_head_stride,
                                        dbias_row_stride, sum_batch != 0, sum_heads != 0, out_batch_stride, out_head_stride,
                                        out_row_stride, vec_store, reinterpret_cast<hipStream_t>(stream)));
  return FA_OK;
}

int fa_rotary(const fa_rotary_args* a) {
  FA_REQUIRE(a && a->struct_bytes == sizeof(fa_rotary_args), "fa_rotary: struct size mismatch");
  FA_REQUIRE(a->dtype == FA_FP16 || a->dtype == FA_BF16, "fa_rotary: dtype must be fp16 or bf16");
  FA_REQUIRE(a->n_rows >= 0 && a->n_parts >= 1 && a->n_rotated >= 0 && a->n_rotated <= a->n_parts && a->n_heads >= 1,
             "fa_rotary: bad sizes");
  FA_REQUIRE(a->head_dim >= 8 && a->head_dim % 8 == 0, "fa_rotary: head_dim must be a multiple of 8");
  if (a->n_rows == 0) return FA_OK;
  FA_REQUIRE(a->src && a->dst && a->cos_table && a->sin_table, "fa_rotary: null pointer");
  FA_REQUIRE(a->table_rows >= 1 && (a->positions || a->seqlen >= 1), "fa_rotary: empty table or no positions");
  FA_REQUIRE(a->positions || a->seqlen <= a->table_rows, "fa_rotary: the tables have %d rows, the sequence %d positions",
             a->table_rows, a->seqlen);
  FA_REQUIRE(aligned16(a->src) && aligned16(a->dst) && (reinterpret_cast<uintptr_t>(a->cos_table) & 7) == 0 &&
                 (reinterpret_cast<uintptr_t>(a->sin_table) & 7) == 0,
             "fa_rotary: pointers must be 16-byte (tensors) / 8-byte (tables) aligned");
  FA_REQUIRE(stride_ok(a->src_row_stride) && stride_ok(a->src_part_stride) && stride_ok(a->src_head_stride) &&
                 stride_ok(a->dst_row_stride) && stride_ok(a->dst_part_stride) && stride_ok(a->dst_head_stride),
             "fa_rotary: strides must be multiples of 8 elements");
  fa::RotaryParams p;
  p.src = a->src; p.dst = a->dst; p.cos = a->cos_table; p.sin = a->sin_table; p.positions = a->positions;
  p.n_rows = a->n_rows;
  p.src_row_stride = a->src_row_stride; p.src_part_stride = a->src_part_stride; p.src_head_stride = a->src_head_stride;
  p.dst_row_stride = a->dst_row_stride; p.dst_part_stride = a->dst_part_stride; p.dst_head_stride = a->dst_head_stride;
  p.n_parts = a->n_parts; p.n_rotated = a->n_rotated; p.n_heads = a->n_heads; p.head_dim = a->head_dim;
  p.seqlen = a->seqlen; p.table_rows = a->table_rows; p.conjugate = a->conjugate;
  p.row_offset = 0;
  FA_LAUNCH(fa::launch_rotary(p, a->dtype, reinterpret_cast<hipStream_t>(a->stream)));
  return FA_OK;
}

int fa_set_launch_policy(int policy) {
  FA_REQUIRE((policy & ~0x73) == 0 && (policy & 3) != 3 && (policy & 0x30) != 0x30,
             "launch policy: tile shape 0 (automatic), 1 (full-size) or 2 (half-size), plus 0x10 (two-kernel backward) or 0x20 "
             "(one-kernel backward where it exists), plus 0x40 (head dim 128: dK/dV kernel of wave pairs where it exists)");
  g_launch_policy.store(policy, std::memory_order_relaxed);
  return FA_OK;
}

const char* fa_last_error(void) { return g_err; }
int fa_abi_version(void) { return FA_ABI_VERSION; }

}  // extern "C"
