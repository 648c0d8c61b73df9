/*
 * flash_attn_gfx950.h -- C ABI of the MI355X (gfx950) FlashAttention engine.
 *
 * This shared library replaces the reference's pybind11 module `flash_attn_cuda`
 * (csrc/flash_attn/fmha_api.cpp:721-727).  Each entry point below is what a binding for one of
 * that module's four functions calls.  Differences from the reference boundary, by design:
 *   - plain pointers, sizes and strides only (no ATen types);
 *   - every buffer is owned by the caller, including outputs and scratch (`workspace`);
 *   - the Philox (seed, offset) pair is passed in instead of being drawn from a generator;
 *   - errors are returned as negative codes with a message in fa_last_error(); nothing here
 *     exits the process (the reference's FMHA_CHECK_CUDA does, fmha_utils.h:39-50);
 *   - work is enqueued on `stream` and never synchronised.
 *
 * Tensor conventions (as fmha_api.cpp:173-186): q is [total_q, nheads, head_dim], k and v are
 * [total_k, nheads, head_dim], element type fp16 or bf16, innermost stride 1, row and head strides
 * given in ELEMENTS (a packed qkv[total,3,H,d] view has row stride 3*H*d).  cu_seqlens_* are int32
 * [batch+1] device arrays of cumulative sequence lengths.
 */
#ifndef FLASH_ATTN_GFX950_H_
#define FLASH_ATTN_GFX950_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FA_ABI_VERSION 5

enum fa_dtype { FA_FP16 = 0, FA_BF16 = 1 };

enum fa_status {
  FA_OK = 0,
  FA_ERR_INVALID_ARGUMENT = -1, /* a TORCH_CHECK of fmha_api.cpp would have thrown */
  FA_ERR_WORKSPACE = -2,        /* workspace missing or smaller than fa_*_workspace_bytes() */
  FA_ERR_LAUNCH = -3,           /* HIP reported a launch error */
  FA_ERR_UNSUPPORTED = -4
};

/* Arguments of the forward pass.  Mirrors mha_fwd (fmha_api.cpp:173-186) and, when `blockmask`
 * is non-NULL, mha_fwd_block (fmha_api.cpp:451-464). */
typedef struct fa_fwd_args {
  uint32_t struct_bytes; /* sizeof(fa_fwd_args), checked */
  int32_t dtype;         /* enum fa_dtype */
  const void* q;
  const void* k;
  const void* v;
  void* o;            /* [total_q, nheads, head_dim], same dtype; written for rows < seqlen_q */
  float* softmax_lse; /* [batch, nheads, max_seqlen_q_rounded] fp32 */
  void* s_dmask;      /* NULL, or [batch, nheads, max_seqlen_q_rounded, max_seqlen_k_rounded] in `dtype`:
                         row-major softmax probabilities, negative sign = dropped (return_softmax) */
  const int32_t* cu_seqlens_q;
  const int32_t* cu_seqlens_k;
  const int32_t* blockmask; /* NULL = dense.  Else the converted block list of
                               flash_blocksparse_attn_interface.py:8-40: int32
                               [max_seqlen_k_rounded/256, max_seqlen_q_rounded/16] */
  int64_t q_row_stride, q_head_stride;
  int64_t k_row_stride, k_head_stride;
  int64_t v_row_stride, v_head_stride;
  int64_t o_row_stride, o_head_stride; /* both >= head_dim: written rows and heads may not overlap */
  int32_t batch, nheads, head_dim;
  int32_t total_q, total_k;
  int32_t max_seqlen_q, max_seqlen_k; /* as given by the caller, before rounding */
  float p_dropout;                    /* probability of DROPPING, in [0,1) (fmha_api.cpp:113) */
  float softmax_scale;
  int32_t zero_tensors; /* pre-fill o=0, lse=-inf, s_dmask=0 (fmha_api.cpp:256-260) */
  int32_t is_causal;
  uint64_t philox_seed, philox_offset;
  void* workspace; /* device scratch of >= fa_fwd_workspace_bytes() bytes (may be NULL if that is 0) */
  size_t workspace_bytes;
  void* stream; /* hipStream_t */
  /* Attention bias (no counterpart in the reference's entry points; its README lists "attention bias (e.g. ALiBi)" as
   * planned, README.md:49-50).  NULL, or a device array of nheads fp32 slopes: softmax_scale * q.k - slope[h] * |i - j|
   * is what the softmax sees, i and j being the positions of query and key in their sequences.  With a blockmask: inside
   * the active blocks. */
  const float* alibi_slopes;
  /* Dropout keep words (no counterpart in the reference, whose backward kernels draw every keep decision again,
   * fmha_dgrad_kernel_1xN_loop.h:337).  NULL, or 16-byte aligned device memory of keep_words_bytes >=
   * fa_keep_words_bytes() bytes: with p_dropout > 0 and no blockmask the forward then also leaves the keep decision of
   * every score there, one bit each, for fa_bwd (fa_bwd_args.keep_words).  o, softmax_lse and s_dmask are what they are
   * without it.  Ignored with p_dropout == 0 or a blockmask. */
  void* keep_words;
  size_t keep_words_bytes;
  /* Attention bias as a tensor (same origin as alibi_slopes: the reference plans it, README.md:50, "relative positional
   * encoding").  NULL, or a device tensor of `dtype` indexed [batch, head, query, key] with the strides below in elements
   * (keys contiguous; batch and head stride may be 0: one bias for all of them): softmax_scale * q.k + bias[b, h, i, j] is
   * what the softmax sees, i < max_seqlen_q and j < max_seqlen_k being positions inside the sequences.  -inf entries mask.
   * 16-byte aligned, bias_row_stride a multiple of 8 and >= max_seqlen_k; every row is read in 16-byte pieces, i.e. up to the
   * next multiple of 8 keys past max_seqlen_k (inside the row stride).  Not with alibi_slopes.  With a blockmask: read inside
   * the active blocks only. */
  const void* attn_bias;
  int64_t bias_batch_stride, bias_head_stride, bias_row_stride;
  /* Block-sparse only (no counterpart in the reference).  NULL, or a device array of max_seqlen_q_rounded / 16 int32: a
   * permutation of the 16-row blocks.  A workgroup of the forward and of the backward's dQ kernel owns eight consecutive
   * entries of it (without it: eight consecutive row blocks) and has to stage every key tile that any of the eight lists;
   * an order that puts row blocks with similar key-block lists next to each other saves that staging (at 25 % of
   * independently drawn blocks about a third of it).  Results do not depend on the order beyond rounding.  The entries
   * must be distinct row blocks (a row block that is not listed is not computed: its rows of o / dq are left unwritten);
   * ignored with is_causal. */
  const int32_t* row_order;
  /* Rotary position embedding inside the kernels (replaces the elementwise passes of the reference's FlashMHA,
   * flash_attention.py:109-113 with rotary.py:90-99, which read and write q and k once more in each direction).  NULL, or
   * the interleaved-pair cos / sin tables of fa_rotary ([rotary_table_rows, head_dim / 2] of `dtype`, contiguous, 16-byte
   * aligned, rotary_table_rows >= max_seqlen_q): the query at position i of its sequence is turned by table row i as
   * it is loaded, with fa_rotary's arithmetic, so o and softmax_lse are bit for bit those of fa_rotary followed by
   * fa_fwd.  k is NOT turned here - key tiles never pass through registers - the caller gives the rotated keys (fa_rotary
   * over the k part only: a third of the bytes of rotating q and k).  q_rot: NULL, or a [total_q, nheads, head_dim] tensor
   * (strides below, 16-byte aligned like q) that receives the rotated queries, which fa_bwd wants.  Not with
   * return-softmax (s_dmask), whose pass reads q itself; not with a blockmask, alibi_slopes or attn_bias. */
  const void* rotary_cos;
  const void* rotary_sin;
  int32_t rotary_table_rows;
  int32_t reserved0; /* 0 */
  void* q_rot;
  int64_t q_rot_row_stride, q_rot_head_stride;
} fa_fwd_args;

/* Arguments of the backward pass.  Mirrors mha_bwd (fmha_api.cpp:302-321) and, when `blockmask`
 * is non-NULL, mha_bwd_block (fmha_api.cpp:575-594).  dq, dk, dv are caller-allocated, possibly
 * strided views written in place. */
typedef struct fa_bwd_args {
  uint32_t struct_bytes;
  int32_t dtype;
  const void* dout; /* [total_q, nheads, head_dim] */
  const void* q;
  const void* k;
  const void* v;
  const void* out;
  const float* softmax_lse; /* [batch, nheads, lse_seq_stride] as written by the forward */
  void* dq;
  void* dk;
  void* dv;
  float* softmax_d; /* [batch, nheads, max_seqlen_q_rounded] fp32: (1 - p_dropout) * rowsum(dout * out), the reference's
                       dp_sum * p_dropout (fmha_dgrad_kernel_1xN_loop.h:15-30,226) */
  const int32_t* cu_seqlens_q;
  const int32_t* cu_seqlens_k;
  const int32_t* blockmask;
  int64_t do_row_stride, do_head_stride;
  int64_t q_row_stride, q_head_stride;
  int64_t k_row_stride, k_head_stride;
  int64_t v_row_stride, v_head_stride;
  int64_t o_row_stride, o_head_stride;
  int64_t dq_row_stride, dq_head_stride;
  int64_t dk_row_stride, dk_head_stride;
  int64_t dv_row_stride, dv_head_stride;
  int32_t lse_seq_stride; /* innermost extent of softmax_lse (the forward's max_seqlen_q_rounded) */
  int32_t batch, nheads, head_dim;
  int32_t total_q, total_k;
  int32_t max_seqlen_q, max_seqlen_k;
  float p_dropout;
  float softmax_scale;
  int32_t zero_tensors; /* pre-fill dq=dk=dv=0, softmax_d=0 (fmha_api.cpp:406-411) */
  int32_t is_causal;
  uint64_t philox_seed, philox_offset; /* the pair the forward was given */
  void* workspace;
  size_t workspace_bytes;
  void* stream;
  const float* alibi_slopes; /* as in fa_fwd_args: the slopes the forward was given */
  /* NULL, or the keep words the forward of this very call (same shapes, cu_seqlens, p_dropout, seed and offset) left in
   * fa_fwd_args.keep_words: with p_dropout > 0 and no blockmask neither backward kernel then runs Philox, they read the
   * decisions (the dropout variants of these kernels spend more than half of their vector instructions drawing them).
   * dq, dk, dv are bit for bit what they are without it.  Ignored with p_dropout == 0 or a blockmask. */
  const void* keep_words;
  size_t keep_words_bytes;
  /* as in fa_fwd_args: the bias the forward was given */
  const void* attn_bias;
  int64_t bias_batch_stride, bias_head_stride, bias_row_stride;
  /* NULL, or where to leave d(loss)/d(attn_bias): a tensor of `dtype` indexed [batch, head, query, key] with the strides
   * below (every (batch, head) has its own slice: row stride >= max_seqlen_k, head stride >= max_seqlen_q rows, batch
   * stride >= nheads head strides; sum over the slices for a shared bias), 2-byte aligned.  Only the (query, key) tiles the backward visits are written (under a causal mask none above the diagonal,
   * none past a sequence's end): the caller clears the tensor first. */
  void* dbias;
  int64_t dbias_batch_stride, dbias_head_stride, dbias_row_stride;
  /* as in fa_fwd_args (the backward need not be given the order the forward had) */
  const int32_t* row_order;
  /* Rotary position embedding inside the kernels.  NULL, or the tables the forward was given (rotary_table_rows >=
   * max(max_seqlen_q, max_seqlen_k)): q and k are then the ROTATED tensors (fa_fwd_args.q_rot and the k the forward
   * read), and dq and dk come out as gradients with respect to the unrotated ones - turned back by the opposite angles in
   * fp32 before their one rounding - so no elementwise pass over them follows. */
  const void* rotary_cos;
  const void* rotary_sin;
  int32_t rotary_table_rows;
  int32_t reserved0; /* 0 */
} fa_bwd_args;

/* replaces flash_attn_cuda.fwd -> mha_fwd, csrc/flash_attn/fmha_api.cpp:173-299 */
int fa_fwd(const fa_fwd_args* args);
/* replaces flash_attn_cuda.bwd -> mha_bwd, csrc/flash_attn/fmha_api.cpp:302-449 */
int fa_bwd(const fa_bwd_args* args);
/* replaces flash_attn_cuda.fwd_block -> mha_fwd_block, csrc/flash_attn/fmha_api.cpp:451-573
 * (args->blockmask must be non-NULL).  is_causal may be set together with a blockmask, here and in fa_bwd_block: a score
 * counts iff its block is listed AND key <= query; blocks that lie wholly above the diagonal may be listed or not.  The
 * reference's kernels take the flag too, but its Python refuses it (flash_blocksparse_attn_interface.py:21). */
int fa_fwd_block(const fa_fwd_args* args);
/* replaces flash_attn_cuda.bwd_block -> mha_bwd_block, csrc/flash_attn/fmha_api.cpp:575-718 */
int fa_bwd_block(const fa_bwd_args* args);

/* No counterpart in the reference.  fa_fwd_block for callers that cannot allocate device memory or carry scratch
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): the block activity maps that
 * fa_fwd_block keeps in `workspace` live in a device array inside the library instead (FA_NOALLOC_SCRATCH_BYTES, held by
 * every GPU the library runs on until the process ends).  args->workspace / workspace_bytes are ignored; inputs and
 * outputs are the caller's as usual.  Layouts whose maps need more (fa_fwd_workspace_bytes() > FA_NOALLOC_SCRATCH_BYTES;
 * the limit is reached between 16384 and 32768 tokens) are refused with FA_ERR_WORKSPACE.  The call allocates nothing
 * and the maps are rebuilt by every call, but all calls on one GPU share the one array: calls that overlap on a GPU
 * (different streams or host threads) race; serialise them.  The first call on a device looks up the array's device
 * address, which is not meant to happen under stream capture: make one eager call per device before capturing.  The
 * current device must be the device of args->stream.  Results are those of fa_fwd_block. */
#define FA_NOALLOC_SCRATCH_BYTES (64u * 1024u)
int fa_fwd_block_noalloc(const fa_fwd_args* args);

/* Scratch the caller provides.  The dense forward and backward need none to be correct
 * (there is no o_tmp / dq_tmp, fmha_api.cpp:247,403-404).  The block-sparse paths need room for their block activity
 * maps (an error without it).  For a dense, non-causal forward with few query rows and many keys (max_seqlen_q <= 128,
 * batch * nheads < 128, max_seqlen_k >= 512: decoding and cross-attention shapes) fa_fwd_workspace_bytes() returns the size of the
 * partial results of a key-split pass: if `workspace` holds that much, fa_fwd shares the keys of each query tile
 * among several workgroups and merges their results; if not, it runs the single pass.  fa_bwd_workspace_bytes() does the
 * same for the dQ kernel of such shapes (fp32 partial dQ per key split), and, under launch policy 0x20, returns the
 * scratch of the one-kernel backward (fp32 running sums of dQ and their hand-over counters: about twice the bytes of dq).
 * Only shapes, is_causal, p_dropout, the bias pointers and blockmask != NULL are read. */
size_t fa_fwd_workspace_bytes(const fa_fwd_args* args);
size_t fa_bwd_workspace_bytes(const fa_bwd_args* args);
/* Size of fa_fwd_args.keep_words / fa_bwd_args.keep_words: one bit per (batch, head, query, key) with both sequence
 * lengths rounded up to 128. */
size_t fa_keep_words_bytes(int32_t batch, int32_t nheads, int32_t max_seqlen_q, int32_t max_seqlen_k);

/* Seqlen rounding used for the shapes of softmax_lse / s_dmask / softmax_d / blockmask
 * (fmha_api.cpp:232-241 dense, :509-514 block-sparse).  Writes the rounded values. */
void fa_round_seqlens(int32_t head_dim, int32_t max_seqlen_q, int32_t max_seqlen_k, int32_t blocksparse,
                      int32_t* max_seqlen_q_rounded, int32_t* max_seqlen_k_rounded);

/* Number of 64-bit Philox offsets one forward call consumes; the caller advances its generator
 * by this much (the role of launch_params.elts_per_thread, fmha_api.cpp:282-292). */
uint64_t fa_philox_offset_increment(void);

/* Row gather / scatter: the device side of unpad_input / pad_input (flash_attn/bert_padding.py:9-95, where they
 * are torch.gather and index assignment inside IndexFirstAxis / IndexPutFirstAxis).  Rows are `row_bytes` wide,
 * `*_row_stride` bytes apart; `indices` is a device array of int64 (what torch.nonzero returns).
 *
 * fa_gather_rows:  dst[i, :] = src[indices[i], :]  for i < n_indices      (IndexFirstAxis.forward :12-19,
 *                  IndexPutFirstAxis.backward :51-57).  An index outside [0, n_src_rows) gives a zero row.
 * fa_scatter_rows: dst[indices[i], :] = src[i, :], every other row of dst[0 .. n_dst_rows) = 0
 *                  (IndexPutFirstAxis.forward :38-48, IndexFirstAxis.backward :21-30).  dst is written exactly once
 *                  and needs no prior zero fill; indices must be unique (duplicates: one of the rows wins); indices
 *                  outside [0, n_dst_rows) are ignored.  `workspace`: fa_scatter_rows_workspace_bytes(n_dst_rows)
 *                  bytes of device scratch (the inverse index; its contents on entry do not matter). */
int fa_gather_rows(const void* src, void* dst, const int64_t* indices, int64_t n_indices, int64_t n_src_rows,
                   int64_t row_bytes, int64_t src_row_stride, int64_t dst_row_stride, void* stream);
int fa_scatter_rows(const void* src, void* dst, const int64_t* indices, int64_t n_indices, int64_t n_dst_rows,
                    int64_t row_bytes, int64_t src_row_stride, int64_t dst_row_stride, void* workspace,
                    size_t workspace_bytes, void* stream);
size_t fa_scatter_rows_workspace_bytes(int64_t n_dst_rows);

/* Sum of the bias gradient over the batch entries and / or heads that shared one bias (no counterpart in the
 * reference, which takes no bias).  fa_bwd writes `dbias` per (batch, head); a bias of batch or head extent 1 that
 * was broadcast wants the sum.  dbias: [batch, heads, rows, >= cols rounded up to 8] in `dtype` (strides in elements,
 * multiples of 8, base 16-byte aligned: the rows are read as whole 16-byte chunks).  out: [sum_batch ? 1 : batch,
 * sum_heads ? 1 : heads, rows, cols] in the same dtype, any strides with innermost stride 1.  One pass; the slices are
 * added in fp32 in a fixed order (batch outer, head inner) and rounded once, so the result is reproducible bit for
 * bit. */
int fa_bias_grad_reduce(const void* dbias, void* out, int32_t dtype, int32_t batch, int32_t heads, int32_t rows,
                        int32_t cols, int64_t dbias_batch_stride, int64_t dbias_head_stride, int64_t dbias_row_stride,
                        int32_t sum_batch, int32_t sum_heads, int64_t out_batch_stride, int64_t out_head_stride,
                        int64_t out_row_stride, void* stream);

/* Rotary position embedding of the query and key parts of a packed tensor in one pass: what
 * RotaryEmbedding.forward / apply_rotary_pos_emb compute with elementwise torch ops (flash_attn/rotary.py:22-42,
 * 89-100; FlashMHA applies it to q and k before attention, flash_attention.py:109-113).
 * src / dst: [n_rows, n_parts, n_heads, head_dim] views (strides in elements, innermost stride 1; dst may equal
 * src).  Parts 0 .. n_rotated-1 are rotated, the remaining parts are copied (packed qkv: n_parts 3, n_rotated 2).
 * Pair (x[2i], x[2i+1]) of a row at position t becomes (x[2i] c - x[2i+1] s, x[2i+1] c + x[2i] s) with
 * c = cos_table[t, i], s = sin_table[t, i]; tables are [table_rows, head_dim / 2] in the tensor's dtype;
 * t = positions[row] if positions != NULL (entries outside [0, table_rows) are clamped to the nearest table row: callers
 * that cannot vouch for them check positions themselves), else row % seqlen (seqlen <= table_rows is required).
 * conjugate != 0 negates s (the backward pass).
 * head_dim must be a multiple of 8; base pointers and strides must keep 16-byte alignment. */
typedef struct fa_rotary_args {
  uint32_t struct_bytes;
  int32_t dtype;
  const void* src;
  void* dst;
  const void* cos_table;
  const void* sin_table;
  const int32_t* positions;
  int64_t n_rows;
  int64_t src_row_stride, src_part_stride, src_head_stride;
  int64_t dst_row_stride, dst_part_stride, dst_head_stride;
  int32_t n_parts, n_rotated, n_heads, head_dim;
  int32_t seqlen, table_rows, conjugate;
  void* stream;
} fa_rotary_args;
int fa_rotary(const fa_rotary_args* args);

/* Host-side helper of the block-sparse entry points (no GPU work, no counterpart in the reference): an order of the 16-row
 * blocks for fa_fwd_args.row_order / fa_bwd_args.row_order that puts row blocks with similar key-block lists into the same
 * workgroup (eight consecutive entries) and wave (two).  layout: HOST array [n_row_blocks][n_col_blocks] of bytes, non-zero
 * = the 16 x 256 block is listed (the layout before convert_blockmask); order: HOST array of n_row_blocks int32, written:
 * a permutation of 0 .. n_row_blocks - 1, the identity if reordering would save less than 5 % of the staged key blocks.
 * Deterministic; a greedy grouping followed by 2000 * n_row_blocks exchange attempts, four million at most (tens of
 * milliseconds for 4096 tokens, about a second for 65536). */
int fa_blocksparse_row_order(const uint8_t* layout, int32_t n_row_blocks, int32_t n_col_blocks, int32_t* order);

/* Launch policy (process-wide state; no counterpart in the reference, whose launchers pick their tile by head size
 * and sequence length alone, fmha_api.cpp:232-241).  policy = tile shape | backward plan.
 * Tile shape (bits 0-1): 0 (default): short-sequence launches that would leave compute units idle with the full-size
 * tiles (128 query rows / 128 keys per workgroup) use the half-size variants where they exist (head_dim <= 64, no
 * blockmask, no alibi_slopes); 1: always full-size; 2: always half-size where they exist.
 * Backward plan (bits 4-5): 0 (default): two kernels (dQ with softmax_d, then dK/dV), no scratch - as two launches, or, for
 * short launches at head_dim 64 (where the dQ kernel takes its half-size tiles), as one launch that holds both kinds of
 * workgroup, with bit-identical results; 0x10: always two launches; 0x20: one kernel
 * that also passes dQ from key tile to key tile through fp32 scratch, where it exists (head_dim 64, no blockmask, mask,
 * dropout or bias, max_seqlen_k <= 4096) and only if the caller brings the scratch fa_bwd_workspace_bytes() then asks for.
 * Bit 6 (0x40): at head_dim 128 without dropout, blockmask or bias the dK/dV kernel runs as wave pairs (one wave holds K and
 * owns dV, its partner holds V and owns dK; 64 keys per workgroup) instead of four waves with 32 keys each and V in LDS.
 * The defaults are the faster choices on the shapes measured; the others are kept for parts and shapes where the balance differs.
 * Results agree within rounding between the choices (the order of fp32 summation differs), not bit for bit; each choice is
 * reproducible bit for bit from run to run. */
int fa_set_launch_policy(int policy);

/* Message for the last non-zero status returned on the calling thread. */
const char* fa_last_error(void);
int fa_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* FLASH_ATTN_GFX950_H_ */
