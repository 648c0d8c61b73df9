// Kernel parameter blocks (passed by value to the kernels) and launcher entry points shared
// between the C-ABI front end and the kernel translation units.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fa_common.h"

namespace fa {

// Block-sparse activity, built on the device from the reference's converted block list
// (flash_blocksparse_attn_interface.py:8-40) by launch_build_sparse_maps(): the 16-row x 256-key block (rb, cb) is
// computed iff its bit is set.  Bit sets (bit j of 64-bit word w <-> block 64 w + j), so that a kernel holds what it
// needs in a register pair and re-reads memory only every 64 blocks.
struct SparseMaps {
  const uint64_t* rbits;  // [nrb][ncw]: 16-row block -> its active 256-key column blocks
  const uint64_t* qbits;  // [nqt][ncw]: forward query tile -> column blocks active for any of its row blocks
  const uint64_t* cbits;  // [ncb][nrw]: column block -> its active 16-row blocks
  int nrb;   // 16-row blocks  (= max_seqlen_q_rounded / 16)
  int ncb;   // 256-key blocks (= max_seqlen_k_rounded / 256)
  int nqt;   // forward query tiles
  int ncw;   // 64-bit words per row of rbits / qbits
  int nrw;   // 64-bit words per row of cbits
  // Row order (or null = 0, 1, 2, ...): a permutation of the 16-row blocks.  The forward and the dQ kernel give query tile t
  // the row blocks order[8 t .. 8 t + 7] (qbits is built for those), so that a caller who lists row blocks with similar key
  // blocks next to each other makes a workgroup stage few tiles that only one of its row blocks needs.  Not used under a
  // causal mask (the tile ranges there follow the rows' positions).
  const int32_t* order;
};

// The two 16-row blocks of the 32-row slab `slab` (0 .. 3) of query tile qt: positions 8 qt + 2 slab and + 1 of the row
// order; -1 = none (past the last row block, or an entry that is not a row block).
FA_DEVICE void slab_row_blocks(const SparseMaps& sp, bool ordered, int qt, int slab, int* a, int* b) {
  const int pos = 8 * qt + 2 * slab;
  int ra = pos < sp.nrb ? pos : -1, rb = pos + 1 < sp.nrb ? pos + 1 : -1;
  if (ordered) {
    if (ra >= 0) ra = sp.order[pos];
    if (rb >= 0) rb = sp.order[pos + 1];
    if (ra >= sp.nrb) ra = -1;
    if (rb >= sp.nrb) rb = -1;
  }
  *a = __builtin_amdgcn_readfirstlane(ra);
  *b = __builtin_amdgcn_readfirstlane(rb);
}

// What is added to the scaled scores before the softmax (template parameter kBias of the kernels)
constexpr int kBiasNone = 0;    // nothing
constexpr int kBiasAlibi = 1;   // -slope[head] * |query - key| (alibi)
constexpr int kBiasTensor = 2;  // bias[b, h, query, key] (bias, strides in elements; batch and head stride may be 0)

struct FwdParams {
  const void* q;
  const void* k;
  const void* v;
  void* o;
  float* lse;
  const int32_t* cu_q;
  const int32_t* cu_k;
  int64_t q_rs, q_hs, k_rs, k_hs, v_rs, v_hs, o_rs, o_hs;  // strides in elements
  int B, H;
  int total_q, total_k;
  int max_sq, max_sk;  // caller's bounds on the sequence lengths; longer sequences are truncated to them
  int sq_r;  // rounded max_seqlen_q = innermost extent of lse
  int nq_tiles;
  int tile_group;    // causal launches: (batch, head) pairs of an XCD in flight together (map_tile); 0 = all
  float scale;       // softmax_scale
  float scale_log2;  // softmax_scale * log2(e)
  float rp_keep;     // 1 / keep probability
  uint32_t keep_thr; // floor(keep * 65535)
  PhiloxKey pk;
  SparseMaps sp;
  // Key-split forward (few query tiles, many keys): split s of n_splits handles a contiguous share of the key tiles
  // and writes its normalised fp32 output and its lse to o_part [n_splits, total_q, H, d] / lse_part
  // [n_splits, B, H, sq_r]; fwd_combine_kernel merges them into o / lse.  n_splits <= 1: single pass.
  int n_splits;
  float* o_part;
  float* lse_part;
  const float* alibi;  // null, or one slope per head: the score of (query i, key j) gets -slope * |i - j| added
  const void* bias;    // null, or a tensor of the element type added to the scaled scores: [b, h, query, key]
  int64_t bias_bs, bias_hs, bias_rs;  // its batch, head (0: shared) and row strides in elements; keys are contiguous
  // Rotary position embedding of the queries inside the kernel (null: none): cos / sin tables [rot_rows, head_dim / 2] of
  // the element type; the row at position i of its sequence is turned by table row i when its Q fragment is loaded (the
  // keys come in rotated: their tiles go to LDS without passing through registers).  q_rot: null, or where the rotated
  // queries are left for the backward ([total_q, H, d], strides in elements).
  const void* rot_cos;
  const void* rot_sin;
  int rot_rows;
  void* q_rot;
  int64_t qr_rs, qr_hs;
  // Dropout keep words (fa_common.h), or null: the keep decisions of every score, left for the backward
  uint32_t* keep_words;
  int kw_q;   // query extent of the buffer (max_seqlen_q rounded up to 128)
  int kw_kb;  // 32-key blocks (max_seqlen_k rounded up to 128, / 32)
};

struct DumpParams {  // return_softmax path
  const void* q;
  const void* k;
  const float* lse;
  void* s;  // [B, H, sq_r, sk_r]
  const int32_t* cu_q;
  const int32_t* cu_k;
  int64_t q_rs, q_hs, k_rs, k_hs;
  int B, H, D;
  int total_q, total_k;
  int max_sq, max_sk;
  int sq_r, sk_r;
  float scale;
  int causal, dropout, sparse;
  uint32_t keep_thr;
  PhiloxKey pk;
  SparseMaps sp;
  const float* alibi;
  const void* bias;  // as in FwdParams
  int64_t bias_bs, bias_hs, bias_rs;
};

struct BwdParams {
  const void* dout;
  const void* q;
  const void* k;
  const void* v;
  const void* out;
  const float* lse;
  float* dsoftmax;  // softmax_d [B, H, sq_r]
  void* dq;
  void* dk;
  void* dv;
  const int32_t* cu_q;
  const int32_t* cu_k;
  int64_t do_rs, do_hs, q_rs, q_hs, k_rs, k_hs, v_rs, v_hs, o_rs, o_hs;
  int64_t dq_rs, dq_hs, dk_rs, dk_hs, dv_rs, dv_hs;
  int B, H;
  int total_q, total_k;
  int max_sq, max_sk;
  int sq_r;        // innermost extent of dsoftmax
  int lse_stride;  // innermost extent of lse
  int nk_tiles;      // key tiles of the dK/dV kernel
  int merged_dkdv_blocks, merged_nq_tiles;  // fa_bwd_merged_kernel: its dK/dV workgroups come first; query tiles of the dQ part
  int nq_tiles;      // query tiles of the dQ kernel
  int tile_group;    // causal launches: (batch, head) pairs of an XCD in flight together (map_tile); 0 = all
  float scale;
  float scale_log2;
  float p_keep;
  float rp_keep;
  uint32_t keep_thr;
  PhiloxKey pk;
  SparseMaps sp;
  // Key-split dQ (one query tile, many keys; see FwdParams): split s of n_splits walks its share of the key tiles and
  // writes its scaled fp32 partial dQ to dq_part [n_splits, total_q, H, d]; dq_combine_kernel sums them into dq.
  int n_splits;
  float* dq_part;
  const float* alibi;  // as in FwdParams
  const void* bias;    // as in FwdParams
  int64_t bias_bs, bias_hs, bias_rs;
  void* dbias;         // null, or where the dK/dV kernel leaves d(loss)/d(bias) = dS / keep: [b, h, query, key], written for the
  int64_t dbias_bs, dbias_hs, dbias_rs;  // (query, key) tiles it visits (the caller clears the tensor)
  // Rotary position embedding (as in FwdParams; null: none): q and k are the rotated tensors, and dq and dk are turned back
  // by the opposite angles in the kernels' epilogues, before they are rounded
  const void* rot_cos;
  const void* rot_sin;
  int rot_rows;
  // Dropout keep words (fa_common.h) as the forward left them, or null: read by both kernels in place of Philox
  const uint32_t* keep_words;
  int kw_q;   // query extent of the buffer (max_seqlen_q rounded up to 128)
  int kw_kb;  // 32-key blocks (max_seqlen_k rounded up to 128, / 32)
  // One-kernel backward (fa_bwd_fused_kernel.h): fp32 running sums of dQ [B * H, nqt_ring tiles, 2048] and their hand-over
  // counters [B * H, nqt_ring, 4]
  float* dq_acc;
  int* dq_flags;
  int nqt_ring;     // query tiles of max_seqlen_q
  int ring_stride;  // tiles between the starting points of consecutive key tiles (0: the kernel's default)
};

// Sequence extent of batch entry b, clamped so that a cu_seqlens array that disagrees with the declared
// totals or maxima can never index outside the tensors: returns false if the entry must be skipped.
FA_DEVICE bool seq_extent(const int32_t* cu, int b, int total, int max_len, int* begin, int* len) {
  const int s = cu[b], e = cu[b + 1];
  int n = e - s;
  if (s < 0 || n <= 0 || e > total) return false;
  *begin = s;
  *len = n < max_len ? n : max_len;
  return true;
}

// Ragged batches: workgroup ids enumerate the batch entries longest first.  A launch deals its workgroups out in id order;
// the entries with the longest walks should be under way first and - in a grid that is resident all at once - spread over
// the compute units instead of arriving together as some units' third workgroup.  Slot `slot` of the launch's batch
// dimension therefore goes to the entry with the slot-th largest length in cu (ties: lower index first, so a batch of
// equal lengths keeps its order).  Every wave finds the entry itself: lane i holds entry i's length, counts the entries
// that precede it (one readlane and compare per entry), and the lane whose count is `slot` is the answer.  Batches of
// more than 64 entries keep their order.  The search costs every workgroup's prologue a few instructions per batch entry,
// so the launchers ask for it (tile_group < 0 in a launch without a mask) only for grids that are resident all at once
// (longest_first_launch), where the spreading is what it buys.
FA_DEVICE int longest_first(const int32_t* cu, int B, int slot) {
  if (B > 64 || B < 2) return slot;
  const int lane = threadIdx.x & 63;
  const int i = lane < B ? lane : B - 1;
  const int len = cu[i + 1] - cu[i];
  int before = 0;
  for (int j = 0; j < B; j++) {
    const int lj = __builtin_amdgcn_readlane(len, j);
    before += (lj > len || (lj == len && j < lane)) ? 1 : 0;
  }
  const uint64_t hit = __builtin_amdgcn_ballot_w64(lane < B && before == slot);
  return __builtin_amdgcn_readfirstlane(hit != 0 ? (int)__builtin_ctzll(hit) : slot);
}

// Workgroup id -> (batch*head, tile rank).  The hardware deals consecutive workgroup ids to the 8 XCDs in turn
// (id % 8), and each XCD has its own L2.
//   kTileMajor = false (tiles of equal cost): the tiles of one (batch, head) are consecutive in one XCD's share of the
//     ids, so they run on one XCD at about the same time and share its L2 copy of the streamed operand.
//   kTileMajor = true (causal: tile cost grows with the rank reversed): ids enumerate tile ranks outermost, so the
//     most expensive tiles of all (batch, head) pairs start first; batch*head is padded to a multiple of 8 so that a
//     given (batch, head) still always lands on the same XCD.
template <bool kTileMajor>
FA_DEVICE bool map_tile(int block, int tiles_per_bh, int BH, int* bh, int* rank, int group = 0) {
  if (kTileMajor) {
    const int bhp = (BH + 7) & ~7;
    const int P = bhp >> 3;  // (batch, head) pairs per XCD
    if (group > 0 && group < P) {
      // Long sequences: an XCD that streams the K and V of all its pairs at once reads them from memory again for every
      // query tile (they exceed its L2 many times over).  The pairs of an XCD are therefore taken `group` at a time -
      // ranks outermost inside a group, the groups one after the other - so that what is in flight shares a few pairs' keys.
      const int x = block & 7, j = block >> 3;
      const int g = j / (group * tiles_per_bh);
      const int r = j - g * group * tiles_per_bh;
      const int members = P - g * group < group ? P - g * group : group;
      *rank = r / members;
      *bh = x + 8 * (g * group + (r - *rank * members));
      return *bh < BH && *rank < tiles_per_bh;
    }
    // A grid small enough to be resident all at once (up to 4 workgroups on each of the 256 compute units) is dealt
    // out in one go, compute unit c getting ids c, c + 256, ...: then every odd group of 256 ids is walked backwards
    // (in steps of 8, so that id % 8 is kept), and a compute unit that got one of the dearest tiles of a group gets
    // one of the cheapest of the next.  Larger grids are scheduled as workgroups retire; plain dearest-first is best.
    const int grp = block >> 8;
    if ((grp & 1) && bhp * tiles_per_bh <= 1024) {
      const int left = bhp * tiles_per_bh - (grp << 8);
      const int size8 = (left < 256 ? left : 256) >> 3;
      const int pos = block & 255;
      block = (grp << 8) + ((size8 - 1 - (pos >> 3)) << 3) + (pos & 7);
    }
    *rank = block / bhp;
    *bh = block - *rank * bhp;
    return *bh < BH && *rank < tiles_per_bh;
  }
  // XCD x takes the (batch, head) pairs x, x + 8, x + 16, ... and all their tiles: the heads of one batch entry - which
  // share its sequence length - are spread over the XCDs, so a ragged batch loads the XCDs evenly
  // The tile ranks are rotated from one pair to the next: the hardware deals consecutive ids of an XCD to its compute
  // units in turn, so with a power-of-two tile count a compute unit would always get the same rank - and in a ragged
  // batch the last ranks are the ones that often lie beyond a sequence's end.
  const int j = block >> 3;
  const int q = j / tiles_per_bh;
  *bh = (block & 7) + 8 * q;
  *rank = (j - q * tiles_per_bh + q) % tiles_per_bh;
  return *bh < BH;
}
inline int tile_grid(bool tile_major, int tiles_per_bh, int BH) {
  return ((BH + 7) & ~7) * tiles_per_bh;
}
// see longest_first: dense launches without a mask whose grid is resident all at once (at most 4 workgroups on each of the
// 256 compute units), 2 to 64 batch entries
inline bool longest_first_launch(bool causal, bool sparse, int grid, int B) {
  return !causal && !sparse && grid <= 1024 && B >= 2 && B <= 64;
}

// Launch shape: with 128-row tiles a short-sequence batch gives the compute units one or two workgroups each, and one
// workgroup's walk over its keys is the launch's critical path; the forward and the dQ kernel then run their half-size
// tile variants (64 query rows, wave pairs split the keys: twice the workgroups, half the serial work of each).  The rule is
// read off a sweep over batch size, sequence length, mask and dropout (bench.py --tile-sweep): with x = full-size
// workgroups per compute unit,
//   forward: half-size for x < 2 (more than one key tile pair to split: sequences beyond 128), and up to x < 3 with dropout
//            (whose Philox work makes the serial walk longer);
//   dQ:      half-size for 1 <= x < 2 under a causal mask or with dropout; the plain kernel gains nothing from it.
// launch_policy() & 3: 0 = by this rule, 1 = always the full-size tiles, 2 = the half-size tiles wherever they exist
// (fa_set_launch_policy; the parity tests run both shapes on the same inputs).
int launch_policy();
constexpr int kSmallLaunchFwd = 0, kSmallLaunchDq = 1;
inline bool small_launch(int kernel, int BH, int max_s, bool causal, bool dropout) {
  const int policy = launch_policy() & 3;
  if (policy != 0) return policy == 2;
  const int64_t wgs = (int64_t)BH * ((max_s + 127) / 128);  // x = wgs / 256 compute units
  if (kernel == kSmallLaunchFwd) return max_s > 128 && (wgs < 2 * 256 || (dropout && wgs < 3 * 256));
  return wgs >= 256 && wgs < 2 * 256 && (causal || dropout);
}

// Short backward launches run dQ and dK/dV as one grid (fa_bwd_merged_kernel): where the dQ kernel takes its half-size tiles
// (small_launch), at head dim 64, dense, no score bias, no rotation, no key split, dropout off or read from the keep words.
inline bool merged_backward_launch(int head_dim, int BH, int max_sq, bool causal, bool dropout, bool keep_words, bool sparse,
                                   bool bias, bool rotary, int n_splits) {
  if ((launch_policy() & 0x30) == 0x10) return false;  // (the two-kernel plan was asked for)
  return head_dim == 64 && !sparse && !bias && !rotary && n_splits <= 1 && (!dropout || keep_words) &&
         small_launch(kSmallLaunchDq, BH, max_sq, causal, dropout);
}

// Launchers (defined in fa_fwd.hip / fa_bwd.hip / fa_aux.hip).  Return hipError_t of the launch.
// p.alibi != null selects the ALiBi variants (not available together with sparse)
hipError_t launch_fwd(const FwdParams& p, int dtype, int head_dim, bool causal, bool dropout, bool sparse,
                      hipStream_t stream);
hipError_t launch_fwd_combine(const FwdParams& p, int dtype, int head_dim, hipStream_t stream);
hipError_t launch_dq_combine(const BwdParams& p, int dtype, int head_dim, hipStream_t stream);
// The whole backward in one kernel (fa_bwd_fused_kernel.h; head_dim 64, dense, no mask, no dropout, no bias): softmax_d pass, then
// the kernel.  ev_start / ev_stop: null, or events recorded around the main kernel.
hipError_t launch_bwd_fused(const BwdParams& p, int dtype, hipStream_t stream, hipEvent_t ev_start, hipEvent_t ev_stop);
// fa_rotary: rotate the first n_rotated of n_parts (row, part, head, head_dim) slices, copy the others
struct RotaryParams {
  const void* src;
  void* dst;
  const void* cos;          // [table_rows, head_dim / 2], tensor dtype
  const void* sin;
  const int32_t* positions; // [n_rows] or null: position = row % seqlen
  int64_t n_rows;
  int64_t src_row_stride, src_part_stride, src_head_stride;  // elements
  int64_t dst_row_stride, dst_part_stride, dst_head_stride;
  int n_parts, n_rotated, n_heads, head_dim, seqlen, table_rows, conjugate;
  int64_t row_offset;  // set by launch_rotary: index of this launch's first row in the caller's tensor (position = row % seqlen)
};
hipError_t launch_rotary(const RotaryParams& p, int dtype, hipStream_t stream);
hipError_t launch_gather_rows(const void* src, void* dst, const int64_t* idx, int64_t n_idx, int64_t n_src,
                              int64_t row_bytes, int64_t src_stride, int64_t dst_stride, int vec, hipStream_t stream);
hipError_t launch_scatter_rows(const void* src, void* dst, const int64_t* idx, int64_t n_idx, int64_t n_dst,
                               int64_t row_bytes, int64_t src_stride, int64_t dst_stride, int vec, int32_t* inv,
                               hipStream_t stream);
hipError_t launch_bias_grad_reduce(const void* in, void* out, int dtype, int nb, int nh, int rows, int cols, int64_t in_bs,
                                   int64_t in_hs, int64_t in_rs, int sum_batch, int sum_heads, int64_t out_bs, int64_t out_hs,
                                   int64_t out_rs, bool vec_store, hipStream_t stream);
hipError_t launch_dump_probs(const DumpParams& p, int dtype, hipStream_t stream);
// which: 0 = dQ kernel, 1 = dK/dV kernel
hipError_t launch_bwd(const BwdParams& p, int which, int dtype, int head_dim, bool causal, bool dropout, bool sparse,
                      hipStream_t stream);
// order / inv: null, or the row order (SparseMaps::order) and nrb ints of scratch for its inverse
hipError_t launch_build_sparse_maps(const int32_t* blockmask, uint64_t* rbits, uint64_t* qbits, uint64_t* cbits, int nrb,
                                    int ncb, int rows_per_qt, int nqt, int ncw, int nrw, const int32_t* order, int32_t* inv,
                                    hipStream_t stream);
hipError_t launch_fill_f32(float* p, size_t n, float value, hipStream_t stream);
// Zero a strided [total, H, D] tensor of 16-bit elements.
hipError_t launch_zero_rows(void* base, int64_t row_stride, int64_t head_stride, int total, int H, int D,
                            hipStream_t stream);
// softmax_d = keep * rowsum(dO o O) (fmha_dgrad_kernel_1xN_loop.h:15-30).

// Tile shapes, needed by the front end for grid sizes and workspace layout.
constexpr int kFwdBM = 128;   // query rows per forward workgroup
constexpr int kBwdBN = 128;   // keys per dK/dV workgroup
constexpr int kFusedBM = 32;  // query rows per step of the one-kernel backward

}  // namespace fa
