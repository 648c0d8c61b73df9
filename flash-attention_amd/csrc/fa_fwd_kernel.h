// Forward attention kernel for gfx950.
//
// Computes what the reference's device_1xN_loop does (csrc/flash_attn/src/fmha_fprop_kernel_1xN.h:199-671):
// O = dropout(softmax(scale * Q K^T + mask)) V and lse = logsumexp(scale * Q K^T + mask), but organised
// query-tile-outer: one workgroup owns 128 query rows of one (batch, head), keeps the output accumulator
// and the running (max, sum) in registers, streams K/V tiles through LDS, and writes o and lse once.
// There is no fp32 o_tmp round trip through global memory.
//
// Everything is computed transposed so that one lane owns one query row:
//   S^T = K Q^T   (A = K tile from LDS, B = Q fragment held in registers), C layout: lane -> query
//                 column l%32, registers -> 16 keys.  Row max / row sum are in-lane plus ONE exchange with lane l^32.
//   O^T = V^T P^T (A = V^T read from the row-major V tile with ds_read_b64_tr_b16, B = P^T taken straight from the
//                 S^T accumulator registers, rounded to fp16/bf16).  The contraction runs over keys in the order the
//                 accumulator registers hold them; the V^T fragment is fetched in the same order.
#pragma once

#include "fa_common.h"
#include "fa_params.h"
#include "fa_stage.h"

// Measurement variants (-DFA_ABLATE_FWD=<bits> through FA_EXTRA_HIPCC_FLAGS; results are wrong, never a product build):
// what one part of the main loop costs is read off the kernel's time without it.  1: no wait for the staged tile and no
// workgroup barrier; 2: a multiplication in place of every exponential; 4: no P V products; 8: no Q K^T products; 16: the K
// and V fragments not read from LDS (registers stand in); 32: no row sums of P and no test of them.
#ifndef FA_ABLATE_FWD
#define FA_ABLATE_FWD 0
#endif

namespace fa {

// KS (key split) = 1: the workgroup's four waves own 32 of its 128 query rows each and every wave sees all keys of a tile.
// KS = 2 (short sequences, where 128-row tiles are too few workgroups to fill the chip and one workgroup's walk over the
// keys is the launch's critical path): 64 query rows per workgroup; waves w and w + 2 share 32 rows and split the keys
// of every tile between them, each with its own running maximum, sum and output accumulator, merged in the epilogue.
template <typename T, int D, int BN, int KS = 1>
struct FwdCfg {
  static constexpr int BM = kFwdBM / KS;
  static constexpr int NW = 4;                 // waves per workgroup
  static constexpr int RW = NW / KS;           // 32-row slabs per workgroup
  static constexpr int KBW = BN / 32 / KS;     // 32-key blocks of a tile per wave
  static_assert(KS == 1 || (KS == 2 && BN == 64), "key split: two waves per 32 rows, one 32-key block each");
  static constexpr int DV = D < 32 ? 32 : D;   // rows of the V^T MFMA operand (for D = 16 the upper 16 are don't-care)
  static constexpr int OS = D + 8;             // epilogue staging row stride
  // K tile (read as row fragments) followed by V tile (read transposed), double buffered; see fa_stage.h
  typedef TilePairStager<D, BN, kSwzRow, kSwzTr> Stager;
  static constexpr int kBufBytes = Stager::kPairBytes;
  static constexpr int kSlack = D < 32 ? 64 : 0;                // the 32-wide transposed reads run past a 16-wide V row
  static constexpr int kTileBytes = 2 * kBufBytes + kSlack;
  static constexpr int kEpiBytes = BM * OS * 2;
  static constexpr int kMergeBytes = KS > 1 ? RW * (DV / 32 * 16 + 2) * 64 * 4 : 0;  // partial (O, max, sum) of RW waves
  static constexpr int kLdsBytes0 = kTileBytes > kEpiBytes ? kTileBytes : kEpiBytes;
  static constexpr int kLdsBytes = kLdsBytes0 > kMergeBytes ? kLdsBytes0 : kMergeBytes;
  static constexpr int CH = D / 8;
};

// kBias (fa_params.h): 1 = ALiBi, the score of (query i, key j) gets -slope[head] * |i - j| added after scaling; 2 = it gets
// bias[b, h, i, j] of a tensor added.  The scores are then moved to the softmax's own units (base-2 exponent) before the row
// maximum is taken, and the running maximum is kept in those units.
// kWords (dropout, dense): the keep decisions are also left in p.keep_words for the backward (fa_common.h)
template <typename T, int D, int BN, bool kCausal, bool kDropout, bool kSparse, int kBias = 0, int KS = 1,
          bool kWords = false>
__global__ void __launch_bounds__(256, ((!kDropout || KS == 2) && kBias == 0 && D <= 64) ? 4 : ((!kDropout && kBias == kBiasTensor && D <= 64) ? 3 : 2)) fa_fwd_kernel(const FwdParams p) {
  constexpr bool kAlibi = kBias == kBiasAlibi, kTensorBias = kBias == kBiasTensor;
  static_assert(!kWords || (kDropout && !kSparse), "keep words: dense dropout variants only");
  using Cfg = FwdCfg<T, D, BN, KS>;
  using E = Elem<T>;
  using vec8 = typename E::vec8;
  constexpr int BM = Cfg::BM, DV = Cfg::DV, CH = Cfg::CH, kBufBytes = Cfg::kBufBytes, KBW = Cfg::KBW;
  static_assert(KS == 1 || !kSparse, "the block-sparse maps are built for 128-row query tiles");

  // kTensorBias: behind the tiles, per wave 32 rows x BN keys of bias, rows padded by 8 bytes (see load_bias below)
  constexpr int kBiasRowBytes = BN * 2 + 8, kBiasWaveBytes = 32 * kBiasRowBytes;
  __shared__ __attribute__((aligned(16))) unsigned char lds_raw[Cfg::kLdsBytes + (kTensorBias ? 4 * kBiasWaveBytes : 0)];

  // Workgroup -> (batch, head, query tile), XCD-aware (see map_tile): the query tiles of one (batch, head) share
  // one XCD's L2 copy of K and V.
  int bh, rank;
  const int n_splits = p.n_splits > 1 ? p.n_splits : 1;   // key splits per query tile (see FwdParams)
  if (!map_tile<kCausal>(blockIdx.x, p.nq_tiles * n_splits, p.B * p.H, &bh, &rank, p.tile_group)) return;
  const int split = rank % n_splits;
  rank /= n_splits;
  const int qt = kCausal ? p.nq_tiles - 1 - rank : rank;  // under a causal mask the last query tiles cost most
  const int h = bh % p.H;
  // (dense, no mask: the batch entries are taken longest keys first, see longest_first)
  const int b = (!kCausal && !kSparse && p.tile_group < 0) ? longest_first(p.cu_k, p.B, bh / p.H) : bh / p.H;
  bh = b * p.H + h;  // (what the dropout counters and the keep words are indexed by)

  int q_begin, Lq, k_begin = 0, Lk = 0;
  if (!seq_extent(p.cu_q, b, p.total_q, p.max_sq, &q_begin, &Lq)) return;
  if (!seq_extent(p.cu_k, b, p.total_k, p.max_sk, &k_begin, &Lk)) Lk = 0;  // no keys: o = 0, lse = -inf
  const int m0 = qt * BM;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 31, hf = lane >> 5;
  const int rs = KS > 1 ? wave % Cfg::RW : wave;  // this wave's 32-row slab of the tile
  const int kh = KS > 1 ? wave / Cfg::RW : 0;     // ... and its share of every key tile's 32-key blocks
  const int mw = m0 + rs * 32;    // first query row of this wave
  int qrow = mw + c;              // this lane's query row (sequence-local)
  // Sparse: the wave's 32 rows are two 16-row blocks, consecutive ones or - with a row order (SparseMaps) - two the caller
  // put next to each other; rows of no block count as lying past the end
  int rb_a = -1, rb_b = -1;
  bool wave_live = mw < Lq;  // some row of the wave exists
  if (kSparse) {
    const bool ordered = !kCausal && p.sp.order != nullptr;
    slab_row_blocks(p.sp, ordered, qt, rs, &rb_a, &rb_b);
    const int rbl = c < 16 ? rb_a : rb_b;
    qrow = rbl >= 0 ? rbl * 16 + (c & 15) : 0x3fffffff;
    wave_live = (rb_a >= 0 && rb_a * 16 < Lq) || (rb_b >= 0 && rb_b * 16 < Lq);
    if (ordered) {
      if (!__syncthreads_or(wave_live)) return;  // no row of the workgroup exists
    } else if (m0 >= Lq) {
      return;
    }
  } else if (m0 >= Lq) {
    return;
  }

  // ---- Q fragment (B operand of S^T = K Q^T), held in registers for the whole kernel
  vec8 qreg[D / 16];
  {
    const int qr = qrow < Lq ? qrow : Lq - 1;
    const T* qp = reinterpret_cast<const T*>(p.q) + (int64_t)(q_begin + qr) * p.q_rs + (int64_t)h * p.q_hs + hf * 8;
#pragma unroll
    for (int ks = 0; ks < D / 16; ks++) qreg[ks] = bitcast<vec8>(ld_global16(qp + ks * 16));
    // rows past the end work on a copy of the last row and are never stored (no select on the loaded data here: it
    // would make the wave wait for the load before it has issued its first tile)
  }

  int n_end = Lk;
  if (kCausal) n_end = n_end < m0 + BM ? n_end : m0 + BM;
  const int ntiles_all = (n_end + BN - 1) / BN;
  const int tile0 = (int)((int64_t)split * ntiles_all / n_splits);        // this workgroup's share of the key tiles
  const int ntiles = (int)((int64_t)(split + 1) * ntiles_all / n_splits);

  // ---- K/V staging: global -> LDS without passing through registers (waves 0,1 fetch K tiles, waves 2,3 V tiles)
  typename Cfg::Stager stager;
  stager.init(wave, lane, reinterpret_cast<const T*>(p.k) + (int64_t)k_begin * p.k_rs + (int64_t)h * p.k_hs, p.k_rs,
              reinterpret_cast<const T*>(p.v) + (int64_t)k_begin * p.v_rs + (int64_t)h * p.v_hs, p.v_rs);
  auto stage = [&](int it, int buf) { stager.issue(lds_raw + buf * kBufBytes, it * BN, Lk); };

  // Sparse: tile `it` is computed iff its 256-key block is active for any 16-row block of this query tile.  The tile's
  // and this lane's row block's activity bits of 64 consecutive key blocks (16384 keys) sit in registers.
  uint64_t tile_bits = 0, row_bits = 0;
  int bits_word = -1;
  const int qt_u = __builtin_amdgcn_readfirstlane(qt);
  // First tile >= it whose 256-key block is active (ntiles if none): the bits of the loaded word are searched with a
  // count-trailing-zeros, not tile by tile.
  bool row_on_next = true;  // this lane's row block attends the tile the last next_active() found
  auto next_active = [&](int it) -> int {
    if (!kSparse) return it;
    constexpr int kTilesPerBlock = 256 / BN;
    while (it < ntiles) {
      const int cb = __builtin_amdgcn_readfirstlane((it * BN) >> 8);
      if ((cb >> 6) != bits_word) {
        bits_word = cb >> 6;
        tile_bits = uniform64(p.sp.qbits[(int64_t)qt_u * p.sp.ncw + bits_word]);
        const int rbl = c < 16 ? rb_a : rb_b;
        row_bits = rbl >= 0 ? p.sp.rbits[(int64_t)rbl * p.sp.ncw + bits_word] : 0;
      }
      const uint64_t rest = tile_bits >> (cb & 63);  // bit 0: this tile's block
      if (rest & 1) break;
      // first tile of the next active block of this word, or of the next word
      it = (rest ? cb + (int)__builtin_ctzll(rest) : (cb | 63) + 1) * kTilesPerBlock;
    }
    if (it > ntiles) it = ntiles;
    if (it < ntiles) row_on_next = (row_bits >> (((it * BN) >> 8) & 63)) & 1;
    return it;
  };

  f32x16 o_acc[DV / 32];
#pragma unroll
  for (int i = 0; i < DV / 32; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) o_acc[i][r] = 0.f;
  float m_i = -INFINITY;  // running row max of raw scores (before scaling)
  float l_i = 0.f;        // this lane's share of the running row sum (other share in lane^32)

  const float cs = p.scale_log2;
  const float cse = kBias != 0 ? 1.f : cs;                       // units of the scores the softmax works on
  const float sl2 = kAlibi ? p.alibi[h] * kLog2e : 0.f;          // slope in base-2 exponent units
  // kTensorBias: the wave's 32 rows x BN keys of the bias come in as whole rows - BN / 8 lanes fetch the BN * 2 contiguous
  // bytes of one row, 16 bytes each, so that an instruction touches 8 (16) rows and not 32: read lane by lane in the MFMA
  // layout (every lane another row) the requests, one per row and instruction, took as long as the whole kernel without a
  // bias - and are turned into that layout through LDS (wave-private, rows padded by 8 bytes: 32 lanes reading 8 bytes at the
  // same column of 32 rows hit 32 distinct bank pairs).  Asked for one tile ahead; chunks that begin past the last key are
  // not read, rows past the end read the last row (like Q).
  constexpr int kBiasCPR = BN / 8, kBiasRPI = 64 / kBiasCPR, kBiasNLD = 32 / kBiasRPI;
  const T* const bias_bh =
      kTensorBias ? reinterpret_cast<const T*>(p.bias) + (int64_t)b * p.bias_bs + (int64_t)h * p.bias_hs : nullptr;
  unsigned char* const bias_lds = lds_raw + Cfg::kLdsBytes + wave * kBiasWaveBytes;
  u32x4 braw[kTensorBias ? kBiasNLD : 1];
  auto load_bias = [&](int tile) {
#pragma unroll
    for (int i = 0; i < kBiasNLD; i++) {
      const int lr = i * kBiasRPI + lane / kBiasCPR, k0 = tile * BN + (lane % kBiasCPR) * 8;
      int row = mw + lr;
      if (kSparse) {  // the slab's two row blocks (rows of no block read the last row: their results are never stored)
        const int rbl = lr < 16 ? rb_a : rb_b;
        row = rbl >= 0 ? rbl * 16 + (lr & 15) : Lq;
      }
      braw[i] = u32x4{0, 0, 0, 0};
      if (k0 < Lk) braw[i] = ld_global16(bias_bh + (uint32_t)(row < Lq ? row : Lq - 1) * (uint32_t)p.bias_rs + (uint32_t)k0);
    }
  };
  auto bias_to_lds = [&]() {
#pragma unroll
    for (int i = 0; i < kBiasNLD; i++)
      *reinterpret_cast<u32x4*>(bias_lds + (i * kBiasRPI + lane / kBiasCPR) * kBiasRowBytes + (lane % kBiasCPR) * 16) = braw[i];
  };
  int voff[DV / 32];  // element offsets of this lane's transposed V reads and K row fragments inside a tile
#pragma unroll
  for (int db = 0; db < DV / 32; db++) voff[db] = tr_off<D, kSwzTr>(0, db * 4, lane);
  int koff[D / 16];
#pragma unroll
  for (int ks = 0; ks < D / 16; ks++) koff[ks] = frag_off<D, kSwzRow>(c, ks * 2 + hf);
  int buf = 0;

  // Dropout keep words for the backward (fa_common.h): a tile's words are stored at the top of the next step, ahead of
  // the next prefetch - stored where they are made, their acknowledgements would still be outstanding when the step
  // ends and waits for its prefetched tile (one counter serves loads and stores).
  uint32_t kwout[KBW];
  int kw_pending = -1;  // first key block (of 32) of the words waiting in kwout
  auto flush_keep_words = [&]() {
    if (kWords && kw_pending >= 0) {
      if (hf == 0) {
#pragma unroll
        for (int kb = 0; kb < KBW; kb++)
          p.keep_words[((int64_t)bh * p.kw_kb + kw_pending + kb) * p.kw_q + mw + (keep_word_slot(c) & 31)] = kwout[kb];
      }
      kw_pending = -1;
    }
  };

  int it = next_active(tile0);
  bool row_on_cur = row_on_next;
  if (it < ntiles) {
    stage(it, 0);
    if (kTensorBias) load_bias(it);
  }
  // Rotary embedding of the queries (what the reference's FlashMHA does to q before attention, flash_attention.py:109-113,
  // with elementwise ops): the fragments are turned where they sit, after the first tile has been asked for; the rotated
  // rows are left in q_rot for the backward, whose kernels stream Q through LDS and cannot do the same
  if (p.rot_cos != nullptr) {
    int t = qrow < Lq ? qrow : Lq - 1;
    t = t < p.rot_rows ? t : p.rot_rows - 1;
    const T* const ct = reinterpret_cast<const T*>(p.rot_cos) + (int64_t)t * (D / 2) + hf * 4;
    const T* const st = reinterpret_cast<const T*>(p.rot_sin) + (int64_t)t * (D / 2) + hf * 4;
#pragma unroll
    for (int ks = 0; ks < D / 16; ks++)
      qreg[ks] = rotate8<T>(qreg[ks], *reinterpret_cast<const typename E::vec4*>(ct + ks * 8),
                            *reinterpret_cast<const typename E::vec4*>(st + ks * 8), false);
    if (p.q_rot != nullptr && kh == 0 && split == 0 && qrow < Lq) {
      T* const qo = reinterpret_cast<T*>(p.q_rot) + (int64_t)(q_begin + qrow) * p.qr_rs + (int64_t)h * p.qr_hs + hf * 8;
#pragma unroll
      for (int ks = 0; ks < D / 16; ks++) st_global16(qo + ks * 16, bitcast<u32x4>(qreg[ks]));
    }
  }
  while (it < ntiles) {
    const int n0 = it * BN;
    // Opaque redefinition of the accumulators at the top of every iteration: without it the register allocator
    // ties the last MFMA's result to the registers the epilogue reads and copies all of O back on every trip.
#pragma unroll
    for (int i = 0; i < DV / 32; i++) asm volatile("" : "+v"(o_acc[i]));
    if constexpr ((FA_ABLATE_FWD & 1) == 0) {
      wait_vmem();                       // this wave's share of tile `it` is in LDS
      flush_keep_words();
      __syncthreads();                   // so is everyone else's, and nobody still reads the other buffer
    }
    const int it_next = next_active(it + 1);
    if (it_next < ntiles) stage(it_next, buf ^ 1);
    if (kTensorBias) {  // (the wave's own reads of the last tile's values are behind it: LDS operations of a wave stay in order)
      bias_to_lds();
      if (it_next < ntiles) load_bias(it_next);
    }
    const T* Ks = reinterpret_cast<const T*>(lds_raw + buf * kBufBytes);
    const T* Vs = Ks + BN * D;
    buf ^= 1;

    bool wave_work = wave_live;  // a wave whose 32 rows all lie past the sequence's end only helps with the staging
    if (kCausal && n0 + kh * 32 * KBW > mw + 31) wave_work = false;  // every key of the wave's share is above its diagonal
    if (KS > 1 && n0 + kh * 32 * KBW >= Lk) wave_work = false;       // ... or past the last key
    bool row_on = true;
    if (kSparse) {
      row_on = row_on_cur;
      row_on_cur = row_on_next;  // next_active(it + 1) above has set it
      if (__ballot(row_on) == 0) wave_work = false;
    }

    if (wave_work) {
      // this wave's 32-key blocks of the tile: kb0, kb0 + 1, ... (all of them without a key split)
      const int kb0 = kh * KBW;
      f32x16 s[KBW];
      // ---- S^T = K Q^T, dead scores set to -inf, bias added
      auto scores = [&]() {
        // kTensorBias: the lane's 4 x 4 consecutive bias values per 32-key block (registers 4 j .. 4 j + 3 <-> keys
        // 8 j + 4 hf ..) of its row
        typename E::vec4 bv[kTensorBias ? KBW : 1][4];
        if (kTensorBias) {
#pragma unroll
          for (int kb = 0; kb < KBW; kb++)
#pragma unroll
            for (int j = 0; j < 4; j++)
              bv[kb][j] = *reinterpret_cast<const typename E::vec4*>(bias_lds + c * kBiasRowBytes + ((kb0 + kb) * 32 + 8 * j + 4 * hf) * 2);
        }
#pragma unroll
        for (int kb = 0; kb < KBW; kb++) {
#pragma unroll
          for (int r = 0; r < 16; r++) s[kb][r] = 0.f;
#pragma unroll
          for (int ks = 0; ks < D / 16; ks++) {
            vec8 a = (FA_ABLATE_FWD & 16) ? qreg[(ks + 1) % (D / 16)] : *reinterpret_cast<const vec8*>(Ks + (kb0 + kb) * 32 * D + koff[ks]);
            if constexpr ((FA_ABLATE_FWD & 8) == 0) s[kb] = E::mfma32(a, qreg[ks], s[kb]);
            else s[kb][ks] = (float)a[ks] * (float)qreg[ks][0];
          }
        }
        // mask: only tiles that straddle the key length or the diagonal.  (An inactive row block inside an active tile is
        // not masked score by score: its lanes' exponentials are taken against +inf below.)
        const bool need_mask = (n0 + BN > Lk) || (kCausal && (n0 + BN - 1 > mw));
        if (need_mask) {
#pragma unroll
          for (int kb = 0; kb < KBW; kb++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
              const int key = n0 + (kb0 + kb) * 32 + (r >> 2) * 8 + hf * 4 + (r & 3);
              bool dead = key >= Lk;
              if (kCausal) dead = dead || key > qrow;
              if (dead) s[kb][r] = -INFINITY;
            }
        }
        if (kTensorBias) {  // s <- s * scale * log2(e) + bias * log2(e)
          // Dead scores must stay -inf whatever lies behind them: past the last key a row of the caller's tensor may hold
          // anything, so on a tile that needs a mask +inf and NaN are cut off (fminf returns the number)
#pragma unroll
          for (int kb = 0; kb < KBW; kb++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
              float bf = (float)bv[kb][r >> 2][r & 3];
              if (need_mask) bf = fminf(bf, 3.0e38f);
              s[kb][r] = __builtin_fmaf(bf, kLog2e, s[kb][r] * cs);
            }
        }
        if (kAlibi) {  // s <- s * scale * log2(e) - slope2 * |key - query|; dead scores stay -inf
#pragma unroll
          for (int kb = 0; kb < KBW; kb++) {
            const float dbase = (float)(n0 + (kb0 + kb) * 32 + hf * 4 - qrow);  // key - query of register 0
#pragma unroll
            for (int r = 0; r < 16; r++) {
              const float cr = (float)((r >> 2) * 8 + (r & 3));
              // under a causal mask every live score has key <= query: -|key - query| = key - query, linear in cr
              const float bias = kCausal ? __builtin_fmaf(cr, sl2, sl2 * dbase) : -sl2 * __builtin_fabsf(dbase + cr);
              s[kb][r] = __builtin_fmaf(s[kb][r], cs, bias);
            }
          }
        }
      };
      // ---- P = exp2(scores - reference point m_i), rounded to the tensor dtype (what the P V product consumes); lt = this
      // lane's share of the tile's row sums: of the rounded values, or with dropout of P before the mask, in fp32 as the
      // reference has it (fmha_fprop_kernel_1xN.h:454 vs :471)
      vec8 pb[KBW][2];
      float lt;
      auto probabilities = [&]() {
        float mc = ((m_i == -INFINITY) ? 0.f : m_i) * cse;
        if (kSparse && !row_on) mc = INFINITY;  // this lane's row block does not attend the tile: P = exp2(x - inf) = 0
        lt = 0.f;
#pragma unroll
        for (int kb = 0; kb < KBW; kb++)
#pragma unroll
          for (int r = 0; r < 16; r++) {
            const float pe_arg = kBias != 0 ? s[kb][r] - mc : __builtin_fmaf(s[kb][r], cs, -mc);
            const float pe = (FA_ABLATE_FWD & 2) ? pe_arg * 1e-3f : fast_exp2(pe_arg);
            s[kb][r] = pe;
            if (kDropout) lt += pe;
          }
        if (kDropout) {
#pragma unroll
          for (int kb = 0; kb < KBW; kb++) {
            const KeepFields keep = keep_fields_row_layout(p.pk, (uint32_t)bh, qrow, n0 + (kb0 + kb) * 32, hf);
            if (kWords) {
              // the lane's 16 keep bits are gathered into its share of the row's keep word (fa_common.h) for the backward
              // (dead scores keep whatever bit they drew: their P is 0)
              uint32_t kw = 0;
#pragma unroll
              for (int r = 0; r < 16; r++) {
                const bool kept = keep.keep_row(r, p.keep_thr);
                if (!kept) s[kb][r] = 0.f;
                kw = shift_in_lane_bit(kw, __builtin_amdgcn_ballot_w64(kept));
                if ((r & 3) == 3 && r != 15) kw <<= 4;
                // (a compare's 64-bit result is to be used up before the next is made: all sixteen held at once would
                // overflow the scalar registers into vector ones)
                if ((r & 3) == 3) __builtin_amdgcn_sched_barrier(0);
              }
              kwout[kb] = keep_word_from_shares(kw, hf);
              kw_pending = (n0 >> 5) + kb0;
            } else {
#pragma unroll
              for (int r = 0; r < 16; r++)
                if (!keep.keep_row(r, p.keep_thr)) s[kb][r] = 0.f;
            }
          }
        }
#pragma unroll
        for (int kb = 0; kb < KBW; kb++)
#pragma unroll
          for (int t = 0; t < 2; t++) {
            f32x8 pf;
#pragma unroll
            for (int i = 0; i < 8; i++) pf[i] = s[kb][8 * t + i];
            pb[kb][t] = cvt8<T>(pf);
            if (!kDropout && (FA_ABLATE_FWD & 32) == 0) lt = sum8_acc(pb[kb][t], lt);
          }
      };
      // ---- online softmax (fmha_fprop_kernel_1xN.h:408-454,560-611 restated for a register-resident row).
      // The reference point m_i of the exponentials only moves when it has to: P may exceed 1 by a factor of up to
      // 2^kRescaleLog2, which the fp32 accumulators and the fp16/bf16 rounding of P absorb (numerator and denominator carry
      // the same factor, so the result is unchanged).  Whether it has to move is read off the tile's row sums - if a lane's
      // share is at most 2^kRescaleLog2, so is every P behind it - so the common tile takes no row maximum at all.  A tile
      // that fails the test (the first of a row always does: no reference point yet) is redone the long way: scores again,
      // row maxima, rescaled accumulators, probabilities against the new reference point.
      scores();
      bool redo = __any(m_i == -INFINITY && (!kSparse || row_on));
      if (!redo) {
        probabilities();
        if constexpr ((FA_ABLATE_FWD & 32) == 0) redo = __any(!(lt <= kRescaleLimit));  // also catches inf and NaN
        if (__builtin_expect(redo, 0)) scores();
      }
      if (__builtin_expect(redo, 0)) {
        float mt = s[0][0];
#pragma unroll
        for (int kb = 0; kb < KBW; kb++)
#pragma unroll
          for (int r = 0; r < 16; r++) mt = fmaxf(mt, s[kb][r]);
        mt = half_max(mt);
        if (kSparse && !row_on) mt = -INFINITY;
        const float m_new = fmaxf(m_i, mt);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = fast_exp2(m_i * cse - m_use * cse);
        m_i = m_new;
        l_i *= alpha;
#pragma unroll
        for (int i = 0; i < DV / 32; i++) o_acc[i] = o_acc[i] * alpha;
        probabilities();
      }
      l_i += lt;

      // ---- O^T += V^T P^T
#pragma unroll
      for (int kb = 0; kb < KBW; kb++) {
#pragma unroll
        for (int t = 0; t < 2; t++) {
#pragma unroll
          for (int db = 0; db < DV / 32; db++) {
            const T* vp = Vs + ((kb0 + kb) * 32 + 16 * t) * D + voff[db];
            u32x4 av;
            if constexpr ((FA_ABLATE_FWD & 16) == 0) {
              u32x2 lo = lds_read_tr16(vp);
              u32x2 hi = lds_read_tr16(vp + 8 * D);
              av = u32x4{lo[0], lo[1], hi[0], hi[1]};
            } else {
              av = bitcast<u32x4>(qreg[db]);
            }
            if constexpr ((FA_ABLATE_FWD & 4) == 0) o_acc[db] = E::mfma32(bitcast<vec8>(av), pb[kb][t], o_acc[db]);
            else asm volatile("" ::"v"(av), "v"(pb[kb][t]));
          }
        }
      }
    }
    it = it_next;
  }
  flush_keep_words();

  // ---- key split: the waves kh > 0 hand their partial (O, maximum, sum) to the wave kh == 0 of their rows, in the
  // accumulator's own register order (word (rs * (16 DV/32 + 2) + j) * 64 + lane: consecutive lanes, no bank conflicts)
  if (KS > 1) {
    __syncthreads();  // every wave has left the tiles
    constexpr int NJ = DV / 32 * 16 + 2;
    float* const X = reinterpret_cast<float*>(lds_raw) + rs * NJ * 64 + lane;
    if (kh != 0) {
#pragma unroll
      for (int db = 0; db < DV / 32; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) X[(db * 16 + r) * 64] = o_acc[db][r];
      X[(NJ - 2) * 64] = m_i;
      X[(NJ - 1) * 64] = l_i;
    }
    __syncthreads();
    if (kh == 0) {
      const float m_b = X[(NJ - 2) * 64], l_b = X[(NJ - 1) * 64];
      const float m_new = fmaxf(m_i, m_b);
      const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
      const float wa = fast_exp2(m_i * cse - m_use * cse), wb = fast_exp2(m_b * cse - m_use * cse);  // exp2(-inf) = 0
      m_i = m_new;
      l_i = l_i * wa + l_b * wb;
#pragma unroll
      for (int db = 0; db < DV / 32; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) o_acc[db][r] = o_acc[db][r] * wa + X[(db * 16 + r) * 64] * wb;
    }
    __syncthreads();  // the staging area of the stores below overlaps the exchange area
    if (kh != 0) return;
  }
  // ---- epilogue: normalise, write lse, transpose O^T through LDS for coalesced 16-byte stores
  const float l_tot = half_sum(l_i);
  const bool empty = !(l_tot > 0.f);  // also catches NaN (fmha_fprop_kernel_1xN.h:575,606)
  float inv = empty ? 1.f : fast_rcp(l_tot);
  if (kDropout) inv *= p.rp_keep;
  const float lse_val = empty ? -INFINITY : (m_i * cse + fast_log2(l_tot)) * kLn2;
  if (p.n_splits > 1) {  // partial result of this key split, fp32, merged by fwd_combine_kernel
    if (qrow < Lq) {
      if (hf == 0) p.lse_part[(((int64_t)split * p.B + b) * p.H + h) * p.sq_r + qrow] = lse_val;
      float* op = p.o_part + (((int64_t)split * p.total_q + q_begin + qrow) * p.H + h) * D;
#pragma unroll
      for (int db = 0; db < DV / 32; db++)
#pragma unroll
        for (int g4 = 0; g4 < 4; g4++) {
          const int d0 = db * 32 + g4 * 8 + hf * 4;
          if (d0 < D) {
            f32x4 x;
#pragma unroll
            for (int i = 0; i < 4; i++) x[i] = o_acc[db][g4 * 4 + i] * inv;
            *reinterpret_cast<f32x4*>(op + d0) = x;
          }
        }
    }
    return;
  }
  if (hf == 0 && qrow < Lq) p.lse[((int64_t)b * p.H + h) * p.sq_r + qrow] = lse_val;
  if (KS == 1) __syncthreads();
  constexpr int OS = Cfg::OS;
  T* Os = reinterpret_cast<T*>(lds_raw) + rs * 32 * OS;
#pragma unroll
  for (int db = 0; db < DV / 32; db++)
#pragma unroll
    for (int g4 = 0; g4 < 4; g4++) {
      const int d0 = db * 32 + g4 * 8 + hf * 4;
      if (d0 < D) {
        f32x4 x;
#pragma unroll
        for (int i = 0; i < 4; i++) x[i] = o_acc[db][g4 * 4 + i] * inv;
        *reinterpret_cast<typename E::vec4*>(Os + c * OS + d0) = cvt4<T>(x);
      }
    }
  __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wave's LDS writes have landed
  __builtin_amdgcn_wave_barrier();
  T* obase = reinterpret_cast<T*>(p.o) + (int64_t)q_begin * p.o_rs + (int64_t)h * p.o_hs;
#pragma unroll
  for (int i = 0; i < (32 * CH + 63) / 64; i++) {
    const int ch = lane + i * 64;
    const int row = ch / CH, col = (ch % CH) * 8;
    int orow = mw + row;  // (sparse: the wave's rows are those of its two row blocks)
    if (kSparse) orow = (row < 16 ? rb_a : rb_b) < 0 ? 0x3fffffff : (row < 16 ? rb_a : rb_b) * 16 + (row & 15);
    if ((32 * CH % 64 == 0 || ch < 32 * CH) && orow < Lq) {
      u32x4 val = *reinterpret_cast<const u32x4*>(Os + row * OS + col);
      st_global16(obase + (int64_t)orow * p.o_rs + col, val);
    }
  }
}

}  // namespace fa
