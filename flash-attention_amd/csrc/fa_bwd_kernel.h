// Backward attention kernels for gfx950.
//
// Together they compute what the reference's compute_dq_dk_dv_1xN does
// (csrc/flash_attn/src/fmha_dgrad_kernel_1xN_loop.h:34-700):
//   P  = exp(scale * S - lse) recomputed from Q, K;  dP = dO V^T;  dS' = P o (M o dP - Dk)   (M = dropout keep mask,
//   Dk = keep * rowsum(dO o O));  dV = (P o M)^T dO / keep;  dK = dS'^T Q * scale / keep;  dQ = dS' K * scale / keep.
//
// The work is split in two kernels so that every output has exactly one owner and nothing is accumulated through
// global memory (the reference carries dQ across key blocks in an fp32 dq_tmp buffer, :444-461,571-592; on this
// part fp32 global atomics for that buffer cost more than recomputing S and dP):
//
// fa_bwd_dkdv_kernel  one workgroup owns 128 keys of one (batch, head) (wave w: keys 32w..32w+31), keeps its K and V
//   fragments and the dK^T / dV^T accumulators in registers and streams 64-row tiles of Q, dO, lse, Dk through LDS.
//     S  = Q K^T, dP = dO V^T           A = Q / dO rows from LDS, B = K / V fragments in registers;
//                                       C layout: lane -> key, registers -> 16 query rows
//     dV^T += dO^T P, dK^T += Q^T dS'   B = P / dS' straight from the accumulator registers (rounded to fp16/bf16 as
//                                       the reference does before these GEMMs, :344,435), A = dO^T / Q^T read from the
//                                       same row-major LDS tiles with ds_read_b64_tr_b16
//
// fa_bwd_dq_kernel    (launched first) one workgroup owns 128 query rows (wave w: rows 32w..32w+31), keeps Q, dO
//   fragments, lse and the dQ^T accumulator in registers, computes Dk = keep * rowsum(dO o O) of its rows (stored to
//   softmax_d for the dK/dV kernel) and streams 64-key tiles of K and V through LDS; everything transposed so one
//   lane owns one query row (as in the forward kernel):
//     S^T = K Q^T, dP^T = V dO^T        A = K / V rows from LDS, B = Q / dO fragments in registers
//     dQ^T += K^T dS'^T                 B = dS'^T from the accumulator registers, A = K^T via ds_read_b64_tr_b16
#pragma once

#include "fa_common.h"
#include "fa_params.h"
#include "fa_stage.h"

// Measurement variants of the dK/dV kernel (-DFA_ABLATE_DKDV=<bits>, as FA_ABLATE_FWD in fa_fwd_kernel.h; results are wrong,
// never a product build).  1: no wait for the staged tile and no workgroup barrier; 2: a multiplication in place of every
// exponential; 4: no dV and dK products; 8: no S and dP products.
#ifndef FA_ABLATE_DKDV
#define FA_ABLATE_DKDV 0
#endif

namespace fa {

// ---------------------------------------------------------------------------------------------------------------
// dK, dV
// ---------------------------------------------------------------------------------------------------------------
template <typename T, int D, bool kDropout = false>
struct BwdCfg {
  static constexpr bool kVLds = D == 128 && !kDropout;  // see below
  static constexpr int BM = kVLds ? 32 : 64;  // query rows per step
  static constexpr int BN = kBwdBN;  // keys per workgroup
  static constexpr int DV = D < 32 ? 32 : D;
  // Q tile followed by dO tile, both read as row fragments and transposed, double buffered (see fa_stage.h),
  // then two buffers of per-row statistics (lse and -Dk)
  typedef TilePairStager<D, BM, kSwzDual, kSwzDual> Stager;
  static constexpr int kBufBytes = Stager::kPairBytes;
  static constexpr int kSlack = D < 32 ? 64 : 0;  // the 32-wide transposed reads run past a 16-wide row
  static constexpr int kOffStat = 2 * kBufBytes + kSlack;
  static constexpr int kStatBytes = 2 * BM * 4;   // lse[BM], -Dk[BM]
  // At d = 128 the K and V fragments plus the two accumulators of a wave would be 192 registers: more than two waves per
  // SIMD allow next to the scores.  There (without dropout, whose Philox state needs the registers anyway and which
  // stays at one wave per SIMD) the workgroup's V tile sits in LDS for the whole kernel instead, rows padded by
  // 8 elements (16 lanes reading one 16-byte chunk of 16 consecutive rows then hit 16 distinct bank groups, and a
  // fragment's address is one register plus a constant), and the query tile is one 32-row slab, so that two workgroups
  // fit a compute unit's LDS.
  static constexpr int VS = D + 8;  // V tile row stride in elements
  static constexpr int kOffV = kOffStat + 2 * kStatBytes;
  static constexpr int kTileBytes = kOffV + (kVLds ? BN * VS * 2 : 0);
  static constexpr int kEpiBytes = BN * (D + 8) * 2;
  static constexpr int kLdsBytes = kTileBytes > kEpiBytes ? kTileBytes : kEpiBytes;
  static constexpr int CH = D / 8;
  static constexpr int kMinBlocks = (D == 128 && kDropout) ? 1 : 2;
  static constexpr int kBiasTileBytes = BM * 32 * 2;  // per wave, behind everything else: the bias-tensor variants' tile
};

// kDrop: 0 = no dropout; 1 = the keep decisions are drawn here (Philox); 2 = they are read from the keep words the
// forward left (fa_common.h; dense only): the kernel then has the tile shape of the one without dropout.
// kBias: as in fa_fwd_kernel; with a bias tensor the kernel also leaves d(loss)/d(bias) in p.dbias if that is not null
// kRot: the keys came in rotated (rotary position embedding) and dK goes out turned back (dense variants without score bias
// only; a variant of its own because the plain kernels sit at their register limit)
// (the kernel proper is fa_bwd_dkdv_kernel below: `block` is its workgroup id, `lds_raw` its LDS)
// kOwnD: the kernel forms Dk = keep * rowsum(dO o O) of every tile's rows itself instead of reading what the dQ kernel left in
// p.dsoftmax (four threads per row, 16 elements each, fetched with the tile): it then depends on nothing the dQ kernel writes,
// and the two can share one launch (fa_bwd_merged_kernel).  64-row tiles, head dim 64.
template <typename T, int D, bool kCausal, int kDrop, bool kSparse, int kBias = 0, bool kRot = false, bool kOwnD = false>
FA_DEVICE void fa_bwd_dkdv_body(const BwdParams& p, const int block, unsigned char* const lds_raw) {
  static_assert(!kRot || (!kSparse && kBias == 0), "rotary: dense variants without score bias");
  static_assert(!kOwnD || (D == 64 && !kSparse && kBias == 0 && BwdCfg<T, D, kDrop == 1>::BM == 64), "own Dk: d = 64, dense");
  constexpr bool kDropout = kDrop == 1, kStored = kDrop == 2;
  constexpr bool kAlibi = kBias == kBiasAlibi, kTensorBias = kBias == kBiasTensor;
  static_assert(!(kStored && kSparse), "keep words: dense only");
  using Cfg = BwdCfg<T, D, kDropout>;
  using E = Elem<T>;
  using vec8 = typename E::vec8;
  using vec4 = typename E::vec4;
  constexpr int BM = Cfg::BM, BN = Cfg::BN, DV = Cfg::DV, CH = Cfg::CH, kBufBytes = Cfg::kBufBytes;
  static_assert(BM == 64 || BM == 32, "a tile is one or two 32-row slabs");
  constexpr int RBT = BM / 16;  // 16-row blocks per tile (sparse activity bits per tile)

  // kTensorBias: behind everything else, per wave BM rows x its 32 keys of bias (see load_bias below)
  constexpr int kBiasTileBytes = BM * 32 * 2;
  static_assert(kBiasTileBytes == BwdCfg<T, D, kDrop == 1>::kBiasTileBytes, "LDS size of the kernel");

  // XCD-aware id map (see map_tile): the key tiles of one (batch, head) share one XCD's L2 copy of Q and dO.
  int bh, kt;  // under a causal mask the first key tiles see the most query rows: rank order is already heavy-first
  if (!map_tile<kCausal>(block, p.nk_tiles, p.B * p.H, &bh, &kt, p.tile_group)) return;
  const int h = bh % p.H;
  // (dense, no mask: the batch entries are taken longest first - here by their queries, which a key tile walks; longest_first)
  const int b = (!kCausal && !kSparse && p.tile_group < 0) ? longest_first(p.cu_q, p.B, bh / p.H) : bh / p.H;
  bh = b * p.H + h;  // (what the dropout counters and the keep words are indexed by)

  int q_begin = 0, Lq = 0, k_begin, Lk;
  if (!seq_extent(p.cu_k, b, p.total_k, p.max_sk, &k_begin, &Lk)) return;
  if (!seq_extent(p.cu_q, b, p.total_q, p.max_sq, &q_begin, &Lq)) Lq = 0;  // no queries: dK = dV = 0
  const int n0 = kt * BN;
  if (n0 >= Lk) return;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 31, hf = lane >> 5;
  const int key = n0 + wave * 32 + c;  // this lane's key (sequence-local)

  // ---- K and V fragments of this wave's 32 keys (B operands), registers for the whole kernel (V: LDS with kVLds).
  // Keys past the end are zero: their P is finite, their dK / dV rows are never stored.
  constexpr bool kVLds = Cfg::kVLds;
  // The loads are only issued here; what they bring is looked at after the first tile has been asked for (finish_kv below):
  // a select or an LDS write on a loaded value at this point would hold the first tile back by a global load's latency.
  vec8 kreg[D / 16], vreg[kVLds ? 1 : D / 16];
  u32x4 kraw[D / 16], vraw[kVLds ? BN * CH / 256 : D / 16];
  T* const Vl = reinterpret_cast<T*>(lds_raw + Cfg::kOffV);
  {
    const int kr = key < Lk ? key : Lk - 1;
    const T* kp = reinterpret_cast<const T*>(p.k) + (int64_t)(k_begin + kr) * p.k_rs + (int64_t)h * p.k_hs + hf * 8;
    const T* vp = reinterpret_cast<const T*>(p.v) + (int64_t)(k_begin + kr) * p.v_rs + (int64_t)h * p.v_hs + hf * 8;
#pragma unroll
    for (int ks = 0; ks < D / 16; ks++) {
      kraw[ks] = ld_global16(kp + ks * 16);
      if (!kVLds) vraw[ks] = ld_global16(vp + ks * 16);
    }
    if (kVLds) {
      const T* vt = reinterpret_cast<const T*>(p.v) + (int64_t)k_begin * p.v_rs + (int64_t)h * p.v_hs;
#pragma unroll
      for (int i = 0; i < BN * CH / 256; i++) {
        const int row = (tid + i * 256) / CH, ch = (tid + i * 256) % CH;
        const int vr = n0 + row < Lk ? n0 + row : Lk - 1;
        vraw[i] = ld_global16(vt + (int64_t)vr * p.v_rs + ch * 8);
      }
    }
  }
  auto finish_kv = [&]() {
#pragma unroll
    for (int ks = 0; ks < D / 16; ks++) {
      kreg[ks] = bitcast<vec8>(key < Lk ? kraw[ks] : u32x4{0, 0, 0, 0});
      if (!kVLds) vreg[ks] = bitcast<vec8>(key < Lk ? vraw[ks] : u32x4{0, 0, 0, 0});
    }
    if (kVLds) {  // the first barrier of the main loop orders these writes before the first read
#pragma unroll
      for (int i = 0; i < BN * CH / 256; i++) {
        const int row = (tid + i * 256) / CH, ch = (tid + i * 256) % CH;
        *reinterpret_cast<u32x4*>(Vl + row * Cfg::VS + ch * 8) = n0 + row < Lk ? vraw[i] : u32x4{0, 0, 0, 0};
      }
    }
  };
  const T* const Vfrag = Vl + (wave * 32 + c) * Cfg::VS + hf * 8;  // this lane's V fragments: + 16 * ks elements
  int mt_begin = 0;
  if (kCausal) mt_begin = n0 / BM;  // query rows above the tile's first key see none of its keys
  const int mt_end = (Lq + BM - 1) / BM;

  const float* lsebase = p.lse + ((int64_t)b * p.H + h) * p.lse_stride;
  const float* dsbase = p.dsoftmax + ((int64_t)b * p.H + h) * p.sq_r;

  // ---- staging: Q and dO tiles go global -> LDS directly (waves 0,1: Q, waves 2,3: dO); the 2 x BM row statistics
  // pass through one register of threads 0 .. 2*BM-1 because they are transformed on the way.
  typename Cfg::Stager stager;
  stager.init(wave, lane, reinterpret_cast<const T*>(p.q) + (int64_t)q_begin * p.q_rs + (int64_t)h * p.q_hs, p.q_rs,
              reinterpret_cast<const T*>(p.dout) + (int64_t)q_begin * p.do_rs + (int64_t)h * p.do_hs, p.do_rs);
  // Row statistics of a tile (lse and Dk of its BM rows) wait in a register of threads 0 .. 2*BM-1 and are only
  // converted when the tile is consumed: arithmetic on a loaded value at this point would make the wave wait for the
  // load - and, memory operations completing in order, for everything issued before it - right away.
  float statpre = 0.f;
  // kStored: the keep words of a tile's rows and this wave's 32 keys - one per lane, in the order the masks are needed
  // (fa_common.h) - are fetched with the tile and handed out to the scalar registers by v_readlane, slab by slab.  (Read
  // straight into scalar registers, 128 bytes a slab, they arrive too late: nothing hides a scalar cache miss here.)
  uint32_t kwpre = 0;
  const uint32_t* const kw_wave =
      kStored ? p.keep_words + ((int64_t)bh * p.kw_kb + (n0 >> 5) + wave) * p.kw_q : nullptr;
  // kOwnD: this thread's quarter (16 elements) of row tid / 4 of the tile's dO and O
  u32x4 dopre[kOwnD ? 2 : 1], opre[kOwnD ? 2 : 1];
  const T* const do_quarter = reinterpret_cast<const T*>(p.dout) + (int64_t)q_begin * p.do_rs + (int64_t)h * p.do_hs + (tid & 3) * 16;
  const T* const o_quarter = reinterpret_cast<const T*>(p.out) + (int64_t)q_begin * p.o_rs + (int64_t)h * p.o_hs + (tid & 3) * 16;
  auto stage = [&](int mt, int buf) {
    const int m0 = mt * BM;
    if (tid < BM) {
      const int row = m0 + tid;
      statpre = INFINITY;  // rows past the end are switched off (P = 0)
      if (row < Lq) statpre = lsebase[row];
    } else if (!kOwnD && tid < 2 * BM) {
      const int row = m0 + tid - BM;
      statpre = 0.f;
      if (row < Lq) statpre = dsbase[row];
    }
    if constexpr (kOwnD) {  // (rows past the end read the last row: their P is 0, any finite Dk will do)
      const int row = m0 + (tid >> 2) < Lq ? m0 + (tid >> 2) : Lq - 1;
#pragma unroll
      for (int i = 0; i < 2; i++) {
        dopre[i] = ld_global16(do_quarter + (int64_t)row * p.do_rs + 8 * i);
        opre[i] = ld_global16(o_quarter + (int64_t)row * p.o_rs + 8 * i);
      }
    }
    if (kStored && (BM == 64 || lane < BM)) kwpre = kw_wave[m0 + lane];
    stager.issue(lds_raw + buf * kBufBytes, m0, Lq);
  };
  // lse scaled to base 2, +inf (row off) where the row saw no key; Dk negated: the dP accumulator starts from -Dk
  auto stat_value = [&]() -> float {
    if (tid < BM) return (statpre == -INFINITY) ? INFINITY : statpre * kLog2e;
    return -statpre;
  };
  auto own_dk = [&]() -> float {  // -Dk of row tid / 4, in every thread of its quad; the dQ kernel's order of summation
    float part[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const vec8 dv = bitcast<vec8>(dopre[i]), ov = bitcast<vec8>(opre[i]);
      part[i] = 0.f;
#pragma unroll
      for (int e = 0; e < 8; e++) part[i] = __builtin_fmaf((float)dv[e], (float)ov[e], part[i]);
      part[i] += __uint_as_float(quad_perm<kQuadXor1>(__float_as_uint(part[i])));
      part[i] += __uint_as_float(quad_perm<kQuadXor2>(__float_as_uint(part[i])));
    }
    return -((part[0] + part[1]) * p.p_keep);
  };

  // Sparse: the tiles are not slices of the query side but packed lists of the 16-row blocks that attend this key block
  // (what the reference's converted block list holds per key block, fmha_blockmask.h:41-53): RBT listed blocks make a
  // tile, their rows are gathered when the tile is staged, so no row of an MFMA is masked and no tile is staged for
  // less than RBT active blocks (but the last).  The list is read off the key block's activity bits, 64 row blocks per word.
  struct BlockTile {
    int rb[RBT];  // sequence-local 16-row block indices, ascending; -1 = none (only at the end of the last tile)
  };
  uint64_t word = 0;
  const int nrb_q = (Lq + 15) >> 4;                               // row blocks that hold rows of this sequence
  const int rb_first = kCausal ? (n0 >> 4) : 0;                   // earlier rows see none of this tile's keys
  const int nwords = kSparse ? (((nrb_q < p.sp.nrb ? nrb_q : p.sp.nrb) + 63) >> 6) : 0;
  int wi = (rb_first >> 6) - 1;
  auto next_tile = [&](BlockTile& t) -> bool {  // the next RBT listed blocks; false if there is none
#pragma unroll
    for (int j = 0; j < RBT; j++) {
      while (word == 0 && wi + 1 < nwords) {
        wi = __builtin_amdgcn_readfirstlane(wi + 1);
        word = uniform64(p.sp.cbits[(int64_t)(n0 >> 8) * p.sp.nrw + wi]);
        if (wi * 64 < rb_first) word &= ~uint64_t(0) << (rb_first - wi * 64);        // (only the first word)
        if (nrb_q - wi * 64 < 64) word &= (uint64_t(1) << (nrb_q - wi * 64)) - 1;     // (only the last word)
      }
      t.rb[j] = -1;
      if (word != 0) {
        t.rb[j] = wi * 64 + (int)__builtin_ctzll(word);
        word &= word - 1;
      }
    }
    return t.rb[0] >= 0;
  };
  auto stage_blocks = [&](const BlockTile& t, int buf) {
    if (tid < 2 * BM) {
      const int tr = tid < BM ? tid : tid - BM;
      int blk = -1;
#pragma unroll
      for (int j = 0; j < RBT; j++)
        if ((tr >> 4) == j) blk = t.rb[j];
      const int row = blk * 16 + (tr & 15);
      const bool live = blk >= 0 && row < Lq;
      statpre = tid < BM ? INFINITY : 0.f;  // rows of no block or past the end are switched off (P = 0)
      if (live) statpre = tid < BM ? lsebase[row] : dsbase[row];
    }
    stager.issue_blocks(lds_raw + buf * kBufBytes, t.rb, Lq);
  };

  f32x16 acc_dk[DV / 32], acc_dv[DV / 32];
#pragma unroll
  for (int i = 0; i < DV / 32; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) {
      acc_dk[i][r] = 0.f;
      acc_dv[i][r] = 0.f;
    }

  const float cs = p.scale_log2;
  const float sl2 = kAlibi ? p.alibi[h] * kLog2e : 0.f;  // ALiBi slope in base-2 exponent units (see fa_fwd_kernel)
  // kTensorBias: this lane's column (key) of the bias and of its gradient; row q is q * stride further
  // kTensorBias: the bias of a tile's BM query rows and the wave's 32 keys comes in as whole rows (4 lanes fetch the 64 bytes of a
  // row, 16 bytes each, one tile ahead), is written to a wave-private piece of LDS laid out like a Q tile of 32 columns, and is
  // read back with the transposed reads that give the MFMA's B operand order: register r <-> row 8 (r / 4) + 4 hf + r % 4 of the
  // lane's key, the accumulators' order.  (Read straight from global memory in that order - 16 two-byte loads per slab in front
  // of the MFMAs whose results need them - the kernel took 274 us at the headline shape where it takes 198 us without a bias.)
  // (wave-uniform bases and 32-bit element offsets: a (batch, head) slice holds fewer than 2^31 elements, the front end checks)
  const T* const bias_bh =
      kTensorBias ? reinterpret_cast<const T*>(p.bias) + (int64_t)b * p.bias_bs + (int64_t)h * p.bias_hs : nullptr;
  T* const dbias_bh =
      (kTensorBias && p.dbias) ? reinterpret_cast<T*>(p.dbias) + (int64_t)b * p.dbias_bs + (int64_t)h * p.dbias_hs : nullptr;
  const uint32_t bias_rs = (uint32_t)p.bias_rs, dbias_rs = (uint32_t)p.dbias_rs;
  T* const bias_lds = reinterpret_cast<T*>(lds_raw + Cfg::kLdsBytes + wave * kBiasTileBytes);
  constexpr int kBiasNLD = BM * 4 / 64;  // 16-byte loads per lane and tile
  u32x4 bpre[kTensorBias ? kBiasNLD : 1];
  // (q_first: the tile's first query row; sparse: the packed tile's list of 16-row blocks instead, -1 = no block)
  auto load_bias = [&](int q_first, const int* rb) {
#pragma unroll
    for (int i = 0; i < kBiasNLD; i++) {
      const int k0 = n0 + wave * 32 + (lane & 3) * 8;
      int qr = q_first + i * 16 + (lane >> 2);
      if (kSparse) qr = rb[i] >= 0 ? rb[i] * 16 + (lane >> 2) : Lq;
      bpre[i] = u32x4{0, 0, 0, 0};  // chunks that begin past the last key are not read; rows past the end read the last row
      if (k0 < Lk) bpre[i] = ld_global16(bias_bh + (uint32_t)(qr < Lq ? qr : Lq - 1) * bias_rs + (uint32_t)k0);
    }
  };
  auto bias_to_lds = [&]() {
#pragma unroll
    for (int i = 0; i < kBiasNLD; i++)
      *reinterpret_cast<u32x4*>(bias_lds + frag_off<32, kSwzDual>(i * 16 + (lane >> 2), lane & 3)) = bpre[i];
  };
  const int bt_lo = tr_off<32, kSwzDual>(0, 0, lane), bt_hi = tr_off<32, kSwzDual>(8, 0, lane);
  // element offsets inside a tile of this lane's row fragments and of its transposed reads (rows +0 and +8)
  int foff[D / 16], tlo[DV / 32], thi[DV / 32];
#pragma unroll
  for (int ks = 0; ks < D / 16; ks++) foff[ks] = frag_off<D, kSwzDual>(c, ks * 2 + hf);
#pragma unroll
  for (int db = 0; db < DV / 32; db++) {
    tlo[db] = tr_off<D, kSwzDual>(0, db * 4, lane);
    thi[db] = tr_off<D, kSwzDual>(8, db * 4, lane);
  }
  int buf = 0;

  int mt = mt_begin;          // dense: the query tile in use
  BlockTile tc, tn;           // sparse: the packed tile in use / being staged
  bool more = kSparse ? next_tile(tc) : mt < mt_end;
  if (more) {
    if (kSparse) stage_blocks(tc, 0);
    else stage(mt, 0);
  }
  finish_kv();
  if (kTensorBias && more) load_bias(mt * BM, tc.rb);
  while (more) {
    const int m0 = mt * BM;
    if constexpr ((FA_ABLATE_DKDV & 1) == 0) wait_vmem();  // this thread's share of the tile has arrived (LDS) / is in statpre
    float* const lse_l = reinterpret_cast<float*>(lds_raw + Cfg::kOffStat + buf * Cfg::kStatBytes);
    float* const dk_l = lse_l + BM;
    if constexpr (kOwnD) {
      if (tid < BM) lse_l[tid] = stat_value();
      const float nd = own_dk();
      if ((tid & 3) == 0) dk_l[tid >> 2] = nd;
    } else {
      if (tid < 2 * BM) lse_l[tid] = stat_value();
    }
    const uint32_t kwcur = kwpre;
    if constexpr ((FA_ABLATE_DKDV & 1) == 0) __syncthreads();  // the tile is complete, and nobody still reads the other buffer
    if (kSparse) {
      more = next_tile(tn);
      if (more) stage_blocks(tn, buf ^ 1);
    } else {
      more = mt + 1 < mt_end;
      if (more) stage(mt + 1, buf ^ 1);
    }
    if (kTensorBias) {  // (the wave's own reads of the last tile's values are behind it: LDS operations of a wave stay in order)
      bias_to_lds();
      if (more) load_bias((mt + 1) * BM, tn.rb);
    }
    const T* const Ql = reinterpret_cast<const T*>(lds_raw + buf * kBufBytes);
    const T* const dOl = Ql + BM * D;
    buf ^= 1;


    // LDS fragment fetches sit next to their use; the other waves of the SIMD hide their latency.
    auto load_rows = [&](int qb, vec8* aq, vec8* ad) {
#pragma unroll
      for (int ks = 0; ks < D / 16; ks++) aq[ks] = *reinterpret_cast<const vec8*>(Ql + qb * 32 * D + foff[ks]);
#pragma unroll
      for (int ks = 0; ks < D / 16; ks++) ad[ks] = *reinterpret_cast<const vec8*>(dOl + qb * 32 * D + foff[ks]);
    };
    auto load_tr = [&](int qb, int t, u32x4* avs, u32x4* aqs) {
      const int off = (qb * 32 + 16 * t) * D;
#pragma unroll
      for (int db = 0; db < DV / 32; db++) {
        u32x2 lo = lds_read_tr16(dOl + off + tlo[db]), hi = lds_read_tr16(dOl + off + thi[db]);
        avs[db] = u32x4{lo[0], lo[1], hi[0], hi[1]};
        lo = lds_read_tr16(Ql + off + tlo[db]);
        hi = lds_read_tr16(Ql + off + thi[db]);
        aqs[db] = u32x4{lo[0], lo[1], hi[0], hi[1]};
      }
    };
#pragma unroll
    for (int qb = 0; qb < BM / 32; qb++) {
      // dropout: the two slabs' Philox streams are not to be interleaved by the scheduler (it would, for the sake of
      // instruction-level parallelism, and need 70 more registers: one wave per SIMD fewer)
      if (kDropout || kTensorBias) __builtin_amdgcn_sched_barrier(0);  // (kTensorBias: nor the two slabs' bias loads)
      // first query rows of the slab's two 16-row halves (sparse: of the two listed blocks; ascending)
      const int q_lo = kSparse ? tc.rb[2 * qb] * 16 : m0 + qb * 32;
      const int q_hi = kSparse ? tc.rb[2 * qb + 1] * 16 : q_lo + 16;
      if (kSparse && q_lo < 0) continue;  // the last tile's list ended before this slab
      const bool diag = kCausal && ((kSparse ? q_lo : m0) < n0 + wave * 32 + 32);  // some (q, key) of the wave's has key > q
      // ---- S = Q K^T and dP = dO V^T for 32 query rows x this wave's 32 keys
      // dP starts from -Dk of its query row (fmha_dgrad_kernel_1xN_loop.h:361-371), so the MFMA delivers dP - Dk
      f32x16 s, dp;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const f32x4 nd4 = *reinterpret_cast<const f32x4*>(dk_l + qb * 32 + 8 * j + 4 * hf);
#pragma unroll
        for (int i = 0; i < 4; i++) { s[4 * j + i] = 0.f; dp[4 * j + i] = nd4[i]; }
      }
      // kTensorBias: the bias of this lane's key for the slab's 16 query rows of the lane (register r <-> row
      // 8 (r / 4) + 4 hf + r % 4), asked for before the MFMAs; rows past the end read the last row (their P is 0)
      T braw[kTensorBias ? 16 : 1];
      if (kTensorBias) {
#pragma unroll
        for (int t = 0; t < 2; t++) {
          const T* bp = bias_lds + (qb * 32 + 16 * t) * 32;
          const u32x2 lo = lds_read_tr16(bp + bt_lo), hi = lds_read_tr16(bp + bt_hi);
          const vec8 bv = bitcast<vec8>(u32x4{lo[0], lo[1], hi[0], hi[1]});
#pragma unroll
          for (int i = 0; i < 8; i++) braw[8 * t + i] = bv[i];
        }
      }
      vec8 aq[D / 16], ad[D / 16];
      load_rows(qb, aq, ad);
      if constexpr ((FA_ABLATE_DKDV & 8) == 0) {
#pragma unroll
        for (int ks = 0; ks < D / 16; ks++) s = E::mfma32(aq[ks], kreg[ks], s);
#pragma unroll
        for (int ks = 0; ks < D / 16; ks++)
          dp = E::mfma32(ad[ks], kVLds ? *reinterpret_cast<const vec8*>(Vfrag + ks * 16) : vreg[ks], dp);
      } else {
#pragma unroll
        for (int ks = 0; ks < D / 16; ks++) { s[ks] += (float)aq[ks][0] * (float)kreg[ks][0]; dp[ks] += (float)ad[ks][0]; }
      }
      // ---- P and dS'
      KeepFields keep;
      if (kDropout) {  // this lane draws micro-block 2 (key % 4) + hf of the slab's eight (four query rows each)
        const int mb = 2 * (key & 3) + hf;
        keep = keep_fields_col_layout_q4(p.pk, (uint32_t)bh, (uint32_t)((mb < 4 ? q_lo : q_hi) >> 2) + (mb & 3), key);
      }
      // -Dk is read a second time where a dropped element needs it; the opaque zero keeps the compiler from holding
      // the 16 values it read for the accumulator's start in registers until then instead
      int again = 0;
      if (kStored) asm volatile("" : "+s"(again));
      if (kCausal && diag) {  // only slabs that straddle the diagonal: scores above it become -inf (P = 0)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int qrow = kSparse ? (r < 8 ? q_lo : q_hi) + 8 * ((r >> 2) & 1) + 4 * hf + (r & 3)
                                   : q_lo + 8 * (r >> 2) + 4 * hf + (r & 3);
          if (key > qrow) s[r] = -INFINITY;
        }
      }
      uint64_t km[16];  // kStored: the keep mask of register r over the wave's 64 lanes
      if (kStored) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)kwcur, (qb * 32 + 2 * r) & 63);
          const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)kwcur, (qb * 32 + 2 * r + 1) & 63);
          km[r] = ((uint64_t)hi << 32) | lo;
        }
      }
      // kAlibi: key - query of register 0, and (sparse: the slab's second row block is any later one) of register 8 plus 16
      const float dbase = kSparse ? (float)(key - q_lo - 4 * hf) : (float)(key - m0 - qb * 32 - 4 * hf);
      const float dbase_hi = kSparse ? (float)(key - q_hi + 16 - 4 * hf) : dbase;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const f32x4 lse4 = *reinterpret_cast<const f32x4*>(lse_l + qb * 32 + 8 * j + 4 * hf);
        f32x4 nd4 = {0.f, 0.f, 0.f, 0.f};
        if (kDrop != 0) nd4 = *reinterpret_cast<const f32x4*>(dk_l + again + qb * 32 + 8 * j + 4 * hf);
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const int r = 4 * j + i;
          float e = -lse4[i];
          if (kAlibi) e = __builtin_fmaf(__builtin_fabsf((j < 2 ? dbase : dbase_hi) - (float)(8 * j + i)), -sl2, -lse4[i]);
          if (kTensorBias) e = __builtin_fmaf((float)braw[r], kLog2e, -lse4[i]);
          const float pe = (FA_ABLATE_DKDV & 2) ? __builtin_fmaf(s[r], cs, e) * 1e-3f : fast_exp2(__builtin_fmaf(s[r], cs, e));
          float dpe = dp[r];  // dP - Dk
          float pm = pe;
          if (kDropout && !keep.keep_col(r, p.keep_thr)) { dpe = nd4[i]; pm = 0.f; }  // dropped: M o dP = 0
          if (kStored && !lane_bit(km[r])) { dpe = nd4[i]; pm = 0.f; }
          s[r] = pm;          // P o M, feeds dV
          dp[r] = pe * dpe;   // dS' = P o (M o dP - Dk), feeds dK
        }
      }
      if (kTensorBias && dbias_bh != nullptr && key < Lk) {  // d(loss)/d(bias) = dS = dS' / keep
        const uint32_t q0 = (uint32_t)(q_lo + 4 * hf), q8 = (uint32_t)(q_hi - 16 + 4 * hf);  // (dense: q8 == q0)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const uint32_t qr = (kSparse && r >= 8 ? q8 : q0) + 8 * (r >> 2) + (r & 3);
          if (qr < (uint32_t)Lq) dbias_bh[qr * dbias_rs + (uint32_t)key] = (T)(dp[r] * p.rp_keep);
        }
      }
      // ---- dV^T += dO^T P; dK^T += Q^T dS'
#pragma unroll
      for (int t = 0; t < 2; t++) {
        f32x8 pf, df;
#pragma unroll
        for (int i = 0; i < 8; i++) { pf[i] = s[8 * t + i]; df[i] = dp[8 * t + i]; }
        const vec8 pb = cvt8<T>(pf);
        const vec8 db8 = cvt8<T>(df);
        u32x4 avs[DV / 32], aqs[DV / 32];
        load_tr(qb, t, avs, aqs);
#pragma unroll
        for (int db = 0; db < DV / 32; db++) {
          if constexpr ((FA_ABLATE_DKDV & 4) == 0) {
            acc_dv[db] = E::mfma32(bitcast<vec8>(avs[db]), pb, acc_dv[db]);
            acc_dk[db] = E::mfma32(bitcast<vec8>(aqs[db]), db8, acc_dk[db]);
          } else {
            asm volatile("" ::"v"(avs[db]), "v"(aqs[db]), "v"(pb), "v"(db8));
          }
        }
      }
    }
    if (kSparse) tc = tn;
    else mt++;
  }

  // ---- rotary: k came in rotated; dk goes out turned back by the angles of this lane's key (linear, so it can precede the
  // scaling), in fp32 before its one rounding
  if constexpr (kRot) {
    const int krow = n0 + wave * 32 + (int)(threadIdx.x & 31);
    const int t = krow < p.rot_rows ? krow : p.rot_rows - 1;
#pragma unroll
    for (int db = 0; db < DV / 32; db++)
#pragma unroll
      for (int g4 = 0; g4 < 4; g4++) {
        const int d0 = db * 32 + g4 * 8 + (int)(threadIdx.x >> 5 & 1) * 4;
        if (d0 < D) {
          f32x4 x;
#pragma unroll
          for (int i = 0; i < 4; i++) x[i] = acc_dk[db][g4 * 4 + i];
          x = unrotate4<T>(x, p.rot_cos, p.rot_sin, t, D / 2, d0);
#pragma unroll
          for (int i = 0; i < 4; i++) acc_dk[db][g4 * 4 + i] = x[i];
        }
      }
  }

  // ---- epilogue: scale, transpose dK^T / dV^T through LDS, coalesced stores
  __syncthreads();
  constexpr int ES = D + 8;
  T* Stg = reinterpret_cast<T*>(lds_raw) + wave * 32 * ES;  // 32 keys x D per wave
  const float fv = p.rp_keep, fk = p.scale * p.rp_keep;
#pragma unroll
  for (int which = 0; which < 2; which++) {
#pragma unroll
    for (int db = 0; db < DV / 32; db++)
#pragma unroll
      for (int g4 = 0; g4 < 4; g4++) {
        const int d0 = db * 32 + g4 * 8 + hf * 4;
        if (d0 < D) {
          f32x4 x;
#pragma unroll
          for (int i = 0; i < 4; i++)
            x[i] = which == 0 ? acc_dk[db][g4 * 4 + i] * fk : acc_dv[db][g4 * 4 + i] * fv;
          *reinterpret_cast<vec4*>(Stg + c * ES + d0) = cvt4<T>(x);
        }
      }
    __builtin_amdgcn_wave_barrier();
    T* gbase = which == 0
                   ? reinterpret_cast<T*>(p.dk) + (int64_t)k_begin * p.dk_rs + (int64_t)h * p.dk_hs
                   : reinterpret_cast<T*>(p.dv) + (int64_t)k_begin * p.dv_rs + (int64_t)h * p.dv_hs;
    const int64_t grs = which == 0 ? p.dk_rs : p.dv_rs;
#pragma unroll
    for (int i = 0; i < (32 * CH + 63) / 64; i++) {
      const int ch = lane + i * 64;
      const int row = ch / CH, col = (ch % CH) * 8;
      const int krow = n0 + wave * 32 + row;
      if ((32 * CH % 64 == 0 || ch < 32 * CH) && krow < Lk) {
        u32x4 val = *reinterpret_cast<const u32x4*>(Stg + row * ES + col);
        st_global16(gbase + (int64_t)krow * grs + col, val);
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
}

template <typename T, int D, bool kCausal, int kDrop, bool kSparse, int kBias = 0, bool kRot = false>
__global__ void __launch_bounds__(256, (kDrop == 0 && D <= 64 && kBias != kBiasTensor) ? 3 : ((D == 128 && kBias == kBiasTensor) ? 1 : BwdCfg<T, D, kDrop == 1>::kMinBlocks)) fa_bwd_dkdv_kernel(const BwdParams p) {
  using Cfg = BwdCfg<T, D, kDrop == 1>;
  __shared__ __attribute__((aligned(16))) unsigned char lds_raw[Cfg::kLdsBytes + (kBias == kBiasTensor ? 4 * Cfg::kBiasTileBytes : 0)];
  fa_bwd_dkdv_body<T, D, kCausal, kDrop, kSparse, kBias, kRot>(p, blockIdx.x, lds_raw);
}

// ---------------------------------------------------------------------------------------------------------------
// dK, dV at head dim 128 without dropout, mask layout or score bias: wave pairs
// ---------------------------------------------------------------------------------------------------------------
// At d = 128 one wave cannot hold K, V and both accumulators of 32 keys next to the scores at more than two waves per SIMD
// (fa_bwd_dkdv_kernel keeps its V tile in LDS for that reason and reads every V fragment from there).  Here two waves share
// 32 keys: the first holds the K fragments, forms S = Q K^T and P and owns dV^T += dO^T P; the second holds the V
// fragments, forms dP - D = dO V^T - D, takes P from the first through LDS (rounded to the element type, as dV's MFMA
// takes it; the accumulator layout on both sides: a straight copy), forms dS' = P o (dP - D) and owns dK^T += Q^T dS'.
// Each wave then needs one operand's fragments and one accumulator: three waves per SIMD, and no V fragment is read from
// LDS.  The second wave runs one 32-row slab behind the first, so that it never waits for its partner inside a step: in
// step i it finishes slab i - 1 (P from LDS, Q^T of slab i - 1: the Q tile has three buffers, dO two) and then starts
// slab i.  A workgroup is two pairs (64 keys); a step is one 32-row slab of Q and dO and has one barrier.
struct PairCfg {
  static constexpr int D = 128, BM = 32, BN = 64, CH = D / 8;
  typedef TilePairStager<D, BM, kSwzDual, kSwzDual> Stager;
  static constexpr int kTile = Stager::kTileBytes;        // one 32 x 128 tile
  static constexpr int kOffQ = 0;                         // three Q tiles
  static constexpr int kOffdO = 3 * kTile;                // two dO tiles
  static constexpr int kOffStat = 5 * kTile;
  static constexpr int kStatBytes = 2 * BM * 4;           // lse[BM], -Dk[BM]
  static constexpr int kOffP = kOffStat + 2 * kStatBytes;
  static constexpr int kPBytes = 2 * 64 * 16;             // one pair's P of one slab: 2 x 64 lanes x 8 elements
  static constexpr int kTileBytes = kOffP + 4 * kPBytes;  // two pairs, two slabs in flight
  static constexpr int ES = D + 8;
  static constexpr int kEpiBytes = 4 * 32 * ES * 2;
  static constexpr int kLdsBytes = kTileBytes > kEpiBytes ? kTileBytes : kEpiBytes;
};

template <typename T, bool kCausal, bool kRot>
__global__ void __launch_bounds__(256, 3) fa_bwd_dkdv_pair_kernel(const BwdParams p) {
  using Cfg = PairCfg;
  using E = Elem<T>;
  using vec8 = typename E::vec8;
  using vec4 = typename E::vec4;
  constexpr int D = Cfg::D, BM = Cfg::BM, BN = Cfg::BN, CH = Cfg::CH;
  __shared__ __attribute__((aligned(16))) unsigned char lds_raw[Cfg::kLdsBytes];

  int bh, kt;
  if (!map_tile<kCausal>(blockIdx.x, p.nk_tiles, p.B * p.H, &bh, &kt, p.tile_group)) return;
  const int b = bh / p.H, h = bh % p.H;
  int q_begin = 0, Lq = 0, k_begin, Lk;
  if (!seq_extent(p.cu_k, b, p.total_k, p.max_sk, &k_begin, &Lk)) return;
  if (!seq_extent(p.cu_q, b, p.total_q, p.max_sq, &q_begin, &Lq)) Lq = 0;  // no queries: dK = dV = 0
  const int n0 = kt * BN;
  if (n0 >= Lk) return;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int pr = wave >> 1;        // the pair, i.e. which 32 of the workgroup's 64 keys
  const bool second = wave & 1;    // false: S, P, dV;  true: dP, dS', dK
  const int c = lane & 31, hf = lane >> 5;
  const int key = n0 + pr * 32 + c;  // this lane's key (sequence-local)

  // ---- this wave's B operand: the K (first wave) or V (second wave) fragments of the pair's 32 keys; keys past the end
  // are zero.  Issued here, looked at after the first tile has been asked for.
  vec8 breg[D / 16];
  u32x4 braw[D / 16];
  {
    const int kr = key < Lk ? key : Lk - 1;
    const T* bp = second ? reinterpret_cast<const T*>(p.v) + (int64_t)(k_begin + kr) * p.v_rs + (int64_t)h * p.v_hs
                         : reinterpret_cast<const T*>(p.k) + (int64_t)(k_begin + kr) * p.k_rs + (int64_t)h * p.k_hs;
#pragma unroll
    for (int ks = 0; ks < D / 16; ks++) braw[ks] = ld_global16(bp + hf * 8 + ks * 16);
  }
  const int mt_begin = kCausal ? n0 / BM : 0;  // query rows above the tile's first key see none of its keys
  const int mt_end = (Lq + BM - 1) / BM;
  const int n_slabs = mt_end > mt_begin ? mt_end - mt_begin : 0;
  const float* lsebase = p.lse + ((int64_t)b * p.H + h) * p.lse_stride;
  const float* dsbase = p.dsoftmax + ((int64_t)b * p.H + h) * p.sq_r;

  typename Cfg::Stager stager;
  stager.init(wave, lane, reinterpret_cast<const T*>(p.q) + (int64_t)q_begin * p.q_rs + (int64_t)h * p.q_hs, p.q_rs,
              reinterpret_cast<const T*>(p.dout) + (int64_t)q_begin * p.do_rs + (int64_t)h * p.do_hs, p.do_rs);
  float statpre = 0.f;  // a slab's lse (threads 0 .. BM-1) and Dk (BM .. 2 BM-1), converted when the slab is consumed
  // q3 / d2: which of the three Q and of the two dO buffers the slab goes to (the stager adds one tile's size for the waves
  // that fetch the second tensor)
  auto stage = [&](int m0, int q3, int d2) {
    if (tid < BM) {
      statpre = INFINITY;  // rows past the end are switched off (P = 0)
      if (m0 + tid < Lq) statpre = lsebase[m0 + tid];
    } else if (tid < 2 * BM) {
      statpre = 0.f;
      if (m0 + tid - BM < Lq) statpre = dsbase[m0 + tid - BM];
    }
    stager.issue(lds_raw + (stager.second ? Cfg::kOffdO + (d2 - 1) * Cfg::kTile : Cfg::kOffQ + q3 * Cfg::kTile), m0, Lq);
  };
  auto stat_value = [&]() -> float {
    if (tid < BM) return (statpre == -INFINITY) ? INFINITY : statpre * kLog2e;
    return -statpre;
  };

  f32x16 acc[D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[i][r] = 0.f;
  const float cs = p.scale_log2;
  int foff[D / 16], tlo[D / 32], thi[D / 32];
#pragma unroll
  for (int ks = 0; ks < D / 16; ks++) foff[ks] = frag_off<D, kSwzDual>(c, ks * 2 + hf);
#pragma unroll
  for (int db = 0; db < D / 32; db++) {
    tlo[db] = tr_off<D, kSwzDual>(0, db * 4, lane);
    thi[db] = tr_off<D, kSwzDual>(8, db * 4, lane);
  }
  // P of a slab: [slab parity][pair][half t][lane] x 16 bytes
  u32x4* const Pl = reinterpret_cast<u32x4*>(lds_raw + Cfg::kOffP + pr * Cfg::kPBytes) + lane;

  if (n_slabs > 0) stage(mt_begin * BM, 0, 0);
#pragma unroll
  for (int ks = 0; ks < D / 16; ks++) breg[ks] = bitcast<vec8>(key < Lk ? braw[ks] : u32x4{0, 0, 0, 0});

  f32x16 x;  // first wave: S, then P of the slab;  second wave: dP - Dk of the slab it has started
  auto accumulate = [&](const T* cols, vec8 x0, vec8 x1) {  // acc += cols^T (x0 | x1)
#pragma unroll
    for (int t = 0; t < 2; t++) {
      u32x4 at[D / 32];
#pragma unroll
      for (int db = 0; db < D / 32; db++) {
        const u32x2 lo = lds_read_tr16(cols + 16 * t * D + tlo[db]), hi = lds_read_tr16(cols + 16 * t * D + thi[db]);
        at[db] = u32x4{lo[0], lo[1], hi[0], hi[1]};
      }
#pragma unroll
      for (int db = 0; db < D / 32; db++) acc[db] = E::mfma32(bitcast<vec8>(at[db]), t == 0 ? x0 : x1, acc[db]);
    }
  };
  int q3 = 0, d2 = 0;  // buffers of slab i
  for (int i = 0; i <= n_slabs; i++) {  // (the last round only lets the second waves finish the last slab)
    if (n_slabs == 0) break;
    const bool cur = i < n_slabs;
    const int m0 = (mt_begin + i) * BM;
    wait_vmem();
    float* const lse_l = reinterpret_cast<float*>(lds_raw + Cfg::kOffStat + d2 * Cfg::kStatBytes);
    float* const dk_l = lse_l + BM;
    if (cur && tid < 2 * BM) lse_l[tid] = stat_value();
    __syncthreads();  // slab i is complete, P of slab i - 1 is there, nobody still reads what slab i + 1 will overwrite
    const int q3n = q3 == 2 ? 0 : q3 + 1, q3p = q3 == 0 ? 2 : q3 - 1;
    if (i + 1 < n_slabs) stage(m0 + BM, q3n, d2 ^ 1);
    const T* const Ql = reinterpret_cast<const T*>(lds_raw + Cfg::kOffQ + q3 * Cfg::kTile);
    const T* const dOl = reinterpret_cast<const T*>(lds_raw + Cfg::kOffdO + d2 * Cfg::kTile);

    if (second && i > 0) {  // ---- finish slab i - 1: dS' = P o (dP - Dk), dK^T += Q^T dS'
      const vec8 p0 = bitcast<vec8>(Pl[(d2 ^ 1) * (2 * Cfg::kPBytes / 16)]);
      const vec8 p1 = bitcast<vec8>(Pl[(d2 ^ 1) * (2 * Cfg::kPBytes / 16) + 64]);
      f32x8 d0, d1;
#pragma unroll
      for (int e = 0; e < 8; e++) {
        d0[e] = (float)p0[e] * x[e];
        d1[e] = (float)p1[e] * x[8 + e];
      }
      accumulate(reinterpret_cast<const T*>(lds_raw + Cfg::kOffQ + q3p * Cfg::kTile), cvt8<T>(d0), cvt8<T>(d1));
    }
    if (cur) {
      // ---- S = Q K^T (first wave) or dP - Dk = dO V^T - Dk (second wave: the accumulator starts from -Dk of its rows)
#pragma unroll
      for (int j = 0; j < 4; j++) {
        f32x4 nd4 = {0.f, 0.f, 0.f, 0.f};
        if (second) nd4 = *reinterpret_cast<const f32x4*>(dk_l + 8 * j + 4 * hf);
#pragma unroll
        for (int e = 0; e < 4; e++) x[4 * j + e] = nd4[e];
      }
      {
        const T* const rows = second ? dOl : Ql;
        vec8 a[D / 16];
#pragma unroll
        for (int ks = 0; ks < D / 16; ks++) a[ks] = *reinterpret_cast<const vec8*>(rows + foff[ks]);
#pragma unroll
        for (int ks = 0; ks < D / 16; ks++) x = E::mfma32(a[ks], breg[ks], x);
      }
      if (!second) {  // ---- P, left for the partner; dV^T += dO^T P
        if (kCausal && m0 < n0 + pr * 32 + 32) {  // the slab straddles the diagonal: scores above it become -inf (P = 0)
#pragma unroll
          for (int r = 0; r < 16; r++)
            if (key > m0 + 8 * (r >> 2) + 4 * hf + (r & 3)) x[r] = -INFINITY;
        }
        f32x8 pf0, pf1;
#pragma unroll
        for (int j = 0; j < 4; j++) {
          const f32x4 lse4 = *reinterpret_cast<const f32x4*>(lse_l + 8 * j + 4 * hf);
#pragma unroll
          for (int e = 0; e < 4; e++) {
            const float pe = fast_exp2(__builtin_fmaf(x[4 * j + e], cs, -lse4[e]));
            if (j < 2) pf0[4 * j + e] = pe;
            else pf1[4 * (j - 2) + e] = pe;
          }
        }
        const vec8 p0 = cvt8<T>(pf0), p1 = cvt8<T>(pf1);
        Pl[d2 * (2 * Cfg::kPBytes / 16)] = bitcast<u32x4>(p0);
        Pl[d2 * (2 * Cfg::kPBytes / 16) + 64] = bitcast<u32x4>(p1);
        accumulate(dOl, p0, p1);
      }
    }
    q3 = q3n;
    d2 ^= 1;
  }

  // ---- rotary: k came in rotated; dk goes out turned back by the angles of this lane's key, in fp32 before its rounding
  if constexpr (kRot) {
    if (second) {
      const int t = key < p.rot_rows ? key : p.rot_rows - 1;
#pragma unroll
      for (int db = 0; db < D / 32; db++)
#pragma unroll
        for (int g4 = 0; g4 < 4; g4++) {
          f32x4 xr;
#pragma unroll
          for (int i = 0; i < 4; i++) xr[i] = acc[db][g4 * 4 + i];
          xr = unrotate4<T>(xr, p.rot_cos, p.rot_sin, t, D / 2, db * 32 + g4 * 8 + hf * 4);
#pragma unroll
          for (int i = 0; i < 4; i++) acc[db][g4 * 4 + i] = xr[i];
        }
    }
  }

  // ---- epilogue: scale, transpose this wave's dV^T or dK^T through LDS, coalesced stores
  __syncthreads();
  constexpr int ES = Cfg::ES;
  T* Stg = reinterpret_cast<T*>(lds_raw) + wave * 32 * ES;  // 32 keys x D per wave
  const float f = second ? p.scale * p.rp_keep : p.rp_keep;
#pragma unroll
  for (int db = 0; db < D / 32; db++)
#pragma unroll
    for (int g4 = 0; g4 < 4; g4++) {
      f32x4 xo;
#pragma unroll
      for (int i = 0; i < 4; i++) xo[i] = acc[db][g4 * 4 + i] * f;
      *reinterpret_cast<vec4*>(Stg + c * ES + db * 32 + g4 * 8 + hf * 4) = cvt4<T>(xo);
    }
  __builtin_amdgcn_wave_barrier();
  T* const gbase = second ? reinterpret_cast<T*>(p.dk) + (int64_t)k_begin * p.dk_rs + (int64_t)h * p.dk_hs
                          : reinterpret_cast<T*>(p.dv) + (int64_t)k_begin * p.dv_rs + (int64_t)h * p.dv_hs;
  const int64_t grs = second ? p.dk_rs : p.dv_rs;
#pragma unroll
  for (int i = 0; i < 32 * CH / 64; i++) {
    const int ch = lane + i * 64;
    const int row = ch / CH, col = (ch % CH) * 8;
    const int krow = n0 + pr * 32 + row;
    if (krow < Lk) st_global16(gbase + (int64_t)krow * grs + col, *reinterpret_cast<const u32x4*>(Stg + row * ES + col));
  }
}

// ---------------------------------------------------------------------------------------------------------------
// dQ
// ---------------------------------------------------------------------------------------------------------------
// KS: key split as in the forward kernel (FwdCfg): 1 = four waves with 32 of the workgroup's 128 query rows each;
// 2 = 64 query rows, the waves w and w + 2 share 32 rows, split every key tile's two 32-key blocks between them and add
// up their partial dQ in the epilogue.
template <typename T, int D, int BN, int KS = 1>
struct DqCfg {
  static constexpr int BM = kFwdBM / KS;  // query rows per workgroup (KS = 1: the forward's tiling, shares its sparse map)
  static constexpr int RW = 4 / KS;       // 32-row slabs per workgroup
  static constexpr int KBW = BN / 32 / KS;  // 32-key blocks of a tile per wave
  static_assert(KS == 1 || (KS == 2 && BN == 64), "key split: two waves per 32 rows, one 32-key block each");
  static constexpr int DV = D < 32 ? 32 : D;
  static constexpr int OS = D + 8;
  // K tile (read as row fragments and transposed) followed by V tile (row fragments), double buffered (fa_stage.h)
  typedef TilePairStager<D, BN, kSwzDual, kSwzRow> Stager;
  static constexpr int kBufBytes = Stager::kPairBytes;
  static constexpr int kSlack = D < 32 ? 64 : 0;  // the 32-wide transposed reads run past a 16-wide K row
  static constexpr int kTileBytes = 2 * kBufBytes + kSlack;
  static constexpr int kEpiBytes = BM * OS * 2;
  static constexpr int kMergeBytes = KS > 1 ? RW * (DV / 32 * 16) * 64 * 4 : 0;  // partial dQ of RW waves
  static constexpr int kLdsBytes0 = kTileBytes > kEpiBytes ? kTileBytes : kEpiBytes;
  static constexpr int kLdsBytes = kLdsBytes0 > kMergeBytes ? kLdsBytes0 : kMergeBytes;
  static constexpr int CH = D / 8;
  static constexpr int kBiasWaveBytes = 32 * (BN * 2 + 8);  // per wave, behind the tiles: the bias-tensor variants' rows
};

// kDrop: as in fa_bwd_dkdv_kernel
// (the kernel proper is fa_bwd_dq_kernel below: `block` is its workgroup id, `lds_raw` its LDS)
template <typename T, int D, int BN, bool kCausal, int kDrop, bool kSparse, int kBias = 0, int KS = 1>
FA_DEVICE void fa_bwd_dq_body(const BwdParams& p, const int block, unsigned char* const lds_raw) {
  constexpr bool kDropout = kDrop == 1, kStored = kDrop == 2;
  constexpr bool kAlibi = kBias == kBiasAlibi, kTensorBias = kBias == kBiasTensor;
  static_assert(!(kStored && kSparse), "keep words: dense only");
  constexpr bool kRotCapable = !kSparse && kBias == 0;  // rotary (p.rot_cos): dense variants without score bias
  using Cfg = DqCfg<T, D, BN, KS>;
  using E = Elem<T>;
  using vec8 = typename E::vec8;
  constexpr int BM = Cfg::BM, DV = Cfg::DV, CH = Cfg::CH, kBufBytes = Cfg::kBufBytes, KBW = Cfg::KBW;
  static_assert(KS == 1 || !kSparse, "the block-sparse maps are built for 128-row query tiles");

  // kTensorBias: behind the tiles, per wave 32 rows x BN keys of bias, rows padded by 8 bytes (as in fa_fwd_kernel)
  constexpr int kBiasRowBytes = BN * 2 + 8, kBiasWaveBytes = 32 * kBiasRowBytes;
  static_assert(kBiasWaveBytes == Cfg::kBiasWaveBytes, "LDS size of the kernel");

  int bh, rank;
  const int n_splits = p.n_splits > 1 ? p.n_splits : 1;  // key splits per query tile (see BwdParams)
  if (!map_tile<kCausal>(block, p.nq_tiles * n_splits, p.B * p.H, &bh, &rank, p.tile_group)) return;
  const int split = rank % n_splits;
  rank /= n_splits;
  const int qt = kCausal ? p.nq_tiles - 1 - rank : rank;
  const int h = bh % p.H;
  // (dense, no mask: the batch entries are taken longest keys first, see longest_first)
  const int b = (!kCausal && !kSparse && p.tile_group < 0) ? longest_first(p.cu_k, p.B, bh / p.H) : bh / p.H;
  bh = b * p.H + h;  // (what the dropout counters and the keep words are indexed by)

  int q_begin, Lq, k_begin = 0, Lk = 0;
  if (!seq_extent(p.cu_q, b, p.total_q, p.max_sq, &q_begin, &Lq)) return;
  if (!seq_extent(p.cu_k, b, p.total_k, p.max_sk, &k_begin, &Lk)) Lk = 0;  // no keys: dQ = 0
  const int m0 = qt * BM;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 31, hf = lane >> 5;
  const int rs = KS > 1 ? wave % Cfg::RW : wave;  // this wave's 32-row slab of the tile
  const int kh = KS > 1 ? wave / Cfg::RW : 0;     // ... and its share of every key tile's 32-key blocks
  const int mw = m0 + rs * 32;
  int qrow = mw + c;
  // Sparse: the wave's 32 rows are two 16-row blocks, consecutive ones or two that the row order puts next to each other
  // (as in fa_fwd_kernel); rows of no block count as lying past the end
  int rb_a = -1, rb_b = -1;
  bool wave_live = mw < Lq;
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

  // ---- Q and dO fragments (B operands), lse and Dk of this lane's query row.  Dk = keep * rowsum(dO o O) is computed
  // here (fmha_dgrad_kernel_1xN_loop.h:15-30 does it on the first column block) and stored to softmax_d, which the
  // dK/dV kernel, launched after this one, reads.
  // The loads are only issued here; what they bring is looked at after the first key tile has been asked for (below):
  // arithmetic on a loaded value at this point would hold that tile back by a global load's latency.
  vec8 qreg[D / 16], doreg[D / 16];
  u32x4 qraw[D / 16], doraw[D / 16], oraw[D / 16];
  float lse_raw = 0.f;
  {
    const int qr = qrow < Lq ? qrow : Lq - 1;
    const T* qp = reinterpret_cast<const T*>(p.q) + (int64_t)(q_begin + qr) * p.q_rs + (int64_t)h * p.q_hs + hf * 8;
    const T* dp_ = reinterpret_cast<const T*>(p.dout) + (int64_t)(q_begin + qr) * p.do_rs + (int64_t)h * p.do_hs + hf * 8;
    const T* op = reinterpret_cast<const T*>(p.out) + (int64_t)(q_begin + qr) * p.o_rs + (int64_t)h * p.o_hs + hf * 8;
#pragma unroll
    for (int ks = 0; ks < D / 16; ks++) {
      qraw[ks] = ld_global16(qp + ks * 16);
      doraw[ks] = ld_global16(dp_ + ks * 16);
      oraw[ks] = ld_global16(op + ks * 16);
    }
    lse_raw = p.lse[((int64_t)b * p.H + h) * p.lse_stride + qr];
  }
  // For d <= 64 the dP^T accumulator starts from -Dk of this lane's query row (16 registers that save 16 subtractions
  // per 32x32 tile); at d = 128 those registers would push the kernel below two waves per SIMD.
  constexpr bool kInitNegD = D <= 64 || !kDropout;
  f32x16 negd;
  float lse2 = INFINITY, dkv = 0.f;  // +inf switches the row off
  int n_end = Lk;
  if (kCausal) n_end = n_end < m0 + BM ? n_end : m0 + BM;
  const int ntiles_all = (n_end + BN - 1) / BN;
  const int tile0 = (int)((int64_t)split * ntiles_all / n_splits);  // this workgroup's share of the key tiles
  const int ntiles = (int)((int64_t)(split + 1) * ntiles_all / n_splits);

  // ---- K/V staging: global -> LDS without passing through registers (waves 0,1 fetch K tiles, waves 2,3 V tiles).
  // Keys past the end re-read the last key: their P is masked to 0 below, so they add 0 * finite to dQ.
  typename Cfg::Stager stager;
  stager.init(wave, lane, reinterpret_cast<const T*>(p.k) + (int64_t)k_begin * p.k_rs + (int64_t)h * p.k_hs, p.k_rs,
              reinterpret_cast<const T*>(p.v) + (int64_t)k_begin * p.v_rs + (int64_t)h * p.v_hs, p.v_rs);
  // kStored: the keep words of this lane's query row for the wave's 32-key blocks of a tile travel with the tile
  uint32_t kwpre[KBW];
  const uint32_t* const kw_row =
      kStored ? p.keep_words + ((int64_t)bh * p.kw_kb + kh * KBW) * p.kw_q + mw + (keep_word_slot(c) & 31) : nullptr;
  auto stage = [&](int it, int buf) {
    if (kStored) {
#pragma unroll
      for (int kbi = 0; kbi < KBW; kbi++) kwpre[kbi] = kw_row[(int64_t)(it * (BN / 32) + kbi) * p.kw_q];
    }
    stager.issue(lds_raw + buf * kBufBytes, it * BN, Lk);
  };

  // Sparse: the tile's and this lane's row block's activity bits of 64 consecutive key blocks sit in registers
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

  f32x16 acc[DV / 32];
#pragma unroll
  for (int i = 0; i < DV / 32; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[i][r] = 0.f;

  const float cs = p.scale_log2;
  const float sl2 = kAlibi ? p.alibi[h] * kLog2e : 0.f;  // ALiBi slope in base-2 exponent units (see fa_fwd_kernel)
  // kTensorBias: as in the forward kernel - whole rows of the wave's 32 x BN bias values fetched 16 bytes a lane one tile ahead,
  // turned into the MFMA layout through a wave-private piece of LDS
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
  // element offsets inside a tile: row fragments of K (dual swizzle) and V, transposed reads of K (rows +0, +8)
  int kfoff[D / 16], vfoff[D / 16], tlo[DV / 32], thi[DV / 32];
#pragma unroll
  for (int ks = 0; ks < D / 16; ks++) {
    kfoff[ks] = frag_off<D, kSwzDual>(c, ks * 2 + hf);
    vfoff[ks] = frag_off<D, kSwzRow>(c, ks * 2 + hf);
  }
#pragma unroll
  for (int db = 0; db < DV / 32; db++) {
    tlo[db] = tr_off<D, kSwzDual>(0, db * 4, lane);
    thi[db] = tr_off<D, kSwzDual>(8, db * 4, lane);
  }
  int buf = 0;

  int it = next_active(tile0);
  bool row_on_cur = row_on_next;
  if (it < ntiles) {
    stage(it, 0);
    if (kTensorBias) load_bias(it);
  }
  // ---- now the fragments: rows past the end are zero; Dk and -Dk, lse in base-2 units (+inf switches a row off)
  {
    // (summed as the dK/dV kernel's own_dk sums it - eight elements in a chain, the chains pairwise - so that both give the same bits)
    float dpart[D / 16];
#pragma unroll
    for (int ks = 0; ks < D / 16; ks++) {
      const vec8 ov = bitcast<vec8>(oraw[ks]);
      qreg[ks] = bitcast<vec8>(qrow < Lq ? qraw[ks] : u32x4{0, 0, 0, 0});
      doreg[ks] = bitcast<vec8>(qrow < Lq ? doraw[ks] : u32x4{0, 0, 0, 0});
      dpart[ks] = 0.f;
#pragma unroll
      for (int i = 0; i < 8; i++) dpart[ks] = __builtin_fmaf((float)doreg[ks][i], (float)ov[i], dpart[ks]);
    }
#pragma unroll
    for (int step = 1; step < D / 16; step *= 2)
#pragma unroll
      for (int ks = 0; ks + step < D / 16; ks += 2 * step) dpart[ks] += dpart[ks + step];
    float dsum = half_sum(dpart[0]) * p.p_keep;  // lanes l and l^32 hold the two halves of each 16-element group of the row
    if (qrow < Lq) {
      lse2 = (lse_raw == -INFINITY) ? INFINITY : lse_raw * kLog2e;
      dkv = dsum;
      if (hf == 0 && split == 0 && kh == 0) p.dsoftmax[((int64_t)b * p.H + h) * p.sq_r + qrow] = dsum;
    }
  }
#pragma unroll
  for (int r = 0; r < 16; r++) negd[r] = kInitNegD ? -dkv : 0.f;
  while (it < ntiles) {
    const int n0 = it * BN;
    // Opaque redefinition of the accumulators (keeps the register allocator from copying them around the loop)
#pragma unroll
    for (int i = 0; i < DV / 32; i++) asm volatile("" : "+v"(acc[i]));
    wait_vmem();      // this wave's share of tile `it` is in LDS
    uint32_t kwcur[KBW];
#pragma unroll
    for (int kbi = 0; kbi < KBW; kbi++) kwcur[kbi] = kStored ? kwpre[kbi] >> (4 * hf) : 0u;  // bit 8 (r / 4) + r % 4 <-> register r
    __syncthreads();  // so is everyone else's, and nobody still reads the other buffer
    const int it_next = next_active(it + 1);
    if (it_next < ntiles) stage(it_next, buf ^ 1);
    if (kTensorBias) {
      bias_to_lds();
      if (it_next < ntiles) load_bias(it_next);
    }
    const T* const Ks = reinterpret_cast<const T*>(lds_raw + buf * kBufBytes);
    const T* const Vs = Ks + BN * D;
    buf ^= 1;

    bool wave_work = wave_live;  // a wave whose 32 rows all lie past the sequence's end only helps with the staging
    const int kb0 = kh * KBW;  // this wave's 32-key blocks of the tile: kb0, kb0 + 1, ... (all of them without a key split)
    if (kCausal && n0 + kb0 * 32 > mw + 31) wave_work = false;  // every key of the wave's share is above its diagonal
    if (KS > 1 && n0 + kb0 * 32 >= Lk) wave_work = false;       // ... or past the last key
    bool row_on = true;
    if (kSparse) {
      row_on = row_on_cur;
      row_on_cur = row_on_next;  // next_active(it + 1) above has set it
      if (__ballot(row_on) == 0) wave_work = false;
    }
    if (wave_work) {
      // tiles that straddle the key length, the diagonal or an inactive row block get their dead scores set to -inf
      // (an inactive row block inside an active tile is switched off through its lanes' lse, not score by score)
      const bool need_mask = (n0 + BN > Lk) || (kCausal && (n0 + BN - 1 > mw));
      const float lse_t = (kSparse && !row_on) ? INFINITY : lse2;  // P = exp2(finite - inf) = 0
#pragma unroll
      for (int kbi = 0; kbi < KBW; kbi++) {
        const int kb = kb0 + kbi;
        f32x16 s, dp = negd;
#pragma unroll
        for (int r = 0; r < 16; r++) s[r] = 0.f;
        typename E::vec4 bv[4];  // kTensorBias: the lane's 4 x 4 consecutive values of this 32-key block
        if (kTensorBias) {
#pragma unroll
          for (int j = 0; j < 4; j++)
            bv[j] = *reinterpret_cast<const typename E::vec4*>(bias_lds + c * kBiasRowBytes + (kb * 32 + 8 * j + 4 * hf) * 2);
        }
#pragma unroll
        for (int ks = 0; ks < D / 16; ks++) {
          vec8 a = *reinterpret_cast<const vec8*>(Ks + kb * 32 * D + kfoff[ks]);
          s = E::mfma32(a, qreg[ks], s);
        }
#pragma unroll
        for (int ks = 0; ks < D / 16; ks++) {
          vec8 a = *reinterpret_cast<const vec8*>(Vs + kb * 32 * D + vfoff[ks]);
          dp = E::mfma32(a, doreg[ks], dp);
        }
        if (need_mask) {
#pragma unroll
          for (int r = 0; r < 16; r++) {
            const int key = n0 + kb * 32 + (r >> 2) * 8 + hf * 4 + (r & 3);
            bool dead = key >= Lk;
            if (kCausal) dead = dead || key > qrow;
            if (dead) s[r] = -INFINITY;
          }
        }
        KeepFields keep;
        if (kDropout) keep = keep_fields_row_layout(p.pk, (uint32_t)bh, qrow, n0 + kb * 32, hf);
        const float dbase = (float)(n0 + kb * 32 + hf * 4 - qrow);  // key - query of register 0 (kAlibi)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          float e = -lse_t;
          if (kAlibi) {  // -slope2 * |key - query| - lse; under a causal mask live scores have key <= query
            const float cr = (float)((r >> 2) * 8 + (r & 3));
            e = kCausal ? __builtin_fmaf(cr, sl2, __builtin_fmaf(dbase, sl2, -lse_t))
                        : __builtin_fmaf(__builtin_fabsf(dbase + cr), -sl2, -lse_t);
          }
          if (kTensorBias) {  // (past the last key the caller's rows may hold anything: +inf and NaN are cut off there)
            float bf = (float)bv[r >> 2][r & 3];
            if (need_mask) bf = fminf(bf, 3.0e38f);
            e = __builtin_fmaf(bf, kLog2e, -lse_t);
          }
          const float pe = fast_exp2(__builtin_fmaf(s[r], cs, e));  // 0 for dead scores and switched-off rows
          float dpe = kInitNegD ? dp[r] : dp[r] - dkv;  // dP - Dk
          if (kDropout && !keep.keep_row(r, p.keep_thr)) dpe = -dkv;
          if (kStored) dpe = keep_word_select(kwcur[kbi], 8 * (r >> 2) + (r & 3), dpe, -dkv);
          s[r] = pe * dpe;  // dS'
        }
#pragma unroll
        for (int t = 0; t < 2; t++) {
          f32x8 df;
#pragma unroll
          for (int i = 0; i < 8; i++) df[i] = s[8 * t + i];
          const vec8 dsb = cvt8<T>(df);
#pragma unroll
          for (int db = 0; db < DV / 32; db++) {
            const T* kp = Ks + (kb * 32 + 16 * t) * D;
            u32x2 lo = lds_read_tr16(kp + tlo[db]), hi = lds_read_tr16(kp + thi[db]);
            u32x4 av = {lo[0], lo[1], hi[0], hi[1]};
            acc[db] = E::mfma32(bitcast<vec8>(av), dsb, acc[db]);
          }
        }
      }
    }
    it = it_next;
  }

  // ---- key split: the waves kh > 0 hand their partial dQ to the wave kh == 0 of their rows, in the accumulator's own
  // register order (word (rs * 16 DV/32 + j) * 64 + lane: consecutive lanes, no bank conflicts)
  if (KS > 1) {
    __syncthreads();  // every wave has left the tiles
    float* const X = reinterpret_cast<float*>(lds_raw) + rs * (DV / 32 * 16) * 64 + lane;
    if (kh != 0) {
#pragma unroll
      for (int db = 0; db < DV / 32; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) X[(db * 16 + r) * 64] = acc[db][r];
    }
    __syncthreads();
    if (kh == 0) {
#pragma unroll
      for (int db = 0; db < DV / 32; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[db][r] += X[(db * 16 + r) * 64];
    }
    __syncthreads();  // the staging area of the stores below overlaps the exchange area
    if (kh != 0) return;
  }
  // ---- epilogue: dQ = dQ^T acc * scale / keep, transposed through LDS, coalesced stores
  const float f = p.scale * p.rp_keep;
  if (p.n_splits > 1) {  // partial sum of this key split, fp32, added up by dq_combine_kernel
    if (qrow < Lq) {
      float* op = p.dq_part + (((int64_t)split * p.total_q + q_begin + qrow) * p.H + h) * D;
#pragma unroll
      for (int db = 0; db < DV / 32; db++)
#pragma unroll
        for (int g4 = 0; g4 < 4; g4++) {
          const int d0 = db * 32 + g4 * 8 + hf * 4;
          if (d0 < D) {
            f32x4 x;
#pragma unroll
            for (int i = 0; i < 4; i++) x[i] = acc[db][g4 * 4 + i] * f;
            if (kRotCapable && p.rot_cos != nullptr)  // rotary: the turn back is linear, so every partial sum takes it
              x = unrotate4<T>(x, p.rot_cos, p.rot_sin, qrow < p.rot_rows ? qrow : p.rot_rows - 1, D / 2, d0);
            *reinterpret_cast<f32x4*>(op + d0) = x;
          }
        }
    }
    return;
  }
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
        for (int i = 0; i < 4; i++) x[i] = acc[db][g4 * 4 + i] * f;
        // rotary: q came in rotated; dq goes out turned back (this lane's query row sits at table row `qrow`)
        if (kRotCapable && p.rot_cos != nullptr) {
          int t = qrow < Lq ? qrow : Lq - 1;
          x = unrotate4<T>(x, p.rot_cos, p.rot_sin, t < p.rot_rows ? t : p.rot_rows - 1, D / 2, d0);
        }
        *reinterpret_cast<typename E::vec4*>(Os + c * OS + d0) = cvt4<T>(x);
      }
    }
  __builtin_amdgcn_wave_barrier();
  T* gbase = reinterpret_cast<T*>(p.dq) + (int64_t)q_begin * p.dq_rs + (int64_t)h * p.dq_hs;
#pragma unroll
  for (int i = 0; i < (32 * CH + 63) / 64; i++) {
    const int ch = lane + i * 64;
    const int row = ch / CH, col = (ch % CH) * 8;
    int orow = mw + row;  // (sparse: the wave's rows are those of its two row blocks)
    if (kSparse) orow = (row < 16 ? rb_a : rb_b) < 0 ? 0x3fffffff : (row < 16 ? rb_a : rb_b) * 16 + (row & 15);
    if ((32 * CH % 64 == 0 || ch < 32 * CH) && orow < Lq) {
      u32x4 val = *reinterpret_cast<const u32x4*>(Os + row * OS + col);
      st_global16(gbase + (int64_t)orow * p.dq_rs + col, val);
    }
  }
}

template <typename T, int D, int BN, bool kCausal, int kDrop, bool kSparse, int kBias = 0, int KS = 1>
__global__ void __launch_bounds__(256, (D <= 64 && kDrop == 0 && kBias != kBiasTensor) ? 3 : 2) fa_bwd_dq_kernel(const BwdParams p) {
  using Cfg = DqCfg<T, D, BN, KS>;
  __shared__ __attribute__((aligned(16))) unsigned char lds_raw[Cfg::kLdsBytes + (kBias == kBiasTensor ? 4 * Cfg::kBiasWaveBytes : 0)];
  fa_bwd_dq_body<T, D, BN, kCausal, kDrop, kSparse, kBias, KS>(p, blockIdx.x, lds_raw);
}

// ---------------------------------------------------------------------------------------------------------------
// Short launches: dQ and dK/dV in one launch
// ---------------------------------------------------------------------------------------------------------------
// A launch of a few hundred short workgroups spends a third of its time filling and draining the chip, and the backward
// pays that twice.  Here the workgroups of the dK/dV kernel (ids below p.merged_dkdv_blocks; they form their own Dk, kOwnD) and
// the half-size workgroups of the dQ kernel (the ids after them) make one grid: one fill, one drain, and the two kinds run
// side by side.  Head dim 64, dense, no score bias; kDrop 0 or 2.
template <typename T, bool kCausal, int kDrop>
__global__ void __launch_bounds__(256, 2) fa_bwd_merged_kernel(const BwdParams p) {
  constexpr int D = 64;
  using CfgK = BwdCfg<T, D, kDrop == 1>;
  using CfgQ = DqCfg<T, D, 64, 2>;
  constexpr int kLds = CfgK::kLdsBytes > CfgQ::kLdsBytes ? CfgK::kLdsBytes : CfgQ::kLdsBytes;
  __shared__ __attribute__((aligned(16))) unsigned char lds_raw[kLds];
  const int block = blockIdx.x;
  if (block < p.merged_dkdv_blocks) {
    fa_bwd_dkdv_body<T, D, kCausal, kDrop, false, 0, false, true>(p, block, lds_raw);
  } else {
    BwdParams pq = p;
    pq.nq_tiles = p.merged_nq_tiles;
    fa_bwd_dq_body<T, D, 64, kCausal, kDrop, false, 0, 2>(pq, block - p.merged_dkdv_blocks, lds_raw);
  }
}

}  // namespace fa
