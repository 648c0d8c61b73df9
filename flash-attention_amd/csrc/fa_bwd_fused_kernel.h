// One-kernel backward for gfx950: the dK/dV kernel of fa_bwd_kernel.h that also produces dQ, so that S and dP are computed
// once per (query, key) pair instead of twice (five GEMMs per pair of tiles instead of the two-kernel backward's seven).
// It computes what the reference's compute_dq_dk_dv_1xN does (csrc/flash_attn/src/fmha_dgrad_kernel_1xN_loop.h:34-700); where
// the reference carries dQ across key blocks in an fp32 dq_tmp with one CTA per (batch, head) walking all key blocks
// (:444-461,571-592), here the key tiles of a (batch, head) are separate workgroups that pass the running sum of each query
// tile from one to the next.  An alternative to the two-kernel backward, selected by the launch policy (fa_api.hip): the
// matrix work it saves is, on this part, about what its hand-over costs.
//
// A workgroup (four waves) owns 128 keys of one (batch, head) as in fa_bwd_dkdv_kernel and walks the 32-row query tiles.  Per
// step: S = Q K^T, dP = dO V^T - D, P, dS' (one 32-row slab, as in that kernel); dS' (rounded, as it feeds dK) also goes to
// LDS, [key][query]; dV^T += dO^T P, dK^T += Q^T dS'; and, at the top of the NEXT step, from the double-buffered dS' tile,
// the previous tile's partial dQ (32 x 64) = dS' K over the workgroup's 128 keys with v_mfma_f32_16x16x32: wave w owns
// columns 16 w .. 16 w + 15 of d for both 16-row halves (8 MFMAs; A = dS'^T and B = K^T fragments by transposed LDS reads).
// One barrier per step.
//
// The partial sums of the (batch, head)'s key tiles are added up in fp32 scratch with exactly one owner at a time and in a
// fixed order (so the result is reproducible bit for bit, which sums by atomics would not be):
//   * the ring: key tile j starts at query tile j * stride and walks all query tiles cyclically, so the key tiles follow each
//     other `stride` tiles apart and only stride * nkt tiles of Q, dO and running sums are live at a time;
//   * a tile is added to in the order in which the key tiles reach it (rank_of); a wave adds its block when the block's
//     counter says that the wave before it is done, and then sets the counter to rank + 1; the first one stores without
//     loading, the last one scales, rounds and writes dq itself;
//   * the scratch is laid out as the waves hold the blocks ([tile][wave][register][lane]: every load and store instruction
//     moves 256 contiguous bytes).
// What the hand-over costs is decided by where the running sums live between two owners.  A workgroup stores its block, the
// next owner loads it about two steps later; in between every other resident workgroup of the XCD streams its own tiles and
// blocks through the same 4 MB L2, and what is pushed out of it is written back to memory and fetched again.  With 64-row
// tiles and the key tiles spread over the whole ring that was nearly every block (805 MB written, 420 MB re-read per launch at
// B=8, H=12, N=2048 by the L2's counters); 32-row tiles (a step is half as long) and the short ring bring it to 290 MB and
// 100 MB.
// The hand-over needs no atomics and no cache write-back: the key tiles of a (batch, head) run on one XCD (map_tile), whose L2
// is the point of coherence for them.  Stores are complete (vmcnt) when the L2 has them; the counter is written after that;
// the next owner reads counter and block with device-scope loads, which bypass its compute unit's L1.  Every workgroup checks
// that it runs on the XCD its id implies (workgroup ids are dealt to the XCDs in turn) and poisons its dq with NaN if not.
// A wave that waits for its turn gives up after a bounded number of polls and poisons its block with NaN: the grid always
// drains, and a schedule that broke the assumptions above shows instead of hanging.  The front end only launches the kernel
// when all key tiles of a (batch, head) fit one XCD at once with room to spare (fused_bwd_bytes in fa_api.hip).
#pragma once

#include "fa_bwd_kernel.h"

namespace fa {

constexpr int kFusedPollLimit = 1 << 18;

// The XCD this workgroup runs on (gfx940 and later: XCC_ID of the wave's hardware id registers)
FA_DEVICE int xcc_id() {
  uint32_t x;
  asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(x));
  return (int)(x & 15u);
}

// softmax_d = keep * rowsum(dO o O) (fmha_dgrad_kernel_1xN_loop.h:15-30) for the one-kernel backward, which has no dQ kernel
// in front of it to do it on the way; the same pass clears the hand-over counters.  One row per 8 lanes (a lane takes 8 of the
// 64 columns); block x of a (batch, head) covers rows 32 x .. 32 x + 31.
template <typename T>
__global__ void __launch_bounds__(256) fused_prepass_kernel(const BwdParams p) {
  typedef typename Elem<T>::vec8 vec8;
  const int bh = blockIdx.y, b = bh / p.H, h = bh % p.H;
  if (threadIdx.x < 4 && (int)blockIdx.x < p.nqt_ring)
    p.dq_flags[((int64_t)bh * p.nqt_ring + blockIdx.x) * 4 + threadIdx.x] = 0;
  int q_begin, Lq;
  if (!seq_extent(p.cu_q, b, p.total_q, p.max_sq, &q_begin, &Lq)) return;
  const int row = blockIdx.x * 32 + (threadIdx.x >> 3), ch = threadIdx.x & 7;
  float s = 0.f;
  if (row < Lq) {
    const vec8 a = bitcast<vec8>(ld_global16(reinterpret_cast<const T*>(p.dout) + (int64_t)(q_begin + row) * p.do_rs +
                                             (int64_t)h * p.do_hs + ch * 8));
    const vec8 o = bitcast<vec8>(ld_global16(reinterpret_cast<const T*>(p.out) + (int64_t)(q_begin + row) * p.o_rs +
                                             (int64_t)h * p.o_hs + ch * 8));
#pragma unroll
    for (int i = 0; i < 8; i++) s = __builtin_fmaf((float)a[i], (float)o[i], s);
  }
  s += __shfl_xor(s, 1);
  s += __shfl_xor(s, 2);
  s += __shfl_xor(s, 4);
  if (row < Lq && ch == 0) p.dsoftmax[(int64_t)bh * p.sq_r + row] = s * p.p_keep;
  // a batch entry without keys has no key tile to write its dq: zero
  int k_begin, Lk;
  if (row < Lq && !seq_extent(p.cu_k, b, p.total_k, p.max_sk, &k_begin, &Lk))
    st_global16(reinterpret_cast<T*>(p.dq) + (int64_t)(q_begin + row) * p.dq_rs + (int64_t)h * p.dq_hs + ch * 8, u32x4{0, 0, 0, 0});
}

template <typename T, int D>
struct FusedCfg {
  static_assert(D == 64, "one-kernel backward: head dimension 64");
  static constexpr int BM = kFusedBM, BN = kBwdBN;
  typedef TilePairStager<D, BM, kSwzDual, kSwzDual> Stager;
  static constexpr int kBufBytes = Stager::kPairBytes;
  static constexpr int kOffStat = 2 * kBufBytes;
  static constexpr int kStatBytes = 2 * BM * 4;
  static constexpr int kOffK = kOffStat + 2 * kStatBytes;  // K tile [key][d] for the dQ GEMM
  static constexpr int kSBytes = BN * BM * 2;              // dS' tile [key][query]
  static constexpr int kOffS = kOffK + BN * D * 2;
  static constexpr int kLdsBytes = kOffS + 2 * kSBytes;
  static_assert(kLdsBytes >= BN * (D + 8) * 2, "epilogue staging");
  static constexpr int kTileFloats = BM * D;  // running sums of one tile
};

// Chunk permutations (XOR on the 16-byte chunk index inside a row) of the two tiles the dQ GEMM reads with 16-lane
// transposed reads: a group of 16 lanes fetches 4 consecutive rows x 16 columns (two chunks), the LDS serves two groups
// (rows r .. r + 3 and r + 8 .. r + 11) at a time, and their 8 row pieces must fall on 8 distinct 32-byte bank groups.
FA_DEVICE int swz_k16(int r) { return 2 * ((r >> 1) & 1) + 4 * ((r >> 3) & 1); }   // 128-byte rows (two per bank line)
FA_DEVICE int swz_s16(int r) { return 2 * ((r >> 3) & 1) + ((r >> 2) & 1); }        // 64-byte rows (four per bank line)

// kMode: 0 = the kernel.  1 .. 4 only exist for measurements (build with -DFA_FUSED_EXPERIMENTS; dq is wrong): 1 = every partial
// block is stored, nothing is handed over; 2 = the partial blocks are computed and dropped; 3 = stored to a small region that
// stays in the L2; 4 = added to what that region holds and stored back, without counters.
template <typename T, int D, int kMode = 0>
__global__ void __launch_bounds__(256, 2) fa_bwd_fused_kernel(const BwdParams p) {
  using Cfg = FusedCfg<T, D>;
  using E = Elem<T>;
  using vec8 = typename E::vec8;
  using vec4 = typename E::vec4;
  constexpr int BM = Cfg::BM, BN = Cfg::BN, CH = D / 8, kBufBytes = Cfg::kBufBytes;
  static_assert(BM == 32, "one 32-row slab per step");

  __shared__ __attribute__((aligned(16))) unsigned char lds_raw[Cfg::kLdsBytes];

  int bh, kt;
  if (!map_tile<false>(blockIdx.x, p.nk_tiles, p.B * p.H, &bh, &kt)) return;
  const int b = bh / p.H, h = bh % p.H;
  int q_begin = 0, Lq = 0, k_begin, Lk;
  if (!seq_extent(p.cu_k, b, p.total_k, p.max_sk, &k_begin, &Lk)) return;
  if (!seq_extent(p.cu_q, b, p.total_q, p.max_sq, &q_begin, &Lq)) Lq = 0;
  const int n0 = kt * BN;
  if (n0 >= Lk) return;
  const int nkt = (Lk + BN - 1) / BN, nqt = (Lq + BM - 1) / BM;  // key tiles that add to dQ, query tiles
  const bool xcd_ok = xcc_id() == (int)(blockIdx.x & 7u);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 31, hf = lane >> 5;
  const int key = n0 + wave * 32 + c;

  vec8 kreg[D / 16], vreg[D / 16];
  {
    const int kr = key < Lk ? key : Lk - 1;
    const T* kp = reinterpret_cast<const T*>(p.k) + (int64_t)(k_begin + kr) * p.k_rs + (int64_t)h * p.k_hs + hf * 8;
    const T* vp = reinterpret_cast<const T*>(p.v) + (int64_t)(k_begin + kr) * p.v_rs + (int64_t)h * p.v_hs + hf * 8;
#pragma unroll
    for (int ks = 0; ks < D / 16; ks++) {
      u32x4 a = ld_global16(kp + ks * 16), bb = ld_global16(vp + ks * 16);
      if (key >= Lk) { a = u32x4{0, 0, 0, 0}; bb = u32x4{0, 0, 0, 0}; }
      kreg[ks] = bitcast<vec8>(a);
      vreg[ks] = bitcast<vec8>(bb);
    }
  }
  T* const Kl = reinterpret_cast<T*>(lds_raw + Cfg::kOffK);
  T* const dSl = reinterpret_cast<T*>(lds_raw + Cfg::kOffS);
  const int krow = wave * 32 + c;  // this lane's key inside the tile
#pragma unroll
  for (int ks = 0; ks < D / 16; ks++)  // (the main loop's first barrier orders these writes before the first read)
    *reinterpret_cast<vec8*>(Kl + krow * D + (((ks * 2 + hf) ^ swz_k16(krow)) << 3)) = kreg[ks];

  const float* lsebase = p.lse + (int64_t)bh * p.lse_stride;
  const float* dsbase = p.dsoftmax + (int64_t)bh * p.sq_r;

  typename Cfg::Stager stager;
  stager.init(wave, lane, reinterpret_cast<const T*>(p.q) + (int64_t)q_begin * p.q_rs + (int64_t)h * p.q_hs, p.q_rs,
              reinterpret_cast<const T*>(p.dout) + (int64_t)q_begin * p.do_rs + (int64_t)h * p.do_hs, p.do_rs);
  float statpre = 0.f;
  auto stage = [&](int mt, int buf) {
    const int m0 = mt * BM;
    if (tid < BM) {
      const int row = m0 + tid;
      statpre = INFINITY;
      if (row < Lq) statpre = lsebase[row];
    } else if (tid < 2 * BM) {
      const int row = m0 + tid - BM;
      statpre = 0.f;
      if (row < Lq) statpre = dsbase[row];
    }
    stager.issue(lds_raw + buf * kBufBytes, m0, Lq);
  };
  auto stat_value = [&]() -> float {
    if (tid < BM) return (statpre == -INFINITY) ? INFINITY : statpre * kLog2e;
    return -statpre;
  };

  f32x16 acc_dk[D / 32], acc_dv[D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) {
      acc_dk[i][r] = 0.f;
      acc_dv[i][r] = 0.f;
    }

  const float cs = p.scale_log2;
  int foff[D / 16], tlo[D / 32], thi[D / 32];
#pragma unroll
  for (int ks = 0; ks < D / 16; ks++) foff[ks] = frag_off<D, kSwzDual>(c, ks * 2 + hf);
#pragma unroll
  for (int db = 0; db < D / 32; db++) {
    tlo[db] = tr_off<D, kSwzDual>(0, db * 4, lane);
    thi[db] = tr_off<D, kSwzDual>(8, db * 4, lane);
  }
  // dS' row of this lane's key: its 4 values per 16-row half and lane half go to chunk 2 t (+ 1), half hf
  const int sswz = swz_s16(krow);
  const int ds_row = krow * BM + 4 * hf;
  // dQ GEMM operands: 16-lane group g of lane j16 fetches keys 8 g + j16 / 4 (+ 4: second read) of a 32-key step, columns
  // 4 (j16 % 4) .. + 3 of a 16-column block (query rows 16 b .. of dS', columns 16 wave .. of K)
  const int j16 = lane & 15, g16 = lane >> 4;
  int offk[2], offs[2][2];
#pragma unroll
  for (int rd = 0; rd < 2; rd++) {
    const int row = 8 * g16 + (j16 >> 2) + 4 * rd;
    offk[rd] = row * D + (((2 * wave + ((j16 >> 1) & 1)) ^ swz_k16(row)) << 3) + 4 * (j16 & 1);
#pragma unroll
    for (int bq = 0; bq < 2; bq++)
      offs[bq][rd] = row * BM + (((2 * bq + ((j16 >> 1) & 1)) ^ swz_s16(row)) << 3) + 4 * (j16 & 1);
  }

  // K^T fragments of the dQ GEMM (columns 16 wave .. of d, all 128 keys): loop invariant, read once
  __syncthreads();
  vec8 ktf[BN / 32];
#pragma unroll
  for (int kk = 0; kk < BN / 32; kk++) {
    const u32x2 lo = lds_read_tr16(Kl + kk * 32 * D + offk[0]), hi = lds_read_tr16(Kl + kk * 32 * D + offk[1]);
    ktf[kk] = bitcast<vec8>(u32x4{lo[0], lo[1], hi[0], hi[1]});
  }

  // running sums of this (batch, head): [nqt][4 waves][2 halves][64 lanes][4] fp32; counters [nqt][4 waves]
  float* const accbase = p.dq_acc + (int64_t)bh * p.nqt_ring * Cfg::kTileFloats;
  int* const flagbase = p.dq_flags + (int64_t)bh * p.nqt_ring * 4 + wave;
  const __amdgpu_buffer_rsrc_t acc_rsrc =
      __builtin_amdgcn_make_buffer_rsrc(accbase, 0, p.nqt_ring * Cfg::kTileFloats * 4, 0x00020000);
  const int blk_off = (wave * 2 * 64 + lane) * 16;  // bytes; 16-row half bq: + 1024 bq; tile: + kTileFloats * 4
  const float fq = p.scale * p.rp_keep;

  // The ring: key tile j starts at query tile o_j = floor(j * W / nkt), W = min(nqt, stride * nkt), and walks all nqt tiles
  // cyclically.  Tile i is added to first by the key tiles that started at or before it, the later starters first (they
  // reach it first), then by the others in the same order: rank_of() below.
  const int stride = p.ring_stride > 0 ? p.ring_stride : 2;
  const int W = nqt < stride * nkt ? nqt : stride * nkt;
  const int o_j = nkt > 0 ? (int)((int64_t)kt * W / nkt) : 0;
  // cnt(i) = min(nkt, ceil((i + 1) nkt / W)) key tiles have started at or before tile i; carried along from tile to tile
  int cnt_num = (o_j + 1) * nkt, cnt_i = (cnt_num + W - 1) / (W > 0 ? W : 1);
  auto rank_of = [&](int i) -> int { return (i >= o_j ? 0 : nkt) + (cnt_i < nkt ? cnt_i : nkt) - 1 - kt; };
  auto advance_cnt = [&](int i_next) {  // the walk moved on to tile i_next (the successor of the last tile, cyclically)
    if (i_next == 0) { cnt_num = 0; cnt_i = 0; }
    cnt_num += nkt;
    while (cnt_i * W < cnt_num) cnt_i++;
  };

  f32x4 dq_pend[2], ld[2];
  int rel_mt = -1, rel_rank = 0;
  auto release = [&]() {  // the block's stores have been acknowledged: pass it on
    if (rel_mt < 0) return;
    if (lane == 0) __hip_atomic_store(flagbase + rel_mt * 4, rel_rank + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    rel_mt = -1;
  };
  auto load_sum = [&](int mt_) {
    const int toff = mt_ * Cfg::kTileFloats * 4 + blk_off;
#pragma unroll
    for (int bq = 0; bq < 2; bq++)
      ld[bq] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(acc_rsrc, toff + bq * 1024, 0, 16));
  };

  int buf = 0;
  int mt = o_j, pend = -1;
  if (nqt > 0) stage(mt, 0);
  for (int s = 0; s <= nqt; s++) {  // steps 0 .. nqt - 1 and one more for the last tile's dQ block
    const bool work = s < nqt;
    int mt_next = mt + 1;
    if (mt_next == nqt) mt_next = 0;
    wait_vmem();
    float* const lse_l = reinterpret_cast<float*>(lds_raw + Cfg::kOffStat + buf * Cfg::kStatBytes);
    float* const dk_l = lse_l + BM;
    if (work && tid < 2 * BM) lse_l[tid] = stat_value();
    __syncthreads();  // tile s is complete, so is the dS' tile of step s - 1; nobody still reads the other buffers
    if (kMode == 0) release();  // (the stores of the block passed on are older than the wait above)
    if (s + 1 < nqt) stage(mt_next, buf ^ 1);
    const T* const Ql = reinterpret_cast<const T*>(lds_raw + buf * kBufBytes);
    const T* const dOl = Ql + BM * D;
    buf ^= 1;

    // ---- the previous tile's dQ block; its running sum is asked for as soon as its counter allows
    int rank = 0, seen = 0;
    bool loaded = false;
    int* const flag = flagbase + (pend < 0 ? 0 : pend) * 4;
    if (pend >= 0) {
      rank = rank_of(pend);
      if (kMode == 0 && rank > 0) seen = __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const T* const dSp = dSl + ((s - 1) & 1) * (Cfg::kSBytes / 2);
#pragma unroll
      for (int bq = 0; bq < 2; bq++)
#pragma unroll
        for (int i = 0; i < 4; i++) dq_pend[bq][i] = 0.f;
#pragma unroll
      for (int kk = 0; kk < BN / 32; kk++) {
#pragma unroll
        for (int bq = 0; bq < 2; bq++) {
          const u32x2 lo = lds_read_tr16(dSp + kk * 32 * BM + offs[bq][0]), hi = lds_read_tr16(dSp + kk * 32 * BM + offs[bq][1]);
          dq_pend[bq] = E::mfma16(bitcast<vec8>(u32x4{lo[0], lo[1], hi[0], hi[1]}), ktf[kk], dq_pend[bq]);
        }
      }
      if (kMode == 0 && rank > 0 && !loaded && seen >= rank) {
        load_sum(pend);
        loaded = true;
      }
    }

    // ---- this tile: S = Q K^T, dP = dO V^T - D, P, dS'
    f32x16 sc, dp;
    vec8 pb[2], db8[2];
    if (work) {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const f32x4 nd4 = *reinterpret_cast<const f32x4*>(dk_l + 8 * j + 4 * hf);
#pragma unroll
        for (int i = 0; i < 4; i++) { sc[4 * j + i] = 0.f; dp[4 * j + i] = nd4[i]; }
      }
      vec8 aq[D / 16], ad[D / 16];
#pragma unroll
      for (int ks = 0; ks < D / 16; ks++) aq[ks] = *reinterpret_cast<const vec8*>(Ql + foff[ks]);
#pragma unroll
      for (int ks = 0; ks < D / 16; ks++) ad[ks] = *reinterpret_cast<const vec8*>(dOl + foff[ks]);
#pragma unroll
      for (int ks = 0; ks < D / 16; ks++) sc = E::mfma32(aq[ks], kreg[ks], sc);
#pragma unroll
      for (int ks = 0; ks < D / 16; ks++) dp = E::mfma32(ad[ks], vreg[ks], dp);
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const f32x4 lse4 = *reinterpret_cast<const f32x4*>(lse_l + 8 * j + 4 * hf);
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const int r = 4 * j + i;
          const float pe = fast_exp2(__builtin_fmaf(sc[r], cs, -lse4[i]));
          sc[r] = pe;
          dp[r] = pe * dp[r];
        }
      }
      T* const dSc = dSl + (s & 1) * (Cfg::kSBytes / 2);
#pragma unroll
      for (int t = 0; t < 2; t++) {
        f32x8 pf, df;
#pragma unroll
        for (int i = 0; i < 8; i++) { pf[i] = sc[8 * t + i]; df[i] = dp[8 * t + i]; }
        pb[t] = cvt8<T>(pf);
        db8[t] = cvt8<T>(df);
        // dS' of query rows 16 t + 4 hf + {0..3} and + 8 + {0..3} of this lane's key
        *reinterpret_cast<vec4*>(dSc + ds_row + (((2 * t) ^ sswz) << 3)) = __builtin_shufflevector(db8[t], db8[t], 0, 1, 2, 3);
        *reinterpret_cast<vec4*>(dSc + ds_row + (((2 * t + 1) ^ sswz) << 3)) = __builtin_shufflevector(db8[t], db8[t], 4, 5, 6, 7);
      }
    }

    // ---- the previous tile's block joins the running sum
    if (pend >= 0 && (kMode == 3 || kMode == 4)) {  // measurement: blocks go to (and come from) a small region that stays in the L2
      const int toff = (kt % p.nqt_ring) * Cfg::kTileFloats * 4 + blk_off;
      if (kMode == 4) {
#pragma unroll
        for (int bq = 0; bq < 2; bq++)
          dq_pend[bq] = dq_pend[bq] + __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(acc_rsrc, toff + bq * 1024, 0, 16));
      }
      char* const dst = reinterpret_cast<char*>(accbase) + toff;
#pragma unroll
      for (int bq = 0; bq < 2; bq++) *reinterpret_cast<f32x4*>(dst + bq * 1024) = dq_pend[bq];
    }
    if (pend >= 0 && kMode < 2) {
      bool ok = xcd_ok;
      if (kMode == 0 && rank > 0 && !loaded) {  // its turn had not come at the top of the step
        int polls = 0;
#pragma unroll 1
        while (seen < rank) {
          if (++polls > kFusedPollLimit) { ok = false; break; }
          __builtin_amdgcn_s_sleep(2);
          seen = __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        load_sum(pend);
      }
      if (kMode == 0 && rank > 0) {
#pragma unroll
        for (int bq = 0; bq < 2; bq++) dq_pend[bq] = dq_pend[bq] + ld[bq];
      }
      if (!ok) {  // wrong XCD, or the block's turn never came
#pragma unroll
        for (int bq = 0; bq < 2; bq++)
#pragma unroll
          for (int i = 0; i < 4; i++) dq_pend[bq][i] = __builtin_nanf("");
      }
      if (kMode == 0 && rank == nkt - 1) {  // the last one writes dq itself
        const int row0 = pend * BM + 4 * g16;
        T* op = reinterpret_cast<T*>(p.dq) + (int64_t)(q_begin + row0) * p.dq_rs + (int64_t)h * p.dq_hs + 16 * wave + j16;
#pragma unroll
        for (int bq = 0; bq < 2; bq++)
#pragma unroll
          for (int i = 0; i < 4; i++)
            if (row0 + 16 * bq + i < Lq) op[(int64_t)(16 * bq + i) * p.dq_rs] = (T)(dq_pend[bq][i] * fq);
      } else {
        char* const dst = reinterpret_cast<char*>(accbase) + pend * Cfg::kTileFloats * 4 + blk_off;
#pragma unroll
        for (int bq = 0; bq < 2; bq++) *reinterpret_cast<f32x4*>(dst + bq * 1024) = dq_pend[bq];
        rel_mt = pend;
        rel_rank = rank;
      }
    }
    if (kMode == 2 && pend >= 0) {
#pragma unroll
      for (int i = 0; i < 4; i++) acc_dk[0][i] += (dq_pend[0][i] + dq_pend[1][i]) * 1e-30f;
    }

    // ---- dV^T += dO^T P; dK^T += Q^T dS'
    if (work) {
#pragma unroll
      for (int t = 0; t < 2; t++) {
        const int off = 16 * t * D;
#pragma unroll
        for (int db = 0; db < D / 32; db++) {
          u32x2 lo = lds_read_tr16(dOl + off + tlo[db]), hi = lds_read_tr16(dOl + off + thi[db]);
          const u32x4 av = {lo[0], lo[1], hi[0], hi[1]};
          lo = lds_read_tr16(Ql + off + tlo[db]);
          hi = lds_read_tr16(Ql + off + thi[db]);
          const u32x4 aqs = {lo[0], lo[1], hi[0], hi[1]};
          acc_dv[db] = E::mfma32(bitcast<vec8>(av), pb[t], acc_dv[db]);
          acc_dk[db] = E::mfma32(bitcast<vec8>(aqs), db8[t], acc_dk[db]);
        }
      }
    }
    if (pend >= 0) advance_cnt(mt);  // (the count belongs to `pend`: it follows one step behind mt)
    pend = work ? mt : -1;
    mt = mt_next;
  }
  if (kMode == 0) {
    wait_vmem();
    release();
  }

  // ---- epilogue: scale, transpose dK^T / dV^T through LDS, coalesced stores
  __syncthreads();
  constexpr int ES = D + 8;
  T* Stg = reinterpret_cast<T*>(lds_raw) + wave * 32 * ES;
  const float fv = p.rp_keep, fk = p.scale * p.rp_keep;
#pragma unroll
  for (int which = 0; which < 2; which++) {
#pragma unroll
    for (int db = 0; db < D / 32; db++)
#pragma unroll
      for (int g4 = 0; g4 < 4; g4++) {
        const int d0 = db * 32 + g4 * 8 + hf * 4;
        f32x4 x;
#pragma unroll
        for (int i = 0; i < 4; i++) x[i] = which == 0 ? acc_dk[db][g4 * 4 + i] * fk : acc_dv[db][g4 * 4 + i] * fv;
        *reinterpret_cast<vec4*>(Stg + c * ES + d0) = cvt4<T>(x);
      }
    __builtin_amdgcn_wave_barrier();
    T* gbase = which == 0 ? reinterpret_cast<T*>(p.dk) + (int64_t)k_begin * p.dk_rs + (int64_t)h * p.dk_hs
                          : reinterpret_cast<T*>(p.dv) + (int64_t)k_begin * p.dv_rs + (int64_t)h * p.dv_hs;
    const int64_t grs = which == 0 ? p.dk_rs : p.dv_rs;
#pragma unroll
    for (int i = 0; i < 32 * CH / 64; i++) {
      const int ch = lane + i * 64;
      const int row = ch / CH, col = (ch % CH) * 8;
      const int kr = n0 + wave * 32 + row;
      if (kr < Lk) st_global16(gbase + (int64_t)kr * grs + col, *reinterpret_cast<const u32x4*>(Stg + row * ES + col));
    }
    __builtin_amdgcn_wave_barrier();
  }
}

}  // namespace fa
