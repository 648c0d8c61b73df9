// Backward attention kernel for gfx950.
//
// Computes what the reference's compute_dq_dk_dv_1xN does (csrc/flash_attn/src/fmha_dgrad_kernel_1xN_loop.h:34-700):
//   P  = exp(scale * S - lse) recomputed from Q, K;  dP = dO V^T;  dS' = P o (M o dP - Dk)   (M = dropout keep mask,
//   Dk = keep * rowsum(dO o O));  dV = (P o M)^T dO / keep;  dK = dS'^T Q * scale / keep;  dQ = dS' K * scale / keep.
// Organisation: one workgroup owns a tile of BN = 128 keys of one (batch, head) (wave w owns keys 32w..32w+31), keeps
// its K and V fragments and the dK^T / dV^T accumulators in registers, and streams 64-row tiles of Q, dO, lse, Dk
// through LDS.  Per step:
//   S  = Q K^T, dP = dO V^T   A = Q / dO rows from LDS, B = K / V fragments in registers; C layout: lane -> key,
//                             registers -> 16 query rows
//   dV^T += dO^T P, dK^T += Q^T dS'   B = P / dS' straight from the accumulator registers (rounded to fp16/bf16, as the
//                             reference does before these GEMMs), A = dO^T / Q^T via ds_read_b64_tr_b16
//   dQ += dS' K               dS' goes through LDS once ([key][query] layout); the (64 x D) dQ tile of the step is split
//                             over the 4 waves as 32x32 tiles, contraction over the 128 keys, both operands read with
//                             ds_read_b64_tr_b16; the result is added to an fp32 accumulator in global memory with
//                             atomics (the reference's dq_tmp, fmha_dgrad_kernel_1xN_loop.h:444-461,571-592) and is
//                             converted to fp16/bf16 by a separate pass.
#pragma once

#include "fa_common.h"
#include "fa_params.h"

namespace fa {

template <typename T, int D>
struct BwdCfg {
  static constexpr int BM = kBwdBM;  // query rows per step
  static constexpr int BN = 128;     // keys per workgroup
  static constexpr int NW = 4;
  static constexpr int DV = D < 32 ? 32 : D;
  static constexpr int RS = DV + 8;   // row stride (elements) of the K, Q, dO tiles in LDS
  static constexpr int DSS = BM + 8;  // row stride of the dS'^T tile [key][query]
  static constexpr int kOffK = 0;
  static constexpr int kOffQ = kOffK + BN * RS * 2;
  static constexpr int kOffDO = kOffQ + BM * RS * 2;
  static constexpr int kOffDS = kOffDO + BM * RS * 2;
  static constexpr int kOffLse = kOffDS + BN * DSS * 2;
  static constexpr int kOffDk = kOffLse + BM * 4;
  static constexpr int kLdsBytes = kOffDk + BM * 4;
  static constexpr int CH = D / 8;
  static constexpr int CPT = (BM * CH + 255) / 256;   // 16-byte chunks per thread for a Q / dO tile
  static constexpr int CPTK = (BN * CH + 255) / 256;  // for the K tile
  static constexpr int kMinBlocks = D <= 64 ? 2 : 1;
};

template <typename T, int D, bool kCausal, bool kDropout, bool kSparse>
__global__ void __launch_bounds__(256, (BwdCfg<T, D>::kMinBlocks)) fa_bwd_kernel(const BwdParams p) {
  using Cfg = BwdCfg<T, D>;
  using E = Elem<T>;
  using vec8 = typename E::vec8;
  using vec4 = typename E::vec4;
  constexpr int BM = Cfg::BM, BN = Cfg::BN, DV = Cfg::DV, RS = Cfg::RS, DSS = Cfg::DSS, CH = Cfg::CH;
  constexpr int CPT = Cfg::CPT, CPTK = Cfg::CPTK;

  __shared__ __attribute__((aligned(16))) unsigned char lds_raw[Cfg::kLdsBytes];
  T* Kl = reinterpret_cast<T*>(lds_raw + Cfg::kOffK);
  T* Ql = reinterpret_cast<T*>(lds_raw + Cfg::kOffQ);
  T* dOl = reinterpret_cast<T*>(lds_raw + Cfg::kOffDO);
  T* dSl = reinterpret_cast<T*>(lds_raw + Cfg::kOffDS);
  float* lse_l = reinterpret_cast<float*>(lds_raw + Cfg::kOffLse);
  float* dk_l = reinterpret_cast<float*>(lds_raw + Cfg::kOffDk);

  // XCD-aware id remap: all key tiles of one (batch, head) run on one XCD and share its L2 for Q, dO and
  // the dQ accumulator.
  const int per_xcd = (p.total_tiles + 7) >> 3;
  const int vid = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (vid >= p.total_tiles) return;
  const int bh = vid / p.nk_tiles;
  const int kt = vid % p.nk_tiles;
  const int b = bh / p.H, h = bh % p.H;

  int q_begin = 0, Lq = 0, k_begin, Lk;
  if (!seq_extent(p.cu_k, b, p.total_k, p.max_sk, &k_begin, &Lk)) return;
  if (!seq_extent(p.cu_q, b, p.total_q, p.max_sq, &q_begin, &Lq)) Lq = 0;  // no queries: dK = dV = 0
  const int n0 = kt * BN;
  if (n0 >= Lk) return;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c = lane & 31, hf = lane >> 5;
  const int j16 = lane & 15, g16 = lane >> 4;
  const int key = n0 + wave * 32 + c;  // this lane's key (sequence-local)

  // ---- K and V fragments of this wave's 32 keys (B operands), registers for the whole kernel
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
  // ---- K tile, row-major in LDS (B operand of the dQ GEMM)
  {
    const T* kbase = reinterpret_cast<const T*>(p.k) + (int64_t)k_begin * p.k_rs + (int64_t)h * p.k_hs;
#pragma unroll
    for (int i = 0; i < CPTK; i++) {
      const int ch = tid + i * 256;
      const int row = ch / CH, col = (ch % CH) * 8;
      if (BN * CH % 256 == 0 || ch < BN * CH) {
        u32x4 a = u32x4{0, 0, 0, 0};
        if (n0 + row < Lk) a = ld_global16(kbase + (int64_t)(n0 + row) * p.k_rs + col);
        *reinterpret_cast<u32x4*>(Kl + row * RS + col) = a;
      }
    }
    if (D < 32) {  // zero padding columns of all three row-major tiles
      for (int i = tid; i < BN * (DV - D); i += 256) Kl[(i / (DV - D)) * RS + D + i % (DV - D)] = (T)0.f;
      for (int i = tid; i < BM * (DV - D); i += 256) {
        Ql[(i / (DV - D)) * RS + D + i % (DV - D)] = (T)0.f;
        dOl[(i / (DV - D)) * RS + D + i % (DV - D)] = (T)0.f;
      }
    }
  }

  int mt_begin = 0;
  if (kCausal) mt_begin = n0 / BM;  // query rows above the tile's first key see none of its keys
  const int mt_end = (Lq + BM - 1) / BM;

  const T* qbase = reinterpret_cast<const T*>(p.q) + (int64_t)q_begin * p.q_rs + (int64_t)h * p.q_hs;
  const T* dobase = reinterpret_cast<const T*>(p.dout) + (int64_t)q_begin * p.do_rs + (int64_t)h * p.do_hs;
  const float* lsebase = p.lse + ((int64_t)b * p.H + h) * p.lse_stride;
  const float* dsbase = p.dsoftmax + ((int64_t)b * p.H + h) * p.sq_r;
  float* dqbase = p.dq_acc + (int64_t)q_begin * p.H * D + (int64_t)h * D;

  u32x4 qpre[CPT], dopre[CPT];
  float statpre = 0.f;
  auto prefetch = [&](int mt) {
    const int m0 = mt * BM;
#pragma unroll
    for (int i = 0; i < CPT; i++) {
      const int ch = tid + i * 256;
      const int row = ch / CH, col = (ch % CH) * 8;
      if ((BM * CH % 256 == 0 || ch < BM * CH) && m0 + row < Lq) {
        qpre[i] = ld_global16(qbase + (int64_t)(m0 + row) * p.q_rs + col);
        dopre[i] = ld_global16(dobase + (int64_t)(m0 + row) * p.do_rs + col);
      } else {
        qpre[i] = u32x4{0, 0, 0, 0};
        dopre[i] = u32x4{0, 0, 0, 0};
      }
    }
    if (tid < BM) {  // lse (scaled to base 2; +inf switches a row off)
      const int row = m0 + tid;
      float x = INFINITY;
      if (row < Lq) {
        x = lsebase[row];
        x = (x == -INFINITY) ? INFINITY : x * kLog2e;
      }
      statpre = x;
    } else if (tid < 2 * BM) {
      const int row = m0 + tid - BM;
      statpre = row < Lq ? dsbase[row] : 0.f;
    }
  };
  auto commit = [&]() {
#pragma unroll
    for (int i = 0; i < CPT; i++) {
      const int ch = tid + i * 256;
      const int row = ch / CH, col = (ch % CH) * 8;
      if (BM * CH % 256 == 0 || ch < BM * CH) {
        *reinterpret_cast<u32x4*>(Ql + row * RS + col) = qpre[i];
        *reinterpret_cast<u32x4*>(dOl + row * RS + col) = dopre[i];
      }
    }
    if (tid < BM) lse_l[tid] = statpre;
    else if (tid < 2 * BM) dk_l[tid - BM] = statpre;
  };

  auto tile_active = [&](int mt) -> bool {
    if (!kSparse) return true;
    return p.sp.actk[(n0 >> 8) * p.sp.nqt2 + mt] != 0;
  };
  auto next_active = [&](int mt) -> int {
    while (mt < mt_end && !tile_active(mt)) mt++;
    return mt;
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
  // element offset of a transposed read: row (4*hf + j16/4) [+8], column 16*(g16&1) + 4*(j16&3)
  const int tr_row = 4 * hf + (j16 >> 2);
  const int tr_col = 16 * (g16 & 1) + 4 * (j16 & 3);

  int mt = next_active(mt_begin);
  if (mt < mt_end) prefetch(mt);
  while (mt < mt_end) {
    const int m0 = mt * BM;
    __syncthreads();
    commit();
    __syncthreads();
    const int mt_next = next_active(mt + 1);
    if (mt_next < mt_end) prefetch(mt_next);

    const bool diag = kCausal && (m0 < n0 + wave * 32 + 32);  // some (q, key) of this wave's slab has key > q

#pragma unroll
    for (int qb = 0; qb < BM / 32; qb++) {
      // ---- S = Q K^T and dP = dO V^T for 32 query rows x this wave's 32 keys
      f32x16 s, dp;
#pragma unroll
      for (int r = 0; r < 16; r++) { s[r] = 0.f; dp[r] = 0.f; }
#pragma unroll
      for (int ks = 0; ks < D / 16; ks++) {
        vec8 aq = *reinterpret_cast<const vec8*>(Ql + (qb * 32 + c) * RS + ks * 16 + hf * 8);
        s = E::mfma32(aq, kreg[ks], s);
      }
#pragma unroll
      for (int ks = 0; ks < D / 16; ks++) {
        vec8 ad = *reinterpret_cast<const vec8*>(dOl + (qb * 32 + c) * RS + ks * 16 + hf * 8);
        dp = E::mfma32(ad, vreg[ks], dp);
      }
      // ---- P and dS'
      bool rb_on[2] = {true, true};
      if (kSparse) {
#pragma unroll
        for (int u = 0; u < 2; u++) {
          int rb = (m0 + qb * 32 + u * 16) >> 4;
          rb = rb < p.sp.nrb ? rb : p.sp.nrb - 1;
          rb_on[u] = p.sp.act16[rb * p.sp.ncb + (n0 >> 8)] != 0;
        }
      }
      uint32_t keepbits[4];
      if (kDropout) {
        const int t = c & 3;
        const uint32_t K4 = (uint32_t)key >> 2;
        const uint32_t Q4 = ((uint32_t)(m0 + qb * 32) >> 2) + 2 * t + hf;
        const uint32_t mine = dropout_keep_bits16(p.pk, (uint32_t)bh, Q4, K4, p.keep_thr);
        keepbits[0] = quad_bcast<0>(mine) >> t;
        keepbits[1] = quad_bcast<1>(mine) >> t;
        keepbits[2] = quad_bcast<2>(mine) >> t;
        keepbits[3] = quad_bcast<3>(mine) >> t;
      }
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const f32x4 lse4 = *reinterpret_cast<const f32x4*>(lse_l + qb * 32 + 8 * j + 4 * hf);
        const f32x4 dk4 = *reinterpret_cast<const f32x4*>(dk_l + qb * 32 + 8 * j + 4 * hf);
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const int r = 4 * j + i;
          float pe = fast_exp2(__builtin_fmaf(s[r], cs, -lse4[i]));
          if (kCausal && diag) {
            const int qrow = m0 + qb * 32 + 8 * j + 4 * hf + i;
            if (key > qrow) pe = 0.f;
          }
          if (kSparse && !rb_on[j >> 1]) pe = 0.f;
          float dpe = dp[r];
          float pm = pe;
          if (kDropout) {
            const bool keep = (keepbits[j] >> (4 * i)) & 1u;
            if (!keep) { dpe = 0.f; pm = 0.f; }
          }
          s[r] = pm;                      // P o M, feeds dV
          dp[r] = pe * (dpe - dk4[i]);    // dS', feeds dK and dQ
        }
      }
      // ---- round to the element type; dS'^T to LDS ([key][query]); dV^T += dO^T P; dK^T += Q^T dS'
#pragma unroll
      for (int j = 0; j < 4; j++) {
        f32x4 x;
#pragma unroll
        for (int i = 0; i < 4; i++) x[i] = dp[4 * j + i];
        *reinterpret_cast<vec4*>(dSl + (wave * 32 + c) * DSS + qb * 32 + 8 * j + 4 * hf) = cvt4<T>(x);
      }
#pragma unroll
      for (int t = 0; t < 2; t++) {
        f32x8 pf, df;
#pragma unroll
        for (int i = 0; i < 8; i++) { pf[i] = s[8 * t + i]; df[i] = dp[8 * t + i]; }
        const vec8 pb = cvt8<T>(pf);
        const vec8 db8 = cvt8<T>(df);
#pragma unroll
        for (int db = 0; db < DV / 32; db++) {
          const int off = (qb * 32 + 16 * t + tr_row) * RS + db * 32 + tr_col;
          u32x2 lo = lds_read_tr16(dOl + off), hi = lds_read_tr16(dOl + off + 8 * RS);
          u32x4 av = {lo[0], lo[1], hi[0], hi[1]};
          acc_dv[db] = E::mfma32(bitcast<vec8>(av), pb, acc_dv[db]);
          lo = lds_read_tr16(Ql + off);
          hi = lds_read_tr16(Ql + off + 8 * RS);
          u32x4 aq = {lo[0], lo[1], hi[0], hi[1]};
          acc_dk[db] = E::mfma32(bitcast<vec8>(aq), db8, acc_dk[db]);
        }
      }
    }
    __syncthreads();  // dS'^T of all four waves is in LDS

    // ---- dQ (BM x D) = dS' (BM x BN) K (BN x D); 32x32 tiles over the waves
    constexpr int kTiles = (BM / 32) * (DV / 32);
#pragma unroll
    for (int tile = 0; tile < (kTiles + 3) / 4; tile++) {
      const int tl = wave + tile * 4;
      if (kTiles % 4 == 0 || tl < kTiles) {
        const int qtile = tl / (DV / 32), dtile = tl % (DV / 32);
        f32x16 acc;
#pragma unroll
        for (int r = 0; r < 16; r++) acc[r] = 0.f;
#pragma unroll
        for (int kk = 0; kk < BN / 16; kk++) {
          const int offa = (kk * 16 + tr_row) * DSS + qtile * 32 + tr_col;
          const int offb = (kk * 16 + tr_row) * RS + dtile * 32 + tr_col;
          u32x2 alo = lds_read_tr16(dSl + offa), ahi = lds_read_tr16(dSl + offa + 8 * DSS);
          u32x2 blo = lds_read_tr16(Kl + offb), bhi = lds_read_tr16(Kl + offb + 8 * RS);
          u32x4 av = {alo[0], alo[1], ahi[0], ahi[1]};
          u32x4 bv = {blo[0], blo[1], bhi[0], bhi[1]};
          acc = E::mfma32(bitcast<vec8>(av), bitcast<vec8>(bv), acc);
        }
        if (dtile * 32 + c < D) {
#pragma unroll
          for (int r = 0; r < 16; r++) {
            const int qrow = m0 + qtile * 32 + (r >> 2) * 8 + hf * 4 + (r & 3);
            if (qrow < Lq) atomicAdd(dqbase + (int64_t)qrow * p.H * D + dtile * 32 + c, acc[r]);
          }
        }
      }
    }
    mt = mt_next;
  }

  // ---- epilogue: scale, transpose dK^T / dV^T through LDS, coalesced stores
  __syncthreads();
  T* Stg = reinterpret_cast<T*>(lds_raw) + wave * 32 * RS;  // 32 keys x D per wave, reusing the K tile region
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
          *reinterpret_cast<vec4*>(Stg + c * RS + d0) = cvt4<T>(x);
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
        u32x4 val = *reinterpret_cast<const u32x4*>(Stg + row * RS + col);
        st_global16(gbase + (int64_t)krow * grs + col, val);
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
}

}  // namespace fa
