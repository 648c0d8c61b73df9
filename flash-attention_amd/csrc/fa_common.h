// Shared device-side building blocks of the gfx950 attention kernels: vector types, MFMA wrappers,
// LDS transposed reads, half-wave exchange, Philox dropout bits.
//
// MFMA register layouts used throughout (wave64, v_mfma_f32_32x32x16_{f16,bf16}):
//   A operand: lane l holds row (l % 32), contraction indices 8*(l / 32) .. +7
//   B operand: lane l holds column (l % 32), contraction indices 8*(l / 32) .. +7
//   C/D:       lane l holds column (l % 32); register r (0..15) holds row 8*(r/4) + 4*(l/32) + r%4
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fa {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef short i16x4 __attribute__((ext_vector_type(4)));

#define FA_DEVICE __device__ __forceinline__
#define FA_LDS __attribute__((address_space(3)))

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

template <typename T>
struct Elem;

template <>
struct Elem<_Float16> {
  typedef f16x8 vec8;
  typedef f16x4 vec4;
  static FA_DEVICE f32x16 mfma32(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static FA_DEVICE f32x4 mfma16(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};

template <>
struct Elem<__bf16> {
  typedef bf16x8 vec8;
  typedef bf16x4 vec4;
  static FA_DEVICE f32x16 mfma32(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static FA_DEVICE f32x4 mfma16(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};

template <typename To, typename From>
FA_DEVICE To bitcast(const From& x) {
  static_assert(sizeof(To) == sizeof(From), "bitcast size");
  return __builtin_bit_cast(To, x);
}

// Round 8 floats to the 16-bit element type (round-to-nearest-even, v_cvt_pk_*).
template <typename T>
FA_DEVICE typename Elem<T>::vec8 cvt8(f32x8 x) {
  return __builtin_convertvector(x, typename Elem<T>::vec8);
}
template <typename T>
FA_DEVICE typename Elem<T>::vec4 cvt4(f32x4 x) {
  return __builtin_convertvector(x, typename Elem<T>::vec4);
}

// acc + sum of 8 half-precision values, accumulated in fp32 (v_dot2c_f32_{f16,bf16} against (1, 1)): the forward
// kernel's row sum costs half the VALU instructions of fp32 adds and sums exactly the rounded probabilities that
// multiply V.
FA_DEVICE float sum8_acc(f16x8 v, float acc) {
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  const h2 one = {(_Float16)1.f, (_Float16)1.f};
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const h2 x = {v[2 * i], v[2 * i + 1]};
    acc = __builtin_amdgcn_fdot2(x, one, acc, false);
  }
  return acc;
}
FA_DEVICE float sum8_acc(bf16x8 v, float acc) {
  typedef __bf16 b2 __attribute__((ext_vector_type(2)));
  const b2 one = {(__bf16)1.f, (__bf16)1.f};
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const b2 x = {v[2 * i], v[2 * i + 1]};
    acc = __builtin_amdgcn_fdot2_f32_bf16(x, one, acc, false);
  }
  return acc;
}

// Threshold (log2 units) of the forward kernel's lazy accumulator rescale.
constexpr float kRescaleLog2 = 8.f;
constexpr float kRescaleLimit = 256.f;  // 2^kRescaleLog2

// A wave-uniform 64-bit value moved to scalar registers (the compiler cannot always prove uniformity of a load)
FA_DEVICE uint64_t uniform64(uint64_t x) {
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)x);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(x >> 32));
  return ((uint64_t)hi << 32) | lo;
}

FA_DEVICE float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
FA_DEVICE float fast_log2(float x) { return __builtin_amdgcn_logf(x); }
FA_DEVICE float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

// Values of the two lanes l and l^32 (the two halves of a wave that share an MFMA column).
// v_permlane32_swap with both operands equal returns (lower half's value, upper half's value) in
// every lane, so symmetric reductions need no lane select.
FA_DEVICE float half_max(float x) {
  uint32_t u = __float_as_uint(x);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
FA_DEVICE float half_sum(float x) {
  uint32_t u = __float_as_uint(x);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Rotary position embedding of one 16-byte chunk: pairs (x[2e], x[2e+1]) turned by the angles whose cosines / sines are
// c4[e] / s4[e] (rounded to the tensor dtype, as the reference's cached tables are: flash_attn/rotary.py:66-87), products
// and sums in fp32, one rounding.  The one definition serves the stand-alone pass (fa_rotary.hip) and the attention
// kernels, so both give the same bits.
template <typename T>
FA_DEVICE typename Elem<T>::vec8 rotate8(typename Elem<T>::vec8 x, typename Elem<T>::vec4 c4, typename Elem<T>::vec4 s4,
                                         bool conjugate) {
  typename Elem<T>::vec8 y;
#pragma unroll
  for (int e = 0; e < 4; e++) {
    const float a = (float)x[2 * e], b = (float)x[2 * e + 1];
    const float c = (float)c4[e], s = conjugate ? -(float)s4[e] : (float)s4[e];
    y[2 * e] = (T)(a * c - b * s);
    y[2 * e + 1] = (T)(b * c + a * s);
  }
  return y;
}
// The opposite rotation of four consecutive fp32 values (two pairs; d0 = index of the first inside the head dimension) of
// the row at table position t: what turns a gradient with respect to rotated queries or keys into the gradient with respect
// to the unrotated ones, before it is rounded.
template <typename T>
FA_DEVICE f32x4 unrotate4(f32x4 x, const void* cos_table, const void* sin_table, int t, int half_dim, int d0) {
  typedef T t2 __attribute__((ext_vector_type(2)));
  const int64_t off = (int64_t)t * half_dim + (d0 >> 1);
  const t2 c2 = *reinterpret_cast<const t2*>(reinterpret_cast<const T*>(cos_table) + off);
  const t2 s2 = *reinterpret_cast<const t2*>(reinterpret_cast<const T*>(sin_table) + off);
  f32x4 y;
#pragma unroll
  for (int e = 0; e < 2; e++) {
    const float c = (float)c2[e], s = (float)s2[e];
    y[2 * e] = x[2 * e] * c + x[2 * e + 1] * s;
    y[2 * e + 1] = x[2 * e + 1] * c - x[2 * e] * s;
  }
  return y;
}

// 16-byte global load/store helpers.
FA_DEVICE u32x4 ld_global16(const void* p) { return *reinterpret_cast<const u32x4*>(p); }
FA_DEVICE void st_global16(void* p, u32x4 v) { *reinterpret_cast<u32x4*>(p) = v; }

// ds_read_b64_tr_b16: within each group of 16 lanes, lane j supplies the address of 4 consecutive
// 16-bit elements M[j][0..3]; lane i receives { M[4e + i/4][i%4] : e = 0..3 }.  With lane j pointing
// at row (j/4), columns 4*(j%4).. of a row-major [k][n] tile, lane i ends up with column i of rows
// 0..3, i.e. a k-contiguous MFMA operand fragment read from an n-contiguous tile.
FA_DEVICE u32x2 lds_read_tr16(const void* lds_ptr) {
  i16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FA_LDS i16x4*)(lds_ptr));
  return bitcast<u32x2>(v);
}

// ---------------------------------------------------------------------------------------------
// Dropout.  The keep/drop decision of score element (b, h, q, key) is a pure function of
// (seed, offset, b*H+h, q, key), so forward, backward and the probability dump agree whatever
// their tiling.  Philox-4x32 with 7 rounds (the round function and count of the reference's
// philox.cuh:35-42,121-135).  One 4x4 micro-block of the score matrix (rows 4*Q4.., keys 4*K4..)
// draws two Philox outputs (call 0: rows 0,1; call 1: rows 2,3 of the micro-block); element
// (q%4, key%4) uses 16-bit field  hw = 4*(q%4) + key%4  of the 16 fields, field f being bits
// 16*(f%2).. of word (f/2)%4 of call f/8.  keep  <=>  field <= keep_threshold
// (threshold = floor(keep_prob * 65535), fmha_api.cpp:110).
// ---------------------------------------------------------------------------------------------
struct PhiloxKey {
  uint32_t k0, k1;  // seed_lo, seed_hi ^ offset_hi
  uint32_t c3;      // offset_lo
};

// a ^ b ^ c in one instruction (v_bitop3_b32 with the parity truth table)
FA_DEVICE uint32_t xor3(uint32_t a, uint32_t b, uint32_t c) { return __builtin_amdgcn_bitop3_b32(a, b, c, 0x96); }

FA_DEVICE u32x4 philox4x32_7(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1) {
#pragma unroll
  for (int i = 0; i < 7; i++) {
    uint64_t p0 = (uint64_t)0xD2511F53u * c0;
    uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    uint32_t n0 = xor3((uint32_t)(p1 >> 32), c1, k0);
    uint32_t n1 = (uint32_t)p1;
    uint32_t n2 = xor3((uint32_t)(p0 >> 32), c3, k1);
    uint32_t n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  u32x4 r = {c0, c1, c2, c3};
  return r;
}

// 16 keep bits of micro-block (Q4, K4): bit (4*(q%4) + key%4) set <=> keep.
FA_DEVICE uint32_t dropout_keep_bits16(const PhiloxKey& pk, uint32_t bh, uint32_t Q4, uint32_t K4, uint32_t thr) {
  uint32_t bits = 0;
#pragma unroll
  for (int call = 0; call < 2; call++) {
    u32x4 r = philox4x32_7((K4 << 1) | call, Q4, bh, pk.c3, pk.k0, pk.k1);
#pragma unroll
    for (int w = 0; w < 4; w++) {
      uint32_t lo = r[w] & 0xffffu, hi = r[w] >> 16;
      bits |= (lo <= thr ? 1u : 0u) << (call * 8 + w * 2);
      bits |= (hi <= thr ? 1u : 0u) << (call * 8 + w * 2 + 1);
    }
  }
  return bits;
}

// dest lane i of every quad reads lane P_i of its quad (CTRL = P0 | P1 << 2 | P2 << 4 | P3 << 6)
template <int CTRL>
FA_DEVICE uint32_t quad_perm(uint32_t x) {
  return (uint32_t)__builtin_amdgcn_mov_dpp((int)x, CTRL, 0xf, 0xf, true);
}
constexpr int kQuadXor1 = 0xB1, kQuadXor2 = 0x4E;  // lane ^ 1, lane ^ 2

// The 16 random 16-bit fields that decide the 16 score elements one lane owns in a 32x32 MFMA accumulator tile.
// "Row layout" (S^T = K Q^T tiles: lane -> query row `qrow`, register r -> key key0 + 8*(r/4) + 4*hf + r%4) and
// "column layout" (S = Q K^T tiles: lane -> key `key`, register r -> query row q0 + 8*(r/4) + 4*hf + r%4).
// The four lanes of a quad own the four rows (columns) of the same four micro-blocks.  Lane t of the quad draws the
// two Philox outputs of micro-block t (8 words = 4 rows of 2 words) and the quad then transposes - every lane needs
// row (column) lane%4 of all four micro-blocks - in two DPP butterfly stages.  The raw fields travel: nothing is
// compared, packed into bit masks and unpacked again on the way; the consumer compares a half-word with the threshold.
struct KeepFields {
  uint32_t w[8];
  // row layout: w[2 tt + h] holds row lane%4 of micro-block tt = r / 4, columns 2h (low half) and 2h + 1 (high half)
  FA_DEVICE bool keep_row(int r, uint32_t thr) const { return ((w[r >> 1] >> (16 * (r & 1))) & 0xffffu) <= thr; }
  // column layout: w[4 pi + rho] holds row rho = r % 4, column lane%4 of micro-blocks 2 pi (low half), 2 pi + 1 (high)
  FA_DEVICE bool keep_col(int r, uint32_t thr) const {
    return ((w[4 * (r >> 3) + (r & 3)] >> (16 * ((r >> 2) & 1))) & 0xffffu) <= thr;
  }
};

FA_DEVICE void philox_micro_block(const PhiloxKey& pk, uint32_t bh, uint32_t Q4, uint32_t K4, uint32_t (&a)[8]) {
  const u32x4 r0 = philox4x32_7((K4 << 1) | 0u, Q4, bh, pk.c3, pk.k0, pk.k1);
  const u32x4 r1 = philox4x32_7((K4 << 1) | 1u, Q4, bh, pk.c3, pk.k0, pk.k1);
#pragma unroll
  for (int i = 0; i < 4; i++) { a[i] = r0[i]; a[4 + i] = r1[i]; }  // row rho of the micro-block: a[2 rho], a[2 rho + 1]
}

FA_DEVICE KeepFields keep_fields_row_layout(const PhiloxKey& pk, uint32_t bh, int qrow, int key0, int hf) {
  const int t = qrow & 3;
  uint32_t a[8];
  philox_micro_block(pk, bh, (uint32_t)qrow >> 2, ((uint32_t)key0 >> 2) + 2 * t + hf, a);
  // 4 x 4 transpose over (lane, row): swap bit 0 of both, then bit 1
  const bool t0 = (t & 1) != 0, t1 = (t & 2) != 0;
  uint32_t c[8];
  KeepFields e;
#pragma unroll
  for (int rho = 0; rho < 4; rho++)
#pragma unroll
    for (int h = 0; h < 2; h++) {
      const uint32_t nb = quad_perm<kQuadXor1>(a[2 * (rho ^ 1) + h]);
      c[2 * rho + h] = (((rho & 1) != 0) == t0) ? a[2 * rho + h] : nb;
    }
#pragma unroll
  for (int rho = 0; rho < 4; rho++)
#pragma unroll
    for (int h = 0; h < 2; h++) {
      const uint32_t nb = quad_perm<kQuadXor2>(c[2 * (rho ^ 2) + h]);
      e.w[2 * rho + h] = (((rho & 2) != 0) == t1) ? c[2 * rho + h] : nb;
    }
  return e;
}

// Q4: the micro-block row (query row / 4) this lane draws - micro-block 2 (key % 4) + hf of the eight that cover the
// tile's 32 query rows
FA_DEVICE KeepFields keep_fields_col_layout_q4(const PhiloxKey& pk, uint32_t bh, uint32_t Q4, int key) {
  const int t = key & 3;
  uint32_t a[8];
  philox_micro_block(pk, bh, Q4, (uint32_t)key >> 2, a);
  // Column c of a micro-block is half (c & 1) of its words of parity c >> 1.  Stage 1 swaps lane bit 1 against the
  // word parity; stage 2 swaps lane bit 0 against the half, by a byte permute whose selector depends on the lane:
  // even lanes keep their low half and take the neighbour's low half as high half, odd lanes the reverse.
  const bool t1 = (t & 2) != 0;
  const uint32_t sel = (t & 1) ? 0x03020706u : 0x05040100u;
  KeepFields g;
#pragma unroll
  for (int pi = 0; pi < 2; pi++)
#pragma unroll
    for (int rho = 0; rho < 4; rho++) {
      const uint32_t nb2 = quad_perm<kQuadXor2>(a[2 * rho + (pi ^ 1)]);
      const uint32_t cw = ((pi != 0) == t1) ? a[2 * rho + pi] : nb2;  // from lane (lane & 1) | pi << 1, parity lane / 2
      g.w[4 * pi + rho] = __builtin_amdgcn_perm(quad_perm<kQuadXor1>(cw), cw, sel);
    }
  return g;
}
// ... for 32 consecutive query rows q0 .. q0 + 31
FA_DEVICE KeepFields keep_fields_col_layout(const PhiloxKey& pk, uint32_t bh, int q0, int key, int hf) {
  return keep_fields_col_layout_q4(pk, bh, ((uint32_t)q0 >> 2) + 2 * (key & 3) + hf, key);
}

// ---------------------------------------------------------------------------------------------
// Dropout keep words.  All three kernels decide the same keep bits.  When the caller offers a buffer (one bit per score),
// the forward - which draws them with Philox - leaves them there and the backward's kernels read them instead of
// drawing them again:
// keep_words[(bh * n_key_blocks + kb) * q_extent + keep_word_slot(q)], bit j <=> the score of query q (sequence-local) and
// key 32 kb + j is kept.
//   * The dQ kernel (lane -> query row, like the forward) loads its row's word and tests the bits of its 16 keys.
//   * The dK/dV kernel (lane l owns key l % 32 and, in accumulator register r, query row 8 (r / 4) + 4 (l / 32) + r % 4 of
//     its 32) needs, for register r, a mask over its 64 lanes = the words of two rows 4 apart: keep_word_slot() makes them
//     neighbours, the kernel fetches a tile's words one per lane and moves them to scalar registers (v_readlane), where
//     v_cndmask takes them as they are.
// ---------------------------------------------------------------------------------------------
FA_DEVICE int keep_word_slot(int q) { return (q & ~31) | (q & 24) | ((q & 3) << 1) | ((q >> 2) & 1); }
inline size_t keep_words_q_extent(int max_sq) { return (size_t)((max_sq + 127) & ~127); }
inline size_t keep_words_key_blocks(int max_sk) { return (size_t)(((max_sk + 127) & ~127) / 32); }

// bit `pos` (a constant) of w ? a : b, as a sign-extended one-bit field and a bitwise select: two instructions
FA_DEVICE float keep_word_select(uint32_t w, int pos, float a, float b) {
  const uint32_t m = (uint32_t)((int32_t)(w << (31 - pos)) >> 31);
  return __uint_as_float((m & __float_as_uint(a)) | (~m & __float_as_uint(b)));
}
// w <- 2 w + (this lane's bit of `mask`): one v_addc with the mask as carry-in
FA_DEVICE uint32_t shift_in_lane_bit(uint32_t w, uint64_t mask) {
  asm("v_addc_co_u32_e64 %0, vcc, %1, %1, %2" : "=v"(w) : "v"(w), "s"(mask) : "vcc");
  return w;
}
// this lane's bit of a wave-uniform mask, as a condition the compiler selects on with the mask register as it is
FA_DEVICE bool lane_bit(uint64_t mask) { return __builtin_amdgcn_inverse_ballot_w64(mask); }
// The 16 keep bits of a lane in the row layout (register r <-> key 8 (r / 4) + 4 hf + r % 4 of a 32-key block), shifted in
// register by register with shift_in_lane_bit and a 4-bit gap after every fourth: turned into the lane's share of the
// 32-bit keep word of its query row, then joined with the share of the lane that holds the row's other 16 keys.
FA_DEVICE uint32_t keep_word_from_shares(uint32_t w, int hf) {
  w = __builtin_bitreverse32(w) >> (hf ? 0 : 4);  // register r of half hf now sits at bit 8 (r / 4) + 4 hf + r % 4
  auto r = __builtin_amdgcn_permlane32_swap(w, w, false, false);
  return r[0] | r[1];
}

}  // namespace fa
