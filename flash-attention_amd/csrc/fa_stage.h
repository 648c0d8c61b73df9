// Global -> LDS tile staging shared by the forward and backward kernels.
//
// A tile is ROWS rows of D 16-bit elements (CH = D/8 chunks of 16 bytes per row) of a strided global tensor.  It is
// brought into LDS by direct-to-LDS loads (global_load_lds_dwordx4): the data never passes through registers, the
// issuing wave does not wait for it, and one wave instruction deposits the 64 lanes' 16-byte chunks at 64 consecutive
// chunk slots.  The tile is therefore stored unpadded (row stride D elements); LDS bank conflicts are avoided by
// permuting the chunks inside a row instead: chunk ch of tile row r is stored at position ch ^ tile_swz(r).  Each
// lane chooses the global chunk that belongs in its slot, so the permutation costs nothing at load time; readers
// apply the same XOR to the chunk index (frag_off / tr_off below).
//
// The LDS pipe serves 16 lanes (a 256-byte line of 64 banks) per cycle.  Three read patterns occur:
//   row fragments  (ds_read_b128, MFMA A operand of X Y^T): 16 lanes read the same chunk of 16 consecutive rows;
//   transposed     (ds_read_b64_tr_b16, MFMA A operand of X^T P): 16 lanes read an aligned chunk pair of 4
//                  consecutive rows;
//   both.
// kSwzRow, kSwzTr and kSwzDual are conflict-free for these respectively.  kSwzTr has period 2 to 8 rows, the other two
// period 16 rows.
#pragma once

#include "fa_common.h"

namespace fa {

enum { kSwzRow = 0, kSwzTr = 1, kSwzDual = 2 };

template <int D, int KIND>
FA_DEVICE int tile_swz(int r) {
  constexpr int CH = D / 8;
  constexpr int RPB = CH >= 16 ? 1 : 16 / CH;  // tile rows per 256-byte LDS line
  const int u = (r / RPB) % CH;
  if (KIND == kSwzRow) return u;
  if (KIND == kSwzTr) {
    // A transposed read touches 4 consecutive rows, and the two 16-lane groups that the LDS serves together 64 bytes
    // (4 chunks) of each: the 4 rows must land in 4 distinct 64-byte bank groups of the 256-byte line.  128-element rows
    // (one per line): chunk ^= 4 * (r % 4); 64-element rows (two per line, the odd row in the upper half anyway): rows r and
    // r + 2 must differ, chunk ^= 4 * ((r / 2) % 2).  Both have period <= 4 rows, so rows r + 8 and r + 16 keep r's value.
    if (CH == 16) return 4 * (r % 4);
    if (CH == 8) return 4 * ((r >> 1) & 1);
    return CH >= 4 ? 2 * (u % (CH / 2)) : 0;
  }
  // dual: a bijection of u (row fragments) whose values for the 4 rows of a transposed read fall in distinct pairs
  if (CH == 16) return ((u & 3) << 2) | (u >> 2);
  if (CH == 8) return ((u & 1) << 2) | (u >> 1);
  return u;
}

// Element offset inside a tile of the row fragment (8 elements) `chunk` of row r.
template <int D, int KIND>
FA_DEVICE int frag_off(int r, int chunk) {
  return r * D + ((chunk ^ tile_swz<D, KIND>(r)) * 8);
}

// Element offset of a lane's 4-element piece of a transposed read (see lds_read_tr16): the 16-lane group g16 of lane
// j16 fetches rows r0 + 4*hf + j16/4 and the aligned chunk pair starting at chunk cp (even) + 2*(g16 & 1).
template <int D, int KIND>
FA_DEVICE int tr_off(int r0, int cp, int lane) {
  const int j16 = lane & 15, g16 = lane >> 4, hf = lane >> 5;
  const int r = r0 + 4 * hf + (j16 >> 2);
  const int chunk = cp + 2 * (g16 & 1) + ((j16 >> 1) & 1);
  return r * D + ((chunk ^ tile_swz<D, KIND>(r)) * 8) + 4 * (j16 & 1);
}

// Stages a pair of ROWS x D tiles per step: tile 0 (swizzle KIND0) by waves 0 and 1, tile 1 (KIND1) by waves 2 and 3,
// into [lds, lds + kTileBytes) and [lds + kTileBytes, lds + 2 * kTileBytes).  A workgroup has 4 waves.
template <int D, int ROWS, int KIND0, int KIND1>
struct TilePairStager {
  static constexpr int CH = D / 8;
  static constexpr int RPI = 64 / CH;                       // tile rows per wave instruction
  static constexpr int TI = 2 * ROWS * CH / 64;             // wave instructions per tile pair
  static constexpr int NI = TI / 4;                         // per wave
  static constexpr int NOFF = 16 / RPI > 0 ? 16 / RPI : 1;  // distinct per-lane source offsets (swizzle period 16 rows)
  static constexpr int kTileBytes = ROWS * D * 2;
  static constexpr int kPairBytes = 2 * kTileBytes;
  static_assert(TI % 4 == 0 && NI % NOFF == 0 && (ROWS / 2) % 16 == 0, "tile does not split evenly over 4 waves");

  typedef __attribute__((address_space(1))) const void* gptr_t;
  typedef __attribute__((address_space(3))) void* lptr_t;

  const char* base;          // wave-uniform: first row of this wave's tensor
  int64_t rsb;               // wave-uniform: row stride in bytes
  int dst0;                  // wave-uniform: byte offset of this wave's first chunk slot inside the pair
  int row0;                  // wave-uniform: first tile row this wave fetches
  int rl, pch;               // lane: row within an instruction, chunk slot within the row
  bool second;               // wave-uniform: this wave fetches tile 1
  uint32_t src_off[NOFF];    // lane: byte offset from the instruction's first row to the chunk this lane fetches

  // `wave` must be wave-uniform (readfirstlane).  t0 / t1 point at row 0 of the two tensors (head offset applied),
  // rs0 / rs1 are their row strides in elements.
  FA_DEVICE void init(int wave, int lane, const void* t0, int64_t rs0, const void* t1, int64_t rs1) {
    second = wave >= 2;
    base = reinterpret_cast<const char*>(second ? t1 : t0);
    rsb = (second ? rs1 : rs0) * 2;
    row0 = (wave & 1) * NI * RPI;
    dst0 = (second ? kTileBytes : 0) + (wave & 1) * NI * 1024;
    rl = lane / CH;
    pch = lane % CH;
#pragma unroll
    for (int j = 0; j < NOFF; j++) src_off[j] = (uint32_t)(rl * rsb) + 16u * (uint32_t)(pch ^ swz(j * RPI + rl));
  }
  FA_DEVICE int swz(int r) const { return second ? tile_swz<D, KIND1>(r) : tile_swz<D, KIND0>(r); }

  // One direct-to-LDS wave instruction: lane l's 16 bytes at (uniform base + per-lane offset) go to lds_dst + 16 * l.
  // Written as inline assembly on purpose: the compiler makes every ds_read_b64_tr_b16 that follows a direct-to-LDS
  // load it knows about wait for vmcnt(0) (it cannot tell that they touch different buffers), which would serialise the
  // prefetch of the next tile with the use of the current one.  The kernels order these loads against their LDS
  // reads themselves (wait_vmem() + workgroup barrier).  M0 carries the LDS address, as the instruction requires.
  static FA_DEVICE void dma16(const char* base, uint32_t lane_off, unsigned char* lds_dst) {
    const uint32_t lds_addr = (uint32_t)(uintptr_t)(lptr_t)lds_dst;
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(lane_off), "s"(base), "s"(lds_addr)
                 : "memory", "m0");
  }

  // Issues the loads of tile rows [first_row, first_row + ROWS) of both tensors; rows >= n_rows (the tensors' valid
  // extent, > first_row) re-read the last valid row so that LDS never holds anything but real tensor data.
  FA_DEVICE void issue(unsigned char* lds, int first_row, int n_rows) const {
    if (__builtin_expect(first_row + ROWS <= n_rows, 1)) {
      const char* const tb = base + ((int64_t)first_row + row0) * rsb;
#pragma unroll
      for (int i = 0; i < NI; i++) dma16(tb + i * RPI * rsb, src_off[i % NOFF], lds + dst0 + i * 1024);
    } else {
      const char* const tb = base + (int64_t)first_row * rsb;
      // The opaque copies keep this rarely taken path's per-lane arithmetic inside it: hoisted out of the caller's main
      // loop (it is loop invariant) it would occupy, or spill, a dozen registers for the whole kernel.
      int rlv = rl, pchv = pch;
      asm volatile("" : "+v"(rlv), "+v"(pchv));
#pragma unroll
      for (int i = 0; i < NI; i++) {
        const int r = row0 + i * RPI + rlv;
        const int rc = first_row + r < n_rows ? r : n_rows - 1 - first_row;
        dma16(tb, (uint32_t)(rc * rsb) + 16u * (uint32_t)(pchv ^ swz(r)), lds + dst0 + i * 1024);
      }
    }
  }

  // The same for a tile whose rows are gathered from 16-row blocks of the tensors: tile rows 16 j .. 16 j + 15 are tensor
  // rows 16 blk[j] .. 16 blk[j] + 15 (blk[j] wave-uniform; < 0: no block - some valid row is fetched and the caller
  // switches those tile rows off).  Rows >= n_rows re-read the last valid row.
  FA_DEVICE void issue_blocks(unsigned char* lds, const int (&blk)[ROWS / 16], int n_rows) const {
    constexpr int SEG = RPI < 16 ? RPI : 16;  // rows of one block that one instruction covers
    const int jb = row0 >> 4;                 // first block this wave fetches from
#pragma unroll
    for (int i = 0; i < NI; i++) {
#pragma unroll
      for (int sg = 0; sg < RPI / SEG; sg++) {  // two segments when an instruction spans two blocks (16-element rows)
        const int tr = i * RPI + sg * 16;       // first tile row of the segment, relative to row0 (a multiple of 16)
        int b = -1;
#pragma unroll
        for (int j = 0; j < ROWS / 16; j++)
          if (jb + (tr >> 4) == j) b = blk[j];
        int srow = (b < 0 ? 0 : b * 16) + (tr & 15);  // tensor row of the segment's first tile row
        if (srow > n_rows - 1) srow = n_rows - 1;
        const bool mine = RPI / SEG == 1 || (rl >> 4) == sg;
        if (__builtin_expect(srow + SEG <= n_rows, 1)) {
          // lane offsets count rows from the instruction's first tile row: rl rows (sg * 16 of them before this segment)
          if (mine) dma16(base + ((int64_t)srow - sg * 16) * rsb, src_off[i % NOFF], lds + dst0 + i * 1024);
        } else {
          int rlv = rl, pchv = pch;
          asm volatile("" : "+v"(rlv), "+v"(pchv));
          const int within = rlv - sg * 16;
          const int rc = srow + within < n_rows ? within : n_rows - 1 - srow;
          if (mine)
            dma16(base + (int64_t)srow * rsb, (uint32_t)(rc * rsb) + 16u * (uint32_t)(pchv ^ swz(row0 + i * RPI + rlv)),
                  lds + dst0 + i * 1024);
        }
      }
    }
  }
};

// s_waitcnt vmcnt(0): every global load this wave has issued, direct-to-LDS ones included, has completed.
FA_DEVICE void wait_vmem() { __builtin_amdgcn_s_waitcnt(0x0f70); }
}  // namespace fa
