// Rotary position embedding kernel behind fa_rotary: what apply_rotary_pos_emb does with torch elementwise ops
// (flash_attn/rotary.py:22-42 in the reference: x * cos + rotate_half(x) * sin, pairs (x[2i], x[2i+1]) interleaved),
// for the query and key parts of a packed qkv tensor in ONE pass, optionally in place.  HBM-bound: each element is read
// once and written once; cos / sin come from the caller's tables (position x pair, rounded to the tensor's dtype as the
// reference's cached tables are), products and sums are formed in fp32 and rounded once.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "fa_common.h"
#include "fa_params.h"

namespace fa {

namespace {

// work_parts: the parts of a row the kernel visits - all of them, or only the rotated ones when the pass is in place (the
// others are already where they belong: copying v onto itself would be a third of the traffic for nothing).
//
// Index arithmetic decides this kernel's speed, not its eight multiply-adds per 16 bytes: a thread owns one 16-byte chunk
// position (part, head, chunk) of a row - found with three divisions, once - and walks kRotaryRows consecutive rows with
// it (blockIdx.y picks the group of rows); the position in the sequence is carried along with a compare instead of a
// modulo per row.  (One flat index per chunk, decomposed by 64-bit divisions for every 16 bytes, ran at 40 % of this.)
constexpr int kRotaryRows = 8;

template <typename T>
__global__ void __launch_bounds__(512) rotary_kernel(const RotaryParams p, int work_parts) {
  typedef typename Elem<T>::vec8 vec8;
  typedef typename Elem<T>::vec4 vec4;
  const int cpr = p.head_dim / 8;                      // 16-byte chunks per (row, part, head)
  const int per_row = work_parts * p.n_heads * cpr;
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= per_row) return;
  const int part = j / (p.n_heads * cpr);
  const int rem = j - part * p.n_heads * cpr;
  const int head = rem / cpr, ch = rem - head * cpr;
  const bool rot = part < p.n_rotated;
  const int64_t row0 = (int64_t)blockIdx.y * kRotaryRows;
  const int nrows = (int)(p.n_rows - row0 < kRotaryRows ? p.n_rows - row0 : kRotaryRows);
  const T* src = reinterpret_cast<const T*>(p.src) + row0 * p.src_row_stride + (int64_t)part * p.src_part_stride +
                 (int64_t)head * p.src_head_stride + ch * 8;
  T* dst = reinterpret_cast<T*>(p.dst) + row0 * p.dst_row_stride + (int64_t)part * p.dst_part_stride +
           (int64_t)head * p.dst_head_stride + ch * 8;
  int pos0 = p.positions ? 0 : (int)((p.row_offset + row0) % p.seqlen);  // (wave-uniform: one division per workgroup)
  vec8 x[kRotaryRows];
  vec4 c4[kRotaryRows], s4[kRotaryRows];
#pragma unroll
  for (int i = 0; i < kRotaryRows; i++) {  // every load of the thread is in flight before the first is used
    if (i < nrows) {
      x[i] = bitcast<vec8>(ld_global16(src + (int64_t)i * p.src_row_stride));
      if (rot) {
        int pos = p.positions ? p.positions[row0 + i] : pos0;
        pos = pos < 0 ? 0 : (pos >= p.table_rows ? p.table_rows - 1 : pos);
        const int64_t toff = (int64_t)pos * (p.head_dim / 2) + ch * 4;
        c4[i] = *reinterpret_cast<const vec4*>(reinterpret_cast<const T*>(p.cos) + toff);
        s4[i] = *reinterpret_cast<const vec4*>(reinterpret_cast<const T*>(p.sin) + toff);
        if (++pos0 == p.seqlen) pos0 = 0;
      }
    }
  }
#pragma unroll
  for (int i = 0; i < kRotaryRows; i++) {
    if (i < nrows) {
      vec8 y = x[i];
      if (rot) y = rotate8<T>(x[i], c4[i], s4[i], p.conjugate != 0);
      st_global16(dst + (int64_t)i * p.dst_row_stride, bitcast<u32x4>(y));
    }
  }
}

}  // namespace

hipError_t launch_rotary(const RotaryParams& p, int dtype, hipStream_t stream) {
  const bool in_place = p.src == p.dst && p.src_row_stride == p.dst_row_stride && p.src_part_stride == p.dst_part_stride &&
                        p.src_head_stride == p.dst_head_stride;
  const int work_parts = in_place ? p.n_rotated : p.n_parts;
  const int64_t per_row = (int64_t)work_parts * p.n_heads * (p.head_dim / 8);
  if (p.n_rows == 0 || per_row == 0) return hipSuccess;
  if (per_row > (int64_t)1 << 30) return hipErrorInvalidValue;
  const int64_t row_groups = (p.n_rows + kRotaryRows - 1) / kRotaryRows;
  // grid.y holds the row groups: up to 65535 of them per launch
  // a row's chunks go to one workgroup of whole waves if at most 512, else to 256-thread workgroups (the last one partly idle)
  const int threads = per_row <= 512 ? (int)((per_row + 63) / 64 * 64) : 256;
  const unsigned gx = (unsigned)((per_row + threads - 1) / threads);
  for (int64_t g0 = 0; g0 < row_groups; g0 += 65535) {
    const int64_t ng = row_groups - g0 < 65535 ? row_groups - g0 : 65535;
    RotaryParams q = p;
    const int64_t r0 = g0 * kRotaryRows;
    q.src = reinterpret_cast<const char*>(p.src) + r0 * p.src_row_stride * 2;
    q.dst = reinterpret_cast<char*>(p.dst) + r0 * p.dst_row_stride * 2;
    q.n_rows = p.n_rows - r0 < ng * kRotaryRows ? p.n_rows - r0 : ng * kRotaryRows;
    if (p.positions) q.positions = p.positions + r0;
    q.row_offset = p.row_offset + r0;
    if (dtype == 0) hipLaunchKernelGGL(rotary_kernel<_Float16>, dim3(gx, (unsigned)ng), dim3(threads), 0, stream, q, work_parts);
    else hipLaunchKernelGGL(rotary_kernel<__bf16>, dim3(gx, (unsigned)ng), dim3(threads), 0, stream, q, work_parts);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

}  // namespace fa
