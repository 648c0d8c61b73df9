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

template <typename T>
__global__ void __launch_bounds__(256) rotary_kernel(const RotaryParams p) {
  typedef typename Elem<T>::vec8 vec8;
  typedef typename Elem<T>::vec4 vec4;
  const int cpr = p.head_dim / 8;                      // 16-byte chunks per (row, part, head)
  const int64_t per_row = (int64_t)p.n_parts * p.n_heads * cpr;
  const int64_t total = p.n_rows * per_row;
  for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < total; t += (int64_t)gridDim.x * 256) {
    const int64_t row = t / per_row;
    int rem = (int)(t - row * per_row);
    const int part = rem / (p.n_heads * cpr);
    rem -= part * p.n_heads * cpr;
    const int head = rem / cpr, ch = rem - head * cpr;
    const T* src = reinterpret_cast<const T*>(p.src) + row * p.src_row_stride + (int64_t)part * p.src_part_stride +
                   (int64_t)head * p.src_head_stride + ch * 8;
    T* dst = reinterpret_cast<T*>(p.dst) + row * p.dst_row_stride + (int64_t)part * p.dst_part_stride +
             (int64_t)head * p.dst_head_stride + ch * 8;
    const vec8 x = bitcast<vec8>(ld_global16(src));
    vec8 y = x;
    if (part < p.n_rotated) {
      int pos = p.positions ? p.positions[row] : (int)(row % p.seqlen);
      pos = pos < 0 ? 0 : (pos >= p.table_rows ? p.table_rows - 1 : pos);
      const int64_t toff = (int64_t)pos * (p.head_dim / 2) + ch * 4;
      const vec4 c4 = *reinterpret_cast<const vec4*>(reinterpret_cast<const T*>(p.cos) + toff);
      const vec4 s4 = *reinterpret_cast<const vec4*>(reinterpret_cast<const T*>(p.sin) + toff);
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const float a = (float)x[2 * i], b = (float)x[2 * i + 1];
        const float c = (float)c4[i], s = p.conjugate ? -(float)s4[i] : (float)s4[i];
        y[2 * i] = (T)(a * c - b * s);
        y[2 * i + 1] = (T)(b * c + a * s);
      }
    }
    st_global16(dst, bitcast<u32x4>(y));
  }
}

}  // namespace

hipError_t launch_rotary(const RotaryParams& p, int dtype, hipStream_t stream) {
  const int64_t total = p.n_rows * p.n_parts * p.n_heads * (p.head_dim / 8);
  if (total == 0) return hipSuccess;
  int64_t blocks = (total + 255) / 256;
  if (blocks > 256 * 32) blocks = 256 * 32;
  if (dtype == 0) hipLaunchKernelGGL(rotary_kernel<_Float16>, dim3((unsigned)blocks), dim3(256), 0, stream, p);
  else hipLaunchKernelGGL(rotary_kernel<__bf16>, dim3((unsigned)blocks), dim3(256), 0, stream, p);
  return hipGetLastError();
}

}  // namespace fa
