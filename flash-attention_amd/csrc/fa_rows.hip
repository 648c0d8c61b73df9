// Row gather / scatter kernels behind fa_gather_rows / fa_scatter_rows: the device side of unpad_input / pad_input
// (flash_attn/bert_padding.py:9-95 in the reference, where they are torch.gather / index assignment).  Pure HBM-bound
// byte movement: every row is moved as 16-byte chunks by consecutive lanes (narrower chunks when the row width or an
// address is not 16-byte aligned), each output byte is written exactly once, and no output is zero-filled beforehand.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "fa_params.h"

namespace fa {

namespace {

template <int V> struct Chunk;
template <> struct Chunk<16> { typedef uint4 type; };
template <> struct Chunk<8> { typedef uint2 type; };
template <> struct Chunk<4> { typedef uint32_t type; };
template <> struct Chunk<2> { typedef uint16_t type; };
template <> struct Chunk<1> { typedef uint8_t type; };

// dst[i, :] = src[idx[i], :] for i < n_idx; an index outside [0, n_src) yields a zero row
template <int V>
__global__ void __launch_bounds__(256) gather_rows_kernel(const unsigned char* __restrict__ src, unsigned char* __restrict__ dst,
                                                          const int64_t* __restrict__ idx, int64_t n_idx, int64_t n_src,
                                                          int64_t cpr, int64_t src_stride, int64_t dst_stride) {
  typedef typename Chunk<V>::type C;
  const int64_t total = n_idx * cpr;
  for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < total; t += (int64_t)gridDim.x * 256) {
    const int64_t row = t / cpr, ch = t - row * cpr;
    const int64_t s = idx[row];
    C v = C{};
    if (s >= 0 && s < n_src) v = *reinterpret_cast<const C*>(src + s * src_stride + ch * V);
    *reinterpret_cast<C*>(dst + row * dst_stride + ch * V) = v;
  }
}

// inv[idx[i]] = i (inv pre-filled with -1): the inverse of the index list, for the single-pass scatter below
__global__ void __launch_bounds__(256) invert_index_kernel(const int64_t* __restrict__ idx, int64_t n_idx, int64_t n_dst,
                                                           int32_t* __restrict__ inv) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n_idx) return;
  const int64_t d = idx[i];
  if (d >= 0 && d < n_dst) inv[d] = (int32_t)i;
}

// dst[r, :] = src[s, :] if some idx[s] == r, else 0, for every r < n_dst.  inv is NOT initialised before
// invert_index_kernel writes the entries that have a source: an entry is trusted only if it points back (idx[inv[r]] == r),
// which stale scratch contents can satisfy only by naming the right source row, the indices being unique.
template <int V>
__global__ void __launch_bounds__(256) scatter_rows_kernel(const unsigned char* __restrict__ src, unsigned char* __restrict__ dst,
                                                           const int32_t* __restrict__ inv, const int64_t* __restrict__ idx,
                                                           int64_t n_idx, int64_t n_dst, int64_t cpr, int64_t src_stride,
                                                           int64_t dst_stride) {
  typedef typename Chunk<V>::type C;
  const int64_t total = n_dst * cpr;
  for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < total; t += (int64_t)gridDim.x * 256) {
    const int64_t row = t / cpr, ch = t - row * cpr;
    const int64_t s = inv[row];
    C v = C{};
    if (s >= 0 && s < n_idx && idx[s] == row) v = *reinterpret_cast<const C*>(src + s * src_stride + ch * V);
    *reinterpret_cast<C*>(dst + row * dst_stride + ch * V) = v;
  }
}

unsigned grid_for(int64_t total) {
  int64_t blocks = (total + 255) / 256;
  const int64_t cap = 256 * 32;  // 32 workgroups per CU, grid-stride beyond that
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  return (unsigned)blocks;
}

}  // namespace

#define FA_DISPATCH_V(V, KERNEL, ...)                                                                                 \
  switch (V) {                                                                                                        \
    case 16: hipLaunchKernelGGL(KERNEL<16>, dim3(grid), dim3(256), 0, stream, __VA_ARGS__); break;                    \
    case 8: hipLaunchKernelGGL(KERNEL<8>, dim3(grid), dim3(256), 0, stream, __VA_ARGS__); break;                      \
    case 4: hipLaunchKernelGGL(KERNEL<4>, dim3(grid), dim3(256), 0, stream, __VA_ARGS__); break;                      \
    case 2: hipLaunchKernelGGL(KERNEL<2>, dim3(grid), dim3(256), 0, stream, __VA_ARGS__); break;                      \
    default: hipLaunchKernelGGL(KERNEL<1>, dim3(grid), dim3(256), 0, stream, __VA_ARGS__); break;                     \
  }

hipError_t launch_gather_rows(const void* src, void* dst, const int64_t* idx, int64_t n_idx, int64_t n_src,
                              int64_t row_bytes, int64_t src_stride, int64_t dst_stride, int vec, hipStream_t stream) {
  if (n_idx == 0 || row_bytes == 0) return hipSuccess;
  const int64_t cpr = row_bytes / vec;
  const unsigned grid = grid_for(n_idx * cpr);
  FA_DISPATCH_V(vec, gather_rows_kernel, reinterpret_cast<const unsigned char*>(src), reinterpret_cast<unsigned char*>(dst),
                idx, n_idx, n_src, cpr, src_stride, dst_stride)
  return hipGetLastError();
}

hipError_t launch_scatter_rows(const void* src, void* dst, const int64_t* idx, int64_t n_idx, int64_t n_dst,
                               int64_t row_bytes, int64_t src_stride, int64_t dst_stride, int vec, int32_t* inv,
                               hipStream_t stream) {
  if (n_dst == 0 || row_bytes == 0) return hipSuccess;
  if (n_idx > 0)
    hipLaunchKernelGGL(invert_index_kernel, dim3((unsigned)((n_idx + 255) / 256)), dim3(256), 0, stream, idx, n_idx, n_dst, inv);
  const int64_t cpr = row_bytes / vec;
  const unsigned grid = grid_for(n_dst * cpr);
  FA_DISPATCH_V(vec, scatter_rows_kernel, reinterpret_cast<const unsigned char*>(src), reinterpret_cast<unsigned char*>(dst),
                inv, idx, n_idx, n_dst, cpr, src_stride, dst_stride)
  return hipGetLastError();
}

}  // namespace fa
