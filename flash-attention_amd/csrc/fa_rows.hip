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

// Work shape of both kernels: a thread owns one chunk position of a row and moves it for kRowsPerBlock consecutive output
// rows (blockIdx.y picks the group of rows), index loads first, then all data loads, then the stores - no division per
// chunk, and a row's source index is one wave-uniform load.
constexpr int kRowsPerBlock = 8;

// dst[i, :] = src[idx[i], :] for i < n_idx; an index outside [0, n_src) yields a zero row
template <int V>
__global__ void __launch_bounds__(512) gather_rows_kernel(const unsigned char* __restrict__ src, unsigned char* __restrict__ dst,
                                                          const int64_t* __restrict__ idx, int64_t n_idx, int64_t n_src,
                                                          int cpr, int64_t src_stride, int64_t dst_stride) {
  typedef typename Chunk<V>::type C;
  const int ch = blockIdx.x * blockDim.x + threadIdx.x;
  if (ch >= cpr) return;
  const int64_t row0 = (int64_t)blockIdx.y * kRowsPerBlock;
  const int nrows = (int)(n_idx - row0 < kRowsPerBlock ? n_idx - row0 : kRowsPerBlock);
  int64_t s[kRowsPerBlock];
  C v[kRowsPerBlock];
#pragma unroll
  for (int i = 0; i < kRowsPerBlock; i++) s[i] = i < nrows ? idx[row0 + i] : -1;
#pragma unroll
  for (int i = 0; i < kRowsPerBlock; i++) {
    v[i] = C{};
    if (s[i] >= 0 && s[i] < n_src) v[i] = *reinterpret_cast<const C*>(src + s[i] * src_stride + (int64_t)ch * V);
  }
#pragma unroll
  for (int i = 0; i < kRowsPerBlock; i++)
    if (i < nrows) *reinterpret_cast<C*>(dst + (row0 + i) * dst_stride + (int64_t)ch * V) = v[i];
}

// inv[idx[i]] = i for the entries that have a source (the others keep whatever the scratch held: see scatter_rows_kernel):
// the inverse of the index list, for the single-pass scatter below
__global__ void __launch_bounds__(256) invert_index_kernel(const int64_t* __restrict__ idx, int64_t n_idx, int64_t n_dst,
                                                           int32_t* __restrict__ inv) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n_idx) return;
  const int64_t d = idx[i];
  if (d >= 0 && d < n_dst) inv[d] = (int32_t)i;
}

// dst[r, :] = src[s, :] if some idx[s] == row_base + r, else 0, for every r < n_dst (the rows of this launch).  inv is NOT initialised before
// invert_index_kernel writes the entries that have a source: an entry is trusted only if it points back (idx[inv[r]] == r),
// which stale scratch contents can satisfy only by naming the right source row, the indices being unique.
template <int V>
__global__ void __launch_bounds__(512) scatter_rows_kernel(const unsigned char* __restrict__ src, unsigned char* __restrict__ dst,
                                                           const int32_t* __restrict__ inv, const int64_t* __restrict__ idx,
                                                           int64_t n_idx, int64_t n_dst, int64_t row_base, int cpr,
                                                           int64_t src_stride, int64_t dst_stride) {
  typedef typename Chunk<V>::type C;
  const int ch = blockIdx.x * blockDim.x + threadIdx.x;
  if (ch >= cpr) return;
  const int64_t row0 = (int64_t)blockIdx.y * kRowsPerBlock;
  const int nrows = (int)(n_dst - row0 < kRowsPerBlock ? n_dst - row0 : kRowsPerBlock);
  int64_t s[kRowsPerBlock];
  C v[kRowsPerBlock];
#pragma unroll
  for (int i = 0; i < kRowsPerBlock; i++) s[i] = i < nrows ? (int64_t)inv[row0 + i] : -1;
#pragma unroll
  for (int i = 0; i < kRowsPerBlock; i++)
    if (!(s[i] >= 0 && s[i] < n_idx && idx[s[i]] == row_base + row0 + i)) s[i] = -1;
#pragma unroll
  for (int i = 0; i < kRowsPerBlock; i++) {
    v[i] = C{};
    if (s[i] >= 0) v[i] = *reinterpret_cast<const C*>(src + s[i] * src_stride + (int64_t)ch * V);
  }
#pragma unroll
  for (int i = 0; i < kRowsPerBlock; i++)
    if (i < nrows) *reinterpret_cast<C*>(dst + (row0 + i) * dst_stride + (int64_t)ch * V) = v[i];
}

// Launch shape: a row's chunks go to one workgroup of whole waves if at most 512, else to 256-thread workgroups; grid.y
// holds the groups of rows (at most 65535 per launch: longer tensors take several launches, see the launchers).
struct RowGrid {
  int threads;
  unsigned gx;
};
RowGrid row_grid(int64_t cpr) {
  RowGrid g;
  g.threads = cpr <= 512 ? (int)((cpr + 63) / 64 * 64) : 256;
  g.gx = (unsigned)((cpr + g.threads - 1) / g.threads);
  return g;
}
constexpr int64_t kMaxRowsPerLaunch = (int64_t)65535 * kRowsPerBlock;

}  // namespace

#define FA_DISPATCH_V(V, KERNEL, ...)                                                                                 \
  switch (V) {                                                                                                        \
    case 16: hipLaunchKernelGGL(KERNEL<16>, grid, dim3(g.threads), 0, stream, __VA_ARGS__); break;                    \
    case 8: hipLaunchKernelGGL(KERNEL<8>, grid, dim3(g.threads), 0, stream, __VA_ARGS__); break;                      \
    case 4: hipLaunchKernelGGL(KERNEL<4>, grid, dim3(g.threads), 0, stream, __VA_ARGS__); break;                      \
    case 2: hipLaunchKernelGGL(KERNEL<2>, grid, dim3(g.threads), 0, stream, __VA_ARGS__); break;                      \
    default: hipLaunchKernelGGL(KERNEL<1>, grid, dim3(g.threads), 0, stream, __VA_ARGS__); break;                     \
  }

hipError_t launch_gather_rows(const void* src, void* dst, const int64_t* idx, int64_t n_idx, int64_t n_src,
                              int64_t row_bytes, int64_t src_stride, int64_t dst_stride, int vec, hipStream_t stream) {
  if (n_idx == 0 || row_bytes == 0) return hipSuccess;
  const int64_t cpr = row_bytes / vec;
  if (cpr > (int64_t)1 << 30) return hipErrorInvalidValue;
  const RowGrid g = row_grid(cpr);
  for (int64_t r0 = 0; r0 < n_idx; r0 += kMaxRowsPerLaunch) {  // (one launch unless there are more than 524 280 rows)
    const int64_t n = n_idx - r0 < kMaxRowsPerLaunch ? n_idx - r0 : kMaxRowsPerLaunch;
    const dim3 grid(g.gx, (unsigned)((n + kRowsPerBlock - 1) / kRowsPerBlock));
    FA_DISPATCH_V(vec, gather_rows_kernel, reinterpret_cast<const unsigned char*>(src),
                  reinterpret_cast<unsigned char*>(dst) + r0 * dst_stride, idx + r0, n, n_src, (int)cpr, src_stride, dst_stride)
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

hipError_t launch_scatter_rows(const void* src, void* dst, const int64_t* idx, int64_t n_idx, int64_t n_dst,
                               int64_t row_bytes, int64_t src_stride, int64_t dst_stride, int vec, int32_t* inv,
                               hipStream_t stream) {
  if (n_dst == 0 || row_bytes == 0) return hipSuccess;
  if (n_idx > 0)
    hipLaunchKernelGGL(invert_index_kernel, dim3((unsigned)((n_idx + 255) / 256)), dim3(256), 0, stream, idx, n_idx, n_dst, inv);
  const int64_t cpr = row_bytes / vec;
  if (cpr > (int64_t)1 << 30) return hipErrorInvalidValue;
  const RowGrid g = row_grid(cpr);
  for (int64_t r0 = 0; r0 < n_dst; r0 += kMaxRowsPerLaunch) {  // (one launch unless there are more than 524 280 rows)
    const int64_t n = n_dst - r0 < kMaxRowsPerLaunch ? n_dst - r0 : kMaxRowsPerLaunch;
    const dim3 grid(g.gx, (unsigned)((n + kRowsPerBlock - 1) / kRowsPerBlock));
    // inv and dst start at this launch's first row; row_base tells the kernel which destination rows these are
    FA_DISPATCH_V(vec, scatter_rows_kernel, reinterpret_cast<const unsigned char*>(src),
                  reinterpret_cast<unsigned char*>(dst) + r0 * dst_stride, inv + r0, idx, n_idx, n, r0, (int)cpr, src_stride,
                  dst_stride)
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

}  // namespace fa
