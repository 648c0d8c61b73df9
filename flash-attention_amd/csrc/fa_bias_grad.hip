// Reduction of the bias gradient behind fa_bias_grad_reduce.  The dK/dV kernel writes the gradient of an attn_bias tensor
// per (batch, head); a bias that was broadcast over the batch and/or the heads wants the sum over the entries that shared
// it.  One pass: every thread owns 8 consecutive keys of one output row, adds the slices in a fixed order (batch outer,
// head inner) in fp32 and rounds once.  HBM-bound: each input element is read once, each output element written once.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "fa_params.h"

namespace fa {

namespace {

template <typename T, bool kVecStore>
__global__ void __launch_bounds__(256) bias_grad_reduce_kernel(const T* __restrict__ in, T* __restrict__ out, int nb, int nh,
                                                               int rows, int cols, int64_t in_bs, int64_t in_hs,
                                                               int64_t in_rs, int64_t out_bs, int64_t out_hs, int64_t out_rs,
                                                               int sum_batch, int sum_heads) {
  typedef Elem<T> E;
  const int cpr = (cols + 7) >> 3;  // chunks of 8 keys per row (the input rows are padded to whole chunks)
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (int64_t)rows * cpr) return;
  const int row = (int)(i / cpr), ch = (int)(i % cpr);
  const int ho = blockIdx.y, bo = blockIdx.z;
  const int b0 = sum_batch ? 0 : bo, b1 = sum_batch ? nb : bo + 1;
  const int h0 = sum_heads ? 0 : ho, h1 = sum_heads ? nh : ho + 1;
  float acc[8];
#pragma unroll
  for (int j = 0; j < 8; j++) acc[j] = 0.f;
  const T* const src = in + (int64_t)row * in_rs + ch * 8;
  for (int b = b0; b < b1; b++)
    for (int h = h0; h < h1; h++) {
      const typename E::vec8 v = *reinterpret_cast<const typename E::vec8*>(src + (int64_t)b * in_bs + (int64_t)h * in_hs);
#pragma unroll
      for (int j = 0; j < 8; j++) acc[j] += (float)v[j];
    }
  T* const dst = out + (int64_t)bo * out_bs + (int64_t)ho * out_hs + (int64_t)row * out_rs + ch * 8;
  if (kVecStore && ch * 8 + 8 <= cols) {
    typename E::vec8 r;
#pragma unroll
    for (int j = 0; j < 8; j++) r[j] = (T)acc[j];
    *reinterpret_cast<typename E::vec8*>(dst) = r;
  } else {
#pragma unroll
    for (int j = 0; j < 8; j++)
      if (ch * 8 + j < cols) dst[j] = (T)acc[j];
  }
}

}  // namespace

hipError_t launch_bias_grad_reduce(const void* in, void* out, int dtype, int nb, int nh, int rows, int cols, int64_t in_bs,
                                   int64_t in_hs, int64_t in_rs, int sum_batch, int sum_heads, int64_t out_bs, int64_t out_hs,
                                   int64_t out_rs, bool vec_store, hipStream_t stream) {
  if (nb == 0 || nh == 0 || rows == 0 || cols == 0) return hipSuccess;
  const int64_t n = (int64_t)rows * ((cols + 7) >> 3);
  const dim3 grid((unsigned)((n + 255) / 256), (unsigned)(sum_heads ? 1 : nh), (unsigned)(sum_batch ? 1 : nb));
#define FA_BGR(T, V)                                                                                                   \
  hipLaunchKernelGGL((bias_grad_reduce_kernel<T, V>), grid, dim3(256), 0, stream, reinterpret_cast<const T*>(in),      \
                     reinterpret_cast<T*>(out), nb, nh, rows, cols, in_bs, in_hs, in_rs, out_bs, out_hs, out_rs, sum_batch, \
                     sum_heads)
  if (dtype == 0) {
    if (vec_store) FA_BGR(_Float16, true); else FA_BGR(_Float16, false);
  } else {
    if (vec_store) FA_BGR(__bf16, true); else FA_BGR(__bf16, false);
  }
#undef FA_BGR
  return hipGetLastError();
}

}  // namespace fa
