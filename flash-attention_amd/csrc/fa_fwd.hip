// Forward launcher: picks the head-dimension specialisation (the role of run_fmha_fp16_sm80,
// csrc/flash_attn/src/fmha_fprop_fp16_kernel.sm80.cu:84-146).
#include "fa_common.h"
#include "fa_params.h"

namespace fa {

template <int D>
hipError_t launch_fwd_d(const FwdParams& p, int dtype, bool causal, bool dropout, bool sparse, hipStream_t stream);
template <> hipError_t launch_fwd_d<16>(const FwdParams&, int, bool, bool, bool, hipStream_t);
template <> hipError_t launch_fwd_d<32>(const FwdParams&, int, bool, bool, bool, hipStream_t);
template <> hipError_t launch_fwd_d<64>(const FwdParams&, int, bool, bool, bool, hipStream_t);
template <> hipError_t launch_fwd_d<128>(const FwdParams&, int, bool, bool, bool, hipStream_t);

hipError_t launch_fwd(const FwdParams& p, int dtype, int head_dim, bool causal, bool dropout, bool sparse,
                      hipStream_t stream) {
  switch (head_dim) {
    case 16: return launch_fwd_d<16>(p, dtype, causal, dropout, sparse, stream);
    case 32: return launch_fwd_d<32>(p, dtype, causal, dropout, sparse, stream);
    case 64: return launch_fwd_d<64>(p, dtype, causal, dropout, sparse, stream);
    case 128: return launch_fwd_d<128>(p, dtype, causal, dropout, sparse, stream);
    default: return hipErrorInvalidValue;
  }
}

// Merges the partial results of a key-split forward: lse = log sum_s exp(lse_s), o = sum_s exp(lse_s - lse) o_s.
// One thread per (batch, head, query row, 4 output columns).
template <typename T>
__global__ void __launch_bounds__(256) fwd_combine_kernel(const FwdParams p, int D) {
  const int cpr = D / 4;
  const int64_t total = (int64_t)p.B * p.H * p.max_sq * cpr;
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= total) return;
  const int ch = (int)(t % cpr);
  const int row = (int)((t / cpr) % p.max_sq);
  const int h = (int)((t / cpr / p.max_sq) % p.H);
  const int b = (int)(t / cpr / p.max_sq / p.H);
  int q_begin, Lq;
  if (!seq_extent(p.cu_q, b, p.total_q, p.max_sq, &q_begin, &Lq) || row >= Lq) return;
  // The splits are read eight at a time, all loads of a group in flight together: with few query rows (decoding) the
  // kernel has a handful of workgroups and its time is the latency of this loop, not bandwidth.
  constexpr int U = 8;
  const float* lp = p.lse_part + ((int64_t)b * p.H + h) * p.sq_r + row;
  const int64_t lstep = (int64_t)p.B * p.H * p.sq_r;
  const float* opart = p.o_part + ((int64_t)(q_begin + row) * p.H + h) * D + ch * 4;
  const int64_t ostep = (int64_t)p.total_q * p.H * D;
  float m = -INFINITY;
  for (int s0 = 0; s0 < p.n_splits; s0 += U) {
    float l[U];
#pragma unroll
    for (int u = 0; u < U; u++) l[u] = s0 + u < p.n_splits ? lp[(s0 + u) * lstep] : -INFINITY;
#pragma unroll
    for (int u = 0; u < U; u++) m = fmaxf(m, l[u]);
  }
  float sum = 0.f;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  if (m > -INFINITY) {
    for (int s0 = 0; s0 < p.n_splits; s0 += U) {
      float l[U];
      f32x4 o[U];
#pragma unroll
      for (int u = 0; u < U; u++) {
        const bool in = s0 + u < p.n_splits;
        l[u] = in ? lp[(s0 + u) * lstep] : -INFINITY;
        o[u] = in ? *reinterpret_cast<const f32x4*>(opart + (s0 + u) * ostep) : f32x4{0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
      for (int u = 0; u < U; u++) {
        const float w = __expf(l[u] - m);  // 0 for a split past the end or without keys
        sum += w;
        acc = acc + o[u] * w;
      }
    }
    acc = acc * (1.f / sum);
  }
  if (ch == 0) p.lse[((int64_t)b * p.H + h) * p.sq_r + row] = m > -INFINITY ? m + __logf(sum) : -INFINITY;
  T* op = reinterpret_cast<T*>(p.o) + (int64_t)(q_begin + row) * p.o_rs + (int64_t)h * p.o_hs + ch * 4;
  *reinterpret_cast<typename Elem<T>::vec4*>(op) = cvt4<T>(acc);
}

hipError_t launch_fwd_combine(const FwdParams& p, int dtype, int head_dim, hipStream_t stream) {
  const int64_t total = (int64_t)p.B * p.H * p.max_sq * (head_dim / 4);
  if (total == 0) return hipSuccess;
  const unsigned grid = (unsigned)((total + 255) / 256);
  if (dtype == 0) hipLaunchKernelGGL(fwd_combine_kernel<_Float16>, dim3(grid), dim3(256), 0, stream, p, head_dim);
  else hipLaunchKernelGGL(fwd_combine_kernel<__bf16>, dim3(grid), dim3(256), 0, stream, p, head_dim);
  return hipGetLastError();
}

}  // namespace fa
