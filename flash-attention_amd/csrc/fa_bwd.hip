// Backward launcher: picks the head-dimension specialisation (the role of run_fmha_dgrad_fp16_sm80,
// csrc/flash_attn/src/fmha_dgrad_fp16_kernel_loop.sm80.cu:54-102).
#include "fa_params.h"

namespace fa {

template <int D>
hipError_t launch_bwd_d(const BwdParams& p, int which, int dtype, bool causal, bool dropout, bool sparse,
                        hipStream_t stream);
template <> hipError_t launch_bwd_d<16>(const BwdParams&, int, int, bool, bool, bool, hipStream_t);
template <> hipError_t launch_bwd_d<32>(const BwdParams&, int, int, bool, bool, bool, hipStream_t);
template <> hipError_t launch_bwd_d<64>(const BwdParams&, int, int, bool, bool, bool, hipStream_t);
template <> hipError_t launch_bwd_d<128>(const BwdParams&, int, int, bool, bool, bool, hipStream_t);

hipError_t launch_bwd(const BwdParams& p, int which, int dtype, int head_dim, bool causal, bool dropout, bool sparse,
                      hipStream_t stream) {
  switch (head_dim) {
    case 16: return launch_bwd_d<16>(p, which, dtype, causal, dropout, sparse, stream);
    case 32: return launch_bwd_d<32>(p, which, dtype, causal, dropout, sparse, stream);
    case 64: return launch_bwd_d<64>(p, which, dtype, causal, dropout, sparse, stream);
    case 128: return launch_bwd_d<128>(p, which, dtype, causal, dropout, sparse, stream);
    default: return hipErrorInvalidValue;
  }
}

// Adds up the partial dQ of a key-split backward (BwdParams::dq_part) and writes dq in the tensor dtype.
// One thread per (batch, head, query row, 4 columns).
template <typename T>
__global__ void __launch_bounds__(256) dq_combine_kernel(const BwdParams p, int D) {
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
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  constexpr int U = 8;  // eight splits' loads in flight at a time (see fwd_combine_kernel)
  const float* part = p.dq_part + ((int64_t)(q_begin + row) * p.H + h) * D + ch * 4;
  const int64_t step = (int64_t)p.total_q * p.H * D;
  for (int s0 = 0; s0 < p.n_splits; s0 += U) {
    f32x4 x[U];
#pragma unroll
    for (int u = 0; u < U; u++)
      x[u] = s0 + u < p.n_splits ? *reinterpret_cast<const f32x4*>(part + (s0 + u) * step) : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < U; u++) acc = acc + x[u];
  }
  T* op = reinterpret_cast<T*>(p.dq) + (int64_t)(q_begin + row) * p.dq_rs + (int64_t)h * p.dq_hs + ch * 4;
  *reinterpret_cast<typename Elem<T>::vec4*>(op) = cvt4<T>(acc);
}

hipError_t launch_dq_combine(const BwdParams& p, int dtype, int head_dim, hipStream_t stream) {
  const int64_t total = (int64_t)p.B * p.H * p.max_sq * (head_dim / 4);
  if (total == 0) return hipSuccess;
  const unsigned grid = (unsigned)((total + 255) / 256);
  if (dtype == 0) hipLaunchKernelGGL(dq_combine_kernel<_Float16>, dim3(grid), dim3(256), 0, stream, p, head_dim);
  else hipLaunchKernelGGL(dq_combine_kernel<__bf16>, dim3(grid), dim3(256), 0, stream, p, head_dim);
  return hipGetLastError();
}

}  // namespace fa
