// Launcher of the one-kernel backward (fa_bwd_fused_kernel.h): softmax_d pass (which also clears the hand-over counters),
// then the kernel.
#include "fa_bwd_fused_kernel.h"

#ifdef FA_FUSED_EXPERIMENTS
#include <cstdio>
#include <cstdlib>
#endif

namespace fa {

namespace {
template <typename T>
hipError_t launch_fused_t(const BwdParams& p0, hipStream_t stream, hipEvent_t ev_start, hipEvent_t ev_stop) {
  BwdParams p = p0;
  const int BH = p.B * p.H;
#ifdef FA_FUSED_EXPERIMENTS
  static const int ring_stride = getenv("FA_RING_STRIDE") ? atoi(getenv("FA_RING_STRIDE")) : 0;
  p.ring_stride = ring_stride;
#endif
  const dim3 gd((p.max_sq + 31) / 32, BH);
  hipLaunchKernelGGL(fused_prepass_kernel<T>, gd, dim3(256), 0, stream, p);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  const int grid = tile_grid(false, p.nk_tiles, BH);
  if (ev_start && (e = hipEventRecord(ev_start, stream)) != hipSuccess) return e;
#ifdef FA_FUSED_EXPERIMENTS
  static const int mode = getenv("FA_FUSED_MODE") ? atoi(getenv("FA_FUSED_MODE")) : 0;
  if (mode == 1) hipLaunchKernelGGL((fa_bwd_fused_kernel<T, 64, 1>), dim3(grid), dim3(256), 0, stream, p);
  else if (mode == 2) hipLaunchKernelGGL((fa_bwd_fused_kernel<T, 64, 2>), dim3(grid), dim3(256), 0, stream, p);
  else if (mode == 3) hipLaunchKernelGGL((fa_bwd_fused_kernel<T, 64, 3>), dim3(grid), dim3(256), 0, stream, p);
  else if (mode == 4) hipLaunchKernelGGL((fa_bwd_fused_kernel<T, 64, 4>), dim3(grid), dim3(256), 0, stream, p);

  else
#endif
  hipLaunchKernelGGL((fa_bwd_fused_kernel<T, 64, 0>), dim3(grid), dim3(256), 0, stream, p);
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  if (ev_stop && (e = hipEventRecord(ev_stop, stream)) != hipSuccess) return e;
  return hipSuccess;
}
}  // namespace

hipError_t launch_bwd_fused(const BwdParams& p, int dtype, hipStream_t stream, hipEvent_t ev_start, hipEvent_t ev_stop) {
  if (p.B * p.H == 0) return hipSuccess;
  if (dtype == 0) return launch_fused_t<_Float16>(p, stream, ev_start, ev_stop);
  return launch_fused_t<__bf16>(p, stream, ev_start, ev_stop);
}

}  // namespace fa
