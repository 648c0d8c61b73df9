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

}  // namespace fa
