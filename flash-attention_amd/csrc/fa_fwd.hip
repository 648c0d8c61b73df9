// Forward launcher: picks the head-dimension specialisation (the role of run_fmha_fp16_sm80,
// csrc/flash_attn/src/fmha_fprop_fp16_kernel.sm80.cu:84-146).
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

}  // namespace fa
