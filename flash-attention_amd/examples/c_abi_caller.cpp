// A caller of libflash_attn_gfx950.so that knows nothing of Python or torch: device buffers from hipMalloc, the
// argument structs of include/flash_attn_gfx950.h, one forward and one backward of a small ragged batch, and a check of
// o, lse, dq, dk, dv against the closed form evaluated in double precision on the host
// (softmax(scale Q K^T) V and its gradients; the formulas of flash_attn/flash_attn_interface.py's attention).
// Exit status 0 and "PASS" if every output is within the stated tolerance.
//
// Build: hipcc -O2 -std=c++17 -I include flash-attention_amd/examples/c_abi_caller.cpp \
//              -L flash-attention_amd/flash_attn -lflash_attn_gfx950 -Wl,-rpath,'$ORIGIN/../flash_attn' -o c_abi_caller
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "flash_attn_gfx950.h"

#define HIP_OK(x)                                                                       \
  do {                                                                                  \
    hipError_t e_ = (x);                                                                \
    if (e_ != hipSuccess) {                                                             \
      std::fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));                      \
      return 2;                                                                         \
    }                                                                                   \
  } while (0)

namespace {

typedef _Float16 half_t;

// deterministic pseudo-normal values (sum of uniforms), exactly representable after the fp16 rounding both sides see
float next_value(uint64_t* state) {
  float acc = 0.f;
  for (int i = 0; i < 4; i++) {
    *state = *state * 6364136223846793005ull + 1442695040888963407ull;
    acc += (float)((*state >> 40) & 0xffff) / 65536.f - 0.5f;
  }
  return acc * 1.7f;
}

template <typename T>
T* to_device(const std::vector<T>& h) {
  T* d = nullptr;
  if (hipMalloc(&d, h.size() * sizeof(T)) != hipSuccess) return nullptr;
  if (hipMemcpy(d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice) != hipSuccess) return nullptr;
  return d;
}

double max_err(const std::vector<half_t>& got, const std::vector<double>& want) {
  double m = 0;
  for (size_t i = 0; i < want.size(); i++) m = std::fmax(m, std::fabs((double)(float)got[i] - want[i]));
  return m;
}

}  // namespace

int main() {
  const int B = 3, H = 2, D = 64;
  const int lens[B] = {100, 37, 129};
  const bool causal = true;
  const float scale = 0.125f;
  std::vector<int32_t> cu(B + 1, 0);
  for (int b = 0; b < B; b++) cu[b + 1] = cu[b] + lens[b];
  const int total = cu[B], max_len = 129;
  const size_t n = (size_t)total * H * D;

  // packed qkv [total, 3, H, D] as the reference's qkv-packed interface holds it, dout [total, H, D]
  std::vector<half_t> qkv(3 * n), dout(n);
  uint64_t st = 42;
  for (auto& x : qkv) x = (half_t)next_value(&st);
  for (auto& x : dout) x = (half_t)next_value(&st);
  auto at = [&](int which, int row, int h, int d) { return (double)(float)qkv[(((size_t)row * 3 + which) * H + h) * D + d]; };

  int32_t sq_r = 0, sk_r = 0;
  fa_round_seqlens(D, max_len, max_len, 0, &sq_r, &sk_r);

  half_t* d_qkv = to_device(qkv);
  half_t* d_dout = to_device(dout);
  int32_t* d_cu = to_device(cu);
  half_t *d_o = nullptr, *d_dqkv = nullptr;
  float *d_lse = nullptr, *d_sd = nullptr;
  HIP_OK(hipMalloc(&d_o, n * sizeof(half_t)));
  HIP_OK(hipMalloc(&d_dqkv, 3 * n * sizeof(half_t)));
  HIP_OK(hipMalloc(&d_lse, (size_t)B * H * sq_r * sizeof(float)));
  HIP_OK(hipMalloc(&d_sd, (size_t)B * H * sq_r * sizeof(float)));
  if (!d_qkv || !d_dout || !d_cu) return 2;
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));

  fa_fwd_args f;
  std::memset(&f, 0, sizeof(f));
  f.struct_bytes = sizeof(f);
  f.dtype = FA_FP16;
  f.q = d_qkv; f.k = d_qkv + (size_t)H * D; f.v = d_qkv + 2 * (size_t)H * D;
  f.o = d_o; f.softmax_lse = d_lse;
  f.cu_seqlens_q = d_cu; f.cu_seqlens_k = d_cu;
  f.q_row_stride = f.k_row_stride = f.v_row_stride = 3 * H * D;
  f.q_head_stride = f.k_head_stride = f.v_head_stride = D;
  f.o_row_stride = H * D; f.o_head_stride = D;
  f.batch = B; f.nheads = H; f.head_dim = D;
  f.total_q = f.total_k = total; f.max_seqlen_q = f.max_seqlen_k = max_len;
  f.p_dropout = 0.f; f.softmax_scale = scale; f.is_causal = causal;
  f.stream = stream;
  if (fa_fwd_workspace_bytes(&f) != 0) { std::fprintf(stderr, "dense forward must not need scratch\n"); return 1; }
  if (fa_fwd(&f) != FA_OK) { std::fprintf(stderr, "fa_fwd: %s\n", fa_last_error()); return 1; }

  fa_bwd_args g;
  std::memset(&g, 0, sizeof(g));
  g.struct_bytes = sizeof(g);
  g.dtype = FA_FP16;
  g.dout = d_dout; g.q = f.q; g.k = f.k; g.v = f.v; g.out = d_o; g.softmax_lse = d_lse;
  g.dq = d_dqkv; g.dk = d_dqkv + (size_t)H * D; g.dv = d_dqkv + 2 * (size_t)H * D; g.softmax_d = d_sd;
  g.cu_seqlens_q = d_cu; g.cu_seqlens_k = d_cu;
  g.do_row_stride = g.o_row_stride = H * D; g.do_head_stride = g.o_head_stride = D;
  g.q_row_stride = g.k_row_stride = g.v_row_stride = g.dq_row_stride = g.dk_row_stride = g.dv_row_stride = 3 * H * D;
  g.q_head_stride = g.k_head_stride = g.v_head_stride = g.dq_head_stride = g.dk_head_stride = g.dv_head_stride = D;
  g.lse_seq_stride = sq_r;
  g.batch = B; g.nheads = H; g.head_dim = D;
  g.total_q = g.total_k = total; g.max_seqlen_q = g.max_seqlen_k = max_len;
  g.p_dropout = 0.f; g.softmax_scale = scale; g.is_causal = causal;
  g.stream = stream;
  if (fa_bwd_workspace_bytes(&g) != 0) { std::fprintf(stderr, "dense backward must not need scratch\n"); return 1; }
  if (fa_bwd(&g) != FA_OK) { std::fprintf(stderr, "fa_bwd: %s\n", fa_last_error()); return 1; }
  HIP_OK(hipStreamSynchronize(stream));

  std::vector<half_t> o(n), dqkv(3 * n);
  std::vector<float> lse((size_t)B * H * sq_r);
  HIP_OK(hipMemcpy(o.data(), d_o, n * sizeof(half_t), hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(dqkv.data(), d_dqkv, 3 * n * sizeof(half_t), hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(lse.data(), d_lse, lse.size() * sizeof(float), hipMemcpyDeviceToHost));

  // ---- closed form in double precision
  std::vector<double> o_ref(n, 0.0), dq_ref(n, 0.0), dk_ref(n, 0.0), dv_ref(n, 0.0);
  double lse_err = 0;
  for (int b = 0; b < B; b++)
    for (int h = 0; h < H; h++) {
      const int L = lens[b], r0 = cu[b];
      std::vector<double> P((size_t)L * L, 0.0);
      for (int i = 0; i < L; i++) {
        const int jmax = causal ? i : L - 1;
        double m = -1e300, l = 0;
        std::vector<double> s(L, 0.0);
        for (int j = 0; j <= jmax; j++) {
          double acc = 0;
          for (int d = 0; d < D; d++) acc += at(0, r0 + i, h, d) * at(1, r0 + j, h, d);
          s[j] = acc * scale;
          m = std::fmax(m, s[j]);
        }
        for (int j = 0; j <= jmax; j++) l += std::exp(s[j] - m);
        lse_err = std::fmax(lse_err, std::fabs((double)lse[((size_t)b * H + h) * sq_r + i] - (m + std::log(l))));
        for (int j = 0; j <= jmax; j++) {
          P[(size_t)i * L + j] = std::exp(s[j] - m) / l;
          for (int d = 0; d < D; d++) o_ref[((size_t)(r0 + i) * H + h) * D + d] += P[(size_t)i * L + j] * at(2, r0 + j, h, d);
        }
      }
      for (int i = 0; i < L; i++) {
        std::vector<double> dP(L, 0.0);
        double Dk = 0;
        for (int j = 0; j < L; j++) {
          const double p = P[(size_t)i * L + j];
          if (p == 0.0) continue;
          for (int d = 0; d < D; d++) dP[j] += (double)(float)dout[((size_t)(r0 + i) * H + h) * D + d] * at(2, r0 + j, h, d);
          Dk += p * dP[j];
        }
        for (int j = 0; j < L; j++) {
          const double p = P[(size_t)i * L + j];
          if (p == 0.0) continue;
          const double dS = p * (dP[j] - Dk) * scale;
          for (int d = 0; d < D; d++) {
            dq_ref[((size_t)(r0 + i) * H + h) * D + d] += dS * at(1, r0 + j, h, d);
            dk_ref[((size_t)(r0 + j) * H + h) * D + d] += dS * at(0, r0 + i, h, d);
            dv_ref[((size_t)(r0 + j) * H + h) * D + d] += p * (double)(float)dout[((size_t)(r0 + i) * H + h) * D + d];
          }
        }
      }
    }
  std::vector<half_t> dq(n), dk(n), dv(n);
  for (int row = 0; row < total; row++)
    for (int hd = 0; hd < H * D; hd++) {
      dq[(size_t)row * H * D + hd] = dqkv[((size_t)row * 3 + 0) * H * D + hd];
      dk[(size_t)row * H * D + hd] = dqkv[((size_t)row * 3 + 1) * H * D + hd];
      dv[(size_t)row * H * D + hd] = dqkv[((size_t)row * 3 + 2) * H * D + hd];
    }
  const double e_o = max_err(o, o_ref), e_dq = max_err(dq, dq_ref), e_dk = max_err(dk, dk_ref), e_dv = max_err(dv, dv_ref);
  std::printf("max |error|: o %.2e  lse %.2e  dq %.2e  dk %.2e  dv %.2e\n", e_o, lse_err, e_dq, e_dk, e_dv);
  // fp16 outputs of magnitude O(1): half an ulp is 5e-4; the gradients sum up to 129 rounded terms
  const bool ok = e_o < 2e-3 && lse_err < 1e-3 && e_dq < 8e-3 && e_dk < 8e-3 && e_dv < 8e-3;
  std::printf(ok ? "PASS\n" : "FAIL\n");
  hipFree(d_qkv); hipFree(d_dout); hipFree(d_cu); hipFree(d_o); hipFree(d_dqkv); hipFree(d_lse); hipFree(d_sd);
  hipStreamDestroy(stream);
  return ok ? 0 : 1;
}
