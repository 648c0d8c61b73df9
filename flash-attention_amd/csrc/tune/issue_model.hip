// Micro-benchmarks of the gfx950 compute unit that the attention kernels' tile shapes are argued from:
//   1. sustained MFMA rate (v_mfma_f32_32x32x16_f16) and the clock it runs at,
//   2. whether VALU work overlaps with MFMA work, within one wave and across waves of one SIMD,
//   3. issue cost of the VALU instructions the softmax uses (fma, exp2, max, integer multiply),
//   4. LDS read bandwidth of ds_read_b128 and ds_read_b64_tr_b16 for the row strides the kernels use.
// Build and run:  hipcc --offload-arch=gfx950 -O3 issue_model.hip -o issue_model && ./issue_model
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
#define LDSA __attribute__((address_space(3)))

static float* g_out = nullptr;

template <typename F>
static float time_ms(F launch) {
  hipEvent_t e0, e1;
  hipEventCreate(&e0);
  hipEventCreate(&e1);
  launch();
  hipEventRecord(e0);
  launch();
  hipEventRecord(e1);
  hipEventSynchronize(e1);
  float ms;
  hipEventElapsedTime(&ms, e0, e1);
  return ms;
}

// ---- 1 + 2a: NACC independent MFMA chains, each MFMA followed by NV independent fp32 FMAs, in one wave
template <int NACC, int NV>
__global__ void __launch_bounds__(256) mfma_valu_kernel(float* out, int iters, long long* clk) {
  f16x8 a, b;
  for (int i = 0; i < 8; i++) { a[i] = (_Float16)(threadIdx.x * 0.001f + i); b[i] = (_Float16)(i * 0.5f); }
  f32x16 acc[NACC];
  for (int n = 0; n < NACC; n++) for (int i = 0; i < 16; i++) acc[n][i] = 0;
  float xs[8];
  for (int i = 0; i < 8; i++) xs[i] = threadIdx.x + i;
  const float y = 1.0001f;
  const long long t0 = __builtin_readcyclecounter(), w0 = wall_clock64();
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int n = 0; n < NACC; n++) {
      acc[n] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[n], 0, 0, 0);
#pragma unroll
      for (int v = 0; v < NV; v++) xs[v & 7] = __builtin_fmaf(xs[v & 7], y, 0.5f);
    }
  }
  const long long t1 = __builtin_readcyclecounter(), w1 = wall_clock64();
  float s = 0;
  for (int i = 0; i < 8; i++) s += xs[i];
  for (int n = 0; n < NACC; n++) s += acc[n][0] + acc[n][7];
  out[blockIdx.x * 256 + threadIdx.x] = s;
  if (blockIdx.x == 0 && threadIdx.x == 0) { clk[0] = t1 - t0; clk[1] = w1 - w0; }
}

template <int NACC, int NV>
static void run_mfma_valu(int blocks) {
  static long long* clk = nullptr;
  if (!clk) hipMalloc(&clk, 16);
  const int iters = 4000;
  const float ms = time_ms([&] { mfma_valu_kernel<NACC, NV><<<blocks, 256>>>(g_out, iters, clk); });
  long long h[2];
  hipMemcpy(h, clk, 16, hipMemcpyDeviceToHost);
  const double flops = (double)blocks * 4 * iters * NACC * 32768.0;
  printf("  1 MFMA + %2d FMA per step, %d wave(s)/SIMD: %8.1f TFLOP/s of MFMA work, shader clock %.2f GHz\n", NV, blocks / 256,
         flops / ms / 1e9, h[0] / (h[1] / 100.0) / 1e3);
}

// ---- 2b: two waves per SIMD; waves 0-3 of a 512-thread block only issue MFMAs, waves 4-7 only VALU
template <int MODE, bool EXP>
__global__ void __launch_bounds__(512) roles_kernel(float* out, int n_mfma, int n_valu) {
  const int wave = threadIdx.x >> 6;
  f16x8 a, b;
  for (int i = 0; i < 8; i++) { a[i] = (_Float16)(threadIdx.x * 0.001f + i); b[i] = (_Float16)(i * 0.5f); }
  f32x16 acc[4];
  for (int n = 0; n < 4; n++) for (int i = 0; i < 16; i++) acc[n][i] = 0;
  float xs[8];
  for (int i = 0; i < 8; i++) xs[i] = threadIdx.x * 1e-3f + i;
  const float y = 1.0001f;
  if (MODE == 0 || (MODE == 2 && wave < 4)) {
    for (int it = 0; it < n_mfma; it++) {
#pragma unroll
      for (int n = 0; n < 4; n++) acc[n] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[n], 0, 0, 0);
    }
  }
  if (MODE == 1 || (MODE == 2 && wave >= 4)) {
    for (int it = 0; it < n_valu; it++) {
#pragma unroll
      for (int v = 0; v < 32; v++) xs[v & 7] = EXP ? __builtin_amdgcn_exp2f(xs[v & 7]) : __builtin_fmaf(xs[v & 7], y, 0.5f);
    }
  }
  float s = 0;
  for (int i = 0; i < 8; i++) s += xs[i];
  for (int n = 0; n < 4; n++) s += acc[n][0] + acc[n][7];
  out[blockIdx.x * 512 + threadIdx.x] = s;
}

// ---- 3: issue cost of single instruction kinds (2 waves per SIMD, 8 independent chains)
template <int OP>
__global__ void __launch_bounds__(512) op_kernel(float* out, int iters) {
  float xs[8];
  unsigned us[8];
  for (int i = 0; i < 8; i++) { xs[i] = threadIdx.x * 1e-3f + i * 0.01f; us[i] = threadIdx.x + i; }
  const float y = 1.0001f;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int v = 0; v < 32; v++) {
      const int i = v & 7;
      if (OP == 0) xs[i] = __builtin_fmaf(xs[i], y, 0.5f);
      if (OP == 1) xs[i] = __builtin_amdgcn_exp2f(xs[i]);
      if (OP == 2) xs[i] = fmaxf(xs[i], xs[(i + 1) & 7]);
      if (OP == 3) us[i] = us[i] * 0x9E3779B9u + 12345u;
      if (OP == 4) us[i] = __umulhi(us[i], 0xD2511F53u);
      if (OP == 5) xs[i] = __builtin_amdgcn_rcpf(xs[i]);
    }
  }
  float s = 0;
  for (int i = 0; i < 8; i++) s += xs[i] + (float)us[i];
  out[blockIdx.x * 512 + threadIdx.x] = s;
}

template <int OP>
static void run_op(const char* name, double ghz) {
  const int iters = 2000;
  const float ms = time_ms([&] { op_kernel<OP><<<256, 512>>>(g_out, iters); });
  printf("  %-24s %5.2f cycles per wave64 instruction per SIMD\n", name, ms * 1e-3 * ghz * 1e9 / (2.0 * iters * 32));
}

// ---- 4: LDS read bandwidth for a given per-lane byte offset pattern
template <int MODE>
__global__ void __launch_bounds__(256) lds_kernel(const int* offs, int iters, uint32_t* out) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[65536];
  for (int i = threadIdx.x; i < 65536 / 4; i += 256) ((uint32_t*)lds)[i] = i;
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int off = (offs[lane] + wave * 4096) & 0xffff;
  uint32_t acc = 0;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int u = 0; u < 16; u++) {
      if (MODE == 0) { u32x4 v = *(volatile LDSA u32x4*)(LDSA char*)(lds + off); acc += v[0] ^ v[3]; }
      if (MODE == 1) { i16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDSA i16x4*)(LDSA char*)(lds + off)); acc += v[0] ^ v[3]; asm volatile("" ::: "memory"); }
    }
  }
  out[blockIdx.x * 256 + threadIdx.x] = acc;
}

static void run_lds(const char* name, int mode, const int* offs, double ghz) {
  static int* d_offs = nullptr;
  if (!d_offs) hipMalloc(&d_offs, 256);
  hipMemcpy(d_offs, offs, 256, hipMemcpyHostToDevice);
  const int iters = 2000, blocks = 512;
  const float ms = mode == 0 ? time_ms([&] { lds_kernel<0><<<blocks, 256>>>(d_offs, iters, (uint32_t*)g_out); })
                             : time_ms([&] { lds_kernel<1><<<blocks, 256>>>(d_offs, iters, (uint32_t*)g_out); });
  const double bytes = (double)blocks * 4 * 64 * (mode == 0 ? 16 : 8) * 16 * iters;
  printf("  %-52s %6.1f B/clk/CU\n", name, bytes / 256 / (ms * 1e-3 * ghz * 1e9));
}

int main() {
  hipMalloc(&g_out, 4 * 512 * 4096);
  printf("1. MFMA rate, and 2a. MFMA followed by independent FMAs in the same wave\n");
  run_mfma_valu<4, 0>(256);
  run_mfma_valu<4, 0>(512);
  run_mfma_valu<4, 4>(512);
  run_mfma_valu<4, 8>(512);
  run_mfma_valu<4, 12>(512);
  run_mfma_valu<4, 16>(512);

  printf("2b. one MFMA-only wave and one VALU-only wave on each SIMD (same instruction counts per SIMD in all three runs)\n");
  const int nm = 4000, nv = 4000;
  const float t_m = time_ms([&] { roles_kernel<0, false><<<256, 512>>>(g_out, nm / 2, 0); });
  const float t_v = time_ms([&] { roles_kernel<1, false><<<256, 512>>>(g_out, 0, nv / 2); });
  const float t_x = time_ms([&] { roles_kernel<2, false><<<256, 512>>>(g_out, nm, nv); });
  const float t_e = time_ms([&] { roles_kernel<1, true><<<256, 512>>>(g_out, 0, nv / 2); });
  const float t_xe = time_ms([&] { roles_kernel<2, true><<<256, 512>>>(g_out, nm, nv); });
  printf("  fma : MFMA only %.3f ms, VALU only %.3f ms, both %.3f ms (sum %.3f, max %.3f)\n", t_m, t_v, t_x, t_m + t_v, t_m > t_v ? t_m : t_v);
  printf("  exp2: MFMA only %.3f ms, VALU only %.3f ms, both %.3f ms (sum %.3f, max %.3f)\n", t_m, t_e, t_xe, t_m + t_e, t_m > t_e ? t_m : t_e);

  const double ghz = 2.4;  // VALU-only kernels run at the boost clock
  printf("3. issue cost of VALU instructions (assuming %.1f GHz)\n", ghz);
  run_op<0>("v_fma_f32", ghz);
  run_op<1>("v_exp_f32", ghz);
  run_op<5>("v_rcp_f32", ghz);
  run_op<2>("v_max_f32", ghz);
  run_op<3>("v_mul_lo_u32 + add", ghz);
  run_op<4>("v_mul_hi_u32", ghz);

  printf("4. LDS read bandwidth (assuming %.1f GHz), 8 waves per CU\n", ghz);
  int offs[64];
  for (int l = 0; l < 64; l++) offs[l] = l * 16;
  run_lds("ds_read_b128, contiguous", 0, offs, ghz);
  const int bstr[] = {128, 144, 272, 304, 80, 48};
  for (int s : bstr) {
    for (int l = 0; l < 64; l++) offs[l] = (l % 32) * s + (l / 32) * 16;
    char nm_[80];
    snprintf(nm_, 80, "ds_read_b128 row fragment, row stride %d B", s);
    run_lds(nm_, 0, offs, ghz);
  }
  for (int l = 0; l < 64; l++) offs[l] = l * 8;
  run_lds("ds_read_b64_tr_b16, contiguous", 1, offs, ghz);
  const int tstr[] = {128, 144, 272, 288, 304, 80, 48};
  for (int s : tstr) {
    for (int l = 0; l < 64; l++) {
      const int j = l & 15, g = l >> 4, hf = l >> 5;
      offs[l] = (4 * hf + (j >> 2)) * s + (16 * (g & 1) + 4 * (j & 3)) * 2;
    }
    char nm_[80];
    snprintf(nm_, 80, "ds_read_b64_tr_b16 transposed fragment, row stride %d B", s);
    run_lds(nm_, 1, offs, ghz);
  }
  printf("done: %s\n", hipGetErrorString(hipDeviceSynchronize()));
  return 0;
}
