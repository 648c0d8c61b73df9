// Micro-benchmarks of the gfx950 compute unit that the attention kernels' design is argued from:
//   1. sustained MFMA rate (v_mfma_f32_32x32x16_f16) and the shader clock it settles at, with constant and with
//      random operands (the part is power limited: toggling operands lower the clock),
//   2. cost of VALU / transcendental instructions issued between MFMAs (they do not run underneath an MFMA, whether
//      they come from the same wave or from another wave of the SIMD), and what the accumulators' register file costs,
//   3. issue cost of the VALU instructions the softmax uses, on their own,
//   4. LDS read bandwidth of ds_read_b128 row fragments and ds_read_b64_tr_b16 transposed fragments for padded row
//      strides and for the unpadded, chunk-swizzled tile layouts of fa_stage.h.
// Every measurement runs under sustained load (the clock governor needs tens of milliseconds to settle) and reads the
// shader clock inside the kernel (cycle counter against the 100 MHz wall clock).
// Build and run, from the repository root, with the flags the kernels are built with:
//   hipcc --offload-arch=gfx950 -O3 -std=c++17 -Xclang -target-feature -Xclang -packed-fp32-ops
//         flash-attention_amd/csrc/tune/issue_model.hip -o issue_model && ./issue_model
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <vector>

#include "../fa_stage.h"

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
using fa::f16x8;
using fa::u32x4;
#define LDSA __attribute__((address_space(3)))

__device__ long long g_clk[2];
static float* g_out = nullptr;
static f16x8* g_src = nullptr;  // 4096 fragments of operand data

// Launches `launch` repeatedly (settle launches untimed, then `n` timed ones); returns ms per launch and the shader
// clock (GHz) that workgroup 0 observed during the last launch.
template <typename F>
static float time_ms(F launch, double* ghz, int settle = 40, int n = 10) {
  hipEvent_t e0, e1;
  hipEventCreate(&e0);
  hipEventCreate(&e1);
  for (int i = 0; i < settle; i++) launch();
  hipEventRecord(e0);
  for (int i = 0; i < n; i++) launch();
  hipEventRecord(e1);
  hipEventSynchronize(e1);
  float ms;
  hipEventElapsedTime(&ms, e0, e1);
  long long hc[2];
  hipMemcpyFromSymbol(hc, HIP_SYMBOL(g_clk), 16);
  if (ghz) *ghz = hc[0] / (hc[1] / 100.0) / 1e3;
  return ms / n;
}

struct ClockProbe {
  long long c0 = 0, w0 = 0;
  __device__ void start() {
    if (blockIdx.x == 0 && threadIdx.x == 0) { c0 = __builtin_readcyclecounter(); w0 = wall_clock64(); }
  }
  __device__ void stop() {
    if (blockIdx.x == 0 && threadIdx.x == 0) { g_clk[0] = __builtin_readcyclecounter() - c0; g_clk[1] = wall_clock64() - w0; }
  }
};

// ---- 1 + 2: 8 MFMAs per trip over 4 independent accumulators; operands rotate over 8 A and 8 B fragments taken from
// `src`; NV independent fp32 FMAs and NE exp2 follow every MFMA.
// FORM 0: the compiler's choice for this kernel, accumulators in AccVGPRs (it has the whole register file);
// FORM 1: accumulators in ordinary VGPRs, the form the attention kernels' MFMAs have (their results feed the VALU).
// SPLIT: workgroups with an even id only issue the MFMAs, those with an odd id only the VALU work; at two workgroups per
// compute unit every SIMD then holds one wave of each kind.
template <int NV, int NE, int FORM = 0, bool SPLIT = false>
__global__ void __launch_bounds__(256) mfma_mix_kernel(const f16x8* __restrict__ src, float* out, int iters) {
  ClockProbe probe;
  probe.start();
  const int tid = threadIdx.x, lane = tid & 63;
  f16x8 A[8], Bv[8];
  for (int i = 0; i < 8; i++) {
    A[i] = src[(lane * 8 + i + blockIdx.x * 3) & 4095];
    Bv[i] = src[(lane * 8 + i + 2048 + tid) & 4095];
  }
  f32x16 acc[4];
  for (int n = 0; n < 4; n++)
    for (int i = 0; i < 16; i++) acc[n][i] = 0;
  float xs[8];
  for (int i = 0; i < 8; i++) xs[i] = lane * 0.37f + i;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int u = 0; u < 8; u++) {
      if (!SPLIT || (blockIdx.x & 1) == 0) {
        if (FORM == 1)
          asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc[u & 3]) : "v"(A[u]), "v"(Bv[(u * 3 + 1) & 7]));
        else
          acc[u & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A[u], Bv[(u * 3 + 1) & 7], acc[u & 3], 0, 0, 0);
      }
      if (!SPLIT || (blockIdx.x & 1) == 1) {
#pragma unroll
        for (int v = 0; v < NV; v++) xs[v & 7] = __builtin_fmaf(xs[v & 7], 0.999f, 0.37f);
#pragma unroll
        for (int v = 0; v < NE; v++) xs[(v + 4) & 7] = __builtin_amdgcn_exp2f(xs[(v + 4) & 7] * 0.03f);
      }
    }
    if ((it & 63) == 63)
      for (int n = 0; n < 4; n++) acc[n] = acc[n] * 0.001f;  // keep the accumulators bounded
  }
  float s = 0;
  for (int i = 0; i < 8; i++) s += xs[i];
  for (int n = 0; n < 4; n++)
    for (int i = 0; i < 16; i++) s += acc[n][i];
  out[blockIdx.x * 256 + tid] = s;
  probe.stop();
}

template <int NV, int NE, int FORM = 0, bool SPLIT = false>
static void run_mix(const char* name, int waves_per_simd) {
  const int iters = 2000, blocks = 256 * waves_per_simd;
  double ghz;
  const float ms = time_ms([&] { mfma_mix_kernel<NV, NE, FORM, SPLIT><<<blocks, 256>>>(g_src, g_out, iters); }, &ghz);
  const int mfma_waves = SPLIT ? waves_per_simd / 2 : waves_per_simd;  // waves per SIMD that issue MFMAs
  const double flops = (double)blocks / waves_per_simd * mfma_waves * 4 * iters * 8 * 32768.0;
  printf("  %-34s %d wave(s)/SIMD: %7.1f TFLOP/s, clock %.2f GHz, %5.1f cycles per MFMA slot\n", name, waves_per_simd,
         flops / ms / 1e9, ghz, ms * 1e-3 * ghz * 1e9 / ((double)iters * 8 * mfma_waves));
}

static void fill_src(int mode) {  // 0: uniform random in [-2, 2), 1: zeros
  std::vector<uint16_t> h(4096 * 8);
  unsigned s = 12345;
  for (auto& x : h) {
    s = s * 1664525u + 1013904223u;
    const _Float16 v = (_Float16)(mode == 1 ? 0.f : ((s >> 8) & 0xffff) / 65536.f * 4.f - 2.f);
    x = *(const uint16_t*)&v;
  }
  hipMemcpy(g_src, h.data(), h.size() * 2, hipMemcpyHostToDevice);
}

// ---- 3: issue cost of single instruction kinds (2 waves per SIMD, 8 independent chains)
template <int OP>
__global__ void __launch_bounds__(512) op_kernel(float* out, int iters) {
  ClockProbe probe;
  probe.start();
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
      if (OP == 6) {  // 32 x 32 -> 64-bit product, both halves used (one Philox multiply): v_mad_u64_u32
        const unsigned long long pr = (unsigned long long)us[i] * 0xD2511F53u;
        us[i] = (unsigned)(pr >> 32) ^ (unsigned)pr ^ us[(i + 1) & 7];
      }
      if (OP == 7) us[i] = us[i] ^ us[(i + 1) & 7] ^ us[(i + 3) & 7];  // v_bitop3_b32
    }
  }
  float s = 0;
  for (int i = 0; i < 8; i++) s += xs[i] + (float)us[i];
  out[blockIdx.x * 512 + threadIdx.x] = s;
  probe.stop();
}

template <int OP>
static void run_op(const char* name) {
  const int iters = 2000;
  double ghz;
  const float ms = time_ms([&] { op_kernel<OP><<<256, 512>>>(g_out, iters); }, &ghz);
  printf("  %-24s %5.2f cycles per wave64 instruction per SIMD (clock %.2f GHz)\n", name,
         ms * 1e-3 * ghz * 1e9 / (2.0 * iters * 32), ghz);
}

// ---- 4: LDS read bandwidth for a given per-lane byte offset pattern
template <int MODE>
__global__ void __launch_bounds__(256) lds_kernel(const int* offs, int iters, uint32_t* out) {
  ClockProbe probe;
  probe.start();
  __shared__ __attribute__((aligned(16))) unsigned char lds[65536];
  for (int i = threadIdx.x; i < 65536 / 4; i += 256) ((uint32_t*)lds)[i] = i;
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int off = (offs[lane] + wave * 8192) & 0xffff;
  uint32_t acc = 0;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int u = 0; u < 16; u++) {
      if (MODE == 0) { u32x4 v = *(volatile LDSA u32x4*)(LDSA char*)(lds + off); acc += v[0] ^ v[3]; }
      if (MODE == 1) { i16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDSA i16x4*)(LDSA char*)(lds + off)); acc += v[0] ^ v[3]; asm volatile("" ::: "memory"); }
    }
  }
  out[blockIdx.x * 256 + threadIdx.x] = acc;
  probe.stop();
}

static void run_lds(const char* name, int mode, const int* offs) {
  static int* d_offs = nullptr;
  if (!d_offs) hipMalloc(&d_offs, 256);
  hipMemcpy(d_offs, offs, 256, hipMemcpyHostToDevice);
  const int iters = 2000, blocks = 512;
  double ghz;
  const float ms = mode == 0 ? time_ms([&] { lds_kernel<0><<<blocks, 256>>>(d_offs, iters, (uint32_t*)g_out); }, &ghz, 4, 4)
                             : time_ms([&] { lds_kernel<1><<<blocks, 256>>>(d_offs, iters, (uint32_t*)g_out); }, &ghz, 4, 4);
  const double bytes = (double)blocks * 4 * 64 * (mode == 0 ? 16 : 8) * 16 * iters;
  printf("  %-64s %6.1f B/clk/CU\n", name, bytes / 256 / (ms * 1e-3 * ghz * 1e9));
}

// host copies of the tile addressing of fa_stage.h (element offsets -> bytes)
template <int D, int KIND>
static void frag_pattern(int* offs) {  // the row-fragment read of chunk 2*ks + hf with ks = 1
  for (int l = 0; l < 64; l++) {
    const int c = l & 31, hf = l >> 5, CH = D / 8, RPB = CH >= 16 ? 1 : 16 / CH;
    const int u = (c / RPB) % CH;
    int f = u;
    if (KIND == fa::kSwzTr) f = CH >= 4 ? 2 * (u % (CH / 2)) : 0;
    if (KIND == fa::kSwzDual && CH == 16) f = ((u & 3) << 2) | (u >> 2);
    if (KIND == fa::kSwzDual && CH == 8) f = ((u & 1) << 2) | (u >> 1);
    if (KIND < 0) f = 0;
    offs[l] = (c * D + (((2 + hf) ^ f) * 8)) * 2;
  }
}
template <int D, int KIND>
static void tr_pattern(int* offs) {  // the transposed read of rows 4*hf + j/4, chunk pair 4 + 2*(g&1)
  for (int l = 0; l < 64; l++) {
    const int j = l & 15, g = l >> 4, hf = l >> 5, CH = D / 8, RPB = CH >= 16 ? 1 : 16 / CH;
    const int r = 4 * hf + (j >> 2);
    const int u = (r / RPB) % CH;
    int f = u;
    if (KIND == fa::kSwzTr) f = CH >= 4 ? 2 * (u % (CH / 2)) : 0;
    if (KIND == fa::kSwzDual && CH == 16) f = ((u & 3) << 2) | (u >> 2);
    if (KIND == fa::kSwzDual && CH == 8) f = ((u & 1) << 2) | (u >> 1);
    if (KIND < 0) f = 0;
    const int chunk = 4 + 2 * (g & 1) + ((j >> 1) & 1);
    offs[l] = (r * D + ((chunk ^ f) * 8) + 4 * (j & 1)) * 2;
  }
}

int main() {
  hipMalloc(&g_out, 4 * 512 * 4096);
  hipMalloc(&g_src, 4096 * 16);

  printf("1. MFMA rate and clock: constant (zero) operands, then random operands\n");
  fill_src(1);
  run_mix<0, 0>("MFMA only, zero operands", 1);
  run_mix<0, 0>("MFMA only, zero operands", 2);
  fill_src(0);
  run_mix<0, 0>("MFMA only, random operands", 1);
  run_mix<0, 0>("MFMA only, random operands", 2);

  printf("2. independent VALU work after every MFMA (random operands)\n");
  run_mix<4, 0>("MFMA + 4 v_fma_f32", 2);
  run_mix<8, 0>("MFMA + 8 v_fma_f32", 2);
  run_mix<0, 2>("MFMA + 2 v_exp_f32 (+2 v_mul)", 2);
  run_mix<8, 2>("MFMA + 8 v_fma_f32 + 2 v_exp_f32", 2);
  run_mix<8, 2>("MFMA + 8 v_fma_f32 + 2 v_exp_f32", 3);
  printf("2b. accumulators in VGPRs (as in the attention kernels) instead of AccVGPRs; MFMA and VALU work in separate waves\n");
  run_mix<0, 0, 1>("VGPR acc: MFMA only", 2);
  run_mix<8, 0, 1>("VGPR acc: MFMA + 8 v_fma_f32", 2);
  run_mix<8, 2, 1>("VGPR acc: MFMA + 8 fma + 2 exp", 2);
  run_mix<8, 0, 0, true>("MFMA wave | 8 v_fma_f32 wave", 2);

  printf("3. issue cost of VALU instructions on their own, 2 waves per SIMD\n");
  run_op<0>("v_fma_f32");
  run_op<1>("v_exp_f32");
  run_op<5>("v_rcp_f32");
  run_op<2>("v_max_f32");
  run_op<3>("v_mul_lo_u32 + add");
  run_op<4>("v_mul_hi_u32");
  run_op<6>("v_mad_u64_u32 + v_bitop3");
  run_op<7>("v_bitop3_b32");

  printf("4. LDS read bandwidth, 8 waves per CU\n");
  int offs[64];
  for (int l = 0; l < 64; l++) offs[l] = l * 16;
  run_lds("ds_read_b128, contiguous", 0, offs);
  const int bstr[] = {128, 144, 256, 272};
  for (int s : bstr) {
    for (int l = 0; l < 64; l++) offs[l] = (l % 32) * s + (l / 32) * 16;
    char nm_[96];
    snprintf(nm_, 96, "ds_read_b128 row fragment, padded row stride %d B", s);
    run_lds(nm_, 0, offs);
  }
  frag_pattern<64, fa::kSwzRow>(offs);   run_lds("ds_read_b128 row fragment, d=64 unpadded, row swizzle", 0, offs);
  frag_pattern<64, fa::kSwzDual>(offs);  run_lds("ds_read_b128 row fragment, d=64 unpadded, dual swizzle", 0, offs);
  frag_pattern<128, fa::kSwzRow>(offs);  run_lds("ds_read_b128 row fragment, d=128 unpadded, row swizzle", 0, offs);
  frag_pattern<128, fa::kSwzDual>(offs); run_lds("ds_read_b128 row fragment, d=128 unpadded, dual swizzle", 0, offs);
  frag_pattern<32, fa::kSwzDual>(offs);  run_lds("ds_read_b128 row fragment, d=32 unpadded, dual swizzle", 0, offs);
  for (int l = 0; l < 64; l++) offs[l] = l * 8;
  run_lds("ds_read_b64_tr_b16, contiguous", 1, offs);
  tr_pattern<64, -1>(offs);              run_lds("ds_read_b64_tr_b16 transposed, d=64 unpadded, no swizzle", 1, offs);
  tr_pattern<64, fa::kSwzTr>(offs);      run_lds("ds_read_b64_tr_b16 transposed, d=64 unpadded, tr swizzle", 1, offs);
  tr_pattern<64, fa::kSwzDual>(offs);    run_lds("ds_read_b64_tr_b16 transposed, d=64 unpadded, dual swizzle", 1, offs);
  tr_pattern<64, fa::kSwzRow>(offs);     run_lds("ds_read_b64_tr_b16 transposed, d=64 unpadded, row swizzle", 1, offs);
  tr_pattern<128, -1>(offs);             run_lds("ds_read_b64_tr_b16 transposed, d=128 unpadded, no swizzle", 1, offs);
  tr_pattern<128, fa::kSwzTr>(offs);     run_lds("ds_read_b64_tr_b16 transposed, d=128 unpadded, tr swizzle", 1, offs);
  tr_pattern<128, fa::kSwzDual>(offs);   run_lds("ds_read_b64_tr_b16 transposed, d=128 unpadded, dual swizzle", 1, offs);
  tr_pattern<32, fa::kSwzDual>(offs);    run_lds("ds_read_b64_tr_b16 transposed, d=32 unpadded, dual swizzle", 1, offs);
  printf("done: %s\n", hipGetErrorString(hipDeviceSynchronize()));
  return 0;
}
