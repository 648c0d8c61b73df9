// Micro-benchmark: is an attention-shaped loop on gfx950 limited by instruction issue or by power?
//
// One step of the loop is what a forward wave does per 64-key tile at head dim 64, without LDS, barriers or memory
// traffic (operands stay in registers): S = K Q^T (8 MFMAs), the softmax VALU work on the 32 scores a lane owns (max3,
// fma, exp2, convert, dot2 row sum, a rarely taken rescale branch), O += V P (8 MFMAs that consume the converted P).
// Written three ways:
//   chain      S -> softmax -> PV, each stage waiting for the one before (what a straightforward kernel does),
//   ahead      the S MFMAs of the next step are issued before this step's exponentials (independent work for the matrix
//              pipe while the VALU runs),
//   ahead + PV the S MFMAs of the next step and the PV MFMAs of the previous step are interleaved with this step's
//              exponentials, one MFMA per N VALU instructions (scheduling-group barriers), i.e. the matrix pipe and the
//              VALU of ONE wave always have independent work,
// next to the MFMAs alone and the VALU work alone, and the chain with the K and V fragments fetched from LDS every step
// as a kernel must (8 ds_read_b128 + 16 ds_read_b64 per wave and step, no staging traffic), once for 32 query rows per
// wave and once for 64 (two row blocks share every fragment read; the time is quoted per 32 rows).  Every line reports time and, from the cycle counter read against
// the 100 MHz wall clock inside the kernel, the shader clock: when the interleaved forms need fewer cycles but the clock
// falls by as much, the loop is power limited, not issue limited.
// Build and run from the repository root with the kernels' flags:
//   hipcc --offload-arch=gfx950 -O3 -std=c++17 -Xclang -target-feature -Xclang -packed-fp32-ops
//         flash-attention_amd/csrc/tune/overlap_model.hip -o overlap_model && ./overlap_model
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <vector>

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

struct PFrag { f16x8 v[4]; };  // the converted probabilities of a step: B operands of its four PV MFMA pairs
__device__ long long g_clk[2];

enum { kMfmaOnly, kValuOnly, kChain, kAhead, kAheadPV, kChainLds, kChainLds2 };

__device__ __forceinline__ void s_mfma(f32x16* s, const f16x8* K, const f16x8* Q) {
#pragma unroll
  for (int kb = 0; kb < 2; kb++) {
    for (int i = 0; i < 16; i++) s[kb][i] = 0.f;
#pragma unroll
    for (int ks = 0; ks < 4; ks++) s[kb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(K[kb * 4 + ks], Q[ks], s[kb], 0, 0, 0);
  }
}
__device__ __forceinline__ void pv_mfma(f32x16* o, const f16x8* V, const PFrag& p) {
#pragma unroll
  for (int j = 0; j < 4; j++)
#pragma unroll
    for (int db = 0; db < 2; db++) o[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(V[db * 2 + (j & 1)], p.v[j], o[db], 0, 0, 0);
}
// row maximum and the (rare) move of the reference point; `pending` are probabilities not yet accumulated into o
__device__ __forceinline__ void softmax_max(f32x16* s, float& m, float& l, f32x16* o, float cs, PFrag* pending) {
  float mt = s[0][0];
#pragma unroll
  for (int kb = 0; kb < 2; kb++)
#pragma unroll
    for (int r = 0; r < 16; r++) mt = fmaxf(mt, s[kb][r]);
  if (__builtin_expect(__any((mt - m) * cs > 8.f), 0)) {
    m = mt;
    l *= 0.5f;
    o[0] = o[0] * 0.5f;
    o[1] = o[1] * 0.5f;
    if (pending)
      for (int j = 0; j < 4; j++) pending->v[j] = pending->v[j] * (_Float16)0.5f;
  }
}
__device__ __forceinline__ void softmax_exp(f32x16* s, float m, float& l, float cs, PFrag& p) {
  const float mc = m * cs;
#pragma unroll
  for (int kb = 0; kb < 2; kb++)
#pragma unroll
    for (int t = 0; t < 2; t++) {
      f16x8 pb;
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const float a = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kb][8 * t + 2 * i], cs, -mc));
        const float b = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kb][8 * t + 2 * i + 1], cs, -mc));
        const f16x2 h = __builtin_bit_cast(f16x2, __builtin_amdgcn_cvt_pkrtz(a, b));
        pb[2 * i] = h[0];
        pb[2 * i + 1] = h[1];
        l = __builtin_amdgcn_fdot2(h, f16x2{(_Float16)1, (_Float16)1}, l, false);
      }
      p.v[kb * 2 + t] = pb;
    }
}

// VPM: VALU instructions per MFMA in the interleaved region (0: leave the order to the compiler)
template <int FORM, int VPM, int WAVES>
__global__ void __launch_bounds__(256, WAVES) step_kernel(const f16x8* __restrict__ src, float* out, int iters) {
  const int tid = threadIdx.x, lane = tid & 63;
  long long c0 = 0, w0 = 0;
  if (blockIdx.x == 0 && tid == 0) { c0 = __builtin_readcyclecounter(); w0 = wall_clock64(); }
  f16x8 K[8], Q[4], V[4];
  for (int i = 0; i < 8; i++) K[i] = src[(lane * 8 + i + blockIdx.x * 3) & 4095];
  for (int i = 0; i < 4; i++) {
    Q[i] = src[(lane * 4 + i + 2048 + tid) & 4095];
    V[i] = src[(lane * 4 + i + 1024 + tid) & 4095];
  }
  f32x16 o[2];
  for (int n = 0; n < 2; n++)
    for (int i = 0; i < 16; i++) o[n][i] = 0;
  float m = 0.5f, l = 0.f;
  const float cs = 0.18f;
  f32x16 sa[2], sb[2];
  PFrag pa, pb;
  for (int j = 0; j < 4; j++) pa.v[j] = K[j];
  if (FORM == kAhead || FORM == kAheadPV) s_mfma(sa, K, Q);
  constexpr bool kLds = FORM == kChainLds || FORM == kChainLds2;
  __shared__ __attribute__((aligned(16))) unsigned char lds[kLds ? 32768 : 16];
  f16x8 Q2[4];   // second row block of kChainLds2
  f32x16 o2[2];
  float m2 = 0.5f, l2 = 0.f;
  for (int i = 0; i < 4; i++) Q2[i] = src[(lane * 4 + i + 3072 + tid) & 4095];
  for (int n = 0; n < 2; n++)
    for (int i = 0; i < 16; i++) o2[n][i] = 0;
  if (kLds) {
    for (int i = tid; i < 2048; i += 256) reinterpret_cast<f16x8*>(lds)[i] = src[(i * 7 + blockIdx.x) & 4095];
    __syncthreads();
  }
  int it_ = 0;
  // one step; the two score buffers and the two probability buffers swap roles from step to step
  auto step = [&](f32x16* sc, f32x16* sn, PFrag& pp, PFrag& pc) {
    asm volatile("" : "+v"(o[0]), "+v"(o[1]));
    asm volatile("" : "+v"(Q[0]), "+v"(Q[1]), "+v"(Q[2]), "+v"(Q[3]));  // keeps the S MFMAs inside the loop
    if (FORM == kChainLds2) asm volatile("" : "+v"(o2[0]), "+v"(o2[1]), "+v"(Q2[0]), "+v"(Q2[1]), "+v"(Q2[2]), "+v"(Q2[3]));
    if (FORM == kMfmaOnly) {
      s_mfma(sc, K, Q);
      for (int j = 0; j < 4; j++) pc.v[j] = __builtin_bit_cast(f16x8, __builtin_shufflevector(sc[j >> 1], sc[j >> 1], 0, 1, 2, 3));
      pv_mfma(o, V, pc);
    } else if (FORM == kValuOnly) {
      for (int kb = 0; kb < 2; kb++)
        for (int i = 0; i < 16; i++) sc[kb][i] = o[kb][i] + l;  // 32 adds stand in for the scores
      asm volatile("" : "+v"(sc[0]), "+v"(sc[1]));
      softmax_max(sc, m, l, o, cs, nullptr);
      softmax_exp(sc, m, l, cs, pc);
      for (int j = 0; j < 4; j++) asm volatile("" ::"v"(pc.v[j]));
    } else if (FORM == kChainLds) {
      // fragments of this step from one of two LDS copies in turn (so the reads stay inside the loop)
      const unsigned char* base = lds + ((it_ & 1) ? 16384 : 0);
      f16x8 Kl[8], Vl[4];
#pragma unroll
      for (int i = 0; i < 8; i++) Kl[i] = *reinterpret_cast<const f16x8*>(base + i * 1024 + lane * 16);
      s_mfma(sc, Kl, Q);
      softmax_max(sc, m, l, o, cs, nullptr);
      softmax_exp(sc, m, l, cs, pc);
#pragma unroll
      for (int j = 0; j < 4; j++) {
#pragma unroll
        for (int db = 0; db < 2; db++) {
          typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
          typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
          const u32x2 lo = *reinterpret_cast<const u32x2*>(base + 8192 + (j * 4 + db * 2) * 512 + lane * 8);
          const u32x2 hi = *reinterpret_cast<const u32x2*>(base + 8192 + (j * 4 + db * 2 + 1) * 512 + lane * 8);
          const u32x4 av = {lo[0], lo[1], hi[0], hi[1]};
          o[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, av), pc.v[j], o[db], 0, 0, 0);
        }
      }
    } else if (FORM == kChainLds2) {
      // as kChainLds for two blocks of 32 query rows that share the fragment reads (second block: sn, pp, o2, m2, l2)
      const unsigned char* base = lds + ((it_ & 1) ? 16384 : 0);
      f16x8 Kl[8];
#pragma unroll
      for (int i = 0; i < 8; i++) Kl[i] = *reinterpret_cast<const f16x8*>(base + i * 1024 + lane * 16);
      s_mfma(sc, Kl, Q);
      s_mfma(sn, Kl, Q2);
      softmax_max(sc, m, l, o, cs, nullptr);
      softmax_exp(sc, m, l, cs, pc);
      softmax_max(sn, m2, l2, o2, cs, nullptr);
      softmax_exp(sn, m2, l2, cs, pp);
#pragma unroll
      for (int j = 0; j < 4; j++) {
#pragma unroll
        for (int db = 0; db < 2; db++) {
          typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
          typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
          const u32x2 lo = *reinterpret_cast<const u32x2*>(base + 8192 + (j * 4 + db * 2) * 512 + lane * 8);
          const u32x2 hi = *reinterpret_cast<const u32x2*>(base + 8192 + (j * 4 + db * 2 + 1) * 512 + lane * 8);
          const u32x4 av = {lo[0], lo[1], hi[0], hi[1]};
          o[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, av), pc.v[j], o[db], 0, 0, 0);
          o2[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, av), pp.v[j], o2[db], 0, 0, 0);
        }
      }
    } else if (FORM == kChain) {
      s_mfma(sc, K, Q);
      softmax_max(sc, m, l, o, cs, nullptr);
      softmax_exp(sc, m, l, cs, pc);
      pv_mfma(o, V, pc);
    } else if (FORM == kAhead) {
      softmax_max(sc, m, l, o, cs, nullptr);
      s_mfma(sn, K, Q);
      softmax_exp(sc, m, l, cs, pc);
      if (VPM) {
#pragma unroll
        for (int g = 0; g < 8; g++) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, VPM, 0);
        }
      }
      pv_mfma(o, V, pc);
    } else {
      softmax_max(sc, m, l, o, cs, &pp);
      s_mfma(sn, K, Q);
      pv_mfma(o, V, pp);
      softmax_exp(sc, m, l, cs, pc);
      if (VPM) {
#pragma unroll
        for (int g = 0; g < 16; g++) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, VPM, 0);
        }
      }
    }
  };
  for (int it = 0; it < iters; it += 2) {
    it_ = it >> 1;
    step(sa, sb, pa, pb);
    step(sb, sa, pb, pa);
  }
  if (FORM == kAheadPV) pv_mfma(o, V, pa);
  float acc = l + m + l2 + m2;
  for (int n = 0; n < 2; n++)
    for (int i = 0; i < 16; i++) acc += o[n][i] + sa[n][i] + o2[n][i];
  out[blockIdx.x * 256 + tid] = acc;
  if (blockIdx.x == 0 && tid == 0) { g_clk[0] = __builtin_readcyclecounter() - c0; g_clk[1] = wall_clock64() - w0; }
}

static f16x8* g_src;
static float* g_out;

template <int FORM, int VPM, int WAVES>
static void run(const char* name) {
  const int iters = 2000, blocks = 256 * WAVES;
  hipEvent_t e0, e1;
  hipEventCreate(&e0);
  hipEventCreate(&e1);
  for (int r = 0; r < 20; r++) step_kernel<FORM, VPM, WAVES><<<blocks, 256>>>(g_src, g_out, iters);  // clock settles
  hipEventRecord(e0);
  for (int r = 0; r < 5; r++) step_kernel<FORM, VPM, WAVES><<<blocks, 256>>>(g_src, g_out, iters);
  hipEventRecord(e1);
  hipEventSynchronize(e1);
  float ms;
  hipEventElapsedTime(&ms, e0, e1);
  ms /= 5;
  long long hc[2];
  hipMemcpyFromSymbol(hc, HIP_SYMBOL(g_clk), 16);
  const int units = FORM == kChainLds2 ? 2 : 1;  // blocks of 32 query rows per wave and step
  const double ghz = hc[0] / (hc[1] / 100.0) / 1e3, ns = ms * 1e6 / (iters * (double)WAVES * units);
  printf("  %-46s %d waves/SIMD: %6.1f ns = %5.0f cycles per wave and 32-row step, clock %.2f GHz", name, WAVES, ns, ns * ghz, ghz);
  if (FORM != kValuOnly) printf(", %6.1f TFLOP/s", (double)blocks * 4 * iters * units * 16 * 32768.0 / ms / 1e9);
  printf("\n");
}

int main() {
  hipMalloc(&g_src, 4096 * 16);
  hipMalloc(&g_out, 1024 * 256 * 4);
  std::vector<uint16_t> h(4096 * 8);
  unsigned s = 12345;
  for (auto& x : h) {
    s = s * 1664525u + 1013904223u;
    const _Float16 v = (_Float16)(((s >> 8) & 0xffff) / 65536.f * 2.f - 1.f);
    x = *(const uint16_t*)&v;
  }
  hipMemcpy(g_src, h.data(), h.size() * 2, hipMemcpyHostToDevice);
  printf("forward-shaped step: 16 MFMAs 32x32x16 f16 + softmax VALU work of 32 scores per lane, operands in registers\n");
  run<kMfmaOnly, 0, 2>("MFMAs only");
  run<kValuOnly, 0, 2>("VALU work only");
  run<kChain, 0, 2>("chain: S -> softmax -> PV");
  run<kChain, 0, 3>("chain: S -> softmax -> PV");
  run<kChainLds, 0, 2>("chain, K and V fragments read from LDS");
  run<kChainLds, 0, 4>("chain, K and V fragments read from LDS");
  run<kChainLds2, 0, 2>("chain from LDS, 64 query rows per wave");
  run<kAhead, 0, 2>("next S ahead of the exponentials");
  run<kAhead, 16, 2>("next S ahead, 1 MFMA : 16 VALU");
  run<kAheadPV, 0, 2>("next S and previous PV ahead");
  run<kAheadPV, 8, 2>("next S and previous PV ahead, 1 MFMA : 8 VALU");
  run<kAheadPV, 6, 2>("next S and previous PV ahead, 1 MFMA : 6 VALU");
  printf("done: %s\n", hipGetErrorString(hipGetLastError()));
  return 0;
}
