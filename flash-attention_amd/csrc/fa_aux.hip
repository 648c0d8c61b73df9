// Small HBM-bound helper kernels around the attention kernels: fills, the block-sparse activity maps and the
// probability dump behind return_softmax.
#include "fa_params.h"

namespace fa {

namespace {

__global__ void fill_f32_kernel(float* p, size_t n, float value) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) p[i] = value;
}

__global__ void zero_rows_kernel(uint16_t* base, int64_t rs, int64_t hs, int total, int H, int D) {
  const int64_t n = (int64_t)total * H * (D / 8);
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    const int ch = (int)(i % (D / 8));
    const int64_t rh = i / (D / 8);
    const int h = (int)(rh % H);
    const int64_t row = rh / H;
    st_global16(base + row * rs + h * hs + ch * 8, u32x4{0, 0, 0, 0});
  }
}

// blockmask: [ncb][nrb] int32, entries 4*rowblock + flags for the active 16-row blocks of each 256-key
// column block, -1 padded (flash_blocksparse_attn_interface.py:8-40; read as fmha_blockmask.h:41-53 does).
// inv[order[i]] = i + 1: where each row block stands in the row order (entries that are no row block are skipped; inv was
// cleared: 0 = the order does not list the row block, it belongs to no tile)
__global__ void invert_order_kernel(const int32_t* order, int32_t* inv, int nrb) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= nrb) return;
  const int rb = order[i];
  if (rb >= 0 && rb < nrb) inv[rb] = i + 1;
}

// inv: null, or the position of every row block in the row order (then query tile t owns the row blocks at positions
// rpq t .. rpq t + rpq - 1, not the row blocks with those numbers)
__global__ void sparse_maps_kernel(const int32_t* blockmask, uint32_t* rbits, uint32_t* qbits, uint32_t* cbits, int nrb,
                                   int ncb, int rpq, int nqt, int ncw, int nrw, const int32_t* inv) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= nrb * ncb) return;
  const int cb = i / nrb;
  const int e = blockmask[i];
  if (e < 0) return;
  const int rb = e >> 2;
  if (rb >= nrb) return;
  // the 64-bit words are addressed as pairs of 32-bit words (bit b of a word: half b / 32, bit b % 32)
  atomicOr(rbits + ((int64_t)rb * ncw * 2 + (cb >> 5)), 1u << (cb & 31));
  const int pos = inv ? inv[rb] - 1 : rb;
  if (pos >= 0 && pos / rpq < nqt) atomicOr(qbits + ((int64_t)(pos / rpq) * ncw * 2 + (cb >> 5)), 1u << (cb & 31));
  atomicOr(cbits + ((int64_t)cb * nrw * 2 + (rb >> 5)), 1u << (rb & 31));
}

// One thread per (query row, key) element of S_dmask.  Slow scalar dot products: this path exists for tests
// (flash_attn_interface.py:163-173).  The value is the normalised probability exp(scale*s - lse); its sign
// bit is set when dropout dropped the element.
template <typename T>
__global__ void __launch_bounds__(256) dump_probs_kernel(const DumpParams p) {
  const int key = blockIdx.x * 256 + threadIdx.x;
  const int qrow = blockIdx.y;
  const int bh = blockIdx.z;
  const int b = bh / p.H, h = bh % p.H;
  int q_begin = 0, Lq = 0, k_begin = 0, Lk = 0;
  if (!seq_extent(p.cu_q, b, p.total_q, p.max_sq, &q_begin, &Lq)) Lq = 0;
  if (!seq_extent(p.cu_k, b, p.total_k, p.max_sk, &k_begin, &Lk)) Lk = 0;
  if (key >= p.sk_r) return;
  float val = 0.f;
  bool dropped = false;
  bool live = qrow < Lq && key < Lk;
  if (p.causal && key > qrow) live = false;
  if (live && p.sparse) {
    const int rb = qrow >> 4, cb = key >> 8;
    live = rb < p.sp.nrb && cb < p.sp.ncb && ((p.sp.rbits[(int64_t)rb * p.sp.ncw + (cb >> 6)] >> (cb & 63)) & 1) != 0;
  }
  if (live) {
    const T* qp = reinterpret_cast<const T*>(p.q) + (int64_t)(q_begin + qrow) * p.q_rs + (int64_t)h * p.q_hs;
    const T* kp = reinterpret_cast<const T*>(p.k) + (int64_t)(k_begin + key) * p.k_rs + (int64_t)h * p.k_hs;
    float s = 0.f;
    for (int d = 0; d < p.D; d++) s += (float)qp[d] * (float)kp[d];
    const float lse = p.lse[((int64_t)b * p.H + h) * p.sq_r + qrow];
    float x = s * p.scale;
    if (p.alibi) x -= p.alibi[h] * fabsf((float)(key - qrow));
    if (p.bias)
      x += (float)reinterpret_cast<const T*>(p.bias)[(int64_t)b * p.bias_bs + (int64_t)h * p.bias_hs + (int64_t)qrow * p.bias_rs + key];
    val = __expf(x - lse);
    if (p.dropout) {
      const uint32_t bits = dropout_keep_bits16(p.pk, (uint32_t)bh, (uint32_t)qrow >> 2, (uint32_t)key >> 2, p.keep_thr);
      dropped = !((bits >> (4 * (qrow & 3) + (key & 3))) & 1u);
    }
  }
  T out = (T)val;
  if (dropped) out = -out;
  reinterpret_cast<T*>(p.s)[(((int64_t)b * p.H + h) * p.sq_r + qrow) * p.sk_r + key] = out;
}

}  // namespace

hipError_t launch_fill_f32(float* p, size_t n, float value, hipStream_t stream) {
  if (n == 0) return hipSuccess;
  size_t blocks = (n + 255) / 256;
  if (blocks > 65535) blocks = 65535;
  hipLaunchKernelGGL(fill_f32_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, p, n, value);
  return hipGetLastError();
}

hipError_t launch_zero_rows(void* base, int64_t row_stride, int64_t head_stride, int total, int H, int D,
                            hipStream_t stream) {
  const int64_t n = (int64_t)total * H * (D / 8);
  if (n == 0) return hipSuccess;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 65535) blocks = 65535;
  hipLaunchKernelGGL(zero_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, stream,
                     reinterpret_cast<uint16_t*>(base), row_stride, head_stride, total, H, D);
  return hipGetLastError();
}

hipError_t launch_build_sparse_maps(const int32_t* blockmask, uint64_t* rbits, uint64_t* qbits, uint64_t* cbits, int nrb,
                                    int ncb, int rows_per_qt, int nqt, int ncw, int nrw, const int32_t* order, int32_t* inv,
                                    hipStream_t stream) {
  const int n = nrb * ncb;
  if (order && inv) {  // (inv was cleared by the caller)
    hipLaunchKernelGGL(invert_order_kernel, dim3((nrb + 255) / 256), dim3(256), 0, stream, order, inv, nrb);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
  } else {
    inv = nullptr;
  }
  hipLaunchKernelGGL(sparse_maps_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, blockmask,
                     reinterpret_cast<uint32_t*>(rbits), reinterpret_cast<uint32_t*>(qbits),
                     reinterpret_cast<uint32_t*>(cbits), nrb, ncb, rows_per_qt / 16, nqt, ncw, nrw, inv);
  return hipGetLastError();
}

hipError_t launch_dump_probs(const DumpParams& p, int dtype, hipStream_t stream) {
  dim3 grid((p.sk_r + 255) / 256, p.sq_r, p.B * p.H);
  if (dtype == 0) hipLaunchKernelGGL(dump_probs_kernel<_Float16>, grid, dim3(256), 0, stream, p);
  else hipLaunchKernelGGL(dump_probs_kernel<__bf16>, grid, dim3(256), 0, stream, p);
  return hipGetLastError();
}

}  // namespace fa
