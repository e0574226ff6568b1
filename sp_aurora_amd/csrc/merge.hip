// Ring-step merge and final cast: plain coalesced HBM streams.
//   merge    : (out_acc, lse_acc) <- logaddexp-combine with one block's (out, lse)
//              stands in for update_out_and_lse (sp_aurora/utils.py:47-147)
//   finalize : out = cast(out_acc)   (sp_aurora/intel_ring_flash_attn.py:141-143)
//   delta    : delta = rowsum(dout * out), first pass of the block-wise backward
// One thread owns 8 consecutive head dims of one (b, h, s) row; the D/8 threads
// of a row sit in one wavefront, so every lane of the row has read lse_acc before
// the row's first lane overwrites it.
#include "spa_common.h"

namespace {

struct RowIdx {
  int b, h, s;
};

// rows are enumerated with the head index fastest after the sequence index of
// the [B,S,H,D] accumulator: row = (b*Sq + s)*H + h.
static __device__ __forceinline__ RowIdx decode_row(int64_t row, int H, int Sq) {
  RowIdx r;
  r.h = (int)(row % H);
  const int64_t t = row / H;
  r.s = (int)(t % Sq);
  r.b = (int)(t / Sq);
  return r;
}

template <typename T>
struct Load8;  // 8 consecutive elements as floats

template <>
struct Load8<float> {
  static __device__ __forceinline__ void ld(const float* p, float* x) {
    const f32x4 a = *(const f32x4*)p, b = *(const f32x4*)(p + 4);
    x[0] = a[0]; x[1] = a[1]; x[2] = a[2]; x[3] = a[3];
    x[4] = b[0]; x[5] = b[1]; x[6] = b[2]; x[7] = b[3];
  }
  static __device__ __forceinline__ void st(float* p, const float* x) {
    f32x4 a, b;
    a[0] = x[0]; a[1] = x[1]; a[2] = x[2]; a[3] = x[3];
    b[0] = x[4]; b[1] = x[5]; b[2] = x[6]; b[3] = x[7];
    *(f32x4*)p = a;
    *(f32x4*)(p + 4) = b;
  }
};

template <>
struct Load8<__bf16> {
  static __device__ __forceinline__ void ld(const __bf16* p, float* x) {
    const u32x4 a = *(const u32x4*)p;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      x[2 * i] = __builtin_bit_cast(float, a[i] << 16);
      x[2 * i + 1] = __builtin_bit_cast(float, a[i] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ void st(__bf16* p, const float* x) {
    u32x4 a;
#pragma unroll
    for (int i = 0; i < 4; ++i) a[i] = Mma16<__bf16>::pack2(x[2 * i], x[2 * i + 1]);
    *(u32x4*)p = a;
  }
};

template <>
struct Load8<_Float16> {
  static __device__ __forceinline__ void ld(const _Float16* p, float* x) {
    const f16x8 a = *(const f16x8*)p;
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = (float)a[i];
  }
  static __device__ __forceinline__ void st(_Float16* p, const float* x) {
    u32x4 a;
#pragma unroll
    for (int i = 0; i < 4; ++i) a[i] = Mma16<_Float16>::pack2(x[2 * i], x[2 * i + 1]);
    *(u32x4*)p = a;
  }
};

template <typename T, bool INIT>
__global__ void __launch_bounds__(256) merge_kernel(float* __restrict__ out_acc, float* __restrict__ lse_acc,
                                                    const T* __restrict__ blk_out,
                                                    const float* __restrict__ blk_lse, int H, int Sq,
                                                    int cpr /* D/8 */, int64_t nrows, Strides3 as,
                                                    Strides3 bs, int64_t acc_lse_bh) {
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t row = gid / cpr;
  const int ch = (int)(gid % cpr);
  if (row >= nrows) return;
  const RowIdx r = decode_row(row, H, Sq);
  const int64_t li = ((int64_t)r.b * H + r.h) * Sq + r.s;          // block lse: contiguous [B,H,Sq]
  const int64_t la_i = ((int64_t)r.b * H + r.h) * acc_lse_bh + r.s;  // running lse: row pitch acc_lse_bh
  float* ap = out_acc + r.b * as.b + r.h * as.h + (int64_t)r.s * as.s + ch * 8;
  const T* bp = blk_out + r.b * bs.b + r.h * bs.h + (int64_t)r.s * bs.s + ch * 8;
  float xb[8];
  Load8<T>::ld(bp, xb);
  const float lb = blk_lse[li];
  if (INIT) {
    Load8<float>::st(ap, xb);
    if (ch == 0) lse_acc[la_i] = lb;
    return;
  }
  const float la = lse_acc[la_i];
  float xa[8];
  Load8<float>::ld(ap, xa);
  // w = sigmoid(lb - la); lse' = max + log1p(exp(-|lb - la|))
  const float d = lb - la;
  float w, ln;
  if (d == d) {  // also covers +-inf on one side
    const float e = __expf(-fabsf(d));
    const float inv = 1.f / (1.f + e);
    w = d >= 0.f ? inv : e * inv;
    ln = fmaxf(la, lb) + log1pf(e);
  } else {  // both -inf: nothing accumulated on either side
    w = 0.f;
    ln = la;
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) xa[i] = xa[i] - w * (xa[i] - xb[i]);
  Load8<float>::st(ap, xa);
  if (ch == 0) lse_acc[la_i] = ln;
}

template <typename T>
__global__ void __launch_bounds__(256) finalize_kernel(T* __restrict__ out, const float* __restrict__ out_acc,
                                                       int H, int Sq, int cpr, int64_t nrows, Strides3 os,
                                                       Strides3 as) {
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t row = gid / cpr;
  const int ch = (int)(gid % cpr);
  if (row >= nrows) return;
  const RowIdx r = decode_row(row, H, Sq);
  float x[8];
  Load8<float>::ld(out_acc + r.b * as.b + r.h * as.h + (int64_t)r.s * as.s + ch * 8, x);
  Load8<T>::st(out + r.b * os.b + r.h * os.h + (int64_t)r.s * os.s + ch * 8, x);
}

// delta[b,h,s] = sum_d dout*out; the D/8 lanes of a row reduce with DPP-free shuffles.
template <typename T>
__global__ void __launch_bounds__(256) delta_kernel(const T* __restrict__ out, const T* __restrict__ dout,
                                                    float* __restrict__ delta, int H, int Sq, int cpr,
                                                    int64_t nrows, Strides3 os, Strides3 ds) {
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  int64_t row = gid / cpr;
  const int ch = (int)(gid % cpr);
  const bool valid = row < nrows;
  if (!valid) row = nrows - 1;
  const RowIdx r = decode_row(row, H, Sq);
  float a[8], g[8];
  Load8<T>::ld(out + r.b * os.b + r.h * os.h + (int64_t)r.s * os.s + ch * 8, a);
  Load8<T>::ld(dout + r.b * ds.b + r.h * ds.h + (int64_t)r.s * ds.s + ch * 8, g);
  float acc = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) acc = __builtin_fmaf(a[i], g[i], acc);
  for (int off = cpr >> 1; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
  if (valid && ch == 0) delta[((int64_t)r.b * H + r.h) * Sq + r.s] = acc;
}

}  // namespace

hipError_t spa_launch_merge(float* out_acc, float* lse_acc, const void* blk_out, const float* blk_lse, int B,
                            int H, int Sq, int D, Strides3 as, Strides3 bs, int dtype, int init,
                            int64_t acc_lse_bh, hipStream_t stream) {
  const int cpr = D / 8;
  const int64_t nrows = (int64_t)B * H * Sq;
  const int64_t nthreads = nrows * cpr;
  const dim3 grid((unsigned)((nthreads + 255) / 256));
#define SPA_MERGE(T, I)                                                                              \
  hipLaunchKernelGGL((merge_kernel<T, I>), grid, dim3(256), 0, stream, out_acc, lse_acc, (const T*)blk_out, \
                     blk_lse, H, Sq, cpr, nrows, as, bs, acc_lse_bh)
  if (dtype == 0) { if (init) SPA_MERGE(float, true); else SPA_MERGE(float, false); }
  else if (dtype == 1) { if (init) SPA_MERGE(__bf16, true); else SPA_MERGE(__bf16, false); }
  else if (dtype == 2) { if (init) SPA_MERGE(_Float16, true); else SPA_MERGE(_Float16, false); }
  else return hipErrorInvalidValue;
#undef SPA_MERGE
  return hipGetLastError();
}

hipError_t spa_launch_finalize(void* out, const float* out_acc, int B, int H, int Sq, int D, Strides3 os,
                               Strides3 as, int dtype, hipStream_t stream) {
  const int cpr = D / 8;
  const int64_t nrows = (int64_t)B * H * Sq;
  const dim3 grid((unsigned)((nrows * cpr + 255) / 256));
  if (dtype == 0)
    hipLaunchKernelGGL((finalize_kernel<float>), grid, dim3(256), 0, stream, (float*)out, out_acc, H, Sq, cpr, nrows, os, as);
  else if (dtype == 1)
    hipLaunchKernelGGL((finalize_kernel<__bf16>), grid, dim3(256), 0, stream, (__bf16*)out, out_acc, H, Sq, cpr, nrows, os, as);
  else if (dtype == 2)
    hipLaunchKernelGGL((finalize_kernel<_Float16>), grid, dim3(256), 0, stream, (_Float16*)out, out_acc, H, Sq, cpr, nrows, os, as);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

hipError_t spa_launch_delta(const void* out, const void* dout, float* delta, int B, int H, int Sq, int D,
                            Strides3 os, Strides3 ds, int dtype, hipStream_t stream) {
  const int cpr = D / 8;
  const int64_t nrows = (int64_t)B * H * Sq;
  const dim3 grid((unsigned)((nrows * cpr + 255) / 256));
  if (dtype == 0)
    hipLaunchKernelGGL((delta_kernel<float>), grid, dim3(256), 0, stream, (const float*)out, (const float*)dout, delta, H, Sq, cpr, nrows, os, ds);
  else if (dtype == 1)
    hipLaunchKernelGGL((delta_kernel<__bf16>), grid, dim3(256), 0, stream, (const __bf16*)out, (const __bf16*)dout, delta, H, Sq, cpr, nrows, os, ds);
  else if (dtype == 2)
    hipLaunchKernelGGL((delta_kernel<_Float16>), grid, dim3(256), 0, stream, (const _Float16*)out, (const _Float16*)dout, delta, H, Sq, cpr, nrows, os, ds);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}
