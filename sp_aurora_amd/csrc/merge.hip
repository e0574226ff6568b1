// Ring-step merge and final cast: plain coalesced HBM streams.
//   merge    : (out_acc, lse_acc) <- logaddexp-combine with one block's (out, lse)
//              stands in for update_out_and_lse (sp_aurora/utils.py:47-147)
//   finalize : out = cast(out_acc)   (sp_aurora/intel_ring_flash_attn.py:141-143)
//   delta    : delta = rowsum(dout * out), first pass of the block-wise backward
// One thread owns 8 consecutive head dims of two (b, h, s) rows (all loads of both rows are
// issued before the first store); the D/8 threads of a row sit in one wavefront, so every lane of
// the row has read lse_acc before the row's first lane overwrites it.  32-bit row arithmetic,
// the batch index comes from the grid.
#include "spa_common.h"

namespace {

struct RowIdx {
  int b, h, s;
};

// Rows of one batch entry are enumerated with the head index fastest after the sequence index of
// the [B,S,H,D] accumulator: row = s*H + h (32-bit: a batch entry holds fewer than 2^31 rows, the
// launchers check it); the batch index is the grid's y dimension.
static __device__ __forceinline__ RowIdx decode_row(unsigned row, int H) {
  RowIdx r;
  r.s = (int)(row / (unsigned)H);
  r.h = (int)(row - (unsigned)r.s * (unsigned)H);
  r.b = (int)blockIdx.y;
  return r;
}

constexpr int ROWS_PER_THREAD = 1;  // rows a thread takes (two, `half` rows apart with all loads first, measured 10 % slower on the merge)

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

// A thread owns chunk `ch` (8 head dims) of ROWS_PER_THREAD rows, `half` rows apart; the D/8
// lanes of a row share a wave, so every lane of the row has read lse_acc before lane 0 rewrites it.
template <typename T, bool INIT>
__global__ void __launch_bounds__(256) merge_kernel(float* __restrict__ out_acc, float* __restrict__ lse_acc,
                                                    const T* __restrict__ blk_out,
                                                    const float* __restrict__ blk_lse, int H, int Sq,
                                                    int cpr_shift /* log2(D/8) */, unsigned nrows, unsigned half,
                                                    Strides3 as, Strides3 bs, int64_t acc_lse_bh) {
  const unsigned gid = blockIdx.x * 256u + threadIdx.x;
  const unsigned row0 = gid >> cpr_shift;
  const int ch = (int)(gid & ((1u << cpr_shift) - 1u));
  float xb[ROWS_PER_THREAD][8], xa[ROWS_PER_THREAD][8], lb[ROWS_PER_THREAD], la[ROWS_PER_THREAD];
  float* ap[ROWS_PER_THREAD];
  int64_t la_i[ROWS_PER_THREAD];
  bool on[ROWS_PER_THREAD];
#pragma unroll
  for (int k = 0; k < ROWS_PER_THREAD; ++k) {
    const unsigned row = row0 + k * half;
    on[k] = row0 < half && row < nrows;
    const RowIdx r = decode_row(on[k] ? row : 0u, H);
    const int64_t li = ((int64_t)r.b * H + r.h) * Sq + r.s;     // block lse: contiguous [B,H,Sq]
    la_i[k] = ((int64_t)r.b * H + r.h) * acc_lse_bh + r.s;        // running lse: row pitch acc_lse_bh
    ap[k] = out_acc + r.b * as.b + r.h * as.h + (int64_t)r.s * as.s + ch * 8;
    if (on[k]) {
      Load8<T>::ld(blk_out + r.b * bs.b + r.h * bs.h + (int64_t)r.s * bs.s + ch * 8, xb[k]);
      lb[k] = blk_lse[li];
      if (!INIT) {
        la[k] = lse_acc[la_i[k]];
        Load8<float>::ld(ap[k], xa[k]);
      }
    }
  }
#pragma unroll
  for (int k = 0; k < ROWS_PER_THREAD; ++k) {
    if (!on[k]) continue;
    if (INIT) {
      Load8<float>::st(ap[k], xb[k]);
      if (ch == 0) lse_acc[la_i[k]] = lb[k];
      continue;
    }
    // w = sigmoid(lb - la); lse' = max + log1p(exp(-|lb - la|))
    const float d = lb[k] - la[k];
    float w, ln;
    if (d == d) {  // also covers +-inf on one side
      const float e = __expf(-fabsf(d));
      const float inv = 1.f / (1.f + e);
      w = d >= 0.f ? inv : e * inv;
      ln = fmaxf(la[k], lb[k]) + log1pf(e);
    } else {  // both -inf: nothing accumulated on either side
      w = 0.f;
      ln = la[k];
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) xa[k][i] = xa[k][i] - w * (xa[k][i] - xb[k][i]);
    Load8<float>::st(ap[k], xa[k]);
    if (ch == 0) lse_acc[la_i[k]] = ln;
  }
}

template <typename T>
__global__ void __launch_bounds__(256) finalize_kernel(T* __restrict__ out, const float* __restrict__ out_acc,
                                                       int H, int cpr_shift, unsigned nrows, unsigned half,
                                                       Strides3 os, Strides3 as) {
  const unsigned gid = blockIdx.x * 256u + threadIdx.x;
  const unsigned row0 = gid >> cpr_shift;
  const int ch = (int)(gid & ((1u << cpr_shift) - 1u));
  float x[ROWS_PER_THREAD][8];
  T* op[ROWS_PER_THREAD];
  bool on[ROWS_PER_THREAD];
#pragma unroll
  for (int k = 0; k < ROWS_PER_THREAD; ++k) {
    const unsigned row = row0 + k * half;
    on[k] = row0 < half && row < nrows;
    const RowIdx r = decode_row(on[k] ? row : 0u, H);
    op[k] = out + r.b * os.b + r.h * os.h + (int64_t)r.s * os.s + ch * 8;
    if (on[k]) Load8<float>::ld(out_acc + r.b * as.b + r.h * as.h + (int64_t)r.s * as.s + ch * 8, x[k]);
  }
#pragma unroll
  for (int k = 0; k < ROWS_PER_THREAD; ++k)
    if (on[k]) Load8<T>::st(op[k], x[k]);
}

// Merge of the n block results a key-split forward left behind (rows j * Sq .. of `part`, [B, n * Sq, H, D] in T, and of
// part_lse, [B, H, n * Sq]): update_out_and_lse (sp_aurora/utils.py:103-104) over all of them at once, as a running
// (weighted sum, weight sum) relative to the largest lse so far.  All lse are finite (every chunk holds a key).
template <typename T>
__global__ void __launch_bounds__(256) splitkv_combine_kernel(T* __restrict__ out, float* __restrict__ lse, const T* __restrict__ part,
                                                              const float* __restrict__ part_lse, int n, int H, int Sq, int D,
                                                              int cpr_shift, unsigned nrows, Strides3 os, int64_t lse_bh) {
  const unsigned gid = blockIdx.x * 256u + threadIdx.x;
  const unsigned row = gid >> cpr_shift;
  const int ch = (int)(gid & ((1u << cpr_shift) - 1u));
  if (row >= nrows) return;
  const RowIdx r = decode_row(row, H);
  const int64_t prow = (int64_t)H * D;                                  // elements between rows of `part`
  const T* pp = part + ((int64_t)r.b * n * Sq + r.s) * prow + r.h * D + ch * 8;
  const float* pl = part_lse + ((int64_t)r.b * H + r.h) * ((int64_t)n * Sq) + r.s;
  float x[8], xb[8], lb = pl[0], wsum = 1.f;
  Load8<T>::ld(pp, x);
  for (int j = 1; j < n; ++j) {
    Load8<T>::ld(pp + (int64_t)j * Sq * prow, xb);
    const float lj = pl[(int64_t)j * Sq];
    const float mx = fmaxf(lb, lj);
    const float wa = __expf(lb - mx), wb = __expf(lj - mx);
    wsum = wsum * wa + wb;
    lb = mx;
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = x[i] * wa + xb[i] * wb;
  }
  const float inv = 1.f / wsum;
#pragma unroll
  for (int i = 0; i < 8; ++i) x[i] *= inv;
  Load8<T>::st(out + r.b * os.b + r.h * os.h + (int64_t)r.s * os.s + ch * 8, x);
  if (ch == 0) lse[((int64_t)r.b * H + r.h) * lse_bh + r.s] = lb + __logf(wsum);
}

// delta[b,h,s] = sum_d dout*out; the D/8 lanes of a row reduce with DPP-free shuffles.
template <typename T>
__global__ void __launch_bounds__(256) delta_kernel(const T* __restrict__ out, const T* __restrict__ dout,
                                                    float* __restrict__ delta, int H, int Sq, int cpr_shift,
                                                    unsigned nrows, unsigned half, Strides3 os, Strides3 ds) {
  const unsigned gid = blockIdx.x * 256u + threadIdx.x;
  const unsigned row0 = gid >> cpr_shift;
  const int cpr = 1 << cpr_shift;
  const int ch = (int)(gid & (unsigned)(cpr - 1));
  float a[ROWS_PER_THREAD][8], g[ROWS_PER_THREAD][8];
  int64_t di[ROWS_PER_THREAD];
  bool on[ROWS_PER_THREAD];
#pragma unroll
  for (int k = 0; k < ROWS_PER_THREAD; ++k) {
    const unsigned row = row0 + k * half;
    on[k] = row0 < half && row < nrows;
    const RowIdx r = decode_row(on[k] ? row : 0u, H);  // (rows past the end reread row 0: every lane takes part in the shuffles)
    di[k] = ((int64_t)r.b * H + r.h) * Sq + r.s;
    Load8<T>::ld(out + r.b * os.b + r.h * os.h + (int64_t)r.s * os.s + ch * 8, a[k]);
    Load8<T>::ld(dout + r.b * ds.b + r.h * ds.h + (int64_t)r.s * ds.s + ch * 8, g[k]);
  }
#pragma unroll
  for (int k = 0; k < ROWS_PER_THREAD; ++k) {
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc = __builtin_fmaf(a[k][i], g[k][i], acc);
    for (int off = cpr >> 1; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
    if (on[k] && ch == 0) delta[di[k]] = acc;
  }
}

// Grid of the three kernels: x covers half the rows of one batch entry (a thread takes a row of
// each half), y the batch.
struct RowGrid {
  dim3 grid;
  unsigned nrows, half;
  int cpr_shift;
  bool ok;
};
RowGrid row_grid(int B, int H, int Sq, int D) {
  RowGrid g;
  const int64_t nrows = (int64_t)H * Sq;
  g.cpr_shift = __builtin_ctz((unsigned)(D / 8));
  g.ok = nrows < 0x7fffffffLL / (D / 8) && B <= 65535;
  g.nrows = (unsigned)nrows;
  g.half = (unsigned)((nrows + ROWS_PER_THREAD - 1) / ROWS_PER_THREAD);
  const int64_t threads = (int64_t)g.half * (D / 8);
  g.grid = dim3((unsigned)((threads + 255) / 256), (unsigned)B);
  return g;
}

}  // namespace

hipError_t spa_launch_merge(float* out_acc, float* lse_acc, const void* blk_out, const float* blk_lse, int B,
                            int H, int Sq, int D, Strides3 as, Strides3 bs, int dtype, int init,
                            int64_t acc_lse_bh, hipStream_t stream) {
  const RowGrid g = row_grid(B, H, Sq, D);
  if (!g.ok) return hipErrorInvalidValue;
#define SPA_MERGE(T, I)                                                                              \
  hipLaunchKernelGGL((merge_kernel<T, I>), g.grid, dim3(256), 0, stream, out_acc, lse_acc, (const T*)blk_out, \
                     blk_lse, H, Sq, g.cpr_shift, g.nrows, g.half, as, bs, acc_lse_bh)
  if (dtype == 0) { if (init) SPA_MERGE(float, true); else SPA_MERGE(float, false); }
  else if (dtype == 1) { if (init) SPA_MERGE(__bf16, true); else SPA_MERGE(__bf16, false); }
  else if (dtype == 2) { if (init) SPA_MERGE(_Float16, true); else SPA_MERGE(_Float16, false); }
  else return hipErrorInvalidValue;
#undef SPA_MERGE
  return hipGetLastError();
}

hipError_t spa_launch_finalize(void* out, const float* out_acc, int B, int H, int Sq, int D, Strides3 os,
                               Strides3 as, int dtype, hipStream_t stream) {
  const RowGrid g = row_grid(B, H, Sq, D);
  if (!g.ok) return hipErrorInvalidValue;
  if (dtype == 0)
    hipLaunchKernelGGL((finalize_kernel<float>), g.grid, dim3(256), 0, stream, (float*)out, out_acc, H, g.cpr_shift, g.nrows, g.half, os, as);
  else if (dtype == 1)
    hipLaunchKernelGGL((finalize_kernel<__bf16>), g.grid, dim3(256), 0, stream, (__bf16*)out, out_acc, H, g.cpr_shift, g.nrows, g.half, os, as);
  else if (dtype == 2)
    hipLaunchKernelGGL((finalize_kernel<_Float16>), g.grid, dim3(256), 0, stream, (_Float16*)out, out_acc, H, g.cpr_shift, g.nrows, g.half, os, as);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

hipError_t spa_launch_delta(const void* out, const void* dout, float* delta, int B, int H, int Sq, int D,
                            Strides3 os, Strides3 ds, int dtype, hipStream_t stream) {
  const RowGrid g = row_grid(B, H, Sq, D);
  if (!g.ok) return hipErrorInvalidValue;
  if (dtype == 0)
    hipLaunchKernelGGL((delta_kernel<float>), g.grid, dim3(256), 0, stream, (const float*)out, (const float*)dout, delta, H, Sq, g.cpr_shift, g.nrows, g.half, os, ds);
  else if (dtype == 1)
    hipLaunchKernelGGL((delta_kernel<__bf16>), g.grid, dim3(256), 0, stream, (const __bf16*)out, (const __bf16*)dout, delta, H, Sq, g.cpr_shift, g.nrows, g.half, os, ds);
  else if (dtype == 2)
    hipLaunchKernelGGL((delta_kernel<_Float16>), g.grid, dim3(256), 0, stream, (const _Float16*)out, (const _Float16*)dout, delta, H, Sq, g.cpr_shift, g.nrows, g.half, os, ds);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

hipError_t spa_launch_splitkv_combine(void* out, float* lse, const void* part, const float* part_lse, int n, int B, int H, int Sq,
                                      int D, Strides3 os, int64_t lse_bh, int dtype, hipStream_t stream) {
  const RowGrid g = row_grid(B, H, Sq, D);
  if (!g.ok || n < 1) return hipErrorInvalidValue;
  if (dtype == 1)
    hipLaunchKernelGGL((splitkv_combine_kernel<__bf16>), g.grid, dim3(256), 0, stream, (__bf16*)out, lse, (const __bf16*)part, part_lse, n, H,
                       Sq, D, g.cpr_shift, g.nrows, os, lse_bh);
  else if (dtype == 2)
    hipLaunchKernelGGL((splitkv_combine_kernel<_Float16>), g.grid, dim3(256), 0, stream, (_Float16*)out, lse, (const _Float16*)part,
                       part_lse, n, H, Sq, D, g.cpr_shift, g.nrows, os, lse_bh);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}
