// Ulysses re-layout as one coalesced HBM pass per direction (pure byte movement).
// With the P ranks' shards stacked on a leading axis of one buffer:
//   s2h:  y[r][b, q*s+t, c, j, :] = x[q][b, t, c, r*h+j, :]     (h = H/P)
//   h2s:  x[r][b, t, c, q*h+j, :] = y[q][b, r*s+t, c, j, :]
// which is what the reference builds from reshape -> transpose -> contiguous ->
// all_to_all_single -> reshape -> transpose -> contiguous
// (sp_aurora/intel_ulysses_attn.py:86-140, sp_aurora/comm/all_to_all.py:266-333):
// three HBM passes there, one here.  The unit that moves is a run of h*D elements,
// contiguous on both sides; a thread moves one VB-byte vector of a run and the
// destination is walked linearly, so stores are fully coalesced and loads are
// coalesced within each run.
#include "spa_common.h"

namespace {

template <int VB>
struct Vec;
template <> struct Vec<16> { typedef u32x4 type; };
template <> struct Vec<8> { typedef u32x2 type; };
template <> struct Vec<4> { typedef unsigned int type; };
template <> struct Vec<2> { typedef unsigned short type; };
template <> struct Vec<1> { typedef unsigned char type; };

struct RelayoutParams {
  int P, B, s, pack;
  int run;      // vectors per (h*D) run
  int64_t total;  // vectors in the whole tensor
};

// S2H = true: dst is y (head-sharded), src is x (sequence-sharded); false: the inverse.
template <int VB, bool S2H>
__global__ void __launch_bounds__(256) relayout_kernel(const typename Vec<VB>::type* __restrict__ src,
                                                       typename Vec<VB>::type* __restrict__ dst,
                                                       const RelayoutParams p) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= p.total) return;
  int64_t t = idx;
  const int ju = (int)(t % p.run);
  t /= p.run;
  int64_t so;
  if (S2H) {
    // dst index (r, b, q, t, c, ju)
    const int c = (int)(t % p.pack); t /= p.pack;
    const int ts = (int)(t % p.s); t /= p.s;
    const int q = (int)(t % p.P); t /= p.P;
    const int b = (int)(t % p.B);
    const int r = (int)(t / p.B);
    // src x[q][b][ts][c][r*h + j]
    so = (((((int64_t)q * p.B + b) * p.s + ts) * p.pack + c) * p.P + r) * p.run + ju;
  } else {
    // dst index (r, b, ts, c, q, ju)
    const int q = (int)(t % p.P); t /= p.P;
    const int c = (int)(t % p.pack); t /= p.pack;
    const int ts = (int)(t % p.s); t /= p.s;
    const int b = (int)(t % p.B);
    const int r = (int)(t / p.B);
    // src y[q][b][r*s + ts][c][j]
    so = (((((int64_t)q * p.B + b) * p.P + r) * p.s + ts) * p.pack + c) * p.run + ju;
  }
  dst[idx] = src[so];
}

template <int VB>
hipError_t launch_vb(const void* src, void* dst, const RelayoutParams& p, bool s2h, hipStream_t stream) {
  typedef typename Vec<VB>::type V;
  const dim3 grid((unsigned)((p.total + 255) / 256));
  if (s2h)
    hipLaunchKernelGGL((relayout_kernel<VB, true>), grid, dim3(256), 0, stream, (const V*)src, (V*)dst, p);
  else
    hipLaunchKernelGGL((relayout_kernel<VB, false>), grid, dim3(256), 0, stream, (const V*)src, (V*)dst, p);
  return hipGetLastError();
}

}  // namespace

hipError_t spa_launch_relayout(const void* src, void* dst, int P, int B, int s, int H, int D, int pack,
                               int elem_bytes, bool s2h, hipStream_t stream) {
  const int64_t run_bytes = (int64_t)(H / P) * D * elem_bytes;
  int vb = 16;
  while (vb > 1 && (run_bytes % vb != 0 || ((uintptr_t)src % vb) != 0 || ((uintptr_t)dst % vb) != 0)) vb >>= 1;
  RelayoutParams p;
  p.P = P; p.B = B; p.s = s; p.pack = pack;
  p.run = (int)(run_bytes / vb);
  p.total = (int64_t)P * B * s * pack * P * p.run;
  if (p.total == 0) return hipSuccess;
  if ((p.total + 255) / 256 > 0x7fffffffLL) return hipErrorInvalidValue;
  switch (vb) {
    case 16: return launch_vb<16>(src, dst, p, s2h, stream);
    case 8: return launch_vb<8>(src, dst, p, s2h, stream);
    case 4: return launch_vb<4>(src, dst, p, s2h, stream);
    case 2: return launch_vb<2>(src, dst, p, s2h, stream);
    default: return launch_vb<1>(src, dst, p, s2h, stream);
  }
}
