// Ulysses re-layout as one coalesced HBM pass per direction (pure byte movement).
// With the P ranks' shards stacked on a leading axis of one buffer:
//   s2h:  y[r][b, q*s+t, c, j, :] = x[q][b, t, c, r*h+j, :]     (h = H/P)
//   h2s:  x[r][b, t, c, q*h+j, :] = y[q][b, r*s+t, c, j, :]
// which is what the reference builds from reshape -> transpose -> contiguous ->
// all_to_all_single -> reshape -> transpose -> contiguous
// (sp_aurora/intel_ulysses_attn.py:86-140, sp_aurora/comm/all_to_all.py:266-333):
// three HBM passes there, one here.
//
// The unit that moves is a RUN of h*D elements, contiguous on both sides.  Both directions are
// the same permutation of runs, indexed (r, b, q, t, c) with r the rank that owns the head
// group, q the rank that owns the sequence shard, t the row inside the shard:
//   head-sharded side   y: run index (((r*B + b)*P + q)*s + t)*pack + c
//   seq-sharded side    x: run index ((((q*B + b)*s + t)*pack + c)*P + r
// so one kernel serves both with the roles of source and destination swapped.  The grid carries
// (t tile, q*pack + c, [r*B +] b) in its three dimensions: a workgroup decodes its run strides once,
// from scalars; a thread needs one or two 32-bit divisions (shifts when the run holds a
// power-of-two number of vectors) per 16-byte vector, and moves four vectors with all loads issued
// before the first store.
#include "spa_common.h"

namespace {

template <int VB>
struct Vec;
template <> struct Vec<16> { typedef u32x4 type; };
template <> struct Vec<8> { typedef u32x2 type; };
template <> struct Vec<4> { typedef unsigned int type; };
template <> struct Vec<2> { typedef unsigned short type; };
template <> struct Vec<1> { typedef unsigned char type; };

constexpr int RL_THREADS = 256;
constexpr int RL_UNROLL = 4;  // vectors per thread in flight

struct RelayoutParams {
  int P, B, s, pack;
  unsigned run;       // vectors per run
  int run_shift;      // log2(run) when run is a power of two, else -1
  int line_shift;     // the same for run * P
  unsigned rows_tile; // rows t per workgroup
};

// S2H = true: dst is y (head-sharded), src is x (sequence-sharded); false: the inverse.
// Either way the DESTINATION is written in long contiguous stretches (scattered 1 KiB writes cost
// more than scattered 1 KiB reads):
//   s2h: a workgroup owns rows t0.. of one (r, b, q, c): y is contiguous over t (pack = 1), the
//        source runs sit pack*P runs apart;
//   h2s: a workgroup owns rows t0.. of one (q, b, c) for ALL r: x is contiguous over (r, vector)
//        within a row, rows pack*P runs apart; the source is P stretches, one per r, each
//        contiguous over t.
template <int VB, bool S2H>
__global__ void __launch_bounds__(RL_THREADS) relayout_kernel(const typename Vec<VB>::type* __restrict__ src,
                                                              typename Vec<VB>::type* __restrict__ dst,
                                                              const RelayoutParams p) {
  typedef typename Vec<VB>::type V;
  const unsigned t0 = blockIdx.x * p.rows_tile;
  const unsigned q = blockIdx.y / (unsigned)p.pack, c = blockIdx.y % (unsigned)p.pack;
  const unsigned r = S2H ? blockIdx.z / (unsigned)p.B : 0u, b = blockIdx.z % (unsigned)p.B;
  // first vector of run (r, b, q, t = 0, c) on either side, the step of one row t and of one rank r
  const int64_t y0 = ((((int64_t)r * p.B + b) * p.P + q) * p.s * p.pack + c) * p.run;
  const int64_t x0 = ((((int64_t)q * p.B + b) * p.s * p.pack + c) * p.P + r) * p.run;
  const int64_t ys = (int64_t)p.pack * p.run, xs = (int64_t)p.pack * p.P * p.run;
  const int64_t yr = (int64_t)p.B * p.P * p.s * p.pack * p.run;  // y: from one rank r to the next
  const unsigned rows = p.s - t0 < p.rows_tile ? p.s - t0 : p.rows_tile;  // rows of this tile
  const unsigned line = S2H ? p.run : p.run * (unsigned)p.P;              // contiguous destination vectors per row
  const int line_shift = S2H ? p.run_shift : p.line_shift;
  const unsigned total = rows * line;                                      // vectors of this tile
  // thread i of pass k moves vector i + k * RL_THREADS of the tile, counted row-major (row, [r,] vec)
  for (unsigned base = threadIdx.x; base < total; base += RL_THREADS * RL_UNROLL) {
    V val[RL_UNROLL];
    int64_t doff[RL_UNROLL];
    bool on[RL_UNROLL];
#pragma unroll
    for (int k = 0; k < RL_UNROLL; ++k) {
      const unsigned i = base + k * RL_THREADS;
      on[k] = i < total;
      const unsigned ii = on[k] ? i : 0;
      const unsigned row = line_shift >= 0 ? ii >> line_shift : ii / line;
      const unsigned rem = ii - row * line;
      const int64_t tt = (int64_t)(t0 + row);
      int64_t so;
      if (S2H) {
        doff[k] = y0 + tt * ys + rem;
        so = x0 + tt * xs + rem;
      } else {
        const unsigned rr = p.run_shift >= 0 ? rem >> p.run_shift : rem / p.run;
        const unsigned vec = rem - rr * p.run;
        doff[k] = x0 + tt * xs + rem;  // (r, vec) are contiguous in x
        so = y0 + rr * yr + tt * ys + vec;
      }
      if (on[k]) val[k] = __builtin_nontemporal_load(src + so);
    }
#pragma unroll
    for (int k = 0; k < RL_UNROLL; ++k)
      if (on[k]) __builtin_nontemporal_store(val[k], dst + doff[k]);
  }
}

template <int VB>
hipError_t launch_vb(const void* src, void* dst, const RelayoutParams& p, bool s2h, hipStream_t stream) {
  typedef typename Vec<VB>::type V;
  const dim3 grid((p.s + p.rows_tile - 1) / p.rows_tile, (unsigned)(p.P * p.pack), (unsigned)(s2h ? p.P * p.B : p.B));
  if (s2h)
    hipLaunchKernelGGL((relayout_kernel<VB, true>), grid, dim3(RL_THREADS), 0, stream, (const V*)src, (V*)dst, p);
  else
    hipLaunchKernelGGL((relayout_kernel<VB, false>), grid, dim3(RL_THREADS), 0, stream, (const V*)src, (V*)dst, p);
  return hipGetLastError();
}

}  // namespace

hipError_t spa_launch_relayout(const void* src, void* dst, int P, int B, int s, int H, int D, int pack,
                               int elem_bytes, bool s2h, hipStream_t stream) {
  const int64_t run_bytes = (int64_t)(H / P) * D * elem_bytes;
  int vb = 16;
  while (vb > 1 && (run_bytes % vb != 0 || ((uintptr_t)src % vb) != 0 || ((uintptr_t)dst % vb) != 0)) vb >>= 1;
  if ((int64_t)P * B * s * pack * P == 0 || run_bytes == 0) return hipSuccess;
  if (run_bytes / vb > 0x7fffffffLL / (RL_THREADS * RL_UNROLL)) return hipErrorInvalidValue;
  if ((int64_t)P * pack > 65535 || (int64_t)P * B > 65535) return hipErrorInvalidValue;
  RelayoutParams p;
  p.P = P; p.B = B; p.s = s; p.pack = pack;
  p.run = (unsigned)(run_bytes / vb);
  p.run_shift = (p.run & (p.run - 1)) == 0 ? __builtin_ctz(p.run) : -1;
  if ((int64_t)p.run * P > 0x7fffffffLL / (RL_THREADS * RL_UNROLL)) return hipErrorInvalidValue;
  const unsigned line = s2h ? p.run : p.run * (unsigned)P;
  p.line_shift = (line & (line - 1)) == 0 ? __builtin_ctz(line) : -1;
  // a workgroup takes enough rows t to give every thread RL_UNROLL vectors (one pass), at least one row
  const unsigned want = RL_THREADS * RL_UNROLL;
  p.rows_tile = line >= want ? 1u : (want + line - 1) / line;
  switch (vb) {
    case 16: return launch_vb<16>(src, dst, p, s2h, stream);
    case 8: return launch_vb<8>(src, dst, p, s2h, stream);
    case 4: return launch_vb<4>(src, dst, p, s2h, stream);
    case 2: return launch_vb<2>(src, dst, p, s2h, stream);
    default: return launch_vb<1>(src, dst, p, s2h, stream);
  }
}
