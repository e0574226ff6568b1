// Block-wise attention backward for gfx950 with the GLOBAL lse / delta of the query rows:
//   P = exp(q k^T * scale + mask - lse);  dV += P^T dO;  dP = dO V^T;
//   dS = P * (dP - delta);  dQ += dS K * scale;  dK += dS^T Q * scale.
// Stands in for the per-step body of intel_ring_flash_attn_backward
// (sp_aurora/intel_ring_flash_attn.py:192-258), which re-runs autograd on each block.
//
// Two kernels, no atomics, every output row has one owner (deterministic):
//   dq kernel   : workgroup = 128 or 256 query rows (4 or 8 waves x 32), walks key tiles of 64.
//                 S^T = K Q^T and dP^T = V dO^T land with a lane owning one query row,
//                 so lse/delta are per-lane scalars and dS^T is, register for register,
//                 the B operand of dQ^T = K^T dS^T.
//   dkdv kernel : workgroup = 128 keys (4 waves x 32), walks query tiles of 64.
//                 S = Q K^T and dP = dO V^T land with a lane owning one key, so P and dS
//                 are the B operands of dV^T = dO^T P and dK^T = Q^T dS.
//
// Streamed tiles (K, V / Q, dO; 64 rows) travel from global memory straight into LDS, several
// tiles ahead, rows back to back with their 16-byte chunks XOR-permuted so that both ways of
// reading a tile run without bank conflicts: rows as 16-byte reads (A operands of the S / dP
// contractions) and, through the transposing read, columns (A operands K^T, Q^T, dO^T of the
// gradient contractions).  No transposed copies exist.
//
// One wave per SIMD (the 8-wave dq kernel: two, which also halves the K/V traffic per query row),
// software-pipelined inside the wave at half-tile (32 rows) granularity:
// the MFMAs that produce S and dP of half-tile g+1 are interleaved, one to one, with the
// element-wise work (exp, dS) on half-tile g, followed by the gradient MFMAs of half-tile g.
// MFMA operands come from LDS through a rolling window that runs ahead of the MFMAs and is
// carried across loop iterations; one workgroup barrier per 64-row tile.
// Accumulators are fp32 in HBM and are ADDED to (read-modify-write by the owning lane).
// In the one-wave-per-SIMD kernels the MFMAs are written with their register files spelled out
// (gradient accumulators in AGPRs, S / dP tiles in VGPRs), see MmaAsm.
#include "spa_common.h"
#include "spa_host.h"
#include <stdlib.h>

namespace {

constexpr int BWD_THREADS = 256;
constexpr int BWD_ROWS = 64;    // rows (keys or queries) per streamed LDS tile
constexpr int BWD_STAGES = 4;   // tiles resident or on their way
constexpr int BWD_LOOK_MAX = 8; // operands are fetched from LDS up to this many MFMAs ahead
constexpr unsigned OFF_NONE = 0x80000000u;  // a buffer offset beyond any tensor: the load stores zeros

template <int D, int THREADS = BWD_THREADS>
struct BwdCfg {
  static constexpr int ROWB = D * 2;             // bytes per tile row
  static constexpr int TILEB = BWD_ROWS * ROWB;  // one tile
  static constexpr int CPR = D / 8;              // 16-byte chunks per row
  static constexpr int NDMA = TILEB / (THREADS * 16);  // direct loads per thread and tile
  static_assert(NDMA >= 1, "a tile must give every thread at least one 16-byte slot");
  static constexpr int RPD = THREADS / CPR;  // rows one round of the workgroup's loads covers
};

// Chunk permutation of a tile row, good for both read patterns: 16 consecutive rows at one chunk
// index fall into 16 different 16-byte bank groups, and so do the 4 rows x 4 chunks a half wave
// covers with one transposing read.  Depends on row % 16 only.
template <int D>
__device__ __forceinline__ int tile_swizzle(int row) {
  return D == 128 ? ((row & 3) << 2) | ((row >> 2) & 3)
         : D == 64 ? (((row >> 1) & 1) << 2) | ((row >> 2) & 3)
                   : (row >> 2) & 3;
}

// Per-lane LDS offsets (relative to a tile) of the two read patterns.
template <int D>
struct TileReads {
  unsigned row[D / 16];     // chunk 2 ks + hh of row ln (+ 32 rows: second half)
  unsigned tr[D / 32][2];   // transposing read of 4 dims of row 8 h8 + 4 hh + e (+ 16 u rows, + 32 rows)
  __device__ __forceinline__ void init(int lane) {
    typedef BwdCfg<D> C;
    const int ln = lane & 31, hh = lane >> 5;
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) row[ks] = ln * C::ROWB + (((2 * ks + hh) ^ tile_swizzle<D>(ln)) * 16);
    const int blk = lane >> 4, e = (lane >> 2) & 3, c4 = lane & 3;
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
      for (int h8 = 0; h8 < 2; ++h8) {
        const int r = 8 * h8 + 4 * hh + e;
        const int chunk = db * 4 + (blk & 1) * 2 + (c4 >> 1);
        tr[db][h8] = r * C::ROWB + ((chunk ^ tile_swizzle<D>(r)) * 16) + (c4 & 1) * 8;
      }
  }
};

// Global side of the direct loads: thread tid owns 16-byte slot tid of every round of 256 slots;
// round j covers rows j * RPD + tid / CPR.  Slot (row, pos) receives chunk pos ^ swizzle(row).
// BIG: the tensor's rows of one (batch, head) may span 2 GiB or more; the descriptor is re-based per tile
// (buffer_window) instead of covering the whole tensor.
template <typename T, int D, int THREADS = BWD_THREADS, bool BIG = false>
struct TileLoader {
  u32x4 rsrc;
  unsigned lane_off;  // bytes
  unsigned row_b;     // bytes per tensor row
  const T* base_;             // BIG only
  unsigned long long total_;  // BIG only: bytes from base_ to the end of the last row
  __device__ __forceinline__ void init(const T* base, int64_t row_stride, int rows, int tid) {
    typedef BwdCfg<D, THREADS> C;
    total_ = (unsigned long long)((((int64_t)rows - 1) * row_stride + D) * (int64_t)sizeof(T));
    base_ = base;
    rsrc = buffer_descriptor(base, BIG ? 0u : (unsigned)total_);  // (BIG: an empty range, for tiles that are not wanted)
    const int drow = tid / C::CPR, dpos = tid % C::CPR;
    lane_off = (unsigned)((drow * row_stride + ((dpos ^ tile_swizzle<D>(drow)) * 8)) * (int64_t)sizeof(T));
    row_b = (unsigned)(row_stride * (int64_t)sizeof(T));
  }
  // round q of the tile whose first tensor row is row0 (on = false: store zeros) into LDS at lds_wave
  __device__ __forceinline__ void load(int q, bool on, int row0, unsigned lds_wave) const {
    typedef BwdCfg<D, THREADS> C;
    if constexpr (BIG) {
      unsigned rel = OFF_NONE;
      u32x4 rs = rsrc;
      if (on) rs = buffer_window(base_, total_, (unsigned long long)(unsigned)row0 * row_b, rel);
      load_to_lds_b128(rs, lane_off + rel + (unsigned)(q * C::RPD) * row_b, lds_wave + q * (THREADS * 16));
      return;
    }
    const unsigned u = on ? (unsigned)(row0 + q * C::RPD) * row_b : OFF_NONE;
    load_to_lds_b128(rsrc, lane_off + u, lds_wave + q * (THREADS * 16));
  }
};

// One MFMA operand from two transposing reads (rows 0..3 and 8..11 of a lane's group of 16).
template <typename F>
__device__ __forceinline__ F frag_tr(unsigned addr_lo, unsigned addr_hi) {
  const u32x2 r0 = lds_read_tr16_b64(addr_lo);
  const u32x2 r1 = lds_read_tr16_b64(addr_hi);
  u32x4 x;
  x[0] = r0[0];
  x[1] = r0[1];
  x[2] = r1[0];
  x[3] = r1[1];
  return as_frag<F>(x);
}

__device__ __forceinline__ void zero16(f32x16& x) {
#pragma unroll
  for (int v = 0; v < 16; ++v) x[v] = 0.f;
}

template <int N>
__device__ __forceinline__ void wait_loads_but() {  // until at most N of this wave's loads are in flight
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

// MFMAs with the accumulator's register file spelled out.  The compiler gives every MFMA of a
// function the same form; the one-wave-per-SIMD kernels want both: the gradient accumulators
// (touched by MFMAs only) in AGPRs, the S / dP tiles, which the VALU works on, in VGPRs, so that
// no v_accvgpr_read / v_accvgpr_write copies are needed between the matrix pipe and the VALU.
// The compiler does not see these as MFMAs: the code keeps the distances the hardware needs
// (a VALU read of a tile comes at least 16 MFMAs after the tile's last MFMA; srcC is the
// destination itself or the literal 0, never a register a VALU instruction has just written).
template <typename T>
struct MmaAsm;
template <>
struct MmaAsm<__bf16> {
  typedef bf16x8 frag;
  static __device__ __forceinline__ void first_v(f32x16& c, frag a, frag b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void acc_v(f32x16& c, frag a, frag b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void acc_a(f32x16& c, frag a, frag b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
};
template <>
struct MmaAsm<_Float16> {
  typedef f16x8 frag;
  static __device__ __forceinline__ void first_v(f32x16& c, frag a, frag b) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void acc_v(f32x16& c, frag a, frag b) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void acc_a(f32x16& c, frag a, frag b) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
};

// ------------------------------------------------------------------------------------------
// dQ kernel
// ------------------------------------------------------------------------------------------
template <int D, int NW = 4>
struct DqCfg {
  typedef BwdCfg<D, NW * 64> C;
  static constexpr int STAGE = 2 * C::TILEB;  // K tile, V tile
  static constexpr int SMEM = BWD_STAGES * STAGE;
  static constexpr int NL = 2 * C::NDMA;      // loads per thread and stage
};

// Variable-length batch: sequence b owns rows cu_q[b] .. cu_q[b+1] of the query-side tensors and
// cu_k[b] .. cu_k[b+1] of the key-side ones; the kernel then works on that sequence as on batch 0
// of a batch whose bases and sizes are the sequence's.
template <typename T>
__device__ __forceinline__ void select_sequence(BwdParams& p, int& b) {
  if (!p.cu_q) return;
  const int q_lo = p.cu_q[b], k_lo = p.cu_k[b];
  p.Sq = p.cu_q[b + 1] - q_lo;
  p.Sk = p.cu_k[b + 1] - k_lo;
  p.q = (const T*)p.q + (int64_t)q_lo * p.qs.s;
  p.dout = (const T*)p.dout + (int64_t)q_lo * p.dos.s;
  p.k = (const T*)p.k + (int64_t)k_lo * p.ks.s;
  p.v = (const T*)p.v + (int64_t)k_lo * p.vs.s;
  const int64_t gsz = p.grads_in_t ? (int64_t)sizeof(T) : 4;  // gradients written in T, or fp32 accumulators
  p.dq = (float*)((char*)p.dq + q_lo * p.dqs.s * gsz);
  p.dk = (float*)((char*)p.dk + k_lo * p.dks.s * gsz);
  p.dv = (float*)((char*)p.dv + k_lo * p.dvs.s * gsz);
  p.lse += q_lo;
  p.delta += q_lo;
  b = 0;
}

// A row of a gradient that is written (BwdParams::grads_in_t) and that no tile contributes to: the
// lane's share of the row (the columns the epilogues give it) is set to zero.
template <typename E, int D>
__device__ __forceinline__ void zero_grad_row(E* rowp, int hh) {
#pragma unroll
  for (int db = 0; db < D / 32; ++db)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      if constexpr (sizeof(E) == 2) {
        const u32x2 z = {0u, 0u};
        *(u32x2*)(rowp + db * 32 + 8 * g + 4 * hh) = z;
      } else {
        const f32x4 z = {0.f, 0.f, 0.f, 0.f};
        *(f32x4*)(rowp + db * 32 + 8 * g + 4 * hh) = z;
      }
    }
}

template <typename T, int D, int NW, bool BIG = false>
__global__ void __launch_bounds__(NW * 64, 1) flash_bwd_dq_kernel(const BwdParams pk) {
  BwdParams p = pk;  // a variable-length batch rewrites the sizes and bases for its sequence below
  typedef BwdCfg<D, NW * 64> C;
  typedef DqCfg<D, NW> G;
  typedef Mma16<T> M;
  typedef MmaAsm<T> MA;
  // one wave per SIMD: AGPRs are there for the dq accumulators.  D = 128 only: its 8 gradient
  // MFMAs (with their operand reads) between a tile's last MFMA and the first VALU read of the
  // tile give the matrix pipe the time it needs; the shorter lists of smaller D would not.
  constexpr bool MIXED = NW == 4 && D == 128;
  typedef typename M::frag frag;
  extern __shared__ __align__(16) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63, ln = lane & 31, hh = lane >> 5;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);

  int bid = blockIdx.x;
  const int bh = bid % (p.B * p.H);  // (batch, head) pairs first: each keeps to one XCD also when H < 8
  const int h = bh % p.H;
  int b = bh / p.H;
  const int qt = p.nqt - 1 - bid / (p.B * p.H);
  const int q0 = qt * (NW * 32);
  const int qw0 = q0 + w * 32;
  select_sequence<T>(p, b);
  if (q0 >= p.Sq || p.Sk <= 0) {  // (variable-length batches only) no keys: nothing to add to dq, a written dq is zero
    if (p.grads_in_t && qw0 + ln < p.Sq)
      zero_grad_row<T, D>((T*)p.dq + b * p.dqs.b + h * p.dqs.h + (int64_t)(qw0 + ln) * p.dqs.s, hh);
    return;
  }

  const T* qp = (const T*)p.q + b * p.qs.b + h * p.qs.h;
  const T* kp = (const T*)p.k + b * p.ks.b + h * p.ks.h;
  const T* vp = (const T*)p.v + b * p.vs.b + h * p.vs.h;
  const T* dop = (const T*)p.dout + b * p.dos.b + h * p.dos.h;

  const int qrow = qw0 + ln;
  const int qrow_c = qrow < p.Sq ? qrow : p.Sq - 1;

  frag qf[D / 16], dof[D / 16];
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks) {
    qf[ks] = as_frag<frag>(*(const u32x4*)(qp + (int64_t)qrow_c * p.qs.s + ks * 16 + hh * 8));
    dof[ks] = as_frag<frag>(*(const u32x4*)(dop + (int64_t)qrow_c * p.dos.s + ks * 16 + hh * 8));
  }
  const int64_t li = ((int64_t)b * p.H + h) * p.lse_bh + qrow_c;
  const float l2 = p.lse[li] * 1.4426950408889634f;
  const float dl = p.delta[li];
  const float c = p.scale_log2;
  const float hidden = c < 0.f ? INFINITY : -INFINITY;  // a hidden score: exp2(hidden * c - lse) = 0 for either sign of the scale
  const int lim = p.causal ? (qrow < p.Sk - 1 ? qrow : p.Sk - 1) : p.Sk - 1;  // last visible key

  const int kv_end = p.causal ? (q0 + NW * 32 < p.Sk ? q0 + NW * 32 : p.Sk) : p.Sk;
  const int nt = (kv_end + BWD_ROWS - 1) / BWD_ROWS;  // key tiles this workgroup visits

  TileLoader<T, D, NW * 64, BIG> kld, vld;
  kld.init(kp, p.ks.s, p.Sk, tid);
  vld.init(vp, p.vs.s, p.Sk, tid);
  TileReads<D> rd;
  rd.init(lane);
  const unsigned lds0 = (unsigned)(uintptr_t)(lds_u8*)smem;
  auto stage_of = [&](int i) { return lds0 + (unsigned)((i & (BWD_STAGES - 1)) * G::STAGE); };
  auto issue_tile = [&](int i) {  // K and V tile i -> its stage
    const unsigned dst = stage_of(i) + w * 1024;
#pragma unroll
    for (int q = 0; q < C::NDMA; ++q) kld.load(q, i < nt, i * BWD_ROWS, dst);
#pragma unroll
    for (int q = 0; q < C::NDMA; ++q) vld.load(q, i < nt, i * BWD_ROWS, dst + C::TILEB);
  };
  auto issue_one = [&](int i, int n) {  // load n of tile i's G::NL, in issue_tile's order
    const unsigned dst = stage_of(i) + w * 1024;
    if (n < C::NDMA)
      kld.load(n, i < nt, i * BWD_ROWS, dst);
    else
      vld.load(n - C::NDMA, i < nt, i * BWD_ROWS, dst + C::TILEB);
  };

  f32x16 dq[D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; ++i) zero16(dq[i]);

  // Half-tile g = 2 i + t is keys [32 g, 32 g + 32).  One pass of the loop body handles tile i:
  //   list 2i  : S^T, dP^T of half 2i+1 (tile i, rows 32..63)   | dS^T of half 2i   | dQ of half 2i
  //   list 2i+1: S^T, dP^T of half 2i+2 (tile i+1, rows 0..31)  | dS^T of half 2i+1 | dQ of half 2i+1
  // NA MFMAs produce, the element-wise work rides between them, NB MFMAs consume.
  constexpr int NA = 2 * (D / 16), NB = 2 * (D / 32), NLIST = NA + NB, NBODY = 2 * NLIST;
  constexpr int LOOK_CAP = NW == 8 ? 4 : BWD_LOOK_MAX;  // two waves per SIMD: 256 registers each, and the other wave covers LDS latency
  constexpr int BWD_LOOK = NA < LOOK_CAP ? NA : LOOK_CAP;
  static_assert(NBODY % BWD_LOOK == 0 && BWD_LOOK <= NA, "the operand window must tile the loop body");

  issue_tile(0);
  issue_tile(1);
  issue_tile(2);
  wait_loads_but<2 * G::NL>();
  __syncthreads();

  f32x16 sc, dc, sn, dn;  // S^T, dP^T of the current / next half-tile
  {
    if (!MIXED) {
      zero16(sc);
      zero16(dc);
    }
    const unsigned kb = stage_of(0);
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) {
      const frag a0 = as_frag<frag>(lds_read_b128(kb + rd.row[ks]));
      const frag a1 = as_frag<frag>(lds_read_b128(kb + C::TILEB + rd.row[ks]));
      if (MIXED) {
        if (ks == 0) {
          MA::first_v(sc, a0, qf[0]);
          MA::first_v(dc, a1, dof[0]);
        } else {
          MA::acc_v(sc, a0, qf[ks]);
          MA::acc_v(dc, a1, dof[ks]);
        }
      } else {
        sc = M::run(a0, qf[ks], sc);
        dc = M::run(a1, dof[ks], dc);
      }
    }
  }

  // operand fetch number J of the body of tile i (J >= NBODY: the first operands of the next body)
  unsigned row_cur[D / 16], row_nxt[D / 16], tr_cur[D / 32][2];
  auto set_addresses = [&](int i) {
    const unsigned a = stage_of(i), n = stage_of(i + 1);
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) {
      row_cur[ks] = a + rd.row[ks];
      row_nxt[ks] = n + rd.row[ks];
    }
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
      for (int h8 = 0; h8 < 2; ++h8) tr_cur[db][h8] = a + rd.tr[db][h8];
  };
  auto fetch = [&](int J) -> frag {
    const int body = J / NBODY, j2 = J % NBODY;
    const int list = j2 / NLIST, j = j2 % NLIST;
    if (j < NA) {  // j = 2 ks + which: K row (S^T) or V row (dP^T) of the half-tile being produced
      const int ks = j >> 1, which = j & 1;
      // list 0 of this body: tile i rows 32..; list 1: tile i+1 rows 0..; list 0 of the next body: tile i+1 rows 32..
      const unsigned base = (body == 0 && list == 0) ? row_cur[ks] + 32 * C::ROWB
                            : (body == 0)           ? row_nxt[ks]
                                                    : row_nxt[ks] + 32 * C::ROWB;
      return as_frag<frag>(lds_read_b128(base + which * C::TILEB));
    }
    const int jb = j - NA;  // jb = u * (D/32) + db : K^T operand of half-tile `list` of tile i
    const int db = jb % (D / 32), u = jb / (D / 32);
    const unsigned off = (list * 32 + u * 16) * C::ROWB;
    return frag_tr<frag>(tr_cur[db][0] + off, tr_cur[db][1] + off);
  };

  frag win[BWD_LOOK];
  frag dsf[2];
  set_addresses(0);
#pragma unroll
  for (int j = 0; j < BWD_LOOK; ++j) win[j] = fetch(j);
  // The loads of tile i + 3 go out one at a time between the MFMAs of the pass: issued in one burst
  // after the barrier, they hold up the wave's instruction stream while the memory pipeline takes them in.
  constexpr int LOAD_GAP = NBODY / G::NL;
  for (int i = 0; i < nt; ++i) {
    // tile i+1 must have landed before this body reads it; tile i-1 is free for tile i+3
    wait_loads_but<G::NL>();
    __syncthreads();
    set_addresses(i);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int list = 0; list < 2; ++list) {
      const int key0 = (2 * i + list) * 32;  // first key of the half-tile whose dS is formed in this list
      // diagonal: hide the keys after each lane's query; last tile: hide the keys past the end (their K
      // and V rows arrive as zeros, but P = exp(0 - lse) overflows for lse < -88 and inf * 0 is NaN)
      if ((p.causal && key0 + 31 > qw0) || key0 + 31 >= p.Sk) {
#pragma unroll
        for (int v = 0; v < 16; ++v)
          if (key0 + 8 * (v >> 2) + 4 * hh + (v & 3) > lim) sc[v] = hidden;
      }
      if (!MIXED) {
        zero16(sn);
        zero16(dn);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int j = 0; j < NLIST; ++j) {
        const int J = list * NLIST + j;
        const frag a = win[J % BWD_LOOK];
        win[J % BWD_LOOK] = fetch(J + BWD_LOOK);
        __builtin_amdgcn_sched_barrier(0);
        if (j < NA) {
          const int ks = j >> 1;
          if (MIXED) {
            if (j & 1) {
              if (ks == 0) MA::first_v(dn, a, dof[0]); else MA::acc_v(dn, a, dof[ks]);
            } else {
              if (ks == 0) MA::first_v(sn, a, qf[0]); else MA::acc_v(sn, a, qf[ks]);
            }
          } else if (j & 1) {
            dn = M::run(a, dof[ks], dn);
          } else {
            sn = M::run(a, qf[ks], sn);
          }
          // element-wise work on the current half-tile, spread over the producing MFMAs
#pragma unroll
          for (int v = 0; v < 16; ++v)
            if (v * NA / 16 == j) {
              const float pr = fast_exp2(__builtin_fmaf(sc[v], c, -l2));
              sc[v] = pr * (dc[v] - dl);
            }
          if (j == NA / 2 - 1)
            dsf[0] = M::pack(sc[0], sc[1], sc[2], sc[3], sc[4], sc[5], sc[6], sc[7]);
          if (j == NA - 1) dsf[1] = M::pack(sc[8], sc[9], sc[10], sc[11], sc[12], sc[13], sc[14], sc[15]);
        } else {
          const int jb = j - NA;
          const int db = jb % (D / 32), u = jb / (D / 32);
          if (MIXED)
            MA::acc_a(dq[db], a, dsf[u]);
          else
            dq[db] = M::run(a, dsf[u], dq[db]);
        }
        if (J % LOAD_GAP == LOAD_GAP / 2 && J / LOAD_GAP < G::NL) issue_one(i + 3, J / LOAD_GAP);
        __builtin_amdgcn_sched_barrier(0);
      }
      sc = sn;
      dc = dn;
    }
  }
  wait_loads_but<0>();  // nothing may still be writing LDS when the workgroup ends
  // The last MFMAs must have written dq before it is read.  The accumulators are operands of the
  // wait, so no read of them can be scheduled above it.
  if constexpr (MIXED) asm volatile("s_nop 15\n s_nop 15" : "+a"(dq[0]), "+a"(dq[1]), "+a"(dq[2]), "+a"(dq[3])::"memory");

  if (qrow < p.Sq && p.grads_in_t) {
    // the whole gradient of the row: written in q's element type, nothing read
    T* dqp = (T*)p.dq + b * p.dqs.b + h * p.dqs.h + (int64_t)qrow * p.dqs.s;
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2 st;
        st[0] = Mma16<T>::pack2(dq[db][4 * g + 0] * p.scale, dq[db][4 * g + 1] * p.scale);
        st[1] = Mma16<T>::pack2(dq[db][4 * g + 2] * p.scale, dq[db][4 * g + 3] * p.scale);
        *(u32x2*)(dqp + db * 32 + 8 * g + 4 * hh) = st;
      }
  } else if (qrow < p.Sq) {
    float* dqp = p.dq + b * p.dqs.b + h * p.dqs.h + (int64_t)qrow * p.dqs.s;
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        f32x4* dst = (f32x4*)(dqp + db * 32 + 8 * g + 4 * hh);
        f32x4 x = *dst;
        x[0] += dq[db][4 * g + 0] * p.scale;
        x[1] += dq[db][4 * g + 1] * p.scale;
        x[2] += dq[db][4 * g + 2] * p.scale;
        x[3] += dq[db][4 * g + 3] * p.scale;
        *dst = x;
      }
  }
}

// ------------------------------------------------------------------------------------------
// dK / dV kernel
// ------------------------------------------------------------------------------------------
template <int D>
struct DkvCfg {
  typedef BwdCfg<D> C;
  static constexpr int STAT = 2 * BWD_ROWS * 4;       // lse and delta of the tile's query rows
  static constexpr int STAGE = 2 * C::TILEB + STAT;   // Q tile, dO tile, stats
  static constexpr int SMEM = BWD_STAGES * STAGE;
  static constexpr int NL = 2 * C::NDMA + 1;          // loads per thread and stage
};

// ASM = false: the D = 128 kernel with every MFMA left to the compiler (its uniform accumulator
// form, its own hazard handling): slower, kept as the test twin of the hand-issued form.
template <typename T, int D, bool ASM = true, bool BIG = false>
__global__ void __launch_bounds__(BWD_THREADS, 1) flash_bwd_dkdv_kernel(const BwdParams pk) {
  BwdParams p = pk;  // a variable-length batch rewrites the sizes and bases for its sequence below
  typedef BwdCfg<D> C;
  typedef DkvCfg<D> G;
  typedef Mma16<T> M;
  typedef MmaAsm<T> MA;
  constexpr bool MIXED = D == 128 && ASM;  // see the dq kernel; here 16 gradient MFMAs separate a tile's MFMAs from its VALU reads
  typedef typename M::frag frag;
  extern __shared__ __align__(16) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63, ln = lane & 31, hh = lane >> 5;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);

  int bid = blockIdx.x;
  const int bh = bid % (p.B * p.H);  // (batch, head) pairs first: each keeps to one XCD also when H < 8
  const int h = bh % p.H;
  int b = bh / p.H;
  const int kt = bid / (p.B * p.H);  // causal: low key tiles see the most query tiles, they go first
  const int k0 = kt * 128;
  const int kw0 = k0 + w * 32;
  select_sequence<T>(p, b);
  if (k0 >= p.Sk || p.Sq <= 0 || (p.causal && k0 >= p.Sq)) {  // no query sees these keys: nothing to add to dk, dv
    if (p.grads_in_t && kw0 + ln < p.Sk) {                     // written gradients of such keys are zero
      zero_grad_row<T, D>((T*)p.dk + b * p.dks.b + h * p.dks.h + (int64_t)(kw0 + ln) * p.dks.s, hh);
      zero_grad_row<T, D>((T*)p.dv + b * p.dvs.b + h * p.dvs.h + (int64_t)(kw0 + ln) * p.dvs.s, hh);
    }
    return;
  }

  const T* qp = (const T*)p.q + b * p.qs.b + h * p.qs.h;
  const T* kp = (const T*)p.k + b * p.ks.b + h * p.ks.h;
  const T* vp = (const T*)p.v + b * p.vs.b + h * p.vs.h;
  const T* dop = (const T*)p.dout + b * p.dos.b + h * p.dos.h;
  const float* lsep = p.lse + ((int64_t)b * p.H + h) * p.lse_bh;
  const float* delp = p.delta + ((int64_t)b * p.H + h) * p.lse_bh;

  const int krow = kw0 + ln;
  const int krow_c = krow < p.Sk ? krow : p.Sk - 1;

  frag kf[D / 16], vf[D / 16];
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks) {
    kf[ks] = as_frag<frag>(*(const u32x4*)(kp + (int64_t)krow_c * p.ks.s + ks * 16 + hh * 8));
    vf[ks] = as_frag<frag>(*(const u32x4*)(vp + (int64_t)krow_c * p.vs.s + ks * 16 + hh * 8));
  }
  const float c = p.scale_log2;
  const float hidden = c < 0.f ? INFINITY : -INFINITY;  // a hidden score: exp2(hidden * c - lse) = 0 for either sign of the scale

  // causal: query rows before the first key of this workgroup see none of its keys
  const int it0 = p.causal ? k0 / BWD_ROWS : 0;
  const int nt = (p.Sq + BWD_ROWS - 1) / BWD_ROWS;  // query tiles it0 .. nt-1 are visited

  TileLoader<T, D, BWD_THREADS, BIG> qld, dold;
  qld.init(qp, p.qs.s, p.Sq, tid);
  dold.init(dop, p.dos.s, p.Sq, tid);
  // per-row statistics: waves 0, 2 fetch the tile's 64 lse values, waves 1, 3 its 64 delta values
  // (the pairs store the same bytes to the same place, which keeps every wave's load count equal)
  const u32x4 stat_rsrc = buffer_descriptor((w & 1) ? delp : lsep, (unsigned)p.Sq * 4u);
  TileReads<D> rd;
  rd.init(lane);
  const unsigned lds0 = (unsigned)(uintptr_t)(lds_u8*)smem;
  auto stage_of = [&](int i) { return lds0 + (unsigned)((i & (BWD_STAGES - 1)) * G::STAGE); };
  auto issue_tile = [&](int i) {  // Q and dO tile i and their statistics -> stage
    const unsigned st = stage_of(i);
    const unsigned dst = st + w * 1024;
#pragma unroll
    for (int q = 0; q < C::NDMA; ++q) qld.load(q, i < nt, i * BWD_ROWS, dst);
#pragma unroll
    for (int q = 0; q < C::NDMA; ++q) dold.load(q, i < nt, i * BWD_ROWS, dst + C::TILEB);
    load_to_lds_b32(stat_rsrc, i < nt ? (unsigned)(i * BWD_ROWS + lane) * 4u : OFF_NONE,
                    st + 2 * C::TILEB + (w & 1) * (BWD_ROWS * 4));
  };
  auto issue_one = [&](int i, int n) {  // load n of tile i's G::NL, in issue_tile's order
    const unsigned st = stage_of(i);
    const unsigned dst = st + w * 1024;
    if (n < C::NDMA)
      qld.load(n, i < nt, i * BWD_ROWS, dst);
    else if (n < 2 * C::NDMA)
      dold.load(n - C::NDMA, i < nt, i * BWD_ROWS, dst + C::TILEB);
    else
      load_to_lds_b32(stat_rsrc, i < nt ? (unsigned)(i * BWD_ROWS + lane) * 4u : OFF_NONE,
                      st + 2 * C::TILEB + (w & 1) * (BWD_ROWS * 4));
  };

  f32x16 dk[D / 32], dv[D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; ++i) {
    zero16(dk[i]);
    zero16(dv[i]);
  }

  // Half-tile g = 2 i + t is query rows [32 g, 32 g + 32).  Body of tile i:
  //   list 2i  : S, dP of half 2i+1 (tile i rows 32..63)  | P, dS of half 2i   | dV, dK from half 2i
  //   list 2i+1: S, dP of half 2i+2 (tile i+1 rows 0..31) | P, dS of half 2i+1 | dV, dK from half 2i+1
  constexpr int NA = 2 * (D / 16), NB = 4 * (D / 32), NLIST = NA + NB, NBODY = 2 * NLIST;
  constexpr int BWD_LOOK = NA < BWD_LOOK_MAX ? NA : BWD_LOOK_MAX;
  static_assert(NBODY % BWD_LOOK == 0 && BWD_LOOK <= NA, "the operand window must tile the loop body");

  if (it0 < nt) {  // uniform; a workgroup whose keys no query sees adds nothing
    issue_tile(it0);
    issue_tile(it0 + 1);
    issue_tile(it0 + 2);
    wait_loads_but<2 * G::NL>();
    __syncthreads();

    f32x16 sc, dc, sn, dn;
    {
      const unsigned qb = stage_of(it0);
#pragma unroll
      for (int ks = 0; ks < D / 16; ++ks) {
        const frag a0 = as_frag<frag>(lds_read_b128(qb + rd.row[ks]));
        const frag a1 = as_frag<frag>(lds_read_b128(qb + C::TILEB + rd.row[ks]));
        if (!MIXED) {
          if (ks == 0) {
            zero16(sc);
            zero16(dc);
          }
          sc = M::run(a0, kf[ks], sc);
          dc = M::run(a1, vf[ks], dc);
        } else if (ks == 0) {
          MA::first_v(sc, a0, kf[0]);
          MA::first_v(dc, a1, vf[0]);
        } else {
          MA::acc_v(sc, a0, kf[ks]);
          MA::acc_v(dc, a1, vf[ks]);
        }
      }
    }

    unsigned row_cur[D / 16], row_nxt[D / 16], tr_cur[D / 32][2];
    unsigned stat_cur;
    auto set_addresses = [&](int i) {
      const unsigned a = stage_of(i), n = stage_of(i + 1);
#pragma unroll
      for (int ks = 0; ks < D / 16; ++ks) {
        row_cur[ks] = a + rd.row[ks];
        row_nxt[ks] = n + rd.row[ks];
      }
#pragma unroll
      for (int db = 0; db < D / 32; ++db)
#pragma unroll
        for (int h8 = 0; h8 < 2; ++h8) tr_cur[db][h8] = a + rd.tr[db][h8];
      stat_cur = a + 2 * C::TILEB + 16 * hh;
    };
    auto fetch = [&](int J) -> frag {
      const int body = J / NBODY, j2 = J % NBODY;
      const int list = j2 / NLIST, j = j2 % NLIST;
      if (j < NA) {  // j = 2 ks + which: Q row (S) or dO row (dP) of the half-tile being produced
        const int ks = j >> 1, which = j & 1;
        const unsigned base = (body == 0 && list == 0) ? row_cur[ks] + 32 * C::ROWB
                              : (body == 0)           ? row_nxt[ks]
                                                      : row_nxt[ks] + 32 * C::ROWB;
        return as_frag<frag>(lds_read_b128(base + which * C::TILEB));
      }
      // jb = (u * (D/32) + db) * 2 + which: dO^T (for dV) or Q^T (for dK) operand of half-tile `list`
      const int jb = j - NA;
      const int which = jb & 1, db = (jb >> 1) % (D / 32), u = (jb >> 1) / (D / 32);
      const unsigned off = (which ? 0 : C::TILEB) + (list * 32 + u * 16) * C::ROWB;
      return frag_tr<frag>(tr_cur[db][0] + off, tr_cur[db][1] + off);
    };

    frag win[BWD_LOOK];
    frag pf[2], dsf[2];
    set_addresses(it0);
#pragma unroll
    for (int j = 0; j < BWD_LOOK; ++j) win[j] = fetch(j);
    // The loads of tile i + 3 go out one at a time between the MFMAs of the pass: issued in one
    // burst after the barrier, they hold up the wave's instruction stream while the memory pipeline
    // takes them in.
    constexpr int LOAD_GAP = NBODY / G::NL;
    for (int i = it0; i < nt; ++i) {
      wait_loads_but<G::NL>();
      __syncthreads();
      set_addresses(i);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int list = 0; list < 2; ++list) {
        const int r0 = (2 * i + list) * 32;  // first query row of the half-tile whose P, dS are formed here
        if (p.causal && kw0 + 31 > r0) {     // diagonal: a key sees only the queries at or after it
#pragma unroll
          for (int v = 0; v < 16; ++v)
            if (krow > r0 + 8 * (v >> 2) + 4 * hh + (v & 3)) sc[v] = hidden;
        }
        // lse (times -log2 e) and delta of this lane's 16 query rows
        float nl[16], de[16];
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          // (whole-vector casts: a bit cast of one element of a vector reads element 0)
          const f32x4 l4 = __builtin_bit_cast(f32x4, lds_read_b128(stat_cur + (list * 32 + 8 * g4) * 4));
          const f32x4 d4 = __builtin_bit_cast(f32x4, lds_read_b128(stat_cur + (BWD_ROWS + list * 32 + 8 * g4) * 4));
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            nl[4 * g4 + e] = l4[e] * -1.4426950408889634f;
            de[4 * g4 + e] = d4[e];
          }
        }
        if (!MIXED) {
          zero16(sn);
          zero16(dn);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < NLIST; ++j) {
          const int J = list * NLIST + j;
          const frag a = win[J % BWD_LOOK];
          win[J % BWD_LOOK] = fetch(J + BWD_LOOK);
          __builtin_amdgcn_sched_barrier(0);
          if (j < NA) {
            const int ks = j >> 1;
            if (!MIXED) {
              if (j & 1)
                dn = M::run(a, vf[ks], dn);
              else
                sn = M::run(a, kf[ks], sn);
            } else if (j & 1) {
              if (ks == 0) MA::first_v(dn, a, vf[0]); else MA::acc_v(dn, a, vf[ks]);
            } else {
              if (ks == 0) MA::first_v(sn, a, kf[0]); else MA::acc_v(sn, a, kf[ks]);
            }
#pragma unroll
            for (int v = 0; v < 16; ++v)
              if (v * NA / 16 == j) {
                const float pr = fast_exp2(__builtin_fmaf(sc[v], c, nl[v]));
                sc[v] = pr;
                dc[v] = pr * (dc[v] - de[v]);
              }
            if (j == NA / 2 - 1) {
              pf[0] = M::pack(sc[0], sc[1], sc[2], sc[3], sc[4], sc[5], sc[6], sc[7]);
              dsf[0] = M::pack(dc[0], dc[1], dc[2], dc[3], dc[4], dc[5], dc[6], dc[7]);
            }
            if (j == NA - 1) {
              pf[1] = M::pack(sc[8], sc[9], sc[10], sc[11], sc[12], sc[13], sc[14], sc[15]);
              dsf[1] = M::pack(dc[8], dc[9], dc[10], dc[11], dc[12], dc[13], dc[14], dc[15]);
            }
          } else {
            const int jb = j - NA;
            const int which = jb & 1, db = (jb >> 1) % (D / 32), u = (jb >> 1) / (D / 32);
            if (!MIXED) {
              if (which)
                dk[db] = M::run(a, dsf[u], dk[db]);
              else
                dv[db] = M::run(a, pf[u], dv[db]);
            } else if (which) {
              MA::acc_a(dk[db], a, dsf[u]);
            } else {
              MA::acc_a(dv[db], a, pf[u]);
            }
          }
          if (J % LOAD_GAP == LOAD_GAP / 2 && J / LOAD_GAP < G::NL) issue_one(i + 3, J / LOAD_GAP);
          __builtin_amdgcn_sched_barrier(0);
        }
        sc = sn;
        dc = dn;
      }
    }
    wait_loads_but<0>();
  }
  // The last MFMAs must have written dk / dv before they are read; the accumulators are operands of
  // the wait, so no read of them can be scheduled above it.
  if constexpr (MIXED)
    asm volatile("s_nop 15\n s_nop 15"
                 : "+a"(dk[0]), "+a"(dk[1]), "+a"(dk[2]), "+a"(dk[3]), "+a"(dv[0]), "+a"(dv[1]), "+a"(dv[2]), "+a"(dv[3])::"memory");

  if (krow < p.Sk && p.grads_in_t) {
    T* dkp = (T*)p.dk + b * p.dks.b + h * p.dks.h + (int64_t)krow * p.dks.s;
    T* dvp = (T*)p.dv + b * p.dvs.b + h * p.dvs.h + (int64_t)krow * p.dvs.s;
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2 x, y;
        x[0] = Mma16<T>::pack2(dk[db][4 * g + 0] * p.scale, dk[db][4 * g + 1] * p.scale);
        x[1] = Mma16<T>::pack2(dk[db][4 * g + 2] * p.scale, dk[db][4 * g + 3] * p.scale);
        y[0] = Mma16<T>::pack2(dv[db][4 * g + 0], dv[db][4 * g + 1]);
        y[1] = Mma16<T>::pack2(dv[db][4 * g + 2], dv[db][4 * g + 3]);
        *(u32x2*)(dkp + db * 32 + 8 * g + 4 * hh) = x;
        *(u32x2*)(dvp + db * 32 + 8 * g + 4 * hh) = y;
      }
  } else if (krow < p.Sk) {
    float* dkp = p.dk + b * p.dks.b + h * p.dks.h + (int64_t)krow * p.dks.s;
    float* dvp = p.dv + b * p.dvs.b + h * p.dvs.h + (int64_t)krow * p.dvs.s;
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        f32x4* d1 = (f32x4*)(dkp + db * 32 + 8 * g + 4 * hh);
        f32x4* d2 = (f32x4*)(dvp + db * 32 + 8 * g + 4 * hh);
        f32x4 x = *d1, y = *d2;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          x[e] += dk[db][4 * g + e] * p.scale;
          y[e] += dv[db][4 * g + e];
        }
        *d1 = x;
        *d2 = y;
      }
  }
}

// ------------------------------------------------------------------------------------------
// fp32 kernels: the same two-kernel scheme on v_mfma_f32_32x32x2_f32 (fp32 products and
// accumulation, P and dS stay fp32).  Correctness path for fp32 inputs: tiles of 32 rows staged
// through registers, no software pipeline.  The contraction index of the gradient products is the
// row an accumulator register holds (8*(v/4) + 4*hh + v%4), so P and dS are used where they are.
// ------------------------------------------------------------------------------------------
constexpr int B32_ROWS = 32;

template <int D>
struct Bwd32Cfg {
  static constexpr int PITCH = D + 4;              // floats per LDS row
  static constexpr int TILE = B32_ROWS * PITCH;    // floats per tile
  static constexpr int STAT = 2 * B32_ROWS;        // lse * log2 e and delta of a query tile
  static constexpr int SMEM_DQ = 2 * 2 * TILE * 4;
  static constexpr int SMEM_DKV = 2 * (2 * TILE + STAT) * 4;
  static constexpr int CPR = D / 4;
  static constexpr int RPP = BWD_THREADS / CPR;
  static constexpr int PASS = (B32_ROWS + RPP - 1) / RPP;
};

// two row-major tiles of 32 rows (a, b) of tensors with the same row count, staged together
template <int D>
struct PairStage {
  typedef Bwd32Cfg<D> C;
  f32x4 ra[C::PASS], rb[C::PASS];
  __device__ __forceinline__ void gload(const float* a, int64_t as, const float* b, int64_t bs, int row0, int nrows, int tid) {
    const int cc = tid % C::CPR, cr = tid / C::CPR;
#pragma unroll
    for (int i = 0; i < C::PASS; ++i) {
      const int lr = cr + i * C::RPP;
      if (lr < B32_ROWS) {
        int r = row0 + lr;
        r = r < nrows ? r : nrows - 1;
        ra[i] = *(const f32x4*)(a + (int64_t)r * as + cc * 4);
        rb[i] = *(const f32x4*)(b + (int64_t)r * bs + cc * 4);
      }
    }
  }
  __device__ __forceinline__ void lstore(float* ta, float* tb, int tid) const {
    const int cc = tid % C::CPR, cr = tid / C::CPR;
#pragma unroll
    for (int i = 0; i < C::PASS; ++i) {
      const int lr = cr + i * C::RPP;
      if (lr < B32_ROWS) {
        *(f32x4*)(ta + lr * C::PITCH + cc * 4) = ra[i];
        *(f32x4*)(tb + lr * C::PITCH + cc * 4) = rb[i];
      }
    }
  }
};

template <int D>
__global__ void __launch_bounds__(BWD_THREADS, 1) flash_bwd32_dq_kernel(const BwdParams pk) {
  BwdParams p = pk;  // a variable-length batch rewrites the sizes and bases for its sequence below
  typedef Bwd32Cfg<D> C;
  extern __shared__ __align__(16) unsigned char smem[];
  float* sm = (float*)smem;
  const int tid = threadIdx.x;
  const int lane = tid & 63, w = tid >> 6, ln = lane & 31, hh = lane >> 5;

  int bid = blockIdx.x;
  const int bh = bid % (p.B * p.H);  // (batch, head) pairs first: each keeps to one XCD also when H < 8
  const int h = bh % p.H;
  int b = bh / p.H;
  const int qt = p.nqt - 1 - bid / (p.B * p.H);
  const int q0 = qt * 128;
  const int qw0 = q0 + w * 32;
  select_sequence<float>(p, b);
  if (q0 >= p.Sq || p.Sk <= 0) {  // (variable-length batches only) no keys: nothing to add to dq, a written dq is zero
    if (p.grads_in_t && qw0 + ln < p.Sq)
      zero_grad_row<float, D>(p.dq + b * p.dqs.b + h * p.dqs.h + (int64_t)(qw0 + ln) * p.dqs.s, hh);
    return;
  }

  const float* qp = (const float*)p.q + b * p.qs.b + h * p.qs.h;
  const float* kp = (const float*)p.k + b * p.ks.b + h * p.ks.h;
  const float* vp = (const float*)p.v + b * p.vs.b + h * p.vs.h;
  const float* dop = (const float*)p.dout + b * p.dos.b + h * p.dos.h;

  const int qrow = qw0 + ln;
  const int qrow_c = qrow < p.Sq ? qrow : p.Sq - 1;
  // contraction step of the first products: head dim 8*g + 4*hh + e
  f32x4 qf[D / 8], dof[D / 8];
#pragma unroll
  for (int g = 0; g < D / 8; ++g) {
    qf[g] = *(const f32x4*)(qp + (int64_t)qrow_c * p.qs.s + 8 * g + 4 * hh);
    dof[g] = *(const f32x4*)(dop + (int64_t)qrow_c * p.dos.s + 8 * g + 4 * hh);
  }
  const int64_t li = ((int64_t)b * p.H + h) * p.lse_bh + qrow_c;
  const float l2 = p.lse[li] * 1.4426950408889634f;
  const float dl = p.delta[li];
  const float c = p.scale_log2;
  const int lim = p.causal ? (qrow < p.Sk - 1 ? qrow : p.Sk - 1) : p.Sk - 1;  // last visible key

  const int kv_end = p.causal ? (q0 + 128 < p.Sk ? q0 + 128 : p.Sk) : p.Sk;
  const int nt = (kv_end + B32_ROWS - 1) / B32_ROWS;

  f32x16 dq[D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; ++i) zero16(dq[i]);

  PairStage<D> st;
  st.gload(kp, p.ks.s, vp, p.vs.s, 0, p.Sk, tid);
  st.lstore(sm, sm + C::TILE, tid);
  __syncthreads();

  for (int it = 0; it < nt; ++it) {
    const int cur = it & 1;
    const int key0 = it * B32_ROWS;
    const bool more = it + 1 < nt;
    if (more) st.gload(kp, p.ks.s, vp, p.vs.s, key0 + B32_ROWS, p.Sk, tid);
    if (!(p.causal && key0 > qw0 + 31)) {
      const float* kb = sm + cur * 2 * C::TILE;
      const float* vb = kb + C::TILE;
      f32x16 s, dp;
      zero16(s);
      zero16(dp);
#pragma unroll
      for (int g = 0; g < D / 8; ++g) {
        const f32x4 a = *(const f32x4*)(kb + ln * C::PITCH + 8 * g + 4 * hh);
        const f32x4 a2 = *(const f32x4*)(vb + ln * C::PITCH + 8 * g + 4 * hh);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          s = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], qf[g][e], s, 0, 0, 0);
          dp = __builtin_amdgcn_mfma_f32_32x32x2f32(a2[e], dof[g][e], dp, 0, 0, 0);
        }
      }
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int key = key0 + 8 * (v >> 2) + 4 * hh + (v & 3);
        const float pr = key > lim ? 0.f : fast_exp2(__builtin_fmaf(s[v], c, -l2));
        s[v] = pr * (dp[v] - dl);
      }
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int kl = 8 * (v >> 2) + 4 * hh + (v & 3);
#pragma unroll
        for (int db = 0; db < D / 32; ++db)
          dq[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(kb[kl * C::PITCH + db * 32 + ln], s[v], dq[db], 0, 0, 0);
      }
    }
    if (more) st.lstore(sm + (cur ^ 1) * 2 * C::TILE, sm + (cur ^ 1) * 2 * C::TILE + C::TILE, tid);
    __syncthreads();
  }

  if (qrow < p.Sq) {
    float* dqp = p.dq + b * p.dqs.b + h * p.dqs.h + (int64_t)qrow * p.dqs.s;
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        f32x4* dst = (f32x4*)(dqp + db * 32 + 8 * g + 4 * hh);
        f32x4 x = {0.f, 0.f, 0.f, 0.f};
        if (!p.grads_in_t) x = *dst;
#pragma unroll
        for (int e = 0; e < 4; ++e) x[e] += dq[db][4 * g + e] * p.scale;
        *dst = x;
      }
  }
}

template <int D>
__global__ void __launch_bounds__(BWD_THREADS, 1) flash_bwd32_dkdv_kernel(const BwdParams pk) {
  BwdParams p = pk;  // a variable-length batch rewrites the sizes and bases for its sequence below
  typedef Bwd32Cfg<D> C;
  extern __shared__ __align__(16) unsigned char smem[];
  float* sm = (float*)smem;
  const int tid = threadIdx.x;
  const int lane = tid & 63, w = tid >> 6, ln = lane & 31, hh = lane >> 5;

  int bid = blockIdx.x;
  const int bh = bid % (p.B * p.H);  // (batch, head) pairs first: each keeps to one XCD also when H < 8
  const int h = bh % p.H;
  int b = bh / p.H;
  const int kt = bid / (p.B * p.H);
  const int k0 = kt * 128;
  const int kw0 = k0 + w * 32;
  select_sequence<float>(p, b);
  if (k0 >= p.Sk || p.Sq <= 0 || (p.causal && k0 >= p.Sq)) {  // no query sees these keys: nothing to add to dk, dv
    if (p.grads_in_t && kw0 + ln < p.Sk) {                     // written gradients of such keys are zero
      zero_grad_row<float, D>(p.dk + b * p.dks.b + h * p.dks.h + (int64_t)(kw0 + ln) * p.dks.s, hh);
      zero_grad_row<float, D>(p.dv + b * p.dvs.b + h * p.dvs.h + (int64_t)(kw0 + ln) * p.dvs.s, hh);
    }
    return;
  }

  const float* qp = (const float*)p.q + b * p.qs.b + h * p.qs.h;
  const float* kp = (const float*)p.k + b * p.ks.b + h * p.ks.h;
  const float* vp = (const float*)p.v + b * p.vs.b + h * p.vs.h;
  const float* dop = (const float*)p.dout + b * p.dos.b + h * p.dos.h;
  const float* lsep = p.lse + ((int64_t)b * p.H + h) * p.lse_bh;
  const float* delp = p.delta + ((int64_t)b * p.H + h) * p.lse_bh;

  const int krow = kw0 + ln;
  const int krow_c = krow < p.Sk ? krow : p.Sk - 1;
  f32x4 kf[D / 8], vf[D / 8];
#pragma unroll
  for (int g = 0; g < D / 8; ++g) {
    kf[g] = *(const f32x4*)(kp + (int64_t)krow_c * p.ks.s + 8 * g + 4 * hh);
    vf[g] = *(const f32x4*)(vp + (int64_t)krow_c * p.vs.s + 8 * g + 4 * hh);
  }
  const float c = p.scale_log2;

  const int it0 = p.causal ? k0 / B32_ROWS : 0;  // earlier query rows see none of these keys
  const int nt = (p.Sq + B32_ROWS - 1) / B32_ROWS;
  constexpr int STAGE = 2 * C::TILE + C::STAT;

  f32x16 dk[D / 32], dv[D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; ++i) {
    zero16(dk[i]);
    zero16(dv[i]);
  }

  PairStage<D> st;
  float st_l = 0.f, st_d = 0.f;
  auto gload = [&](int it) {
    st.gload(qp, p.qs.s, dop, p.dos.s, it * B32_ROWS, p.Sq, tid);
    if (tid < B32_ROWS) {
      int r = it * B32_ROWS + tid;
      r = r < p.Sq ? r : p.Sq - 1;
      st_l = lsep[r] * 1.4426950408889634f;
      st_d = delp[r];
    }
  };
  auto lstore = [&](int stage) {
    float* sb = sm + stage * STAGE;
    st.lstore(sb, sb + C::TILE, tid);
    if (tid < B32_ROWS) {
      sb[2 * C::TILE + tid] = st_l;
      sb[2 * C::TILE + B32_ROWS + tid] = st_d;
    }
  };

  if (it0 < nt) {
    gload(it0);
    lstore(it0 & 1);
  }
  __syncthreads();

  for (int it = it0; it < nt; ++it) {
    const int cur = it & 1;
    const int r0 = it * B32_ROWS;
    const bool more = it + 1 < nt;
    if (more) gload(it + 1);
    if (!(p.causal && r0 + B32_ROWS - 1 < kw0)) {
      const float* qb = sm + cur * STAGE;
      const float* dob = qb + C::TILE;
      const float* stp = dob + C::TILE;
      f32x16 s, dp;
      zero16(s);
      zero16(dp);
#pragma unroll
      for (int g = 0; g < D / 8; ++g) {
        const f32x4 a = *(const f32x4*)(qb + ln * C::PITCH + 8 * g + 4 * hh);
        const f32x4 a2 = *(const f32x4*)(dob + ln * C::PITCH + 8 * g + 4 * hh);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          s = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], kf[g][e], s, 0, 0, 0);
          dp = __builtin_amdgcn_mfma_f32_32x32x2f32(a2[e], vf[g][e], dp, 0, 0, 0);
        }
      }
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int ql = 8 * (v >> 2) + 4 * hh + (v & 3);
        const int qi = r0 + ql;
        const bool dead = qi >= p.Sq || (p.causal && krow > qi);
        const float pr = dead ? 0.f : fast_exp2(__builtin_fmaf(s[v], c, -stp[ql]));
        s[v] = pr;
        dp[v] = pr * (dp[v] - stp[B32_ROWS + ql]);
      }
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int ql = 8 * (v >> 2) + 4 * hh + (v & 3);
#pragma unroll
        for (int db = 0; db < D / 32; ++db) {
          dv[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(dob[ql * C::PITCH + db * 32 + ln], s[v], dv[db], 0, 0, 0);
          dk[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(qb[ql * C::PITCH + db * 32 + ln], dp[v], dk[db], 0, 0, 0);
        }
      }
    }
    if (more) lstore(cur ^ 1);
    __syncthreads();
  }

  if (krow < p.Sk && p.grads_in_t) {
    float* dkp = p.dk + b * p.dks.b + h * p.dks.h + (int64_t)krow * p.dks.s;
    float* dvp = p.dv + b * p.dvs.b + h * p.dvs.h + (int64_t)krow * p.dvs.s;
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        f32x4 x, y;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          x[e] = dk[db][4 * g + e] * p.scale;
          y[e] = dv[db][4 * g + e];
        }
        *(f32x4*)(dkp + db * 32 + 8 * g + 4 * hh) = x;
        *(f32x4*)(dvp + db * 32 + 8 * g + 4 * hh) = y;
      }
  } else if (krow < p.Sk) {
    float* dkp = p.dk + b * p.dks.b + h * p.dks.h + (int64_t)krow * p.dks.s;
    float* dvp = p.dv + b * p.dvs.b + h * p.dvs.h + (int64_t)krow * p.dvs.s;
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        f32x4* d1 = (f32x4*)(dkp + db * 32 + 8 * g + 4 * hh);
        f32x4* d2 = (f32x4*)(dvp + db * 32 + 8 * g + 4 * hh);
        f32x4 x = *d1, y = *d2;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          x[e] += dk[db][4 * g + e] * p.scale;
          y[e] += dv[db][4 * g + e];
        }
        *d1 = x;
        *d2 = y;
      }
  }
}

template <auto kernel>
hipError_t launch(int smem, unsigned blocks, const BwdParams& p, hipStream_t stream, int threads = BWD_THREADS) {
  const hipError_t e = spa_allow_dynamic_lds<kernel>(smem);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(threads), smem, stream, p);
  return hipGetLastError();
}

template <typename T, int D>
hipError_t launch_both(const BwdParams& p, hipStream_t stream) {
  const unsigned kblocks = (unsigned)((int64_t)p.B * p.H * p.nkt);
  // dq kernel: 256-row workgroups (two waves per SIMD, the K/V stream shared by twice the rows) once
  // there are enough of them to occupy every CU; spa_tune() can force 4 or 8 waves (experiments, tests)
  const int nqt8 = (p.Sq + 255) / 256;
  const int forced = spa_knob(SPA_KNOB_BWD_DQ_WAVES);
  hipError_t e = hipErrorInvalidValue;
  bool wide = false;
  if constexpr (D >= 64) {  // a D = 32 tile has fewer 16-byte slots than 512 threads
    wide = forced ? forced == 8 : (int64_t)p.B * p.H * nqt8 >= spa_device_cus();
    if (wide) {
      BwdParams p8 = p;
      p8.nqt = nqt8;
      e = launch<flash_bwd_dq_kernel<T, D, 8>>(DqCfg<D, 8>::SMEM, (unsigned)((int64_t)p.B * p.H * nqt8), p8, stream, 512);
    }
  }
  if (!wide) e = launch<flash_bwd_dq_kernel<T, D, 4>>(DqCfg<D, 4>::SMEM, (unsigned)((int64_t)p.B * p.H * p.nqt), p, stream);
  if (e != hipSuccess) return e;
  if constexpr (D == 128)
    if (spa_knob(SPA_KNOB_BWD_DKDV_FORM) == 1) return launch<flash_bwd_dkdv_kernel<T, D, false>>(DkvCfg<D>::SMEM, kblocks, p, stream);
  return launch<flash_bwd_dkdv_kernel<T, D>>(DkvCfg<D>::SMEM, kblocks, p, stream);
}

// A tensor of 2 GiB or more per (batch, head): the re-based variants, 128-row dq workgroups.
template <typename T, int D>
hipError_t launch_both_big(const BwdParams& p, hipStream_t stream) {
  const hipError_t e = launch<flash_bwd_dq_kernel<T, D, 4, true>>(DqCfg<D, 4>::SMEM, (unsigned)((int64_t)p.B * p.H * p.nqt), p, stream);
  if (e != hipSuccess) return e;
  return launch<flash_bwd_dkdv_kernel<T, D, true, true>>(DkvCfg<D>::SMEM, (unsigned)((int64_t)p.B * p.H * p.nkt), p, stream);
}

}  // namespace

// This file makes two objects: compiled with SPA_BWD_BIG_UNIT it holds the re-based variants of the 16-bit kernels
// and nothing else, without it everything else (so that the two parts compile side by side).
#ifdef SPA_BWD_BIG_UNIT
hipError_t spa_launch_bwd16_big(const BwdParams& p, int D, int dtype, hipStream_t stream) {
  if (dtype == 1) {
    if (D == 128) return launch_both_big<__bf16, 128>(p, stream);
    if (D == 64) return launch_both_big<__bf16, 64>(p, stream);
    if (D == 32) return launch_both_big<__bf16, 32>(p, stream);
  } else if (dtype == 2) {
    if (D == 128) return launch_both_big<_Float16, 128>(p, stream);
    if (D == 64) return launch_both_big<_Float16, 64>(p, stream);
    if (D == 32) return launch_both_big<_Float16, 32>(p, stream);
  }
  return hipErrorInvalidValue;
}
#else
hipError_t spa_launch_bwd16_big(const BwdParams& p, int D, int dtype, hipStream_t stream);

// Returns hipSuccess, or hipErrorInvalidValue for an unsupported (dtype, D).
hipError_t spa_launch_flash_bwd(BwdParams p, int D, int dtype, hipStream_t stream) {
  p.nqt = (p.Sq + 127) / 128;
  p.nkt = (p.Sk + 127) / 128;
  if (p.big && dtype != 0) return spa_launch_bwd16_big(p, D, dtype, stream);
  if (dtype == 1) {
    if (D == 128) return launch_both<__bf16, 128>(p, stream);
    if (D == 64) return launch_both<__bf16, 64>(p, stream);
    if (D == 32) return launch_both<__bf16, 32>(p, stream);
  } else if (dtype == 2) {
    if (D == 128) return launch_both<_Float16, 128>(p, stream);
    if (D == 64) return launch_both<_Float16, 64>(p, stream);
    if (D == 32) return launch_both<_Float16, 32>(p, stream);
  } else if (dtype == 0) {
    const unsigned qblocks = (unsigned)((int64_t)p.B * p.H * p.nqt);
    const unsigned kblocks = (unsigned)((int64_t)p.B * p.H * p.nkt);
    hipError_t e = hipErrorInvalidValue;
    if (D == 128) e = launch<flash_bwd32_dq_kernel<128>>(Bwd32Cfg<128>::SMEM_DQ, qblocks, p, stream);
    if (D == 64) e = launch<flash_bwd32_dq_kernel<64>>(Bwd32Cfg<64>::SMEM_DQ, qblocks, p, stream);
    if (D == 32) e = launch<flash_bwd32_dq_kernel<32>>(Bwd32Cfg<32>::SMEM_DQ, qblocks, p, stream);
    if (e != hipSuccess) return e;
    if (D == 128) return launch<flash_bwd32_dkdv_kernel<128>>(Bwd32Cfg<128>::SMEM_DKV, kblocks, p, stream);
    if (D == 64) return launch<flash_bwd32_dkdv_kernel<64>>(Bwd32Cfg<64>::SMEM_DKV, kblocks, p, stream);
    if (D == 32) return launch<flash_bwd32_dkdv_kernel<32>>(Bwd32Cfg<32>::SMEM_DKV, kblocks, p, stream);
  }
  return hipErrorInvalidValue;
}
#endif  // SPA_BWD_BIG_UNIT
