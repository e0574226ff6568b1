// Block flash-attention forward for gfx950: out = softmax(q k^T * scale + mask) v and
// fp32 lse = logsumexp(q k^T * scale + mask), for one (q chunk, kv chunk) pair or for a whole
// ring schedule of kv chunks per launch.
// Stands in for intel_flash_attn_forward (sp_aurora/intel_flash_attn.py:18-126) /
// intel_flash_attn_forward_optimized (sp_aurora/intel_flash_attn_optimized.py:95-225) and, with
// the schedule, for the step loop around it (sp_aurora/intel_ring_flash_attn.py:72-148):
// one Q.K^T instead of the reference's two, scores never leave the CU.
//
// Work decomposition (16-bit kernel)
//   workgroup = 128 query rows of one (batch, head, rank); a wave owns 32 of them.
//   Both contractions are computed TRANSPOSED on v_mfma_f32_32x32x16:
//     S^T[key][qrow] = K[key][:] . Q[qrow][:]      A = K tile (LDS), B = Q (registers)
//     O^T[d][qrow]  += V^T[d][key] . P^T[key][qrow] A = V^T tile (LDS), B = P^T (registers)
//   In the 32x32 accumulator layout a lane owns ONE query row (column lane%32)
//   and 16 of the 32 block rows, so the row max / row sum of the softmax is a
//   per-lane reduction plus one exchange with lane^32, the rescale of O is a
//   per-lane scalar, and the S^T accumulators are, register for register,
//   the B operand of the second contraction: P never touches LDS.
//
//   K and V sub-tiles (64 keys) travel from global memory straight into LDS (buffer loads
//   with the LDS bit), rows back to back with their 16-byte chunks XOR-permuted against bank
//   conflicts.  K operands are 16-byte LDS reads; V stays row-major in LDS and is transposed
//   by the read (ds_read_b64_tr_b16), two reads per operand.
//
//   Two wave groups (8 waves, two per SIMD) share the query rows and take alternate
//   64-key sub-tiles; each group streams its own sub-tiles through its own
//   double-buffered LDS.  A wave's loop is software-pipelined into two phases,
//       VALU phase:  softmax of S(i) -> P(i);  wait for the loads issued one phase ago
//       MFMA phase:  O += V(i)^T P(i);  S(i+1) = K(i+1) Q^T;  loads of V(i+1), K(i+2) in between
//   separated by workgroup barriers, and group 1 runs one barrier behind group 0, so at
//   any time one wave of a SIMD is in its MFMA phase while its neighbour is in its VALU
//   phase (ping-pong).  The groups' partial (O, m, l) are combined through LDS at the end.
#include <type_traits>

#include "spa_common.h"
#include "spa_host.h"

namespace {

constexpr int FWD_BM = 128;  // query rows per workgroup
// Keys per LDS sub-tile (one VALU phase + one MFMA phase of a wave).  The kernel is written for 64 or
// 128.  128-key sub-tiles for D = 64 (whose phases hold half the MFMA work against the same softmax
// work) were measured 5-8 % slower than 64-key ones on every shape tried, long rows included:
// fewer barriers do not pay for the coarser ping-pong and the 247-register VALU phase.
template <int D>
constexpr int fwd_bn() { return 64; }
constexpr int FWD_THREADS = 256;  // threads of one wave group (4 waves x 32 query rows)
constexpr int FWD_LOOK = 8;       // MFMA operands are fetched from LDS this many MFMAs ahead

// SHARE = false: the NG wave groups work on the same 128 query rows and take alternate sub-tiles,
// each through LDS buffers of its own.  SHARE = true (NG = 2): the groups work on different query
// rows (256 per workgroup), every group takes every sub-tile, and all 8 waves fill one set of
// buffers together: half the global -> LDS traffic per FLOP and half as many workgroups.
template <int D, int NG, bool SHARE>
struct Fwd16Cfg {
  static constexpr int BN = fwd_bn<D>();       // keys per sub-tile
  static constexpr int NT = BN / 32;           // 32-key score tiles per sub-tile
  static constexpr int ROWB = D * 2;           // bytes per K / V row in LDS: no padding, the tiles are swizzled
  static constexpr int TILEB = BN * ROWB;      // one K or V sub-tile
  static constexpr int GROUP = 4 * TILEB;      // one set of K[2] and V[2] buffers
  static constexpr int BMW = SHARE ? NG * FWD_BM : FWD_BM;  // query rows per workgroup
  static constexpr int EPI = (NG * FWD_BM * (D + 4) + NG * FWD_BM * 2 + BMW) * 4;  // epilogue staging
  static constexpr int TILES = SHARE ? GROUP : NG * GROUP;
  static constexpr int SMEM = TILES > EPI ? TILES : EPI;
  static constexpr int CPR = D / 8;                         // 16-byte chunks per row
  static constexpr int DTHREADS = SHARE ? NG * FWD_THREADS : FWD_THREADS;  // threads filling one buffer
  static constexpr int NDMA = TILEB / (DTHREADS * 16);      // direct loads per thread and sub-tile
  static constexpr int RPD = DTHREADS / CPR;                // rows one round of loads covers
  static_assert(!SHARE || (NG == 2 && NDMA >= 1), "shared buffers: two groups, at least one load per thread");
};

// A sub-tile lives in LDS as its rows back to back, each row's 16-byte chunks permuted by an XOR
// with a function of the row, so that the reads of one instruction spread over all banks:
// K is read 16 bytes per lane by 16 consecutive rows at one chunk index; V is read by the
// transposing 8-byte read, a half wave covering 4 rows x 64 bytes.
template <int D>
__device__ __forceinline__ int k_swizzle(int row) {
  constexpr int CPR = D / 8;
  return (row / (16 / CPR)) % CPR;
}
template <int D>
__device__ __forceinline__ int v_swizzle(int row) {
  return D == 128 ? (row & 3) << 2 : D == 64 ? ((row >> 1) & 1) << 2 : 0;
}

// KV8: K and V hold OCP e4m3 bytes (K = k8 * k_scale[b,h], V = v8 * v_scale[b,h]).  The tiles travel
// global -> registers -> LDS and are widened to T on the way (every e4m3 value is exact in bf16 and
// fp16), once per workgroup, so LDS holds the same swizzled 16-bit tiles as without KV8 and both
// contractions run unchanged; k_scale folds into the softmax scale, v_scale into the final 1 / l.
// (With shared buffers every thread of the workgroup stages its share of a tile and writes it before
// the barrier at which the direct loads of the 16-bit form are waited for.)
// FINALN: the variant for a rank's last ring step (epilogue SPA_EPI_FINALN); the others write a
// block result as it is (SPA_EPI_PLAIN / SPA_EPI_PART).
// ZZ: the variant for zigzag shards (FwdParams::zigzag); the others carry none of its bookkeeping.
// BIG: the variant for K / V whose rows of one (batch, head) span 2 GiB or more: the buffer descriptors are
// re-based per sub-tile (a few scalar instructions per tile that the others do without).
// QK8 (with KV8, D = 128): q is e4m3 as well (Q = q8 * q_scale[b,h]) and S^T = K Q^T runs on the 8-bit matrix
// instruction (v_mfma_f32_32x32x64_f8f6f4, twice the rate of the 16-bit one; products of two e4m3 values are exact
// in fp32): K tiles stay bytes in LDS (direct loads again, half the size), Q fragments are 32 bytes per lane and
// 64-deep step; V is widened to T as with KV8 and P V stays a 16-bit contraction.
// WAIT: the variant for a ring rank whose chunks arrive while its launch runs (FwdParams::arrive): a bounded wait for
// a chunk's flag before the chunk's first tile is loaded.
// KS: the variant that splits the KEYS of a call with few query rows over grid.z (FwdParams::sk_last): "rank" z takes
// chunk z of the keys for the SAME query rows and writes its block result to rows z * Sq .. of (out, lse), which the
// launcher points at a scratch tensor; a second kernel merges the z results.
// VR: the variant for a ring over a packed variable-length batch (FwdParams::chunk_rows, rank_rows): chunks and ranks
// lie a shard apart, not a sequence length apart.
template <typename T, int D, int NG, bool SHARE, bool KV8 = false, bool FINALN = false, bool ZZ = false, bool BIG = false,
          bool QK8 = false, bool WAIT = false, bool KS = false, bool VR = false>
__global__ void __launch_bounds__(FWD_THREADS * NG, 1) flash_fwd16_kernel(const FwdParams pk) {
  static_assert(!(FINALN && SHARE), "the merging epilogue goes with 128-row workgroups");
  static_assert(!KS || (!SHARE && !FINALN && !ZZ && !BIG && !QK8 && !WAIT), "split keys: 128-row workgroups, plain results");
  static_assert(!QK8 || (KV8 && D == 128 && !ZZ && !BIG), "8-bit scores: e4m3 q, k, v, head dim 128, contiguous chunks");
  typedef typename std::conditional<KV8, unsigned char, T>::type KVT;  // element type of K / V in memory
  typedef typename std::conditional<QK8, unsigned char, T>::type QT;   // element type of q in memory
  constexpr bool KSTAGE = KV8 && !QK8;  // K tiles go through registers (widened on the way); V tiles do whenever KV8
  typedef Fwd16Cfg<D, NG, SHARE> C;
  FwdParams p = pk;  // a variable-length batch rewrites the sizes and bases for its sequence below
  typedef Mma16<T> M;
  typedef typename M::frag frag;
  extern __shared__ __align__(16) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int w = wave & 3;     // which 32 query rows
  const int grp = wave >> 2;  // wave group: which key sub-tiles (or, with shared buffers, which 128 query rows)
  const int tg = SHARE ? tid : tid & (FWD_THREADS - 1);  // thread index among those filling one buffer
  const int ln = lane & 31;
  const int hh = lane >> 5;

  // Consecutive workgroup ids walk the (batch, head) pairs first: with round-robin placement of
  // workgroups on the 8 XCDs, all query tiles of a head share one XCD's L2 for K/V.
  // Then query tiles and ranks, heaviest first.
  // (grid.x = (batch, head) pairs, grid.y = query tiles, grid.z = ranks: workgroups are dispatched
  // x first, and the decomposition costs no divisions)
  const int bh = blockIdx.x;  // (batch, head) pairs first: each keeps to one XCD also when H < 8
  const int h = bh % p.H;
  int b = bh / p.H;
  // dequantisation scales of this (batch or sequence, head): K = k8 * ksc, V = v8 * vsc
  const float ksc = KV8 ? p.k_scale[bh] * (QK8 ? p.q_scale[bh] : 1.f) : 1.f;  // (with e4m3 q its scale rides along)
  const float vsc = KV8 ? p.v_scale[bh] : 1.f;
  const int qt = p.nqt - 1 - (int)blockIdx.y;
  // Zigzag shards: the tiles of the two halves of the chunk are laid out one half after the other (a tile
  // never holds rows of both), the second (heavier) half first in dispatch order.
  constexpr bool zz = ZZ;
  const int zz_hs = p.Sq >> 1;                                    // rows per half-chunk
  const int zz_nqh = p.zz_half ? p.nqt : p.nqt >> 1;              // tiles per half
  const bool zhalf = zz && (p.zz_half || qt >= zz_nqh);           // this workgroup's rows lie in the second half
  const int q0 = zz ? (zhalf ? zz_hs : 0) + (qt - (zhalf && !p.zz_half ? zz_nqh : 0)) * C::BMW : qt * C::BMW;
  // Ranks heaviest first: the last rank with contiguous chunks.  With zigzag shards the second half of a shard's
  // rows is heavier the lower the rank and the first half the higher, and every grid plane z holds the same work.
  const int rank = zz && zhalf ? p.rank0 + (int)blockIdx.z : p.rank0 + p.nranks - 1 - (int)blockIdx.z;
  // WAIT: the flag of the first chunk is requested before anything else (such a load takes microseconds; it is looked
  // at when the first tiles are about to be requested)
  auto flag_of = [&](int ch) { return __hip_atomic_load(p.arrive + ch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM); };
  int ahead_ch = -1;   // the chunk whose flag was fetched ahead of time, and what it read
  unsigned ahead = 0;
  if constexpr (WAIT) {
    ahead_ch = rank - p.t_begin;
    ahead_ch = ahead_ch < 0 ? ahead_ch + p.P : ahead_ch;
    ahead = flag_of(ahead_ch);
  }
  if (p.cu_q) {
    const int q_lo = p.cu_q[b], k_lo = p.cu_k[b];
    p.Sq = p.cu_q[b + 1] - q_lo;
    p.Sk = p.cu_k[b + 1] - k_lo;
    p.q = (const QT*)p.q + (int64_t)q_lo * p.qs.s;
    p.k = (const KVT*)p.k + (int64_t)k_lo * p.ks.s;
    p.v = (const KVT*)p.v + (int64_t)k_lo * p.vs.s;
    p.out = (T*)p.out + (int64_t)q_lo * p.os.s;
    p.lse += q_lo;
    b = 0;
    if (q0 >= p.Sq) return;  // this sequence is shorter than the longest one
    if (p.Sk <= 0) {
      // no keys: the empty sum, out = 0 and lse = -inf
      for (int idx = tid; idx < C::BMW * (D / 8); idx += FWD_THREADS * NG) {
        const int grow = q0 + idx / (D / 8), ch = idx % (D / 8);
        if (grow >= p.Sq) break;
        u32x4 z = {0u, 0u, 0u, 0u};
        *(u32x4*)((T*)p.out + h * p.os.h + (int64_t)grow * p.os.s + ch * 8) = z;
        if (ch == 0) p.lse[(int64_t)h * p.lse_bh + grow] = -INFINITY;
      }
      return;
    }
  }
  const int q_lim = zz && !zhalf ? zz_hs : p.Sq;  // one past the last row this workgroup may own
  const int qw0 = q0 + (SHARE ? grp * FWD_BM : 0) + w * 32;
  const int64_t qoff = (int64_t)rank * (VR ? p.rank_rows : p.Sq);  // first row of this rank's query chunk
  const int crow = VR ? p.chunk_rows : p.Sk;                         // rows from one K / V chunk to the next

  const QT* qp = (const QT*)p.q + b * p.qs.b + h * p.qs.h + (KS ? 0 : qoff * p.qs.s);  // (KS: every chunk of keys meets the same rows)
  const KVT* kp = (const KVT*)p.k + b * p.ks.b + h * p.ks.h;
  const KVT* vp = (const KVT*)p.v + b * p.vs.b + h * p.vs.h;

  const int qrow = qw0 + ln;
  const int qrow_c = qrow < q_lim ? qrow : q_lim - 1;

  frag qf[QK8 ? 1 : D / 16];
  i32x8 qf8[QK8 ? D / 64 : 1];  // QK8: 32 bytes per lane and 64-deep contraction step (bytes 32 hh .. 32 hh + 31 of the step)
  const unsigned qsign = p.negq ? (QK8 ? 0x80808080u : 0x80008000u) : 0u;  // negative softmax scale: -q with |scale|
  if constexpr (QK8) {
#pragma unroll
    for (int kk = 0; kk < D / 64; ++kk) {
      const u32x4 x0 = *(const u32x4*)(qp + (int64_t)qrow_c * p.qs.s + kk * 64 + hh * 32);
      const u32x4 x1 = *(const u32x4*)(qp + (int64_t)qrow_c * p.qs.s + kk * 64 + hh * 32 + 16);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        qf8[kk][i] = (int)(x0[i] ^ qsign);
        qf8[kk][4 + i] = (int)(x1[i] ^ qsign);
      }
    }
  } else {
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) {
      u32x4 x = *(const u32x4*)(qp + (int64_t)qrow_c * p.qs.s + ks * 16 + hh * 8);
      x[0] ^= qsign; x[1] ^= qsign; x[2] ^= qsign; x[3] ^= qsign;
      qf[ks] = as_frag<frag>(x);
    }
  }

  // ---- the schedule of this workgroup ----
  // K/V hold P chunks of Sk keys.  Ring step t of rank r uses chunk (r - t) mod P; a causal ring
  // has steps 0..r and masks step 0 (the rank's own chunk) only.  The launch covers steps
  // [t_begin, t_end) of that schedule; a plain block call is P = 1, one step.
  // A group's work is a sequence of 64-key sub-tiles: first those of the masked (diagonal)
  // chunk up to the last key any row of the workgroup sees, then every full chunk.
  constexpr int BN = C::BN, NT = C::NT;
  constexpr int TILE = SHARE ? BN : BN * NG;  // keys between two sub-tiles of one group
  constexpr int KSTEP = SHARE ? 1 : NG;
  // A zigzag ring has P steps for the second half of a chunk's rows and steps 0..r for the first half;
  // steps 1..r use the first half of their chunk's keys (zz_last_half: the last such step, -1 without zigzag).
  const int nsteps = p.causal ? (zhalf ? p.P : rank + 1 < p.P ? rank + 1 : p.P) : p.P;
  const int t_end = p.t_count < 0 || p.t_begin + p.t_count > nsteps ? nsteps : p.t_begin + p.t_count;
  const bool diag = p.causal && p.t_begin == 0;
  const int kv_end = q0 + C::BMW < p.Sk ? q0 + C::BMW : p.Sk;  // keys of the diagonal chunk in use
  const int n_diag = diag ? (kv_end + TILE - 1) / TILE : 0;
  // (KS: one step, the rank's own chunk; the last chunk of the keys may be shorter than the others)
  const int ks_klen = KS && rank == p.P - 1 ? p.sk_last : p.Sk;
  const int npc = ((KS ? ks_klen : p.Sk) + TILE - 1) / TILE;   // sub-tiles per full chunk
  const int zz_last_half = zz ? rank : -1;
  const int klen_h = zz ? zz_hs : p.Sk;                        // keys of a half step
  const int npc_h = (klen_h + TILE - 1) / TILE;                // sub-tiles of a half step
  const int t_full0 = p.t_begin + (diag ? 1 : 0);              // first unmasked step
  const int t_half_end = t_end < zz_last_half + 1 ? t_end : zz_last_half + 1;  // unmasked steps before this one are half steps
  const int n_hsteps = t_half_end > t_full0 ? t_half_end - t_full0 : 0;
  const int n_fsteps = t_end - t_full0 - n_hsteps > 0 ? t_end - t_full0 - n_hsteps : 0;
  const int n = n_diag + n_hsteps * npc_h + n_fsteps * npc;
  if constexpr (FINALN && ZZ) {
    if (n == 0) {
      // The launch of a zigzag rank's last step, first half of the rows: no block here (their last block was
      // step `rank`), so the workgroup only applies update_out_and_lse (sp_aurora/utils.py:103-104) to the
      // slots of steps 0 .. rank, in that order, and writes the rows' final (out, lse).
      typedef Mma16<T> MM;
      constexpr float LOG2E = 1.4426950408889634f;
      const int nslot = rank + 1 < p.npart ? rank + 1 : p.npart;
      const RingSlots slots(p.B, p.H, p.Sq, D);
      const int64_t slot_rs = (int64_t)p.H * D;  // a slot is contiguous [B, Sq, H, D]
      const int64_t slot_bh = (int64_t)b * p.Sq * slot_rs + h * D;
      const int64_t qoff0 = (int64_t)rank * p.Sq;
      T* const out0 = (T*)p.out + b * p.os.b + h * p.os.h + qoff0 * p.os.s;
      float* const lse0 = p.lse + ((int64_t)b * p.H + h) * p.lse_bh + qoff0;
      for (int idx = tid; idx < C::BMW * (D / 8); idx += FWD_THREADS * NG) {
        const int grow = q0 + idx / (D / 8), ch = idx % (D / 8);
        if (grow >= q_lim) break;
        float x[8], lb = -INFINITY, wsum = 0.f;
#pragma unroll
        for (int k2 = 0; k2 < 8; ++k2) x[k2] = 0.f;
        for (int j = 0; j < nslot; ++j) {
          const u32x4 raw = *(const u32x4*)(slots.template out<T>(p.part, j) + slot_bh + (int64_t)grow * slot_rs + ch * 8);
          const float lj = (slots.lse(p.part, p.P, j) + ((int64_t)b * p.H + h) * p.Sq)[grow];
          const float mx = fmaxf(lb, lj);  // slot 0, the diagonal block, is finite in every row
          const float wa = fast_exp2((lb - mx) * LOG2E), wb = fast_exp2((lj - mx) * LOG2E);
          wsum = wsum * wa + wb;
          lb = mx;
#pragma unroll
          for (int k2 = 0; k2 < 4; ++k2) {
            float lo, hi;
            MM::unpack2(raw[k2], lo, hi);
            x[2 * k2] = x[2 * k2] * wa + lo * wb;
            x[2 * k2 + 1] = x[2 * k2 + 1] * wa + hi * wb;
          }
        }
        const float inv = 1.f / wsum;
        u32x4 st;
#pragma unroll
        for (int k2 = 0; k2 < 4; ++k2) st[k2] = MM::pack2(x[2 * k2] * inv, x[2 * k2 + 1] * inv);
        *(u32x4*)(out0 + (int64_t)grow * p.os.s + ch * 8) = st;
        if (ch == 0) lse0[grow] = lb + fast_log2(wsum) * 0.6931471805599453f;
      }
      return;
    }
  }

  struct Sub {
    int krel;   // first key of the sub-tile, relative to its chunk
    int krow;   // the same as a row of the K/V tensors
    int kend;   // one past the chunk's last row
    int klen;   // keys of the chunk this step may use (half a chunk in some steps of a zigzag ring)
    int ch;     // the chunk's number (read by the WAIT variants only)
    bool masked;
  };
  // The loop walks the sub-tiles in order with three cursors (softmax at i, V loads at i+1,
  // K loads at i+2); a cursor steps without divisions.
  struct Cursor {
    int i, j, t;
    Sub sb;
  };
  auto cursor_next = [&](Cursor& c) {
    ++c.i;
    ++c.j;
    if (c.i == n_diag) {
      c.j = 0;
      c.t = t_full0;
    } else if (c.i > n_diag && c.j == (c.t <= zz_last_half ? npc_h : npc)) {
      c.j = 0;
      ++c.t;
    }
    int ch = rank - c.t;
    ch = ch < 0 ? ch + p.P : ch;
    ch = ch < 0 ? 0 : ch;  // only past the end of the schedule, where nothing is used
    c.sb.masked = c.i < n_diag;
    c.sb.ch = ch;
    c.sb.klen = KS ? ks_klen : c.i >= n_diag && c.t <= zz_last_half ? klen_h : p.Sk;
    c.sb.krel = (c.j * KSTEP + (SHARE ? 0 : grp)) * BN;
    c.sb.krow = ch * crow + c.sb.krel;
    c.sb.kend = ch * crow + p.Sk;
  };
  // ---- global -> LDS: direct loads, no registers in between ----
  // Thread tg of the group owns slot tg of every round of 256 16-byte slots; round j of a
  // sub-tile covers rows j * RPD + tg / CPR.  LDS slot (row, pos) receives the row's chunk
  // pos ^ swizzle(row), so the permutation happens on the global side, in the lane's offset.
  // Buffer loads: a wave-uniform descriptor per tensor and a 32-bit byte offset per lane (a lane
  // constant plus the sub-tile's uniform row offset), and the hardware's range check instead of
  // clamps and branches: a row past the end of the tensor arrives as zeros, a row past the end of
  // its chunk but inside the tensor is the next chunk's data; both are keys >= Sk, which the
  // softmax masks to P = 0.  The whole offset travels in the per-lane register: a scalar offset is taken off the
  // range before the comparison (a lane is out of range when voffset >= num_records - soffset, unsigned), which
  // is only safe while soffset <= num_records; carrying the tile's row offset there instead (one vector add per
  // load less, all of them outside the MFMA phase) was measured: bit-identical results, +-1 %.
  // A load that is not wanted (past the end of the schedule) gets an offset beyond
  // any tensor and stores zeros into a buffer nobody reads.
  constexpr unsigned OFF_NONE = 0x80000000u;
  const int drow = tg / C::CPR, dpos = tg % C::CPR;
  // QK8: a K row is D bytes = D / 16 slots; rows 2 r, 2 r + 1 share a permutation (16 consecutive rows at one
  // slot index then hit 16 different bank groups); NK direct loads per thread fill a sub-tile
  constexpr int CPR8 = D / 16, ROWB8 = D;
  constexpr int NK = QK8 ? (C::BN * ROWB8) / (C::DTHREADS * 16) : C::NDMA;
  constexpr int RPD_K = QK8 ? C::DTHREADS / CPR8 : C::RPD;
  static_assert(NK >= 1, "a K sub-tile must give every thread a load");
  auto k8_swizzle = [](int row) { return (row >> 1) & (CPR8 - 1); };
  const unsigned kdoff = QK8 ? (unsigned)((tg / CPR8) * p.ks.s + (((tg % CPR8) ^ k8_swizzle(tg / CPR8)) * 16))
                             : (unsigned)((drow * p.ks.s + ((dpos ^ k_swizzle<D>(drow)) * 8)) * (int64_t)sizeof(KVT));
  const unsigned vdoff = (unsigned)((drow * p.vs.s + ((dpos ^ v_swizzle<D>(drow)) * 8)) * (int64_t)sizeof(KVT));
  const unsigned krow_b = (unsigned)(p.ks.s * (int64_t)sizeof(KVT));  // bytes per K row
  const unsigned vrow_b = (unsigned)(p.vs.s * (int64_t)sizeof(KVT));
  const int64_t rows_all = KS ? (int64_t)(p.P - 1) * p.Sk + p.sk_last : (int64_t)(p.P - 1) * crow + p.Sk;
  const unsigned long long kbytes = (unsigned long long)(((rows_all - 1) * p.ks.s + D) * (int64_t)sizeof(KVT));
  const unsigned long long vbytes = (unsigned long long)(((rows_all - 1) * p.vs.s + D) * (int64_t)sizeof(KVT));
  static_assert(!(BIG && KV8), "the re-based variants are built for 16-bit K / V");
  const u32x4 krsrc = buffer_descriptor(kp, BIG ? 0u : (unsigned)kbytes);  // (BIG: an empty range, for loads that are not wanted)
  const u32x4 vrsrc = buffer_descriptor(vp, BIG ? 0u : (unsigned)vbytes);
  // LDS byte addresses of this group's buffers and of this wave's 1 KB share of a round
  const unsigned lds_group = (unsigned)(uintptr_t)(lds_u8*)smem + (SHARE ? 0 : grp * C::GROUP);
  const unsigned lds_wave = lds_group + (SHARE ? wave : w) * 1024;
  auto k_lds = [&](int i) { return (unsigned)((i & 1) * C::TILEB); };                  // relative to lds_group
  auto v_lds = [&](int i) { return (unsigned)(2 * C::TILEB + (i & 1) * C::TILEB); };
  // load number q of the pair (K sub-tile with first row k_row into buffer kb, V sub-tile v_row into vb)
  constexpr int NLOADS = NK + C::NDMA;
  // the same two descriptors as compiler-visible resources, for loads into registers
  const __amdgpu_buffer_rsrc_t krs = __builtin_amdgcn_make_buffer_rsrc((void*)kp, 0, (int)krsrc[2], 0x00020000);
  const __amdgpu_buffer_rsrc_t vrs = __builtin_amdgcn_make_buffer_rsrc((void*)vp, 0, (int)vrsrc[2], 0x00020000);
  // KV8: a thread's 8 e4m3 bytes per slot wait in registers from the MFMA phase that loads them to
  // the next VALU phase, which widens them and writes the 16-byte LDS slot (store_staged).
  u32x2 stage[KV8 ? NLOADS : 1];
  // (k_end / v_end: one past the chunk's last row; the WAIT variants give lanes beyond it the offset of a load that
  // is not wanted, so that no byte of a chunk whose flag has not been seen is requested - a row past the end of a
  // chunk is the next chunk's first - and no cache can hold a line of the receive buffer from before its arrival)
  // Split keys, 16-bit K/V, D = 128: a chunk's tiles are read by the one workgroup of their (batch, head) when the rows fit a
  // tile, so they carry the non-temporal hint (3-9 % on five decode shapes; slower for e4m3 K/V and D = 64).
  constexpr bool KS_NT = KS && !KV8 && D == 128;
  auto load_one = [&](int q, bool kon, int k_row, unsigned kb, bool von, int v_row, unsigned vb, int k_end = 0x7fffffff,
                      int v_end = 0x7fffffff) {
    if constexpr (WAIT) {
      // the descriptor's range ends with the chunk (a scalar per load instead of a compare per lane): what lies past
      // it arrives as zeros like everything past the tensor
      if (q < NK) {
        const unsigned u = kon ? (unsigned)(k_row + q * RPD_K) * krow_b : OFF_NONE;
        const unsigned end = (unsigned)k_end * krow_b;
        const unsigned lim = end < krsrc[2] ? end : krsrc[2];
        if constexpr (KSTAGE) {
          stage[q] = __builtin_bit_cast(
              u32x2, __builtin_amdgcn_raw_buffer_load_b64(__builtin_amdgcn_make_buffer_rsrc((void*)kp, 0, (int)lim, 0x00020000), kdoff + u, 0, 0));
        } else {
          u32x4 rs = krsrc;
          rs[2] = lim;
          load_to_lds_b128(rs, kdoff + u, lds_wave + kb + q * (C::DTHREADS * 16));
        }
      } else {
        const int r = q - NK;
        const unsigned u = von ? (unsigned)(v_row + r * C::RPD) * vrow_b : OFF_NONE;
        const unsigned end = (unsigned)v_end * vrow_b;
        const unsigned lim = end < vrsrc[2] ? end : vrsrc[2];
        if constexpr (KV8) {
          stage[q] = __builtin_bit_cast(
              u32x2, __builtin_amdgcn_raw_buffer_load_b64(__builtin_amdgcn_make_buffer_rsrc((void*)vp, 0, (int)lim, 0x00020000), vdoff + u, 0, 0));
        } else {
          u32x4 rs = vrsrc;
          rs[2] = lim;
          load_to_lds_b128(rs, vdoff + u, lds_wave + vb + r * (C::DTHREADS * 16));
        }
      }
      return;
    }
    if (q < NK) {
      if constexpr (BIG) {
        // the sub-tile's first row as a 64-bit byte offset -> window descriptor + offset inside it
        unsigned rel = OFF_NONE;
        u32x4 rs = krsrc;
        if (kon) rs = buffer_window(kp, kbytes, (unsigned long long)(unsigned)k_row * krow_b, rel);
        load_to_lds_b128(rs, kdoff + rel + (unsigned)(q * C::RPD) * krow_b, lds_wave + kb + q * (C::DTHREADS * 16));
        return;
      }
      const unsigned u = kon ? (unsigned)(k_row + q * RPD_K) * krow_b : OFF_NONE;
      if constexpr (KSTAGE)
        stage[q] = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(krs, kdoff + u, 0, 0));
      else if constexpr (KS_NT)
        load_to_lds_b128_nt(krsrc, kdoff + u, lds_wave + kb + q * (C::DTHREADS * 16));
      else
        load_to_lds_b128(krsrc, kdoff + u, lds_wave + kb + q * (C::DTHREADS * 16));
    } else {
      const int r = q - NK;
      if constexpr (BIG) {
        unsigned rel = OFF_NONE;
        u32x4 rs = vrsrc;
        if (von) rs = buffer_window(vp, vbytes, (unsigned long long)(unsigned)v_row * vrow_b, rel);
        load_to_lds_b128(rs, vdoff + rel + (unsigned)(r * C::RPD) * vrow_b, lds_wave + vb + r * (C::DTHREADS * 16));
        return;
      }
      const unsigned u = von ? (unsigned)(v_row + r * C::RPD) * vrow_b : OFF_NONE;
      if constexpr (KV8)
        stage[q] = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(vrs, vdoff + u, 0, 0));
      else if constexpr (KS_NT)
        load_to_lds_b128_nt(vrsrc, vdoff + u, lds_wave + vb + r * (C::DTHREADS * 16));
      else
        load_to_lds_b128(vrsrc, vdoff + u, lds_wave + vb + r * (C::DTHREADS * 16));
    }
  };
  // 8 e4m3 bytes -> 8 elements of T, 16 bytes
  auto widen = [&](u32x2 x) {
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      if constexpr (std::is_same<T, __bf16>::value) {
        r[2 * i] = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(x[i], 1.0f, false));
        r[2 * i + 1] = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(x[i], 1.0f, true));
      } else {
        r[2 * i] = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(x[i], 1.0f, false));
        r[2 * i + 1] = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(x[i], 1.0f, true));
      }
    }
    return r;
  };
  // the staged K sub-tile goes to the K buffer at kb, the staged V sub-tile to the V buffer at vb
  // (slot of thread tg in round q: the 16 bytes the direct load would have written)
  auto store_staged = [&](unsigned kb, unsigned vb) {
    if constexpr (KV8) {
      const unsigned slot = lds_group + (unsigned)tg * 16;
#pragma unroll
      for (int q = KSTAGE ? 0 : NK; q < NLOADS; ++q) {
        const unsigned a = slot + (q < NK ? kb + q * (C::DTHREADS * 16) : vb + (q - NK) * (C::DTHREADS * 16));
        *(__attribute__((address_space(3))) u32x4*)(lds_u8*)(uintptr_t)a = widen(stage[q]);
      }
    }
  };
  auto loads_landed = [&]() { __builtin_amdgcn_s_waitcnt(0x0F70); };  // vmcnt(0)

  // ---- LDS -> MFMA operands ----
  // K (A operand of S^T = K Q^T): lane (key = ln, half hh) reads chunk 2 ks + hh of its row.
  // V (A operand of O^T += V^T P^T): the transposing read hands lane (dim, hh) four consecutive
  // keys of one head dim; in a block of 16 lanes, lane 4 e + c supplies the address of 8 bytes
  // (4 dims) of key e, and lane x receives dim x of keys 0..3.
  // (QK8: the operand of step kk is bytes 64 kk + 32 hh .. + 31 of the key's row: two 16-byte reads, kra[2 kk], kra[2 kk + 1])
  constexpr int NKA = QK8 ? 2 * (D / 64) : D / 16;  // 16-byte K reads per lane and 32-key tile
  unsigned kra[NKA], vra[D / 32];
  if constexpr (QK8) {
#pragma unroll
    for (int u = 0; u < 2 * (D / 64); ++u)
      kra[u] = lds_group + ln * ROWB8 + ((((u >> 1) * 4 + 2 * hh + (u & 1)) ^ k8_swizzle(ln)) * 16);
  } else {
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) kra[ks] = lds_group + ln * C::ROWB + (((2 * ks + hh) ^ k_swizzle<D>(ln)) * 16);
  }
  {
    const int blk = lane >> 4, e = (lane >> 2) & 3, c4 = lane & 3;
    const int krl = 4 * hh + e;
#pragma unroll
    for (int db = 0; db < D / 32; ++db) {
      const int chunk = db * 4 + (blk & 1) * 2 + (c4 >> 1);
      vra[db] = lds_group + krl * C::ROWB + ((chunk ^ v_swizzle<D>(krl)) * 16) + (c4 & 1) * 8;
    }
  }

  f32x16 s[NT];
  f32x16 o[D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[i][v] = 0.f;
  float m_run = -INFINITY;  // reference row max of the raw scores (may lag the true max, see below)
  float l_run = 0.f;        // this lane's share of the running row sum
  const float c = p.scale_log2 * ksc;  // scores are q . k8: the scale of K rides on the softmax scale

  // per-lane LDS addresses of the operands of MFMA phase i: V(i) and K(i+1); computed before the
  // barrier that opens the phase
  auto operand_addresses = [&](int i, unsigned (&va)[D / 32], unsigned (&ka)[NKA]) {
    const unsigned vb = v_lds(i), kb = k_lds(i + 1);
#pragma unroll
    for (int db = 0; db < D / 32; ++db) va[db] = vra[db] + vb;
#pragma unroll
    for (int ks = 0; ks < NKA; ++ks) ka[ks] = kra[ks] + kb;
  };

  // MFMA phase of step i: O += V(i)^T P(i) (if PV) followed by S(i+1) = K(i+1) Q^T (if NS).
  // The LDS operand of MFMA number j is fetched LOOK MFMAs ahead of its use, so the whole
  // phase runs off a rolling window of LOOK fragments instead of stalling on every read.
  auto mfma_phase = [&](auto do_pv, auto do_s, const unsigned (&va)[D / 32], const unsigned (&ka)[NKA], frag (&pfr)[NT][2], auto&& side) {
    constexpr bool PV = decltype(do_pv)::value, NS = decltype(do_s)::value;
    constexpr int NPV = PV ? (D / 32) * (BN / 16) : 0;
    constexpr int NSS = NS ? NKA * NT : 0;  // 16-byte K reads: one per 16-bit MFMA, two per 8-bit one
    constexpr int TOTAL = NPV + NSS;
    constexpr int LOOK = KV8 && D == 64 ? FWD_LOOK - 2 : FWD_LOOK;  // (the staged e4m3 bytes take the registers of two fragments)
    auto fetch = [&](int j) -> frag {
      if (j < NPV) {  // j = (t*2+u)*(D/32) + db : consecutive MFMAs hit different accumulators
        const int db = j % (D / 32), tu = j / (D / 32);
        const lds_u8* a = (const lds_u8*)(uintptr_t)va[db] + tu * 16 * C::ROWB;
        const u32x2 r0 = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)a));
        const u32x2 r1 = __builtin_bit_cast(
            u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a + 8 * C::ROWB)));
        u32x4 x;
        x[0] = r0[0];
        x[1] = r0[1];
        x[2] = r1[0];
        x[3] = r1[1];
        return as_frag<frag>(x);
      }
      const int jj = j - NPV;  // jj = ks*NT + t;  QK8: jj = (kk*NT + t)*2 + which half of the 32 bytes
      if constexpr (QK8) {
        const int half = jj & 1, t = (jj >> 1) % NT, kk = (jj >> 1) / NT;
        return as_frag<frag>(*(const __attribute__((address_space(3))) u32x4*)((const lds_u8*)(uintptr_t)ka[2 * kk + half] + t * 32 * ROWB8));
      }
      const int t = jj % NT, ks = jj / NT;
      return as_frag<frag>(*(const __attribute__((address_space(3))) u32x4*)((const lds_u8*)(uintptr_t)ka[ks] + t * 32 * C::ROWB));
    };
    frag win[LOOK];
#pragma unroll
    for (int j = 0; j < LOOK && j < TOTAL; ++j) win[j] = fetch(j);
    // scheduling fences keep the compiler from sinking each read back next to its use
    __builtin_amdgcn_sched_barrier(0);
    frag klo;  // QK8: the first half of an 8-bit operand waits here for the second
#pragma unroll
    for (int j = 0; j < TOTAL; ++j) {
      const frag a = win[j % LOOK];
      if (j + LOOK < TOTAL) win[j % LOOK] = fetch(j + LOOK);
      __builtin_amdgcn_sched_barrier(0);
      if (j < NPV) {
        const int db = j % (D / 32), tu = j / (D / 32);
        o[db] = M::run(a, pfr[tu >> 1][tu & 1], o[db]);
      } else if constexpr (QK8) {
        const int jj = j - NPV;
        const int half = jj & 1, t = (jj >> 1) % NT, kk = (jj >> 1) / NT;
        if (half == 0) {
          klo = a;
        } else {
          const u32x4 x0 = __builtin_bit_cast(u32x4, klo), x1 = __builtin_bit_cast(u32x4, a);
          i32x8 ka8;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            ka8[i] = (int)x0[i];
            ka8[4 + i] = (int)x1[i];
          }
          f32x16 acc;
          if (kk == 0) {
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[v] = 0.f;
          } else {
            acc = s[t];
          }
          s[t] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ka8, qf8[kk], acc, 0, 0, 0, 0, 0, 0);  // e4m3 x e4m3, unscaled
        }
      } else {
        const int jj = j - NPV;
        const int t = jj % NT, ks = jj / NT;
        if (ks == 0) {
          f32x16 z;
#pragma unroll
          for (int v = 0; v < 16; ++v) z[v] = 0.f;
          s[t] = M::run(a, qf[0], z);
        } else {
          s[t] = M::run(a, qf[ks], s[t]);
        }
      }
      side(j);
    }
  };

  // VALU phase of step i: softmax of S(i) -> P(i) as MFMA operands, O rescaled if needed.
  auto softmax_phase = [&](const Sub& sb, frag (&pfr)[NT][2]) {
    const int key0 = sb.krel;
    const bool causal_here = sb.masked;
    const bool need_mask = (causal_here && key0 + BN - 1 > qw0) || (key0 + BN > sb.klen);
    if (need_mask) {
      const int lim = causal_here ? (qrow < sb.klen - 1 ? qrow : sb.klen - 1) : sb.klen - 1;  // last visible key
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int key = key0 + t * 32 + 8 * (v >> 2) + 4 * hh + (v & 3);
          if (key > lim) s[t][v] = -INFINITY;
        }
    }

    // row max of the lane's 32 NT scores: 3-input maxima, two independent chains per 32-key tile.
    // (Through the instruction itself: fmaxf() makes the compiler quiet possible signalling NaNs
    // first, one extra instruction per MFMA result; the scores are finite or -inf here.)
    auto max3 = [](float a, float b, float c3) {
      float r;
      asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c3));
      return r;
    };
    float mxa[NT], mxb[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      mxa[t] = max3(s[t][0], s[t][1], s[t][2]);
      mxb[t] = max3(s[t][8], s[t][9], s[t][10]);
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      mxa[t] = max3(mxa[t], s[t][3], s[t][4]);
      mxb[t] = max3(mxb[t], s[t][11], s[t][12]);
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      mxa[t] = max3(mxa[t], s[t][5], s[t][6]);
      mxb[t] = max3(mxb[t], s[t][13], s[t][14]);
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) mxa[t] = max3(mxa[t], s[t][7], mxb[t]);
    float mx;
    if constexpr (NT == 2) {
      mx = max3(mxa[0], mxa[1], fmaxf(s[0][15], s[1][15]));
    } else {
      static_assert(NT == 4, "sub-tiles of 64 or 128 keys");
      const float u = max3(mxa[0], mxa[1], s[0][15]), w2 = max3(mxa[2], mxa[3], s[1][15]);
      mx = max3(u, w2, fmaxf(s[2][15], s[3][15]));
    }
    mx = halves_max(mx);
    // Lazy rescale: the reference max only moves when some row's max grew by more than
    // 2^8 in the exp2 domain; until then P <= 256, harmless in fp32 sums and bf16 operands.
    if (__builtin_amdgcn_ballot_w64((mx - m_run) * c > 8.f) != 0) {
      const float m_new = fmaxf(m_run, mx);
      // (a lane whose row has seen no key yet, here or before, while another row of the wave asks for the
      // rescale: -inf - -inf; nothing of that row needs scaling.  Rows of a wave differ in this only when
      // the tile's first row is not a multiple of the sub-tile size: the second half of a zigzag shard.)
      const float alpha = ZZ && m_new == -INFINITY ? 1.f : fast_exp2((m_run - m_new) * c);
      m_run = m_new;
      l_run *= alpha;
#pragma unroll
      for (int d = 0; d < D / 32; ++d)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[d][v] *= alpha;
    }
    // a row that has seen no key yet (a ragged chunk can leave a whole sub-tile empty) keeps m = -inf
    const float mc = m_run == -INFINITY ? 0.f : m_run * c;

    float ps[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const float e = fast_exp2(__builtin_fmaf(s[t][v], c, -mc));
        s[t][v] = e;
        ps[v & 3] += e;
      }
    l_run += (ps[0] + ps[1]) + (ps[2] + ps[3]);
    asm volatile("" : "+v"(l_run));  // keep the row sum in this phase as well (see below)

#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int u = 0; u < 2; ++u)
        pfr[t][u] = M::pack(s[t][8 * u + 0], s[t][8 * u + 1], s[t][8 * u + 2], s[t][8 * u + 3],
                            s[t][8 * u + 4], s[t][8 * u + 5], s[t][8 * u + 6], s[t][8 * u + 7]);
    // P must exist in registers when the phase ends: without this the compiler sinks the
    // exponentials past the barrier into the MFMA phase they are meant to overlap with.
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        u32x4 x = __builtin_bit_cast(u32x4, pfr[t][u]);
        asm volatile("" : "+v"(x));
        pfr[t][u] = __builtin_bit_cast(frag, x);
      }
  };

  // ---- prologue: K(0), V(0), K(1) on their way into LDS together with Q into registers ----
  // The three cursors of the loop (softmax at i, V loads at i + 1, K loads at i + 2) start at
  // sub-tiles 0, 1, 2; the first loads take their rows from them (no divisions).
  Cursor cs, cv, ck;
  cs.i = 0;
  cs.j = 0;
  cs.t = n_diag > 0 ? 0 : t_full0;
  {
    int ch = rank - cs.t;
    ch = ch < 0 ? ch + p.P : ch;
    cs.sb.masked = n_diag > 0;
    cs.sb.ch = ch;
    cs.sb.klen = KS ? ks_klen : n_diag == 0 && cs.t <= zz_last_half ? klen_h : p.Sk;
    cs.sb.krel = (SHARE ? 0 : grp) * BN;
    cs.sb.krow = ch * crow + cs.sb.krel;
    cs.sb.kend = ch * crow + p.Sk;
  }
  cv = cs;
  cursor_next(cv);
  ck = cv;
  cursor_next(ck);
  // WAIT: no tile of a chunk is requested before the chunk's arrival flag has been seen (each wave polls for itself;
  // the acquire at system scope also drops cache lines that could hold the buffer's earlier contents).
  // The flag is read with a relaxed load at system scope (it bypasses the caches; nothing is invalidated: K/V lines can
  // not be stale, see load_one).  Such a load takes microseconds, so the flag of the chunk that follows in ring order
  // is fetched when a chunk is entered and looked at a chunk later; only a flag that was not up yet is polled.
  auto wait_chunk = [&](int ch) {
    if constexpr (WAIT) {
      unsigned seen = ch == ahead_ch ? ahead : flag_of(ch);
      unsigned spins = 0;
      while (__builtin_amdgcn_readfirstlane(seen) < p.epoch) {
        if (++spins >= p.spin_limit) {  // the bound every wave reaches: note the failure and go on
          if (lane == 0) __hip_atomic_store(p.fault, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
          break;
        }
        __builtin_amdgcn_s_sleep(8);
        seen = flag_of(ch);
      }
      ahead_ch = ch > 0 ? ch - 1 : p.P - 1;
      ahead = flag_of(ahead_ch);
    }
  };
  if constexpr (WAIT) {
    if (0 < n) wait_chunk(cs.sb.ch);
    if (1 < n && cv.sb.ch != cs.sb.ch) wait_chunk(cv.sb.ch);
    if (2 < n && ck.sb.ch != cv.sb.ch) wait_chunk(ck.sb.ch);
  }
#pragma unroll
  for (int q = 0; q < NK; ++q) load_one(q, 0 < n, cs.sb.krow, k_lds(0), false, 0, 0, cs.sb.kend, 0);     // K(0)
#pragma unroll
  for (int q = 0; q < C::NDMA; ++q) load_one(NK + q, false, 0, 0, 0 < n, cs.sb.krow, v_lds(0), 0, cs.sb.kend);  // V(0)
  if constexpr (KSTAGE) {
    // K(0) goes to LDS now; V(0) stays staged together with K(1), loaded next, and both are written
    // by the first VALU phase like every later pair
#pragma unroll
    for (int q = 0; q < NK; ++q)
      *(__attribute__((address_space(3))) u32x4*)(lds_u8*)(uintptr_t)(lds_group + (unsigned)tg * 16 + k_lds(0) + q * (C::DTHREADS * 16)) = widen(stage[q]);
  }
#pragma unroll
  for (int q = 0; q < NK; ++q) load_one(q, 1 < n, cv.sb.krow, k_lds(1), false, 0, 0, cv.sb.kend, 0);     // K(1)
  // S(0) needs Q and K(0) only: loads complete in the order of issue, so at most the loads of V(0)
  // and K(1) may still be in flight here; they are waited for before the barrier that
  // opens the first MFMA phase reading them.
  __builtin_amdgcn_s_waitcnt(0x0F70 | ((NK + C::NDMA) & 15) | (((NK + C::NDMA) >> 4) << 14));  // vmcnt(loads of V(0), K(1))
  __syncthreads();
  {
    frag none[NT][2];
    unsigned va[D / 32], ka[NKA];
    operand_addresses(-1, va, ka);
    mfma_phase(std::false_type{}, std::true_type{}, va, ka, none, [](int) {});  // S(0)
  }
  __syncthreads();
  if (NG > 1 && grp == 1) {  // group 1 runs one phase behind group 0
    loads_landed();          // (with shared buffers group 0 reads this group's share of V(0), K(1) after this barrier)
    if constexpr (SHARE) store_staged(k_lds(1), v_lds(0));
    __syncthreads();
  }

  // One loop, no branch around an MFMA, the same barriers per step for every wave of a group.  A wave
  // whose rows see none of a diagonal sub-tile's keys (at most the last two sub-tiles of the
  // diagonal chunk) simply gets P = 0 from the mask.
  // MFMA phase i reads V(i) and K(i+1); the other two buffers are free then and receive V(i+1)
  // and K(i+2), which must have landed when the next VALU phase ends.
  // With shared buffers both groups load their share of the same two sub-tiles in the same
  // phase of the workgroup: group 0 during its MFMA phase, group 1 (one phase behind) at the start
  // of its VALU phase; each waits for its loads before the barrier two phases later.
  const bool early = SHARE && grp == 1;  // wave-uniform
  // The loop body comes in two copies, one per buffer parity of the step, so that every LDS address of
  // the MFMA phase is a per-lane constant plus an immediate offset (no address arithmetic per step).
  auto body = [&](auto parity, int i) __attribute__((always_inline)) {
    constexpr int PAR = decltype(parity)::value;  // == i & 1
    frag pf[NT][2];
    const bool kon = ck.i < n, von = cv.i < n;
    constexpr unsigned kb = (unsigned)(PAR * C::TILEB), vb = (unsigned)(2 * C::TILEB + (PAR ^ 1) * C::TILEB);  // k_lds(i), v_lds(i + 1)
    if (early) {
#pragma unroll
      for (int q = 0; q < NLOADS; ++q) load_one(q, kon, ck.sb.krow, kb, von, cv.sb.krow, vb, ck.sb.kend, cv.sb.kend);
    }
    softmax_phase(cs.sb, pf);
    unsigned va[D / 32], ka[NKA];
#pragma unroll
    for (int db = 0; db < D / 32; ++db) va[db] = vra[db] + (unsigned)(2 * C::TILEB + PAR * C::TILEB);  // v_lds(i)
#pragma unroll
    for (int ks = 0; ks < NKA; ++ks) ka[ks] = kra[ks] + (unsigned)((PAR ^ 1) * C::TILEB);               // k_lds(i + 1)
    // Shared buffers need one barrier per step and group (after the wait for the loads: group 0
    // at the end of its VALU phase, group 1 at the end of its MFMA phase, the same physical
    // barrier); the other one only holds the two groups in step, and they drift little without it.
    if (!early) {
      loads_landed();
      store_staged((unsigned)((PAR ^ 1) * C::TILEB), (unsigned)(2 * C::TILEB + PAR * C::TILEB));  // K(i + 1), V(i)
    }
    if constexpr (WAIT) {
      // the MFMA phase below requests K of sub-tile i + 2 (V of the same sub-tile follows one step later): its chunk's
      // first tile?  (Here, where every load has landed anyway: looking at the flag fetched ahead waits for no other load.)
      if (kon && ck.j == 0) wait_chunk(ck.sb.ch);
    }
    if (!SHARE || !early) __syncthreads();
    __builtin_amdgcn_s_setprio(3);
    mfma_phase(std::true_type{}, std::true_type{}, va, ka, pf, [&](int j) {
      constexpr int TOTAL = (D / 32) * (BN / 16) + NKA * NT;
#pragma unroll
      for (int q = 0; q < NLOADS; ++q)
        if ((q * TOTAL + TOTAL / 2) / NLOADS == j && !early) load_one(q, kon, ck.sb.krow, kb, von, cv.sb.krow, vb, ck.sb.kend, cv.sb.kend);
    });
    __builtin_amdgcn_s_setprio(0);
    cursor_next(cs);
    cursor_next(cv);
    cursor_next(ck);
    if (early) {
      loads_landed();
      store_staged(kb, vb);  // this group's share of K(i + 2), V(i + 1), loaded at the top of the step
    }
    if (!SHARE || early) __syncthreads();
  };
  {
    int i = 0;
    for (; i + 2 < n; i += 2) {
      body(std::integral_constant<int, 0>{}, i);
      body(std::integral_constant<int, 1>{}, i + 1);
    }
    if (i + 1 < n) body(std::integral_constant<int, 0>{}, i);
  }
  {  // last sub-tile: nothing to prepare behind it
    frag pf[NT][2];
    softmax_phase(cs.sb, pf);
    unsigned va[D / 32], ka[NKA];
    operand_addresses(n - 1, va, ka);
    loads_landed();
    if (!early) store_staged(k_lds(n), v_lds(n - 1));  // V(n - 1) (and whatever K(n) stands for: never read)
    if (!SHARE || !early) __syncthreads();
    mfma_phase(std::true_type{}, std::false_type{}, va, ka, pf, [](int) {});
    if (!SHARE || early) __syncthreads();
  }
  if (NG > 1 && grp == 0) __syncthreads();  // matches group 1's leading barrier

  // ---- epilogue ----
  // The groups exchange only (m, l) per row; each scales its own partial O by
  // exp2((m - m_all) c) / l_all and stages it as fp32 rows in LDS (free now); then all
  // waves walk the 128 x D tile row-major, add the groups' partials and write full rows:
  // 16-byte coalesced stores instead of 8-byte pieces scattered over 32 rows per wave.
  // A rank's last ring step (the FINALN variants) merges the earlier steps' results, which lie in the
  // slots of p.part, in the same pass.  A step that is not the rank's last needs nothing of its own:
  // the host points out / lse and their strides at the step's slot (in q's element type, as the
  // reference keeps a block's output: sp_aurora/intel_ring_flash_attn.py:96-108).
  T* const out_bh = (T*)p.out + b * p.os.b + h * p.os.h + qoff * p.os.s;
  const int64_t out_rs = p.os.s;
  float* const lse_bh = p.lse + ((int64_t)b * p.H + h) * p.lse_bh + qoff;
  // Rows leave straight from the registers wherever nothing is merged into them (every variant but a rank's
  // last ring step).  A lane holds 4 consecutive head dims per register group and its partner 32 lanes on the
  // next 4; one v_permlane32_swap per dword pairs them up so that every lane stores 16-byte pieces, the two
  // lanes of a row side by side.  `other`: the same rows' partial sums of the other wave group, staged in LDS
  // in the accumulator's own layout (128 rows of D + 4 floats), or null.
  auto store_rows = [&](float a_own, auto with_other, const float* other, float a_other, float lse_val) {
    constexpr bool OTHER = decltype(with_other)::value;
    if (hh == 0 && qrow < q_lim) lse_bh[qrow] = lse_val;
    T* const orow = out_bh + qrow_c * out_rs;
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
      for (int gp = 0; gp < 2; ++gp) {
        float e[8];  // this lane's 4 dims of the even and of the odd register group
#pragma unroll
        for (int i = 0; i < 8; ++i) e[i] = o[db][8 * gp + i] * a_own;
        if constexpr (OTHER) {
          const f32x4 p0 = *(const f32x4*)(other + db * 32 + 8 * (2 * gp) + 4 * hh);
          const f32x4 p1 = *(const f32x4*)(other + db * 32 + 8 * (2 * gp + 1) + 4 * hh);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            e[i] = __builtin_fmaf(p0[i], a_other, e[i]);
            e[4 + i] = __builtin_fmaf(p1[i], a_other, e[4 + i]);
          }
        }
        unsigned x[2], y[2];  // as two packed pairs each
#pragma unroll
        for (int k = 0; k < 2; ++k) {
          x[k] = M::pack2(e[2 * k], e[2 * k + 1]);
          y[k] = M::pack2(e[4 + 2 * k], e[4 + 2 * k + 1]);
        }
        u32x4 st;
#pragma unroll
        for (int k = 0; k < 2; ++k) {
          const auto r = __builtin_amdgcn_permlane32_swap(x[k], y[k], false, false);
          st[k] = r[0];      // lanes 0-31: own dims 0-3 of the even group; lanes 32-63: partner's dims 0-3 of the odd group
          st[2 + k] = r[1];  // lanes 0-31: partner's dims 4-7 of the even group; lanes 32-63: own dims 4-7 of the odd group
        }
        if (qrow < q_lim) *(u32x4*)(orow + db * 32 + 8 * (2 * gp + hh)) = st;
      }
  };
  if constexpr (SHARE || (NG == 1 && !FINALN)) {
    // a wave's rows are complete: no LDS round trip, no barrier
    const float l_tot = halves_sum(l_run);
    store_rows(vsc / l_tot, std::false_type{}, nullptr, 0.f, (m_run * c + fast_log2(l_tot)) * 0.6931471805599453f);
    return;
  } else if constexpr (!FINALN) {
    // Two groups hold partial sums of the same rows.  Group 1 stages its unscaled partial O (fp32, its own
    // register layout) and (m, l) in LDS, free now, and leaves; group 0 weighs both by exp2((m - m_all) c) / l_all
    // and stores the rows from its registers.  One barrier, one staged tile.
    constexpr int TP = D + 4;  // floats per staged row
    float* const tile = (float*)smem;
    float* const ml = tile + FWD_BM * TP;  // [128](m, l) of group 1
    const int rloc = w * 32 + ln;
    const float l_own = halves_sum(l_run);
    if (grp == 1) {
#pragma unroll
      for (int db = 0; db < D / 32; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          f32x4 st;
          st[0] = o[db][4 * g + 0];
          st[1] = o[db][4 * g + 1];
          st[2] = o[db][4 * g + 2];
          st[3] = o[db][4 * g + 3];
          *(f32x4*)(tile + rloc * TP + db * 32 + 8 * g + 4 * hh) = st;
        }
      if (hh == 0) {
        ml[rloc * 2] = m_run;
        ml[rloc * 2 + 1] = l_own;
      }
    }
    __syncthreads();
    if (grp == 1) return;
    const float m2 = ml[rloc * 2], l2 = ml[rloc * 2 + 1];
    const float m_all = fmaxf(m_run, m2);  // finite: some group has seen key 0 of the first chunk
    const float a1 = fast_exp2((m_run - m_all) * c);
    const float a2 = fast_exp2((m2 - m_all) * c);
    const float l_all = l_own * a1 + l2 * a2;
    const float sc = vsc / l_all;
    store_rows(a1 * sc, std::true_type{}, tile + rloc * TP, a2 * sc, (m_all * c + fast_log2(l_all)) * 0.6931471805599453f);
    return;
  } else {
    constexpr int TP = D + 4;  // floats per staged row
    float* const tile = (float*)smem + grp * (FWD_BM * TP);
    float* const ml = (float*)smem + NG * FWD_BM * TP;  // [NG][128](m, l), then lse_b[rows of the workgroup]
    float* const lsb = ml + NG * FWD_BM * 2;
    const int rloc = w * 32 + ln;
    // The final pass walks the tile row-major, a thread owning 8 head dims of NIT rows; the CH lanes of
    // a row share a wave.
    constexpr int CH = D / 8;                                   // 8-element chunks per row
    constexpr int NIT = C::BMW * CH / (FWD_THREADS * NG);       // chunks per thread
    static_assert(NIT * FWD_THREADS * NG == C::BMW * CH, "the final pass must tile the workgroup's rows");
    int crow[NIT], cch[NIT];
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int cidx = tid + it * (FWD_THREADS * NG);
      crow[it] = cidx / CH;
      cch[it] = cidx % CH;
    }
    // The rank's last step fetches the first slots NOW, so that their latency passes under the
    // exchange and the staging below; NB slots are in flight at a time.
    constexpr int NB = 2;
    void* const part = FINALN ? p.part : nullptr;
    const int npart = FINALN ? p.npart : 0;
    const RingSlots slots(p.B, p.H, p.Sq, D);
    const int64_t slot_rs = (int64_t)p.H * D;  // a slot is contiguous [B, Sq, H, D]
    const int64_t slot_bh = (int64_t)b * p.Sq * slot_rs + h * D;
    u32x4 raw[NB][NIT];
    float rl[NB][NIT];
    auto fetch_slots = [&](int j0) {
#pragma unroll
      for (int jj = 0; jj < NB; ++jj)
        if (j0 + jj < npart) {
          const T* so = slots.template out<T>(part, j0 + jj) + slot_bh;
          const float* sl = slots.lse(part, p.P, j0 + jj) + ((int64_t)b * p.H + h) * p.Sq;
#pragma unroll
          for (int it = 0; it < NIT; ++it) {
            const int grow = q0 + crow[it];
            if (grow < q_lim) {
              raw[jj][it] = *(const u32x4*)(so + (int64_t)grow * slot_rs + cch[it] * 8);
              rl[jj][it] = sl[grow];
            }
          }
        }
    };
    if constexpr (FINALN) fetch_slots(0);
    const float l_own = halves_sum(l_run);
    float scale, lse_b;
    if (NG > 1) {
      if (hh == 0) {
        ml[(grp * FWD_BM + rloc) * 2] = m_run;
        ml[(grp * FWD_BM + rloc) * 2 + 1] = l_own;
      }
      __syncthreads();
      const float m2 = ml[((grp ^ 1) * FWD_BM + rloc) * 2];
      const float l2 = ml[((grp ^ 1) * FWD_BM + rloc) * 2 + 1];
      const float m_all = fmaxf(m_run, m2);  // finite: some group has seen key 0 of the first chunk
      const float a1 = fast_exp2((m_run - m_all) * c);
      const float a2 = fast_exp2((m2 - m_all) * c);
      const float l_all = l_own * a1 + l2 * a2;
      scale = a1 * vsc / l_all;
      lse_b = (m_all * c + fast_log2(l_all)) * 0.6931471805599453f;
    } else {
      scale = vsc / l_own;
      lse_b = (m_run * c + fast_log2(l_own)) * 0.6931471805599453f;
    }
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        f32x4 st;
        st[0] = o[db][4 * g + 0] * scale;
        st[1] = o[db][4 * g + 1] * scale;
        st[2] = o[db][4 * g + 2] * scale;
        st[3] = o[db][4 * g + 3] * scale;
        *(f32x4*)(tile + rloc * TP + db * 32 + 8 * g + 4 * hh) = st;
      }
    if (grp == 0 && hh == 0) lsb[rloc] = lse_b;
    __syncthreads();
    const float* t0 = (const float*)smem;
    float x[NIT][8], lb[NIT];
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int row = crow[it], ch = cch[it];
      const f32x4 a = *(const f32x4*)(t0 + row * TP + ch * 8);
      const f32x4 bq = *(const f32x4*)(t0 + row * TP + ch * 8 + 4);
      x[it][0] = a[0]; x[it][1] = a[1]; x[it][2] = a[2]; x[it][3] = a[3];
      x[it][4] = bq[0]; x[it][5] = bq[1]; x[it][6] = bq[2]; x[it][7] = bq[3];
      if (NG > 1) {
        const float* t1 = t0 + FWD_BM * TP;
        const f32x4 a2 = *(const f32x4*)(t1 + row * TP + ch * 8);
        const f32x4 b2 = *(const f32x4*)(t1 + row * TP + ch * 8 + 4);
        x[it][0] += a2[0]; x[it][1] += a2[1]; x[it][2] += a2[2]; x[it][3] += a2[3];
        x[it][4] += b2[0]; x[it][5] += b2[1]; x[it][6] += b2[2]; x[it][7] += b2[3];
      }
      lb[it] = lsb[row];
    }
    if constexpr (FINALN) {
      // update_out_and_lse over all of the rank's steps at once (sp_aurora/utils.py:103-104 applied
      // npart times): out = sum_j e^(lse_j - L) out_j, L = log sum_j e^(lse_j), carried as a running
      // (weighted sum, weight sum) relative to the largest lse so far, starting from this step's block.
      constexpr float LOG2E = 1.4426950408889634f;
      float wsum[NIT];
#pragma unroll
      for (int it = 0; it < NIT; ++it) wsum[it] = 1.f;
      for (int j0 = 0; j0 < npart; j0 += NB) {
        u32x4 cur[NB][NIT];
        float cul[NB][NIT];
#pragma unroll
        for (int jj = 0; jj < NB; ++jj)
#pragma unroll
          for (int it = 0; it < NIT; ++it) {
            cur[jj][it] = raw[jj][it];
            cul[jj][it] = rl[jj][it];
          }
        fetch_slots(j0 + NB);
#pragma unroll
        for (int jj = 0; jj < NB; ++jj)
          if (j0 + jj < npart) {
#pragma unroll
            for (int it = 0; it < NIT; ++it) {
              const float lj = cul[jj][it];
              const float mx = fmaxf(lb[it], lj);  // lb is finite: the last step's block hides no key of a row
              const float wa = fast_exp2((lb[it] - mx) * LOG2E);
              const float wb = fast_exp2((lj - mx) * LOG2E);
              wsum[it] = wsum[it] * wa + wb;
              lb[it] = mx;
#pragma unroll
              for (int k = 0; k < 4; ++k) {
                float lo, hi;
                M::unpack2(cur[jj][it][k], lo, hi);
                x[it][2 * k] = x[it][2 * k] * wa + lo * wb;
                x[it][2 * k + 1] = x[it][2 * k + 1] * wa + hi * wb;
              }
            }
          }
      }
#pragma unroll
      for (int it = 0; it < NIT; ++it) {
        const float inv = 1.f / wsum[it];
#pragma unroll
        for (int k = 0; k < 8; ++k) x[it][k] *= inv;
        lb[it] += fast_log2(wsum[it]) * 0.6931471805599453f;
      }
    }
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int grow = q0 + crow[it];
      if (grow >= q_lim) continue;
      u32x4 st;
      st[0] = M::pack2(x[it][0], x[it][1]);
      st[1] = M::pack2(x[it][2], x[it][3]);
      st[2] = M::pack2(x[it][4], x[it][5]);
      st[3] = M::pack2(x[it][6], x[it][7]);
      *(u32x4*)(out_bh + (int64_t)grow * out_rs + cch[it] * 8) = st;
      if (cch[it] == 0) lse_bh[grow] = lb[it];
    }
  }
}

// ---------------------------------------------------------------------------------
// fp32 kernel: same transposed formulation on v_mfma_f32_32x32x2_f32 (full fp32
// products and accumulation, P stays fp32).  Correctness path for fp32 inputs; the
// contraction-index freedom makes V usable row-major, so nothing is transposed.
// ---------------------------------------------------------------------------------
constexpr int F32_BN = 32;  // keys per LDS tile

template <int D>
struct Fwd32Cfg {
  static constexpr int PITCH = D + 4;  // floats per LDS row (+4: bank spread for 16-byte reads)
  static constexpr int TILE = F32_BN * PITCH;  // floats per K or V tile
  static constexpr int SMEM = 2 * 2 * TILE * 4;
  static constexpr int CPR = D / 4;             // 16-byte chunks per row
  static constexpr int RPP = FWD_THREADS / CPR;  // rows fetched per pass
  static constexpr int PASS = (F32_BN + RPP - 1) / RPP;
};

template <int D>
__global__ void __launch_bounds__(FWD_THREADS, 1) flash_fwd32_kernel(const FwdParams pk) {
  typedef Fwd32Cfg<D> C;
  FwdParams p = pk;  // a variable-length batch rewrites the sizes and bases for its sequence below
  extern __shared__ __align__(16) unsigned char smem[];
  float* sm = (float*)smem;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int w = tid >> 6;
  const int ln = lane & 31;
  const int hh = lane >> 5;

  const int h = blockIdx.x % p.H;
  int b = blockIdx.x / p.H;
  const int qt = p.nqt - 1 - (int)blockIdx.y;
  const int q0 = qt * FWD_BM;
  const int qw0 = q0 + w * 32;
  if (p.cu_q) {
    const int q_lo = p.cu_q[b], k_lo = p.cu_k[b];
    p.Sq = p.cu_q[b + 1] - q_lo;
    p.Sk = p.cu_k[b + 1] - k_lo;
    p.q = (const float*)p.q + (int64_t)q_lo * p.qs.s;
    p.k = (const float*)p.k + (int64_t)k_lo * p.ks.s;
    p.v = (const float*)p.v + (int64_t)k_lo * p.vs.s;
    p.out = (float*)p.out + (int64_t)q_lo * p.os.s;
    p.lse += q_lo;
    b = 0;
    if (q0 >= p.Sq) return;
    if (p.Sk <= 0) {
      for (int idx = tid; idx < FWD_BM * (D / 4); idx += FWD_THREADS) {
        const int grow = q0 + idx / (D / 4), ch = idx % (D / 4);
        if (grow >= p.Sq) break;
        f32x4 z = {0.f, 0.f, 0.f, 0.f};
        *(f32x4*)((float*)p.out + h * p.os.h + (int64_t)grow * p.os.s + ch * 4) = z;
        if (ch == 0) p.lse[(int64_t)h * p.lse_bh + grow] = -INFINITY;
      }
      return;
    }
  }

  const float* qp = (const float*)p.q + b * p.qs.b + h * p.qs.h;
  const float* kp = (const float*)p.k + b * p.ks.b + h * p.ks.h;
  const float* vp = (const float*)p.v + b * p.vs.b + h * p.vs.h;

  const int qrow = qw0 + ln;
  const int qrow_c = qrow < p.Sq ? qrow : p.Sq - 1;

  // Contraction step u (0..D/2-1) of the first product uses head dim
  // 8*(u/4) + 4*hh + (u%4): a lane's dims come as 16-byte groups.
  f32x4 qf[D / 8];
#pragma unroll
  for (int g = 0; g < D / 8; ++g) {
    qf[g] = *(const f32x4*)(qp + (int64_t)qrow_c * p.qs.s + 8 * g + 4 * hh);
    if (p.negq) qf[g] = -qf[g];  // negative softmax scale: -q with |scale|
  }

  const int kv_end = p.causal ? (q0 + FWD_BM < p.Sk ? q0 + FWD_BM : p.Sk) : p.Sk;
  const int nt = (kv_end + F32_BN - 1) / F32_BN;

  const int cc = tid % C::CPR;
  const int cr = tid / C::CPR;
  f32x4 kreg[C::PASS], vreg[C::PASS];

  auto gload = [&](int it) {
    const int key0 = it * F32_BN;
#pragma unroll
    for (int i = 0; i < C::PASS; ++i) {
      const int lr = cr + i * C::RPP;
      if (lr < F32_BN) {
        int r = key0 + lr;
        r = r < p.Sk ? r : p.Sk - 1;
        kreg[i] = *(const f32x4*)(kp + (int64_t)r * p.ks.s + cc * 4);
        vreg[i] = *(const f32x4*)(vp + (int64_t)r * p.vs.s + cc * 4);
      }
    }
  };
  auto lstore = [&](int stage) {
    float* kb = sm + stage * 2 * C::TILE;
    float* vb = kb + C::TILE;
#pragma unroll
    for (int i = 0; i < C::PASS; ++i) {
      const int lr = cr + i * C::RPP;
      if (lr < F32_BN) {
        *(f32x4*)(kb + lr * C::PITCH + cc * 4) = kreg[i];
        *(f32x4*)(vb + lr * C::PITCH + cc * 4) = vreg[i];
      }
    }
  };

  f32x16 o[D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[i][v] = 0.f;
  float m_run = -INFINITY;
  float l_run = 0.f;

  gload(0);
  lstore(0);
  __syncthreads();

  const float c = p.scale_log2;

  for (int it = 0; it < nt; ++it) {
    const int cur = it & 1;
    const int key0 = it * F32_BN;
    const bool more = it + 1 < nt;
    if (more) gload(it + 1);

    const bool active = !(p.causal && key0 > qw0 + 31);
    if (active) {
      const float* kb = sm + cur * 2 * C::TILE;
      const float* vb = kb + C::TILE;

      f32x16 s;
#pragma unroll
      for (int v = 0; v < 16; ++v) s[v] = 0.f;
#pragma unroll
      for (int g = 0; g < D / 8; ++g) {
        const f32x4 a = *(const f32x4*)(kb + ln * C::PITCH + 8 * g + 4 * hh);
#pragma unroll
        for (int e = 0; e < 4; ++e)
          s = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], qf[g][e], s, 0, 0, 0);
      }

      const bool need_mask = (p.causal && key0 + F32_BN - 1 > qw0) || (key0 + F32_BN > p.Sk);
      if (need_mask) {
        const int lim = p.causal ? (qrow < p.Sk - 1 ? qrow : p.Sk - 1) : p.Sk - 1;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int key = key0 + 8 * (v >> 2) + 4 * hh + (v & 3);
          if (key > lim) s[v] = -INFINITY;
        }
      }

      float mx = s[0];
#pragma unroll
      for (int v = 1; v < 16; ++v) mx = fmaxf(mx, s[v]);
      mx = halves_max(mx);
      const float m_new = fmaxf(m_run, mx);
      const float alpha = fast_exp2((m_run - m_new) * c);
      const float mc = m_new * c;
      m_run = m_new;

      float ps = 0.f;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const float e = fast_exp2(__builtin_fmaf(s[v], c, -mc));
        s[v] = e;
        ps += e;
      }
      l_run = l_run * alpha + ps;

#pragma unroll
      for (int i = 0; i < D / 32; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[i][v] *= alpha;

      // Contraction step v of the second product is the key that accumulator
      // register v holds for this lane: 8*(v/4) + 4*hh + (v%4).
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int kl = 8 * (v >> 2) + 4 * hh + (v & 3);
#pragma unroll
        for (int db = 0; db < D / 32; ++db) {
          const float a = vb[kl * C::PITCH + db * 32 + ln];
          o[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, s[v], o[db], 0, 0, 0);
        }
      }
    }

    if (more) lstore(cur ^ 1);
    __syncthreads();
  }

  const float l_tot = halves_sum(l_run);
  const float inv = 1.f / l_tot;
  if (qrow < p.Sq) {
    float* op = (float*)p.out + b * p.os.b + h * p.os.h + (int64_t)qrow * p.os.s;
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        f32x4 st;
        st[0] = o[db][4 * g + 0] * inv;
        st[1] = o[db][4 * g + 1] * inv;
        st[2] = o[db][4 * g + 2] * inv;
        st[3] = o[db][4 * g + 3] * inv;
        *(f32x4*)(op + db * 32 + 8 * g + 4 * hh) = st;
      }
    if (hh == 0)
      p.lse[((int64_t)b * p.H + h) * p.lse_bh + qrow] = (m_run * c + fast_log2(l_tot)) * 0.6931471805599453f;
  }
}


// ---------------------------------------------------------------------------------
// fp32, few query rows: a launch of the kernel above with fewer workgroups than CUs lasts as long as one wave's
// chain of fp32 MFMAs over all key tiles (64 MFMAs of 64 cycles per 32 keys).  Here a workgroup owns 32 query rows
// and its NW waves take every NW-th key tile, each through an LDS tile pair of its own (no workgroup barrier in the
// loop); the waves' (O, m, l) are combined through LDS at the end.  Same arithmetic per tile as above.
// ---------------------------------------------------------------------------------
template <int D, int NW>
struct Fwd32SplitCfg {
  static constexpr int PITCH = D + 4;
  static constexpr int TILE = F32_BN * PITCH;          // floats per K or V tile
  static constexpr int WAVE = 2 * TILE;                // one wave's K and V tile
  static constexpr int SMEM = NW * WAVE * 4;           // the combine reuses it: NW x (32 x D + 64) floats fit
  static constexpr int CPR = D / 4;                    // 16-byte chunks per row
  static constexpr int RPP = 64 / CPR;                 // rows a wave fetches per pass
  static constexpr int PASS = F32_BN / RPP;
  static_assert(D <= 64, "built for head dims whose tile pair fits a wave's registers");
};

template <int D, int NW>
__global__ void __launch_bounds__(64 * NW, 1) flash_fwd32_splitk_kernel(const FwdParams p) {
  typedef Fwd32SplitCfg<D, NW> C;
  extern __shared__ __align__(16) unsigned char smem[];
  float* const sm = (float*)smem;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ln = lane & 31;
  const int hh = lane >> 5;
  const int h = blockIdx.x % p.H;
  const int b = blockIdx.x / p.H;
  const int qt = p.nqt - 1 - (int)blockIdx.y;
  const int q0 = qt * 32;
  const float* qp = (const float*)p.q + b * p.qs.b + h * p.qs.h;
  const float* kp = (const float*)p.k + b * p.ks.b + h * p.ks.h;
  const float* vp = (const float*)p.v + b * p.vs.b + h * p.vs.h;
  const int qrow = q0 + ln;
  const int qrow_c = qrow < p.Sq ? qrow : p.Sq - 1;
  f32x4 qf[D / 8];
#pragma unroll
  for (int g = 0; g < D / 8; ++g) {
    qf[g] = *(const f32x4*)(qp + (int64_t)qrow_c * p.qs.s + 8 * g + 4 * hh);
    if (p.negq) qf[g] = -qf[g];
  }
  const int kv_end = p.causal ? (q0 + 32 < p.Sk ? q0 + 32 : p.Sk) : p.Sk;
  const int nt = (kv_end + F32_BN - 1) / F32_BN;
  float* const kb = sm + w * C::WAVE;  // this wave's tiles
  float* const vb = kb + C::TILE;
  const int cc = lane % C::CPR, cr = lane / C::CPR;
  f32x4 kreg[C::PASS], vreg[C::PASS];
  auto gload = [&](int it) {
    const int key0 = it * F32_BN;
#pragma unroll
    for (int i = 0; i < C::PASS; ++i) {
      int r = key0 + cr + i * C::RPP;
      r = r < p.Sk ? r : p.Sk - 1;
      kreg[i] = *(const f32x4*)(kp + (int64_t)r * p.ks.s + cc * 4);
      vreg[i] = *(const f32x4*)(vp + (int64_t)r * p.vs.s + cc * 4);
    }
  };
  auto lstore = [&]() {
#pragma unroll
    for (int i = 0; i < C::PASS; ++i) {
      const int lr = cr + i * C::RPP;
      *(f32x4*)(kb + lr * C::PITCH + cc * 4) = kreg[i];
      *(f32x4*)(vb + lr * C::PITCH + cc * 4) = vreg[i];
    }
  };
  f32x16 o[D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[i][v] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  const float c = p.scale_log2;
  if (w < nt) gload(w);
  for (int it = w; it < nt; it += NW) {
    const int key0 = it * F32_BN;
    // the tile is this wave's alone: its own LDS reads of the tile before are done (in order), and a wave's LDS
    // writes are visible to its own later reads
    lstore();
    if (it + NW < nt) gload(it + NW);
    f32x16 s;
#pragma unroll
    for (int v = 0; v < 16; ++v) s[v] = 0.f;
#pragma unroll
    for (int g = 0; g < D / 8; ++g) {
      const f32x4 a = *(const f32x4*)(kb + ln * C::PITCH + 8 * g + 4 * hh);
#pragma unroll
      for (int e = 0; e < 4; ++e) s = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], qf[g][e], s, 0, 0, 0);
    }
    const bool need_mask = (p.causal && key0 + F32_BN - 1 > q0) || (key0 + F32_BN > p.Sk);
    if (need_mask) {
      const int lim = p.causal ? (qrow < p.Sk - 1 ? qrow : p.Sk - 1) : p.Sk - 1;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int key = key0 + 8 * (v >> 2) + 4 * hh + (v & 3);
        if (key > lim) s[v] = -INFINITY;
      }
    }
    float mx = s[0];
#pragma unroll
    for (int v = 1; v < 16; ++v) mx = fmaxf(mx, s[v]);
    mx = halves_max(mx);
    const float m_new = fmaxf(m_run, mx);
    // (a row past the last key of a causal tile that starts beyond it has seen nothing yet: -inf - -inf)
    const float alpha = m_new == -INFINITY ? 1.f : fast_exp2((m_run - m_new) * c);
    const float mc = m_new == -INFINITY ? 0.f : m_new * c;
    m_run = m_new;
    float ps = 0.f;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const float e = fast_exp2(__builtin_fmaf(s[v], c, -mc));
      s[v] = e;
      ps += e;
    }
    l_run = l_run * alpha + ps;
#pragma unroll
    for (int i = 0; i < D / 32; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) o[i][v] *= alpha;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int kl = 8 * (v >> 2) + 4 * hh + (v & 3);
#pragma unroll
      for (int db = 0; db < D / 32; ++db) {
        const float a = vb[kl * C::PITCH + db * 32 + ln];
        o[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, s[v], o[db], 0, 0, 0);
      }
    }
  }
  // ---- combine: every wave leaves its unscaled O (lane-private order) and (m, l); wave j then finishes the
  // 16-byte pieces j, j + NW, ... of every row ----
  constexpr int NPC = D / 8;           // 16-byte pieces per lane: (db, g)
  constexpr int REC = 64 * NPC * 4;    // floats of one wave's O
  const float l_own = halves_sum(l_run);
  __syncthreads();                     // every wave is done with its tiles
  float* const orec = sm + w * (REC + 128);
#pragma unroll
  for (int db = 0; db < D / 32; ++db)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      f32x4 st;
      st[0] = o[db][4 * g + 0]; st[1] = o[db][4 * g + 1]; st[2] = o[db][4 * g + 2]; st[3] = o[db][4 * g + 3];
      *(f32x4*)(orec + ((db * 4 + g) * 64 + lane) * 4) = st;
    }
  if (hh == 0) {
    orec[REC + ln] = m_run;
    orec[REC + 32 + ln] = l_own;
  }
  __syncthreads();
  float mw[NW], m_all = -INFINITY;
#pragma unroll
  for (int j = 0; j < NW; ++j) {
    mw[j] = sm[j * (REC + 128) + REC + ln];
    m_all = fmaxf(m_all, mw[j]);
  }
  float aw[NW], l_all = 0.f;
#pragma unroll
  for (int j = 0; j < NW; ++j) {
    aw[j] = mw[j] == -INFINITY ? 0.f : fast_exp2((mw[j] - m_all) * c);  // a wave without a visible key
    l_all += aw[j] * sm[j * (REC + 128) + REC + 32 + ln];
  }
  const float inv = 1.f / l_all;
  if (qrow < p.Sq) {
    float* const op = (float*)p.out + b * p.os.b + h * p.os.h + (int64_t)qrow * p.os.s;
    for (int pc = w; pc < NPC; pc += NW) {
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < NW; ++j) {
        const f32x4 x = *(const f32x4*)(sm + j * (REC + 128) + (pc * 64 + lane) * 4);
        acc[0] += aw[j] * x[0]; acc[1] += aw[j] * x[1]; acc[2] += aw[j] * x[2]; acc[3] += aw[j] * x[3];
      }
      acc[0] *= inv; acc[1] *= inv; acc[2] *= inv; acc[3] *= inv;
      const int db = pc / 4, g = pc % 4;
      *(f32x4*)(op + db * 32 + 8 * g + 4 * hh) = acc;
    }
    if (w == 0 && hh == 0) p.lse[((int64_t)b * p.H + h) * p.lse_bh + qrow] = (m_all * c + fast_log2(l_all)) * 0.6931471805599453f;
  }
}

template <auto kernel>
hipError_t launch(int threads, int smem, const FwdParams& p, hipStream_t stream) {
  const hipError_t e = spa_allow_dynamic_lds<kernel>(smem);
  if (e != hipSuccess) return e;
  if (p.nqt > 65535 || p.nranks > 65535) return hipErrorInvalidValue;
  const dim3 grid((unsigned)((int64_t)p.B * p.H), (unsigned)p.nqt, (unsigned)p.nranks);
  hipLaunchKernelGGL(kernel, grid, dim3(threads), smem, stream, p);
  return hipGetLastError();
}

// Query tiles of `bm` rows per (batch, head, rank): zigzag shards are tiled half by half (no tile holds
// rows of both halves); a launch for the second half only (zz_half) has that half's tiles.
int fwd_tiles(const FwdParams& p, int bm) {
  if (!p.zigzag) return (p.Sq + bm - 1) / bm;
  const int per_half = (p.Sq / 2 + bm - 1) / bm;
  return p.zz_half ? per_half : 2 * per_half;
}

// Two wave groups once there are at least two 64-key sub-tiles to split; 256-row workgroups with
// shared K/V buffers once that still leaves every CU at least two workgroups.  spa_tune() can
// force either choice (experiments and tests).
template <typename T, int D, bool ZZ>
hipError_t launch16(FwdParams p, hipStream_t stream) {
  const int force = spa_knob(SPA_KNOB_FWD_GROUPS);
  const int force_share = spa_knob(SPA_KNOB_FWD_SHARE);
  const bool two = force ? force == 2 : p.Sk > fwd_bn<D>();
  if (p.epi == SPA_EPI_FINALN) {
    if (two) return launch<flash_fwd16_kernel<T, D, 2, false, false, true, ZZ>>(2 * FWD_THREADS, Fwd16Cfg<D, 2, false>::SMEM, p, stream);
    return launch<flash_fwd16_kernel<T, D, 1, false, false, true, ZZ>>(FWD_THREADS, Fwd16Cfg<D, 1, false>::SMEM, p, stream);
  }
  if (two && D >= 64) {
    const int nqt2 = fwd_tiles(p, 2 * FWD_BM);
    const int64_t wgs = (int64_t)p.B * p.H * nqt2 * p.nranks;
    const bool share = force_share ? force_share == 2 : wgs >= 2 * (int64_t)spa_device_cus();
    if (share) {
      p.nqt = nqt2;
      return launch<flash_fwd16_kernel<T, D, 2, (D >= 64), false, false, ZZ>>(2 * FWD_THREADS, Fwd16Cfg<D, 2, (D >= 64)>::SMEM, p, stream);
    }
  }
  if (two) return launch<flash_fwd16_kernel<T, D, 2, false, false, false, ZZ>>(2 * FWD_THREADS, Fwd16Cfg<D, 2, false>::SMEM, p, stream);
  return launch<flash_fwd16_kernel<T, D, 1, false, false, false, ZZ>>(FWD_THREADS, Fwd16Cfg<D, 1, false>::SMEM, p, stream);
}

// e4m3 K/V: the register-staged variants, chosen like the 16-bit ones.
template <typename T, int D, bool ZZ>
hipError_t launch16_kv8(FwdParams p, hipStream_t stream) {
  const int force = spa_knob(SPA_KNOB_FWD_GROUPS);
  const int force_share = spa_knob(SPA_KNOB_FWD_SHARE);
  const bool two = force ? force == 2 : p.Sk > fwd_bn<D>();
  if (p.epi == SPA_EPI_FINALN) {
    if (two) return launch<flash_fwd16_kernel<T, D, 2, false, true, true, ZZ>>(2 * FWD_THREADS, Fwd16Cfg<D, 2, false>::SMEM, p, stream);
    return launch<flash_fwd16_kernel<T, D, 1, false, true, true, ZZ>>(FWD_THREADS, Fwd16Cfg<D, 1, false>::SMEM, p, stream);
  }
  if (two) {
    const int nqt2 = fwd_tiles(p, 2 * FWD_BM);
    const int64_t wgs = (int64_t)p.B * p.H * nqt2 * p.nranks;
    const bool share = force_share ? force_share == 2 : wgs >= 2 * (int64_t)spa_device_cus();
    if (share) {
      p.nqt = nqt2;
      return launch<flash_fwd16_kernel<T, D, 2, true, true, false, ZZ>>(2 * FWD_THREADS, Fwd16Cfg<D, 2, true>::SMEM, p, stream);
    }
  }
  if (two) return launch<flash_fwd16_kernel<T, D, 2, false, true, false, ZZ>>(2 * FWD_THREADS, Fwd16Cfg<D, 2, false>::SMEM, p, stream);
  return launch<flash_fwd16_kernel<T, D, 1, false, true, false, ZZ>>(FWD_THREADS, Fwd16Cfg<D, 1, false>::SMEM, p, stream);
}

// K / V spanning 2 GiB or more per (batch, head): the re-based variants, 128-row workgroups with two wave groups
// (such a tensor has more than enough rows for them).
template <typename T, int D>
hipError_t launch16_big(const FwdParams& p, hipStream_t stream) {
  if (p.epi == SPA_EPI_FINALN)
    return launch<flash_fwd16_kernel<T, D, 2, false, false, true, false, true>>(2 * FWD_THREADS, Fwd16Cfg<D, 2, false>::SMEM, p, stream);
  return launch<flash_fwd16_kernel<T, D, 2, false, false, false, false, true>>(2 * FWD_THREADS, Fwd16Cfg<D, 2, false>::SMEM, p, stream);
}

// e4m3 q, k, v with the scores on the 8-bit matrix instruction (D = 128, block and ring calls): chosen like the others.
template <typename T>
hipError_t launch16_qk8(FwdParams p, hipStream_t stream) {
  constexpr int D = 128;
  const int force = spa_knob(SPA_KNOB_FWD_GROUPS);
  const int force_share = spa_knob(SPA_KNOB_FWD_SHARE);
  const bool two = force ? force == 2 : p.Sk > fwd_bn<D>();
  if (p.epi == SPA_EPI_FINALN) {
    if (two) return launch<flash_fwd16_kernel<T, D, 2, false, true, true, false, false, true>>(2 * FWD_THREADS, Fwd16Cfg<D, 2, false>::SMEM, p, stream);
    return launch<flash_fwd16_kernel<T, D, 1, false, true, true, false, false, true>>(FWD_THREADS, Fwd16Cfg<D, 1, false>::SMEM, p, stream);
  }
  if (two) {
    const int nqt2 = fwd_tiles(p, 2 * FWD_BM);
    const int64_t wgs = (int64_t)p.B * p.H * nqt2 * p.nranks;
    const bool share = force_share ? force_share == 2 : wgs >= 2 * (int64_t)spa_device_cus();
    if (share) {
      p.nqt = nqt2;
      return launch<flash_fwd16_kernel<T, D, 2, true, true, false, false, false, true>>(2 * FWD_THREADS, Fwd16Cfg<D, 2, true>::SMEM, p, stream);
    }
    return launch<flash_fwd16_kernel<T, D, 2, false, true, false, false, false, true>>(2 * FWD_THREADS, Fwd16Cfg<D, 2, false>::SMEM, p, stream);
  }
  return launch<flash_fwd16_kernel<T, D, 1, false, true, false, false, false, true>>(FWD_THREADS, Fwd16Cfg<D, 1, false>::SMEM, p, stream);
}

// One launch for a rank whose chunks arrive while it runs: 128-row workgroups, one or two wave groups.
template <typename T, int D>
hipError_t launch16_wait(const FwdParams& p, hipStream_t stream) {
  const int force = spa_knob(SPA_KNOB_FWD_GROUPS);
  const bool two = force ? force == 2 : p.Sk > fwd_bn<D>();
  if (two) return launch<flash_fwd16_kernel<T, D, 2, false, false, false, false, false, false, true>>(2 * FWD_THREADS, Fwd16Cfg<D, 2, false>::SMEM, p, stream);
  return launch<flash_fwd16_kernel<T, D, 1, false, false, false, false, false, false, true>>(FWD_THREADS, Fwd16Cfg<D, 1, false>::SMEM, p, stream);
}

// The same for e4m3 q, k, v with the scores on the 8-bit matrix instruction (D = 128).
template <typename T>
hipError_t launch16_wait_qk8(const FwdParams& p, hipStream_t stream) {
  constexpr int D = 128;
  const int force = spa_knob(SPA_KNOB_FWD_GROUPS);
  const bool two = force ? force == 2 : p.Sk > fwd_bn<D>();
  if (two) return launch<flash_fwd16_kernel<T, D, 2, false, true, false, false, false, true, true>>(2 * FWD_THREADS, Fwd16Cfg<D, 2, false>::SMEM, p, stream);
  return launch<flash_fwd16_kernel<T, D, 1, false, true, false, false, false, true, true>>(FWD_THREADS, Fwd16Cfg<D, 1, false>::SMEM, p, stream);
}

// (dtype, D) -> kernel family; the zigzag variants are instantiated beside the plain ones
template <bool ZZ>
hipError_t launch16_any(const FwdParams& p, int D, int dtype, hipStream_t stream) {
  if (p.k_scale) {  // K / V are e4m3 bytes, q / out of type `dtype`
    if (!p.v_scale) return hipErrorInvalidValue;
    if (dtype == 1) {
      if (D == 128) return launch16_kv8<__bf16, 128, ZZ>(p, stream);
      if (D == 64) return launch16_kv8<__bf16, 64, ZZ>(p, stream);
    } else if (dtype == 2) {
      if (D == 128) return launch16_kv8<_Float16, 128, ZZ>(p, stream);
      if (D == 64) return launch16_kv8<_Float16, 64, ZZ>(p, stream);
    }
    return hipErrorInvalidValue;
  }
  if (dtype == 1) {
    if (D == 128) return launch16<__bf16, 128, ZZ>(p, stream);
    if (D == 64) return launch16<__bf16, 64, ZZ>(p, stream);
    if (D == 32) return launch16<__bf16, 32, ZZ>(p, stream);
  } else if (dtype == 2) {
    if (D == 128) return launch16<_Float16, 128, ZZ>(p, stream);
    if (D == 64) return launch16<_Float16, 64, ZZ>(p, stream);
    if (D == 32) return launch16<_Float16, 32, ZZ>(p, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace

// This file makes four objects: compiled with SPA_FWD_ZIGZAG_UNIT it holds the zigzag variants of the 16-bit
// kernel and nothing else, with SPA_FWD_SPLITKV_UNIT those that split the keys over the grid and those for a ring over a
// packed variable-length batch, with SPA_FWD_BIG_UNIT the
// re-based variants, those with 8-bit scores and those that wait for chunk arrival flags, without any of them
// everything else (so that the parts compile side by side).
#if defined(SPA_FWD_SPLITKV_UNIT)
// Keys split over grid.z (the caller has set P, Sk, sk_last, nranks = P and pointed out / lse at the scratch tensors).
hipError_t spa_launch_fwd16_splitkv(FwdParams p, int D, int dtype, hipStream_t stream) {
  if (p.causal || p.P < 2 || p.nranks != p.P || p.rank0 != 0 || p.t_begin != 0 || p.t_count != 1 || p.sk_last <= 0 || p.sk_last > p.Sk ||
      p.Sk <= fwd_bn<128>() || p.zigzag || p.big || p.arrive || p.q_scale || p.cu_q || p.epi != SPA_EPI_PLAIN || (p.k_scale && !p.v_scale))
    return hipErrorInvalidValue;
  p.nqt = fwd_tiles(p, FWD_BM);
#define SPA_KS(T, DD, KV8) \
  launch<flash_fwd16_kernel<T, DD, 2, false, KV8, false, false, false, false, false, true>>(2 * FWD_THREADS, Fwd16Cfg<DD, 2, false>::SMEM, p, stream)
  if (p.k_scale) {
    if (dtype == 1) { if (D == 128) return SPA_KS(__bf16, 128, true); if (D == 64) return SPA_KS(__bf16, 64, true); }
    if (dtype == 2) { if (D == 128) return SPA_KS(_Float16, 128, true); if (D == 64) return SPA_KS(_Float16, 64, true); }
    return hipErrorInvalidValue;
  }
  if (dtype == 1) { if (D == 128) return SPA_KS(__bf16, 128, false); if (D == 64) return SPA_KS(__bf16, 64, false); }
  if (dtype == 2) { if (D == 128) return SPA_KS(_Float16, 128, false); if (D == 64) return SPA_KS(_Float16, 64, false); }
#undef SPA_KS
  return hipErrorInvalidValue;
}
// A ring over a packed variable-length batch (cu_q, P > 1, chunk_rows / rank_rows = rows of a shard): 128-row workgroups.
hipError_t spa_launch_fwd16_varlen_ring(FwdParams p, int D, int dtype, hipStream_t stream) {
  if (!p.cu_q || !p.cu_k || p.chunk_rows <= 0 || p.rank_rows <= 0 || p.zigzag || p.big || p.arrive || p.k_scale || p.q_scale ||
      p.epi != SPA_EPI_PLAIN)
    return hipErrorInvalidValue;
  p.nqt = fwd_tiles(p, FWD_BM);
  const int force = spa_knob(SPA_KNOB_FWD_GROUPS);
  const bool two = force ? force == 2 : p.Sk > fwd_bn<128>();
#define SPA_VR(T, DD)                                                                                                                     \
  (two ? launch<flash_fwd16_kernel<T, DD, 2, false, false, false, false, false, false, false, false, true>>(2 * FWD_THREADS, Fwd16Cfg<DD, 2, false>::SMEM, p, stream) \
       : launch<flash_fwd16_kernel<T, DD, 1, false, false, false, false, false, false, false, false, true>>(FWD_THREADS, Fwd16Cfg<DD, 1, false>::SMEM, p, stream))
  if (dtype == 1) { if (D == 128) return SPA_VR(__bf16, 128); if (D == 64) return SPA_VR(__bf16, 64); if (D == 32) return SPA_VR(__bf16, 32); }
  if (dtype == 2) { if (D == 128) return SPA_VR(_Float16, 128); if (D == 64) return SPA_VR(_Float16, 64); if (D == 32) return SPA_VR(_Float16, 32); }
#undef SPA_VR
  return hipErrorInvalidValue;
}
#elif defined(SPA_FWD_ZIGZAG_UNIT)
hipError_t spa_launch_fwd16_zigzag(const FwdParams& p, int D, int dtype, hipStream_t stream) {
  return launch16_any<true>(p, D, dtype, stream);
}
#elif defined(SPA_FWD_BIG_UNIT)
hipError_t spa_launch_fwd16_qk8(const FwdParams& p, int D, int dtype, hipStream_t stream) {
  if (D != 128 || !p.q_scale || !p.k_scale || !p.v_scale || p.zigzag || p.big || p.cu_q) return hipErrorInvalidValue;
  if (dtype == 1) return launch16_qk8<__bf16>(p, stream);
  if (dtype == 2) return launch16_qk8<_Float16>(p, stream);
  return hipErrorInvalidValue;
}
hipError_t spa_launch_fwd16_wait(const FwdParams& p, int D, int dtype, hipStream_t stream) {
  if (!p.arrive || !p.fault || p.zigzag || p.big || p.epi != SPA_EPI_PLAIN || p.cu_q) return hipErrorInvalidValue;
  if (p.k_scale || p.v_scale || p.q_scale) {  // e4m3 tensors: all three, 8-bit scores
    if (!p.k_scale || !p.v_scale || !p.q_scale || D != 128) return hipErrorInvalidValue;
    if (dtype == 1) return launch16_wait_qk8<__bf16>(p, stream);
    if (dtype == 2) return launch16_wait_qk8<_Float16>(p, stream);
    return hipErrorInvalidValue;
  }
  if (dtype == 1) {
    if (D == 128) return launch16_wait<__bf16, 128>(p, stream);
    if (D == 64) return launch16_wait<__bf16, 64>(p, stream);
  } else if (dtype == 2) {
    if (D == 128) return launch16_wait<_Float16, 128>(p, stream);
    if (D == 64) return launch16_wait<_Float16, 64>(p, stream);
  }
  return hipErrorInvalidValue;
}
hipError_t spa_launch_fwd16_big(const FwdParams& p, int D, int dtype, hipStream_t stream) {
  if (p.k_scale || p.zigzag) return hipErrorInvalidValue;  // no re-based e4m3 or zigzag variants
  if (dtype == 1) {
    if (D == 128) return launch16_big<__bf16, 128>(p, stream);
    if (D == 64) return launch16_big<__bf16, 64>(p, stream);
    if (D == 32) return launch16_big<__bf16, 32>(p, stream);
  } else if (dtype == 2) {
    if (D == 128) return launch16_big<_Float16, 128>(p, stream);
    if (D == 64) return launch16_big<_Float16, 64>(p, stream);
    if (D == 32) return launch16_big<_Float16, 32>(p, stream);
  }
  return hipErrorInvalidValue;
}
#else
hipError_t spa_launch_fwd16_zigzag(const FwdParams& p, int D, int dtype, hipStream_t stream);
hipError_t spa_launch_fwd16_big(const FwdParams& p, int D, int dtype, hipStream_t stream);
hipError_t spa_launch_fwd16_qk8(const FwdParams& p, int D, int dtype, hipStream_t stream);
hipError_t spa_launch_fwd16_wait(const FwdParams& p, int D, int dtype, hipStream_t stream);
hipError_t spa_launch_fwd16_varlen_ring(FwdParams p, int D, int dtype, hipStream_t stream);

// Returns hipSuccess, or hipErrorInvalidValue for an unsupported (dtype, D).
hipError_t spa_launch_flash_fwd(FwdParams p, int D, int dtype, hipStream_t stream) {
  if (p.zigzag && (dtype == 0 || !p.causal || (p.Sq & 1) || p.cu_q)) return hipErrorInvalidValue;  // 16-bit causal rings only
  p.nqt = fwd_tiles(p, FWD_BM);
  if (p.epi == SPA_EPI_PART) {
    // A ring step that is not the rank's last: the kernel writes the block as it would write any
    // result, and out / lse are pointed at the step's slot here.  The kernel adds the rank's row
    // offset (rank0 * Sq rows) to both, so the slot's addresses go in with that offset taken off.
    if (dtype == 0 || p.nranks != 1 || !p.part) return hipErrorInvalidValue;
    const RingSlots slots(p.B, p.H, p.Sq, D);
    p.os.b = (int64_t)p.Sq * p.H * D; p.os.s = (int64_t)p.H * D; p.os.h = D;
    p.lse_bh = p.Sq;
    const int64_t row0 = (int64_t)p.rank0 * p.Sq;
    p.out = (char*)slots.out<char>(p.part, p.part_slot) - row0 * p.os.s * 2;
    p.lse = slots.lse(p.part, p.P, p.part_slot) - row0;
  }
  if ((dtype == 1 || dtype == 2) && p.chunk_rows) return spa_launch_fwd16_varlen_ring(p, D, dtype, stream);
  if ((dtype == 1 || dtype == 2) && p.arrive) return spa_launch_fwd16_wait(p, D, dtype, stream);
  if ((dtype == 1 || dtype == 2) && p.q_scale) return spa_launch_fwd16_qk8(p, D, dtype, stream);
  if (dtype == 1 || dtype == 2)
    return p.big ? spa_launch_fwd16_big(p, D, dtype, stream)
                 : p.zigzag ? spa_launch_fwd16_zigzag(p, D, dtype, stream) : launch16_any<false>(p, D, dtype, stream);
  if (dtype == 0) {
    if (p.epi != SPA_EPI_PLAIN) return hipErrorInvalidValue;  // fp32 ring steps merge with the separate kernel
    // Few 128-row workgroups (fewer than half the CUs), a head dim whose tile pair fits a wave's registers: 32-row
    // workgroups whose 8 waves share the key tiles.  spa_tune("fwd32_split"): 1 never, 2 whenever D <= 64.
    const int knob = spa_knob(SPA_KNOB_FWD32_SPLIT);
    const bool few = 2 * (int64_t)p.B * p.H * p.nqt <= spa_device_cus() && p.Sk > 4 * F32_BN;
    if (D <= 64 && !p.cu_q && p.nranks == 1 && p.P == 1 && knob != 1 && (few || knob == 2)) {
      FwdParams ps = p;
      ps.nqt = (p.Sq + 31) / 32;
      if (D == 64) return launch<flash_fwd32_splitk_kernel<64, 8>>(512, Fwd32SplitCfg<64, 8>::SMEM, ps, stream);
      return launch<flash_fwd32_splitk_kernel<32, 8>>(512, Fwd32SplitCfg<32, 8>::SMEM, ps, stream);
    }
    if (D == 128) return launch<flash_fwd32_kernel<128>>(FWD_THREADS, Fwd32Cfg<128>::SMEM, p, stream);
    if (D == 64) return launch<flash_fwd32_kernel<64>>(FWD_THREADS, Fwd32Cfg<64>::SMEM, p, stream);
    if (D == 32) return launch<flash_fwd32_kernel<32>>(FWD_THREADS, Fwd32Cfg<32>::SMEM, p, stream);
  }
  return hipErrorInvalidValue;
}
#endif  // SPA_FWD_SPLITKV_UNIT / SPA_FWD_ZIGZAG_UNIT / SPA_FWD_BIG_UNIT
