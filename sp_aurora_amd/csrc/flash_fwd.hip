// Block flash-attention forward for gfx950: out = softmax(q k^T * scale + mask) v and
// fp32 lse = logsumexp(q k^T * scale + mask), one launch per (q chunk, kv chunk) pair.
// Stands in for intel_flash_attn_forward (sp_aurora/intel_flash_attn.py:18-126) /
// intel_flash_attn_forward_optimized (sp_aurora/intel_flash_attn_optimized.py:95-225):
// one Q.K^T instead of the reference's two, scores never leave the CU.
//
// Work decomposition (16-bit kernel)
//   workgroup = 128 query rows of one (batch, head), 4 wavefronts x 32 rows;
//   KV is walked in tiles of 64 keys, double-buffered in LDS.
//   Both contractions are computed TRANSPOSED on v_mfma_f32_32x32x16:
//     S^T[key][qrow] = K[key][:] . Q[qrow][:]      A = K tile (LDS), B = Q (registers)
//     O^T[d][qrow]  += V^T[d][key] . P^T[key][qrow] A = V^T tile (LDS), B = P^T (registers)
//   In the 32x32 accumulator layout a lane owns ONE query row (column lane%32)
//   and 16 of the 32 block rows, so the row max / row sum of the softmax is a
//   per-lane reduction plus one exchange with lane^32, the rescale of O is a
//   per-lane scalar, and the S^T accumulators are, register for register,
//   the B operand of the second contraction: P never touches LDS.
//   The contraction index of an MFMA may be permuted freely as long as A and
//   B agree; V^T is stored in LDS with keys permuted (bits 2 and 3 of the key
//   index within a 32-key block swapped) so that the 8 keys a lane needs for
//   one P^T operand are one 16-byte LDS read.
#include <stdlib.h>

#include "spa_common.h"

namespace {

constexpr int FWD_BM = 128;  // query rows per workgroup
constexpr int FWD_BN = 64;   // keys per LDS sub-tile (one per wave group)
constexpr int FWD_THREADS = 256;  // threads of one wave group (4 waves x 32 query rows)

// NG wave groups share the 128 query rows and split the keys: in every step group g works on
// the g-th 64-key sub-tile of a 64*NG-key tile, so 4*NG waves sit on the CU's 4 SIMDs and the
// MFMA phase of one wave overlaps the softmax (VALU) phase of its SIMD neighbour.  The groups'
// partial (O, m, l) are combined through LDS after the key loop.
template <int D, int NG>
struct Fwd16Cfg {
  static constexpr int THREADS = FWD_THREADS * NG;
  static constexpr int KP = D * 2 + 16;       // K tile row pitch in bytes (+16: bank spread)
  static constexpr int VP = FWD_BN * 2 + 16;  // V^T tile row pitch in bytes
  static constexpr int KBYTES = FWD_BN * KP;
  static constexpr int VBYTES = D * VP;
  static constexpr int SUB = KBYTES + VBYTES;  // one 64-key sub-tile: K rows, then V^T
  static constexpr int STAGE = NG * SUB;
  static constexpr int XCH = NG > 1 ? 4 * (D / 2 + 2) * 64 * 4 : 0;  // group exchange area
  static constexpr int SMEM = 2 * STAGE > XCH ? 2 * STAGE : XCH;
  static constexpr int CPR = D / 8;              // 16-byte chunks per row
  static constexpr int RPP = THREADS / CPR;      // K rows fetched per pass
  static constexpr int KPASS = FWD_BN * NG / RPP;  // passes per K tile
  static constexpr int VUNITS = 16 * NG * CPR;   // (4 keys x 8 dims) units per V tile
};

template <typename T, int D, int NG>
__global__ void __launch_bounds__(FWD_THREADS * NG, 1) flash_fwd16_kernel(const FwdParams p) {
  typedef Fwd16Cfg<D, NG> C;
  typedef Mma16<T> M;
  typedef typename M::frag frag;
  extern __shared__ __align__(16) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int w = wave & 3;    // which 32 query rows
  const int grp = wave >> 2;  // which key sub-tile
  const int ln = lane & 31;
  const int hh = lane >> 5;

  // Consecutive workgroup ids walk the heads first: with round-robin placement of
  // workgroups on the 8 XCDs, all query tiles of a head share one XCD's L2 for K/V.
  int bid = blockIdx.x;
  const int h = bid % p.H;
  bid /= p.H;
  const int qt = p.nqt - 1 - (bid % p.nqt);  // heaviest causal tiles first
  const int b = bid / p.nqt;
  const int q0 = qt * FWD_BM;
  const int qw0 = q0 + w * 32;

  const T* qp = (const T*)p.q + b * p.qs.b + h * p.qs.h;
  const T* kp = (const T*)p.k + b * p.ks.b + h * p.ks.h;
  const T* vp = (const T*)p.v + b * p.vs.b + h * p.vs.h;

  const int qrow = qw0 + ln;
  const int qrow_c = qrow < p.Sq ? qrow : p.Sq - 1;

  frag qf[D / 16];
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks)
    qf[ks] = as_frag<frag>(*(const u32x4*)(qp + (int64_t)qrow_c * p.qs.s + ks * 16 + hh * 8));

  constexpr int TILE = FWD_BN * NG;
  const int kv_end = p.causal ? (q0 + FWD_BM < p.Sk ? q0 + FWD_BM : p.Sk) : p.Sk;
  const int nt = (kv_end + TILE - 1) / TILE;

  // ---- global -> register staging of one K / V tile ----
  const int kc = tid % C::CPR;
  const int kr = tid / C::CPR;
  const int vkg = tid & (16 * NG - 1);  // group of 4 consecutive keys
  const int vdc = tid / (16 * NG);      // chunk of 8 head dims
  const bool vact = tid < C::VUNITS;
  // position of this key group inside the permuted 64-key row of its sub-tile's V^T
  const int vsub = vkg >> 4;
  const int vpos = ((vkg >> 3) & 1) * 32 + ((vkg >> 2) & 1) * 16 + (vkg & 1) * 8 + ((vkg >> 1) & 1) * 4;

  u32x4 kreg[C::KPASS];
  u32x4 vreg[4];

  auto gload = [&](int it) {
    const int key0 = it * TILE;
#pragma unroll
    for (int i = 0; i < C::KPASS; ++i) {
      int r = key0 + kr + i * C::RPP;
      r = r < p.Sk ? r : p.Sk - 1;
      kreg[i] = *(const u32x4*)(kp + (int64_t)r * p.ks.s + kc * 8);
    }
    if (vact) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        int r = key0 + vkg * 4 + j;
        r = r < p.Sk ? r : p.Sk - 1;
        vreg[j] = *(const u32x4*)(vp + (int64_t)r * p.vs.s + vdc * 8);
      }
    }
  };

  auto lstore = [&](int stage) {
    unsigned char* sb = smem + stage * C::STAGE;
#pragma unroll
    for (int i = 0; i < C::KPASS; ++i) {
      const int r = kr + i * C::RPP;
      *(u32x4*)(sb + (r >> 6) * C::SUB + (r & 63) * C::KP + kc * 16) = kreg[i];
    }
    if (vact) {
      unsigned char* vb = sb + vsub * C::SUB + C::KBYTES;
      // 4 keys x 8 dims in registers -> 8 rows (dims) of 4 consecutive keys
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        const unsigned a0 = vreg[0][m], a1 = vreg[1][m], a2 = vreg[2][m], a3 = vreg[3][m];
        u32x2 even, odd;
        even[0] = (a0 & 0xffffu) | (a1 << 16);
        even[1] = (a2 & 0xffffu) | (a3 << 16);
        odd[0] = (a0 >> 16) | (a1 & 0xffff0000u);
        odd[1] = (a2 >> 16) | (a3 & 0xffff0000u);
        *(u32x2*)(vb + (vdc * 8 + 2 * m) * C::VP + vpos * 2) = even;
        *(u32x2*)(vb + (vdc * 8 + 2 * m + 1) * C::VP + vpos * 2) = odd;
      }
    }
  };

  f32x16 o[D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[i][v] = 0.f;
  float m_run = -INFINITY;  // reference row max of the raw scores (may lag the true max, see below)
  float l_run = 0.f;        // this lane's share of the running row sum

  gload(0);
  lstore(0);
  __syncthreads();

  const float c = p.scale_log2;

  for (int it = 0; it < nt; ++it) {
    const int cur = it & 1;
    const int key0 = it * TILE + grp * FWD_BN;
    const bool more = it + 1 < nt;
    if (more) gload(it + 1);

    // a wave whose rows all precede its sub-tile, or whose sub-tile lies past the keys, idles
    const bool active = key0 < kv_end && !(p.causal && key0 > qw0 + 31);
    if (active) {
      const unsigned char* kb = smem + cur * C::STAGE + grp * C::SUB;
      const unsigned char* vb = kb + C::KBYTES;

      f32x16 s[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
#pragma unroll
        for (int v = 0; v < 16; ++v) s[t][v] = 0.f;
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks) {
          const frag a = as_frag<frag>(*(const u32x4*)(kb + (t * 32 + ln) * C::KP + (ks * 16 + hh * 8) * 2));
          s[t] = M::run(a, qf[ks], s[t]);
        }
      }

      const bool need_mask = (p.causal && key0 + FWD_BN - 1 > qw0) || (key0 + FWD_BN > p.Sk);
      if (need_mask) {
        const int lim = p.causal ? (qrow < p.Sk - 1 ? qrow : p.Sk - 1) : p.Sk - 1;  // last visible key
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int key = key0 + t * 32 + 8 * (v >> 2) + 4 * hh + (v & 3);
            if (key > lim) s[t][v] = -INFINITY;
          }
      }

      float mx = s[0][0];
#pragma unroll
      for (int v = 1; v < 16; ++v) mx = fmaxf(mx, s[0][v]);
#pragma unroll
      for (int v = 0; v < 16; ++v) mx = fmaxf(mx, s[1][v]);
      mx = fmaxf(mx, xhalf(mx));
      // Lazy rescale: the reference max only moves when some row's max grew by more than
      // 2^8 in the exp2 domain; until then P <= 256, harmless in fp32 sums and bf16 operands.
      if (__builtin_amdgcn_ballot_w64((mx - m_run) * c > 8.f) != 0) {
        const float m_new = fmaxf(m_run, mx);
        const float alpha = fast_exp2((m_run - m_new) * c);
        m_run = m_new;
        l_run *= alpha;
#pragma unroll
        for (int i = 0; i < D / 32; ++i)
#pragma unroll
          for (int v = 0; v < 16; ++v) o[i][v] *= alpha;
      }
      const float mc = m_run * c;

      float ps = 0.f;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const float e = fast_exp2(__builtin_fmaf(s[t][v], c, -mc));
          s[t][v] = e;
          ps += e;
        }
      l_run += ps;

      frag pf[2][2];
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int u = 0; u < 2; ++u)
          pf[t][u] = M::pack(s[t][8 * u + 0], s[t][8 * u + 1], s[t][8 * u + 2], s[t][8 * u + 3],
                             s[t][8 * u + 4], s[t][8 * u + 5], s[t][8 * u + 6], s[t][8 * u + 7]);

#pragma unroll
      for (int db = 0; db < D / 32; ++db)
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int u = 0; u < 2; ++u) {
            const frag a = as_frag<frag>(
                *(const u32x4*)(vb + (db * 32 + ln) * C::VP + (t * 32 + u * 16 + hh * 8) * 2));
            o[db] = M::run(a, pf[t][u], o[db]);
          }
    }

    if (more) lstore(cur ^ 1);
    __syncthreads();
  }

  // ---- combine the wave groups: groups 1.. hand (O, m, l) to group 0 through LDS ----
  if (NG > 1) {
    float* xch = (float*)smem;  // [w][slot][lane], slot = D/2 accumulators, then m, then l
    constexpr int SLOTS = D / 2 + 2;
    if (grp == 1) {
      float* dst = xch + (w * SLOTS) * 64 + lane;
#pragma unroll
      for (int i = 0; i < D / 32; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) dst[(i * 16 + v) * 64] = o[i][v];
      dst[(D / 2) * 64] = m_run;
      dst[(D / 2 + 1) * 64] = l_run;
    }
    __syncthreads();
    if (grp == 0) {
      const float* src = xch + (w * SLOTS) * 64 + lane;
      const float m1 = src[(D / 2) * 64];
      const float l1 = src[(D / 2 + 1) * 64];
      const float m_new = fmaxf(m_run, m1);  // finite: group 0 always sees key 0
      const float a0 = fast_exp2((m_run - m_new) * c);
      const float a1 = fast_exp2((m1 - m_new) * c);
      m_run = m_new;
      l_run = l_run * a0 + l1 * a1;
#pragma unroll
      for (int i = 0; i < D / 32; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[i][v] = o[i][v] * a0 + src[(i * 16 + v) * 64] * a1;
    }
  }

  // ---- epilogue: normalise, store out and lse ----
  if (grp == 0) {
    const float l_tot = l_run + xhalf(l_run);
    const float inv = 1.f / l_tot;
    if (qrow < p.Sq) {
      T* op = (T*)p.out + b * p.os.b + h * p.os.h + (int64_t)qrow * p.os.s;
#pragma unroll
      for (int db = 0; db < D / 32; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          u32x2 st;
          st[0] = M::pack2(o[db][4 * g + 0] * inv, o[db][4 * g + 1] * inv);
          st[1] = M::pack2(o[db][4 * g + 2] * inv, o[db][4 * g + 3] * inv);
          *(u32x2*)(op + db * 32 + 8 * g + 4 * hh) = st;
        }
      if (hh == 0)
        p.lse[((int64_t)b * p.H + h) * p.Sq + qrow] = (m_run * c + fast_log2(l_tot)) * 0.6931471805599453f;
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
__global__ void __launch_bounds__(FWD_THREADS, 1) flash_fwd32_kernel(const FwdParams p) {
  typedef Fwd32Cfg<D> C;
  extern __shared__ __align__(16) unsigned char smem[];
  float* sm = (float*)smem;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int w = tid >> 6;
  const int ln = lane & 31;
  const int hh = lane >> 5;

  int bid = blockIdx.x;
  const int h = bid % p.H;
  bid /= p.H;
  const int qt = p.nqt - 1 - (bid % p.nqt);
  const int b = bid / p.nqt;
  const int q0 = qt * FWD_BM;
  const int qw0 = q0 + w * 32;

  const float* qp = (const float*)p.q + b * p.qs.b + h * p.qs.h;
  const float* kp = (const float*)p.k + b * p.ks.b + h * p.ks.h;
  const float* vp = (const float*)p.v + b * p.vs.b + h * p.vs.h;

  const int qrow = qw0 + ln;
  const int qrow_c = qrow < p.Sq ? qrow : p.Sq - 1;

  // Contraction step u (0..D/2-1) of the first product uses head dim
  // 8*(u/4) + 4*hh + (u%4): a lane's dims come as 16-byte groups.
  f32x4 qf[D / 8];
#pragma unroll
  for (int g = 0; g < D / 8; ++g)
    qf[g] = *(const f32x4*)(qp + (int64_t)qrow_c * p.qs.s + 8 * g + 4 * hh);

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
      mx = fmaxf(mx, xhalf(mx));
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

  const float l_tot = l_run + xhalf(l_run);
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
      p.lse[((int64_t)b * p.H + h) * p.Sq + qrow] = (m_run * c + fast_log2(l_tot)) * 0.6931471805599453f;
  }
}

template <typename K>
hipError_t launch(K kernel, int threads, int smem, const FwdParams& p, hipStream_t stream) {
  hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
  if (e != hipSuccess) return e;
  const dim3 grid((unsigned)((int64_t)p.B * p.H * p.nqt));
  hipLaunchKernelGGL(kernel, grid, dim3(threads), smem, stream, p);
  return hipGetLastError();
}

// Two wave groups once there are at least two 64-key sub-tiles to split.
template <typename T, int D>
hipError_t launch16(const FwdParams& p, hipStream_t stream) {
  static const int force = []() {
    const char* e = getenv("SPA_FWD_GROUPS");
    return e ? atoi(e) : 0;
  }();
  const bool two = force ? force == 2 : p.Sk > FWD_BN;
  if (two) return launch(flash_fwd16_kernel<T, D, 2>, 2 * FWD_THREADS, Fwd16Cfg<D, 2>::SMEM, p, stream);
  return launch(flash_fwd16_kernel<T, D, 1>, FWD_THREADS, Fwd16Cfg<D, 1>::SMEM, p, stream);
}

}  // namespace

// Returns hipSuccess, or hipErrorInvalidValue for an unsupported (dtype, D).
hipError_t spa_launch_flash_fwd(FwdParams p, int D, int dtype, hipStream_t stream) {
  p.nqt = (p.Sq + FWD_BM - 1) / FWD_BM;
  if (dtype == 1) {
    if (D == 128) return launch16<__bf16, 128>(p, stream);
    if (D == 64) return launch16<__bf16, 64>(p, stream);
    if (D == 32) return launch16<__bf16, 32>(p, stream);
  } else if (dtype == 2) {
    if (D == 128) return launch16<_Float16, 128>(p, stream);
    if (D == 64) return launch16<_Float16, 64>(p, stream);
    if (D == 32) return launch16<_Float16, 32>(p, stream);
  } else if (dtype == 0) {
    if (D == 128) return launch(flash_fwd32_kernel<128>, FWD_THREADS, Fwd32Cfg<128>::SMEM, p, stream);
    if (D == 64) return launch(flash_fwd32_kernel<64>, FWD_THREADS, Fwd32Cfg<64>::SMEM, p, stream);
    if (D == 32) return launch(flash_fwd32_kernel<32>, FWD_THREADS, Fwd32Cfg<32>::SMEM, p, stream);
  }
  return hipErrorInvalidValue;
}
