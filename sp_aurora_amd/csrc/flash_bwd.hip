// Block-wise attention backward for gfx950 with the GLOBAL lse / delta of the query rows:
//   P = exp(q k^T * scale + mask - lse);  dV += P^T dO;  dP = dO V^T;
//   dS = P * (dP - delta);  dQ += dS K * scale;  dK += dS^T Q * scale.
// Stands in for the per-step body of intel_ring_flash_attn_backward
// (sp_aurora/intel_ring_flash_attn.py:192-258), which re-runs autograd on each block.
//
// Two kernels, no atomics, every output row has one owner (deterministic):
//   dq kernel   : workgroup = 128 query rows (4 waves x 32), walks key tiles of 64.
//                 S^T = K Q^T and dP^T = V dO^T land with a lane owning one query row,
//                 so lse/delta are per-lane scalars and dS^T is, register for register,
//                 the B operand of dQ^T = K^T dS^T (K^T staged transposed in LDS).
//   dkdv kernel : workgroup = 128 keys (4 waves x 32), walks query tiles of 64.
//                 S = Q K^T and dP = dO V^T land with a lane owning one key, so P and dS
//                 are the B operands of dV^T = dO^T P and dK^T = Q^T dS (Q^T, dO^T staged
//                 transposed in LDS).
// The MFMA contraction index is permuted the same way on both operands (bits 2 and 3 of the
// index inside a 32-block swapped) so that every operand is one 16-byte LDS read.
// Accumulators are fp32 in HBM and are ADDED to (read-modify-write by the owning lane).
#include "spa_common.h"

namespace {

constexpr int BWD_THREADS = 256;
constexpr int BWD_ROWS = 64;  // rows (keys or queries) per streamed LDS tile

template <int D>
struct TileCfg {
  static constexpr int KP = D * 2 + 16;          // row pitch of a row-major tile, bytes
  static constexpr int VP = BWD_ROWS * 2 + 16;   // row pitch of a transposed tile, bytes
  static constexpr int ROWB = BWD_ROWS * KP;     // bytes of a row-major tile
  static constexpr int TRB = D * VP;             // bytes of a transposed tile
  static constexpr int CPR = D / 8;
  static constexpr int RPP = BWD_THREADS / CPR;
  static constexpr int PASS = BWD_ROWS / RPP;
  static constexpr int UNITS = 16 * CPR;
};

// ---- streamed tile, row-major: 64 rows x D elements ----
template <typename T, int D>
__device__ __forceinline__ void rows_gload(u32x4 (&reg)[TileCfg<D>::PASS], const T* base, int64_t stride,
                                           int row0, int nrows, int tid) {
  typedef TileCfg<D> C;
#pragma unroll
  for (int i = 0; i < C::PASS; ++i) {
    int r = row0 + tid / C::CPR + i * C::RPP;
    r = r < nrows ? r : nrows - 1;
    reg[i] = *(const u32x4*)(base + (int64_t)r * stride + (tid % C::CPR) * 8);
  }
}

template <int D>
__device__ __forceinline__ void rows_lstore(unsigned char* lds, const u32x4 (&reg)[TileCfg<D>::PASS], int tid) {
  typedef TileCfg<D> C;
#pragma unroll
  for (int i = 0; i < C::PASS; ++i)
    *(u32x4*)(lds + (tid / C::CPR + i * C::RPP) * C::KP + (tid % C::CPR) * 16) = reg[i];
}

// ---- streamed tile, transposed: D rows x 64 (permuted) columns; a thread moves 4 rows x 8 dims ----
template <typename T, int D>
__device__ __forceinline__ void tr_gload(u32x4 (&reg)[4], const T* base, int64_t stride, int row0, int nrows,
                                         int tid) {
  if (tid < TileCfg<D>::UNITS) {
    const int g = tid & 15, dc = tid >> 4;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int r = row0 + g * 4 + j;
      r = r < nrows ? r : nrows - 1;
      reg[j] = *(const u32x4*)(base + (int64_t)r * stride + dc * 8);
    }
  }
}

template <int D>
__device__ __forceinline__ void tr_lstore(unsigned char* lds, const u32x4 (&reg)[4], int tid) {
  typedef TileCfg<D> C;
  if (tid < C::UNITS) {
    const int g = tid & 15, dc = tid >> 4;
    const int pos = (g >> 3) * 32 + ((g >> 2) & 1) * 16 + (g & 1) * 8 + ((g >> 1) & 1) * 4;
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const unsigned a0 = reg[0][m], a1 = reg[1][m], a2 = reg[2][m], a3 = reg[3][m];
      u32x2 even, odd;
      even[0] = (a0 & 0xffffu) | (a1 << 16);
      even[1] = (a2 & 0xffffu) | (a3 << 16);
      odd[0] = (a0 >> 16) | (a1 & 0xffff0000u);
      odd[1] = (a2 >> 16) | (a3 & 0xffff0000u);
      *(u32x2*)(lds + (dc * 8 + 2 * m) * C::VP + pos * 2) = even;
      *(u32x2*)(lds + (dc * 8 + 2 * m + 1) * C::VP + pos * 2) = odd;
    }
  }
}

template <typename F, int D>
__device__ __forceinline__ F row_frag(const unsigned char* lds, int row, int ks, int hh) {
  return as_frag<F>(*(const u32x4*)(lds + row * TileCfg<D>::KP + (ks * 16 + hh * 8) * 2));
}

template <typename F, int D>
__device__ __forceinline__ F tr_frag(const unsigned char* lds, int row, int t, int u, int hh) {
  return as_frag<F>(*(const u32x4*)(lds + row * TileCfg<D>::VP + (t * 32 + u * 16 + hh * 8) * 2));
}

__device__ __forceinline__ void zero16(f32x16& x) {
#pragma unroll
  for (int v = 0; v < 16; ++v) x[v] = 0.f;
}

// ------------------------------------------------------------------------------------------
// dQ kernel
// ------------------------------------------------------------------------------------------
template <int D>
struct DqCfg {
  typedef TileCfg<D> C;
  static constexpr int STAGE = 2 * C::ROWB + C::TRB;  // K rows, V rows, K^T
  static constexpr int SMEM = 2 * STAGE;
};

template <typename T, int D>
__global__ void __launch_bounds__(BWD_THREADS, 1) flash_bwd_dq_kernel(const BwdParams p) {
  typedef TileCfg<D> C;
  typedef Mma16<T> M;
  typedef typename M::frag frag;
  extern __shared__ __align__(16) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63, w = tid >> 6, ln = lane & 31, hh = lane >> 5;

  int bid = blockIdx.x;
  const int h = bid % p.H;
  bid /= p.H;
  const int qt = p.nqt - 1 - (bid % p.nqt);
  const int b = bid / p.nqt;
  const int q0 = qt * 128;
  const int qw0 = q0 + w * 32;

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
  const int64_t li = ((int64_t)b * p.H + h) * p.Sq + qrow_c;
  const float l2 = p.lse[li] * 1.4426950408889634f;
  const float dl = p.delta[li];
  const float c = p.scale_log2;

  const int kv_end = p.causal ? (q0 + 128 < p.Sk ? q0 + 128 : p.Sk) : p.Sk;
  const int nt = (kv_end + BWD_ROWS - 1) / BWD_ROWS;

  u32x4 kreg[C::PASS], vreg[C::PASS], ktreg[4];
  auto gload = [&](int it) {
    rows_gload<T, D>(kreg, kp, p.ks.s, it * BWD_ROWS, p.Sk, tid);
    rows_gload<T, D>(vreg, vp, p.vs.s, it * BWD_ROWS, p.Sk, tid);
    tr_gload<T, D>(ktreg, kp, p.ks.s, it * BWD_ROWS, p.Sk, tid);
  };
  auto lstore = [&](int stage) {
    unsigned char* sb = smem + stage * DqCfg<D>::STAGE;
    rows_lstore<D>(sb, kreg, tid);
    rows_lstore<D>(sb + C::ROWB, vreg, tid);
    tr_lstore<D>(sb + 2 * C::ROWB, ktreg, tid);
  };

  f32x16 dq[D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; ++i) zero16(dq[i]);

  gload(0);
  lstore(0);
  __syncthreads();

  for (int it = 0; it < nt; ++it) {
    const int cur = it & 1;
    const int key0 = it * BWD_ROWS;
    const bool more = it + 1 < nt;
    if (more) gload(it + 1);

    const bool active = !(p.causal && key0 > qw0 + 31);
    if (active) {
      const unsigned char* kb = smem + cur * DqCfg<D>::STAGE;
      const unsigned char* vb = kb + C::ROWB;
      const unsigned char* ktb = kb + 2 * C::ROWB;

      f32x16 s[2], dp[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        zero16(s[t]);
        zero16(dp[t]);
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks) {
          s[t] = M::run(row_frag<frag, D>(kb, t * 32 + ln, ks, hh), qf[ks], s[t]);
          dp[t] = M::run(row_frag<frag, D>(vb, t * 32 + ln, ks, hh), dof[ks], dp[t]);
        }
      }

      const int lim = p.causal ? (qrow < p.Sk - 1 ? qrow : p.Sk - 1) : p.Sk - 1;  // last visible key
      frag dsf[2][2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int key = key0 + t * 32 + 8 * (v >> 2) + 4 * hh + (v & 3);
          const float pr = key > lim ? 0.f : fast_exp2(__builtin_fmaf(s[t][v], c, -l2));
          s[t][v] = pr * (dp[t][v] - dl);
        }
#pragma unroll
        for (int u = 0; u < 2; ++u)
          dsf[t][u] = M::pack(s[t][8 * u + 0], s[t][8 * u + 1], s[t][8 * u + 2], s[t][8 * u + 3],
                              s[t][8 * u + 4], s[t][8 * u + 5], s[t][8 * u + 6], s[t][8 * u + 7]);
      }

#pragma unroll
      for (int db = 0; db < D / 32; ++db)
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int u = 0; u < 2; ++u)
            dq[db] = M::run(tr_frag<frag, D>(ktb, db * 32 + ln, t, u, hh), dsf[t][u], dq[db]);
    }

    if (more) lstore(cur ^ 1);
    __syncthreads();
  }

  if (qrow < p.Sq) {
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
  typedef TileCfg<D> C;
  static constexpr int STAT = 2 * BWD_ROWS * 4;               // lse*log2e and delta of the tile rows
  static constexpr int STAGE = 2 * C::ROWB + 2 * C::TRB + STAT;  // Q rows, dO rows, Q^T, dO^T, stats
  static constexpr int SMEM = 2 * STAGE;
};

template <typename T, int D>
__global__ void __launch_bounds__(BWD_THREADS, 1) flash_bwd_dkdv_kernel(const BwdParams p) {
  typedef TileCfg<D> C;
  typedef Mma16<T> M;
  typedef typename M::frag frag;
  extern __shared__ __align__(16) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63, w = tid >> 6, ln = lane & 31, hh = lane >> 5;

  int bid = blockIdx.x;
  const int h = bid % p.H;
  bid /= p.H;
  const int kt = bid % p.nkt;  // causal: low key tiles see the most query tiles, they go first
  const int b = bid / p.nkt;
  const int k0 = kt * 128;
  const int kw0 = k0 + w * 32;

  const T* qp = (const T*)p.q + b * p.qs.b + h * p.qs.h;
  const T* kp = (const T*)p.k + b * p.ks.b + h * p.ks.h;
  const T* vp = (const T*)p.v + b * p.vs.b + h * p.vs.h;
  const T* dop = (const T*)p.dout + b * p.dos.b + h * p.dos.h;
  const float* lsep = p.lse + ((int64_t)b * p.H + h) * p.Sq;
  const float* delp = p.delta + ((int64_t)b * p.H + h) * p.Sq;

  const int krow = kw0 + ln;
  const int krow_c = krow < p.Sk ? krow : p.Sk - 1;

  frag kf[D / 16], vf[D / 16];
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks) {
    kf[ks] = as_frag<frag>(*(const u32x4*)(kp + (int64_t)krow_c * p.ks.s + ks * 16 + hh * 8));
    vf[ks] = as_frag<frag>(*(const u32x4*)(vp + (int64_t)krow_c * p.vs.s + ks * 16 + hh * 8));
  }
  const float c = p.scale_log2;

  // causal: query rows below the first key of this workgroup see none of its keys
  const int it0 = p.causal ? k0 / BWD_ROWS : 0;
  const int nt = (p.Sq + BWD_ROWS - 1) / BWD_ROWS;

  u32x4 qreg[C::PASS], doreg[C::PASS], qtreg[4], dotreg[4];
  float st_l = 0.f, st_d = 0.f;
  auto gload = [&](int it) {
    const int r0 = it * BWD_ROWS;
    rows_gload<T, D>(qreg, qp, p.qs.s, r0, p.Sq, tid);
    rows_gload<T, D>(doreg, dop, p.dos.s, r0, p.Sq, tid);
    tr_gload<T, D>(qtreg, qp, p.qs.s, r0, p.Sq, tid);
    tr_gload<T, D>(dotreg, dop, p.dos.s, r0, p.Sq, tid);
    if (tid < BWD_ROWS) {
      int r = r0 + tid;
      r = r < p.Sq ? r : p.Sq - 1;
      st_l = lsep[r] * 1.4426950408889634f;
      st_d = delp[r];
    }
  };
  auto lstore = [&](int stage) {
    unsigned char* sb = smem + stage * DkvCfg<D>::STAGE;
    rows_lstore<D>(sb, qreg, tid);
    rows_lstore<D>(sb + C::ROWB, doreg, tid);
    tr_lstore<D>(sb + 2 * C::ROWB, qtreg, tid);
    tr_lstore<D>(sb + 2 * C::ROWB + C::TRB, dotreg, tid);
    if (tid < BWD_ROWS) {
      float* stp = (float*)(sb + 2 * C::ROWB + 2 * C::TRB);
      stp[tid] = st_l;
      stp[BWD_ROWS + tid] = st_d;
    }
  };

  f32x16 dk[D / 32], dv[D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; ++i) {
    zero16(dk[i]);
    zero16(dv[i]);
  }

  if (it0 < nt) {
    gload(it0);
    lstore(it0 & 1);
  }
  __syncthreads();

  for (int it = it0; it < nt; ++it) {
    const int cur = it & 1;
    const int r0 = it * BWD_ROWS;
    const bool more = it + 1 < nt;
    if (more) gload(it + 1);

    // a wave whose keys all come after this query tile contributes nothing to it
    const bool active = !(p.causal && r0 + BWD_ROWS - 1 < kw0);
    if (active) {
      const unsigned char* qb = smem + cur * DkvCfg<D>::STAGE;
      const unsigned char* dob = qb + C::ROWB;
      const unsigned char* qtb = qb + 2 * C::ROWB;
      const unsigned char* dotb = qtb + C::TRB;
      const float* stp = (const float*)(dotb + C::TRB);

      f32x16 s[2], dp[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        zero16(s[t]);
        zero16(dp[t]);
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks) {
          s[t] = M::run(row_frag<frag, D>(qb, t * 32 + ln, ks, hh), kf[ks], s[t]);
          dp[t] = M::run(row_frag<frag, D>(dob, t * 32 + ln, ks, hh), vf[ks], dp[t]);
        }
      }

      frag pf[2][2], dsf[2][2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const f32x4 l4 = *(const f32x4*)(stp + t * 32 + 8 * g + 4 * hh);
          const f32x4 d4 = *(const f32x4*)(stp + BWD_ROWS + t * 32 + 8 * g + 4 * hh);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int v = 4 * g + e;
            const int qi = r0 + t * 32 + 8 * g + 4 * hh + e;  // query row of this accumulator
            const bool dead = qi >= p.Sq || (p.causal && krow > qi);
            const float pr = dead ? 0.f : fast_exp2(__builtin_fmaf(s[t][v], c, -l4[e]));
            s[t][v] = pr;
            dp[t][v] = pr * (dp[t][v] - d4[e]);
          }
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          pf[t][u] = M::pack(s[t][8 * u + 0], s[t][8 * u + 1], s[t][8 * u + 2], s[t][8 * u + 3],
                             s[t][8 * u + 4], s[t][8 * u + 5], s[t][8 * u + 6], s[t][8 * u + 7]);
          dsf[t][u] = M::pack(dp[t][8 * u + 0], dp[t][8 * u + 1], dp[t][8 * u + 2], dp[t][8 * u + 3],
                              dp[t][8 * u + 4], dp[t][8 * u + 5], dp[t][8 * u + 6], dp[t][8 * u + 7]);
        }
      }

#pragma unroll
      for (int db = 0; db < D / 32; ++db)
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int u = 0; u < 2; ++u) {
            dv[db] = M::run(tr_frag<frag, D>(dotb, db * 32 + ln, t, u, hh), pf[t][u], dv[db]);
            dk[db] = M::run(tr_frag<frag, D>(qtb, db * 32 + ln, t, u, hh), dsf[t][u], dk[db]);
          }
    }

    if (more) lstore(cur ^ 1);
    __syncthreads();
  }

  if (krow < p.Sk) {
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

template <typename K>
hipError_t launch(K kernel, int smem, unsigned blocks, const BwdParams& p, hipStream_t stream) {
  hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(BWD_THREADS), smem, stream, p);
  return hipGetLastError();
}

template <typename T, int D>
hipError_t launch_both(const BwdParams& p, hipStream_t stream) {
  const unsigned qblocks = (unsigned)((int64_t)p.B * p.H * p.nqt);
  const unsigned kblocks = (unsigned)((int64_t)p.B * p.H * p.nkt);
  hipError_t e = launch(flash_bwd_dq_kernel<T, D>, DqCfg<D>::SMEM, qblocks, p, stream);
  if (e != hipSuccess) return e;
  return launch(flash_bwd_dkdv_kernel<T, D>, DkvCfg<D>::SMEM, kblocks, p, stream);
}

}  // namespace

// Returns hipSuccess, or hipErrorInvalidValue for an unsupported (dtype, D).
hipError_t spa_launch_flash_bwd(BwdParams p, int D, int dtype, hipStream_t stream) {
  p.nqt = (p.Sq + 127) / 128;
  p.nkt = (p.Sk + 127) / 128;
  if (dtype == 1) {
    if (D == 128) return launch_both<__bf16, 128>(p, stream);
    if (D == 64) return launch_both<__bf16, 64>(p, stream);
    if (D == 32) return launch_both<__bf16, 32>(p, stream);
  } else if (dtype == 2) {
    if (D == 128) return launch_both<_Float16, 128>(p, stream);
    if (D == 64) return launch_both<_Float16, 64>(p, stream);
    if (D == 32) return launch_both<_Float16, 32>(p, stream);
  }
  return hipErrorInvalidValue;
}
