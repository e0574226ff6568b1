// Attention of a handful of query rows over a long K/V (the decode step of a server): the block forward of
// sp_aurora/intel_flash_attn.py:233-296 at Sq <= 3, where the work is reading K and V once.  The MFMA kernels would spend
// a 128-row tile on these rows; here every lane streams 16 bytes of a key row and of a value row per load and the
// scores are plain fused multiply-adds, so that the launch is bound by HBM alone.
//
// Layout of a wave's load: the 64 lanes cover R = 1024 / (D * element size) consecutive key rows, LPR = 64 / R lanes
// a row, lane l holding elements (l % LPR) * E .. + E of row l / LPR (E = 8 for 16-bit, 16 for e4m3 elements).  A
// score is the sum of the LPR lanes' partial dot products (DPP adds inside the 16-lane row); the softmax state
// (running max, running sum, NQ x E accumulators) lives in the group of lanes and covers the rows that group saw.
// At the end the groups of a wave merge by shuffles and the waves of the workgroup through LDS.
//
// Grid: x = batch * head, y = key chunk (the key split of the caller: chunk y writes rows y * Sq .. of the result
// tensors it is given).  256 threads.
#include "spa_common.h"
#include "spa_host.h"

namespace {

constexpr int kWaves = 4;    // waves per workgroup

template <int CTRL>
static __device__ __forceinline__ float dpp_add(float x) {
  const int y = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true);
  return x + __builtin_bit_cast(float, y);
}
// Sum over the LPR (4, 8 or 16) consecutive lanes a key row is spread over; every lane of the group gets it.
template <int LPR>
static __device__ __forceinline__ float group_sum(float x) {
  x = dpp_add<0xB1>(x);                   // quad_perm [1,0,3,2]
  x = dpp_add<0x4E>(x);                   // quad_perm [2,3,0,1]
  if (LPR >= 8) x = dpp_add<0x141>(x);    // row_half_mirror: the other quad of the 8 lanes
  if (LPR >= 16) x = dpp_add<0x140>(x);   // row_mirror: the other half of the 16 lanes
  return x;
}

// 16 bytes of a row as floats.
template <typename T, bool KV8>
struct Piece;
template <typename T>
struct Piece<T, false> {
  static constexpr int E = 8;
  static __device__ __forceinline__ void cvt(u32x4 x, float* f) {
#pragma unroll
    for (int j = 0; j < 4; ++j) Mma16<T>::unpack2(x[j], f[2 * j], f[2 * j + 1]);
  }
};
template <typename T>
struct Piece<T, true> {
  static constexpr int E = 16;
  static __device__ __forceinline__ void cvt(u32x4 x, float* f) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const auto lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)x[j], false);
      const auto hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)x[j], true);
      f[4 * j] = lo[0]; f[4 * j + 1] = lo[1]; f[4 * j + 2] = hi[0]; f[4 * j + 3] = hi[1];
    }
  }
};

// kUnroll: loads of K (and of V) a wave keeps in flight.  NT: the loads carry the non-temporal hint (K and V are read
// once and should not displace anything in the caches).
template <typename T, int D, bool KV8, int NQ, int kUnroll, bool NT>
__global__ void __launch_bounds__(kWaves * 64) fewrows_fwd_kernel(const FwdParams p) {
  constexpr int AUX = NT ? 2 : 0;
  typedef Piece<T, KV8> Pc;
  constexpr int E = Pc::E;
  constexpr int LPR = D / E;        // lanes per key row
  constexpr int R = 64 / LPR;       // key rows per load of a wave
  constexpr int KESZ = KV8 ? 1 : 2;
  static_assert(LPR == 4 || LPR == 8 || LPR == 16, "row spread");

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // Workgroups go to the 8 XCDs round robin.  Where a key row of one head is half a cache line (64 e4m3 elements), two
  // neighbouring heads share every line: they are given to workgroups 8 apart, which run on one XCD at about the same
  // time, so that the line comes from HBM once (3.1 -> 4.6-5.1 TB/s; with rows of a whole line or more the same
  // placement is 3-10 % slower than heads round robin).
  int bh = blockIdx.x;
  if (D * KESZ < 128 && (gridDim.x & 7) == 0) bh = (bh & 7) * (int)(gridDim.x >> 3) + (bh >> 3);
  const int z = blockIdx.y;
  int b = bh / p.H;
  const int h = bh - b * p.H;
  const int c = lane % LPR, g = lane / LPR;
  int k0 = z * p.Sk;
  int k1 = k0 + (z == p.P - 1 ? p.sk_last : p.Sk);
  int nq = NQ;                                   // rows of this (batch or sequence, head) that exist
  int64_t q_row0 = 0, k_row0 = 0;                // first row of the sequence in the packed tensors
  int64_t lse_base = (int64_t)bh * p.lse_bh;     // lse is [B, H, rows], or [H, packed rows] for a packed batch
  if (p.cu_q) {
    // a packed variable-length batch: sequence b owns rows cu_q[b] .. of q / out / lse and cu_k[b] .. of K / V
    // (one chunk: the keys of such a batch are not split)
    q_row0 = p.cu_q[b];
    k_row0 = p.cu_k[b];
    nq = p.cu_q[b + 1] - (int)q_row0;
    nq = nq < NQ ? nq : NQ;
    k0 = 0;
    k1 = p.cu_k[b + 1] - (int)k_row0;
    lse_base = (int64_t)h * p.lse_bh + q_row0;
    b = 0;
    if (nq <= 0) return;
    if (k1 <= 0) {
      // no keys: the empty sum, out = 0 and lse = -inf
      for (int t = threadIdx.x; t < nq * D; t += kWaves * 64) {
        const int i = t / D, d = t - i * D;
        ((T*)p.out)[h * p.os.h + (q_row0 + i) * p.os.s + d] = (T)0.f;
        if (d == 0) p.lse[lse_base + i] = -INFINITY;
      }
      return;
    }
  }

  // the rows' queries, this lane's elements, scaled into the exponent's base-2 domain
  const float qmul = (p.negq ? -p.scale_log2 : p.scale_log2) * (KV8 ? p.k_scale[bh] : 1.f);
  float qf[NQ][E];
#pragma unroll
  for (int i = 0; i < NQ; ++i) {
    const T* qp = (const T*)p.q + b * p.qs.b + h * p.qs.h + (q_row0 + (i < nq ? i : nq - 1)) * p.qs.s + c * E;
#pragma unroll
    for (int e0 = 0; e0 < E; e0 += 8) {
      float t[8];
      Piece<T, false>::cvt(*(const u32x4*)(qp + e0), t);
#pragma unroll
      for (int e = 0; e < 8; ++e) qf[i][e0 + e] = t[e] * qmul;
    }
  }

  // descriptors that end with this chunk's last row: rows past it read as zero and are masked below
  const int64_t krow_b = p.ks.s * KESZ, vrow_b = p.vs.s * KESZ;
  const char* kp = (const char*)p.k + (b * p.ks.b + h * p.ks.h + k_row0 * p.ks.s) * KESZ;
  const char* vp = (const char*)p.v + (b * p.vs.b + h * p.vs.h + k_row0 * p.vs.s) * KESZ;
  const __amdgpu_buffer_rsrc_t krs =
      __builtin_amdgcn_make_buffer_rsrc((void*)kp, 0, (int)((unsigned)((int64_t)(k1 - 1) * krow_b) + D * KESZ), 0x00020000);
  const __amdgpu_buffer_rsrc_t vrs =
      __builtin_amdgcn_make_buffer_rsrc((void*)vp, 0, (int)((unsigned)((int64_t)(k1 - 1) * vrow_b) + D * KESZ), 0x00020000);

  float m[NQ], l[NQ], acc[NQ][E];
#pragma unroll
  for (int i = 0; i < NQ; ++i) {
    m[i] = -INFINITY;
    l[i] = 0.f;
#pragma unroll
    for (int e = 0; e < E; ++e) acc[i][e] = 0.f;
  }

  // The loads of the next pass go out as soon as the registers of this pass are read: K's after the scores, V's after
  // the accumulation, so that half a pass of loads is in flight while the wave computes.
  u32x4 kx[kUnroll], vx[kUnroll];
  const unsigned kcol = (unsigned)(g * krow_b) + c * 16, vcol = (unsigned)(g * vrow_b) + c * 16;
  auto load_k = [&](int row0) {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
      kx[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(krs, (unsigned)((row0 + u * R) * krow_b) + kcol, 0, AUX));
  };
  auto load_v = [&](int row0) {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
      vx[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(vrs, (unsigned)((row0 + u * R) * vrow_b) + vcol, 0, AUX));
  };
  constexpr int kPass = kWaves * kUnroll * R;   // key rows the workgroup takes per pass
  const int first = k0 + wave * (kUnroll * R);
  if (first < k1) {
    load_k(first);
    load_v(first);
  }
  for (int row0 = first; row0 < k1; row0 += kPass) {
    const int row = row0 + g;
    float s[NQ][kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      float kf[E];
      Pc::cvt(kx[u], kf);
      const bool live = row + u * R < k1;
#pragma unroll
      for (int i = 0; i < NQ; ++i) {
        float d = 0.f;
#pragma unroll
        for (int e = 0; e < E; ++e) d = __builtin_fmaf(qf[i][e], kf[e], d);
        d = group_sum<LPR>(d);
        s[i][u] = live ? d : -INFINITY;
      }
    }
    if (row0 + kPass < k1) load_k(row0 + kPass);
#pragma unroll
    for (int i = 0; i < NQ; ++i) {
      float mx = m[i];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) mx = fmaxf(mx, s[i][u]);
      // (row0 < k1 for the wave, but this group's rows may all lie past the end: keep the exponents finite)
      const float ms = mx == -INFINITY ? 0.f : mx;
      const float alpha = __builtin_amdgcn_exp2f(m[i] - ms);
      m[i] = mx;
      l[i] *= alpha;
#pragma unroll
      for (int e = 0; e < E; ++e) acc[i][e] *= alpha;
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        s[i][u] = __builtin_amdgcn_exp2f(s[i][u] - ms);
        l[i] += s[i][u];
      }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      float vf[E];
      Pc::cvt(vx[u], vf);
#pragma unroll
      for (int i = 0; i < NQ; ++i)
#pragma unroll
        for (int e = 0; e < E; ++e) acc[i][e] = __builtin_fmaf(s[i][u], vf[e], acc[i][e]);
    }
    if (row0 + kPass < k1) load_v(row0 + kPass);
  }

  // the R groups of the wave: common max, then sums across the lanes that hold the same elements
  __shared__ float sm_m[NQ][kWaves], sm_l[NQ][kWaves], sm_acc[NQ][kWaves][D];
#pragma unroll
  for (int i = 0; i < NQ; ++i) {
    float mx = m[i];
#pragma unroll
    for (int off = LPR; off < 64; off <<= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
    const float ms = mx == -INFINITY ? 0.f : mx;
    const float w = __builtin_amdgcn_exp2f(m[i] - ms);
    float ls = l[i] * w;
#pragma unroll
    for (int off = LPR; off < 64; off <<= 1) ls += __shfl_xor(ls, off, 64);
#pragma unroll
    for (int e = 0; e < E; ++e) {
      float a = acc[i][e] * w;
#pragma unroll
      for (int off = LPR; off < 64; off <<= 1) a += __shfl_xor(a, off, 64);
      if (g == 0) sm_acc[i][wave][c * E + e] = a;
    }
    if (lane == 0) {
      sm_m[i][wave] = mx;
      sm_l[i][wave] = ls;
    }
  }
  __syncthreads();

  // the waves of the workgroup: thread t takes element t % D of row t / D
  const float vmul = KV8 ? p.v_scale[bh] : 1.f;
  for (int t = threadIdx.x; t < NQ * D; t += kWaves * 64) {
    const int i = t / D, d = t - i * D;
    float mx = sm_m[i][0];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) mx = fmaxf(mx, sm_m[i][w]);
    float ls = 0.f, a = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const float f = __builtin_amdgcn_exp2f(sm_m[i][w] - mx);   // (every chunk holds a key: mx is finite)
      ls += sm_l[i][w] * f;
      a += sm_acc[i][w][d] * f;
    }
    if (i >= nq) break;
    const int64_t orow = (int64_t)z * p.Sq + i;
    T* op = (T*)p.out + b * p.os.b + h * p.os.h + (q_row0 + orow) * p.os.s;
    op[d] = (T)(a * vmul / ls);
    if (d == 0) p.lse[lse_base + orow] = (mx + __builtin_amdgcn_logf(ls)) * 0.6931471805599453f;
  }
}

// Measured on twelve decode shapes: four loads in flight beat eight (6-10 %) except with three rows and with 64-byte
// rows; the non-temporal hint gains 5-15 % on 16-bit K/V and on e4m3 rows of a whole line when the keys are not split,
// and loses where neighbouring workgroups share lines (64-byte rows) and on split e4m3 calls.
template <typename T, int D, bool KV8, int NQ, int U>
hipError_t launch_variant(const FwdParams& p, hipStream_t stream) {
  const dim3 grid((unsigned)(p.B * p.H), (unsigned)p.P), block(kWaves * 64);
  if constexpr (!KV8) {
    hipLaunchKernelGGL((fewrows_fwd_kernel<T, D, KV8, NQ, U, true>), grid, block, 0, stream, p);
  } else if constexpr (D == 64) {
    hipLaunchKernelGGL((fewrows_fwd_kernel<T, D, KV8, NQ, U, false>), grid, block, 0, stream, p);
  } else if (p.P == 1) {
    hipLaunchKernelGGL((fewrows_fwd_kernel<T, D, KV8, NQ, U, true>), grid, block, 0, stream, p);
  } else {
    hipLaunchKernelGGL((fewrows_fwd_kernel<T, D, KV8, NQ, U, false>), grid, block, 0, stream, p);
  }
  return hipGetLastError();
}

// A launch that leaves half of the CUs without a workgroup (a caller who did not split the keys) is bound by what its
// few waves keep in flight: eight loads there too.
template <typename T, int D, bool KV8, int NQ>
hipError_t launch_unroll(const FwdParams& p, hipStream_t stream) {
  constexpr int U = NQ == 3 || (KV8 && D == 64) ? 8 : 4;
  if constexpr (U != 8) {
    if ((int64_t)p.B * p.H * p.P * 2 <= spa_device_cus()) return launch_variant<T, D, KV8, NQ, 8>(p, stream);
  }
  return launch_variant<T, D, KV8, NQ, U>(p, stream);
}

template <typename T, int D, bool KV8>
hipError_t launch_nq(const FwdParams& p, hipStream_t stream) {
  switch (p.Sq) {
    case 1: return launch_unroll<T, D, KV8, 1>(p, stream);
    case 2: return launch_unroll<T, D, KV8, 2>(p, stream);
    case 3: return launch_unroll<T, D, KV8, 3>(p, stream);
    default: return hipErrorInvalidValue;
  }
}

template <typename T>
hipError_t launch_t(const FwdParams& p, int D, hipStream_t stream) {
  const bool kv8 = p.k_scale != nullptr;
  if (D == 128) return kv8 ? launch_nq<T, 128, true>(p, stream) : launch_nq<T, 128, false>(p, stream);
  if (D == 64) return kv8 ? launch_nq<T, 64, true>(p, stream) : launch_nq<T, 64, false>(p, stream);
  return hipErrorInvalidValue;
}

}  // namespace

// The caller's FwdParams as for the key-split launch: Sk = keys per chunk, sk_last = keys of the last chunk, P = number of
// chunks; out / lse take rows z * Sq + i of chunk z.  No mask, 1 <= Sq <= 3, 16-bit q / out, K/V of one
// (batch, head) below 2 GiB, 16-byte aligned K/V rows.  A packed variable-length batch (cu_q, cu_k; Sq = the longest
// sequence's rows, B = sequences) runs as one chunk.
hipError_t spa_launch_fwd_fewrows(FwdParams p, int D, int dtype, hipStream_t stream) {
  if (p.causal || (p.cu_q && p.P != 1) || p.q_scale || p.big || p.Sq < 1 || p.Sq > 3 || p.P < 1 || p.P > 65535) return hipErrorInvalidValue;
  if (dtype == 1) return launch_t<__bf16>(p, D, stream);
  if (dtype == 2) return launch_t<_Float16>(p, D, stream);
  return hipErrorInvalidValue;
}
