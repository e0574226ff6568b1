// Shared device-side types and helpers for the sp_aurora HIP kernels (gfx950).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef int i32x8 __attribute__((ext_vector_type(8)));

struct Strides3 {
  int64_t b, h, s;  // element strides of (batch, head, seq); head-dim stride is 1
};

struct FwdParams {
  const void* q;
  const void* k;
  const void* v;
  void* out;
  float* lse;
  int B, H, Sq, Sk;
  Strides3 qs, ks, vs, os;
  float scale;       // softmax scale
  float scale_log2;  // |scale| * log2(e): the forward kernels take the row max on raw scores, so a
                     // negative scale travels as negq (q is negated on its way into registers)
  int negq;
  int causal;        // 1: query row i sees keys j <= i (top-left aligned)
  int nqt;           // number of query tiles per (batch, head)
  int64_t lse_bh;    // elements between consecutive (batch, head) rows of lse
  // ring schedule (16-bit kernels): K/V hold P chunks of Sk keys, q/out/lse hold P chunks of Sq
  // rows; the launch runs ranks rank0 .. rank0+nranks-1, each over steps [t_begin, t_begin+t_count)
  // of its schedule (t_count < 0: to the end).  A plain block call is P = 1, rank 0, all steps.
  int P, rank0, nranks, t_begin, t_count;
  // ring-step epilogue (16-bit kernels): what happens to the block result.  The results of a
  // rank's earlier steps wait in slots at `part` (see RingSlots): slot j holds step j's block
  // output in q's element type, contiguous [B,Sq,H,D], and its lse, [B*H,Sq] fp32.
  // Only the kernels for a rank's last step read part and npart; part_slot and epi are for the host.
  void* part;
  int part_slot;     // SPA_EPI_PART: the slot this step fills (the launcher points out / lse at it)
  int npart;         // SPA_EPI_FINALN: slots 0 .. npart-1 are merged, in that order, then this step's block
  int epi;
  // variable-length batch (null: every sequence has Sq queries and Sk keys): sequence b owns rows
  // cu_q[b] .. cu_q[b+1] of q/out/lse and cu_k[b] .. cu_k[b+1] of k/v, batch strides are unused,
  // Sq and Sk are the longest sequence's sizes (they shape the grid) and lse is [H][lse_bh]
  const int* cu_q;
  const int* cu_k;
  // e4m3 K/V (16-bit kernels; null: K and V have q's element type): K = k8 * k_scale[b*H + h],
  // V = v8 * v_scale[b*H + h], fp32, one per (batch or sequence, head); strides of k, v in bytes
  const float* k_scale;
  const float* v_scale;
  // e4m3 q as well (null: q has the type of out): Q = q8 * q_scale[b*H + h]; strides of q in bytes
  const float* q_scale = nullptr;
  // zigzag sharding of a causal ring (16-bit kernels; 0: contiguous chunks): the chunk of rank r holds
  // half-chunks r and 2P-1-r of the sequence, Sq/2 rows each.  Step 0 is plain causal attention on the
  // rank's own chunk; at step t >= 1 (chunk c = (r - t) mod P) every local query sees the first half of
  // the chunk when c < r, and only the second half of the queries sees anything, the whole chunk, when
  // c > r.  Query tiles never straddle the two halves.  zz_half = 1: the launch covers the tiles of
  // the second half only (a step with c > r that is not the rank's last).
  int zigzag = 0;
  int zz_half = 0;
  // Chunk arrival flags (the variants for a ring rank whose K/V chunks land while its one launch runs): before a
  // workgroup loads the first tile of chunk c it waits until arrive[c] >= epoch (an acquire load at system scope in
  // a bounded spin: after spin_limit polls the wave gives up, sets *fault = 1 and goes on, so the grid always drains).
  const unsigned* arrive = nullptr;
  unsigned epoch = 0;
  unsigned spin_limit = 0;
  unsigned* fault = nullptr;
  // K / V rows of one (batch, head) span 2 GiB or more: the launcher takes the kernel variants that re-base their
  // buffer descriptors per tile (16-bit kernels; the fp32 kernels address with 64-bit pointers anyway)
  int big = 0;
  // Keys split over grid.z for calls with few query rows (the KS variants): K / V hold P chunks of Sk keys, the last
  // one sk_last keys; plane z computes the block (all Sq query rows) x (chunk z) and writes it to rows z * Sq .. of out / lse.
  int sk_last = 0;
  // A ring over a packed variable-length batch (cu_q set, P > 1): the tensors are P stacked shards of chunk_rows rows,
  // every shard packed as cu_q says, so chunk c of a sequence's keys starts chunk_rows rows after chunk c - 1 and rank
  // r's queries rank_rows rows after rank r - 1's (0: chunks and ranks follow each other, Sk and Sq rows apart).
  int chunk_rows = 0;
  int rank_rows = 0;
};

// Layout of the ring-step slots of one rank in the caller's workspace (16-bit inputs, ring of P):
// P - 1 output slots of out_bytes each, then P - 1 lse slots of lse_bytes each; host and kernels
// derive it from the sizes.
struct RingSlots {
  int64_t out_bytes, lse_bytes;
  __host__ __device__ RingSlots(int B, int H, int64_t s, int D)
      : out_bytes(((int64_t)B * s * H * D * 2 + 255) / 256 * 256), lse_bytes(((int64_t)B * H * s * 4 + 255) / 256 * 256) {}
  __host__ __device__ int64_t total(int P) const { return (int64_t)(P - 1) * (out_bytes + lse_bytes); }
  template <typename T>
  __host__ __device__ T* out(void* part, int j) const { return (T*)((char*)part + j * out_bytes); }
  __host__ __device__ float* lse(void* part, int P, int j) const { return (float*)((char*)part + (P - 1) * out_bytes + j * lse_bytes); }
};

enum {
  SPA_EPI_PLAIN = 0,   // out <- block, lse <- block lse
  SPA_EPI_PART = 1,    // slot part_slot <- (block rounded to q's type, block lse): a step that is not the rank's last
  SPA_EPI_FINALN = 2   // (out, lse) <- the slots merged one after the other (fp32, sp_aurora/utils.py:103-104), then
                       // this step's block: the rank's last step
};

struct BwdParams {
  const void* q;
  const void* k;
  const void* v;
  const void* dout;
  const float* lse;
  const float* delta;
  float* dq;
  float* dk;
  float* dv;
  int B, H, Sq, Sk;
  Strides3 qs, ks, vs, dos, dqs, dks, dvs;
  float scale;
  float scale_log2;
  int causal;
  int nqt;  // number of query tiles per (batch, head)
  int nkt;  // number of key tiles per (batch, head)
  int64_t lse_bh;  // elements between consecutive (batch, head) rows of lse and delta
  // variable-length batch, as in FwdParams: rows cu_q[b] .. cu_q[b+1] of q/dout/dq/lse/delta and
  // cu_k[b] .. cu_k[b+1] of k/v/dk/dv belong to sequence b; lse and delta are [H][lse_bh]
  const int* cu_q;
  const int* cu_k;
  // 0: dq/dk/dv are fp32 accumulators, added to; 1: they are tensors of q's element type (strides in
  // those elements) and are WRITTEN: the whole gradient comes from this one launch
  int grads_in_t;
  // some tensor's rows of one (batch, head) span 2 GiB or more (see FwdParams::big)
  int big = 0;
};

// 16-bit element traits: MFMA 32x32x16 with 8 elements per lane per operand.
template <typename T>
struct Mma16;

template <>
struct Mma16<__bf16> {
  typedef bf16x8 frag;
  static __device__ __forceinline__ f32x16 run(frag a, frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ frag pack(float x0, float x1, float x2, float x3,
                                              float x4, float x5, float x6, float x7) {
    frag r;
    r[0] = (__bf16)x0; r[1] = (__bf16)x1; r[2] = (__bf16)x2; r[3] = (__bf16)x3;
    r[4] = (__bf16)x4; r[5] = (__bf16)x5; r[6] = (__bf16)x6; r[7] = (__bf16)x7;
    return r;
  }
  static __device__ __forceinline__ unsigned pack2(float lo, float hi) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    bf16x2 r;
    r[0] = (__bf16)lo; r[1] = (__bf16)hi;
    return __builtin_bit_cast(unsigned, r);
  }
  static __device__ __forceinline__ void unpack2(unsigned x, float& lo, float& hi) {
    lo = __builtin_bit_cast(float, x << 16);
    hi = __builtin_bit_cast(float, x & 0xffff0000u);
  }
};

template <>
struct Mma16<_Float16> {
  typedef f16x8 frag;
  static __device__ __forceinline__ f32x16 run(frag a, frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ frag pack(float x0, float x1, float x2, float x3,
                                              float x4, float x5, float x6, float x7) {
    frag r;
    r[0] = (_Float16)x0; r[1] = (_Float16)x1; r[2] = (_Float16)x2; r[3] = (_Float16)x3;
    r[4] = (_Float16)x4; r[5] = (_Float16)x5; r[6] = (_Float16)x6; r[7] = (_Float16)x7;
    return r;
  }
  static __device__ __forceinline__ unsigned pack2(float lo, float hi) {
    typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
    f16x2 r;
    r[0] = (_Float16)lo; r[1] = (_Float16)hi;
    return __builtin_bit_cast(unsigned, r);
  }
  static __device__ __forceinline__ void unpack2(unsigned x, float& lo, float& hi) {
    typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
    const f16x2 r = __builtin_bit_cast(f16x2, x);
    lo = (float)r[0];
    hi = (float)r[1];
  }
};

template <typename F>
static __device__ __forceinline__ F as_frag(u32x4 x) {
  return __builtin_bit_cast(F, x);
}

// The two lanes 32 apart share a row of a 32x32 accumulator tile.  v_permlane32_swap hands every
// lane both of them: the value of lane l % 32 and that of lane 32 + l % 32 (one VALU instruction,
// no LDS round trip).  The second operand goes through an empty asm so that the compiler sees two
// distinct registers.
static __device__ __forceinline__ void both_halves(float x, float& lo, float& hi) {
  float y = x;
  asm volatile("" : "+v"(y));
  const auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(unsigned, x), __builtin_bit_cast(unsigned, y), false, false);
  const unsigned u0 = r[0], u1 = r[1];
  lo = __builtin_bit_cast(float, u0);
  hi = __builtin_bit_cast(float, u1);
}
static __device__ __forceinline__ float halves_max(float x) {
  float lo, hi;
  both_halves(x, lo, hi);
  return fmaxf(lo, hi);
}
static __device__ __forceinline__ float halves_sum(float x) {
  float lo, hi;
  both_halves(x, lo, hi);
  return lo + hi;
}

// ---- LDS helpers shared by the attention kernels ----
typedef __attribute__((address_space(3))) unsigned char lds_u8;
typedef short s16x4 __attribute__((ext_vector_type(4)));

// 16 bytes per lane from a buffer straight into LDS at lds_addr + 16 * lane (lds_addr wave-uniform);
// out-of-range lanes store zeros.  Counts on vmcnt like any load.  Issued from inline asm: the
// compiler knows nothing of it, so the caller orders it against LDS reads (vmcnt wait + barrier).
static __device__ __forceinline__ void load_to_lds_b128(u32x4 rsrc, unsigned voffset, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
               :
               : "s"(lds_addr), "v"(voffset), "s"(rsrc)
               : "memory");
}
// The same with the non-temporal hint: for tiles that no other workgroup reads.
static __device__ __forceinline__ void load_to_lds_b128_nt(u32x4 rsrc, unsigned voffset, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen nt lds"
               :
               : "s"(lds_addr), "v"(voffset), "s"(rsrc)
               : "memory");
}
// The same for 4 bytes per lane: LDS at lds_addr + 4 * lane.
static __device__ __forceinline__ void load_to_lds_b32(u32x4 rsrc, unsigned voffset, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, 0 offen lds"
               :
               : "s"(lds_addr), "v"(voffset), "s"(rsrc)
               : "memory");
}
// Raw buffer descriptor (stride 0) over `bytes` bytes at base; every component wave-uniform.
static __device__ __forceinline__ u32x4 buffer_descriptor(const void* base, unsigned bytes) {
  const unsigned long long a = (unsigned long long)base;
  u32x4 r;
  r[0] = __builtin_amdgcn_readfirstlane((unsigned)a);
  r[1] = __builtin_amdgcn_readfirstlane((unsigned)(a >> 32) & 0xffffu);
  r[2] = __builtin_amdgcn_readfirstlane(bytes);
  r[3] = 0x00020000u;
  return r;
}
// For tensors whose rows of one (batch, head) span 2 GiB or more, beyond what a 32-bit per-lane offset with its
// sign bit spare can address: a descriptor over the part of the tensor that starts at the 1 GiB boundary below
// byte offset `off` (wave-uniform) and `rel`, the offset inside that window (< 1 GiB; the lanes add less than
// 1 GiB to it).  The hardware range check still ends at the tensor's last byte when that lies within 4 GiB of the
// window's start, and beyond that every offset a lane can form is inside the tensor.
static __device__ __forceinline__ u32x4 buffer_window(const void* base, unsigned long long total, unsigned long long off,
                                                      unsigned& rel) {
  const unsigned long long w = off & ~0x3fffffffULL;
  rel = __builtin_amdgcn_readfirstlane((unsigned)(off - w));
  const unsigned long long left = total > w ? total - w : 0ULL;
  return buffer_descriptor((const char*)base + w, left > 0xffffffffULL ? 0xffffffffu : (unsigned)left);
}

// Transposing LDS read: in a block of 16 lanes, lane 4 e + c supplies the address of 8 bytes
// (4 elements) of row e, and lane x receives element x (of the 16 the row's four pieces hold)
// of rows 0..3.
static __device__ __forceinline__ u32x2 lds_read_tr16_b64(unsigned lds_addr) {
  return __builtin_bit_cast(
      u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(lds_u8*)(uintptr_t)lds_addr));
}
static __device__ __forceinline__ u32x4 lds_read_b128(unsigned lds_addr) {
  return *(const __attribute__((address_space(3))) u32x4*)(lds_u8*)(uintptr_t)lds_addr;
}

static __device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
static __device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }
