// extern "C" boundary of libsp_aurora_hip.so: argument checks, then a launch.
// No allocation, no synchronisation, no torch types; errors are codes plus a
// thread-local message.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "../../include/sp_aurora_hip.h"
#include "spa_common.h"
#include "spa_host.h"

std::atomic<int> g_spa_knob[SPA_KNOB_COUNT];

// Scratch of spa_ring_fwd_static: lives in the code object, one copy per device the library is
// loaded on, from load to process end.  The name below is a host-side handle only; kernels and
// copies get the device address hipGetSymbolAddress returns for the current device.
static __device__ __align__(256) unsigned char scratch[SPA_STATIC_SCRATCH_BYTES];

hipError_t spa_launch_flash_fwd(FwdParams p, int D, int dtype, hipStream_t stream);
hipError_t spa_launch_fwd16_splitkv(FwdParams p, int D, int dtype, hipStream_t stream);
hipError_t spa_launch_fwd_fewrows(FwdParams p, int D, int dtype, hipStream_t stream);
hipError_t spa_launch_splitkv_combine(void* out, float* lse, const void* part, const float* part_lse, int n, int B, int H, int Sq,
                                      int D, Strides3 os, int64_t lse_bh, int dtype, hipStream_t stream);
hipError_t spa_launch_flash_bwd(BwdParams p, int D, int dtype, hipStream_t stream);
hipError_t spa_launch_merge(float* out_acc, float* lse_acc, const void* blk_out, const float* blk_lse, int B,
                            int H, int Sq, int D, Strides3 as, Strides3 bs, int dtype, int init,
                            int64_t acc_lse_bh, hipStream_t stream);
hipError_t spa_launch_finalize(void* out, const float* out_acc, int B, int H, int Sq, int D, Strides3 os,
                               Strides3 as, int dtype, hipStream_t stream);
hipError_t spa_launch_delta(const void* out, const void* dout, float* delta, int B, int H, int Sq, int D,
                            Strides3 os, Strides3 ds, int dtype, hipStream_t stream);
hipError_t spa_launch_relayout(const void* src, void* dst, int P, int B, int s, int H, int D, int pack,
                               int elem_bytes, bool s2h, hipStream_t stream);

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int elem_size(int dtype) { return dtype == SPA_F32 ? 4 : 2; }

bool dtype_ok(int dtype) { return dtype == SPA_F32 || dtype == SPA_BF16 || dtype == SPA_F16; }

Strides3 S3(const int64_t* s) {
  Strides3 r;
  r.b = s[0]; r.h = s[1]; r.s = s[2];
  return r;
}

// 16-byte alignment of the base pointer and of every row start.
bool aligned16(const void* p, const int64_t* s, int esz) {
  if (((uintptr_t)p & 15) != 0) return false;
  for (int i = 0; i < 3; ++i)
    if ((s[i] * esz) % 16 != 0) return false;
  return true;
}

// The largest element offset a (B,H,S,D) view touches must fit what the kernels index.
bool dims_ok(int B, int H, int S, int D) { return B > 0 && H > 0 && S > 0 && D > 0; }

bool pow2_8_512(int D) { return D >= 8 && D <= 512 && (D & (D - 1)) == 0; }

// The 16-bit kernels address the streamed tensors of one (batch, head) through buffer descriptors with 32-bit
// per-lane offsets: below 2 GiB one descriptor covers the tensor (span_ok); beyond, the variants that re-base
// the descriptor per tile take over, which need a tile of 128 rows to stay below 1 GiB (span_rebasable).
bool span_ok(int64_t rows, int64_t row_stride, int D, int esz) {
  return ((rows - 1) * row_stride + D) * esz < 0x7fffffffLL;
}
bool span_rebasable(int64_t row_stride, int esz) { return row_stride * esz * 128 < 0x40000000LL; }
// Can K / V that span 2 GiB or more be run?  fp32: yes (those kernels address with 64-bit pointers); e4m3: no
// (no re-based variants); 16-bit: when both row strides allow re-basing.  Returns null or what is in the way.
const char* big_kv_obstacle(bool kv8, int dtype, int64_t k_row_stride, int64_t v_row_stride, int esz) {
  if (kv8) return "not supported for e4m3 K/V";
  if (dtype == SPA_F32) return nullptr;
  return span_rebasable(k_row_stride, esz) && span_rebasable(v_row_stride, esz) ? nullptr : "and 128 rows of them 1 GiB or more";
}

// Any finite softmax scale, as in the reference.  Zero is carried as 1e-30: every finite score then
// scales to (practically) zero while a hidden score stays at -inf instead of becoming inf * 0;
// the results differ from exact arithmetic by less than 1e-25.
bool scale_ok(float scale) { return scale == scale && scale > -INFINITY && scale < INFINITY; }
float scale_eff(float scale) { return scale == 0.f ? 1e-30f : scale; }

int launch_result(hipError_t e, const char* what) {
  if (e == hipSuccess) return SPA_OK;
  if (e == hipErrorInvalidValue) return fail(SPA_EUNSUPPORTED, "%s: no kernel for this head dim / dtype", what);
  return fail(SPA_ELAUNCH, "%s: %s", what, hipGetErrorString(e));
}

}  // namespace

extern "C" {

int spa_abi_version(void) { return SPA_ABI_VERSION; }

const char* spa_last_error(void) { return g_err; }

int spa_device_info(char* buf, int n) {
  if (!buf || n <= 0) return fail(SPA_EINVAL, "spa_device_info: null buffer");
  int dev = 0;
  hipDeviceProp_t prop;
  hipError_t e = hipGetDevice(&dev);
  if (e == hipSuccess) e = hipGetDeviceProperties(&prop, dev);
  if (e != hipSuccess) return fail(SPA_ELAUNCH, "spa_device_info: %s", hipGetErrorString(e));
  snprintf(buf, n, "name=%s;arch=%s;cus=%d;lds=%zu;clock_khz=%d;mem_clock_khz=%d;bus_bits=%d;hbm=%zu", prop.name,
           prop.gcnArchName, prop.multiProcessorCount, prop.maxSharedMemoryPerMultiProcessor, prop.clockRate,
           prop.memoryClockRate, prop.memoryBusWidth, prop.totalGlobalMem);
  return SPA_OK;
}

}  // extern "C"

namespace {

// 8-byte alignment of an e4m3 tensor's base and rows (a thread moves 8 elements at a time).
bool aligned8(const void* p, const int64_t* s, int n) {
  if (((uintptr_t)p & 7) != 0) return false;
  for (int i = 0; i < n; ++i)
    if (s[i] % 8 != 0) return false;
  return true;
}

// The key-split forward: how the keys are cut for a wanted number of chunks (chunks of a multiple of 128 keys, the
// last one what is left), and the scratch the chunks' results need.
constexpr int kFewRows = 3;   // query rows the K/V-streaming kernel takes (spa_launch_fwd_fewrows)
struct KeySplit {
  int n, chunk, last;
  KeySplit(int Sk, int nsplit) {
    chunk = nsplit > 1 ? (int)((((int64_t)Sk + nsplit - 1) / nsplit + 127) / 128 * 128) : Sk;
    n = (Sk + chunk - 1) / chunk;
    last = Sk - (n - 1) * chunk;
  }
};
int64_t splitkv_out_bytes(int B, int H, int Sq, int D, int n, int esz) { return ((int64_t)B * n * Sq * H * D * esz + 255) / 256 * 256; }

// k_scale / v_scale non-null: K and V are e4m3 bytes (strides in bytes), q / out of type `dtype`.
// nsplit >= 1 (the key-split entry points; a workspace when more than one chunk comes of it): the keys are cut into
// chunks that run side by side on the same query rows.
int flash_fwd(const char* what, const void* q, const void* k, const void* v, const float* k_scale, const float* v_scale,
              void* out, float* lse, int B, int H, int Sq, int Sk, int D, const int64_t q_strides[3],
              const int64_t k_strides[3], const int64_t v_strides[3], const int64_t o_strides[3], float scale,
              int mask_mode, int dtype, void* stream, void* workspace = nullptr, int nsplit = 0) {
  const bool workspace_call = nsplit >= 1;   // one of the key-split entry points
  const bool kv8 = k_scale || v_scale;
  if (!q || !k || !v || !out || !lse) return fail(SPA_EINVAL, "%s: null pointer", what);
  if (kv8 && (!k_scale || !v_scale)) return fail(SPA_EINVAL, "%s: null scale pointer", what);
  if (!q_strides || !k_strides || !v_strides || !o_strides) return fail(SPA_EINVAL, "%s: null strides", what);
  if (!dims_ok(B, H, Sq, D) || Sk <= 0) return fail(SPA_EINVAL, "%s: sizes must be positive (B=%d H=%d Sq=%d Sk=%d D=%d)", what, B, H, Sq, Sk, D);
  if (!dtype_ok(dtype)) return fail(SPA_EINVAL, "%s: bad dtype %d", what, dtype);
  if (kv8 && dtype == SPA_F32) return fail(SPA_EUNSUPPORTED, "%s: e4m3 K/V go with bf16 or fp16 queries", what);
  if (mask_mode != SPA_MASK_NONE && mask_mode != SPA_MASK_CAUSAL) return fail(SPA_EINVAL, "%s: bad mask_mode %d", what, mask_mode);
  if (!scale_ok(scale)) return fail(SPA_EINVAL, "%s: softmax scale must be finite", what);
  if (D != 32 && D != 64 && D != 128) return fail(SPA_EUNSUPPORTED, "%s: head dim %d not in {32,64,128}", what, D);
  if (kv8 && D == 32) return fail(SPA_EUNSUPPORTED, "%s: e4m3 K/V need head dim 64 or 128", what);
  const int esz = elem_size(dtype), kesz = kv8 ? 1 : esz;
  const bool kv_aligned = kv8 ? aligned8(k, k_strides, 3) && aligned8(v, v_strides, 3) && (((uintptr_t)k_scale | (uintptr_t)v_scale) & 3) == 0
                              : aligned16(k, k_strides, esz) && aligned16(v, v_strides, esz);
  if (!aligned16(q, q_strides, esz) || !kv_aligned || !aligned16(out, o_strides, esz) || ((uintptr_t)lse & 3) != 0)
    return fail(SPA_EALIGN, "%s: pointers and row strides must be 16-byte aligned (8-byte for e4m3 K/V)", what);
  if ((int64_t)B * H > 0x7fffffffLL || (Sq + 127) / 128 > 65535) return fail(SPA_EINVAL, "%s: grid too large", what);
  const bool big = !span_ok(Sk, k_strides[2], D, kesz) || !span_ok(Sk, v_strides[2], D, kesz);
  if (big && big_kv_obstacle(kv8, dtype, k_strides[2], v_strides[2], esz))
    return fail(SPA_EUNSUPPORTED, "%s: K/V of one (batch, head) span 2 GiB or more (%s)", what,
                big_kv_obstacle(kv8, dtype, k_strides[2], v_strides[2], esz));
  FwdParams p;
  p.big = big && dtype != SPA_F32;
  p.q = q; p.k = k; p.v = v; p.out = out; p.lse = lse;
  p.B = B; p.H = H; p.Sq = Sq; p.Sk = Sk;
  p.qs = S3(q_strides); p.ks = S3(k_strides); p.vs = S3(v_strides); p.os = S3(o_strides);
  p.scale = scale_eff(scale);
  p.scale_log2 = fabsf(scale_eff(scale)) * 1.4426950408889634f;
  p.negq = scale < 0.f;
  p.causal = mask_mode == SPA_MASK_CAUSAL;
  p.nqt = 0;
  p.lse_bh = Sq;
  p.part = nullptr; p.part_slot = 0; p.npart = 0;
  p.epi = SPA_EPI_PLAIN;
  p.P = 1; p.rank0 = 0; p.nranks = 1; p.t_begin = 0; p.t_count = -1;
  p.cu_q = nullptr; p.cu_k = nullptr;
  p.k_scale = k_scale; p.v_scale = v_scale;
  {
    if (nsplit > 1024) return fail(SPA_EINVAL, "%s: nsplit %d above 1024", what, nsplit);
    const KeySplit ks(Sk, workspace_call ? nsplit : 1);
    const bool can = !p.causal && dtype != SPA_F32 && D != 32 && !p.big;
    if (ks.n > 1) {
      if (p.causal) return fail(SPA_EUNSUPPORTED, "%s: the keys are split for calls without a mask", what);
      if (!can) return fail(SPA_EUNSUPPORTED, "%s: built for bf16 / fp16, head dim 64 or 128, K/V below 2 GiB per (batch, head)", what);
      if (!workspace || ((uintptr_t)workspace & 15) != 0) return fail(SPA_EINVAL, "%s: the key split needs a 16-byte aligned workspace", what);
    }
    // Up to kFewRows query rows without a mask, split or not: the kernel that streams K and V past them (16 bytes a lane,
    // so e4m3 rows must be 16-byte aligned as well); more rows, or spa_tune(SPA_TUNE_FEW_ROWS, 1): the MFMA kernels (for a
    // split with the chunks as grid planes).
    const bool few = can && Sq <= kFewRows && spa_knob(SPA_KNOB_FEW_ROWS) != 1 &&
                     (!kv8 || (aligned16(k, k_strides, 1) && aligned16(v, v_strides, 1)));
    if (ks.n > 1 || few) {
      p.Sk = ks.chunk; p.sk_last = ks.last;
      p.P = ks.n; p.rank0 = 0; p.nranks = ks.n; p.t_begin = 0; p.t_count = 1;
      char* part_out = (char*)workspace;
      float* part_lse = ks.n > 1 ? (float*)(part_out + splitkv_out_bytes(B, H, Sq, D, nsplit, esz)) : nullptr;
      if (ks.n > 1) {
        // plane z writes rows z * Sq .. of the scratch tensors [B, n * Sq, H, D] and [B, H, n * Sq]
        p.out = part_out; p.lse = part_lse;
        p.os.b = (int64_t)ks.n * Sq * H * D; p.os.s = (int64_t)H * D; p.os.h = D;
        p.lse_bh = (int64_t)ks.n * Sq;
      }
      hipError_t e = few ? spa_launch_fwd_fewrows(p, D, dtype, (hipStream_t)stream) : spa_launch_fwd16_splitkv(p, D, dtype, (hipStream_t)stream);
      if (e == hipSuccess && ks.n > 1)
        e = spa_launch_splitkv_combine(out, lse, part_out, part_lse, ks.n, B, H, Sq, D, S3(o_strides), Sq, dtype, (hipStream_t)stream);
      return launch_result(e, what);
    }
  }
  return launch_result(spa_launch_flash_fwd(p, D, dtype, (hipStream_t)stream), what);
}

}  // namespace

extern "C" {

int spa_flash_fwd(const void* q, const void* k, const void* v, void* out, float* lse, int B, int H, int Sq,
                  int Sk, int D, const int64_t q_strides[3], const int64_t k_strides[3],
                  const int64_t v_strides[3], const int64_t o_strides[3], float scale, int mask_mode,
                  int dtype, void* stream) {
  return flash_fwd("spa_flash_fwd", q, k, v, nullptr, nullptr, out, lse, B, H, Sq, Sk, D, q_strides, k_strides, v_strides,
                   o_strides, scale, mask_mode, dtype, stream);
}

int spa_flash_fwd_fp8kv(const void* q, const void* k8, const void* v8, const float* k_scale, const float* v_scale,
                        void* out, float* lse, int B, int H, int Sq, int Sk, int D, const int64_t q_strides[3],
                        const int64_t k_strides[3], const int64_t v_strides[3], const int64_t o_strides[3],
                        float scale, int mask_mode, int dtype, void* stream) {
  if (!k_scale || !v_scale) return fail(SPA_EINVAL, "spa_flash_fwd_fp8kv: null scale pointer");
  return flash_fwd("spa_flash_fwd_fp8kv", q, k8, v8, k_scale, v_scale, out, lse, B, H, Sq, Sk, D, q_strides, k_strides,
                   v_strides, o_strides, scale, mask_mode, dtype, stream);
}

int64_t spa_flash_fwd_splitkv_workspace_bytes(int B, int H, int Sq, int D, int nsplit, int dtype) {
  if (B <= 0 || H <= 0 || Sq <= 0 || D <= 0 || nsplit < 1 || (dtype != SPA_BF16 && dtype != SPA_F16)) return -1;
  return splitkv_out_bytes(B, H, Sq, D, nsplit, 2) + (int64_t)B * H * nsplit * Sq * 4;
}

int spa_flash_fwd_splitkv_suggest(int B, int H, int Sq, int Sk, int D, int mask_mode, int dtype) {
  if (B <= 0 || H <= 0 || Sq <= 0 || Sk <= 0 || mask_mode != SPA_MASK_NONE || (dtype != SPA_BF16 && dtype != SPA_F16) || (D != 64 && D != 128))
    return 1;
  const int cus = spa_device_cus();
  // Up to kFewRows query rows run on the kernel that streams K and V: one workgroup per CU measured best on ten decode
  // shapes (more chunks: 3 to 15 % slower), chunks of at least 512 keys.
  if (Sq <= kFewRows && spa_knob(SPA_KNOB_FEW_ROWS) != 1) {
    if (Sk < 1024) return 1;
    int64_t n = ((int64_t)cus + (int64_t)B * H / 2) / ((int64_t)B * H);
    if (n > Sk / 512) n = Sk / 512;
    if (n > 64) n = 64;
    return n < 2 ? 1 : KeySplit(Sk, (int)n).n;
  }
  // Otherwise worth it when the 128-row workgroups of the plain launch leave at least half of the CUs idle and every
  // chunk keeps at least 512 keys: as many chunks as give every CU one workgroup (measured on six decode shapes: more
  // chunks only add the workgroups' fixed cost and rows for the merge).
  const int64_t wgs = (int64_t)B * H * ((Sq + 127) / 128);
  if (wgs * 2 > cus || Sk < 2048) return 1;
  int64_t n = ((int64_t)cus + wgs / 2) / wgs;
  if (n > Sk / 512) n = Sk / 512;
  if (n > 64) n = 64;
  return n < 2 ? 1 : KeySplit(Sk, (int)n).n;
}

int spa_flash_fwd_splitkv(const void* q, const void* k, const void* v, void* out, float* lse, void* workspace, int B, int H, int Sq,
                          int Sk, int D, int nsplit, const int64_t q_strides[3], const int64_t k_strides[3],
                          const int64_t v_strides[3], const int64_t o_strides[3], float scale, int dtype, void* stream) {
  if (nsplit < 1) return fail(SPA_EINVAL, "spa_flash_fwd_splitkv: nsplit must be positive");
  return flash_fwd("spa_flash_fwd_splitkv", q, k, v, nullptr, nullptr, out, lse, B, H, Sq, Sk, D, q_strides, k_strides, v_strides,
                   o_strides, scale, SPA_MASK_NONE, dtype, stream, workspace, nsplit);
}

int spa_flash_fwd_splitkv_fp8kv(const void* q, const void* k8, const void* v8, const float* k_scale, const float* v_scale, void* out,
                                float* lse, void* workspace, int B, int H, int Sq, int Sk, int D, int nsplit,
                                const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                                const int64_t o_strides[3], float scale, int dtype, void* stream) {
  if (!k_scale || !v_scale) return fail(SPA_EINVAL, "spa_flash_fwd_splitkv_fp8kv: null scale pointer");
  if (nsplit < 1) return fail(SPA_EINVAL, "spa_flash_fwd_splitkv_fp8kv: nsplit must be positive");
  return flash_fwd("spa_flash_fwd_splitkv_fp8kv", q, k8, v8, k_scale, v_scale, out, lse, B, H, Sq, Sk, D, q_strides, k_strides,
                   v_strides, o_strides, scale, SPA_MASK_NONE, dtype, stream, workspace, nsplit);
}

int spa_flash_fwd_fp8qkv(const void* q8, const void* k8, const void* v8, const float* q_scale, const float* k_scale,
                         const float* v_scale, void* out, float* lse, int B, int H, int Sq, int Sk, int D,
                         const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                         const int64_t o_strides[3], float scale, int mask_mode, int dtype, void* stream) {
  const char* what = "spa_flash_fwd_fp8qkv";
  if (!q8 || !k8 || !v8 || !out || !lse) return fail(SPA_EINVAL, "%s: null pointer", what);
  if (!q_scale || !k_scale || !v_scale) return fail(SPA_EINVAL, "%s: null scale pointer", what);
  if (!q_strides || !k_strides || !v_strides || !o_strides) return fail(SPA_EINVAL, "%s: null strides", what);
  if (!dims_ok(B, H, Sq, D) || Sk <= 0) return fail(SPA_EINVAL, "%s: sizes must be positive (B=%d H=%d Sq=%d Sk=%d D=%d)", what, B, H, Sq, Sk, D);
  if (dtype != SPA_BF16 && dtype != SPA_F16) return fail(dtype == SPA_F32 ? SPA_EUNSUPPORTED : SPA_EINVAL, "%s: out must be bf16 or fp16 (dtype %d)", what, dtype);
  if (mask_mode != SPA_MASK_NONE && mask_mode != SPA_MASK_CAUSAL) return fail(SPA_EINVAL, "%s: bad mask_mode %d", what, mask_mode);
  if (!scale_ok(scale)) return fail(SPA_EINVAL, "%s: softmax scale must be finite", what);
  if (D != 128) return fail(SPA_EUNSUPPORTED, "%s: head dim %d, built for 128", what, D);
  if (!aligned16(q8, q_strides, 1) || !aligned16(k8, k_strides, 1) || !aligned8(v8, v_strides, 3) || !aligned16(out, o_strides, 2) ||
      (((uintptr_t)q_scale | (uintptr_t)k_scale | (uintptr_t)v_scale | (uintptr_t)lse) & 3) != 0)
    return fail(SPA_EALIGN, "%s: q8, k8, out: pointers and rows 16-byte aligned; v8: 8-byte aligned", what);
  if ((int64_t)B * H > 0x7fffffffLL || (Sq + 127) / 128 > 65535) return fail(SPA_EINVAL, "%s: grid too large", what);
  if (!span_ok(Sk, k_strides[2], D, 1) || !span_ok(Sk, v_strides[2], D, 1))
    return fail(SPA_EUNSUPPORTED, "%s: K/V of one (batch, head) span 2 GiB or more (not supported for e4m3 K/V)", what);
  FwdParams p;
  p.q = q8; p.k = k8; p.v = v8; p.out = out; p.lse = lse;
  p.B = B; p.H = H; p.Sq = Sq; p.Sk = Sk;
  p.qs = S3(q_strides); p.ks = S3(k_strides); p.vs = S3(v_strides); p.os = S3(o_strides);
  p.scale = scale_eff(scale);
  p.scale_log2 = fabsf(scale_eff(scale)) * 1.4426950408889634f;
  p.negq = scale < 0.f;
  p.causal = mask_mode == SPA_MASK_CAUSAL;
  p.nqt = 0;
  p.lse_bh = Sq;
  p.part = nullptr; p.part_slot = 0; p.npart = 0;
  p.epi = SPA_EPI_PLAIN;
  p.P = 1; p.rank0 = 0; p.nranks = 1; p.t_begin = 0; p.t_count = -1;
  p.cu_q = nullptr; p.cu_k = nullptr;
  p.k_scale = k_scale; p.v_scale = v_scale; p.q_scale = q_scale;
  return launch_result(spa_launch_flash_fwd(p, D, dtype, (hipStream_t)stream), what);
}

int spa_merge(float* out_acc, float* lse_acc, const void* blk_out, const float* blk_lse, int B, int H, int Sq,
              int D, const int64_t acc_strides[3], const int64_t blk_strides[3], int blk_dtype, int init,
              void* stream) {
  if (!out_acc || !lse_acc || !blk_out || !blk_lse || !acc_strides || !blk_strides)
    return fail(SPA_EINVAL, "spa_merge: null pointer");
  if (!dims_ok(B, H, Sq, D)) return fail(SPA_EINVAL, "spa_merge: sizes must be positive");
  if (!dtype_ok(blk_dtype)) return fail(SPA_EINVAL, "spa_merge: bad dtype %d", blk_dtype);
  if (!pow2_8_512(D)) return fail(SPA_EUNSUPPORTED, "spa_merge: head dim %d must be a power of two in [8,512]", D);
  if (!aligned16(out_acc, acc_strides, 4) || !aligned16(blk_out, blk_strides, elem_size(blk_dtype)))
    return fail(SPA_EALIGN, "spa_merge: pointers and row strides must be 16-byte aligned");
  if (B > 65535 || (int64_t)H * Sq * (D / 8) >= 0x7fffffffLL) return fail(SPA_EINVAL, "spa_merge: grid too large");
  return launch_result(spa_launch_merge(out_acc, lse_acc, blk_out, blk_lse, B, H, Sq, D, S3(acc_strides),
                                        S3(blk_strides), blk_dtype, init, Sq, (hipStream_t)stream),
                       "spa_merge");
}

int64_t spa_ring_fwd_workspace_bytes(int B, int H, int S, int D, int P, int dtype) {
  if (B <= 0 || H <= 0 || S <= 0 || D <= 0 || P <= 0 || S % P != 0 || !dtype_ok(dtype)) return -1;
  const int64_t s = S / P;
  const int64_t acc = (int64_t)B * s * H * D * 4;
  // 16-bit: one slot per step but a rank's last: the block's output in q's type and its lse
  if (dtype != SPA_F32) return RingSlots(B, H, s, D).total(P);
  // fp32: running output, one block's output, one block's lse
  return 2 * acc + (int64_t)B * H * s * 4;
}

}  // extern "C"

namespace {

// Device address of `scratch` on the current device, looked up once per device.
int static_scratch(void** ptr) {
  static std::atomic<void*> addr[SPA_MAX_DEVICES];
  const int dev = spa_current_device();
  if (dev < 0 || dev >= SPA_MAX_DEVICES) return fail(SPA_ELAUNCH, "spa_ring_fwd_static: no current device (or index >= %d)", SPA_MAX_DEVICES);
  void* a = addr[dev].load(std::memory_order_acquire);
  if (!a) {
    const hipError_t e = hipGetSymbolAddress(&a, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !a) return fail(SPA_ELAUNCH, "spa_ring_fwd_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
    addr[dev].store(a, std::memory_order_release);
  }
  *ptr = a;
  return SPA_OK;
}

// The flag-driven launches: no cache line may hold bytes of two chunks (a line fetched with one chunk would keep the
// other's bytes from before their arrival), so every chunk of every (batch, head) must start on a 128-byte boundary.
// Strides in elements of `esz` bytes.
bool chunk_lines_ok(const void* base, const int64_t st[3], int esz, int B, int H, int S, int P) {
  const int64_t chunk = S / P;
  return ((uintptr_t)base & 127) == 0 && (P == 1 || (chunk * st[2] * esz) % 128 == 0) && (B == 1 || (st[0] * esz) % 128 == 0) &&
         (H == 1 || (st[1] * esz) % 128 == 0);
}

// `what` names the entry point in messages; `ws_bytes` < 0: the caller vouches for the workspace size.
// k_scale / v_scale non-null: K and V are e4m3 bytes with one scale per (batch, head) for the whole sequence.
// What the flag variant adds to a ring call: null `arrive` = none.
struct RingFlags {
  const unsigned* arrive = nullptr;
  unsigned epoch = 0, spin_limit = 0;
  unsigned* fault = nullptr;
};

// q_scale non-null (with the other two): q is e4m3 as well and the scores run on the 8-bit matrix instruction (D = 128).
int ring_fwd(const char* what, const void* q, const void* k, const void* v, const float* q_scale, const float* k_scale,
             const float* v_scale, void* out, float* lse, void* workspace,
             int64_t ws_bytes, int B, int H, int S, int D, int P, int rank, const int64_t q_strides[3],
             const int64_t k_strides[3], const int64_t v_strides[3], const int64_t o_strides[3], float scale,
             int mask_mode, int dtype, int fuse, void* stream, const RingFlags flags = RingFlags()) {
  if (!q || !k || !v || !out || !lse) return fail(SPA_EINVAL, "%s: null pointer", what);
  if (!q_strides || !k_strides || !v_strides || !o_strides) return fail(SPA_EINVAL, "%s: null strides", what);
  if (!dims_ok(B, H, S, D)) return fail(SPA_EINVAL, "%s: sizes must be positive", what);
  if (P <= 0 || S % P != 0) return fail(SPA_EINVAL, "%s: ring size %d must divide the sequence length %d", what, P, S);
  if (rank < -1 || rank >= P) return fail(SPA_EINVAL, "%s: rank %d outside [-1, %d)", what, rank, P);
  if (!dtype_ok(dtype)) return fail(SPA_EINVAL, "%s: bad dtype %d", what, dtype);
  if (mask_mode != SPA_MASK_NONE && mask_mode != SPA_MASK_CAUSAL) return fail(SPA_EINVAL, "%s: bad mask_mode %d", what, mask_mode);
  const bool zig_req = (fuse & SPA_RING_ZIGZAG) != 0;
  fuse &= ~SPA_RING_ZIGZAG;
  if (fuse < SPA_RING_PER_STEP || fuse > SPA_RING_ALL_RANKS) return fail(SPA_EINVAL, "%s: bad fuse mode %d", what, fuse);
  if (zig_req && S % (2 * P) != 0)
    return fail(SPA_EINVAL, "%s: zigzag sharding needs 2 * ring size = %d to divide the sequence length %d", what, 2 * P, S);
  if (!scale_ok(scale)) return fail(SPA_EINVAL, "%s: softmax scale must be finite", what);
  if (D != 32 && D != 64 && D != 128) return fail(SPA_EUNSUPPORTED, "%s: head dim %d not in {32,64,128}", what, D);
  const bool kv8 = k_scale || v_scale;
  if (kv8 && (!k_scale || !v_scale)) return fail(SPA_EINVAL, "%s: null scale pointer", what);
  if (kv8 && dtype == SPA_F32) return fail(SPA_EUNSUPPORTED, "%s: e4m3 K/V go with bf16 or fp16 queries", what);
  if (kv8 && D == 32) return fail(SPA_EUNSUPPORTED, "%s: e4m3 K/V need head dim 64 or 128", what);
  const bool qk8 = q_scale != nullptr;
  if (qk8 && !kv8) return fail(SPA_EINVAL, "%s: e4m3 q goes with e4m3 K/V", what);
  if (qk8 && D != 128) return fail(SPA_EUNSUPPORTED, "%s: e4m3 q: head dim %d, built for 128", what, D);
  if (qk8 && zig_req) return fail(SPA_EUNSUPPORTED, "%s: e4m3 q has no zigzag variants", what);
  const int esz = elem_size(dtype), kesz = kv8 ? 1 : esz;
  const bool kv_aligned = qk8   ? aligned16(k, k_strides, 1) && aligned8(v, v_strides, 3) && (((uintptr_t)q_scale | (uintptr_t)k_scale | (uintptr_t)v_scale) & 3) == 0
                          : kv8 ? aligned8(k, k_strides, 3) && aligned8(v, v_strides, 3) && (((uintptr_t)k_scale | (uintptr_t)v_scale) & 3) == 0
                                : aligned16(k, k_strides, esz) && aligned16(v, v_strides, esz);
  if (!aligned16(q, q_strides, qk8 ? 1 : esz) || !kv_aligned ||
      !aligned16(out, o_strides, esz) || ((uintptr_t)lse & 3) != 0 || ((uintptr_t)workspace & 15) != 0)
    return fail(SPA_EALIGN, "%s: pointers and row strides must be 16-byte aligned (8-byte for e4m3 K/V)", what);
  const bool big = !span_ok(S, k_strides[2], D, kesz) || !span_ok(S, v_strides[2], D, kesz);
  if (big && big_kv_obstacle(kv8, dtype, k_strides[2], v_strides[2], esz))
    return fail(SPA_EUNSUPPORTED, "%s: K/V of one (batch, head) span 2 GiB or more (%s)", what,
                big_kv_obstacle(kv8, dtype, k_strides[2], v_strides[2], esz));
  const bool causal = mask_mode == SPA_MASK_CAUSAL;
  const int s = S / P;
  if (dtype == SPA_F32) fuse = SPA_RING_PER_STEP;  // the fp32 kernel handles one block pair per launch
  // zigzag shards only change a causal ring (without a mask the order of the rows does not matter)
  const bool zig = zig_req && causal && P > 1;
  if (zig && big && dtype != SPA_F32)
    return fail(SPA_EUNSUPPORTED, "%s: zigzag shards are not built for K/V of 2 GiB or more per (batch, head)", what);
  const bool multi = P > 1 && (!causal || rank != 0 || zig);  // does some rank visit more than one block?
  if (fuse == SPA_RING_PER_STEP && multi && !workspace)
    return fail(SPA_EINVAL, "%s: workspace required when steps are separate launches", what);
  if (fuse == SPA_RING_PER_STEP && multi && ws_bytes >= 0 && spa_ring_fwd_workspace_bytes(B, H, S, D, P, dtype) > ws_bytes)
    return fail(SPA_EINVAL, "%s: these sizes need %lld bytes of scratch, the built-in buffer holds %lld", what,
                (long long)spa_ring_fwd_workspace_bytes(B, H, S, D, P, dtype), (long long)ws_bytes);
  const int r_lo = rank < 0 ? 0 : rank, r_hi = rank < 0 ? P : rank + 1;
  if ((int64_t)B * H > 0x7fffffffLL || (s + 127) / 128 > 65535 || r_hi - r_lo > 65535) return fail(SPA_EINVAL, "%s: grid too large", what);
  hipStream_t st = (hipStream_t)stream;

  // workspace carve-up; one rank's block output (or, fp32, its running output) is laid out [B, s, H, D]
  float* acc = (float*)workspace;        // fp32 path only
  const int64_t acc_elems = (int64_t)B * s * H * D;
  Strides3 as;
  as.b = (int64_t)s * H * D; as.h = D; as.s = (int64_t)H * D;
  float* blk_out = acc + acc_elems;      // fp32 path only
  float* blk_lse = blk_out + acc_elems;  // fp32 path only

  FwdParams p;
  p.q = q; p.k = k; p.v = v; p.out = out; p.lse = lse;
  p.B = B; p.H = H; p.Sq = s; p.Sk = s;
  p.qs = S3(q_strides); p.ks = S3(k_strides); p.vs = S3(v_strides); p.os = S3(o_strides);
  p.scale = scale_eff(scale);
  p.scale_log2 = fabsf(scale_eff(scale)) * 1.4426950408889634f;
  p.negq = scale < 0.f;
  p.causal = causal;
  p.nqt = 0;
  p.lse_bh = S;
  p.part = workspace;  // 16-bit path: the steps' slots (RingSlots)
  p.part_slot = 0; p.npart = 0;
  p.P = P;
  p.epi = SPA_EPI_PLAIN;
  p.cu_q = nullptr; p.cu_k = nullptr;
  p.k_scale = k_scale; p.v_scale = v_scale; p.q_scale = q_scale;
  p.zigzag = zig && dtype != SPA_F32;
  p.zz_half = 0;
  p.big = big && dtype != SPA_F32;
  if (flags.arrive) {
    if (fuse != SPA_RING_PER_RANK || dtype == SPA_F32 || (kv8 && !qk8) || zig || big || D == 32)
      return fail(SPA_EUNSUPPORTED, "%s: built for one launch per rank, bf16 / fp16 (or e4m3 q, k, v), head dim 64 or 128, contiguous chunks below 2 GiB", what);
    p.arrive = flags.arrive; p.epoch = flags.epoch; p.spin_limit = flags.spin_limit; p.fault = flags.fault;
  }

  if (fuse == SPA_RING_ALL_RANKS) {  // one launch: every requested rank, every step
    p.rank0 = r_lo; p.nranks = r_hi - r_lo; p.t_begin = 0; p.t_count = -1;
    return launch_result(spa_launch_flash_fwd(p, D, dtype, st), what);
  }
  for (int r = r_lo; r < r_hi; ++r) {
    p.rank0 = r; p.nranks = 1;
    if (fuse == SPA_RING_PER_RANK) {  // one launch per rank: the workgroup walks the rank's chunks
      p.t_begin = 0; p.t_count = -1;
      hipError_t e = spa_launch_flash_fwd(p, D, dtype, st);
      if (e != hipSuccess) return launch_result(e, what);
      continue;
    }
    const int nsteps = causal && !zig ? r + 1 : P;  // a zigzag rank has work in every step
    const int hs = s / 2;
    for (int t = 0; t < nsteps; ++t) {
      hipError_t e;
      if (dtype != SPA_F32) {
        p.t_begin = t; p.t_count = 1;
        // every step but the last leaves its block in slot t; the last merges them in ring order and adds its own
        p.epi = nsteps == 1 ? SPA_EPI_PLAIN : t + 1 == nsteps ? SPA_EPI_FINALN : SPA_EPI_PART;
        p.part_slot = t;
        p.npart = nsteps - 1;
        // zigzag, a step past the rank's own number: only the second half of the rows has a block.  The launch
        // covers that half's tiles, except the last step's: there the first half's workgroups merge their slots.
        p.zz_half = zig && t > r && t + 1 < nsteps;
        e = spa_launch_flash_fwd(p, D, dtype, st);
      } else if (zig) {
        // fp32, zigzag: plain block launches on explicit sub-blocks, merged by the stand-alone kernels
        // (step 0: the rank's own chunk, causal; chunk c < r: all rows x first half of the keys; c > r:
        // second half of the rows x all keys, merged into those rows only)
        const int c = ((r - t) % P + P) % P;
        const bool lower = t > r;  // c > r
        const int rows = lower ? hs : s, keys = (t >= 1 && !lower) ? hs : s, row0 = lower ? hs : 0;
        FwdParams pb = p;
        pb.zigzag = 0;
        pb.P = 1; pb.rank0 = 0; pb.nranks = 1; pb.t_begin = 0; pb.t_count = -1;
        pb.Sq = rows; pb.Sk = keys;
        pb.q = (const char*)q + ((int64_t)r * s + row0) * p.qs.s * esz;
        pb.k = (const char*)k + (int64_t)c * s * p.ks.s * esz;
        pb.v = (const char*)v + (int64_t)c * s * p.vs.s * esz;
        pb.causal = t == 0;
        pb.epi = SPA_EPI_PLAIN;
        pb.out = blk_out; pb.os = as; pb.lse = blk_lse; pb.lse_bh = rows;
        e = spa_launch_flash_fwd(pb, D, dtype, st);
        float* lser = lse + (int64_t)r * s;
        if (e == hipSuccess)
          e = spa_launch_merge(acc + (int64_t)row0 * as.s, lser + row0, blk_out, blk_lse, B, H, rows, D, as, as, SPA_F32, t == 0, S, st);
        if (e == hipSuccess && t + 1 == nsteps)
          e = spa_launch_finalize((char*)out + (int64_t)r * s * p.os.s * esz, acc, B, H, s, D, p.os, as, SPA_F32, st);
      } else {
        // fp32: one plain block pair per launch on explicit chunk pointers, merged by the stand-alone kernels
        const int c = ((r - t) % P + P) % P;
        FwdParams pb = p;
        pb.P = 1; pb.rank0 = 0; pb.nranks = 1; pb.t_begin = 0; pb.t_count = -1;
        pb.q = (const char*)q + (int64_t)r * s * p.qs.s * esz;
        pb.k = (const char*)k + (int64_t)c * s * p.ks.s * esz;
        pb.v = (const char*)v + (int64_t)c * s * p.vs.s * esz;
        pb.causal = causal && t == 0;
        pb.epi = SPA_EPI_PLAIN;
        char* outr = (char*)out + (int64_t)r * s * p.os.s * esz;
        float* lser = lse + (int64_t)r * s;
        if (nsteps == 1) {
          pb.out = outr;
          pb.lse = lser;
          pb.lse_bh = S;
          e = spa_launch_flash_fwd(pb, D, dtype, st);
        } else {
          pb.out = blk_out;
          pb.os = as;
          pb.lse = blk_lse;
          pb.lse_bh = s;
          e = spa_launch_flash_fwd(pb, D, dtype, st);
          if (e == hipSuccess)
            e = spa_launch_merge(acc, lser, blk_out, blk_lse, B, H, s, D, as, as, SPA_F32, t == 0, S, st);
          if (e == hipSuccess && t + 1 == nsteps)
            e = spa_launch_finalize(outr, acc, B, H, s, D, p.os, as, SPA_F32, st);
        }
      }
      if (e != hipSuccess) return launch_result(e, what);
    }
  }
  return SPA_OK;
}

}  // namespace

extern "C" {

int spa_ring_fwd(const void* q, const void* k, const void* v, void* out, float* lse, void* workspace, int B,
                 int H, int S, int D, int P, int rank, const int64_t q_strides[3], const int64_t k_strides[3],
                 const int64_t v_strides[3], const int64_t o_strides[3], float scale, int mask_mode, int dtype,
                 int fuse, void* stream) {
  return ring_fwd("spa_ring_fwd", q, k, v, nullptr, nullptr, nullptr, out, lse, workspace, -1, B, H, S, D, P, rank, q_strides, k_strides,
                  v_strides, o_strides, scale, mask_mode, dtype, fuse, stream);
}

int spa_ring_fwd_fp8kv(const void* q, const void* k8, const void* v8, const float* k_scale, const float* v_scale,
                       void* out, float* lse, void* workspace, int B, int H, int S, int D, int P, int rank,
                       const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                       const int64_t o_strides[3], float scale, int mask_mode, int dtype, int fuse, void* stream) {
  if (!k_scale || !v_scale) return fail(SPA_EINVAL, "spa_ring_fwd_fp8kv: null scale pointer");
  return ring_fwd("spa_ring_fwd_fp8kv", q, k8, v8, nullptr, k_scale, v_scale, out, lse, workspace, -1, B, H, S, D, P, rank, q_strides,
                  k_strides, v_strides, o_strides, scale, mask_mode, dtype, fuse, stream);
}

int spa_ring_fwd_flags(const void* q, const void* k, const void* v, void* out, float* lse, const uint32_t* arrive,
                       uint32_t epoch, uint32_t spin_limit, uint32_t* fault, int B, int H, int S, int D, int P, int rank,
                       const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                       const int64_t o_strides[3], float scale, int mask_mode, int dtype, void* stream) {
  if (!arrive || !fault) return fail(SPA_EINVAL, "spa_ring_fwd_flags: null flag pointer");
  if ((((uintptr_t)arrive | (uintptr_t)fault) & 3) != 0) return fail(SPA_EALIGN, "spa_ring_fwd_flags: flags must be 4-byte aligned");
  if (spin_limit == 0) return fail(SPA_EINVAL, "spa_ring_fwd_flags: spin_limit must be positive");
  if (k && v && k_strides && v_strides && P > 0 && S > 0 && S % P == 0 && (dtype == SPA_BF16 || dtype == SPA_F16) &&
      (!chunk_lines_ok(k, k_strides, 2, B, H, S, P) || !chunk_lines_ok(v, v_strides, 2, B, H, S, P)))
    return fail(SPA_EALIGN, "spa_ring_fwd_flags: every K / V chunk of every (batch, head) must start on a 128-byte boundary");
  RingFlags f;
  f.arrive = arrive; f.epoch = epoch; f.spin_limit = spin_limit; f.fault = fault;
  return ring_fwd("spa_ring_fwd_flags", q, k, v, nullptr, nullptr, nullptr, out, lse, nullptr, -1, B, H, S, D, P, rank, q_strides,
                  k_strides, v_strides, o_strides, scale, mask_mode, dtype, SPA_RING_PER_RANK, stream, f);
}

int spa_ring_fwd_flags_fp8qkv(const void* q8, const void* k8, const void* v8, const float* q_scale, const float* k_scale,
                              const float* v_scale, void* out, float* lse, const uint32_t* arrive, uint32_t epoch,
                              uint32_t spin_limit, uint32_t* fault, int B, int H, int S, int D, int P, int rank,
                              const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                              const int64_t o_strides[3], float scale, int mask_mode, int dtype, void* stream) {
  const char* what = "spa_ring_fwd_flags_fp8qkv";
  if (!q_scale || !k_scale || !v_scale) return fail(SPA_EINVAL, "%s: null scale pointer", what);
  if (!arrive || !fault) return fail(SPA_EINVAL, "%s: null flag pointer", what);
  if ((((uintptr_t)arrive | (uintptr_t)fault) & 3) != 0) return fail(SPA_EALIGN, "%s: flags must be 4-byte aligned", what);
  if (spin_limit == 0) return fail(SPA_EINVAL, "%s: spin_limit must be positive", what);
  if (k8 && v8 && k_strides && v_strides && P > 0 && S > 0 && S % P == 0 &&
      (!chunk_lines_ok(k8, k_strides, 1, B, H, S, P) || !chunk_lines_ok(v8, v_strides, 1, B, H, S, P)))
    return fail(SPA_EALIGN, "%s: every K / V chunk of every (batch, head) must start on a 128-byte boundary", what);
  RingFlags f;
  f.arrive = arrive; f.epoch = epoch; f.spin_limit = spin_limit; f.fault = fault;
  return ring_fwd(what, q8, k8, v8, q_scale, k_scale, v_scale, out, lse, nullptr, -1, B, H, S, D, P, rank, q_strides, k_strides,
                  v_strides, o_strides, scale, mask_mode, dtype, SPA_RING_PER_RANK, stream, f);
}

int spa_ring_flag_set(uint32_t* arrive, int chunk, uint32_t epoch, void* stream) {
  if (!arrive || chunk < 0) return fail(SPA_EINVAL, "spa_ring_flag_set: null pointer or negative chunk");
  const hipError_t e = hipStreamWriteValue32((hipStream_t)stream, arrive + chunk, epoch, 0);
  if (e != hipSuccess) return fail(SPA_ELAUNCH, "spa_ring_flag_set: %s", hipGetErrorString(e));
  return SPA_OK;
}

int spa_ring_fwd_fp8qkv(const void* q8, const void* k8, const void* v8, const float* q_scale, const float* k_scale,
                        const float* v_scale, void* out, float* lse, void* workspace, int B, int H, int S, int D, int P, int rank,
                        const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                        const int64_t o_strides[3], float scale, int mask_mode, int dtype, int fuse, void* stream) {
  if (!q_scale || !k_scale || !v_scale) return fail(SPA_EINVAL, "spa_ring_fwd_fp8qkv: null scale pointer");
  return ring_fwd("spa_ring_fwd_fp8qkv", q8, k8, v8, q_scale, k_scale, v_scale, out, lse, workspace, -1, B, H, S, D, P, rank, q_strides,
                  k_strides, v_strides, o_strides, scale, mask_mode, dtype, fuse, stream);
}

int64_t spa_static_scratch_bytes(void) { return (int64_t)SPA_STATIC_SCRATCH_BYTES; }

int spa_static_scratch_init(void) {
  void* ws = nullptr;
  return static_scratch(&ws);
}

int spa_ring_fwd_static(const void* q, const void* k, const void* v, void* out, float* lse, int B, int H, int S,
                        int D, int P, int rank, const int64_t q_strides[3], const int64_t k_strides[3],
                        const int64_t v_strides[3], const int64_t o_strides[3], float scale, int mask_mode,
                        int dtype, int fuse, void* stream) {
  void* ws = nullptr;
  const int rc = static_scratch(&ws);
  if (rc != SPA_OK) return rc;
  return ring_fwd("spa_ring_fwd_static", q, k, v, nullptr, nullptr, nullptr, out, lse, ws, (int64_t)SPA_STATIC_SCRATCH_BYTES, B, H, S, D, P,
                  rank, q_strides, k_strides, v_strides, o_strides, scale, mask_mode, dtype, fuse, stream);
}

int spa_tune(int knob, int value) {
  if (knob < 0 || knob >= SPA_KNOB_COUNT) return fail(SPA_EINVAL, "spa_tune: unknown knob %d", knob);
  g_spa_knob[knob].store(value, std::memory_order_relaxed);
  return SPA_OK;
}

int spa_finalize(void* out, const float* out_acc, int B, int H, int Sq, int D, const int64_t o_strides[3],
                 const int64_t acc_strides[3], int dtype, void* stream) {
  if (!out || !out_acc || !o_strides || !acc_strides) return fail(SPA_EINVAL, "spa_finalize: null pointer");
  if (!dims_ok(B, H, Sq, D)) return fail(SPA_EINVAL, "spa_finalize: sizes must be positive");
  if (!dtype_ok(dtype)) return fail(SPA_EINVAL, "spa_finalize: bad dtype %d", dtype);
  if (!pow2_8_512(D)) return fail(SPA_EUNSUPPORTED, "spa_finalize: head dim %d must be a power of two in [8,512]", D);
  if (!aligned16(out_acc, acc_strides, 4) || !aligned16(out, o_strides, elem_size(dtype)))
    return fail(SPA_EALIGN, "spa_finalize: pointers and row strides must be 16-byte aligned");
  if (B > 65535 || (int64_t)H * Sq * (D / 8) >= 0x7fffffffLL) return fail(SPA_EINVAL, "spa_finalize: grid too large");
  return launch_result(spa_launch_finalize(out, out_acc, B, H, Sq, D, S3(o_strides), S3(acc_strides), dtype,
                                           (hipStream_t)stream),
                       "spa_finalize");
}

static int relayout(const void* src, void* dst, int P, int B, int s, int H, int D, int pack, int elem_bytes,
                    bool s2h, void* stream, const char* what) {
  if (!src || !dst) return fail(SPA_EINVAL, "%s: null pointer", what);
  if (P <= 0 || B <= 0 || s <= 0 || H <= 0 || D <= 0) return fail(SPA_EINVAL, "%s: sizes must be positive", what);
  if (pack < 1 || pack > 3) return fail(SPA_EINVAL, "%s: pack must be 1, 2 or 3", what);
  if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8)
    return fail(SPA_EINVAL, "%s: elem_bytes must be 1, 2, 4 or 8", what);
  if (H % P != 0) return fail(SPA_EINVAL, "%s: heads (%d) not divisible by ranks (%d)", what, H, P);
  if (src == dst) return fail(SPA_EINVAL, "%s: in-place re-layout is not supported", what);
  if ((int64_t)P * pack > 65535 || (int64_t)P * B > 65535) return fail(SPA_EINVAL, "%s: grid too large (P * B and P * pack must stay below 65536)", what);
  return launch_result(spa_launch_relayout(src, dst, P, B, s, H, D, pack, elem_bytes, s2h, (hipStream_t)stream), what);
}

int spa_relayout_s2h(const void* x, void* y, int P, int B, int s, int H, int D, int pack, int elem_bytes,
                     void* stream) {
  return relayout(x, y, P, B, s, H, D, pack, elem_bytes, true, stream, "spa_relayout_s2h");
}

int spa_relayout_h2s(const void* y, void* x, int P, int B, int s, int H, int D, int pack, int elem_bytes,
                     void* stream) {
  return relayout(y, x, P, B, s, H, D, pack, elem_bytes, false, stream, "spa_relayout_h2s");
}

int spa_bwd_delta(const void* out, const void* dout, float* delta, int B, int H, int Sq, int D,
                  const int64_t o_strides[3], const int64_t do_strides[3], int dtype, void* stream) {
  if (!out || !dout || !delta || !o_strides || !do_strides) return fail(SPA_EINVAL, "spa_bwd_delta: null pointer");
  if (!dims_ok(B, H, Sq, D)) return fail(SPA_EINVAL, "spa_bwd_delta: sizes must be positive");
  if (!dtype_ok(dtype)) return fail(SPA_EINVAL, "spa_bwd_delta: bad dtype %d", dtype);
  if (!pow2_8_512(D)) return fail(SPA_EUNSUPPORTED, "spa_bwd_delta: head dim %d must be a power of two in [8,512]", D);
  const int esz = elem_size(dtype);
  if (!aligned16(out, o_strides, esz) || !aligned16(dout, do_strides, esz))
    return fail(SPA_EALIGN, "spa_bwd_delta: pointers and row strides must be 16-byte aligned");
  if (B > 65535 || (int64_t)H * Sq * (D / 8) >= 0x7fffffffLL) return fail(SPA_EINVAL, "spa_bwd_delta: grid too large");
  return launch_result(spa_launch_delta(out, dout, delta, B, H, Sq, D, S3(o_strides), S3(do_strides), dtype,
                                        (hipStream_t)stream),
                       "spa_bwd_delta");
}

namespace {
// grads_in_t: dq / dk / dv are tensors of the inputs' element type and are written (spa_flash_bwd_out);
// else fp32 accumulators that are added to (spa_flash_bwd).
int flash_bwd(const char* what, const void* q, const void* k, const void* v, const void* dout, const float* lse,
              const float* delta, void* dq, void* dk, void* dv, bool grads_in_t, int B, int H, int Sq, int Sk,
              int D, const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
              const int64_t do_strides[3], const int64_t dq_strides[3], const int64_t dk_strides[3],
              const int64_t dv_strides[3], float scale, int mask_mode, int dtype, void* stream) {
  if (!q || !k || !v || !dout || !lse || !delta || !dq || !dk || !dv) return fail(SPA_EINVAL, "%s: null pointer", what);
  if (!q_strides || !k_strides || !v_strides || !do_strides || !dq_strides || !dk_strides || !dv_strides)
    return fail(SPA_EINVAL, "%s: null strides", what);
  if (!dims_ok(B, H, Sq, D) || Sk <= 0) return fail(SPA_EINVAL, "%s: sizes must be positive", what);
  if (!dtype_ok(dtype)) return fail(SPA_EINVAL, "%s: bad dtype %d", what, dtype);
  if (mask_mode != SPA_MASK_NONE && mask_mode != SPA_MASK_CAUSAL) return fail(SPA_EINVAL, "%s: bad mask_mode %d", what, mask_mode);
  if (!scale_ok(scale)) return fail(SPA_EINVAL, "%s: softmax scale must be finite", what);
  if (D != 32 && D != 64 && D != 128) return fail(SPA_EUNSUPPORTED, "%s: head dim %d not in {32,64,128}", what, D);
  const int esz = elem_size(dtype), gsz = grads_in_t ? esz : 4;
  if (!aligned16(q, q_strides, esz) || !aligned16(k, k_strides, esz) || !aligned16(v, v_strides, esz) ||
      !aligned16(dout, do_strides, esz) || !aligned16(dq, dq_strides, gsz) || !aligned16(dk, dk_strides, gsz) ||
      !aligned16(dv, dv_strides, gsz))
    return fail(SPA_EALIGN, "%s: pointers and row strides must be 16-byte aligned", what);
  const bool big = !span_ok(Sq, q_strides[2], D, esz) || !span_ok(Sk, k_strides[2], D, esz) || !span_ok(Sk, v_strides[2], D, esz) ||
                   !span_ok(Sq, do_strides[2], D, esz);
  if (big && dtype != SPA_F32 && !(span_rebasable(q_strides[2], esz) && span_rebasable(k_strides[2], esz) &&
                                   span_rebasable(v_strides[2], esz) && span_rebasable(do_strides[2], esz)))
    return fail(SPA_EUNSUPPORTED, "%s: a tensor of one (batch, head) spans 2 GiB or more and 128 rows of it 1 GiB or more", what);
  if ((int64_t)B * H * ((Sq + 127) / 128) > 0x7fffffffLL || (int64_t)B * H * ((Sk + 127) / 128) > 0x7fffffffLL)
    return fail(SPA_EINVAL, "%s: grid too large", what);
  BwdParams p;
  p.q = q; p.k = k; p.v = v; p.dout = dout; p.lse = lse; p.delta = delta;
  p.dq = (float*)dq; p.dk = (float*)dk; p.dv = (float*)dv;
  p.grads_in_t = grads_in_t;
  p.big = big && dtype != SPA_F32;
  p.B = B; p.H = H; p.Sq = Sq; p.Sk = Sk;
  p.qs = S3(q_strides); p.ks = S3(k_strides); p.vs = S3(v_strides); p.dos = S3(do_strides);
  p.dqs = S3(dq_strides); p.dks = S3(dk_strides); p.dvs = S3(dv_strides);
  p.scale = scale_eff(scale);
  p.scale_log2 = scale_eff(scale) * 1.4426950408889634f;
  p.causal = mask_mode == SPA_MASK_CAUSAL;
  p.nqt = 0;
  p.nkt = 0;
  p.lse_bh = Sq;
  p.cu_q = nullptr; p.cu_k = nullptr;
  return launch_result(spa_launch_flash_bwd(p, D, dtype, (hipStream_t)stream), what);
}
}  // namespace

int spa_flash_bwd(const void* q, const void* k, const void* v, const void* dout, const float* lse,
                  const float* delta, float* dq_acc, float* dk_acc, float* dv_acc, int B, int H, int Sq, int Sk,
                  int D, const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                  const int64_t do_strides[3], const int64_t dq_strides[3], const int64_t dk_strides[3],
                  const int64_t dv_strides[3], float scale, int mask_mode, int dtype, void* stream) {
  return flash_bwd("spa_flash_bwd", q, k, v, dout, lse, delta, dq_acc, dk_acc, dv_acc, false, B, H, Sq, Sk, D, q_strides, k_strides,
                   v_strides, do_strides, dq_strides, dk_strides, dv_strides, scale, mask_mode, dtype, stream);
}

int spa_flash_bwd_out(const void* q, const void* k, const void* v, const void* dout, const float* lse,
                      const float* delta, void* dq, void* dk, void* dv, int B, int H, int Sq, int Sk,
                      int D, const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                      const int64_t do_strides[3], const int64_t dq_strides[3], const int64_t dk_strides[3],
                      const int64_t dv_strides[3], float scale, int mask_mode, int dtype, void* stream) {
  return flash_bwd("spa_flash_bwd_out", q, k, v, dout, lse, delta, dq, dk, dv, true, B, H, Sq, Sk, D, q_strides, k_strides,
                   v_strides, do_strides, dq_strides, dk_strides, dv_strides, scale, mask_mode, dtype, stream);
}

namespace {
// Strides of a packed [rows, H, D] tensor come as (head, row); the batch stride is unused.
Strides3 S2(const int64_t* s) {
  Strides3 r;
  r.b = 0; r.h = s[0]; r.s = s[1];
  return r;
}
bool aligned16v(const void* p, const int64_t* s, int esz) {
  return ((uintptr_t)p & 15) == 0 && (s[0] * esz) % 16 == 0 && (s[1] * esz) % 16 == 0;
}
int varlen_sizes_ok(const char* what, const void* cu_q, const void* cu_k, int nseq, int H, int total_q, int total_k,
                    int max_sq, int max_sk, int D, int dtype, int mask_mode, float scale) {
  if (!cu_q || !cu_k) return fail(SPA_EINVAL, "%s: null cu_seqlens", what);
  if ((((uintptr_t)cu_q | (uintptr_t)cu_k) & 3) != 0) return fail(SPA_EALIGN, "%s: cu_seqlens must be 4-byte aligned", what);
  if (nseq <= 0 || H <= 0 || total_q <= 0 || total_k <= 0 || max_sq <= 0 || max_sk <= 0 || max_sq > total_q || max_sk > total_k)
    return fail(SPA_EINVAL, "%s: sizes must be positive and the longest sequence no longer than the total (nseq=%d H=%d total_q=%d total_k=%d max_sq=%d max_sk=%d)",
                what, nseq, H, total_q, total_k, max_sq, max_sk);
  if (!dtype_ok(dtype)) return fail(SPA_EINVAL, "%s: bad dtype %d", what, dtype);
  if (mask_mode != SPA_MASK_NONE && mask_mode != SPA_MASK_CAUSAL) return fail(SPA_EINVAL, "%s: bad mask_mode %d", what, mask_mode);
  if (!scale_ok(scale)) return fail(SPA_EINVAL, "%s: softmax scale must be finite", what);
  if (D != 32 && D != 64 && D != 128) return fail(SPA_EUNSUPPORTED, "%s: head dim %d not in {32,64,128}", what, D);
  if ((max_sq + 127) / 128 > 65535 || (int64_t)nseq * H * ((max_sq + 127) / 128) > 0x7fffffffLL ||
      (int64_t)nseq * H * ((max_sk + 127) / 128) > 0x7fffffffLL)
    return fail(SPA_EINVAL, "%s: grid too large", what);
  return SPA_OK;
}
}  // namespace

}  // extern "C"

namespace {
int flash_fwd_varlen(const char* what, const void* q, const void* k, const void* v, const float* k_scale,
                     const float* v_scale, void* out, float* lse, const int32_t* cu_seqlens_q,
                     const int32_t* cu_seqlens_k, int nseq, int H, int total_q, int total_k, int max_sq, int max_sk,
                     int D, const int64_t q_strides[2], const int64_t k_strides[2], const int64_t v_strides[2],
                     const int64_t o_strides[2], float scale, int mask_mode, int dtype, void* stream, int P = 1, int rank = -1,
                     int fuse = SPA_RING_PER_RANK) {
  // P > 1: a ring over the packed batch.  The tensors are P stacked shards of total_q = total_k rows, every shard
  // packed as cu_seqlens_q says; rank r (or every rank, -1) walks the shards in ring order, one launch per rank or one for all.
  const bool kv8 = k_scale || v_scale;
  if (!q || !k || !v || !out || !lse) return fail(SPA_EINVAL, "%s: null pointer", what);
  if (kv8 && (!k_scale || !v_scale)) return fail(SPA_EINVAL, "%s: null scale pointer", what);
  if (!q_strides || !k_strides || !v_strides || !o_strides) return fail(SPA_EINVAL, "%s: null strides", what);
  const int rc = varlen_sizes_ok(what, cu_seqlens_q, cu_seqlens_k, nseq, H, total_q, total_k, max_sq, max_sk, D, dtype,
                                 mask_mode, scale);
  if (rc != SPA_OK) return rc;
  if (P < 1 || rank < -1 || rank >= P) return fail(SPA_EINVAL, "%s: ring size %d, rank %d", what, P, rank);
  if (P > 1) {
    if (fuse != SPA_RING_PER_RANK && fuse != SPA_RING_ALL_RANKS) return fail(SPA_EINVAL, "%s: one launch per rank or one for all ranks", what);
    if (dtype == SPA_F32 || kv8) return fail(SPA_EUNSUPPORTED, "%s: the ring over a packed batch is built for bf16 / fp16 tensors", what);
    if (cu_seqlens_q != cu_seqlens_k || total_q != total_k || max_sq != max_sk)
      return fail(SPA_EINVAL, "%s: a ring over a packed batch has one cu_seqlens for queries and keys", what);
    if ((int64_t)P * total_q > 0x7fffffffLL || P > 65535) return fail(SPA_EINVAL, "%s: grid too large", what);
  }
  if (kv8 && dtype == SPA_F32) return fail(SPA_EUNSUPPORTED, "%s: e4m3 K/V go with bf16 or fp16 queries", what);
  if (kv8 && D == 32) return fail(SPA_EUNSUPPORTED, "%s: e4m3 K/V need head dim 64 or 128", what);
  const int esz = elem_size(dtype), kesz = kv8 ? 1 : esz;
  const bool kv_aligned = kv8 ? aligned8(k, k_strides, 2) && aligned8(v, v_strides, 2) && (((uintptr_t)k_scale | (uintptr_t)v_scale) & 3) == 0
                              : aligned16v(k, k_strides, esz) && aligned16v(v, v_strides, esz);
  if (!aligned16v(q, q_strides, esz) || !kv_aligned || !aligned16v(out, o_strides, esz) || ((uintptr_t)lse & 3) != 0)
    return fail(SPA_EALIGN, "%s: pointers and row strides must be 16-byte aligned (8-byte for e4m3 K/V)", what);
  // (a sequence's keys reach from its slice in the first shard to its slice in the last)
  const int64_t key_span = (int64_t)(P - 1) * total_k + max_sk;
  const bool big = key_span > 0x7fffffffLL || !span_ok((int)key_span, k_strides[1], D, kesz) || !span_ok((int)key_span, v_strides[1], D, kesz);
  if (big && (P > 1 || big_kv_obstacle(kv8, dtype, k_strides[1], v_strides[1], esz)))
    return fail(SPA_EUNSUPPORTED, "%s: K/V of one (sequence, head) span 2 GiB or more (%s)", what,
                P > 1 ? "not supported for a ring over a packed batch" : big_kv_obstacle(kv8, dtype, k_strides[1], v_strides[1], esz));
  FwdParams p;
  p.big = big && dtype != SPA_F32;
  p.q = q; p.k = k; p.v = v; p.out = out; p.lse = lse;
  p.B = nseq; p.H = H; p.Sq = max_sq; p.Sk = max_sk;
  p.qs = S2(q_strides); p.ks = S2(k_strides); p.vs = S2(v_strides); p.os = S2(o_strides);
  p.scale = scale_eff(scale);
  p.scale_log2 = fabsf(scale_eff(scale)) * 1.4426950408889634f;
  p.negq = scale < 0.f;
  p.causal = mask_mode == SPA_MASK_CAUSAL;
  p.nqt = 0;
  p.lse_bh = (int64_t)P * total_q;
  p.part = nullptr; p.part_slot = 0; p.npart = 0;
  p.epi = SPA_EPI_PLAIN;
  p.P = 1; p.rank0 = 0; p.nranks = 1; p.t_begin = 0; p.t_count = -1;
  p.cu_q = cu_seqlens_q; p.cu_k = cu_seqlens_k;
  p.k_scale = k_scale; p.v_scale = v_scale;
  // Sequences of up to kFewRows query rows without a mask (a decode step of a batch with ragged caches): the kernel that
  // streams each sequence's K and V past its rows, as in flash_fwd above.
  if (P == 1 && !p.causal && dtype != SPA_F32 && D != 32 && !p.big && max_sq <= kFewRows && spa_knob(SPA_KNOB_FEW_ROWS) != 1 &&
      (!kv8 || (aligned16v(k, k_strides, 1) && aligned16v(v, v_strides, 1)))) {
    p.sk_last = max_sk;
    return launch_result(spa_launch_fwd_fewrows(p, D, dtype, (hipStream_t)stream), what);
  }
  if (P > 1) {
    p.P = P; p.chunk_rows = total_k; p.rank_rows = total_q;
    const int r_lo = rank < 0 ? 0 : rank, r_hi = rank < 0 ? P : rank + 1;
    if (fuse == SPA_RING_ALL_RANKS) {
      p.rank0 = r_lo; p.nranks = r_hi - r_lo;
      return launch_result(spa_launch_flash_fwd(p, D, dtype, (hipStream_t)stream), what);
    }
    for (int r = r_lo; r < r_hi; ++r) {
      p.rank0 = r; p.nranks = 1;
      const hipError_t e = spa_launch_flash_fwd(p, D, dtype, (hipStream_t)stream);
      if (e != hipSuccess) return launch_result(e, what);
    }
    return SPA_OK;
  }
  return launch_result(spa_launch_flash_fwd(p, D, dtype, (hipStream_t)stream), what);
}

// grads_in_t: as in flash_bwd above.
int flash_bwd_varlen(const char* what, const void* q, const void* k, const void* v, const void* dout, const float* lse,
                     const float* delta, void* dq, void* dk, void* dv, bool grads_in_t, const int32_t* cu_seqlens_q,
                     const int32_t* cu_seqlens_k, int nseq, int H, int total_q, int total_k, int max_sq, int max_sk,
                     int D, const int64_t q_strides[2], const int64_t k_strides[2], const int64_t v_strides[2],
                     const int64_t do_strides[2], const int64_t dq_strides[2], const int64_t dk_strides[2],
                     const int64_t dv_strides[2], float scale, int mask_mode, int dtype, void* stream) {
  if (!q || !k || !v || !dout || !lse || !delta || !dq || !dk || !dv) return fail(SPA_EINVAL, "%s: null pointer", what);
  if (!q_strides || !k_strides || !v_strides || !do_strides || !dq_strides || !dk_strides || !dv_strides)
    return fail(SPA_EINVAL, "%s: null strides", what);
  const int rc = varlen_sizes_ok(what, cu_seqlens_q, cu_seqlens_k, nseq, H, total_q, total_k, max_sq, max_sk, D, dtype,
                                 mask_mode, scale);
  if (rc != SPA_OK) return rc;
  const int esz = elem_size(dtype), gsz = grads_in_t ? esz : 4;
  if (!aligned16v(q, q_strides, esz) || !aligned16v(k, k_strides, esz) || !aligned16v(v, v_strides, esz) ||
      !aligned16v(dout, do_strides, esz) || !aligned16v(dq, dq_strides, gsz) || !aligned16v(dk, dk_strides, gsz) ||
      !aligned16v(dv, dv_strides, gsz) || (((uintptr_t)lse | (uintptr_t)delta) & 3) != 0)
    return fail(SPA_EALIGN, "%s: pointers and row strides must be 16-byte aligned", what);
  const bool big = !span_ok(max_sq, q_strides[1], D, esz) || !span_ok(max_sk, k_strides[1], D, esz) ||
                   !span_ok(max_sk, v_strides[1], D, esz) || !span_ok(max_sq, do_strides[1], D, esz);
  if (big && dtype != SPA_F32 && !(span_rebasable(q_strides[1], esz) && span_rebasable(k_strides[1], esz) &&
                                   span_rebasable(v_strides[1], esz) && span_rebasable(do_strides[1], esz)))
    return fail(SPA_EUNSUPPORTED, "%s: a tensor of one (sequence, head) spans 2 GiB or more and 128 rows of it 1 GiB or more", what);
  BwdParams p;
  p.big = big && dtype != SPA_F32;
  p.q = q; p.k = k; p.v = v; p.dout = dout; p.lse = lse; p.delta = delta;
  p.dq = (float*)dq; p.dk = (float*)dk; p.dv = (float*)dv;
  p.grads_in_t = grads_in_t;
  p.B = nseq; p.H = H; p.Sq = max_sq; p.Sk = max_sk;
  p.qs = S2(q_strides); p.ks = S2(k_strides); p.vs = S2(v_strides); p.dos = S2(do_strides);
  p.dqs = S2(dq_strides); p.dks = S2(dk_strides); p.dvs = S2(dv_strides);
  p.scale = scale_eff(scale);
  p.scale_log2 = scale_eff(scale) * 1.4426950408889634f;
  p.causal = mask_mode == SPA_MASK_CAUSAL;
  p.nqt = 0;
  p.nkt = 0;
  p.lse_bh = total_q;
  p.cu_q = cu_seqlens_q; p.cu_k = cu_seqlens_k;
  return launch_result(spa_launch_flash_bwd(p, D, dtype, (hipStream_t)stream), what);
}
}  // namespace

extern "C" {

int spa_flash_fwd_varlen(const void* q, const void* k, const void* v, void* out, float* lse,
                         const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, int nseq, int H, int total_q,
                         int total_k, int max_sq, int max_sk, int D, const int64_t q_strides[2],
                         const int64_t k_strides[2], const int64_t v_strides[2], const int64_t o_strides[2],
                         float scale, int mask_mode, int dtype, void* stream) {
  return flash_fwd_varlen("spa_flash_fwd_varlen", q, k, v, nullptr, nullptr, out, lse, cu_seqlens_q, cu_seqlens_k, nseq, H,
                          total_q, total_k, max_sq, max_sk, D, q_strides, k_strides, v_strides, o_strides, scale,
                          mask_mode, dtype, stream);
}

int spa_ring_fwd_varlen(const void* q, const void* k, const void* v, void* out, float* lse, const int32_t* cu_seqlens, int nseq,
                        int H, int shard_rows, int max_seqlen, int D, int P, int rank, const int64_t q_strides[2],
                        const int64_t k_strides[2], const int64_t v_strides[2], const int64_t o_strides[2], float scale,
                        int mask_mode, int dtype, int fuse, void* stream) {
  return flash_fwd_varlen("spa_ring_fwd_varlen", q, k, v, nullptr, nullptr, out, lse, cu_seqlens, cu_seqlens, nseq, H, shard_rows,
                          shard_rows, max_seqlen, max_seqlen, D, q_strides, k_strides, v_strides, o_strides, scale, mask_mode, dtype,
                          stream, P, rank, fuse);
}

int spa_flash_fwd_varlen_fp8kv(const void* q, const void* k8, const void* v8, const float* k_scale,
                               const float* v_scale, void* out, float* lse, const int32_t* cu_seqlens_q,
                               const int32_t* cu_seqlens_k, int nseq, int H, int total_q, int total_k, int max_sq,
                               int max_sk, int D, const int64_t q_strides[2], const int64_t k_strides[2],
                               const int64_t v_strides[2], const int64_t o_strides[2], float scale, int mask_mode,
                               int dtype, void* stream) {
  if (!k_scale || !v_scale) return fail(SPA_EINVAL, "spa_flash_fwd_varlen_fp8kv: null scale pointer");
  return flash_fwd_varlen("spa_flash_fwd_varlen_fp8kv", q, k8, v8, k_scale, v_scale, out, lse, cu_seqlens_q, cu_seqlens_k,
                          nseq, H, total_q, total_k, max_sq, max_sk, D, q_strides, k_strides, v_strides, o_strides,
                          scale, mask_mode, dtype, stream);
}

int spa_flash_bwd_varlen(const void* q, const void* k, const void* v, const void* dout, const float* lse,
                         const float* delta, float* dq_acc, float* dk_acc, float* dv_acc,
                         const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, int nseq, int H, int total_q,
                         int total_k, int max_sq, int max_sk, int D, const int64_t q_strides[2],
                         const int64_t k_strides[2], const int64_t v_strides[2], const int64_t do_strides[2],
                         const int64_t dq_strides[2], const int64_t dk_strides[2], const int64_t dv_strides[2],
                         float scale, int mask_mode, int dtype, void* stream) {
  return flash_bwd_varlen("spa_flash_bwd_varlen", q, k, v, dout, lse, delta, dq_acc, dk_acc, dv_acc, false, cu_seqlens_q,
                          cu_seqlens_k, nseq, H, total_q, total_k, max_sq, max_sk, D, q_strides, k_strides, v_strides,
                          do_strides, dq_strides, dk_strides, dv_strides, scale, mask_mode, dtype, stream);
}

int spa_flash_bwd_varlen_out(const void* q, const void* k, const void* v, const void* dout, const float* lse,
                             const float* delta, void* dq, void* dk, void* dv, const int32_t* cu_seqlens_q,
                             const int32_t* cu_seqlens_k, int nseq, int H, int total_q, int total_k, int max_sq,
                             int max_sk, int D, const int64_t q_strides[2], const int64_t k_strides[2],
                             const int64_t v_strides[2], const int64_t do_strides[2], const int64_t dq_strides[2],
                             const int64_t dk_strides[2], const int64_t dv_strides[2], float scale, int mask_mode,
                             int dtype, void* stream) {
  return flash_bwd_varlen("spa_flash_bwd_varlen_out", q, k, v, dout, lse, delta, dq, dk, dv, true, cu_seqlens_q,
                          cu_seqlens_k, nseq, H, total_q, total_k, max_sq, max_sk, D, q_strides, k_strides, v_strides,
                          do_strides, dq_strides, dk_strides, dv_strides, scale, mask_mode, dtype, stream);
}

}  // extern "C"
