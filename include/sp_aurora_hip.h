/*
 * sp_aurora_hip.h — C ABI of libsp_aurora_hip.so (gfx950 / MI355X).
 *
 * The library holds the attention hot path of sp_aurora as hand-written HIP
 * kernels: the single-block flash-attention forward that every ring step
 * calls, the update_out_and_lse merge, the Ulysses head-scatter /
 * sequence-gather re-layout, and the block-wise backward.  It is the native
 * plugin that stands where the reference's pybind11/SYCL module
 * `sp_aurora.sycl_flash_attn` stands (sp_aurora/sycl_bindings/bindings.cpp:316-369),
 * but speaks plain C: pointers, sizes, strides, a stream handle.
 *
 * Conventions shared by every entry point
 *   - All pointers are DEVICE pointers owned by the caller.  The library
 *     allocates nothing, frees nothing, and never synchronises: each call
 *     enqueues kernels on `stream` (a hipStream_t passed as void*; NULL is
 *     the default stream) and returns.
 *   - Return value: 0 on success, a negative SPA_E* code on failure; the
 *     message is available from spa_last_error() (thread-local).  Nothing
 *     throws.  On failure no kernel has been launched.
 *   - Strides are in ELEMENTS, given as int64_t[3] = {batch, head, seq}; the
 *     head-dim stride is always 1.  This one convention covers both the
 *     reference's public layout [B,S,H,D] (stride = {S*H*D, D, H*D}) and its
 *     operator layout [B,H,S,D] (stride = {H*S*D, S*D, D}), and the strided
 *     views qkv[:, :, i] of packed tensors.
 *   - Data pointers and row starts must be 16-byte aligned (every stride a
 *     multiple of 8 elements for 16-bit types, 4 for fp32).
 *   - LSE tensors are fp32, contiguous [B, H, Sq], natural log.
 *   - `dtype`: SPA_F32 / SPA_BF16 / SPA_F16 = element type of q,k,v,out.
 *   - Re-entrant; calls on distinct streams may run concurrently.
 */
#ifndef SP_AURORA_HIP_H
#define SP_AURORA_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SPA_ABI_VERSION 1

enum { SPA_F32 = 0, SPA_BF16 = 1, SPA_F16 = 2 };

/* mask_mode of the block operator.  SPA_MASK_CAUSAL is the reference's
 * top-left aligned `triu(diagonal=1)` mask (sp_aurora/intel_flash_attn.py:79-84):
 * query row i sees keys j <= i.  A ring step uses it on the diagonal block
 * pair only (sp_aurora/intel_ring_flash_attn.py:88). */
enum { SPA_MASK_NONE = 0, SPA_MASK_CAUSAL = 1 };

enum {
  SPA_OK = 0,
  SPA_EINVAL = -1,      /* bad argument (null pointer, non-positive size, bad enum) */
  SPA_EUNSUPPORTED = -2,/* head dim / dtype combination without a kernel */
  SPA_EALIGN = -3,      /* pointer or stride not 16-byte aligned */
  SPA_ELAUNCH = -4      /* HIP runtime refused the launch */
};

/* Library identity.  Replaces `is_available()` / `get_device_info()` of the
 * reference plugin (sp_aurora/sycl_bindings/bindings.cpp:298-313,357-368). */
int spa_abi_version(void);
const char* spa_last_error(void);
/* Writes a NUL-terminated "name=..;arch=..;cus=..;lds=..;clock_khz=.." line
 * for the current device into buf (at most n bytes). */
int spa_device_info(char* buf, int n);

/*
 * Block attention forward: out = softmax(q k^T * scale + mask) v,
 * lse = logsumexp(q k^T * scale + mask) over keys, fp32.
 * Replaces intel_flash_attn_forward / _flash_attn_forward
 * (sp_aurora/intel_flash_attn.py:18-126,161-163;
 *  sp_aurora/intel_flash_attn_optimized.py:95-225) and the native
 * `forward(...)` of the reference plugin (sp_aurora/sycl_bindings/bindings.cpp:50-272).
 * q: [B,H,Sq,D] by strides, k,v: [B,H,Sk,D] by strides, out: like q.
 * D in {32, 64, 128}.  Any finite scale (negative and zero included, as in the reference).
 * Any Sq, Sk >= 1.
 */
int spa_flash_fwd(const void* q, const void* k, const void* v, void* out, float* lse,
                  int B, int H, int Sq, int Sk, int D,
                  const int64_t q_strides[3], const int64_t k_strides[3],
                  const int64_t v_strides[3], const int64_t o_strides[3],
                  float scale, int mask_mode, int dtype, void* stream);

/*
 * spa_flash_fwd with K and V held as 8-bit floats (OCP e4m3, "float8_e4m3fn") plus one fp32
 * dequantisation scale per (batch, head): K = k8 * k_scale[b*H + h], V = v8 * v_scale[b*H + h].
 * q and out have element type `dtype` (SPA_BF16 or SPA_F16); k8, v8: [B,H,Sk,D] by strides in
 * ELEMENTS (= bytes), rows 8-byte aligned; k_scale, v_scale: fp32 contiguous [B,H], positive.
 * D in {64, 128}.  The tiles are widened to `dtype` between HBM and LDS (exact: every e4m3 value
 * is a bf16 and an fp16 value), both contractions run on the 16-bit MFMAs with fp32 accumulation,
 * k_scale is folded into the softmax scale and v_scale into the final normalisation, so the
 * result is that of spa_flash_fwd on the dequantised tensors up to fp32 rounding.
 * The reference has no 8-bit path; the call sites this serves are the ones that hand a KV cache
 * to the attention operator: the variable-length adapter
 * (sp_aurora/adapters/hf_adapter.py:141-155) and the call the variable-length tests are written
 * against (test/flash_attention/test_intel_ring_flash_attn_varlen.py:23-26).
 */
int spa_flash_fwd_fp8kv(const void* q, const void* k8, const void* v8,
                        const float* k_scale, const float* v_scale, void* out, float* lse,
                        int B, int H, int Sq, int Sk, int D,
                        const int64_t q_strides[3], const int64_t k_strides[3],
                        const int64_t v_strides[3], const int64_t o_strides[3],
                        float scale, int mask_mode, int dtype, void* stream);

/*
 * The block forward for calls with few query rows and many keys (a decode step against a KV cache: the call sites that hand
 * the operator a cache, adapters/hf_adapter.py:141-155): without a mask the keys can be cut into nsplit chunks that run
 * side by side on the same query rows (grid planes of one launch), each leaving its block result (out in q's type, lse)
 * in the workspace; a second kernel applies update_out_and_lse (sp_aurora/utils.py:103-104) to all of them.  The plain
 * launch has B * H * ceil(Sq / 128) workgroups however long the keys are, which leaves most of the 256 CUs idle for such a call.
 * spa_flash_fwd_splitkv_suggest returns the number of chunks the library would take for a shape (1: do not split);
 * nsplit = 1 is spa_flash_fwd.  Chunks hold a multiple of 128 keys, so fewer than nsplit may run.  bf16 / fp16, D in
 * {64, 128}, mask none, K/V below 2 GiB per (batch, head).  workspace: spa_flash_fwd_splitkv_workspace_bytes() bytes, 16-byte
 * aligned, the caller's.  _fp8kv: K / V as e4m3 bytes with scales, as for spa_flash_fwd_fp8kv.
 * With up to three query rows (and no mask, the same types and sizes; e4m3 K/V rows 16-byte aligned) these entry points and
 * spa_flash_fwd / spa_flash_fwd_fp8kv run a kernel without matrix instructions that streams K and V past the rows at the
 * rate of HBM (a 128-row tile would hold one to three live rows); spa_tune(SPA_TUNE_FEW_ROWS, 1) keeps the other kernels.
 */
int64_t spa_flash_fwd_splitkv_workspace_bytes(int B, int H, int Sq, int D, int nsplit, int dtype);
int spa_flash_fwd_splitkv_suggest(int B, int H, int Sq, int Sk, int D, int mask_mode, int dtype);
int spa_flash_fwd_splitkv(const void* q, const void* k, const void* v, void* out, float* lse, void* workspace,
                          int B, int H, int Sq, int Sk, int D, int nsplit,
                          const int64_t q_strides[3], const int64_t k_strides[3],
                          const int64_t v_strides[3], const int64_t o_strides[3],
                          float scale, int dtype, void* stream);
int spa_flash_fwd_splitkv_fp8kv(const void* q, const void* k8, const void* v8, const float* k_scale, const float* v_scale,
                                void* out, float* lse, void* workspace,
                                int B, int H, int Sq, int Sk, int D, int nsplit,
                                const int64_t q_strides[3], const int64_t k_strides[3],
                                const int64_t v_strides[3], const int64_t o_strides[3],
                                float scale, int dtype, void* stream);

/*
 * spa_flash_fwd_fp8kv with q held as e4m3 as well: Q = q8 * q_scale[b*H + h] (fp32 contiguous [B,H], positive),
 * q8 [B,H,Sq,D] by strides in bytes, rows of q8 and k8 16-byte aligned, rows of v8 8-byte aligned; out (and the
 * softmax) in `dtype` (SPA_BF16 or SPA_F16); D = 128.  The scores q8 . k8 are formed on the 8-bit matrix
 * instruction (twice the rate of the 16-bit one; a product of two e4m3 values is exact in fp32, and the
 * accumulation is fp32), q_scale * k_scale is folded into the softmax scale; V is widened to `dtype` and P V is the
 * same 16-bit contraction as in spa_flash_fwd_fp8kv.  The result is that of spa_flash_fwd on the dequantised
 * tensors up to fp32 rounding.  Same call sites as spa_flash_fwd_fp8kv; the reference has no 8-bit path.
 */
int spa_flash_fwd_fp8qkv(const void* q8, const void* k8, const void* v8,
                         const float* q_scale, const float* k_scale, const float* v_scale,
                         void* out, float* lse,
                         int B, int H, int Sq, int Sk, int D,
                         const int64_t q_strides[3], const int64_t k_strides[3],
                         const int64_t v_strides[3], const int64_t o_strides[3],
                         float scale, int mask_mode, int dtype, void* stream);

/*
 * Merge of one block result into the running (out_acc, lse_acc):
 *   lse' = logaddexp(lse, lse_b);  out' = out - sigmoid(lse_b - lse) * (out - out_b)
 * Replaces update_out_and_lse / _update_out_and_lse (sp_aurora/utils.py:47-147).
 * init != 0 is the first call of a ring (utils.py:116-122): out_acc = float(blk_out),
 * lse_acc = blk_lse.  out_acc is fp32 [B,H,Sq,D] by acc_strides; lse_acc and
 * blk_lse are fp32 contiguous [B,H,Sq]; blk_out has element type blk_dtype.
 * D must be a multiple of 8 (16-bit blocks) or 4 (fp32 blocks).
 */
int spa_merge(float* out_acc, float* lse_acc, const void* blk_out, const float* blk_lse,
              int B, int H, int Sq, int D,
              const int64_t acc_strides[3], const int64_t blk_strides[3],
              int blk_dtype, int init, void* stream);

/*
 * Ring forward of rank `rank` (or of every rank, rank = -1) on ONE device that holds the whole
 * sequence: q, k, v, out are [B,H,S,D] by strides, split into P contiguous chunks of s = S/P
 * rows; lse is fp32 contiguous [B,H,S].  For rank r, step t = 0..P-1 uses KV chunk
 * (r - t) mod P, is computed iff (mask_mode == SPA_MASK_NONE or t <= r), carries the causal
 * mask iff (mask_mode == SPA_MASK_CAUSAL and t == 0), and is merged into the running
 * (out, lse) in step order — the loop of intel_ring_flash_attn_forward
 * (sp_aurora/intel_ring_flash_attn.py:72-148) with update_out_and_lse (sp_aurora/utils.py:103-104)
 * folded into the block kernel for 16-bit types (fp32 uses spa_merge / spa_finalize kernels
 * between steps).
 * `fuse` chooses how the schedule maps onto launches (the results agree to rounding):
 *   SPA_RING_PER_STEP   one block-attention launch per visited (q chunk, kv chunk) pair, as a
 *                       multi-GPU ring would issue them; needs the workspace.  Every step but a
 *                       rank's last leaves its block output (in q's type, as the reference's
 *                       block_out) and lse there; the last step's epilogue applies
 *                       update_out_and_lse to all of them and its own block in one pass.
 *   SPA_RING_PER_RANK   one launch per rank: a workgroup keeps its query tile and its output
 *                       accumulators in registers and walks the rank's KV chunks in ring order,
 *                       so the merge is the online softmax itself and no accumulator leaves the CU.
 *   SPA_RING_ALL_RANKS  one launch for all requested ranks (heaviest first).
 * fp32 always runs per step, whatever `fuse` says.  No collectives: the "ring" is the order in
 * which chunks are visited.
 * workspace: device scratch of spa_ring_fwd_workspace_bytes() bytes (16-byte aligned), owned
 * by the caller; between separate step launches it holds one rank's earlier block results (16-bit
 * types: P - 1 outputs [B,S/P,H,D] in q's type and their lse; fp32: the running output, one block's
 * output and lse).
 * It may be NULL only when no launch needs it: 16-bit types in the fused modes, or a schedule in
 * which no rank visits more than one block (P = 1; causal rank 0).  fp32 inputs with more than
 * one block per rank always need it (SPA_EINVAL otherwise).
 * Zigzag shards: `fuse | SPA_RING_ZIGZAG` declares that the rows of q, k, v (and of out, lse) are in
 * zigzag-sharded order — with the sequence cut into 2P half-chunks, chunk r of the tensors holds
 * half-chunks r and 2P-1-r — the sharding the reference's test names and does not ship
 * (zigzag_sp_aurora_varlen_func, test/flash_attention/test_intel_ring_flash_attn_varlen.py:25,205-215).
 * Every rank of a causal ring then has the same work: step 0 is causal attention on the rank's own
 * chunk; at step t >= 1 (chunk c = (r - t) mod P) all local queries see the first half of the
 * chunk when c < r, and the second half of the local queries sees the whole chunk when c > r; all P
 * steps run for every rank.  Needs S divisible by 2P; without a mask the flag changes nothing.
 */
enum { SPA_RING_PER_STEP = 0, SPA_RING_PER_RANK = 1, SPA_RING_ALL_RANKS = 2 };
#define SPA_RING_ZIGZAG 16
int64_t spa_ring_fwd_workspace_bytes(int B, int H, int S, int D, int P, int dtype);
int spa_ring_fwd(const void* q, const void* k, const void* v, void* out, float* lse, void* workspace,
                 int B, int H, int S, int D, int P, int rank,
                 const int64_t q_strides[3], const int64_t k_strides[3],
                 const int64_t v_strides[3], const int64_t o_strides[3],
                 float scale, int mask_mode, int dtype, int fuse, void* stream);

/*
 * spa_ring_fwd with e4m3 K / V as in spa_flash_fwd_fp8kv: k8, v8 [B,H,S,D] by strides in bytes,
 * k_scale / v_scale fp32 contiguous [B,H] — one scale per (batch, head) for the whole sequence, i.e.
 * every ring chunk quantised on the same grid (a ring whose ranks quantise their chunks on their
 * own would rescale to a common scale before the exchange).  q / out bf16 or fp16, D in {64, 128};
 * all three `fuse` modes; workspace as for spa_ring_fwd.  Same call sites as spa_flash_fwd_fp8kv,
 * seen from the ring loop (sp_aurora/intel_ring_flash_attn.py:72-148).
 */
int spa_ring_fwd_fp8kv(const void* q, const void* k8, const void* v8,
                       const float* k_scale, const float* v_scale,
                       void* out, float* lse, void* workspace,
                       int B, int H, int S, int D, int P, int rank,
                       const int64_t q_strides[3], const int64_t k_strides[3],
                       const int64_t v_strides[3], const int64_t o_strides[3],
                       float scale, int mask_mode, int dtype, int fuse, void* stream);

/*
 * spa_ring_fwd with q, K, V all e4m3 as in spa_flash_fwd_fp8qkv (q_scale, k_scale, v_scale fp32 contiguous [B,H], one
 * scale per (batch, head) for the whole sequence; D = 128; out and the ring-step slots in `dtype`, bf16 or fp16): the
 * scores of every block pair run on the 8-bit matrix instruction.  All three `fuse` modes, contiguous chunks (no
 * SPA_RING_ZIGZAG); workspace as for spa_ring_fwd.  The reference has no 8-bit path.
 */
int spa_ring_fwd_fp8qkv(const void* q8, const void* k8, const void* v8,
                        const float* q_scale, const float* k_scale, const float* v_scale,
                        void* out, float* lse, void* workspace,
                        int B, int H, int S, int D, int P, int rank,
                        const int64_t q_strides[3], const int64_t k_strides[3],
                        const int64_t v_strides[3], const int64_t o_strides[3],
                        float scale, int mask_mode, int dtype, int fuse, void* stream);

/*
 * One launch per rank for a ring whose KV chunks ARRIVE while the launch runs (a receive buffer filled by a
 * communication stream): spa_ring_fwd(fuse = SPA_RING_PER_RANK) whose workgroups, before they request the first tile
 * of chunk c, wait until arrive[c] >= epoch.  The flag is read past the caches (a relaxed load at system scope) in a
 * bounded spin: after spin_limit polls (about 1 us each) a wave gives up, stores 1 to *fault and goes on with whatever
 * the buffer holds, so the grid always drains; the caller checks *fault after synchronising (and clears it before).
 * The kernel requests no byte of a chunk before it has seen the chunk's flag, so no cache can hold the buffer's earlier
 * contents; for that to hold per cache line, every K / V chunk of every (batch, head) must start on a 128-byte boundary
 * (SPA_EALIGN otherwise).  The query tile and
 * the accumulators stay in registers across ring steps, i.e. the per-step loop of intel_ring_flash_attn_forward
 * (sp_aurora/intel_ring_flash_attn.py:72-134: compute step t while chunk t+1 is in flight, :96-134) at the speed of
 * the one-launch form, without a launch, a Q re-read and an (out, lse) round trip per step.  The producer raises a
 * flag AFTER the chunk's bytes are visible device-wide: spa_ring_flag_set on the stream that moved the chunk, or a
 * release store at system scope from a kernel.  The producer must be able to run while the launch waits: HIP streams share
 * a few hardware queues, and work queued behind the waiting launch on the same queue starts only when the launch has
 * given up (use a stream seen to run beside the consumer's, another process or a peer).
 * Epochs let a flag array be reused without clearing (use a larger
 * epoch per call); the rank's own chunk has a flag like the others.  bf16 / fp16, D in {64, 128}, contiguous chunks;
 * rank >= 0 or -1 (every rank, one launch each).  arrive: uint32[P], fault: uint32[1], device memory.
 * The reference has no counterpart (its steps are separate kernel launches around blocking waits).
 */
int spa_ring_fwd_flags(const void* q, const void* k, const void* v, void* out, float* lse,
                       const uint32_t* arrive, uint32_t epoch, uint32_t spin_limit, uint32_t* fault,
                       int B, int H, int S, int D, int P, int rank,
                       const int64_t q_strides[3], const int64_t k_strides[3],
                       const int64_t v_strides[3], const int64_t o_strides[3],
                       float scale, int mask_mode, int dtype, void* stream);
/* The same for e4m3 q, k, v (spa_ring_fwd_fp8qkv's tensors and scales: D = 128, scores on the 8-bit matrix instruction,
 * out in `dtype`; strides of q, k, v in bytes). */
int spa_ring_fwd_flags_fp8qkv(const void* q8, const void* k8, const void* v8, const float* q_scale, const float* k_scale,
                              const float* v_scale, void* out, float* lse, const uint32_t* arrive, uint32_t epoch,
                              uint32_t spin_limit, uint32_t* fault, int B, int H, int S, int D, int P, int rank,
                              const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                              const int64_t o_strides[3], float scale, int mask_mode, int dtype, void* stream);
/* arrive[chunk] = epoch, ordered after everything enqueued before it on `stream` (a stream memory operation: no kernel). */
int spa_ring_flag_set(uint32_t* arrive, int chunk, uint32_t epoch, void* stream);

/*
 * spa_ring_fwd for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): the same call without the workspace
 * argument.  The scratch is a fixed buffer of SPA_STATIC_SCRATCH_BYTES inside the library's
 * code object (every device the library is loaded on holds its own copy until the process
 * ends); the call allocates and frees nothing.  Sizes whose spa_ring_fwd_workspace_bytes()
 * exceed the buffer are rejected with SPA_EINVAL when the schedule needs the scratch.  All calls
 * on one device share that device's buffer: calls that overlap in time on one device (two
 * streams, two threads) race; serialise them.  Same kernels, same results as spa_ring_fwd.
 * Cost: SPA_STATIC_SCRATCH_BYTES (32 MiB) of device memory on every device the library is loaded
 * on, whether or not this entry point is ever called.
 * Before a stream capture: the device address of the buffer is looked up (hipGetSymbolAddress) on
 * the first use per device, and every kernel variant sets its dynamic-LDS attribute on its first
 * launch per device; neither belongs into a capture.  Call spa_static_scratch_init() with the
 * device current, and make one eager call with the shapes to be captured, before capturing.
 * These entry points have no counterpart in the reference.
 */
#define SPA_STATIC_SCRATCH_BYTES (32 << 20)
int64_t spa_static_scratch_bytes(void);
/* Looks up the buffer's address on the current device (idempotent, allocates nothing, launches
 * nothing).  SPA_OK or SPA_ELAUNCH. */
int spa_static_scratch_init(void);
int spa_ring_fwd_static(const void* q, const void* k, const void* v, void* out, float* lse,
                        int B, int H, int S, int D, int P, int rank,
                        const int64_t q_strides[3], const int64_t k_strides[3],
                        const int64_t v_strides[3], const int64_t o_strides[3],
                        float scale, int mask_mode, int dtype, int fuse, void* stream);

/* out = cast(out_acc) — the `out.to(q.dtype)` that closes a ring forward
 * (sp_aurora/intel_ring_flash_attn.py:141-143). */
int spa_finalize(void* out, const float* out_acc,
                 int B, int H, int Sq, int D,
                 const int64_t o_strides[3], const int64_t acc_strides[3],
                 int dtype, void* stream);

/*
 * Ulysses re-layout, all P ranks' shards stacked on a leading axis of one
 * device buffer.  `pack` = 1 for a 4-D tensor, 2 / 3 for kv- / qkv-packed
 * 5-D tensors (the packed axis sits between sequence and heads).
 *   s2h (scatter heads, gather sequence):
 *     x [P][B, s, pack, H, D]  ->  y [P][B, P*s, pack, H/P, D]
 *     y[r][b, q*s+t, c, j, :] = x[q][b, t, c, r*(H/P)+j, :]
 *   h2s (scatter sequence, gather heads) is its inverse.
 * Replaces the reshape/transpose/contiguous + all_to_all_single chains of
 * intel_all_to_all_4d (sp_aurora/intel_ulysses_attn.py:60-143),
 * all_to_all_4D and all_to_all_5D (sp_aurora/comm/all_to_all.py:17-180,228-335).
 * elem_bytes in {1,2,4,8}; H must be divisible by P.  Pure byte movement.
 */
int spa_relayout_s2h(const void* x, void* y, int P, int B, int s, int H, int D,
                     int pack, int elem_bytes, void* stream);
int spa_relayout_h2s(const void* y, void* x, int P, int B, int s, int H, int D,
                     int pack, int elem_bytes, void* stream);

/*
 * delta[b,h,i] = sum_d dout[b,h,i,d] * out[b,h,i,d]   (fp32, [B,H,Sq] contiguous)
 * First pass of the block-wise backward; the reference obtains the same term
 * implicitly through autograd (sp_aurora/intel_ring_flash_attn.py:229-244).
 */
int spa_bwd_delta(const void* out, const void* dout, float* delta,
                  int B, int H, int Sq, int D,
                  const int64_t o_strides[3], const int64_t do_strides[3],
                  int dtype, void* stream);

/*
 * Block-wise backward of one (q chunk, kv chunk) pair with the GLOBAL lse
 * and delta of the q chunk's rows:
 *   P = exp(q k^T * scale + mask - lse);  dV += P^T dO;  dP = dO V^T;
 *   dS = P * (dP - delta);  dQ += dS K * scale;  dK += dS^T Q * scale.
 * dq_acc [B,H,Sq,D], dk_acc / dv_acc [B,H,Sk,D]: fp32, ACCUMULATED into (the
 * caller zeroes them before the first block pair of a chunk); strides as given.
 * Replaces the per-step body of intel_ring_flash_attn_backward
 * (sp_aurora/intel_ring_flash_attn.py:192-258).
 */
int spa_flash_bwd(const void* q, const void* k, const void* v, const void* dout,
                  const float* lse, const float* delta,
                  float* dq_acc, float* dk_acc, float* dv_acc,
                  int B, int H, int Sq, int Sk, int D,
                  const int64_t q_strides[3], const int64_t k_strides[3],
                  const int64_t v_strides[3], const int64_t do_strides[3],
                  const int64_t dq_strides[3], const int64_t dk_strides[3],
                  const int64_t dv_strides[3],
                  float scale, int mask_mode, int dtype, void* stream);

/*
 * spa_flash_bwd for a gradient that ONE call computes in full (a whole block, or a whole simulated
 * ring over the full-sequence tensors): dq [B,H,Sq,D], dk / dv [B,H,Sk,D] have the inputs' element
 * type `dtype` and are WRITTEN, not added to - no fp32 accumulators to zero, read back and cast.
 * The values are those of spa_flash_bwd into zeroed accumulators followed by the reference's final
 * cast to q's type (sp_aurora/intel_ring_flash_attn.py:250-271), bit for bit; rows of dk / dv that
 * no query sees (causal with Sk > Sq) are written as zeros.
 */
int spa_flash_bwd_out(const void* q, const void* k, const void* v, const void* dout,
                      const float* lse, const float* delta,
                      void* dq, void* dk, void* dv,
                      int B, int H, int Sq, int Sk, int D,
                      const int64_t q_strides[3], const int64_t k_strides[3],
                      const int64_t v_strides[3], const int64_t do_strides[3],
                      const int64_t dq_strides[3], const int64_t dk_strides[3],
                      const int64_t dv_strides[3],
                      float scale, int mask_mode, int dtype, void* stream);

/*
 * Block attention over a batch of sequences of different lengths packed back
 * to back (no padding): q / out are [total_q, H, D], k / v [total_k, H, D];
 * sequence b owns query rows cu_seqlens_q[b] .. cu_seqlens_q[b+1] and key rows
 * cu_seqlens_k[b] .. cu_seqlens_k[b+1] and attends to nothing else.
 * cu_seqlens_*: int32[nseq + 1] in DEVICE memory, non-decreasing, first 0,
 * last = total_*; max_sq / max_sk >= the longest sequence (they size the grid:
 * rows past max_sq of a longer sequence would be left unwritten).  The library
 * cannot read the arrays on the host, the caller vouches for them.
 * lse: fp32 [H, total_q].  A sequence with queries but no keys gets out = 0,
 * lse = -inf.  mask_mode causal is aligned top-left within each sequence.
 * *_strides = element strides of (head, row); head-dim stride is 1.
 * This is the call the reference's variable-length entry points are written
 * against: sp_aurora_varlen_func(q, k, v, cu_seqlens_q, cu_seqlens_k,
 * max_seqlen, ...) in test/flash_attention/test_intel_ring_flash_attn_varlen.py:23-26,66-74
 * (the function itself is missing from the reference), and the packed lse
 * layout of flatten_varlen_lse (sp_aurora/utils.py:150-157).
 * With max_sq <= 3 and no mask (a decode step of a batch whose caches differ in length; bf16 / fp16, D in {64, 128}) the call
 * runs on the kernel that streams each sequence's K and V past its rows, as spa_flash_fwd does (also _fp8kv).
 */
int spa_flash_fwd_varlen(const void* q, const void* k, const void* v, void* out, float* lse,
                         const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                         int nseq, int H, int total_q, int total_k, int max_sq, int max_sk, int D,
                         const int64_t q_strides[2], const int64_t k_strides[2],
                         const int64_t v_strides[2], const int64_t o_strides[2],
                         float scale, int mask_mode, int dtype, void* stream);

/*
 * The ring over a packed variable-length batch in one launch per rank (or one for all ranks): the reference's varlen test
 * runs its function under a process group (test/flash_attention/test_intel_ring_flash_attn_varlen.py:150-215), i.e. every
 * rank holds the r-th of P equal slices of EVERY sequence, packed alike on every rank.  q, k, v, out: the P shards stacked,
 * [P * shard_rows, H, D]; cu_seqlens [nseq + 1] describes one shard; lse [H, P * shard_rows].  Rank r walks the shards
 * r, r-1, ... as spa_ring_fwd does (the causal mask inside each sequence at step 0 only), the query tile and the accumulators
 * in registers across the shards.  fuse = SPA_RING_PER_RANK or SPA_RING_ALL_RANKS; rank >= 0 or -1; bf16 / fp16.
 */
int spa_ring_fwd_varlen(const void* q, const void* k, const void* v, void* out, float* lse,
                        const int32_t* cu_seqlens, int nseq, int H, int shard_rows, int max_seqlen, int D, int P, int rank,
                        const int64_t q_strides[2], const int64_t k_strides[2],
                        const int64_t v_strides[2], const int64_t o_strides[2],
                        float scale, int mask_mode, int dtype, int fuse, void* stream);

/*
 * spa_flash_fwd_varlen with e4m3 K / V as in spa_flash_fwd_fp8kv: k8, v8 [total_k, H, D] by
 * (head, row) strides in bytes, k_scale / v_scale fp32 contiguous [nseq, H] (one scale per
 * sequence and head).  Same call sites as spa_flash_fwd_fp8kv.
 */
int spa_flash_fwd_varlen_fp8kv(const void* q, const void* k8, const void* v8,
                               const float* k_scale, const float* v_scale, void* out, float* lse,
                               const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                               int nseq, int H, int total_q, int total_k, int max_sq, int max_sk, int D,
                               const int64_t q_strides[2], const int64_t k_strides[2],
                               const int64_t v_strides[2], const int64_t o_strides[2],
                               float scale, int mask_mode, int dtype, void* stream);

/*
 * Backward of spa_flash_fwd_varlen, same packing.  lse and delta: fp32
 * [H, total_q] (delta from spa_bwd_delta with B = 1, Sq = total_q);
 * dq_acc [total_q, H, D], dk_acc / dv_acc [total_k, H, D]: fp32, ACCUMULATED
 * into, strides (head, row) as given.  What out.backward() of the reference's
 * variable-length test needs (test_intel_ring_flash_attn_varlen.py:85-91).
 */
int spa_flash_bwd_varlen(const void* q, const void* k, const void* v, const void* dout,
                         const float* lse, const float* delta,
                         float* dq_acc, float* dk_acc, float* dv_acc,
                         const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                         int nseq, int H, int total_q, int total_k, int max_sq, int max_sk, int D,
                         const int64_t q_strides[2], const int64_t k_strides[2],
                         const int64_t v_strides[2], const int64_t do_strides[2],
                         const int64_t dq_strides[2], const int64_t dk_strides[2],
                         const int64_t dv_strides[2],
                         float scale, int mask_mode, int dtype, void* stream);

/*
 * spa_flash_bwd_varlen for the whole gradient in one call, as spa_flash_bwd_out is to spa_flash_bwd:
 * dq [total_q, H, D], dk / dv [total_k, H, D] have the inputs' element type and are WRITTEN (zeros
 * where a sequence has queries but no keys, or keys that no query sees).  Rows that belong to no
 * sequence, or that lie past max_sq / max_sk of a longer sequence, are left untouched.  Same
 * call site as spa_flash_bwd_varlen (test_intel_ring_flash_attn_varlen.py:85-91).
 */
int spa_flash_bwd_varlen_out(const void* q, const void* k, const void* v, const void* dout,
                             const float* lse, const float* delta,
                             void* dq, void* dk, void* dv,
                             const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                             int nseq, int H, int total_q, int total_k, int max_sq, int max_sk, int D,
                             const int64_t q_strides[2], const int64_t k_strides[2],
                             const int64_t v_strides[2], const int64_t do_strides[2],
                             const int64_t dq_strides[2], const int64_t dk_strides[2],
                             const int64_t dv_strides[2],
                             float scale, int mask_mode, int dtype, void* stream);

/*
 * Kernel-variant override for experiments and tests; no counterpart in the reference and not
 * needed in production (value 0 restores the library's own choice).  Process-wide.
 *   SPA_TUNE_FWD_GROUPS    1 | 2   wave groups per forward workgroup
 *   SPA_TUNE_FWD_SHARE     1 | 2   1 = 128-row workgroups, private K/V buffers per wave group;
 *                                  2 = 256-row workgroups sharing one set of buffers
 *   SPA_TUNE_BWD_DQ_WAVES  4 | 8   waves per workgroup of the backward's dq kernel
 *   SPA_TUNE_BWD_DKDV_FORM 1       compiler-scheduled MFMAs in the D = 128 dk/dv kernel
 *   SPA_TUNE_FWD32_SPLIT  1 | 2    never / whenever D <= 64: the fp32 forward with 32-row workgroups whose waves share
 *                                  the key tiles (the library takes it when 128-row workgroups would leave half the CUs idle)
 *   SPA_TUNE_FEW_ROWS     1        a key-split forward of up to 4 query rows runs on the MFMA kernels instead of the
 *                                  kernel that streams K and V past those rows
 */
enum { SPA_TUNE_FWD_GROUPS = 0, SPA_TUNE_FWD_SHARE = 1, SPA_TUNE_BWD_DQ_WAVES = 2, SPA_TUNE_BWD_DKDV_FORM = 3, SPA_TUNE_FWD32_SPLIT = 4, SPA_TUNE_FEW_ROWS = 5 };
int spa_tune(int knob, int value);

#ifdef __cplusplus
}
#endif
#endif /* SP_AURORA_HIP_H */
