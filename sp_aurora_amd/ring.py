"""Ring attention with the reference's public signatures, on one GPU.

Mirrors sp_aurora/intel_ring_flash_attn.py: the step schedule of
intel_ring_flash_attn_forward (:72-148) and intel_ring_flash_attn_backward (:153-271),
IntelRingFlashAttnFunc (:274-341) and the three public functions (:344-449) with their
aliases (:453-456).

One GPU holds every rank's shard, so the ring is SIMULATED: rank r's query chunk walks
KV chunks r, r-1, ... in ring order, one block-attention launch per step, merged with
update_out_and_lse semantics.  There are no collectives; passing a process group (or
running under an initialised torch.distributed world of more than one rank) raises.

Additive, keyword-only extensions of the reference signatures:
    ring_size=P   split the given sequence into P contiguous shards and run every rank
                  (ring_size=1 is the reference's single-process path: one block over the
                  whole sequence, sp_aurora/intel_ring_flash_attn.py:415-435).
    sharding="zigzag"   the rows of the given tensors are in zigzag-sharded order (zigzag_order):
                  shard r holds half-chunks r and 2P-1-r of the sequence, so that every rank of a
                  causal ring has the same work; the sharding the reference's test names without
                  shipping it (test/flash_attention/test_intel_ring_flash_attn_varlen.py:25,205-215).
                  Results (and gradients) come back in the same row order.
"""
import torch
import torch.distributed as dist

from . import ops
from .flash_attn import _check_unsupported

__all__ = [
    "zigzag_order", "ring_flash_attn_forward_rank", "ring_flash_attn_forward", "ring_flash_attn_backward", "make_ring_forward_step",
    "RingFlashAttnFunc", "IntelRingFlashAttnFunc",
    "ring_flash_attn_func", "ring_flash_attn_kvpacked_func", "ring_flash_attn_qkvpacked_func",
    "intel_ring_flash_attn_func", "intel_ring_flash_attn_kvpacked_func", "intel_ring_flash_attn_qkvpacked_func",
    "sp_aurora_func", "sp_aurora_kvpacked_func", "sp_aurora_qkvpacked_func",
]


def _no_multi_gpu(group):
    if group is not None or (dist.is_available() and dist.is_initialized() and dist.get_world_size() > 1):
        raise NotImplementedError(
            "this build runs the ring on one GPU (ring_size=P simulates the P ranks); "
            "process groups / multi-GPU rings are not part of it")


def zigzag_order(S, ring_size, device=None):
    """Row order of zigzag shards: idx (int64 [S]) with sharded = natural.index_select(1, idx).  The S rows
    are cut into 2P half-chunks; shard r is half-chunk r followed by half-chunk 2P-1-r."""
    P = int(ring_size)
    if P < 1 or S % (2 * P):
        raise ValueError(f"zigzag sharding needs 2 * ring_size = {2 * P} to divide the sequence length {S}")
    hc = S // (2 * P)
    halves = torch.arange(2 * P, device=device).view(2, P)
    order = torch.stack([halves[0], halves[1].flip(0)], dim=1).reshape(-1)  # r, 2P-1-r for r = 0 .. P-1
    return (order[:, None] * hc + torch.arange(hc, device=device)[None, :]).reshape(-1)


def _check_sharding(sharding, S, P):
    if sharding not in ("contiguous", "zigzag"):
        raise ValueError(f"sharding must be 'contiguous' or 'zigzag', got {sharding!r}")
    if sharding == "zigzag" and S % (2 * P):
        raise ValueError(f"zigzag sharding needs 2 * ring_size = {2 * P} to divide the sequence length {S}")
    return sharding == "zigzag"


class _RingWorkspace:
    """Per-call scratch of the simulated ring: one block result and the fp32 accumulators."""

    def __init__(self, B, s, H, D, dtype, device):
        self.blk_out = torch.empty((B, s, H, D), dtype=dtype, device=device)
        self.blk_lse = torch.empty((B, H, s), dtype=torch.float32, device=device)
        self.acc = torch.empty((B, s, H, D), dtype=torch.float32, device=device)


def ring_flash_attn_forward_rank(q_local, k_chunks, v_chunks, rank, softmax_scale=None, causal=False,
                                 out=None, lse=None, workspace=None):
    """What rank `rank` of a ring of P = len(k_chunks) computes, on this GPU, spelled out with the
    stand-alone kernels: block attention, then update_out_and_lse as its own pass, per step.
    (ring_flash_attn_forward reaches the same result through the C ring driver, which folds the
    merge into the attention kernel's epilogue.)

    Step t uses KV chunk (rank - t) mod P; it is computed iff `not causal or t <= rank`
    and carries the diagonal mask iff `causal and t == 0`
    (sp_aurora/intel_ring_flash_attn.py:75-95); results are merged in step order (:128)
    and cast to q's dtype at the end (:143).
    q_local, chunks: [B,s,H,D].  Returns out [B,s,H,D] (q dtype), lse fp32 [B,H,s].
    """
    P = len(k_chunks)
    B, s, H, D = q_local.shape
    if out is None:
        out = torch.empty((B, s, H, D), dtype=q_local.dtype, device=q_local.device)
    if lse is None:
        lse = torch.empty((B, H, s), dtype=torch.float32, device=q_local.device)
    steps = [t for t in range(P) if not causal or t <= rank]
    if len(steps) == 1:
        # a single visited block: its result is the answer, no accumulator round trip
        c = (rank - steps[0]) % P
        ops.flash_fwd(q_local, k_chunks[c], v_chunks[c], softmax_scale, causal and steps[0] == 0,
                      layout="bshd", out=out, lse=lse)
        return out, lse
    ws = workspace or _RingWorkspace(B, s, H, D, q_local.dtype, q_local.device)
    for i, t in enumerate(steps):
        c = (rank - t) % P
        ops.flash_fwd(q_local, k_chunks[c], v_chunks[c], softmax_scale, causal and t == 0,
                      layout="bshd", out=ws.blk_out, lse=ws.blk_lse)
        ops.merge(ws.acc, lse, ws.blk_out, ws.blk_lse, layout="bshd", init=(i == 0))
    ops.finalize(ws.acc, q_local.dtype, layout="bshd", out=out)
    return out, lse


def ring_flash_attn_forward(q, k, v, softmax_scale=None, causal=False, ring_size=1, out=None, lse=None,
                            workspace=None, fuse="rank", sharding="contiguous"):
    """All ranks of a simulated ring over contiguous shards of q,k,v [B,S,H,D]: one call into the
    C ring driver, which enqueues the block-pair kernels in ring order and merges each step in the
    kernel epilogue.  Returns out [B,S,H,D] (q dtype) and lse fp32 [B,H,S]; `out`, `lse`,
    `workspace` (ops.ring_fwd_workspace) may be passed in to run without allocating.
    sharding="zigzag": the rows are in zigzag-sharded order (see the module docstring)."""
    B, S, H, D = q.shape
    P = int(ring_size)
    if P < 1 or S % P or (P > 1 and k.shape[1] != S):
        raise ValueError(f"ring_size={P} must divide the sequence length {S} (and k/v must match q)")
    _check_sharding(sharding, S, P)
    if P == 1:
        return ops.flash_fwd(q, k, v, softmax_scale, causal, layout="bshd", out=out, lse=lse)
    return ops.ring_fwd(q, k, v, P, softmax_scale, causal, rank=-1, layout="bshd", out=out, lse=lse,
                        workspace=workspace, fuse=fuse, sharding=sharding)


def make_ring_forward_step(q, k, v, softmax_scale=None, causal=False, ring_size=1, fuse="rank", sharding="contiguous"):
    """Preallocates every buffer ring_flash_attn_forward needs and returns a zero-argument
    callable that runs the whole ring forward into them and returns (out, lse)."""
    B, S, H, D = q.shape
    P = int(ring_size)
    out = torch.empty((B, S, H, D), dtype=q.dtype, device=q.device)
    lse = torch.empty((B, H, S), dtype=torch.float32, device=q.device)
    ws = ops.ring_fwd_workspace(q, P) if P > 1 else None

    def step():
        return ring_flash_attn_forward(q, k, v, softmax_scale, causal, P, out=out, lse=lse, workspace=ws, fuse=fuse,
                                       sharding=sharding)

    return step


def _zigzag_pairs(P):
    """The block pairs of a causal zigzag ring, in the ring's order: (rank, chunk, query rows, key rows,
    masked) with rows as 'all', 'first' or 'second' half of the shard."""
    for r in range(P):
        yield r, r, "all", "all", True
        for t in range(1, P):
            c = (r - t) % P
            yield (r, c, "all", "first", False) if c < r else (r, c, "second", "all", False)


def ring_flash_attn_backward(dout, q, k, v, out, softmax_lse, softmax_scale=None, causal=False, ring_size=1,
                             fuse="all", sharding="contiguous"):
    """dq, dk, dv of ring attention by block-wise recompute with the global lse.

    The schedule is the reference's (sp_aurora/intel_ring_flash_attn.py:192-271): per visited
    (q chunk, kv chunk) pair one backward block, dq summed per q chunk in fp32 (:250-255),
    dk/dv summed per kv chunk over the q chunks that visited it (:257-258,267), cast at the
    end (:271).  Each block uses P = exp(S - lse) with the lse of the WHOLE ring, which makes
    the sum the exact gradient (the reference normalises each block on its own, :229-244).

    fuse="step" launches one backward block per visited pair, in the reference's order, adding
    into the fp32 accumulators (what a rank of a real ring does as chunks arrive); fuse="all"
    walks the same pairs inside one launch of each kernel (the blocks of a simulated ring tile
    the causal / full score matrix exactly, and with a shared global lse their sum is the
    backward of attention over the whole sequence), accumulators in registers.

    sharding="zigzag" (rows in zigzag-sharded order, causal): fuse="step" launches the zigzag ring's
    block pairs (own shard masked; all rows x first half of an earlier rank's shard; second half of
    the rows x a later rank's whole shard); fuse="all" brings the rows into natural order with one
    gather per tensor, runs the one-launch backward there and scatters the gradients back.
    """
    if fuse not in ("step", "all"):
        raise ValueError(f"fuse must be 'step' or 'all', got {fuse!r}")
    B, S, H, D = q.shape
    P = int(ring_size)
    zig = _check_sharding(sharding, S, P) and causal and P > 1
    lse = softmax_lse if softmax_lse.is_contiguous() else softmax_lse.contiguous()
    if zig and fuse == "all":
        idx = zigzag_order(S, P, q.device)
        inv = torch.argsort(idx)
        nat = lambda t: t.index_select(1, inv)
        grads = ring_flash_attn_backward(nat(dout), nat(q), nat(k), nat(v), nat(out), lse.index_select(2, inv), softmax_scale,
                                         True, P, fuse="all")
        return tuple(g.index_select(1, idx) for g in grads)
    delta = ops.bwd_delta(out, dout, layout="bshd")
    if zig:
        dq, dk, dv = (torch.zeros((B, S, H, D), dtype=torch.float32, device=q.device) for _ in range(3))
        s, hs = S // P, S // (2 * P)
        rows = lambda r, part: slice(r * s + (hs if part == "second" else 0), r * s + (hs if part == "first" else s))
        for r, c, qpart, kpart, masked in _zigzag_pairs(P):
            qs, ks = rows(r, qpart), rows(c, kpart)
            ops.flash_bwd(q[:, qs], k[:, ks], v[:, ks], dout[:, qs], lse[:, :, qs].contiguous(), delta[:, :, qs].contiguous(),
                          dq[:, qs], dk[:, ks], dv[:, ks], softmax_scale, masked, layout="bshd")
        return dq.to(q.dtype), dk.to(k.dtype), dv.to(v.dtype)
    if P == 1 or fuse == "all":
        # one launch of each kernel computes the whole gradient: written in q's dtype, no fp32 accumulators
        return ops.flash_bwd_out(q, k, v, dout, lse, delta, softmax_scale, causal, layout="bshd")
    dq = torch.zeros((B, S, H, D), dtype=torch.float32, device=q.device)
    dk = torch.zeros((B, k.shape[1], H, D), dtype=torch.float32, device=q.device)
    dv = torch.zeros((B, k.shape[1], H, D), dtype=torch.float32, device=q.device)
    s = S // P
    for r in range(P):
        rs = slice(r * s, (r + 1) * s)
        lse_r = lse[:, :, rs].contiguous()
        delta_r = delta[:, :, rs].contiguous()
        for t in range(P):
            if causal and t > r:
                continue
            c = (r - t) % P
            cs = slice(c * s, (c + 1) * s)
            ops.flash_bwd(q[:, rs], k[:, cs], v[:, cs], dout[:, rs], lse_r, delta_r,
                          dq[:, rs], dk[:, cs], dv[:, cs], softmax_scale, causal and t == 0, layout="bshd")
    return dq.to(q.dtype), dk.to(k.dtype), dv.to(v.dtype)


class RingFlashAttnFunc(torch.autograd.Function):
    """Mirrors IntelRingFlashAttnFunc (sp_aurora/intel_ring_flash_attn.py:274-341)."""

    @staticmethod
    def forward(ctx, q, k, v, dropout_p, softmax_scale, causal, window_size, alibi_slopes, deterministic,
                return_softmax, group, ring_size=1, sharding="contiguous"):
        if softmax_scale is None:
            softmax_scale = q.shape[-1] ** (-0.5)
        _check_unsupported(dropout_p, window_size, alibi_slopes)
        _no_multi_gpu(group)
        out, softmax_lse = ring_flash_attn_forward(q, k, v, softmax_scale, causal, ring_size, sharding=sharding)
        ctx.save_for_backward(q, k, v, out, softmax_lse)
        ctx.softmax_scale = softmax_scale
        ctx.causal = causal
        ctx.ring_size = ring_size
        ctx.sharding = sharding
        ctx.mark_non_differentiable(softmax_lse)
        return out if not return_softmax else (out, softmax_lse, None)

    @staticmethod
    def backward(ctx, dout, *args):
        q, k, v, out, softmax_lse = ctx.saved_tensors
        dq, dk, dv = ring_flash_attn_backward(dout, q, k, v, out, softmax_lse, ctx.softmax_scale, ctx.causal,
                                              ctx.ring_size, sharding=ctx.sharding)
        return dq, dk, dv, None, None, None, None, None, None, None, None, None, None


IntelRingFlashAttnFunc = RingFlashAttnFunc


def ring_flash_attn_qkvpacked_func(qkv, dropout_p=0.0, softmax_scale=None, causal=False, window_size=(-1, -1),
                                   alibi_slopes=None, deterministic=False, return_attn_probs=False, group=None,
                                   *, ring_size=1, sharding="contiguous"):
    """qkv [B,S,3,H,D]; the strided views qkv[:, :, i] go to the kernels as they are
    (sp_aurora/intel_ring_flash_attn.py:344-368)."""
    return RingFlashAttnFunc.apply(qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2], dropout_p, softmax_scale, causal,
                                   window_size, alibi_slopes, deterministic, return_attn_probs, group, ring_size, sharding)


def ring_flash_attn_kvpacked_func(q, kv, dropout_p=0.0, softmax_scale=None, causal=False, window_size=(-1, -1),
                                  alibi_slopes=None, deterministic=False, return_attn_probs=False, group=None,
                                  *, ring_size=1, sharding="contiguous"):
    """q [B,S,H,D], kv [B,S,2,H,D] (sp_aurora/intel_ring_flash_attn.py:371-396)."""
    return RingFlashAttnFunc.apply(q, kv[:, :, 0], kv[:, :, 1], dropout_p, softmax_scale, causal, window_size,
                                   alibi_slopes, deterministic, return_attn_probs, group, ring_size, sharding)


def ring_flash_attn_func(q, k, v, dropout_p=0.0, softmax_scale=None, causal=False, window_size=(-1, -1),
                         alibi_slopes=None, deterministic=False, return_attn_probs=False, group=None,
                         *, ring_size=1, sharding="contiguous"):
    """q,k,v [B,S,H,D] -> out [B,S,H,D], or (out, lse fp32 [B,H,S], None) with return_attn_probs
    (sp_aurora/intel_ring_flash_attn.py:399-449)."""
    return RingFlashAttnFunc.apply(q, k, v, dropout_p, softmax_scale, causal, window_size, alibi_slopes,
                                   deterministic, return_attn_probs, group, ring_size, sharding)


# names the reference package exports (sp_aurora/__init__.py:59-63) and its own
# module-level names (sp_aurora/intel_ring_flash_attn.py:344-456)
intel_ring_flash_attn_func = ring_flash_attn_func
intel_ring_flash_attn_kvpacked_func = ring_flash_attn_kvpacked_func
intel_ring_flash_attn_qkvpacked_func = ring_flash_attn_qkvpacked_func
# names the reference documents (README.md:46,59,78-80)
sp_aurora_func = ring_flash_attn_func
sp_aurora_kvpacked_func = ring_flash_attn_kvpacked_func
sp_aurora_qkvpacked_func = ring_flash_attn_qkvpacked_func
