"""Attention over packed variable-length batches (`cu_seqlens`), on one GPU.

The reference's tests and adapter are written against sp_aurora_varlen_func(q, k, v,
cu_seqlens_q, cu_seqlens_k, max_seqlen=..., dropout_p=..., causal=...)
(test/flash_attention/test_intel_ring_flash_attn_varlen.py:23-26,66-74,85-91) but the
reference does not ship the function; only the lse helpers exist (sp_aurora/utils.py:150-169).
Here it is the block attention kernels run once over the packed batch, every sequence
attending to itself only, with a backward pass.

ring_size=P (keyword-only, additive) simulates a ring over a packed batch on this GPU: every rank
holds the r-th of P equal slices of EVERY sequence, packed the same way on every rank, so the
given tensors are the P shards stacked, [P * total_local, H, D], and cu_seqlens describes one
shard.  Rank r walks the shards r, r-1, ... in ring order exactly as the fixed-length ring does
(sp_aurora/intel_ring_flash_attn.py:72-148): one variable-length block launch per step, the causal
mask inside each sequence only at step 0, steps merged with update_out_and_lse.
"""
import torch

from . import ops
from .flash_attn import _check_unsupported
from .ring import _no_multi_gpu

__all__ = ["sp_aurora_varlen_func", "ring_flash_attn_varlen_func", "VarlenFlashAttnFunc", "VarlenRingFlashAttnFunc",
           "ring_varlen_forward", "ring_varlen_backward"]


class VarlenFlashAttnFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, softmax_scale, causal,
                return_softmax, rows_covered=False):
        if softmax_scale is None:
            softmax_scale = q.shape[-1] ** (-0.5)
        out, lse = ops.flash_fwd_varlen(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
                                        softmax_scale, causal)
        ctx.save_for_backward(q, k, v, out, lse, cu_seqlens_q, cu_seqlens_k)
        ctx.args = (int(max_seqlen_q), int(max_seqlen_k), softmax_scale, causal)
        ctx.rows_covered = bool(rows_covered)
        ctx.mark_non_differentiable(lse)
        return out if not return_softmax else (out, lse, None)

    @staticmethod
    def backward(ctx, dout, *args):
        q, k, v, out, lse, cu_q, cu_k = ctx.saved_tensors
        max_q, max_k, scale, causal = ctx.args
        # delta = rowsum(dout * out) per (row, head): the packed tensors are one batch of total_q rows
        delta = ops.bwd_delta(out.unsqueeze(0), dout.unsqueeze(0), layout="bshd")[0]
        # one call computes the whole gradient: the kernels write it in q's dtype
        dq, dk, dv = ops.flash_bwd_varlen_out(q, k, v, dout, lse, delta, cu_q, cu_k, max_q, max_k, scale, causal,
                                              rows_covered=ctx.rows_covered)
        return dq, dk, dv, None, None, None, None, None, None, None, None


def ring_varlen_forward(q, k, v, cu_seqlens, max_seqlen, softmax_scale, causal, ring_size):
    """All ranks of a simulated ring over a packed batch (see the module docstring): q, k, v [P * T, H, D] =
    P stacked shards of T rows, cu_seqlens [nseq + 1] the layout of one shard.  Returns out like q and
    lse fp32 [H, P * T]."""
    P = int(ring_size)
    PT, H, D = q.shape
    if P < 1 or PT % P or k.shape != q.shape or v.shape != q.shape:
        raise ValueError(f"ring_size={P} must divide the packed rows {PT}, and k, v must have q's shape")
    T = PT // P
    out = torch.empty_like(q)
    lse = torch.empty((H, PT), dtype=torch.float32, device=q.device)
    shard = lambda t, r: t[r * T:(r + 1) * T]
    acc = torch.empty((1, T, H, D), dtype=torch.float32, device=q.device)
    lse_acc = torch.empty((1, H, T), dtype=torch.float32, device=q.device)
    for r in range(P):
        steps = [t for t in range(P) if not causal or t <= r]
        for i, t in enumerate(steps):
            c = (r - t) % P
            bo, bl = ops.flash_fwd_varlen(shard(q, r), shard(k, c), shard(v, c), cu_seqlens, cu_seqlens, max_seqlen, max_seqlen,
                                          softmax_scale, causal and t == 0)
            if len(steps) == 1:
                shard(out, r).copy_(bo)
                lse[:, r * T:(r + 1) * T] = bl
            else:
                ops.merge(acc, lse_acc, bo.unsqueeze(0), bl.unsqueeze(0), layout="bshd", init=(i == 0))
        if len(steps) > 1:
            ops.finalize(acc, q.dtype, layout="bshd", out=shard(out, r).unsqueeze(0))
            lse[:, r * T:(r + 1) * T] = lse_acc[0]
    return out, lse


def ring_varlen_backward(dout, q, k, v, out, lse, cu_seqlens, max_seqlen, softmax_scale, causal, ring_size):
    """Gradients of ring_varlen_forward: one variable-length backward block per visited (rank, shard) pair with the
    lse of the whole ring, summed into fp32 accumulators (the schedule of
    sp_aurora/intel_ring_flash_attn.py:192-271), cast at the end."""
    P = int(ring_size)
    PT, H, D = q.shape
    T = PT // P
    delta = ops.bwd_delta(out.unsqueeze(0), dout.unsqueeze(0), layout="bshd")[0]  # [H, P * T]
    dq, dk, dv = (torch.zeros(q.shape, dtype=torch.float32, device=q.device) for _ in range(3))
    shard = lambda t, r: t[r * T:(r + 1) * T]
    for r in range(P):
        lse_r = lse[:, r * T:(r + 1) * T].contiguous()
        delta_r = delta[:, r * T:(r + 1) * T].contiguous()
        for t in range(P):
            if causal and t > r:
                continue
            c = (r - t) % P
            ops.flash_bwd_varlen(shard(q, r), shard(k, c), shard(v, c), shard(dout, r), lse_r, delta_r, shard(dq, r), shard(dk, c),
                                 shard(dv, c), cu_seqlens, cu_seqlens, max_seqlen, max_seqlen, softmax_scale, causal and t == 0)
    return dq.to(q.dtype), dk.to(k.dtype), dv.to(v.dtype)


class VarlenRingFlashAttnFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, cu_seqlens, max_seqlen, softmax_scale, causal, return_softmax, ring_size):
        if softmax_scale is None:
            softmax_scale = q.shape[-1] ** (-0.5)
        out, lse = ring_varlen_forward(q, k, v, cu_seqlens, max_seqlen, softmax_scale, causal, ring_size)
        ctx.save_for_backward(q, k, v, out, lse, cu_seqlens)
        ctx.args = (int(max_seqlen), softmax_scale, causal, int(ring_size))
        ctx.mark_non_differentiable(lse)
        return out if not return_softmax else (out, lse, None)

    @staticmethod
    def backward(ctx, dout, *args):
        q, k, v, out, lse, cu = ctx.saved_tensors
        max_seqlen, scale, causal, P = ctx.args
        dq, dk, dv = ring_varlen_backward(dout, q, k, v, out, lse, cu, max_seqlen, scale, causal, P)
        return dq, dk, dv, None, None, None, None, None, None


def sp_aurora_varlen_func(q, k, v, cu_seqlens_q, cu_seqlens_k=None, max_seqlen=None, dropout_p=0.0,
                          softmax_scale=None, causal=False, window_size=(-1, -1), alibi_slopes=None,
                          deterministic=False, return_attn_probs=False, group=None, *, max_seqlen_k=None,
                          check_offsets=True, ring_size=1):
    """q [total_q,H,D], k,v [total_k,H,D] packed without padding; sequence b owns rows
    cu_seqlens_q[b]..cu_seqlens_q[b+1] of q and cu_seqlens_k[b]..cu_seqlens_k[b+1] of k, v
    (cu_seqlens_k defaults to cu_seqlens_q).  max_seqlen: the longest sequence (of the queries;
    max_seqlen_k for the keys if different); computed from cu_seqlens (one device-to-host
    read, as in the reference's callers) when omitted.  Returns out [total_q,H,D], or (out, lse
    fp32 [H,total_q], None) with return_attn_probs.

    The kernels index the packed tensors with the offsets, so each distinct cu_seqlens array is
    looked at once on the host (a blocking device-to-host read on its first use; later calls with
    the same array, e.g. the other layers of a model, read nothing).  check_offsets=False skips the
    look (the caller vouches for the offsets); it is also skipped while the current stream is being
    captured into a graph.

    ring_size=P > 1: the tensors are P stacked shards of a simulated ring over the packed batch (rank r holds the
    r-th of P equal slices of every sequence) and cu_seqlens describes one shard; see the module docstring."""
    _check_unsupported(dropout_p, window_size, alibi_slopes)
    _no_multi_gpu(group)
    if cu_seqlens_k is None:
        cu_seqlens_k = cu_seqlens_q
    if max_seqlen is None:
        max_seqlen = int((cu_seqlens_q[1:] - cu_seqlens_q[:-1]).max())
    if max_seqlen_k is None:
        max_seqlen_k = max_seqlen if cu_seqlens_k is cu_seqlens_q else int((cu_seqlens_k[1:] - cu_seqlens_k[:-1]).max())
    if int(ring_size) > 1:
        # P stacked shards, cu_seqlens describes one of them (queries and keys alike)
        if cu_seqlens_k is not cu_seqlens_q or max_seqlen_k != max_seqlen or q.shape[0] % int(ring_size):
            raise ValueError("ring_size > 1 needs one cu_seqlens for queries and keys and packed rows divisible by ring_size")
        if check_offsets:
            ops.check_cu_seqlens_once(cu_seqlens_q, q.shape[0] // int(ring_size), max_seqlen, "cu_seqlens_q")
        return VarlenRingFlashAttnFunc.apply(q, k, v, cu_seqlens_q, max_seqlen, softmax_scale, causal, return_attn_probs, int(ring_size))
    covered = False
    if check_offsets:
        covered = ops.check_cu_seqlens_once(cu_seqlens_q, q.shape[0], max_seqlen, "cu_seqlens_q")
        if cu_seqlens_k is not cu_seqlens_q or k.shape[0] != q.shape[0] or max_seqlen_k != max_seqlen:
            covered = ops.check_cu_seqlens_once(cu_seqlens_k, k.shape[0], max_seqlen_k, "cu_seqlens_k") and covered
    if cu_seqlens_q.numel() != cu_seqlens_k.numel():
        raise ValueError("cu_seqlens_q and cu_seqlens_k must describe the same number of sequences")
    # rows of no sequence are not written by the backward kernels: gradients start as zeros unless the look
    # above has shown that the offsets cover every row
    return VarlenFlashAttnFunc.apply(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen, max_seqlen_k, softmax_scale,
                                     causal, return_attn_probs, covered)


ring_flash_attn_varlen_func = sp_aurora_varlen_func
