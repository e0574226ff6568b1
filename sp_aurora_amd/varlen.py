"""Attention over packed variable-length batches (`cu_seqlens`), on one GPU.

The reference's tests and adapter are written against sp_aurora_varlen_func(q, k, v,
cu_seqlens_q, cu_seqlens_k, max_seqlen=..., dropout_p=..., causal=...)
(test/flash_attention/test_intel_ring_flash_attn_varlen.py:23-26,66-74,85-91) but the
reference does not ship the function; only the lse helpers exist (sp_aurora/utils.py:150-169).
Here it is the block attention kernels run once over the packed batch, every sequence
attending to itself only, with a backward pass.  A ring over packed batches (every rank
holding a slice of every sequence) is not built: with one GPU a ring of one is the whole
computation.
"""
import torch

from . import ops
from .flash_attn import _check_unsupported
from .ring import _no_multi_gpu

__all__ = ["sp_aurora_varlen_func", "ring_flash_attn_varlen_func", "VarlenFlashAttnFunc"]


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


def sp_aurora_varlen_func(q, k, v, cu_seqlens_q, cu_seqlens_k=None, max_seqlen=None, dropout_p=0.0,
                          softmax_scale=None, causal=False, window_size=(-1, -1), alibi_slopes=None,
                          deterministic=False, return_attn_probs=False, group=None, *, max_seqlen_k=None,
                          check_offsets=True):
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
    captured into a graph."""
    _check_unsupported(dropout_p, window_size, alibi_slopes)
    _no_multi_gpu(group)
    if cu_seqlens_k is None:
        cu_seqlens_k = cu_seqlens_q
    if max_seqlen is None:
        max_seqlen = int((cu_seqlens_q[1:] - cu_seqlens_q[:-1]).max())
    if max_seqlen_k is None:
        max_seqlen_k = max_seqlen if cu_seqlens_k is cu_seqlens_q else int((cu_seqlens_k[1:] - cu_seqlens_k[:-1]).max())
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
