"""Ulysses re-layout and attention with the reference's names, on one GPU.

Mirrors sp_aurora/intel_ulysses_attn.py (intel_all_to_all_4d :60-143, IntelSeqAllToAll4D
:25-57, intel_ulysses_flash_attn_forward :184-287, the public functions :501-624) and
sp_aurora/comm/all_to_all.py (all_to_all_4D :17-180, all_to_all_5D :228-335,
SeqAllToAll4D/5D :183-205,338-365).

One GPU holds every rank's shard STACKED on a leading axis, and the whole P-rank exchange
is one permutation kernel:
    scatter heads / gather sequence:  x [P, B, s, H, D]   -> y [P, B, P*s, H/P, D]
    scatter sequence / gather heads:  y [P, B, P*s, h, D] -> x [P, B, s, P*h, D]
(and the same with a packed axis after the sequence axis for kv / qkv tensors).
A per-rank 4-D (or packed 5-D) tensor without a process group is a world of size 1, for
which the reference returns its input unchanged (intel_ulysses_attn.py:80-82); so does this.
"""
import torch
import torch.distributed as dist

from . import ops
from .flash_attn import _check_unsupported
from .ring import _no_multi_gpu

__all__ = [
    "intel_all_to_all_4d", "all_to_all_4D", "all_to_all_5D", "IntelSeqAllToAll4D", "SeqAllToAll4D",
    "SeqAllToAll5D", "intel_ulysses_flash_attn_forward", "ulysses_flash_attn_func",
    "ulysses_flash_attn_kvpacked_func", "ulysses_flash_attn_qkvpacked_func",
    "intel_ulysses_flash_attn_func", "intel_ulysses_flash_attn_kvpacked_func",
    "intel_ulysses_flash_attn_qkvpacked_func",
]


def _stacked_relayout(x, scatter_idx, gather_idx, per_rank_dims, head_idx, what):
    """x carries one more (leading, rank) axis than the reference's per-rank tensor."""
    if x.dim() == per_rank_dims:
        return x  # world size 1
    if x.dim() != per_rank_dims + 1:
        raise AssertionError(f"{what}: expected a {per_rank_dims}-D per-rank tensor or a "
                             f"{per_rank_dims + 1}-D rank-stacked tensor, got {x.dim()}-D")
    P = x.shape[0]
    if P == 1:
        return x
    if scatter_idx == head_idx and gather_idx == 1:
        return ops.relayout_s2h(x, P)
    if scatter_idx == 1 and gather_idx == head_idx:
        return ops.relayout_h2s(x, P)
    raise ValueError(f"Unsupported scatter_idx={scatter_idx}, gather_idx={gather_idx}")


def intel_all_to_all_4d(input, scatter_idx=2, gather_idx=1, group=None):
    """(bs, seq/P, heads, hd) <-> (bs, seq, heads/P, hd) for every rank at once.

    `input` is the rank-stacked [P, bs, ...] tensor; scatter_idx / gather_idx keep the
    reference's per-rank meaning (2,1 = forward, 1,2 = inverse;
    sp_aurora/intel_ulysses_attn.py:84,114,142-143)."""
    _no_multi_gpu(group)
    return _stacked_relayout(input, scatter_idx, gather_idx, 4, 2, "intel_all_to_all_4d")


def all_to_all_4D(input, scatter_idx=2, gather_idx=1, group=None, use_sync=False):
    """Twin of intel_all_to_all_4d (sp_aurora/comm/all_to_all.py:17-180)."""
    _no_multi_gpu(group)
    out = _stacked_relayout(input, scatter_idx, gather_idx, 4, 2, "all_to_all_4D")
    if use_sync:
        torch.cuda.synchronize()
    return out


def all_to_all_5D(input, scatter_idx=3, gather_idx=1, group=None, use_sync=False):
    """Packed variant: (bs, seq/P, 3, heads, hd) <-> (bs, seq, 3, heads/P, hd)
    (sp_aurora/comm/all_to_all.py:228-335); 3,1 = forward, 1,3 = inverse."""
    _no_multi_gpu(group)
    if input.dim() not in (5, 6):
        raise AssertionError(f"input must be 5D tensor, got {input.dim()} and shape {tuple(input.shape)}")
    if scatter_idx not in (1, 3) or gather_idx not in (1, 3):
        raise RuntimeError("scatter_idx must be 1 or 3 and gather_idx must be 1 or 3")
    out = _stacked_relayout(input, scatter_idx, gather_idx, 5, 3, "all_to_all_5D")
    if use_sync:
        torch.cuda.synchronize()
    return out


class IntelSeqAllToAll4D(torch.autograd.Function):
    """Re-layout whose backward is the inverse re-layout (sp_aurora/intel_ulysses_attn.py:25-57)."""

    @staticmethod
    def forward(ctx, group, input, scatter_idx, gather_idx):
        ctx.group = group
        ctx.scatter_idx = scatter_idx
        ctx.gather_idx = gather_idx
        return intel_all_to_all_4d(input, scatter_idx, gather_idx, group)

    @staticmethod
    def backward(ctx, grad_output):
        return None, IntelSeqAllToAll4D.apply(ctx.group, grad_output, ctx.gather_idx, ctx.scatter_idx), None, None


SeqAllToAll4D = IntelSeqAllToAll4D


class SeqAllToAll5D(torch.autograd.Function):
    """sp_aurora/comm/all_to_all.py:338-365."""

    @staticmethod
    def forward(ctx, group, input, scatter_idx=3, gather_idx=1, use_sync=False):
        ctx.group = group
        ctx.scatter_idx = scatter_idx
        ctx.gather_idx = gather_idx
        ctx.use_sync = use_sync
        return all_to_all_5D(input, scatter_idx, gather_idx, group=group, use_sync=use_sync)

    @staticmethod
    def backward(ctx, grad_output):
        return (None, SeqAllToAll5D.apply(ctx.group, grad_output, ctx.gather_idx, ctx.scatter_idx, ctx.use_sync),
                None, None, None)


def intel_ulysses_flash_attn_forward(process_group, q, k, v, softmax_scale, dropout_p=0.0, causal=False,
                                     window_size=(-1, -1), alibi_slopes=None, deterministic=False, *, relayout="auto"):
    """Ulysses forward for all ranks: re-layout q,k,v, attention over the full sequence on
    H/P heads per rank, inverse re-layout of out (sp_aurora/intel_ulysses_attn.py:233-287).

    q,k,v: rank-stacked [P,B,s,H,D] (or a single rank's [B,S,H,D], P = 1).
    Returns out like q and lse fp32 [P,B,H/P,P*s] — head-sharded, as the reference leaves it
    (:284-287).

    relayout (not in the reference): "kernels" runs the four re-layout passes; "views" runs none -
    with B = 1 the rank-stacked tensor IS the full sequence [P*s, H, D], head group r is a strided
    view of it (heads r*h .. r*h+h-1), and the attention kernel reads and writes such views as they
    are, which on one GPU is what peer writes into the head-sharded layout are across GPUs;
    "auto" = "views" where it applies (B = 1, compact tensors), else "kernels"."""
    _no_multi_gpu(process_group)
    _check_unsupported(dropout_p, window_size, alibi_slopes)
    if relayout not in ("auto", "views", "kernels"):
        raise ValueError(f"relayout must be 'auto', 'views' or 'kernels', got {relayout!r}")
    if q.dim() == 4:
        return ops.flash_fwd(q, k, v, softmax_scale, causal, layout="bshd")
    P, B, s, H, D = q.shape
    views_ok = _views_ok(q, k, v)
    if relayout == "views" and not views_ok:
        raise ValueError("relayout='views' needs B = 1 and compact q, k, v of one shape")
    if relayout != "kernels" and views_ok:
        h = H // P
        out = torch.empty_like(q)
        # group r as a batch entry: [P groups, P*s rows, h heads, D] over the [P*s, H, D] sequence
        grp = lambda t: t.as_strided((P, P * s, h, D), (h * D, H * D, D, 1), t.storage_offset())
        _, lse = ops.flash_fwd(grp(q), grp(k), grp(v), softmax_scale, causal, layout="bshd", out=grp(out))
        return out, lse.view(P, B, h, P * s)
    yq, yk, yv = ops.relayout_s2h(q, P), ops.relayout_s2h(k, P), ops.relayout_s2h(v, P)
    h = H // P
    # the P head groups are independent: fold the rank axis into the batch axis
    o, lse = ops.flash_fwd(yq.view(P * B, P * s, h, D), yk.view(P * B, P * s, h, D), yv.view(P * B, P * s, h, D),
                           softmax_scale, causal, layout="bshd")
    out = ops.relayout_h2s(o.view(P, B, P * s, h, D), P)
    return out, lse.view(P, B, h, P * s)


def _views_ok(q, *others):
    """Can head groups be read / written as strided views of these rank-stacked [P,B,s,H,D] tensors?
    B = 1, heads divisible by the ranks, every tensor compact and of q's shape (a view is built
    with q's sizes, so a tensor of another shape would be read wrongly)."""
    P, B, s, H, D = q.shape
    return B == 1 and H % P == 0 and all(t.shape == q.shape and t.is_contiguous() for t in (q,) + others)


class UlyssesFlashAttnFunc(torch.autograd.Function):
    """Mirrors IntelUlyssesFlashAttnFunc (sp_aurora/intel_ulysses_attn.py:436-498).  The backward
    re-lays dout, runs the block backward on the head-sharded tensors and re-lays the gradients
    back, which is the structure of intel_ulysses_flash_attn_backward (:290-433)."""

    @staticmethod
    def forward(ctx, q, k, v, dropout_p, softmax_scale, causal, window_size, alibi_slopes, deterministic,
                return_attn_probs, group):
        if softmax_scale is None:
            softmax_scale = q.shape[-1] ** -0.5
        out, lse = intel_ulysses_flash_attn_forward(group, q, k, v, softmax_scale, dropout_p, causal,
                                                    window_size, alibi_slopes, deterministic)
        ctx.save_for_backward(q, k, v, out, lse)
        ctx.softmax_scale = softmax_scale
        ctx.causal = causal
        return out if not return_attn_probs else (out, None)

    @staticmethod
    def backward(ctx, dout, *args):
        from .ring import ring_flash_attn_backward
        q, k, v, out, lse = ctx.saved_tensors
        if q.dim() == 4:
            dq, dk, dv = ring_flash_attn_backward(dout, q, k, v, out, lse, ctx.softmax_scale, ctx.causal, 1)
        else:
            P, B, s, H, D = q.shape
            h = H // P
            if _views_ok(q, k, v, out) and dout.shape == q.shape:
                # as in the forward: head groups are strided views of the stacked tensors, and the kernels
                # write the gradients through such views of stacked tensors, so nothing is re-laid
                grp = lambda t: t.as_strided((P, P * s, h, D), (h * D, H * D, D, 1), t.storage_offset())
                dout = dout.contiguous()
                delta = ops.bwd_delta(grp(out), grp(dout), layout="bshd")
                grads = [torch.empty_like(t) for t in (q, k, v)]
                ops.flash_bwd_out(grp(q), grp(k), grp(v), grp(dout), lse.view(P, h, P * s), delta, ctx.softmax_scale, ctx.causal,
                                  layout="bshd", dq=grp(grads[0]), dk=grp(grads[1]), dv=grp(grads[2]))
                return tuple(grads) + (None,) * 8
            fold = lambda t: ops.relayout_s2h(t.contiguous(), P).view(P * B, P * s, h, D)
            gq, gk, gv = ring_flash_attn_backward(fold(dout), fold(q), fold(k), fold(v), fold(out),
                                                  lse.view(P * B, h, P * s), ctx.softmax_scale, ctx.causal, 1)
            unfold = lambda t: ops.relayout_h2s(t.view(P, B, P * s, h, D), P)
            dq, dk, dv = unfold(gq), unfold(gk), unfold(gv)
        return dq, dk, dv, None, None, None, None, None, None, None, None


def ulysses_flash_attn_func(q, k, v, dropout_p=0.0, softmax_scale=None, causal=False, window_size=(-1, -1),
                            alibi_slopes=None, deterministic=False, return_attn_probs=False, group=None):
    """sp_aurora/intel_ulysses_attn.py:501-548.  q,k,v rank-stacked [P,B,s,H,D] (or [B,S,H,D])."""
    return UlyssesFlashAttnFunc.apply(q, k, v, dropout_p, softmax_scale, causal, window_size, alibi_slopes,
                                      deterministic, return_attn_probs, group)


def ulysses_flash_attn_qkvpacked_func(qkv, dropout_p=0.0, softmax_scale=None, causal=False,
                                      window_size=(-1, -1), alibi_slopes=None, deterministic=False,
                                      return_attn_probs=False, group=None):
    """qkv [..., s, 3, H, D] (sp_aurora/intel_ulysses_attn.py:551-586)."""
    three = qkv.shape[-3]
    assert three == 3, f"qkv must have size 3 in dim 2, got {three}"
    q, k, v = qkv.unbind(dim=-3)
    return ulysses_flash_attn_func(q, k, v, dropout_p, softmax_scale, causal, window_size, alibi_slopes,
                                   deterministic, return_attn_probs, group)


def ulysses_flash_attn_kvpacked_func(q, kv, dropout_p=0.0, softmax_scale=None, causal=False,
                                     window_size=(-1, -1), alibi_slopes=None, deterministic=False,
                                     return_attn_probs=False, group=None):
    """kv [..., s, 2, H, D] (sp_aurora/intel_ulysses_attn.py:589-624)."""
    two = kv.shape[-3]
    assert two == 2, f"kv must have size 2 in dim 2, got {two}"
    k, v = kv.unbind(dim=-3)
    return ulysses_flash_attn_func(q, k, v, dropout_p, softmax_scale, causal, window_size, alibi_slopes,
                                   deterministic, return_attn_probs, group)


intel_ulysses_flash_attn_func = ulysses_flash_attn_func
intel_ulysses_flash_attn_qkvpacked_func = ulysses_flash_attn_qkvpacked_func
intel_ulysses_flash_attn_kvpacked_func = ulysses_flash_attn_kvpacked_func
