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

sharding="zigzag" (zigzag_sp_aurora_varlen_func, the name the reference's test imports and the reference does not
ship: test/flash_attention/test_intel_ring_flash_attn_varlen.py:25,205-215): every sequence is cut into 2P
half-slices and rank r holds half-slices r and 2P-1-r of each, one after the other, so that a causal ring gives
every rank the same work.  Host code over the same variable-length block kernels: each shard is brought into
half-major order once (the first halves of all sequences packed, then the second halves; a gather), in which the
block pairs of the zigzag ring are contiguous packed batches: at step 0 first x first (causal), second x first,
second x second (causal); at a step with chunk c < r both halves of the queries against the chunk's first halves;
with c > r the second halves of the queries against both halves of the chunk.
"""
import torch

from . import ops
from .flash_attn import _check_unsupported
from .ring import _no_multi_gpu

__all__ = ["sp_aurora_varlen_func", "ring_flash_attn_varlen_func", "zigzag_sp_aurora_varlen_func", "VarlenFlashAttnFunc",
           "VarlenRingFlashAttnFunc", "ring_varlen_forward", "ring_varlen_backward", "zigzag_varlen_order"]


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


def ring_varlen_forward(q, k, v, cu_seqlens, max_seqlen, softmax_scale, causal, ring_size, fuse="rank"):
    """All ranks of a simulated ring over a packed batch (see the module docstring): q, k, v [P * T, H, D] =
    P stacked shards of T rows, cu_seqlens [nseq + 1] the layout of one shard.  Returns out like q and
    lse fp32 [H, P * T].  fuse="rank" / "all": one launch per rank / for all ranks, the rank's query tile and accumulators
    in registers across its shards (spa_ring_fwd_varlen; bf16 / fp16); "step" (and fp32): one variable-length block launch
    per visited shard pair, merged with update_out_and_lse as separate passes."""
    P = int(ring_size)
    PT, H, D = q.shape
    if P < 1 or PT % P or k.shape != q.shape or v.shape != q.shape:
        raise ValueError(f"ring_size={P} must divide the packed rows {PT}, and k, v must have q's shape")
    if fuse not in ("step", "rank", "all"):
        raise ValueError(f"fuse must be 'step', 'rank' or 'all', got {fuse!r}")
    if fuse != "step" and q.dtype in (torch.bfloat16, torch.float16) and P > 1:
        return ops.ring_fwd_varlen(q, k, v, cu_seqlens, max_seqlen, P, softmax_scale, causal, fuse=fuse)
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


def zigzag_varlen_order(seq_lens, P):
    """Where the rows of a zigzag-sharded packed batch come from: for sequences of the given (global) lengths, each
    divisible by 2P, returns the int64 index tensor `idx` with stacked_shards = packed_natural[idx]: rank r's shard
    holds, sequence by sequence, half-slices r and 2P-1-r of the sequence."""
    starts, idx = [0], []
    for n in seq_lens:
        if n % (2 * P):
            raise ValueError(f"zigzag sharding needs 2 * ring_size = {2 * P} to divide every sequence length (got {n})")
        starts.append(starts[-1] + n)
    for r in range(P):
        for i, n in enumerate(seq_lens):
            h = n // (2 * P)
            idx.append(torch.arange(starts[i] + r * h, starts[i] + (r + 1) * h))
            idx.append(torch.arange(starts[i] + (2 * P - 1 - r) * h, starts[i] + (2 * P - r) * h))
    return torch.cat(idx) if idx else torch.zeros(0, dtype=torch.int64)


_HALF_MAJOR = {}


def _half_major(cu_seqlens, T):
    """For one shard whose sequences all have even length: (perm, cu_half), perm int64 [T] on the device with
    half_major = shard[perm] (the first halves of all sequences packed, then the second halves), cu_half the
    offsets of either half.  One device-to-host read per distinct cu_seqlens array."""
    key = (cu_seqlens.data_ptr(), cu_seqlens._version, cu_seqlens.numel(), str(cu_seqlens.device), int(T))
    hit = _HALF_MAJOR.get(key)
    if hit is not None:
        return hit
    cu = cu_seqlens.detach().cpu().to(torch.int64)
    lens = cu[1:] - cu[:-1]
    if int(cu[0]) != 0 or int(cu[-1]) != T or bool((lens < 0).any()) or bool((lens % 2 != 0).any()):
        raise ValueError("zigzag sharding: cu_seqlens must start at 0, end at the rows of one shard and give every sequence an even length")
    first = [torch.arange(int(cu[i]), int(cu[i]) + int(lens[i]) // 2) for i in range(lens.numel())]
    second = [torch.arange(int(cu[i]) + int(lens[i]) // 2, int(cu[i + 1])) for i in range(lens.numel())]
    perm = torch.cat(first + second).to(cu_seqlens.device)
    cu_half = (cu // 2).to(torch.int32).to(cu_seqlens.device)
    if len(_HALF_MAJOR) >= 64:
        _HALF_MAJOR.clear()
    _HALF_MAJOR[key] = (perm, cu_half)
    return perm, cu_half


def _zigzag_block_pairs(P):
    """The block pairs of a causal zigzag ring in half-major shards, rank by rank in ring order:
    (rank, query half, chunk, key half, causal); halves 0 = first, 1 = second."""
    pairs = []
    for r in range(P):
        pairs += [(r, 0, r, 0, True), (r, 1, r, 0, False), (r, 1, r, 1, True)]
        for t in range(1, P):
            c = (r - t) % P
            pairs += [(r, 0, c, 0, False), (r, 1, c, 0, False)] if c < r else [(r, 1, c, 0, False), (r, 1, c, 1, False)]
    return pairs


def zigzag_ring_varlen_forward(q, k, v, cu_seqlens, max_seqlen, softmax_scale, causal, ring_size):
    """ring_varlen_forward for zigzag shards (see the module docstring).  Without a mask the order of the rows does
    not matter and the contiguous ring is run."""
    P = int(ring_size)
    if not causal or P == 1:
        return ring_varlen_forward(q, k, v, cu_seqlens, max_seqlen, softmax_scale, causal, P)
    PT, H, D = q.shape
    if PT % P or k.shape != q.shape or v.shape != q.shape:
        raise ValueError(f"ring_size={P} must divide the packed rows {PT}, and k, v must have q's shape")
    T = PT // P
    perm, cu_h = _half_major(cu_seqlens, T)
    hm = lambda t: t.reshape(P, T, H, D)[:, perm]                      # [P, T, H, D], every shard in half-major order
    qh, kh, vh = hm(q), hm(k), hm(v)
    Th, max_h = T // 2, (int(max_seqlen) + 1) // 2
    half = lambda t, r, w: t[r, w * Th:(w + 1) * Th]
    outh = torch.empty((P, T, H, D), dtype=q.dtype, device=q.device)
    lseh = torch.empty((P, H, T), dtype=torch.float32, device=q.device)
    acc = torch.empty((2, 1, Th, H, D), dtype=torch.float32, device=q.device)
    lse_acc = torch.empty((2, 1, H, Th), dtype=torch.float32, device=q.device)
    started = [False, False]
    pairs = _zigzag_block_pairs(P)
    for n, (r, qw, c, kw, msk) in enumerate(pairs):
        if Th:
            bo, bl = ops.flash_fwd_varlen(half(qh, r, qw), half(kh, c, kw), half(vh, c, kw), cu_h, cu_h, max_h, max_h, softmax_scale, msk)
            ops.merge(acc[qw], lse_acc[qw], bo.unsqueeze(0), bl.unsqueeze(0), layout="bshd", init=not started[qw])
            started[qw] = True
        if n + 1 == len(pairs) or pairs[n + 1][0] != r:   # the rank's last pair: its rows are complete
            for w in (0, 1):
                if Th:
                    ops.finalize(acc[w], q.dtype, layout="bshd", out=outh[r, w * Th:(w + 1) * Th].unsqueeze(0))
                    lseh[r, :, w * Th:(w + 1) * Th] = lse_acc[w, 0]
            started = [False, False]
    out = torch.empty_like(q)
    out.view(P, T, H, D)[:, perm] = outh
    lse = torch.empty((H, PT), dtype=torch.float32, device=q.device)
    lse.view(H, P, T)[:, :, perm] = lseh.permute(1, 0, 2)
    return out, lse


def zigzag_ring_varlen_backward(dout, q, k, v, out, lse, cu_seqlens, max_seqlen, softmax_scale, causal, ring_size):
    """Gradients of zigzag_ring_varlen_forward: one variable-length backward block per block pair of the zigzag ring, on
    the half-major shards, with the lse of the whole ring, into fp32 accumulators; gathered back and cast at the end."""
    P = int(ring_size)
    if not causal or P == 1:
        return ring_varlen_backward(dout, q, k, v, out, lse, cu_seqlens, max_seqlen, softmax_scale, causal, P)
    PT, H, D = q.shape
    T = PT // P
    perm, cu_h = _half_major(cu_seqlens, T)
    hm = lambda t: t.reshape(P, T, H, D)[:, perm]
    qh, kh, vh, doh = hm(q), hm(k), hm(v), hm(dout)
    delta = ops.bwd_delta(out.unsqueeze(0), dout.unsqueeze(0), layout="bshd")[0]      # [H, P * T]
    hm_rows = lambda t: t.reshape(H, P, T)[:, :, perm].permute(1, 0, 2)                # [P, H, T], half-major
    lseh, deltah = hm_rows(lse), hm_rows(delta)
    Th, max_h = T // 2, (int(max_seqlen) + 1) // 2
    half = lambda t, r, w: t[r, w * Th:(w + 1) * Th]
    dqh, dkh, dvh = (torch.zeros((P, T, H, D), dtype=torch.float32, device=q.device) for _ in range(3))
    if Th:
        for r, qw, c, kw, msk in _zigzag_block_pairs(P):
            rows = slice(qw * Th, (qw + 1) * Th)
            ops.flash_bwd_varlen(half(qh, r, qw), half(kh, c, kw), half(vh, c, kw), half(doh, r, qw), lseh[r, :, rows].contiguous(),
                                 deltah[r, :, rows].contiguous(), half(dqh, r, qw), half(dkh, c, kw), half(dvh, c, kw), cu_h, cu_h,
                                 max_h, max_h, softmax_scale, msk)
    grads = []
    for g, like in ((dqh, q), (dkh, k), (dvh, v)):
        nat = torch.empty((P, T, H, D), dtype=like.dtype, device=q.device)
        nat[:, perm] = g.to(like.dtype)
        grads.append(nat.reshape(PT, H, D))
    return tuple(grads)


class VarlenRingFlashAttnFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, cu_seqlens, max_seqlen, softmax_scale, causal, return_softmax, ring_size, zigzag=False):
        if softmax_scale is None:
            softmax_scale = q.shape[-1] ** (-0.5)
        fwd = zigzag_ring_varlen_forward if zigzag else ring_varlen_forward
        out, lse = fwd(q, k, v, cu_seqlens, max_seqlen, softmax_scale, causal, ring_size)
        ctx.save_for_backward(q, k, v, out, lse, cu_seqlens)
        ctx.args = (int(max_seqlen), softmax_scale, causal, int(ring_size), bool(zigzag))
        ctx.mark_non_differentiable(lse)
        return out if not return_softmax else (out, lse, None)

    @staticmethod
    def backward(ctx, dout, *args):
        q, k, v, out, lse, cu = ctx.saved_tensors
        max_seqlen, scale, causal, P, zigzag = ctx.args
        bwd = zigzag_ring_varlen_backward if zigzag else ring_varlen_backward
        dq, dk, dv = bwd(dout, q, k, v, out, lse, cu, max_seqlen, scale, causal, P)
        return dq, dk, dv, None, None, None, None, None, None, None


def sp_aurora_varlen_func(q, k, v, cu_seqlens_q, cu_seqlens_k=None, max_seqlen=None, dropout_p=0.0,
                          softmax_scale=None, causal=False, window_size=(-1, -1), alibi_slopes=None,
                          deterministic=False, return_attn_probs=False, group=None, *, max_seqlen_k=None,
                          check_offsets=True, ring_size=1, sharding="contiguous"):
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
    r-th of P equal slices of every sequence) and cu_seqlens describes one shard; see the module docstring.
    sharding="zigzag" (with ring_size): rank r holds half-slices r and 2P-1-r of every sequence instead
    (zigzag_varlen_order); every sequence's share of a shard must have an even length."""
    if sharding not in ("contiguous", "zigzag"):
        raise ValueError(f"sharding must be 'contiguous' or 'zigzag', got {sharding!r}")
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
        return VarlenRingFlashAttnFunc.apply(q, k, v, cu_seqlens_q, max_seqlen, softmax_scale, causal, return_attn_probs, int(ring_size),
                                             sharding == "zigzag")
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


def zigzag_sp_aurora_varlen_func(q, k, v, cu_seqlens_q, cu_seqlens_k=None, max_seqlen=None, dropout_p=0.0, softmax_scale=None,
                                 causal=False, window_size=(-1, -1), alibi_slopes=None, deterministic=False,
                                 return_attn_probs=False, group=None, **kw):
    """sp_aurora_varlen_func on zigzag shards: the name test/flash_attention/test_intel_ring_flash_attn_varlen.py:25,205-215
    imports (the reference ships no such function).  With ring_size=P the tensors are the P zigzag shards stacked; a ring of
    one is the plain variable-length call."""
    return sp_aurora_varlen_func(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen, dropout_p, softmax_scale, causal, window_size,
                                 alibi_slopes, deterministic, return_attn_probs, group, sharding="zigzag", **kw)
