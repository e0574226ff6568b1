"""CPU oracle for the sp_aurora attention hot path.  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this
module, and only as the checker; nothing under sp_aurora_amd/ imports it.

It restates, with plain torch CPU ops, the algorithms of the reference's Python
path (each function cites the file:line it follows).  Arithmetic runs in
``compute_dtype`` (float64 by default) on the inputs at their storage precision,
i.e. bf16 / fp16 inputs are up-cast exactly; the reference's own habit of keeping
bf16 scores in bf16 (sp_aurora/intel_flash_attn_optimized.py:56,69) is a precision
defect, not part of the function being computed, and is not reproduced.

Pinning (see tests/test_oracle.py): the reference ships no golden vectors for this
path, so every function here is pinned by brute-force loops on tiny inputs, closed
forms (uniform keys, one visible key, constant V), library routines
(torch.softmax / torch.logsumexp / F.scaled_dot_product_attention in fp64), and the
invariants the reference's own tests assert (ring == full attention,
test/test_ring_attention_full_accuracy.py:122-171; packed == unpacked,
test/test_ring_attention_comprehensive.py:205-218; inverse o forward re-layout is
the identity; a zigzag-sharded ring == full causal attention after un-permuting the rows).
No function is left "parity unpinned".

Layouts: the block operator uses the reference's operator layout [B, H, S, D]
(sp_aurora/intel_flash_attn.py:56); the ring and Ulysses drivers use the public
layout [B, S, H, D] (sp_aurora/intel_ring_flash_attn.py:399-435).
"""
import math

import torch
import torch.nn.functional as F

CD = torch.float64


# --------------------------------------------------------------------------------------
# A1/A2: block attention operator
# --------------------------------------------------------------------------------------
def causal_mask(sq, sk):
    """Top-left aligned mask, True = masked: key j > query i.
    sp_aurora/intel_flash_attn.py:79-84 (triu(ones(seq_len, seq_len_k), diagonal=1))."""
    return torch.triu(torch.ones(sq, sk, dtype=torch.bool), diagonal=1)


def attn_block(q, k, v, softmax_scale=None, causal=False, compute_dtype=CD):
    """out = softmax(q k^T * scale + mask) v, lse = logsumexp(q k^T * scale + mask).

    Follows the dense branch of the reference operator
    (sp_aurora/intel_flash_attn.py:95-126; sp_aurora/intel_flash_attn_optimized.py:208-225):
    scores -> masked_fill(-inf) -> logsumexp -> exp(scores - lse) -> matmul with v.
    q [B,H,Sq,D], k,v [B,H,Sk,D]  ->  out [B,H,Sq,D] (compute_dtype), lse [B,H,Sq].
    """
    q, k, v = q.to(compute_dtype), k.to(compute_dtype), v.to(compute_dtype)
    if softmax_scale is None:
        softmax_scale = q.shape[-1] ** (-0.5)
    scores = torch.matmul(q, k.transpose(-2, -1)) * softmax_scale
    if causal:
        scores = scores.masked_fill(causal_mask(q.shape[-2], k.shape[-2]), float("-inf"))
    lse = torch.logsumexp(scores, dim=-1)
    weights = torch.exp(scores - lse.unsqueeze(-1))
    return torch.matmul(weights, v), lse


def attn_block_tiled(q, k, v, softmax_scale=None, causal=False, block_size=128, compute_dtype=CD,
                     literal_rescale=False, literal_mask=False):
    """The reference's Python-level flash attention, tile by tile
    (_flash_attn_forward_tiled, sp_aurora/intel_flash_attn_optimized.py:12-92):
    tile skip `j >= i_end` (:49-50), in-tile causal mask (:59-66), per-tile logsumexp (:69),
    running log-add-exp (:72-75), P = exp(scores - tile_lse) (:78).

    In-tile mask.  Key j+c is hidden from query i+r when j+c > i+r, i.e. c - r >= i - j + 1:
    triu(diagonal = i - j + 1).  The reference writes diagonal = j - i + 1 (:62-63), which is
    the same on the diagonal tile (j == i) and hides every key of every earlier tile (j < i),
    so its causal lse is -inf/NaN beyond the first query tile.  That is a defect of the
    reference; the function computed here uses the intended offset, `literal_mask=True`
    reproduces the line as written.

    Output rescale.  The reference line :85-86 reads
        acc = acc * exp(tile_lse - new_lse) + P v
    i.e. it puts the weight of the NEW tile on the OLD accumulator and weight 1 on the new
    tile.  With more than one visited key tile the weights do not sum to one and `out` is not
    softmax(scores) v (its lse is still right).  That is a defect of the reference, reached
    only for S > 2048 (:198-205); the function computed here is the intended one,
        acc = acc * exp(old_lse - new_lse) + (P v) * exp(tile_lse - new_lse).
    `literal_rescale=True` reproduces the reference line as written, so that a test can show
    the two agree for one tile and differ for more."""
    q, k, v = q.to(compute_dtype), k.to(compute_dtype), v.to(compute_dtype)
    B, H, Sq, D = q.shape
    Sk = k.shape[-2]
    if softmax_scale is None:
        softmax_scale = D ** (-0.5)
    out = torch.zeros(B, H, Sq, D, dtype=compute_dtype)
    lse = torch.full((B, H, Sq), float("-inf"), dtype=compute_dtype)
    for i in range(0, Sq, block_size):
        i_end = min(i + block_size, Sq)
        qb = q[:, :, i:i_end]
        acc = torch.zeros_like(qb)
        run = torch.full((B, H, i_end - i), float("-inf"), dtype=compute_dtype)
        for j in range(0, Sk, block_size):
            j_end = min(j + block_size, Sk)
            if causal and j >= i_end:
                continue
            scores = torch.matmul(qb, k[:, :, j:j_end].transpose(-2, -1)) * softmax_scale
            if causal:
                diag = (j - i + 1) if literal_mask else (i - j + 1)
                m = torch.triu(torch.ones(i_end - i, j_end - j, dtype=torch.bool), diagonal=diag)
                scores = scores.masked_fill(m, float("-inf"))
            tile_lse = torch.logsumexp(scores, dim=-1)
            mx = torch.maximum(run, tile_lse)
            new = mx + torch.log(torch.exp(run - mx) + torch.exp(tile_lse - mx))
            p = torch.exp(scores - tile_lse.unsqueeze(-1))
            pv = torch.matmul(p, v[:, :, j:j_end])
            w_tile = torch.exp(tile_lse - new).unsqueeze(-1)
            if literal_rescale:
                acc = acc * w_tile + pv
            else:
                acc = acc * torch.exp(run - new).unsqueeze(-1) + pv * w_tile
            run = new
        out[:, :, i:i_end] = acc
        lse[:, :, i:i_end] = run
    return out, lse


def attn_block_sdpa(q, k, v, softmax_scale=None, causal=False, compute_dtype=CD):
    """The op sequence the reference actually runs for S <= 2048
    (sp_aurora/intel_flash_attn_optimized.py:156-193): F.scaled_dot_product_attention for
    `out`, then a SECOND q k^T + mask + logsumexp for the lse."""
    q, k, v = q.to(compute_dtype), k.to(compute_dtype), v.to(compute_dtype)
    if softmax_scale is None:
        softmax_scale = q.shape[-1] ** (-0.5)
    mask = None
    if causal:  # is_causal=True in the reference; an explicit top-left mask also covers Sq != Sk
        mask = ~causal_mask(q.shape[-2], k.shape[-2])
    out = F.scaled_dot_product_attention(q, k, v, attn_mask=mask, dropout_p=0.0, scale=softmax_scale)
    scores = torch.matmul(q, k.transpose(-2, -1)) * softmax_scale
    if causal:
        scores = scores.masked_fill(causal_mask(q.shape[-2], k.shape[-2]), float("-inf"))
    return out, torch.logsumexp(scores, dim=-1)


# --------------------------------------------------------------------------------------
# A4: merge
# --------------------------------------------------------------------------------------
def merge(out, lse, block_out, block_lse):
    """One update_out_and_lse step in fp of the inputs' compute dtype
    (sp_aurora/utils.py:103-104):
        out = out - sigmoid(block_lse - lse) * (out - block_out)
        lse = lse - logsigmoid(lse - block_lse)
    out/block_out [..., S, D]-like with lse/block_lse broadcastable as [..., S, 1]."""
    new_out = out - torch.sigmoid(block_lse - lse) * (out - block_out)
    new_lse = lse - F.logsigmoid(lse - block_lse)
    return new_out, new_lse


# --------------------------------------------------------------------------------------
# A5/A6: ring schedule (public layout [B, S, H, D])
# --------------------------------------------------------------------------------------
def ring_forward_rank(q_local, k_chunks, v_chunks, rank, softmax_scale=None, causal=False,
                      compute_dtype=CD, out_dtype=None):
    """What rank `rank` of a ring of P = len(k_chunks) computes
    (intel_ring_flash_attn_forward, sp_aurora/intel_ring_flash_attn.py:72-148):
    at step t the rank holds KV chunk (rank - t) mod P (:75-76,131-134), computes iff
    `not causal or t <= rank` (:79), masks iff `causal and t == 0` (:88), merges in that
    order (:128), finally casts out to q.dtype (:143).
    q_local [B,s,H,D]; k_chunks/v_chunks: lists of [B,s,H,D].  Returns out [B,s,H,D], lse [B,H,s]."""
    P = len(k_chunks)
    out_dtype = out_dtype or q_local.dtype
    q = q_local.transpose(1, 2)
    out = lse = None
    for step in range(P):
        if causal and step > rank:
            continue
        c = (rank - step) % P
        b_out, b_lse = attn_block(q, k_chunks[c].transpose(1, 2), v_chunks[c].transpose(1, 2),
                                  softmax_scale, causal and step == 0, compute_dtype)
        if out is None:  # first update = cast/copy (sp_aurora/utils.py:116-122)
            out, lse = b_out, b_lse.unsqueeze(-1)
        else:
            out, lse = merge(out, lse, b_out, b_lse.unsqueeze(-1))
    return out.transpose(1, 2).to(out_dtype), lse.squeeze(-1)


def ring_forward(q, k, v, P, softmax_scale=None, causal=False, compute_dtype=CD, out_dtype=None):
    """All P ranks, one after the other, on contiguous sequence shards; q,k,v [B,S,H,D]."""
    qs, ks, vs = q.chunk(P, dim=1), list(k.chunk(P, dim=1)), list(v.chunk(P, dim=1))
    outs, lses = zip(*[ring_forward_rank(qs[r], ks, vs, r, softmax_scale, causal, compute_dtype, out_dtype)
                       for r in range(P)])
    return torch.cat(outs, dim=1), torch.cat(lses, dim=2)


def zigzag_order(S, P):
    """Row order of a zigzag-sharded sequence: with the S rows cut into 2P half-chunks, rank r holds
    half-chunk r followed by half-chunk 2P-1-r, and the ranks' shards are stacked in rank order.
    Returns idx (int64 [S]) with sharded = natural.index_select(1, idx).  The sharding the
    reference's test names (zigzag_sp_aurora_varlen_func,
    test/flash_attention/test_intel_ring_flash_attn_varlen.py:25,205-215) without shipping it:
    every rank of a causal ring then has the same amount of work."""
    if S % (2 * P):
        raise ValueError(f"zigzag sharding needs 2 * P = {2 * P} to divide the sequence length {S}")
    hc = S // (2 * P)
    idx = []
    for r in range(P):
        idx += list(range(r * hc, (r + 1) * hc)) + list(range((2 * P - 1 - r) * hc, (2 * P - r) * hc))
    return torch.tensor(idx, dtype=torch.int64)


def ring_forward_zigzag_rank(q_local, k_chunks, v_chunks, rank, softmax_scale=None, compute_dtype=CD, out_dtype=None):
    """Causal ring forward of rank `rank` on zigzag shards: the step loop of
    intel_ring_flash_attn_forward (sp_aurora/intel_ring_flash_attn.py:72-148) with the block of each
    step cut to what a zigzag shard can see.  The rank holds half-chunks (rank, 2P-1-rank); at step t
    it has the shard of rank c = (rank - t) mod P, half-chunks (c, 2P-1-c):
      t == 0       its own shard: plain causal attention on the local rows (the local order is the global one)
      c <  rank    every local query sees the first half of the shard (half-chunk c), none of the second
      c >  rank    only the second half of the local queries sees anything, and it sees the whole shard
    every step is merged with update_out_and_lse (for c > rank into the second half of the rows only)."""
    P = len(k_chunks)
    out_dtype = out_dtype or q_local.dtype
    hs = q_local.shape[1] // 2
    q = q_local.transpose(1, 2)
    out, lse = attn_block(q, k_chunks[rank].transpose(1, 2), v_chunks[rank].transpose(1, 2), softmax_scale, True, compute_dtype)
    lse = lse.unsqueeze(-1)
    for step in range(1, P):
        c = (rank - step) % P
        kc, vc = k_chunks[c].transpose(1, 2), v_chunks[c].transpose(1, 2)
        if c < rank:
            b_out, b_lse = attn_block(q, kc[:, :, :hs], vc[:, :, :hs], softmax_scale, False, compute_dtype)
            out, lse = merge(out, lse, b_out, b_lse.unsqueeze(-1))
        else:
            b_out, b_lse = attn_block(q[:, :, hs:], kc, vc, softmax_scale, False, compute_dtype)
            o2, l2 = merge(out[:, :, hs:], lse[:, :, hs:], b_out, b_lse.unsqueeze(-1))
            out = torch.cat([out[:, :, :hs], o2], dim=2)
            lse = torch.cat([lse[:, :, :hs], l2], dim=2)
    return out.transpose(1, 2).to(out_dtype), lse.squeeze(-1)


def ring_forward_zigzag(q, k, v, P, softmax_scale=None, compute_dtype=CD, out_dtype=None):
    """All P ranks of a causal zigzag ring; q,k,v [B,S,H,D] in zigzag-sharded row order (zigzag_order);
    out and lse come back in the same order."""
    qs, ks, vs = q.chunk(P, dim=1), list(k.chunk(P, dim=1)), list(v.chunk(P, dim=1))
    outs, lses = zip(*[ring_forward_zigzag_rank(qs[r], ks, vs, r, softmax_scale, compute_dtype, out_dtype) for r in range(P)])
    return torch.cat(outs, dim=1), torch.cat(lses, dim=2)


def full_attention(q, k, v, softmax_scale=None, causal=False, compute_dtype=CD):
    """Single-process path of the public function
    (sp_aurora/intel_ring_flash_attn.py:415-435): transpose to [B,H,S,D], block operator,
    transpose back.  q,k,v [B,S,H,D] -> out [B,S,H,D], lse [B,H,S]."""
    o, l = attn_block(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), softmax_scale, causal, compute_dtype)
    return o.transpose(1, 2), l


# --------------------------------------------------------------------------------------
# A7: backward
# --------------------------------------------------------------------------------------
def attn_backward_autograd(q, k, v, dout, softmax_scale=None, causal=False, compute_dtype=CD):
    """dq, dk, dv of full attention by torch autograd through the closed form — the
    'reference autograd' of the single-process path (sp_aurora/intel_ring_flash_attn.py:415-435
    has no autograd.Function, so gradients flow through native torch ops).  [B,S,H,D]."""
    q, k, v = [t.detach().to(compute_dtype).requires_grad_(True) for t in (q, k, v)]
    out, _ = full_attention(q, k, v, softmax_scale, causal, compute_dtype)
    out.backward(dout.to(compute_dtype))
    return q.grad, k.grad, v.grad


def attn_backward_block(q, k, v, dout, lse, delta, softmax_scale=None, causal=False, compute_dtype=CD):
    """Block-wise backward of one (q chunk, kv chunk) pair with the GLOBAL lse and delta:
        P = exp(S - lse); dV = P^T dO; dP = dO V^T; dS = P * (dP - delta);
        dQ = dS K * scale; dK = dS^T Q * scale.
    The schedule is the reference's (sp_aurora/intel_ring_flash_attn.py:192-258); the math is
    the exact gradient of ring attention (the reference back-propagates each block through an
    independently normalised softmax, :229-244, which is not that gradient when P > 1).
    Operator layout [B,H,S,D]; lse, delta [B,H,Sq]."""
    q, k, v, dout = [t.to(compute_dtype) for t in (q, k, v, dout)]
    if softmax_scale is None:
        softmax_scale = q.shape[-1] ** (-0.5)
    s = torch.matmul(q, k.transpose(-2, -1)) * softmax_scale
    if causal:
        s = s.masked_fill(causal_mask(q.shape[-2], k.shape[-2]), float("-inf"))
    p = torch.exp(s - lse.to(compute_dtype).unsqueeze(-1))
    dv = torch.matmul(p.transpose(-2, -1), dout)
    dp = torch.matmul(dout, v.transpose(-2, -1))
    ds = p * (dp - delta.to(compute_dtype).unsqueeze(-1))
    dq = torch.matmul(ds, k) * softmax_scale
    dk = torch.matmul(ds.transpose(-2, -1), q) * softmax_scale
    return dq, dk, dv


def ring_backward(q, k, v, out, lse, dout, P, softmax_scale=None, causal=False, compute_dtype=CD):
    """Ring backward over all ranks with the block-wise recompute: dq accumulated per q chunk
    (sp_aurora/intel_ring_flash_attn.py:250-255), dk/dv per kv chunk summed over the q chunks
    that visited it (:257-258,267).  Public layout [B,S,H,D]; lse [B,H,S]."""
    delta = (out.to(compute_dtype) * dout.to(compute_dtype)).sum(-1).transpose(1, 2)  # [B,H,S]
    B, S, H, D = q.shape
    s = S // P
    dq = torch.zeros(B, S, H, D, dtype=compute_dtype)
    dk = torch.zeros_like(dq)
    dv = torch.zeros_like(dq)
    for r in range(P):
        rs = slice(r * s, (r + 1) * s)
        for step in range(P):
            if causal and step > r:
                continue
            c = (r - step) % P
            cs = slice(c * s, (c + 1) * s)
            bq, bk, bv = attn_backward_block(
                q[:, rs].transpose(1, 2), k[:, cs].transpose(1, 2), v[:, cs].transpose(1, 2),
                dout[:, rs].transpose(1, 2), lse[:, :, rs], delta[:, :, rs], softmax_scale,
                causal and step == 0, compute_dtype)
            dq[:, rs] += bq.transpose(1, 2)
            dk[:, cs] += bk.transpose(1, 2)
            dv[:, cs] += bv.transpose(1, 2)
    return dq, dk, dv


# --------------------------------------------------------------------------------------
# A8: Ulysses re-layout.  all_to_all_single(output, input) on P ranks with equal splits is,
# by definition, output[r].chunk(P)[q] = input[q].chunk(P)[r]; `_a2a` applies it to the
# list of per-rank send buffers.
# --------------------------------------------------------------------------------------
def _a2a(send):
    P = len(send)
    parts = [t.chunk(P, dim=0) for t in send]
    return [torch.cat([parts[q][r] for q in range(P)], dim=0) for r in range(P)]


def all_to_all_4d_s2h(xs):
    """Scatter heads (dim 2), gather sequence (dim 1) — the literal op chain of
    intel_all_to_all_4d, sp_aurora/intel_ulysses_attn.py:86-112, run for every rank.
    xs: list of P tensors [B, s, H, D]  ->  list of P tensors [B, P*s, H/P, D]."""
    P = len(xs)
    send = []
    for x in xs:
        bs, shard_seq, heads, hd = x.shape
        send.append(x.reshape(bs, shard_seq, P, heads // P, hd).transpose(0, 2).contiguous())
    recv = _a2a(send)
    outs = []
    for o in recv:
        _, shard_seq, bs, sh, hd = o.shape
        outs.append(o.reshape(P * shard_seq, bs, sh, hd).transpose(0, 1).contiguous())
    return outs


def all_to_all_4d_h2s(ys):
    """Scatter sequence (dim 1), gather heads (dim 2) — sp_aurora/intel_ulysses_attn.py:114-140.
    ys: list of P tensors [B, P*s, h, D]  ->  list of P tensors [B, s, P*h, D]."""
    P = len(ys)
    send = []
    for y in ys:
        bs, seq, sh, hd = y.shape
        s = seq // P
        t = y.reshape(bs, P, s, sh, hd).transpose(0, 3).transpose(0, 1).contiguous()
        send.append(t.reshape(P, sh, s, bs, hd))
    recv = _a2a(send)
    outs = []
    for o in recv:
        _, sh, s, bs, hd = o.shape
        outs.append(o.reshape(P * sh, s, bs, hd).transpose(0, 2).contiguous())
    return outs


def all_to_all_5d_s2h(xs):
    """Packed qkv variant, forward: sp_aurora/comm/all_to_all.py:266-298.
    xs: list of P tensors [B, s, 3, H, D] -> list of [B, P*s, 3, H/P, D]."""
    P = len(xs)
    send = []
    for x in xs:
        bs, s, t, hc, hs = x.shape
        send.append(x.reshape(bs, s, t, P, hc // P, hs).transpose(0, 3).contiguous())
    recv = _a2a(send)
    outs = []
    for o in recv:
        _, s, t, bs, shc, hs = o.shape
        o = o.reshape(P * s, t, bs, shc, hs).transpose(0, 2).transpose(1, 2).contiguous()
        outs.append(o.reshape(bs, P * s, t, shc, hs))
    return outs


def all_to_all_5d_h2s(ys):
    """Packed qkv variant, inverse: sp_aurora/comm/all_to_all.py:300-333.
    ys: list of P tensors [B, P*s, 3, h, D] -> list of [B, s, 3, P*h, D]."""
    P = len(ys)
    send = []
    for y in ys:
        bs, seq, t, shc, hs = y.shape
        s = seq // P
        x = y.reshape(bs, P, s, t, shc, hs).transpose(0, 4).transpose(0, 1).contiguous()
        send.append(x.reshape(P, shc, s, t, bs, hs))
    recv = _a2a(send)
    outs = []
    for o in recv:
        _, shc, s, t, bs, hs = o.shape
        o = o.reshape(P * shc, s, t, bs, hs).transpose(0, 3).contiguous()
        outs.append(o.reshape(bs, s, t, P * shc, hs))
    return outs


def relayout_s2h_formula(x):
    """Index formula of the same permutation on stacked shards:
    y[r, b, q*s+t, (c,) j, :] = x[q, b, t, (c,) r*h+j, :].   x [P,B,s,(pack,)H,D]."""
    P = x.shape[0]
    if x.dim() == 5:
        _, B, s, H, D = x.shape
        return x.view(P, B, s, P, H // P, D).permute(3, 1, 0, 2, 4, 5).reshape(P, B, P * s, H // P, D)
    _, B, s, c, H, D = x.shape
    return x.view(P, B, s, c, P, H // P, D).permute(4, 1, 0, 2, 3, 5, 6).reshape(P, B, P * s, c, H // P, D)


def relayout_h2s_formula(y):
    """x[r, b, t, (c,) q*h+j, :] = y[q, b, r*s+t, (c,) j, :].   y [P,B,P*s,(pack,)h,D]."""
    P = y.shape[0]
    if y.dim() == 5:
        _, B, S, h, D = y.shape
        return y.view(P, B, P, S // P, h, D).permute(2, 1, 3, 0, 4, 5).reshape(P, B, S // P, P * h, D)
    _, B, S, c, h, D = y.shape
    return y.view(P, B, P, S // P, c, h, D).permute(2, 1, 3, 4, 0, 5, 6).reshape(P, B, S // P, c, P * h, D)


# --------------------------------------------------------------------------------------
# A9: Ulysses forward (composition)
# --------------------------------------------------------------------------------------
def ulysses_forward(qs, ks, vs, softmax_scale=None, causal=False, compute_dtype=CD):
    """intel_ulysses_flash_attn_forward for all ranks (sp_aurora/intel_ulysses_attn.py:233-287):
    re-layout q,k,v (:233), attention over the full sequence on H/P heads (:249-276),
    inverse re-layout of out (:281); lse stays head-sharded (:284-287).
    qs/ks/vs: lists of P tensors [B,s,H,D] -> (list of out [B,s,H,D], list of lse [B,h,S])."""
    yq, yk, yv = all_to_all_4d_s2h(qs), all_to_all_4d_s2h(ks), all_to_all_4d_s2h(vs)
    outs, lses = [], []
    for a, b, c in zip(yq, yk, yv):
        o, l = full_attention(a, b, c, softmax_scale, causal, compute_dtype)
        outs.append(o.to(qs[0].dtype))
        lses.append(l)
    return all_to_all_4d_h2s(outs), lses


# --------------------------------------------------------------------------------------
# brute force (pure Python floats) — used only to pin the functions above on tiny inputs
# --------------------------------------------------------------------------------------
def brute_attention(q, k, v, scale, causal):
    """Triple loop over python floats.  q [Sq][D], k,v [Sk][D] nested lists -> (out, lse)."""
    out, lse = [], []
    for i, qi in enumerate(q):
        sc = []
        for j, kj in enumerate(k):
            if causal and j > i:
                continue
            sc.append((j, scale * sum(a * b for a, b in zip(qi, kj))))
        m = max(s for _, s in sc)
        z = sum(math.exp(s - m) for _, s in sc)
        lse.append(m + math.log(z))
        row = [0.0] * len(v[0])
        for j, s in sc:
            w = math.exp(s - m) / z
            for d in range(len(row)):
                row[d] += w * v[j][d]
        out.append(row)
    return out, lse
