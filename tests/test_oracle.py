"""Pins of the CPU oracle (oracle/attn_oracle.py).  The reference ships no golden vectors for
this path (its tests compare against inline closed forms), so each oracle function is pinned
against something it does not share code with: pure-Python brute force, closed forms,
torch library routines in fp64, and the invariants the reference's own tests assert."""
import math

import pytest
import torch
import torch.nn.functional as F

from conftest import rand, rand_qkv
from oracle import attn_oracle as O

F64 = torch.float64


# ------------------------------------------------------------------ block operator (A1-A3)
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("sq,sk", [(5, 5), (7, 3), (3, 8)])
def test_block_matches_brute_force(sq, sk, causal):
    q, = rand_qkv((sq, 4), 10, F64, n=1)
    k, v = rand_qkv((sk, 4), 11, F64, n=2)
    out, lse = O.attn_block(q[None, None], k[None, None], v[None, None], 0.37, causal)
    b_out, b_lse = O.brute_attention(q.tolist(), k.tolist(), v.tolist(), 0.37, causal)
    assert torch.allclose(out[0, 0], torch.tensor(b_out, dtype=F64), atol=1e-12)
    assert torch.allclose(lse[0, 0], torch.tensor(b_lse, dtype=F64), atol=1e-12)


def test_block_closed_forms():
    B, H, S, D = 2, 3, 9, 8
    q, k, v = rand_qkv((B, H, S, D), 12, F64)
    # identical keys: uniform weights -> out = mean(v), lse = log(S) + scale * q.k0
    k_same = k[:, :, :1].expand(B, H, S, D)
    out, lse = O.attn_block(q, k_same, v, 0.5, False)
    assert torch.allclose(out, v.mean(2, keepdim=True).expand_as(out), atol=1e-12)
    assert torch.allclose(lse, math.log(S) + 0.5 * (q * k[:, :, :1]).sum(-1), atol=1e-12)
    # constant V: rows of P sum to one
    vc = torch.full_like(v, 2.5)
    assert torch.allclose(O.attn_block(q, k, vc, None, True)[0], vc, atol=1e-12)
    # causal row 0 sees key 0 only
    out, lse = O.attn_block(q, k, v, 0.5, True)
    assert torch.allclose(out[:, :, 0], v[:, :, 0], atol=1e-12)
    assert torch.allclose(lse[:, :, 0], 0.5 * (q[:, :, 0] * k[:, :, 0]).sum(-1), atol=1e-12)
    # one dominant key: out -> that key's value, lse -> its score
    kd = k.clone()
    kd[:, :, 4] = q[:, :, 2] * 1e3
    out, lse = O.attn_block(q[:, :, 2:3], kd, v, 1.0, False)
    assert torch.allclose(out[:, :, 0], v[:, :, 4], atol=1e-9)
    assert torch.allclose(lse[:, :, 0], 1e3 * (q[:, :, 2] ** 2).sum(-1), rtol=1e-12)
    # exp(lse) is the partition function
    s = torch.einsum("bhid,bhjd->bhij", q, k) * 0.25
    assert torch.allclose(torch.exp(O.attn_block(q, k, v, 0.25, False)[1]), torch.exp(s).sum(-1), rtol=1e-12)


@pytest.mark.parametrize("causal", [False, True])
def test_block_matches_torch_library(causal):
    """Same comparison the reference's tests make (test/flash_attention/test_flash_attention_validation.py:31-63):
    softmax / logsumexp / SDPA from the library."""
    q, k, v = rand_qkv((2, 4, 33, 16), 13, F64)
    out, lse = O.attn_block(q, k, v, None, causal)
    s = torch.matmul(q, k.transpose(-1, -2)) / 4.0
    if causal:
        s = s.masked_fill(torch.ones(33, 33, dtype=torch.bool).triu(1), float("-inf"))
    assert torch.allclose(out, torch.matmul(torch.softmax(s, -1), v), atol=1e-12)
    assert torch.allclose(lse, torch.logsumexp(s, -1), atol=1e-12)
    assert torch.allclose(out, F.scaled_dot_product_attention(q, k, v, is_causal=causal), atol=1e-12)
    # default scale is D ** -0.5 (sp_aurora/intel_flash_attn.py:46-47)
    assert torch.equal(out, O.attn_block(q, k, v, 16 ** -0.5, causal)[0])


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("block", [4, 16, 64])
def test_tiled_and_sdpa_restatements_agree_with_dense(block, causal):
    q, k, v = rand_qkv((1, 2, 37, 8), 14, F64)
    d_out, d_lse = O.attn_block(q, k, v, None, causal)
    t_out, t_lse = O.attn_block_tiled(q, k, v, None, causal, block)
    s_out, s_lse = O.attn_block_sdpa(q, k, v, None, causal)
    assert torch.allclose(t_out, d_out, atol=1e-12) and torch.allclose(t_lse, d_lse, atol=1e-12)
    assert torch.allclose(s_out, d_out, atol=1e-12) and torch.allclose(s_lse, d_lse, atol=1e-12)


def test_reference_tiled_rescale_defect_is_what_the_docstring_says():
    """The literal line of the reference agrees with attention for one key tile, keeps the lse
    right and gets `out` wrong as soon as a row visits two tiles."""
    q, k, v = rand_qkv((1, 1, 8, 4), 15, F64)
    dense, d_lse = O.attn_block(q, k, v)
    one, lse1 = O.attn_block_tiled(q, k, v, block_size=8, literal_rescale=True)
    two, lse2 = O.attn_block_tiled(q, k, v, block_size=4, literal_rescale=True)
    assert torch.allclose(one, dense, atol=1e-12)
    assert torch.allclose(lse2, d_lse, atol=1e-12)
    assert (two - dense).abs().max() > 1e-2


def test_reference_tiled_mask_defect_is_what_the_docstring_says():
    """diagonal = j - i + 1 as written in the reference equals the causal mask on the diagonal
    tile only; on an earlier key tile it hides every key."""
    q, k, v = rand_qkv((1, 1, 8, 4), 16, F64)
    _, d_lse = O.attn_block(q, k, v, None, True)
    _, one = O.attn_block_tiled(q, k, v, None, True, block_size=8, literal_mask=True)
    _, two = O.attn_block_tiled(q, k, v, None, True, block_size=4, literal_mask=True)
    assert torch.allclose(one, d_lse, atol=1e-12)
    assert torch.allclose(two[..., :4], d_lse[..., :4], atol=1e-12)
    assert not torch.isfinite(two[..., 4:]).any() or (two[..., 4:] - d_lse[..., 4:]).abs().min() > 1e-3


# ------------------------------------------------------------------ merge (A4)
def _partials(seed, S=6, D=4, n=3):
    q, = rand_qkv((1, 2, S, D), seed, F64, n=1)
    parts = []
    for i in range(n):
        k, v = rand_qkv((1, 2, 5 + i, D), seed + 1 + i, F64, n=2)
        parts.append((k, v))
    return q, parts


def test_merge_of_split_kv_equals_unsplit_attention():
    q, parts = _partials(20)
    k_all = torch.cat([p[0] for p in parts], 2)
    v_all = torch.cat([p[1] for p in parts], 2)
    full_out, full_lse = O.attn_block(q, k_all, v_all, 0.3)
    out = lse = None
    for k, v in parts:
        o, l = O.attn_block(q, k, v, 0.3)
        out, lse = (o, l.unsqueeze(-1)) if out is None else O.merge(out, lse, o, l.unsqueeze(-1))
    assert torch.allclose(out, full_out, atol=1e-12)
    assert torch.allclose(lse.squeeze(-1), full_lse, atol=1e-12)


def test_merge_closed_form_and_algebra():
    g = torch.Generator().manual_seed(21)
    o1, o2, o3 = [torch.randn(4, 5, 3, generator=g, dtype=F64) for _ in range(3)]
    l1, l2, l3 = [torch.randn(4, 5, 1, generator=g, dtype=F64) * 3 for _ in range(3)]
    out, lse = O.merge(o1, l1, o2, l2)
    new = torch.logaddexp(l1, l2)
    assert torch.allclose(lse, new, atol=1e-12)
    assert torch.allclose(out, torch.exp(l1 - new) * o1 + torch.exp(l2 - new) * o2, atol=1e-12)
    # commutative
    out_r, lse_r = O.merge(o2, l2, o1, l1)
    assert torch.allclose(out, out_r, atol=1e-12) and torch.allclose(lse, lse_r, atol=1e-12)
    # associative
    a = O.merge(*O.merge(o1, l1, o2, l2), o3, l3)
    b = O.merge(o1, l1, *O.merge(o2, l2, o3, l3))
    assert torch.allclose(a[0], b[0], atol=1e-12) and torch.allclose(a[1], b[1], atol=1e-12)
    # a block that saw nothing (lse = -inf) changes nothing
    out_i, lse_i = O.merge(o1, l1, o2, torch.full_like(l2, float("-inf")))
    assert torch.equal(out_i, o1) and torch.equal(lse_i, l1)
    # fp32 associativity within 1e-6 (the bound the build plan quotes)
    f = lambda *t: [x.float() for x in t]
    a = O.merge(*O.merge(*f(o1, l1, o2, l2)), *f(o3, l3))
    b = O.merge(*f(o1, l1), *O.merge(*f(o2, l2, o3, l3)))
    assert (a[0] - b[0]).abs().max() < 2e-6


# ------------------------------------------------------------------ ring schedule (A5, A6)
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("P", [1, 2, 4])
def test_ring_equals_full_attention(P, causal):
    """The invariant of test/test_ring_attention_full_accuracy.py:122-171."""
    q, k, v = rand_qkv((2, 16, 3, 8), 30, F64)
    f_out, f_lse = O.full_attention(q, k, v, None, causal)
    r_out, r_lse = O.ring_forward(q, k, v, P, None, causal)
    assert torch.allclose(r_out, f_out, atol=1e-12)
    assert torch.allclose(r_lse, f_lse, atol=1e-12)


def test_ring_schedule_visits_chunks_in_ring_order():
    """Rank r, step t holds chunk (r - t) mod P; causal ranks skip t > r and mask only t == 0
    (sp_aurora/intel_ring_flash_attn.py:75-95).  Checked by counting with tagged values."""
    P, s = 4, 2
    # v chunk c is the constant c+1, keys are zero: every visited key gets the same weight
    q = torch.zeros(1, s, 1, 2, dtype=F64)
    ks = [torch.zeros(1, s, 1, 2, dtype=F64) for _ in range(P)]
    vs = [torch.full((1, s, 1, 2), float(c + 1), dtype=F64) for c in range(P)]
    for r in range(P):
        out, lse = O.ring_forward_rank(q, ks, vs, r, 1.0, True)
        # row i of rank r sees chunks 0..r-1 fully and i+1 keys of chunk r
        for i in range(s):
            n = r * s + i + 1
            want = (sum((c + 1) * s for c in range(r)) + (r + 1) * (i + 1)) / n
            assert abs(out[0, i, 0, 0].item() - want) < 1e-12
            assert abs(lse[0, 0, i].item() - math.log(n)) < 1e-12
        out, lse = O.ring_forward_rank(q, ks, vs, r, 1.0, False)
        assert torch.allclose(out, torch.full_like(out, (1 + 2 + 3 + 4) / 4))


@pytest.mark.parametrize("P", [1, 2, 3, 4])
def test_zigzag_ring_equals_full_causal_attention_after_unpermuting(P):
    """The zigzag schedule against the closed form: shard the rows (rank r gets half-chunks r and
    2P-1-r), run the ring, undo the permutation, compare with full causal attention in natural order.
    A wrong half, a wrong comparison (c < rank) or a merge into the wrong rows fails it."""
    S = 8 * P
    q, k, v = rand_qkv((2, S, 3, 8), 31, F64)
    idx = O.zigzag_order(S, P)
    assert sorted(idx.tolist()) == list(range(S))
    hc = S // (2 * P)
    for r in range(P):  # rank r's shard = half-chunk r, then half-chunk 2P-1-r
        assert idx[2 * hc * r:2 * hc * (r + 1)].tolist() == list(range(r * hc, (r + 1) * hc)) + list(range((2 * P - 1 - r) * hc, (2 * P - r) * hc))
    f_out, f_lse = O.full_attention(q, k, v, None, True)
    z_out, z_lse = O.ring_forward_zigzag(q[:, idx], k[:, idx], v[:, idx], P, None)
    inv = torch.argsort(idx)
    assert torch.allclose(z_out[:, inv], f_out, atol=1e-12)
    assert torch.allclose(z_lse[:, :, inv], f_lse, atol=1e-12)


def test_zigzag_ring_balances_the_work_of_the_ranks():
    """Counting with tagged values: keys are zero (every visible key weighs the same), so exp(lse) of a
    row is the number of keys it sees; per rank these sum to the same total, P * s * s / 2 + s / 2."""
    P, s = 4, 4
    S = P * s
    q = torch.zeros(1, S, 1, 2, dtype=F64)
    _, lse = O.ring_forward_zigzag(q, q, q, P, 1.0)
    seen = torch.exp(lse[0, 0]).view(P, s).sum(1)
    assert torch.allclose(seen, torch.full((P,), P * s * s / 2 + s / 2, dtype=F64))
    # and a row at natural position n sees n + 1 keys
    idx = O.zigzag_order(S, P)
    assert torch.allclose(torch.exp(lse[0, 0]), (idx + 1).to(F64))


def test_packed_equals_unpacked():
    """test/test_ring_attention_comprehensive.py:205-218."""
    qkv = rand((1, 8, 3, 2, 4), 31, F64)
    a, _ = O.ring_forward(qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2], 2, None, True)
    b, _ = O.ring_forward(qkv[:, :, 0].contiguous(), qkv[:, :, 1].contiguous(), qkv[:, :, 2].contiguous(), 2, None, True)
    assert torch.equal(a, b)


# ------------------------------------------------------------------ backward (A7)
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("P", [1, 2, 4])
def test_blockwise_backward_equals_autograd(P, causal):
    q, k, v, dout = rand_qkv((1, 8, 2, 4), 40, F64, n=4)
    out, lse = O.full_attention(q, k, v, None, causal)
    want = O.attn_backward_autograd(q, k, v, dout, None, causal)
    got = O.ring_backward(q, k, v, out, lse, dout, P, None, causal)
    for g, w in zip(got, want):
        assert torch.allclose(g, w, atol=1e-12)


def test_backward_matches_finite_differences():
    """test/flash_attention/test_flash_attention_validation.py:394-437 checks gradients this way."""
    q, k, v, dout = rand_qkv((1, 4, 1, 3), 41, F64, n=4)
    dq, dk, dv = O.attn_backward_autograd(q, k, v, dout, 0.7, True)
    loss = lambda a, b, c: (O.full_attention(a, b, c, 0.7, True)[0] * dout).sum()
    eps = 1e-6
    for x, g, idx in ((q, dq, (0, 2, 0, 1)), (k, dk, (0, 1, 0, 2)), (v, dv, (0, 0, 0, 0))):
        xp, xm = x.clone(), x.clone()
        xp[idx] += eps
        xm[idx] -= eps
        args_p = [xp if t is x else t for t in (q, k, v)]
        args_m = [xm if t is x else t for t in (q, k, v)]
        fd = (loss(*args_p) - loss(*args_m)) / (2 * eps)
        assert abs(fd.item() - g[idx].item()) < 1e-7


# ------------------------------------------------------------------ re-layout (A8)
def _tagged(P, B, s, H, D, pack=None):
    """Value encodes (rank, b, t, c, head, d)."""
    shape = (P, B, s) + ((pack,) if pack else ()) + (H, D)
    return torch.arange(math.prod(shape), dtype=torch.int64).view(shape)


@pytest.mark.parametrize("P,B,s,H,D", [(2, 1, 3, 4, 2), (4, 2, 2, 8, 3), (3, 2, 4, 6, 1)])
def test_relayout_4d_lands_where_the_formula_says(P, B, s, H, D):
    x = _tagged(P, B, s, H, D)
    ys = O.all_to_all_4d_s2h(list(x))
    h = H // P
    for r in range(P):
        assert ys[r].shape == (B, P * s, h, D)  # test/ulysses/test_intel_alltoall_4d.py:93-100
        for b in range(B):
            for q in range(P):
                for t in range(s):
                    for j in range(h):
                        assert torch.equal(ys[r][b, q * s + t, j], x[q, b, t, r * h + j])
    y = torch.stack(ys)
    assert torch.equal(y, O.relayout_s2h_formula(x))
    back = O.all_to_all_4d_h2s(ys)
    assert back[0].shape == (B, s, H, D)  # :140-147
    assert torch.equal(torch.stack(back), x)
    assert torch.equal(O.relayout_h2s_formula(y), x)


@pytest.mark.parametrize("P,B,s,H,D", [(2, 1, 3, 4, 2), (4, 2, 2, 8, 3)])
def test_relayout_5d_lands_where_the_formula_says(P, B, s, H, D):
    x = _tagged(P, B, s, H, D, pack=3)
    ys = O.all_to_all_5d_s2h(list(x))
    h = H // P
    for r in range(P):
        assert ys[r].shape == (B, P * s, 3, h, D)
        for q in range(P):
            for t in range(s):
                for c in range(3):
                    assert torch.equal(ys[r][:, q * s + t, c], x[q, :, t, c, r * h:(r + 1) * h])
    y = torch.stack(ys)
    assert torch.equal(y, O.relayout_s2h_formula(x))
    assert torch.equal(torch.stack(O.all_to_all_5d_h2s(ys)), x)
    assert torch.equal(O.relayout_h2s_formula(y), x)
    # the packed re-layout is the 4-D one applied to each of q, k, v
    for c in range(3):
        assert torch.equal(y[:, :, :, c], O.relayout_s2h_formula(x[:, :, :, c].contiguous()))


# ------------------------------------------------------------------ Ulysses (A9)
@pytest.mark.parametrize("causal", [False, True])
def test_ulysses_equals_full_attention(causal):
    """test/verification/test_ulysses_fixed.py:165-344 compares against attention on the gathered sequence."""
    P, B, s, H, D = 2, 1, 4, 4, 8
    q, k, v = rand_qkv((B, P * s, H, D), 50, F64)
    outs, lses = O.ulysses_forward(list(q.chunk(P, 1)), list(k.chunk(P, 1)), list(v.chunk(P, 1)), None, causal)
    f_out, f_lse = O.full_attention(q, k, v, None, causal)
    assert torch.allclose(torch.cat(outs, 1), f_out, atol=1e-12)
    assert torch.allclose(torch.cat(lses, 1), f_lse, atol=1e-12)  # lse stays head-sharded
