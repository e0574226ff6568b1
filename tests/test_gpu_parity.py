"""GPU parity: the HIP path (through the C ABI) against the CPU oracle on the same seeded inputs.

Tolerances: fp32 out atol 1e-5; bf16 out atol 2e-2 / rtol 1.6e-2;
lse atol 1e-3; re-layout bit-exact.  fp16 uses the bf16 bound (it is tighter in practice).
The oracle computes in float64 from the inputs at their storage precision.
"""
import hashlib
import os

import numpy as np
import pytest
import torch

from conftest import rand, rand_qkv
from oracle import attn_oracle as O
import sp_aurora_amd as spa
from sp_aurora_amd import _lib, ops

pytestmark = pytest.mark.gpu
DEV = "cuda"
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

OUT_TOL = {torch.float32: dict(atol=1e-5, rtol=1e-3), torch.bfloat16: dict(atol=2e-2, rtol=1.6e-2),
           torch.float16: dict(atol=2e-2, rtol=1.6e-2)}
LSE_ATOL = 1e-3


def check_out(got, want, dtype, what="out"):
    got = got.detach().cpu().to(torch.float64)
    want = want.to(torch.float64)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    tol = OUT_TOL[dtype]
    assert torch.isfinite(got).all(), f"{what}: {int((~torch.isfinite(got)).sum())} non-finite values"
    bad = (got - want).abs() > tol["atol"] + tol["rtol"] * want.abs()
    assert not bad.any(), f"{what}: {int(bad.sum())} elements out of tolerance, max abs err {(got - want).abs().max():.3e}"


def check_lse(got, want):
    got = got.detach().cpu().to(torch.float64)
    assert got.dtype == torch.float64 and got.shape == want.shape
    err = (got - want.to(torch.float64)).abs().max().item()
    assert err <= LSE_ATOL, f"lse max abs err {err:.3e}"


# ------------------------------------------------------------------ block operator
BLOCK_CASES = [
    # B, H, Sq, Sk, D, causal
    (1, 2, 64, 64, 32, True),     # test/flash_attention/test_flash_attention_simple.py:74-137
    (1, 4, 64, 64, 32, True),     # test_flash_attention_validation.py:76-134, config 1
    (2, 8, 128, 128, 64, False),  # config 2
    (1, 12, 256, 256, 64, True),  # config 3
    (2, 16, 512, 512, 128, False),  # config 4 (batch halved to keep the CPU oracle quick)
    (1, 3, 1, 1, 64, False),      # a single query, a single key
    (1, 2, 1, 200, 128, False),   # decode-like
    (2, 3, 77, 133, 32, False),   # ragged, Sq != Sk
    (1, 2, 200, 200, 64, True),   # ragged causal
    (1, 2, 130, 67, 128, True),   # causal with fewer keys than queries
    (1, 2, 67, 130, 128, True),   # causal with more keys than queries
    (1, 1, 384, 320, 128, False),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,H,Sq,Sk,D,causal", BLOCK_CASES)
def test_block_forward_matches_oracle(B, H, Sq, Sk, D, causal, dtype):
    q, = rand_qkv((B, H, Sq, D), 42, dtype, n=1)
    k, v = rand_qkv((B, H, Sk, D), 43, dtype, n=2)
    want_out, want_lse = O.attn_block(q, k, v, None, causal)
    out, lse = spa._flash_attn_forward(q.to(DEV), k.to(DEV), v.to(DEV), causal=causal)
    assert out.dtype == dtype and lse.dtype == torch.float32
    assert out.shape == (B, H, Sq, D) and lse.shape == (B, H, Sq)
    check_out(out, want_out, dtype)
    check_lse(lse, want_lse)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_block_forward_scale_and_layouts(dtype):
    """softmax_scale is honoured, and [B,S,H,D] / [B,H,S,D] / packed strided views give one answer."""
    B, S, H, D = 2, 96, 3, 64
    qkv = rand((B, S, 3, H, D), 44, dtype)
    q, k, v = qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]
    want_out, want_lse = O.full_attention(q, k, v, 0.2, True)
    dq = qkv.to(DEV)
    o1, l1 = ops.flash_fwd(dq[:, :, 0], dq[:, :, 1], dq[:, :, 2], 0.2, True, layout="bshd")  # strided views
    o2, l2 = ops.flash_fwd(q.to(DEV), k.to(DEV), v.to(DEV), 0.2, True, layout="bshd")
    o3, l3 = spa.intel_flash_attn_forward(q.transpose(1, 2).to(DEV), k.transpose(1, 2).to(DEV),
                                          v.transpose(1, 2).to(DEV), softmax_scale=0.2, causal=True)
    check_out(o1, want_out, dtype)
    check_lse(l1, want_lse)
    assert torch.equal(o1, o2) and torch.equal(l1, l2)
    assert torch.equal(o1, o3.transpose(1, 2)) and torch.equal(l1, l3)


def test_block_forward_special_cases():
    """Closed forms on the device: uniform keys -> mean(V); constant V -> V; causal row 0 -> v[0]."""
    B, H, S, D = 1, 2, 160, 64
    q, k, v = rand_qkv((B, H, S, D), 45, torch.float32)
    k_same = k[:, :, :1].expand(B, H, S, D).contiguous()
    out, lse = spa._flash_attn_forward(q.to(DEV), k_same.to(DEV), v.to(DEV), softmax_scale=0.5)
    assert torch.allclose(out.cpu(), v.mean(2, keepdim=True).expand_as(v), atol=1e-5)
    assert torch.allclose(lse.cpu(), np.log(S) + 0.5 * (q * k[:, :, :1]).sum(-1), atol=1e-4)
    vc = torch.full_like(v, 2.5)
    out, _ = spa._flash_attn_forward(q.to(DEV), k.to(DEV), vc.to(DEV), causal=True)
    assert torch.allclose(out.cpu(), vc, atol=1e-5)
    out, lse = spa._flash_attn_forward(q.to(DEV), k.to(DEV), v.to(DEV), softmax_scale=0.5, causal=True)
    assert torch.allclose(out[:, :, 0].cpu(), v[:, :, 0], atol=1e-6)
    assert torch.allclose(lse[:, :, 0].cpu(), 0.5 * (q[:, :, 0] * k[:, :, 0]).sum(-1), atol=1e-5)


def test_block_forward_is_deterministic():
    """test/flash_attention/test_lse_computation.py:110-112."""
    q, k, v = [t.to(DEV) for t in rand_qkv((1, 4, 300, 128), 46, torch.bfloat16)]
    a = spa._flash_attn_forward(q, k, v, causal=True)
    b = spa._flash_attn_forward(q, k, v, causal=True)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


def test_large_scores_do_not_overflow():
    q, k, v = rand_qkv((1, 2, 128, 64), 47, torch.bfloat16, scale=30.0)
    want_out, want_lse = O.attn_block(q, k, v, None, False)
    out, lse = spa._flash_attn_forward(q.to(DEV), k.to(DEV), v.to(DEV))
    assert torch.isfinite(out).all() and torch.isfinite(lse).all()
    check_out(out, want_out, torch.bfloat16)
    assert torch.allclose(lse.cpu().double(), want_lse, rtol=1e-5, atol=1e-3)


# ------------------------------------------------------------------ golden fixtures
def _digest(*tensors):
    h = hashlib.sha256()
    for t in tensors:
        h.update(t.contiguous().view(torch.uint8).numpy().tobytes())
    return h.hexdigest()


GOLDEN_CASES = {
    "cfg1_fp32_b1_s512_h8_d64": (0, torch.float32, (1, 512, 8, 64), False, 1, 1.0 / 8.0),
    "simple_fp32_b1_s64_h2_d32_causal": (42, torch.float32, (1, 64, 2, 32), True, 1, None),
    "ring4_bf16_b1_s256_h4_d64_causal": (7, torch.bfloat16, (1, 256, 4, 64), True, 4, None),
    "ring2_fp16_b2_s128_h2_d128": (8, torch.float16, (2, 128, 2, 128), False, 2, None),
    "ring4_fp32_b1_s96_h2_d32_causal": (9, torch.float32, (1, 96, 2, 32), True, 4, None),
}


@pytest.mark.parametrize("name", sorted(GOLDEN_CASES))
def test_golden_fixture(name):
    """Committed vectors (tests/golden/make_golden.py); cfg1_* is benchmark config 1."""
    seed, dtype, shape, causal, P, scale = GOLDEN_CASES[name]
    fx = np.load(os.path.join(GOLDEN, name + ".npz"))
    q, k, v = rand_qkv(shape, seed, dtype)
    assert _digest(q, k, v) == str(fx["input_sha256"]), "seeded inputs differ from the ones the fixture was made from"
    res = spa.ring_flash_attn_func(q.to(DEV), k.to(DEV), v.to(DEV), softmax_scale=scale, causal=causal,
                                   return_attn_probs=True, ring_size=P)
    out, lse, none = res
    assert none is None
    check_out(out, torch.from_numpy(fx["out"]), dtype)
    check_lse(lse, torch.from_numpy(fx["lse"]))


# ------------------------------------------------------------------ merge
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_merge_kernel_matches_oracle(dtype):
    B, H, S, D = 2, 3, 50, 64
    g = torch.Generator().manual_seed(60)
    acc = torch.randn(B, S, H, D, generator=g)
    lse = torch.randn(B, H, S, generator=g) * 3
    blk = torch.randn(B, S, H, D, generator=g).to(dtype)
    blk_lse = torch.randn(B, H, S, generator=g) * 3
    blk_lse[0, 0, :5] = float("-inf")   # a block that saw nothing leaves the row alone
    want_out, want_lse = O.merge(acc.double().transpose(1, 2), lse.double().unsqueeze(-1),
                                 blk.double().transpose(1, 2), blk_lse.double().unsqueeze(-1))
    d_acc, d_lse = acc.to(DEV), lse.to(DEV)
    ops.merge(d_acc, d_lse, blk.to(DEV), blk_lse.to(DEV), layout="bshd")
    assert torch.allclose(d_acc.cpu().double(), want_out.transpose(1, 2), atol=2e-6, rtol=1e-6)
    assert torch.allclose(d_lse.cpu().double(), want_lse.squeeze(-1), atol=2e-6, rtol=1e-6)
    assert torch.equal(d_acc[0, :5, 0].cpu(), acc[0, :5, 0])
    # init = cast/copy; finalize = cast
    ops.merge(d_acc, d_lse, blk.to(DEV), blk_lse.to(DEV), layout="bshd", init=True)
    assert torch.equal(d_acc.cpu(), blk.float()) and torch.equal(d_lse.cpu(), blk_lse)
    fin = ops.finalize(acc.to(DEV), dtype, layout="bshd")
    assert torch.equal(fin.cpu(), acc.to(dtype))


def test_update_out_and_lse_follows_the_reference_contract():
    """Shapes of sp_aurora/utils.py:116-122 and the split-KV == unsplit invariant."""
    B, H, S, D = 1, 4, 96, 64
    q, = rand_qkv((B, H, S, D), 61, torch.bfloat16, n=1)
    parts = [rand_qkv((B, H, n, D), 62 + i, torch.bfloat16, n=2) for i, n in enumerate((64, 40, 128))]
    out = lse = None
    for k, v in parts:
        b_out, b_lse = spa._flash_attn_forward(q.to(DEV), k.to(DEV), v.to(DEV))
        out, lse = spa.update_out_and_lse(out, lse, b_out, b_lse)
        assert out.shape == (B, S, H, D) and out.dtype == torch.float32
        assert lse.shape == (B, S, H, 1) and lse.dtype == torch.float32
    k_all = torch.cat([p[0] for p in parts], 2)
    v_all = torch.cat([p[1] for p in parts], 2)
    want_out, want_lse = O.attn_block(q, k_all, v_all)
    check_out(out.transpose(1, 2), want_out, torch.bfloat16)
    check_lse(lse.squeeze(-1).transpose(1, 2), want_lse)
    with pytest.raises(RuntimeError):
        spa.update_out_and_lse(None, None, b_out, b_lse, slice_=(slice(None),))
    # slice_ updates only the addressed rows
    before = out.clone()
    sl = (slice(None), slice(0, 32))
    b_out, b_lse = spa._flash_attn_forward(q[:, :, :32].to(DEV), parts[0][0].to(DEV), parts[0][1].to(DEV))
    out2, lse2 = spa.update_out_and_lse(out, lse, b_out, b_lse, slice_=sl)
    assert torch.equal(out2[:, 32:], before[:, 32:]) and not torch.equal(out2[:, :32], before[:, :32])


# ------------------------------------------------------------------ ring
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("P", [1, 2, 4])
def test_ring_equals_full_attention(P, causal, dtype):
    """test/test_ring_attention_full_accuracy.py:29-171 (B2, s128, H8, D64, gather and compare)."""
    B, s, H, D = 2, 128, 8, 64
    q, k, v = rand_qkv((B, P * s, H, D), 70, dtype)
    want_out, want_lse = O.full_attention(q, k, v, None, causal)
    out, lse, _ = spa.ring_flash_attn_func(q.to(DEV), k.to(DEV), v.to(DEV), causal=causal,
                                           return_attn_probs=True, ring_size=P)
    check_out(out, want_out, dtype)
    check_lse(lse, want_lse)
    only_out = spa.sp_aurora_func(q.to(DEV), k.to(DEV), v.to(DEV), causal=causal, ring_size=P)
    assert torch.equal(only_out, out)


def test_ring_rank_follows_the_oracle_schedule():
    """One rank's chunk against its KV chunks in ring order, as benchmark config 2 (scaled down)."""
    P, B, s, H, D, rank = 4, 2, 96, 4, 64, 2
    q, k, v = rand_qkv((B, P * s, H, D), 71, torch.bfloat16)
    ks, vs = list(k.chunk(P, 1)), list(v.chunk(P, 1))
    q_r = q[:, rank * s:(rank + 1) * s]
    for causal in (True, False):
        want_out, want_lse = O.ring_forward_rank(q_r, ks, vs, rank, None, causal, out_dtype=torch.float64)
        out, lse = spa.ring_flash_attn_forward_rank(q_r.to(DEV), [t.to(DEV) for t in ks], [t.to(DEV) for t in vs],
                                                    rank, None, causal)
        check_out(out, want_out, torch.bfloat16)
        check_lse(lse, want_lse)


def test_packed_equals_unpacked():
    """test/test_ring_attention_comprehensive.py:205-218."""
    B, S, H, D = 1, 256, 4, 64
    qkv = rand((B, S, 3, H, D), 72, torch.bfloat16).to(DEV)
    q, k, v = [qkv[:, :, i].contiguous() for i in range(3)]
    a = spa.ring_flash_attn_func(q, k, v, causal=True, ring_size=2)
    b = spa.ring_flash_attn_qkvpacked_func(qkv, causal=True, ring_size=2)
    c = spa.ring_flash_attn_kvpacked_func(q, qkv[:, :, 1:], causal=True, ring_size=2)
    assert torch.equal(a, b) and torch.equal(a, c)


# ------------------------------------------------------------------ re-layout
def _tagged(shape, dtype):
    n = int(np.prod(shape))
    if dtype in (torch.int16, torch.uint8):
        info = torch.iinfo(dtype)
        return (torch.arange(n, dtype=torch.int64) % (info.max + 1)).to(dtype).view(shape)
    return torch.arange(n, dtype=torch.int64).to(dtype).view(shape)


@pytest.mark.parametrize("dtype", [torch.uint8, torch.int16, torch.int32, torch.int64])
@pytest.mark.parametrize("P,B,s,H,D,pack", [(4, 1, 4, 8, 8, None), (2, 2, 3, 4, 16, None), (8, 1, 5, 16, 32, None),
                                            (4, 2, 4, 8, 8, 3), (2, 1, 6, 2, 64, 2), (3, 2, 2, 3, 5, None)])
def test_relayout_is_bit_exact(P, B, s, H, D, pack, dtype):
    """Tagged integers land where the reference's op chain puts them
    (archived_fallbacks/test_all_to_all_alternatives.py:126-161 uses tagged aranges the same way)."""
    shape = (P, B, s) + ((pack,) if pack else ()) + (H, D)
    x = _tagged(shape, dtype)
    if pack == 3:
        want = torch.stack(O.all_to_all_5d_s2h(list(x)))
    elif pack is None:
        want = torch.stack(O.all_to_all_4d_s2h(list(x)))
    else:
        want = O.relayout_s2h_formula(x)
    y = ops.relayout_s2h(x.to(DEV), P)
    assert y.shape == want.shape and torch.equal(y.cpu(), want)
    back = ops.relayout_h2s(y, P)
    assert torch.equal(back.cpu(), x)  # inverse o forward = identity
    if pack == 3:
        assert torch.equal(back.cpu(), torch.stack(O.all_to_all_5d_h2s(list(want))))
    elif pack is None:
        assert torch.equal(back.cpu(), torch.stack(O.all_to_all_4d_h2s(list(want))))


def test_relayout_api_names():
    P, B, s, H, D = 4, 2, 8, 8, 32
    x = rand((P, B, s, H, D), 80, torch.bfloat16).to(DEV)
    y = spa.intel_all_to_all_4d(x, 2, 1)
    assert y.shape == (P, B, P * s, H // P, D)   # test/ulysses/test_intel_alltoall_4d.py:93-100
    assert torch.equal(y.cpu(), O.relayout_s2h_formula(x.cpu()))
    assert torch.equal(spa.intel_all_to_all_4d(y, 1, 2), x)   # :140-147 and round trip
    assert torch.equal(spa.all_to_all_4D(x, 2, 1), y)
    x5 = rand((P, B, s, 3, H, D), 81, torch.bfloat16).to(DEV)
    y5 = spa.all_to_all_5D(x5, 3, 1)
    assert torch.equal(y5.cpu(), O.relayout_s2h_formula(x5.cpu()))
    assert torch.equal(spa.all_to_all_5D(y5, 1, 3), x5)
    assert spa.intel_all_to_all_4d(x[0]) is x[0] or torch.equal(spa.intel_all_to_all_4d(x[0]), x[0])  # world size 1
    with pytest.raises(ValueError):
        spa.intel_all_to_all_4d(x, 0, 3)
    # autograd: backward of the re-layout is the inverse re-layout
    xr = x.float().requires_grad_(True)
    yr = spa.SeqAllToAll4D.apply(None, xr, 2, 1)
    g = torch.randn_like(yr)
    yr.backward(g)
    assert torch.equal(xr.grad, ops.relayout_h2s(g, P))


# ------------------------------------------------------------------ Ulysses
@pytest.mark.parametrize("causal", [False, True])
def test_ulysses_equals_full_attention(causal):
    """test/verification/test_ulysses_fixed.py:165-344 (fp16, B2, s64, H4, D64) — here with strict bounds."""
    P, B, s, H, D = 4, 2, 64, 4, 64
    q, k, v = rand_qkv((B, P * s, H, D), 90, torch.float16)
    want_out, want_lse = O.full_attention(q, k, v, None, causal)
    stack = lambda t: torch.stack(t.chunk(P, 1)).contiguous().to(DEV)
    out = spa.ulysses_flash_attn_func(stack(q), stack(k), stack(v), causal=causal)
    assert out.shape == (P, B, s, H, D)
    check_out(torch.cat(list(out), 1), want_out, torch.float16)
    out2, lse = spa.intel_ulysses_flash_attn_forward(None, stack(q), stack(k), stack(v), D ** -0.5, causal=causal)
    assert torch.equal(out, out2) and lse.shape == (P, B, H // P, P * s)
    check_lse(torch.cat(list(lse), 1), want_lse)
    qkv = torch.stack([stack(q), stack(k), stack(v)], dim=3)
    assert torch.equal(spa.ulysses_flash_attn_qkvpacked_func(qkv, causal=causal), out)


@pytest.mark.parametrize("P,s,H,D,dtype,causal", [(4, 64, 8, 64, torch.float16, True), (2, 100, 4, 128, torch.bfloat16, True),
                                                  (8, 40, 8, 128, torch.bfloat16, False), (3, 130, 6, 32, torch.float16, True)])
def test_ulysses_through_views_equals_ulysses_through_relayout_kernels(P, s, H, D, dtype, causal):
    """B = 1: head group r read and written in place as a strided view, no re-layout pass, against the four
    re-layout passes around the same attention call (bit for bit) and against the oracle."""
    B = 1
    q, k, v = rand_qkv((B, P * s, H, D), 95, dtype)
    want_out, want_lse = O.full_attention(q, k, v, None, causal)
    stack = lambda t: torch.stack(t.chunk(P, 1)).contiguous().to(DEV)
    xq, xk, xv = stack(q), stack(k), stack(v)
    out_v, lse_v = spa.intel_ulysses_flash_attn_forward(None, xq, xk, xv, D ** -0.5, causal=causal, relayout="views")
    out_k, lse_k = spa.intel_ulysses_flash_attn_forward(None, xq, xk, xv, D ** -0.5, causal=causal, relayout="kernels")
    assert torch.equal(out_v, out_k) and torch.equal(lse_v, lse_k)
    check_out(torch.cat(list(out_v), 1), want_out, dtype)
    check_lse(torch.cat(list(lse_v), 1), want_lse)
    out_a, _ = spa.intel_ulysses_flash_attn_forward(None, xq, xk, xv, D ** -0.5, causal=causal)
    assert torch.equal(out_a, out_v)
    with pytest.raises(ValueError):
        spa.intel_ulysses_flash_attn_forward(None, torch.cat([xq, xq], 1), torch.cat([xk, xk], 1), torch.cat([xv, xv], 1),
                                             D ** -0.5, causal=causal, relayout="views")


@pytest.mark.parametrize("P,B,s,H,D,dtype,causal", [(4, 1, 64, 8, 64, torch.bfloat16, True), (2, 1, 100, 4, 128, torch.float16, False),
                                                    (4, 2, 48, 4, 64, torch.bfloat16, True)])
def test_ulysses_gradients(P, B, s, H, D, dtype, causal):
    """Backward of the Ulysses function on rank-stacked tensors against the oracle's autograd through full
    attention: B = 1 runs on strided views of the stacked tensors, B = 2 through the re-layout passes."""
    q, k, v, dout = rand_qkv((B, P * s, H, D), 97, dtype, n=4)
    want = O.attn_backward_autograd(q, k, v, dout, None, causal)
    stack = lambda t: torch.stack(t.chunk(P, 1)).contiguous().to(DEV)
    xs = [stack(t).requires_grad_(True) for t in (q, k, v)]
    out = spa.ulysses_flash_attn_func(*xs, causal=causal)
    out.backward(stack(dout))
    for x, w, name in zip(xs, want, "qkv"):
        assert x.grad.shape == (P, B, s, H, D) and x.grad.dtype == dtype
        check_grad(torch.cat(list(x.grad), 1), w, dtype, "d" + name)


# ------------------------------------------------------------------ backward
GRAD_TOL = {torch.bfloat16: dict(atol=3e-2, rtol=3e-2), torch.float16: dict(atol=4e-3, rtol=1e-2),
            torch.float32: dict(atol=2e-5, rtol=1e-4)}


def check_grad(got, want, dtype, what):
    got = got.detach().cpu().double()
    tol = GRAD_TOL[dtype]
    assert torch.isfinite(got).all(), f"{what}: {int((~torch.isfinite(got)).sum())} non-finite values"
    bad = (got - want).abs() > tol["atol"] * want.abs().max() + tol["rtol"] * want.abs()
    assert not bad.any(), f"{what}: {int(bad.sum())} out of tolerance, max abs err {(got - want).abs().max():.3e} (scale {want.abs().max():.3e})"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("B,S,H,D,causal,P", [(1, 128, 2, 64, False, 1), (2, 256, 3, 128, True, 1), (1, 256, 2, 32, True, 4),
                                              (1, 192, 2, 128, False, 3), (1, 200, 2, 64, True, 1), (1, 77, 1, 128, False, 1),
                                              (1, 512, 2, 128, True, 4)])
def test_backward_matches_autograd_of_full_attention(B, S, H, D, causal, P, dtype):
    """Gradients against the oracle's autograd through full attention, relative to each gradient's scale."""
    q, k, v, dout = rand_qkv((B, S, H, D), 100, dtype, n=4)
    want = O.attn_backward_autograd(q, k, v, dout, None, causal)
    dq_, dk_, dv_ = [t.to(DEV).requires_grad_(True) for t in (q, k, v)]
    out = spa.ring_flash_attn_func(dq_, dk_, dv_, causal=causal, ring_size=P)
    out.backward(dout.to(DEV))
    for got, w, name in zip((dq_.grad, dk_.grad, dv_.grad), want, "qkv"):
        assert got.dtype == dtype
        check_grad(got, w, dtype, "d" + name)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("B,Sq,Sk,H,D,causal", [(1, 300, 300, 2, 128, True), (2, 130, 257, 3, 64, False), (1, 64, 64, 1, 32, True),
                                                (1, 1000, 1000, 2, 128, True),
                                                # causal with keys that no query sees: whole tiles of zeros
                                                (1, 100, 400, 2, 64, True), (2, 130, 300, 1, 128, True)])
def test_backward_written_in_the_inputs_type_equals_accumulate_then_cast(B, Sq, Sk, H, D, causal, dtype):
    """spa_flash_bwd_out against spa_flash_bwd into zeroed fp32 accumulators followed by the cast
    (sp_aurora/intel_ring_flash_attn.py:250-271): bit for bit, also through strided gradient views."""
    g = torch.Generator().manual_seed(160)
    q, dout = [(torch.randn(B, Sq, H, D, generator=g) * 0.5).to(dtype).to(DEV) for _ in range(2)]
    k, v = [(torch.randn(B, Sk, H, D, generator=g) * 0.5).to(dtype).to(DEV) for _ in range(2)]
    out, lse = ops.flash_fwd(q, k, v, None, causal, layout="bshd")
    delta = ops.bwd_delta(out, dout, layout="bshd")
    acc = [torch.zeros(t.shape, dtype=torch.float32, device=DEV) for t in (q, k, v)]
    ops.flash_bwd(q, k, v, dout, lse, delta, *acc, None, causal, layout="bshd")
    want = [a.to(dtype) for a in acc]
    got = ops.flash_bwd_out(q, k, v, dout, lse, delta, None, causal, layout="bshd")
    for gt, w, name in zip(got, want, "qkv"):
        assert gt.dtype == dtype and torch.equal(gt, w), f"d{name}"
    # gradients written into the halves of packed buffers (row stride 2 H D)
    pq = torch.full((B, Sq, 2, H, D), 7.0, dtype=dtype, device=DEV)
    pkv = torch.full((B, Sk, 2, H, D), 7.0, dtype=dtype, device=DEV)
    ops.flash_bwd_out(q, k, v, dout, lse, delta, None, causal, layout="bshd", dq=pq[:, :, 1], dk=pkv[:, :, 0], dv=pkv[:, :, 1])
    assert torch.equal(pq[:, :, 1], want[0]) and torch.equal(pkv[:, :, 0], want[1]) and torch.equal(pkv[:, :, 1], want[2])
    assert (pq[:, :, 0] == 7.0).all()
    with pytest.raises(ValueError):
        ops.flash_bwd_out(q, k, v, dout, lse, delta, None, causal, layout="bshd", dq=torch.empty_like(k[:, :1]))
    with pytest.raises(ValueError):
        ops.flash_bwd_out(q, k, v, dout, lse, delta, None, causal, layout="bshd", dk=torch.empty(k.shape, dtype=torch.float64, device=DEV))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("Sq,Sk,causal", [(96, 100, False), (130, 70, False), (100, 100, True)])
def test_backward_with_strongly_negative_scores_and_ragged_keys(Sq, Sk, causal, dtype):
    """Scores near -128, so lse < -88 and exp(-lse) overflows fp32: the keys past the end of a
    ragged last tile (zero rows in LDS, score 0) must be masked, not multiplied by zero."""
    B, H, D = 1, 2, 64
    g = torch.Generator().manual_seed(150)
    noise = lambda shape: torch.randn(shape, generator=g) * 0.05
    q = (4.0 + noise((B, Sq, H, D))).to(dtype)
    k = (-4.0 + noise((B, Sk, H, D))).to(dtype)
    v = torch.randn((B, Sk, H, D), generator=g).to(dtype)
    dout = torch.randn((B, Sq, H, D), generator=g).to(dtype)
    want_out, want_lse = O.full_attention(q, k, v, None, causal)
    assert want_lse.max() < -100
    qd, kd, vd, dd = (t.to(DEV) for t in (q, k, v, dout))
    out, lse = ops.flash_fwd(qd, kd, vd, None, causal, layout="bshd")
    check_out(out, want_out, dtype)
    check_lse(lse, want_lse)
    delta = ops.bwd_delta(out, dd, layout="bshd")
    # Expected gradients: the block formula in fp64 with the delta of the ROUNDED out the kernels
    # see.  (K carries a constant offset here, which multiplies the rounding of out in
    # sum_j dS_ij = dO.O_exact - delta by 4 in dq: against autograd of exact attention the
    # comparison would measure that conditioning, not the kernel.)
    tr = lambda t: t.transpose(1, 2)
    want_delta = (out.cpu().double() * dout.double()).sum(-1).transpose(1, 2)
    assert torch.allclose(delta.cpu().double(), want_delta, rtol=1e-4, atol=1e-5)
    want = [tr(g) for g in O.attn_backward_block(tr(q), tr(k), tr(v), tr(dout), want_lse, want_delta, None, causal)]
    dq = torch.zeros((B, Sq, H, D), dtype=torch.float32, device=DEV)
    dk = torch.zeros((B, Sk, H, D), dtype=torch.float32, device=DEV)
    dv = torch.zeros((B, Sk, H, D), dtype=torch.float32, device=DEV)
    ops.flash_bwd(qd, kd, vd, dd, lse, delta, dq, dk, dv, None, causal, layout="bshd")
    # K (and Q) carry an offset 80 times their spread, so the element-wise errors of P and dS do not
    # cancel the way the exact terms do in sum_j dS_ij K_j; the bound is that error itself:
    # |err dq| <= eps * scale * |dS| |K|, likewise dk with |Q| and dv = P^T dO with |dO|, where eps is
    # the relative error of one element of P / dS: 2^-8 for 16-bit types (they enter the gradient
    # MFMAs rounded to the input type), 3e-4 for fp32 (scores near -128 summed from 64 fp32
    # products of size 16 carry ~1e-4 of absolute error, which exp() turns into relative error).
    eps = 3e-4 if dtype == torch.float32 else 2.0 ** -8
    qt, kt, vt, dot = (tr(t).double() for t in (q, k, v, dout))
    sc = D ** -0.5
    sm = torch.matmul(qt, kt.transpose(-2, -1)) * sc
    if causal:
        sm = sm.masked_fill(O.causal_mask(Sq, Sk), float("-inf"))
    pm = torch.exp(sm - want_lse.unsqueeze(-1))
    dsm = (pm * (torch.matmul(dot, vt.transpose(-2, -1)) - want_delta.unsqueeze(-1))).abs()
    bounds = [tr(torch.matmul(dsm, kt.abs()) * sc), tr(torch.matmul(dsm.transpose(-2, -1), qt.abs()) * sc),
              tr(torch.matmul(pm.transpose(-2, -1), dot.abs()))]
    for got, w, bound, name in zip((dq, dk, dv), want, bounds, "qkv"):
        got = got.cpu().double()
        assert torch.isfinite(got).all(), f"d{name}: non-finite values"
        bad = (got - w).abs() > eps * bound + 1e-6
        assert not bad.any(), f"d{name}: {int(bad.sum())} beyond the rounding bound, max abs err {(got - w).abs().max():.3e}"


@pytest.mark.parametrize("causal", [False, True])
def test_ring_backward_schedules_agree(causal):
    """One launch per visited block pair (the reference's schedule, intel_ring_flash_attn.py:192-271)
    and the single pass over the same pairs give the same gradients, both equal to the oracle's."""
    B, S, H, D, P = 1, 384, 2, 128, 3
    q, k, v, dout = rand_qkv((B, S, H, D), 105, torch.bfloat16, n=4)
    want = O.attn_backward_autograd(q, k, v, dout, None, causal)
    qd, kd, vd, dd = (t.to(DEV) for t in (q, k, v, dout))
    out, lse = spa.ring.ring_flash_attn_forward(qd, kd, vd, None, causal, P)
    res = {f: spa.ring.ring_flash_attn_backward(dd, qd, kd, vd, out, lse, None, causal, P, fuse=f) for f in ("step", "all")}
    for f, grads in res.items():
        for got, w, name in zip(grads, want, "qkv"):
            check_grad(got, w, torch.bfloat16, f"{f} d{name}")
    with pytest.raises(ValueError):
        spa.ring.ring_flash_attn_backward(dd, qd, kd, vd, out, lse, None, causal, P, fuse="rank")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,S,H,D,causal", [(1, 300, 2, 128, True), (2, 515, 2, 64, True), (1, 256, 3, 32, False),
                                            (1, 1000, 2, 128, False), (1, 77, 1, 128, True)])
def test_dq_kernel_workgroup_sizes_agree(B, S, H, D, causal, dtype):
    """The dq kernel runs 128-row or 256-row workgroups depending on the grid; both orders of
    accumulation are the same per row, so the gradients must be identical, and right."""
    q, k, v, dout = rand_qkv((B, S, H, D), 140, dtype, n=4)
    want = O.attn_backward_autograd(q, k, v, dout, None, causal)
    got = {}
    try:
        for waves in (4, 8):
            _lib.tune("bwd_dq_waves", waves)
            xs = [t.to(DEV).requires_grad_(True) for t in (q, k, v)]
            spa.ring_flash_attn_func(*xs, causal=causal).backward(dout.to(DEV))
            got[waves] = [x.grad for x in xs]
            for g, w, name in zip(got[waves], want, "qkv"):
                check_grad(g, w, dtype, f"d{name} with {waves} waves")
    finally:
        _lib.tune("bwd_dq_waves", 0)
    for a, b in zip(got[4], got[8]):
        assert torch.equal(a, b)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,S,H,D,causal", [(1, 300, 2, 128, True), (2, 515, 2, 128, False), (1, 1000, 2, 128, True),
                                            (1, 77, 1, 128, True), (1, 2048, 1, 128, True)])
def test_dkdv_kernel_hand_issued_and_compiler_scheduled_forms_agree(B, S, H, D, causal, dtype):
    """The D = 128 dk/dv kernel issues its MFMAs from inline assembly with the MFMA -> VALU hazard
    distances kept by the order of the loop; its twin leaves every MFMA (and every hazard) to the
    compiler.  Same operations in the same order on the same values: the gradients must be
    bit-identical, and right."""
    q, k, v, dout = rand_qkv((B, S, H, D), 141, dtype, n=4)
    want = O.attn_backward_autograd(q, k, v, dout, None, causal)
    got = {}
    try:
        for form in (0, 1):
            _lib.tune("bwd_dkdv_form", form)
            xs = [t.to(DEV).requires_grad_(True) for t in (q, k, v)]
            spa.ring_flash_attn_func(*xs, causal=causal).backward(dout.to(DEV))
            got[form] = [x.grad for x in xs]
            for g, w, name in zip(got[form], want, "qkv"):
                check_grad(g, w, dtype, f"d{name}, form {form}")
    finally:
        _lib.tune("bwd_dkdv_form", 0)
    for a, b in zip(got[0], got[1]):
        assert torch.equal(a, b)


def test_backward_packed_and_operator_entry():
    B, S, H, D = 1, 256, 2, 128
    qkv = rand((B, S, 3, H, D), 101, torch.bfloat16)
    dout = rand((B, S, H, D), 102, torch.bfloat16)
    want = O.attn_backward_autograd(qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2], dout, None, True)
    dqkv = qkv.to(DEV).requires_grad_(True)
    out, lse, _ = spa.ring_flash_attn_qkvpacked_func(dqkv, causal=True, return_attn_probs=True, ring_size=2)
    out.backward(dout.to(DEV))
    for i, name in enumerate("qkv"):
        check_grad(dqkv.grad[:, :, i], want[i], torch.bfloat16, "packed d" + name)
    # operator-level backward ([B,H,S,D], saved out and lse)
    t = lambda x: x.transpose(1, 2).contiguous().to(DEV)
    q, k, v = t(qkv[:, :, 0]), t(qkv[:, :, 1]), t(qkv[:, :, 2])
    o, l = spa._flash_attn_forward(q, k, v, causal=True)
    dq, dk, dv = spa._flash_attn_backward(t(dout), q, k, v, o, l, causal=True)
    for got, w, name in zip((dq, dk, dv), want, "qkv"):
        check_grad(got.transpose(1, 2), w, torch.bfloat16, "operator d" + name)
    # gradients written into tensors the caller passes: as they are when the kernels can write them
    # (here dq, and dk as one half of a packed buffer), through a copy when not (dv is fp32)
    gq = torch.full_like(q, 7.0)
    gkv = torch.full((B, H, S, 2, D), 7.0, dtype=q.dtype, device=DEV)
    gv = torch.full(v.shape, 7.0, dtype=torch.float32, device=DEV)
    r = spa._flash_attn_backward(t(dout), q, k, v, o, l, dq=gq, dk=gkv[:, :, :, 0], dv=gv, causal=True)
    assert r[0] is gq and r[2] is gv and r[1].data_ptr() == gkv.data_ptr()
    assert torch.equal(gq, dq) and torch.equal(gkv[:, :, :, 0], dk) and torch.equal(gv, dv.float())
    assert (gkv[:, :, :, 1] == 7.0).all()


def test_delta_kernel():
    o, do = rand_qkv((2, 40, 3, 64), 103, torch.bfloat16, n=2)
    got = ops.bwd_delta(o.to(DEV), do.to(DEV))
    want = (o.double() * do.double()).sum(-1).transpose(1, 2)
    assert torch.allclose(got.cpu().double(), want, atol=1e-4, rtol=1e-5)


# ------------------------------------------------------------------ C ring driver
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("causal", [False, True])
def test_ring_driver_matches_stepwise_path_and_oracle(causal, dtype):
    """spa_ring_fwd (merge fused into the kernel epilogue) against the step-by-step path through
    spa_flash_fwd + spa_merge + spa_finalize, and against the oracle's ring schedule; also a single
    rank, as benchmark config 2 runs it."""
    P, B, s, H, D = 4, 2, 160, 3, 64
    q, k, v = rand_qkv((B, P * s, H, D), 110, dtype)
    dq, dk, dv = q.to(DEV), k.to(DEV), v.to(DEV)
    out, lse = ops.ring_fwd(dq, dk, dv, P, None, causal, fuse="step")
    want_out, want_lse = O.ring_forward(q, k, v, P, None, causal, out_dtype=torch.float64)
    check_out(out, want_out, dtype)
    check_lse(lse, want_lse)
    for fuse in ("rank", "all"):  # one launch per rank / one launch in all: same schedule, merged in registers
        o_f, l_f = ops.ring_fwd(dq, dk, dv, P, None, causal, fuse=fuse)
        check_out(o_f, want_out, dtype, what=f"out[{fuse}]")
        check_lse(l_f, want_lse)
    ks, vs = list(dk.split(s, 1)), list(dv.split(s, 1))
    for r in range(P):
        o_r, l_r = spa.ring_flash_attn_forward_rank(dq[:, r * s:(r + 1) * s], ks, vs, r, None, causal)
        tol = dict(atol=1e-6, rtol=1e-6) if dtype == torch.float32 else dict(atol=8e-3, rtol=8e-3)
        assert torch.allclose(out[:, r * s:(r + 1) * s].float(), o_r.float(), **tol)
        assert torch.allclose(lse[:, :, r * s:(r + 1) * s], l_r, atol=1e-5)
    # one rank only: the other rows stay untouched
    out2 = torch.full_like(out, 7.0)
    lse2 = torch.full_like(lse, 7.0)
    ops.ring_fwd(dq, dk, dv, P, None, causal, rank=2, out=out2, lse=lse2, fuse="step")
    assert torch.equal(out2[:, 2 * s:3 * s], out[:, 2 * s:3 * s]) and torch.equal(lse2[:, :, 2 * s:3 * s], lse[:, :, 2 * s:3 * s])
    assert (out2[:, :2 * s] == 7).all() and (out2[:, 3 * s:] == 7).all() and (lse2[:, :, :2 * s] == 7).all()


@pytest.mark.parametrize("fuse", ["step", "rank", "all"])
@pytest.mark.parametrize("P,B,s,H,D,causal", [(8, 1, 128, 2, 128, True), (3, 2, 200, 2, 64, True), (4, 1, 72, 3, 32, False),
                                              (2, 1, 1024, 2, 128, True), (5, 1, 64, 1, 128, True),
                                              (16, 1, 40, 2, 64, False), (12, 2, 136, 1, 128, True)])
def test_ring_driver_modes_on_awkward_shapes(P, B, s, H, D, causal, fuse):
    """Chunk lengths that are not multiples of the key tile, odd ring sizes, many ranks (in the per-step
    schedule a rank's last step then merges up to 15 earlier results)."""
    q, k, v = rand_qkv((B, P * s, H, D), 111, torch.bfloat16)
    want_out, want_lse = O.full_attention(q, k, v, None, causal)
    out, lse = ops.ring_fwd(q.to(DEV), k.to(DEV), v.to(DEV), P, None, causal, fuse=fuse)
    check_out(out, want_out, torch.bfloat16)
    check_lse(lse, want_lse)


@pytest.fixture
def shared_buffer_variant():
    """Forces the 256-row forward variant whose wave groups share the K/V buffers (it is otherwise
    chosen only for grids that fill the GPU twice over)."""
    _lib.tune("fwd_share", 2)
    yield
    _lib.tune("fwd_share", 0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,H,Sq,Sk,D,causal", [(1, 2, 256, 256, 128, True), (2, 3, 300, 300, 64, True), (1, 2, 130, 515, 128, False),
                                                (1, 1, 77, 200, 64, True), (1, 2, 512, 129, 128, True), (1, 1, 1, 65, 128, False)])
def test_shared_buffer_variant_block_forward(shared_buffer_variant, B, H, Sq, Sk, D, causal, dtype):
    q = rand((B, H, Sq, D), 120, dtype)
    k = rand((B, H, Sk, D), 121, dtype)
    v = rand((B, H, Sk, D), 122, dtype)
    want_out, want_lse = O.attn_block(q, k, v, None, causal)
    out, lse = ops.flash_fwd(q.to(DEV), k.to(DEV), v.to(DEV), None, causal, layout="bhsd")
    check_out(out, want_out, dtype)
    check_lse(lse, want_lse)


@pytest.mark.parametrize("fuse", ["step", "rank", "all"])
@pytest.mark.parametrize("P,B,s,H,D,causal", [(3, 2, 200, 2, 64, True), (2, 1, 1024, 2, 128, True), (5, 1, 64, 1, 128, True),
                                              (4, 1, 320, 2, 128, False)])
def test_shared_buffer_variant_ring(shared_buffer_variant, P, B, s, H, D, causal, fuse):
    q, k, v = rand_qkv((B, P * s, H, D), 123, torch.bfloat16)
    want_out, want_lse = O.full_attention(q, k, v, None, causal)
    out, lse = ops.ring_fwd(q.to(DEV), k.to(DEV), v.to(DEV), P, None, causal, fuse=fuse)
    check_out(out, want_out, torch.bfloat16)
    check_lse(lse, want_lse)


@pytest.mark.parametrize("fuse", ["step", "all"])
def test_ring_forward_replays_from_a_captured_graph(fuse):
    """The library allocates nothing and never synchronises, so a ring forward can be captured in a
    graph; every replay (with eager work and synchronisations in between) must equal the eager result."""
    B, S, H, D, P = 1, 1024, 4, 128, 4
    q, k, v = (t.to(DEV) for t in rand_qkv((B, S, H, D), 130, torch.bfloat16))
    step = spa.ring.make_ring_forward_step(q, k, v, None, True, P, fuse=fuse)
    eager_out, eager_lse = (t.clone() for t in step())
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()  # warm up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out, lse = step()
    for rep in range(3):
        out.fill_(7)
        lse.fill_(7)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager_out) and torch.equal(lse, eager_lse), f"replay {rep} differs"
        # eager work between replays, with new inputs of the same shape in the captured buffers
        q.mul_(-1)
        k.mul_(-1)
        torch.cuda.synchronize()
        q.mul_(-1)
        k.mul_(-1)


def test_prepared_calls_replay_the_recorded_sequence():
    """ops.prepared records the C calls of a composition once; a replay must do what the direct
    calls do, on the same buffers, as often as asked."""
    B, S, H, D, P = 1, 256, 2, 64, 2
    q, k, v = [t.to(DEV) for t in rand_qkv((B, S, H, D), 160, torch.bfloat16)]
    want_out, want_lse = ops.ring_fwd(q, k, v, P, None, True, fuse="step")
    out = torch.zeros_like(q)
    lse = torch.zeros((B, H, S), dtype=torch.float32, device=DEV)
    ws = ops.ring_fwd_workspace(q, P)
    run, (o2, l2) = ops.prepared(ops.ring_fwd, q, k, v, P, None, True, out=out, lse=lse, workspace=ws, fuse="step")
    assert o2 is out and l2 is lse
    assert torch.count_nonzero(out) == 0  # recording launches nothing
    for _ in range(3):
        out.zero_()
        lse.zero_()
        run()
        assert torch.equal(out, want_out) and torch.equal(lse, want_lse)
    # a composition: re-layout there and back
    x = rand((2, 1, 64, 4, 32), 161, torch.bfloat16).to(DEV)
    y = torch.empty((2, 1, 128, 2, 32), dtype=x.dtype, device=DEV)
    back = torch.empty_like(x)
    run, _ = ops.prepared(lambda: (ops.relayout_s2h(x, 2, out=y), ops.relayout_h2s(y, 2, out=back)))
    run()
    assert torch.equal(back, x) and torch.equal(y, ops.relayout_s2h(x, 2))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("scale", [-0.25, 0.0, -1.0 / 8])
@pytest.mark.parametrize("causal", [False, True])
def test_any_finite_softmax_scale_forward_and_backward(scale, causal, dtype):
    """The reference takes whatever softmax_scale it is given (sp_aurora/intel_flash_attn.py:46-47,
    a plain multiplication); so does the HIP path: negative scales, and zero (uniform attention
    over the visible keys, lse = log of their number, zero gradients for q and k)."""
    B, S, H, D, P = 1, 200, 2, 64, 1
    q, k, v, dout = rand_qkv((B, S, H, D), 170, dtype, n=4)
    want_out, want_lse = O.full_attention(q, k, v, scale, causal)
    want = O.attn_backward_autograd(q, k, v, dout, scale, causal)
    xs = [t.to(DEV).requires_grad_(True) for t in (q, k, v)]
    out, lse, _ = spa.ring_flash_attn_func(*xs, softmax_scale=scale, causal=causal, return_attn_probs=True)
    check_out(out, want_out, dtype)
    check_lse(lse, want_lse)
    out.backward(dout.to(DEV))
    for x, w, name in zip(xs, want, "qkv"):
        if w.abs().max() == 0:
            assert x.grad.abs().max() < 1e-20, f"d{name} should vanish"
        else:
            check_grad(x.grad, w, dtype, "d" + name)
    # the ring schedules take the same scale
    P = 4
    for fuse in ("step", "rank", "all"):
        o2, l2 = spa.ring.ring_flash_attn_forward(q.to(DEV), k.to(DEV), v.to(DEV), scale, causal, P, fuse=fuse)
        check_out(o2, want_out, dtype)
        check_lse(l2, want_lse)
