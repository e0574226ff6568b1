"""GPU parity of the block forward with e4m3 K / V (spa_flash_fwd_fp8kv, spa_flash_fwd_varlen_fp8kv).

The reference has no 8-bit path and therefore no output to compare with: parity is pinned by the
mathematics.  Expected = the oracle's block attention in fp64 on q and on the DEQUANTISED tensors
K = k8 * k_scale[b,h], V = v8 * v_scale[b,h] (every e4m3 value is exact in fp64), to the same
tolerances as the 16-bit kernels: out atol 2e-2 / rtol 1.6e-2 (bf16), lse atol 1e-3.
"""
import pytest
import torch

from conftest import rand
from oracle import attn_oracle as O
import sp_aurora_amd as spa
from sp_aurora_amd import _lib, ops
from test_gpu_parity import DEV, check_lse, check_out
from test_gpu_varlen import cu_of, per_sequence

pytestmark = pytest.mark.gpu


def quantised(shape, seed, layout, spread=1.0):
    """A random tensor, its e4m3 quantisation with per-(batch, head) scales, and the dequantised values."""
    x = rand(shape, seed, torch.float32) * spread
    x8, sc = ops.quantize_fp8_per_head(x, layout)
    bc = sc[:, None, :, None] if layout == "bshd" else sc[:, :, None, None]
    return x8, sc, x8.double() * bc.double()


def test_e4m3_round_trip_of_the_quantiser():
    x8, sc, deq = quantised((2, 40, 3, 64), 500, "bshd", spread=5.0)
    x = rand((2, 40, 3, 64), 500, torch.float32) * 5.0
    # e4m3 keeps 3 mantissa bits: relative error <= 2^-4 for normal values, absolute 2^-10 * scale below
    assert ((deq - x.double()).abs() <= 2.0 ** -4 * x.double().abs() + 2.0 ** -9 * sc.double().max()).all()
    assert (x8.float().abs() <= 448).all()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,H,Sq,Sk,D,causal", [
    (2, 32, 1024, 1024, 64, True),      # one block pair of benchmark config 2 (diagonal)
    (1, 32, 1024, 1024, 128, False),    # one block pair of benchmark config 3 (full)
    (1, 4, 1024, 1024, 128, True),      # config 3, diagonal
    (1, 2, 130, 515, 128, False), (2, 3, 300, 300, 64, True), (1, 1, 77, 200, 64, True),
    (1, 2, 512, 129, 128, True), (1, 1, 1, 65, 128, False), (1, 2, 50, 40, 64, False), (1, 1, 200, 1, 128, False),
])
def test_block_forward_with_e4m3_kv(B, H, Sq, Sk, D, causal, dtype):
    q = rand((B, H, Sq, D), 510, dtype)
    k8, ksc, k_deq = quantised((B, H, Sk, D), 511, "bhsd", spread=1.5)
    v8, vsc, v_deq = quantised((B, H, Sk, D), 512, "bhsd", spread=0.7)
    want_out, want_lse = O.attn_block(q, k_deq, v_deq, None, causal)
    out, lse = ops.flash_fwd(q.to(DEV), k8.to(DEV), v8.to(DEV), None, causal, layout="bhsd", k_scale=ksc, v_scale=vsc)
    assert out.dtype == dtype and lse.dtype == torch.float32
    check_out(out, want_out, dtype)
    check_lse(lse, want_lse)
    # the operator shim takes the same quadruple
    out2, lse2 = spa.intel_flash_attn_forward(q.to(DEV), k8.to(DEV), v8.to(DEV), causal=causal, k_scale=ksc, v_scale=vsc)
    assert torch.equal(out, out2) and torch.equal(lse, lse2)


def test_e4m3_kv_in_the_public_layout_and_strided():
    """[B,S,H,D] tensors and the strided views of a packed kv cache reach the kernel without copies."""
    B, S, H, D = 1, 384, 4, 128
    q = rand((B, S, H, D), 520, torch.bfloat16)
    kv = rand((B, S, 2, H, D), 521, torch.float32)
    k8, ksc = ops.quantize_fp8_per_head(kv[:, :, 0], "bshd")
    v8, vsc = ops.quantize_fp8_per_head(kv[:, :, 1], "bshd")
    kv8 = torch.stack([k8.view(torch.uint8), v8.view(torch.uint8)], dim=2).to(DEV).view(torch.float8_e4m3fn)
    k_deq = k8.double() * ksc[:, None, :, None].double()
    v_deq = v8.double() * vsc[:, None, :, None].double()
    want_out, want_lse = O.full_attention(q, k_deq, v_deq, None, True)
    out, lse = ops.flash_fwd(q.to(DEV), kv8[:, :, 0], kv8[:, :, 1], None, True, layout="bshd", k_scale=ksc, v_scale=vsc)
    check_out(out, want_out, torch.bfloat16)
    check_lse(lse, want_lse)


@pytest.mark.parametrize("groups", [1, 2])
def test_e4m3_kv_with_one_and_two_wave_groups(groups):
    from sp_aurora_amd import _lib
    B, H, Sq, Sk, D = 1, 2, 256, 320, 128
    q = rand((B, H, Sq, D), 530, torch.bfloat16)
    k8, ksc, k_deq = quantised((B, H, Sk, D), 531, "bhsd")
    v8, vsc, v_deq = quantised((B, H, Sk, D), 532, "bhsd")
    want_out, want_lse = O.attn_block(q, k_deq, v_deq, None, True)
    try:
        _lib.tune("fwd_groups", groups)
        out, lse = ops.flash_fwd(q.to(DEV), k8.to(DEV), v8.to(DEV), None, True, layout="bhsd", k_scale=ksc, v_scale=vsc)
    finally:
        _lib.tune("fwd_groups", 0)
    check_out(out, want_out, torch.bfloat16)
    check_lse(lse, want_lse)


@pytest.mark.parametrize("B,H,Sq,Sk,D,causal,dtype", [(1, 2, 512, 512, 128, True, torch.bfloat16),
                                                      (2, 3, 300, 333, 128, False, torch.bfloat16),
                                                      (1, 2, 256, 130, 128, True, torch.float16),
                                                      (1, 4, 640, 640, 64, True, torch.bfloat16),
                                                      (1, 2, 77, 1000, 64, False, torch.float16)])
def test_e4m3_kv_with_shared_buffers(B, H, Sq, Sk, D, causal, dtype):
    """The 256-row workgroups whose two wave groups stage one set of K/V tiles together (large launches pick
    them; here forced), against the oracle, and within rounding of the 128-row form (which sums the keys in
    another order)."""
    from sp_aurora_amd import _lib
    q = rand((B, H, Sq, D), 560, dtype)
    k8, ksc, k_deq = quantised((B, H, Sk, D), 561, "bhsd")
    v8, vsc, v_deq = quantised((B, H, Sk, D), 562, "bhsd")
    want_out, want_lse = O.attn_block(q, k_deq, v_deq, None, causal)
    got = {}
    try:
        for share in (2, 1):
            _lib.tune("fwd_share", share)
            got[share] = ops.flash_fwd(q.to(DEV), k8.to(DEV), v8.to(DEV), None, causal, layout="bhsd", k_scale=ksc, v_scale=vsc)
    finally:
        _lib.tune("fwd_share", 0)
    check_out(got[2][0], want_out, dtype)
    check_lse(got[2][1], want_lse)
    check_out(got[2][0], got[1][0].double().cpu(), dtype)
    check_lse(got[2][1], got[1][1].double().cpu())


def test_ring_all_ranks_with_e4m3_kv_and_shared_buffers():
    """One launch for every rank of a causal ring (the schedule the shared-buffer form serves), forced onto it."""
    from sp_aurora_amd import _lib
    B, S, H, D, P = 1, 1024, 2, 128, 4
    q = rand((B, S, H, D), 570, torch.bfloat16)
    k8, ksc, k_deq = quantised((B, S, H, D), 571, "bshd")
    v8, vsc, v_deq = quantised((B, S, H, D), 572, "bshd")
    want_out, want_lse = O.full_attention(q, k_deq, v_deq, None, True)
    try:
        _lib.tune("fwd_share", 2)
        out, lse = ops.ring_fwd(q.to(DEV), k8.to(DEV), v8.to(DEV), ring_size=P, causal=True, rank=-1, fuse="all", k_scale=ksc, v_scale=vsc)
    finally:
        _lib.tune("fwd_share", 0)
    check_out(out, want_out, torch.bfloat16)
    check_lse(lse, want_lse)


@pytest.mark.parametrize("lengths,H,D,causal", [([128, 256, 128], 8, 64, True), ([1, 77, 300, 5, 129], 3, 128, False),
                                                ([1, 77, 300, 5, 129], 3, 128, True)])
def test_varlen_forward_with_e4m3_kv(lengths, H, D, causal):
    T, n = sum(lengths), len(lengths)
    q = rand((T, H, D), 540, torch.bfloat16)
    k = rand((T, H, D), 541, torch.float32) * 1.3
    v = rand((T, H, D), 542, torch.float32)
    # one scale per (sequence, head)
    k8 = torch.empty((T, H, D), dtype=torch.float8_e4m3fn)
    v8 = torch.empty((T, H, D), dtype=torch.float8_e4m3fn)
    ksc = torch.empty((n, H))
    vsc = torch.empty((n, H))
    k_deq = torch.empty((T, H, D), dtype=torch.float64)
    v_deq = torch.empty((T, H, D), dtype=torch.float64)
    r0 = 0
    for i, ln in enumerate(lengths):
        for src, dst8, sc, deq in ((k, k8, ksc, k_deq), (v, v8, vsc, v_deq)):
            x8, s1 = ops.quantize_fp8_per_head(src[None, r0:r0 + ln], "bshd")
            dst8[r0:r0 + ln] = x8[0]
            sc[i] = s1[0]
            deq[r0:r0 + ln] = x8[0].double() * s1[0][None, :, None].double()
        r0 += ln
    want_out, want_lse = per_sequence(q, k_deq, v_deq, lengths, lengths, causal)
    cu = cu_of(lengths).to(DEV)
    out, lse = ops.flash_fwd_varlen(q.to(DEV), k8.to(DEV), v8.to(DEV), cu, cu, max(lengths), max(lengths), None, causal,
                                    k_scale=ksc, v_scale=vsc)
    check_out(out, want_out, torch.bfloat16)
    check_lse(lse, want_lse)


@pytest.mark.parametrize("fuse", ["step", "rank", "all"])
@pytest.mark.parametrize("B,S,H,D,P,causal", [(1, 512, 2, 128, 4, True), (2, 384, 3, 64, 3, False), (1, 1024, 4, 128, 8, True)])
def test_ring_forward_with_e4m3_kv(B, S, H, D, P, causal, fuse):
    """The three ring schedules over e4m3 K / V (one scale per (batch, head) for the whole sequence)
    against full attention on the dequantised tensors."""
    q = rand((B, S, H, D), 560, torch.bfloat16)
    k8, ksc, k_deq = quantised((B, S, H, D), 561, "bshd", spread=1.2)
    v8, vsc, v_deq = quantised((B, S, H, D), 562, "bshd")
    want_out, want_lse = O.full_attention(q, k_deq, v_deq, None, causal)
    out, lse = ops.ring_fwd(q.to(DEV), k8.to(DEV), v8.to(DEV), P, None, causal, fuse=fuse, k_scale=ksc, v_scale=vsc)
    check_out(out, want_out, torch.bfloat16)
    check_lse(lse, want_lse)


def test_e4m3_kv_argument_checks():
    q = rand((1, 2, 64, 64), 550, torch.bfloat16).to(DEV)
    k8 = torch.zeros((1, 2, 64, 64), dtype=torch.float8_e4m3fn, device=DEV)
    sc = torch.ones((1, 2))
    with pytest.raises(ValueError, match="k_scale and v_scale"):
        ops.flash_fwd(q, k8, k8, layout="bhsd")
    with pytest.raises(ValueError, match="shape"):
        ops.flash_fwd(q, k8, k8, layout="bhsd", k_scale=torch.ones((2, 2)), v_scale=sc)
    with pytest.raises(TypeError):
        ops.flash_fwd(q, k8, q, layout="bhsd", k_scale=sc, v_scale=sc)
    with pytest.raises(spa._lib.SpaError):  # fp32 queries have no e4m3 K/V kernel
        ops.flash_fwd(q.float(), k8, k8, layout="bhsd", k_scale=sc, v_scale=sc)


# ------------------------------------------------------------------ e4m3 q as well: scores on the 8-bit matrix instruction
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,H,Sq,Sk,causal", [
    (1, 32, 1024, 1024, False),    # one block pair of benchmark config 3 (full)
    (1, 4, 1024, 1024, True),      # config 3, diagonal
    (1, 16, 4096, 4096, True),     # enough workgroups for the 256-row form
    (1, 2, 130, 515, False), (2, 3, 300, 300, True), (1, 1, 77, 200, True),
    (1, 2, 512, 129, True), (1, 1, 1, 65, False), (1, 2, 50, 40, False), (1, 1, 200, 1, False), (1, 1, 64, 64, True),
])
def test_block_forward_with_e4m3_q_k_v(B, H, Sq, Sk, causal, dtype):
    """spa_flash_fwd_fp8qkv against the oracle on the dequantised q, k, v: a product of two e4m3 values is exact in
    fp32, so the scores differ from the oracle's only by the order of the fp32 additions; same tolerances as every
    16-bit kernel (out atol 2e-2 / rtol 1.6e-2, lse atol 1e-3).  No reference output exists for an 8-bit path."""
    D = 128
    q8, qsc, q_deq = quantised((B, H, Sq, D), 520, "bhsd", spread=1.2)
    k8, ksc, k_deq = quantised((B, H, Sk, D), 521, "bhsd", spread=1.5)
    v8, vsc, v_deq = quantised((B, H, Sk, D), 522, "bhsd", spread=0.7)
    want_out, want_lse = O.attn_block(q_deq, k_deq, v_deq, None, causal)
    for share, groups in ((0, 0), (1, 1), (1, 2), (2, 2)):
        _lib.tune("fwd_share", share)
        _lib.tune("fwd_groups", groups)
        try:
            out, lse = ops.flash_fwd(q8.to(DEV), k8.to(DEV), v8.to(DEV), None, causal, layout="bhsd", q_scale=qsc, k_scale=ksc,
                                     v_scale=vsc, out_dtype=dtype)
        finally:
            _lib.tune("fwd_share", 0)
            _lib.tune("fwd_groups", 0)
        assert out.dtype == dtype and lse.dtype == torch.float32
        check_out(out, want_out, dtype, f"share={share} groups={groups}")
        check_lse(lse, want_lse)
    out2, lse2 = spa.intel_flash_attn_forward(q8.to(DEV), k8.to(DEV), v8.to(DEV), causal=causal, q_scale=qsc, k_scale=ksc, v_scale=vsc,
                                              out_dtype=dtype)
    check_out(out2, want_out, dtype, "operator shim")


def test_e4m3_q_k_v_public_layout_negative_scale_and_argument_checks():
    B, S, H, D = 2, 200, 3, 128
    q8, qsc, q_deq = quantised((B, S, H, D), 530, "bshd")
    k8, ksc, k_deq = quantised((B, S, H, D), 531, "bshd")
    v8, vsc, v_deq = quantised((B, S, H, D), 532, "bshd")
    for scale in (None, -0.07, 0.0):
        want_out, want_lse = O.full_attention(q_deq, k_deq, v_deq, scale, True)
        out, lse = ops.flash_fwd(q8.to(DEV), k8.to(DEV), v8.to(DEV), scale, True, q_scale=qsc, k_scale=ksc, v_scale=vsc)
        check_out(out, want_out, torch.bfloat16, f"scale {scale}")
        check_lse(lse, want_lse)
    with pytest.raises(ValueError):
        ops.flash_fwd(q8.to(DEV), k8.to(DEV), v8.to(DEV), None, True, k_scale=ksc, v_scale=vsc)             # no q_scale
    with pytest.raises(TypeError):
        ops.flash_fwd(q8.to(DEV), k_deq.bfloat16().to(DEV), v8.to(DEV), None, True, q_scale=qsc, k_scale=ksc, v_scale=vsc)
    q64 = q8[..., :64].contiguous()
    with pytest.raises(_lib.SpaError):  # head dim 64: no 8-bit score variant
        ops.flash_fwd(q64.to(DEV), k8[..., :64].contiguous().to(DEV), v8[..., :64].contiguous().to(DEV), None, True, q_scale=qsc,
                      k_scale=ksc, v_scale=vsc)


@pytest.mark.parametrize("B,H,P,s,causal", [(1, 2, 4, 128, True), (2, 3, 3, 100, True), (1, 2, 2, 260, False), (1, 32, 8, 256, True)])
def test_ring_forward_with_e4m3_q_k_v(B, H, P, s, causal):
    """spa_ring_fwd_fp8qkv in its three schedules (slots and the merging epilogue included) against the oracle's full
    attention on the dequantised tensors."""
    D, S = 128, P * s
    q8, qsc, q_deq = quantised((B, S, H, D), 540, "bshd", spread=1.2)
    k8, ksc, k_deq = quantised((B, S, H, D), 541, "bshd", spread=1.5)
    v8, vsc, v_deq = quantised((B, S, H, D), 542, "bshd", spread=0.7)
    want_out, want_lse = O.full_attention(q_deq, k_deq, v_deq, None, causal)
    for fuse in ("step", "rank", "all"):
        for dtype in (torch.bfloat16, torch.float16):
            out, lse = ops.ring_fwd(q8.to(DEV), k8.to(DEV), v8.to(DEV), P, None, causal, fuse=fuse, q_scale=qsc, k_scale=ksc, v_scale=vsc,
                                    out_dtype=dtype)
            assert out.dtype == dtype
            check_out(out, want_out, dtype, f"{fuse} {dtype}")
            check_lse(lse, want_lse)
    with pytest.raises(_lib.SpaError):
        ops.ring_fwd(q8.to(DEV), k8.to(DEV), v8.to(DEV), P, None, True, q_scale=qsc, k_scale=ksc, v_scale=vsc, sharding="zigzag")
