"""GPU parity at the full sizes of benchmark configs 2-5.

The float64 CPU oracle covers these shapes at reduced sizes in test_gpu_parity.py; here the HIP
path runs at the full size and is checked
  * against a plain fp32 PyTorch evaluation on the same GPU of the same mathematics
    (softmax(q k^T scale + mask) v, logsumexp) for eight (batch, head) slices per config, to the
    stated tolerances (bf16 out atol 2e-2 / rtol 1.6e-2, lse atol 1e-3,
    gradients 3e-2 of the gradient's scale), and
  * against the float64 CPU oracle on a few dozen random query rows per config (which pins the
    on-device fp32 evaluation itself), and
  * through size-independent properties: the three ring schedules and the step-by-step path
    agree, ring == one block call over the same keys, re-layout is a bit-exact permutation whose
    inverse restores the input, a value projection of all ones returns ones, lse of a ring equals
    logsumexp over the chunks' lse.
"""
import math

import pytest
import torch

from conftest import rand_qkv
import sp_aurora_amd as spa
from sp_aurora_amd import _lib, ops

pytestmark = pytest.mark.gpu
DEV = "cuda"
OUT_ATOL, OUT_RTOL, LSE_ATOL = 2e-2, 1.6e-2, 1e-3


def randn(shape, seed, dtype, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float32) * scale).to(dtype).to(DEV)


def config_qkv(shape, seed, scale=1.0, n=3):
    """The input recipe of the benchmark configs: ONE generator seeded with the config's seed, N(0,1) * scale
    drawn in fp32 on the CPU in the order q, k, v (, dout), cast to bf16 (what bench.py feeds the same config)."""
    return [t.to(DEV) for t in rand_qkv(shape, seed, torch.bfloat16, scale, n)]


def ref_head(q, k, v, scale, causal, q_offset=0):
    """fp32 attention of one head on the GPU: q [Sq,D], k,v [Sk,D]; query i sits at absolute
    position q_offset + i and sees keys <= its position when causal."""
    s = (q.float() @ k.float().T) * scale
    if causal:
        qi = torch.arange(q.shape[0], device=q.device)[:, None] + q_offset
        kj = torch.arange(k.shape[0], device=q.device)[None, :]
        s = s.masked_fill(kj > qi, float("-inf"))
    lse = torch.logsumexp(s, -1)
    p = torch.exp(s - lse[:, None])
    return p @ v.float(), lse


def spot_check_rows(out_h, lse_h, q_h, k_h, v_h, scale, causal, what, n_rows=24, seed=0, q_offset=0):
    """Float64 CPU oracle on random query rows of one head: q_h [Sq,D], k_h, v_h [Sk,D],
    out_h [Sq,D], lse_h [Sq]; query i sits at absolute position q_offset + i."""
    from oracle import attn_oracle as O
    g = torch.Generator().manual_seed(seed)
    rows = torch.randperm(q_h.shape[0], generator=g)[:n_rows].tolist() + [0, q_h.shape[0] - 1]
    kc, vc = k_h.cpu(), v_h.cpu()
    for r in rows:
        n_keys = min(q_offset + r + 1, kc.shape[0]) if causal else kc.shape[0]
        # one query against the keys it sees: a non-causal block of the oracle, [B=1,H=1,1,D] x [1,1,n_keys,D]
        want_o, want_l = O.attn_block(q_h[r].cpu()[None, None, None], kc[None, None, :n_keys], vc[None, None, :n_keys], scale, False)
        got_o, got_l = out_h[r].cpu().double(), lse_h[r].cpu().double()
        bad = (got_o - want_o[0, 0, 0]).abs() > OUT_ATOL + OUT_RTOL * want_o[0, 0, 0].abs()
        assert not bad.any(), f"{what} row {r}: out max abs err {(got_o - want_o[0, 0, 0]).abs().max().item():.3e}"
        assert abs(got_l.item() - want_l[0, 0, 0].item()) <= LSE_ATOL, f"{what} row {r}: lse err {abs(got_l.item() - want_l[0, 0, 0].item()):.3e}"


def assert_out(got, want, what):
    got, want = got.float(), want.float()
    assert torch.isfinite(got).all(), f"{what}: non-finite values"
    bad = (got - want).abs() > OUT_ATOL + OUT_RTOL * want.abs()
    assert not bad.any(), f"{what}: {int(bad.sum())} out of tolerance, max abs err {(got - want).abs().max().item():.3e}"


def assert_lse(got, want, what):
    err = (got.float() - want.float()).abs().max().item()
    assert err <= LSE_ATOL, f"{what}: lse max abs err {err:.3e}"


# ------------------------------------------------------------------ config 2
def test_config2_ring_rank2_of_4():
    """bf16, B=2, S=4096 in 4 chunks of 1024, H=32, D=64, causal; rank 2 visits chunks 2, 1, 0."""
    B, S, H, D, P, rank = 2, 4096, 32, 64, 4, 2
    s = S // P
    scale = D ** -0.5
    q, k, v = config_qkv((B, S, H, D), 1)
    q_local = q[:, rank * s:(rank + 1) * s]
    # step by step with stand-alone kernels and update_out_and_lse as its own pass
    out_a, lse_a = spa.ring.ring_flash_attn_forward_rank(q_local, list(k.split(s, 1)), list(v.split(s, 1)), rank, scale, True)
    for b, h in ((0, 0), (1, 31), (0, 17), (1, 4), (0, 9), (1, 13), (0, 22), (1, 26)):
        want_o, want_l = ref_head(q_local[b, :, h], k[b, :(rank + 1) * s, h], v[b, :(rank + 1) * s, h], scale, True, rank * s)
        assert_out(out_a[b, :, h], want_o, f"stepwise b{b} h{h}")
        assert_lse(lse_a[b, h], want_l, f"stepwise b{b} h{h}")
    spot_check_rows(out_a[1, :, 5], lse_a[1, 5], q_local[1, :, 5], k[1, :(rank + 1) * s, 5], v[1, :(rank + 1) * s, 5], scale, True,
                    "cfg2 fp64", q_offset=rank * s)
    # the C driver in its three schedules writes rank 2's rows of the full tensors
    for fuse in ("step", "rank", "all"):
        out = torch.zeros_like(q)
        lse = torch.zeros((B, H, S), dtype=torch.float32, device=DEV)
        ops.ring_fwd(q, k, v, P, scale, True, rank=rank, out=out, lse=lse, fuse=fuse)
        assert_out(out[:, rank * s:(rank + 1) * s], out_a, f"driver {fuse} vs stepwise")
        assert_lse(lse[:, :, rank * s:(rank + 1) * s], lse_a, f"driver {fuse} vs stepwise")
        assert not out[:, :rank * s].any() and not out[:, (rank + 1) * s:].any(), "other ranks' rows were written"
    # one block call over the same keys (causal offset by construction: keys 0..3071, queries 2048..3071)
    # is the same mathematics: compare through the lse of the unmasked part
    o01, l01 = ops.flash_fwd(q_local, k[:, :rank * s], v[:, :rank * s], scale, False)
    o2, l2 = ops.flash_fwd(q_local, k[:, rank * s:(rank + 1) * s], v[:, rank * s:(rank + 1) * s], scale, True)
    assert_lse(torch.logaddexp(l01, l2), lse_a, "lse = logaddexp of the two parts")


# ------------------------------------------------------------------ config 3
def test_config3_ring_sweep_all_ranks():
    """bf16, B=1, S=8192 in 8 chunks of 1024, H=32, D=128, causal, inputs N(0,1)*0.5: 36 block pairs."""
    B, S, H, D, P = 1, 8192, 32, 128, 8
    scale = D ** -0.5
    q, k, v = config_qkv((B, S, H, D), 2, 0.5)
    res = {f: spa.ring.ring_flash_attn_forward(q, k, v, scale, True, P, fuse=f) for f in ("step", "rank", "all")}
    for h in (0, 4, 9, 13, 18, 22, 27, 31):
        want_o, want_l = ref_head(q[0, :, h], k[0, :, h], v[0, :, h], scale, True)
        for f, (o, l) in res.items():
            assert_out(o[0, :, h], want_o, f"{f} h{h}")
            assert_lse(l[0, h], want_l, f"{f} h{h}")
    spot_check_rows(res["all"][0][0, :, 7], res["all"][1][0, 7], q[0, :, 7], k[0, :, 7], v[0, :, 7], scale, True, "cfg3 fp64")
    # ring == the block operator on the undivided sequence (P = 1)
    o1, l1 = spa.ring.ring_flash_attn_forward(q, k, v, scale, True, 1)
    for f, (o, l) in res.items():
        assert_out(o, o1, f"{f} vs P=1")
        assert_lse(l, l1, f"{f} vs P=1")
    # deterministic: the same call twice gives the same bits
    o_again, l_again = spa.ring.ring_flash_attn_forward(q, k, v, scale, True, P, fuse="all")
    assert torch.equal(o_again, res["all"][0]) and torch.equal(l_again, res["all"][1])
    # V of all ones: every output element is 1 whatever the weights
    ones = torch.ones_like(v)
    o_ones, _ = spa.ring.ring_flash_attn_forward(q, k, ones, scale, True, P, fuse="all")
    assert (o_ones.float() - 1).abs().max().item() <= 2 ** -7


def test_config3_zigzag_shards_give_the_same_attention():
    """The config-3 tensors with their rows in zigzag order (rank r holds half-chunks r and 15-r): the three
    schedules against the contiguous ring on the rows in natural order (itself checked above), eight heads
    against the on-device fp32 evaluation, float64 rows of one head."""
    B, S, H, D, P = 1, 8192, 32, 128, 8
    scale = D ** -0.5
    q, k, v = config_qkv((B, S, H, D), 2, 0.5)
    idx = spa.ring.zigzag_order(S, P, DEV)
    qz, kz, vz = (t.index_select(1, idx) for t in (q, k, v))
    o_nat, l_nat = spa.ring.ring_flash_attn_forward(q, k, v, scale, True, P, fuse="all")
    res = {f: spa.ring.ring_flash_attn_forward(qz, kz, vz, scale, True, P, fuse=f, sharding="zigzag") for f in ("step", "rank", "all")}
    for f, (o, l) in res.items():
        assert_out(o, o_nat.index_select(1, idx), f"zigzag {f} vs contiguous ring")
        assert_lse(l, l_nat.index_select(2, idx), f"zigzag {f} vs contiguous ring")
    inv = torch.argsort(idx)
    o_all, l_all = res["all"][0].index_select(1, inv), res["all"][1].index_select(2, inv)
    for h in (1, 5, 10, 14, 19, 23, 28, 30):
        want_o, want_l = ref_head(q[0, :, h], k[0, :, h], v[0, :, h], scale, True)
        assert_out(o_all[0, :, h], want_o, f"zigzag all h{h}")
        assert_lse(l_all[0, h], want_l, f"zigzag all h{h}")
    spot_check_rows(o_all[0, :, 20], l_all[0, 20], q[0, :, 20], k[0, :, 20], v[0, :, 20], scale, True, "cfg3 zigzag fp64", n_rows=12)


# ------------------------------------------------------------------ config 4
def test_config4_ulysses_relayout_and_attention():
    """bf16 [P=8, B=1, s=2048, H=32, D=128] -> [8, 1, 16384, 4, 128], causal attention, and back."""
    P, B, s, H, D = 8, 1, 2048, 32, 128
    scale = D ** -0.5
    q, k, v = config_qkv((P, B, s, H, D), 3)
    h = H // P
    # bit-exact permutation: rank r of the result holds heads r*h..(r+1)*h of the whole sequence
    y = ops.relayout_s2h(q, P)
    assert y.shape == (P, B, P * s, h, D)
    want = q.permute(1, 0, 2, 3, 4).reshape(B, P * s, P, h, D).permute(2, 0, 1, 3, 4)
    assert torch.equal(y, want)
    assert torch.equal(ops.relayout_h2s(y, P), q)
    assert torch.equal(spa.all_to_all_4D(q, 2, 1), y)
    # packed 5-D form
    qkv = torch.stack([q, k, v], dim=3)  # [P,B,s,3,H,D]
    y5 = spa.all_to_all_5D(qkv, 3, 1)
    assert y5.shape == (P, B, P * s, 3, h, D) and torch.equal(y5[:, :, :, 0], y)
    assert torch.equal(spa.all_to_all_5D(y5, 1, 3), qkv)
    # the whole Ulysses forward
    out, lse = spa.intel_ulysses_flash_attn_forward(None, q, k, v, scale, causal=True)
    assert out.shape == q.shape and lse.shape == (P, B, h, P * s)
    full = lambda t: t.permute(1, 0, 2, 3, 4).reshape(B, P * s, H, D)
    qf, kf, vf, of = full(q), full(k), full(v), full(out)
    for hd in (0, 5, 10, 15, 16, 21, 26, 31):  # one head of every head group
        want_o, want_l = ref_head(qf[0, :, hd], kf[0, :, hd], vf[0, :, hd], scale, True)
        assert_out(of[0, :, hd], want_o, f"ulysses h{hd}")
        assert_lse(lse[hd // h, 0, hd % h], want_l, f"ulysses h{hd}")
    spot_check_rows(of[0, :, 9], lse[9 // h, 0, 9 % h], qf[0, :, 9], kf[0, :, 9], vf[0, :, 9], scale, True, "cfg4 fp64", n_rows=12)
    assert torch.equal(spa.ulysses_flash_attn_func(q, k, v, causal=True), out)


# ------------------------------------------------------------------ config 5
def test_config5_qkvpacked_long_context_forward_backward():
    """bf16 qkv [1, 32768, 3, 16, 128], causal, ring of 16 chunks of 2048: out, lse, dq, dk, dv."""
    B, S, H, D, P = 1, 32768, 16, 128, 16
    scale = D ** -0.5
    qkv = randn((B, S, 3, H, D), 4, torch.bfloat16).requires_grad_(True)
    dout = randn((B, S, H, D), 5, torch.bfloat16)
    out, lse, _ = spa.ring_flash_attn_qkvpacked_func(qkv, causal=True, return_attn_probs=True, ring_size=P)
    out.backward(dout)
    g = qkv.grad
    assert g.shape == qkv.shape and g.dtype == torch.bfloat16
    with torch.no_grad():
        # forward: the ring equals the undivided block operator
        o1, l1 = ops.flash_fwd(qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2], scale, True)
        assert_out(out, o1, "ring vs P=1")
        assert_lse(lse, l1, "ring vs P=1")
    with torch.no_grad():
        spot_check_rows(out[0, :, 3], lse[0, 3], qkv[0, :, 0, 3], qkv[0, :, 1, 3], qkv[0, :, 2, 3], scale, True, "cfg5 fp64", n_rows=12)
    for h in (0, 2, 4, 6, 9, 11, 13, 15):
        qh, kh, vh = (qkv.detach()[0, :, i, h].float().requires_grad_(True) for i in range(3))
        want_o, want_l = ref_head(qh, kh, vh, scale, True)
        assert_out(out[0, :, h], want_o.detach(), f"out h{h}")
        assert_lse(lse[0, h], want_l.detach(), f"lse h{h}")
        want_o.backward(dout[0, :, h].float())
        for i, (name, ref) in enumerate((("dq", qh.grad), ("dk", kh.grad), ("dv", vh.grad))):
            got = g[0, :, i, h].float()
            tol = 3e-2 * ref.abs().max() + 3e-2 * ref.abs()
            bad = (got - ref).abs() > tol
            assert not bad.any(), f"{name} h{h}: {int(bad.sum())} out of tolerance, max err {(got - ref).abs().max().item():.3e} (scale {ref.abs().max().item():.3e})"
        del qh, kh, vh, want_o, want_l
        torch.cuda.empty_cache()


def test_config5_zigzag_shards_forward_and_backward():
    """Config 5's tensors in zigzag order, P = 16: forward (one launch per rank) and both backward forms against
    the contiguous ring's results on the rows in natural order (checked against fp32 / float64 above)."""
    B, S, H, D, P = 1, 32768, 16, 128, 16
    scale = D ** -0.5
    qkv = randn((B, S, 3, H, D), 4, torch.bfloat16)
    dout = randn((B, S, H, D), 5, torch.bfloat16)
    q, k, v = qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]
    idx = spa.ring.zigzag_order(S, P, DEV)
    o_nat, l_nat = spa.ring.ring_flash_attn_forward(q, k, v, scale, True, P, fuse="all")
    g_nat = spa.ring.ring_flash_attn_backward(dout, q, k, v, o_nat, l_nat, scale, True, P, fuse="all")
    qz, kz, vz, dz = (t.index_select(1, idx) for t in (q, k, v, dout))
    oz, lz = spa.ring.ring_flash_attn_forward(qz, kz, vz, scale, True, P, fuse="rank", sharding="zigzag")
    assert_out(oz, o_nat.index_select(1, idx), "zigzag rank vs contiguous ring")
    assert_lse(lz, l_nat.index_select(2, idx), "zigzag rank vs contiguous ring")
    for fuse in ("step", "all"):
        gz = spa.ring.ring_flash_attn_backward(dz, qz, kz, vz, oz, lz, scale, True, P, fuse=fuse, sharding="zigzag")
        for name, got, ref in zip(("dq", "dk", "dv"), gz, g_nat):
            ref = ref.index_select(1, idx).float()
            bad = (got.float() - ref).abs() > 3e-2 * ref.abs().max() + 3e-2 * ref.abs()
            assert torch.isfinite(got).all() and not bad.any(), f"zigzag {fuse} {name}: {int(bad.sum())} out of tolerance"


# ------------------------------------------------------------------ beyond the configs: a long sequence
def test_long_sequence_131072_forward_backward_spot_checks():
    """bf16, B=1, S=131072, H=2, D=128, causal (a score matrix no reference can materialise):
    forward rows and gradient rows / columns against float64 evaluations of the defining sums."""
    B, S, H, D = 1, 131072, 2, 128
    scale = D ** -0.5
    q, k, v, dout = (randn((B, S, H, D), 50 + i, torch.bfloat16) for i in range(4))
    out, lse = spa.ring.ring_flash_attn_forward(q, k, v, scale, True, 8, fuse="all")
    o1, l1 = ops.flash_fwd(q, k, v, scale, True)
    assert_out(out, o1, "ring of 8 vs one block call")
    assert_lse(lse, l1, "ring of 8 vs one block call")
    h = 1
    spot_check_rows(out[0, :, h], lse[0, h], q[0, :, h], k[0, :, h], v[0, :, h], scale, True, "S=131072 fp64", n_rows=6)
    dq, dk, dv = spa.ring.ring_flash_attn_backward(dout, q, k, v, out, lse, scale, True, 8, fuse="all")
    # float64 on the CPU, one head
    qc, kc, vc, doc, oc = (t[0, :, h].cpu().double() for t in (q, k, v, dout, out))
    lc = lse[0, h].cpu().double()
    delta = (doc * oc).sum(-1)
    g = torch.Generator().manual_seed(1)
    for i in torch.randint(0, S, (4,), generator=g).tolist() + [0, S - 1]:
        # dq_i = scale * sum_{j<=i} P_ij (dO_i . v_j - delta_i) k_j
        p = torch.exp(kc[:i + 1] @ qc[i] * scale - lc[i])
        ds = p * (vc[:i + 1] @ doc[i] - delta[i])
        want = scale * (ds @ kc[:i + 1])
        err = (dq[0, i, h].cpu().double() - want).abs().max().item()
        assert err <= 3e-2 * max(want.abs().max().item(), 1e-2), f"dq row {i}: err {err:.3e} scale {want.abs().max().item():.3e}"
    for j in torch.randint(0, S, (4,), generator=g).tolist() + [0, S - 1]:
        # dv_j = sum_{i>=j} P_ij dO_i ;  dk_j = scale * sum_{i>=j} P_ij (dO_i . v_j - delta_i) q_i
        p = torch.exp(qc[j:] @ kc[j] * scale - lc[j:])
        want_dv = p @ doc[j:]
        ds = p * (doc[j:] @ vc[j] - delta[j:])
        want_dk = scale * (ds @ qc[j:])
        for name, got, want in (("dv", dv, want_dv), ("dk", dk, want_dk)):
            err = (got[0, j, h].cpu().double() - want).abs().max().item()
            assert err <= 3e-2 * max(want.abs().max().item(), 1e-2), f"{name} row {j}: err {err:.3e} scale {want.abs().max().item():.3e}"


# ------------------------------------------------------------------ beyond 2 GiB per (batch, head)
def test_rows_of_one_head_spanning_more_than_2_gib():
    """bf16 [B=1, S=8448, H=1024, D=128] viewed as H=4 heads of a tensor whose rows are 256 KiB apart: the rows of one
    head span 2.06 GiB, past what one buffer descriptor with 32-bit offsets covers, so the variants that re-base their
    descriptors per tile run (forward, ring forward in its three schedules, backward).  The same four heads packed
    into compact tensors go through the ordinary variants: same mathematics, results within the bf16 tolerances,
    and float64 rows of one head pin both."""
    S, Hs, H, D, P = 8448, 1024, 4, 128, 4
    scale = D ** -0.5
    gen = torch.Generator(device=DEV).manual_seed(60)  # 1.1 G elements per tensor: drawn on the device
    big = [torch.randn((1, S, Hs, D), generator=gen, device=DEV, dtype=torch.bfloat16) for _ in range(4)]
    wide = [t[:, :, ::341] for t in big]  # heads 0, 341, 682, 1023 as strided views (head stride 341 D), no copy
    assert all(w.shape == (1, S, H, D) and w.stride(1) * 2 * (S - 1) > 2 ** 31 for w in wide)
    q, k, v, dout = wide
    qc, kc, vc, dc = (w.contiguous() for w in wide)
    o_ref, l_ref = ops.flash_fwd(qc, kc, vc, scale, True)
    o, l = ops.flash_fwd(q, k, v, scale, True)
    assert_out(o, o_ref, "block forward, rows 256 KiB apart")
    assert_lse(l, l_ref, "block forward, rows 256 KiB apart")
    spot_check_rows(o[0, :, 3], l[0, 3], qc[0, :, 3], kc[0, :, 3], vc[0, :, 3], scale, True, "2 GiB span fp64", n_rows=10)
    for fuse in ("step", "rank", "all"):
        o2, l2 = ops.ring_fwd(q, k, v, P, scale, True, fuse=fuse)
        assert_out(o2, o_ref, f"ring {fuse}, rows 256 KiB apart")
        assert_lse(l2, l_ref, f"ring {fuse}, rows 256 KiB apart")
    delta = ops.bwd_delta(o_ref, dc)
    g_ref = ops.flash_bwd_out(qc, kc, vc, dc, l_ref, delta, scale, True)
    g = ops.flash_bwd_out(q, k, v, dout, l_ref, delta, scale, True)
    for name, got, ref in zip(("dq", "dk", "dv"), g, g_ref):
        ref = ref.float()
        bad = (got.float() - ref).abs() > 3e-2 * ref.abs().max() + 3e-2 * ref.abs()
        assert torch.isfinite(got).all() and not bad.any(), f"{name}: {int(bad.sum())} out of tolerance"


def test_decode_step_against_a_long_cache_with_the_keys_split():
    """The shape of `bench.py --workload decode`: one new token (and a block of 128) per head against 32768 cached keys, the
    library's own choice of chunks.  Every head against the fp32 reference on the GPU, rows of two heads against the fp64
    oracle; the e4m3 cache the same way on its dequantised values."""
    B, H, Sk, D = 1, 32, 32768, 128
    k, v = config_qkv((B, Sk, H, D), 7, n=2)
    assert _lib.load().spa_flash_fwd_splitkv_suggest(B, H, 1, Sk, D, 0, _lib.SPA_BF16) > 1
    for sq in (1, 128):
        (q,) = config_qkv((B, sq, H, D), 8, n=1)
        out, lse = ops.flash_fwd(q, k, v, None, False)                      # split_kv="auto"
        for h in range(H):
            ro, rl = ref_head(q[0, :, h], k[0, :, h], v[0, :, h], D ** -0.5, False)
            assert_out(out[0, :, h], ro, f"decode Sq={sq} head {h}")
            assert_lse(lse[0, h], rl, f"decode Sq={sq} head {h}")
        for h in (0, H - 1):
            spot_check_rows(out[0, :, h], lse[0, h], q[0, :, h], k[0, :, h], v[0, :, h], D ** -0.5, False, f"decode Sq={sq} head {h}", n_rows=3)
        k8, ksc = ops.quantize_fp8_per_head(k.float())
        v8, vsc = ops.quantize_fp8_per_head(v.float())
        out8, lse8 = ops.flash_fwd(q, k8, v8, None, False, k_scale=ksc, v_scale=vsc)
        kd, vd = k8.float() * ksc[:, None, :, None], v8.float() * vsc[:, None, :, None]
        for h in (3, 17):
            ro, rl = ref_head(q[0, :, h], kd[0, :, h], vd[0, :, h], D ** -0.5, False)
            assert_out(out8[0, :, h], ro, f"decode e4m3 Sq={sq} head {h}")
            assert_lse(lse8[0, h], rl, f"decode e4m3 Sq={sq} head {h}")


def test_decode_step_of_a_batch_with_ragged_caches():
    """64 sequences with 1024 to 4096 cached keys each, one new token per sequence, 32 heads (a packed batch through
    flash_fwd_varlen: the kernel that streams K and V): every head of eight sequences against the fp32 reference on the
    GPU, the rows of two (sequence, head) pairs against the fp64 oracle, bf16 and e4m3 caches."""
    import random
    rng = random.Random(11)
    nseq, H, D = 64, 32, 128
    lens_k = [rng.randrange(1024, 4097) for _ in range(nseq)]
    Tk = sum(lens_k)
    (q,) = config_qkv((1, nseq, H, D), 9, n=1)
    k, v = config_qkv((1, Tk, H, D), 10, n=2)
    cu_q = torch.arange(nseq + 1, dtype=torch.int32, device=DEV)
    starts = [0]
    for n in lens_k:
        starts.append(starts[-1] + n)
    cu_k = torch.tensor(starts, dtype=torch.int32, device=DEV)
    out, lse = ops.flash_fwd_varlen(q[0], k[0], v[0], cu_q, cu_k, 1, max(lens_k), None, False)
    k8, ksc = ops.quantize_fp8_per_head(k.float())
    v8, vsc = ops.quantize_fp8_per_head(v.float())
    out8, lse8 = ops.flash_fwd_varlen(q[0], k8[0], v8[0], cu_q, cu_k, 1, max(lens_k), None, False,
                                      k_scale=ksc.expand(nseq, H).contiguous(), v_scale=vsc.expand(nseq, H).contiguous())
    kd, vd = k8.float() * ksc[:, None, :, None], v8.float() * vsc[:, None, :, None]
    for b in list(range(0, nseq, 9)) + [nseq - 1]:
        ks = slice(starts[b], starts[b + 1])
        for h in range(H):
            ro, rl = ref_head(q[0, b:b + 1, h], k[0, ks, h], v[0, ks, h], D ** -0.5, False)
            assert_out(out[b:b + 1, h], ro, f"sequence {b} head {h}")
            assert_lse(lse[h, b:b + 1], rl, f"sequence {b} head {h}")
            ro, rl = ref_head(q[0, b:b + 1, h], kd[0, ks, h], vd[0, ks, h], D ** -0.5, False)
            assert_out(out8[b:b + 1, h], ro, f"e4m3 sequence {b} head {h}")
            assert_lse(lse8[h, b:b + 1], rl, f"e4m3 sequence {b} head {h}")
    for b, h in ((0, 0), (nseq - 1, H - 1)):
        ks = slice(starts[b], starts[b + 1])
        spot_check_rows(out[b:b + 1, h], lse[h, b:b + 1], q[0, b:b + 1, h], k[0, ks, h], v[0, ks, h], D ** -0.5, False,
                        f"sequence {b} head {h}", n_rows=1)

