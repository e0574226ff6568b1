"""GPU parity of the zigzag-sharded causal ring (rank r holds half-chunks r and 2P-1-r): forward in the
three schedules and backward in both forms, against the oracle's full causal attention on the rows in
natural order (un-permuting the HIP results), for every dtype and awkward half-chunk sizes."""
import pytest
import torch

from conftest import rand_qkv
from oracle import attn_oracle as O
import sp_aurora_amd as spa
from sp_aurora_amd import _lib, ops
from test_gpu_parity import DEV, check_grad, check_lse, check_out

pytestmark = pytest.mark.gpu


def zigzag_inputs(shape, seed, dtype, P, n=3):
    """Tensors in natural order (CPU, for the oracle) and the same rows in zigzag order on the device."""
    nat = rand_qkv(shape, seed, dtype, n=n)
    idx = O.zigzag_order(shape[1], P)
    return nat, [t[:, idx].contiguous().to(DEV) for t in nat], idx


CASES = [
    # B, H, P, half-chunk rows, D, dtype
    (1, 2, 2, 64, 128, torch.bfloat16),
    (2, 3, 4, 64, 64, torch.bfloat16),
    (1, 2, 3, 50, 128, torch.float16),     # ragged tiles in both halves
    (1, 1, 5, 16, 32, torch.bfloat16),     # halves shorter than a sub-tile
    (1, 2, 4, 130, 64, torch.float16),     # a half-chunk of two tiles, the second nearly empty
    (2, 2, 2, 192, 128, torch.bfloat16),
    (1, 2, 3, 100, 64, torch.float32),     # fp32: block launches on sub-blocks + merge kernels
    (1, 1, 2, 33, 128, torch.float32),
    (1, 2, 1, 64, 64, torch.bfloat16),     # a ring of one: zigzag order is the natural order
]


@pytest.mark.parametrize("B,H,P,hc,D,dtype", CASES)
def test_zigzag_ring_forward_matches_full_causal_attention(B, H, P, hc, D, dtype):
    S = 2 * P * hc
    (q, k, v), (qz, kz, vz), idx = zigzag_inputs((B, S, H, D), 700, dtype, P)
    want_o, want_l = O.full_attention(q, k, v, None, True)
    for fuse in ("step", "rank", "all"):
        for share, groups in ((0, 0), (1, 1), (2, 2)):
            _lib.tune("fwd_share", share)
            _lib.tune("fwd_groups", groups)
            try:
                out, lse = spa.ring.ring_flash_attn_forward(qz, kz, vz, None, True, P, fuse=fuse, sharding="zigzag")
            finally:
                _lib.tune("fwd_share", 0)
                _lib.tune("fwd_groups", 0)
            got_o = torch.empty_like(out.cpu())
            got_o[:, idx] = out.cpu()          # undo the sharding: row i of the result is natural row idx[i]
            got_l = torch.empty_like(lse.cpu())
            got_l[:, :, idx] = lse.cpu()
            check_out(got_o, want_o, dtype, f"{fuse} share={share} groups={groups}")
            check_lse(got_l, want_l)


def test_zigzag_single_rank_writes_only_its_rows_and_agrees_with_the_sweep():
    B, H, P, hc, D, dtype = 1, 2, 4, 64, 128, torch.bfloat16
    S = 2 * P * hc
    _, (qz, kz, vz), _ = zigzag_inputs((B, S, H, D), 701, dtype, P)
    s = S // P
    for fuse in ("step", "rank", "all"):
        full_o, full_l = ops.ring_fwd(qz, kz, vz, P, None, True, fuse=fuse, sharding="zigzag")
        for r in range(P):
            out = torch.full_like(qz, 7.0)
            lse = torch.full((B, H, S), 7.0, dtype=torch.float32, device=DEV)
            ops.ring_fwd(qz, kz, vz, P, None, True, rank=r, out=out, lse=lse, fuse=fuse, sharding="zigzag")
            rs = slice(r * s, (r + 1) * s)
            assert torch.equal(out[:, rs], full_o[:, rs]) and torch.equal(lse[:, :, rs], full_l[:, :, rs])
            mask = torch.ones(S, dtype=torch.bool)
            mask[rs] = False
            assert (out[:, mask] == 7.0).all() and (lse[:, :, mask] == 7.0).all()


def test_zigzag_without_a_mask_is_the_contiguous_ring_and_bad_sizes_are_refused():
    B, H, P, D, dtype = 1, 2, 2, 64, torch.bfloat16
    q, k, v = (t.to(DEV) for t in rand_qkv((B, 256, H, D), 702, dtype))
    for fuse in ("step", "rank", "all"):
        a = spa.ring.ring_flash_attn_forward(q, k, v, None, False, P, fuse=fuse, sharding="zigzag")
        b = spa.ring.ring_flash_attn_forward(q, k, v, None, False, P, fuse=fuse)
        assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    # 5 ranks divide 255 rows, 10 half-chunks do not
    q5, k5, v5 = (t[:, :255].contiguous() for t in (q, k, v))
    with pytest.raises(ValueError):
        spa.ring.ring_flash_attn_forward(q5, k5, v5, None, True, 5, sharding="zigzag")
    with pytest.raises(_lib.SpaError):  # the C entry point says the same
        ops.ring_fwd(q5, k5, v5, 5, None, True, sharding="zigzag")
    with pytest.raises(ValueError):
        spa.ring.ring_flash_attn_forward(q, k, v, None, True, P, sharding="striped")


@pytest.mark.parametrize("B,H,P,hc,D,dtype", [
    (1, 2, 2, 64, 128, torch.bfloat16),
    (2, 2, 4, 32, 64, torch.bfloat16),
    (1, 2, 3, 50, 64, torch.float16),
    (1, 1, 2, 40, 128, torch.float32),
])
def test_zigzag_ring_backward_matches_autograd_of_full_attention(B, H, P, hc, D, dtype):
    S = 2 * P * hc
    (q, k, v, dout), (qz, kz, vz, dz), idx = zigzag_inputs((B, S, H, D), 703, dtype, P, n=4)
    want = O.attn_backward_autograd(q, k, v, dout, None, True)
    out, lse = spa.ring.ring_flash_attn_forward(qz, kz, vz, None, True, P, sharding="zigzag")
    for fuse in ("step", "all"):
        got = spa.ring.ring_flash_attn_backward(dz, qz, kz, vz, out, lse, None, True, P, fuse=fuse, sharding="zigzag")
        for g, w, name in zip(got, want, "qkv"):
            nat = torch.empty_like(g.cpu())
            nat[:, idx] = g.cpu()
            check_grad(nat, w, dtype, f"{fuse} d{name}")


def test_zigzag_public_function_with_autograd_and_packed_inputs():
    B, H, P, hc, D, dtype = 1, 2, 4, 32, 64, torch.bfloat16
    S = 2 * P * hc
    (q, k, v, dout), (qz, kz, vz, dz), idx = zigzag_inputs((B, S, H, D), 704, dtype, P, n=4)
    want_o, want_l = O.full_attention(q, k, v, None, True)
    want = O.attn_backward_autograd(q, k, v, dout, None, True)
    qkv = torch.stack([qz, kz, vz], dim=2).requires_grad_(True)
    out, lse, _ = spa.sp_aurora_qkvpacked_func(qkv, causal=True, return_attn_probs=True, ring_size=P, sharding="zigzag")
    out.backward(dz)
    nat_o = torch.empty_like(out.detach().cpu())
    nat_o[:, idx] = out.detach().cpu()
    check_out(nat_o, want_o, dtype, "packed zigzag")
    for i, name in enumerate("qkv"):
        nat = torch.empty_like(qkv.grad[:, :, i].cpu())
        nat[:, idx] = qkv.grad[:, :, i].cpu()
        check_grad(nat, want[i], dtype, "packed zigzag d" + name)
    # the built-in scratch and e4m3 K/V take the same flag
    o2, l2 = ops.ring_fwd(qz, kz, vz, P, None, True, fuse="step", static_scratch=True, sharding="zigzag")
    o3, l3 = ops.ring_fwd(qz, kz, vz, P, None, True, fuse="step", sharding="zigzag")
    assert torch.equal(o2, o3) and torch.equal(l2, l3)
    k8, ksc = ops.quantize_fp8_per_head(kz)
    v8, vsc = ops.quantize_fp8_per_head(vz)
    deq = lambda x8, sc: (x8.float() * sc[:, None, :, None]).cpu()
    inv = torch.argsort(idx)
    want8_o, want8_l = O.full_attention(q, deq(k8, ksc)[:, inv], deq(v8, vsc)[:, inv], None, True)
    for fuse in ("step", "rank", "all"):
        o8, l8 = ops.ring_fwd(qz, k8, v8, P, None, True, fuse=fuse, k_scale=ksc, v_scale=vsc, sharding="zigzag")
        check_out(o8.cpu()[:, inv], want8_o, dtype, f"e4m3 zigzag {fuse}")
        check_lse(l8.cpu()[:, :, inv], want8_l)
