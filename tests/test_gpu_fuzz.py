"""A bounded, fixed-seed sweep of random shapes through every entry of the HIP path against the
float64 oracle: block forward, ring forward in its three schedules (contiguous and zigzag shards) and with arrival flags,
e4m3 K/V (block and ring), packed variable-length batches, and the three backward forms.  Shapes are drawn from lists that
straddle the kernels' tile sizes (1, 63..65, 127..130, 255..257, ragged tails) and the
workgroup-form overrides are drawn as well, so that every kernel variant sees awkward sizes.
The sweep stops at its first failure and names the case."""
import random

import pytest
import torch

from oracle import attn_oracle as O
import sp_aurora_amd as spa
from sp_aurora_amd import _lib, ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
N_CASES = 3000
SEED = 20240611

OUT_TOL = {torch.float32: (1e-5, 1e-3), torch.bfloat16: (2e-2, 1.6e-2), torch.float16: (2e-3, 2e-3)}
LSE_ATOL = 1e-3
# gradients: tolerance relative to the gradient's largest magnitude, relative to the element, and a floor
# (rows that see one or two keys cancel in dS = P (dP - delta): what is left is the rounding of delta, a 128-term fp32 dot
# product of values of order one: up to 4e-6 seen)
GRAD_TOL = {torch.float32: (2e-5, 1e-4, 8e-6), torch.bfloat16: (3e-2, 3e-2, 8e-3), torch.float16: (4e-3, 1e-2, 2e-3)}


def _close(name, got, want, atol, rtol, info):
    got = got.detach().cpu().double()
    assert torch.isfinite(got).all() or not torch.isfinite(want).all(), f"{name} not finite: {info}"
    err = (got - want).abs()
    ok = err <= atol + rtol * want.abs()
    both_inf = torch.isinf(got) & torch.isinf(want) & (got == want)  # lse = -inf of a sequence without keys
    assert bool((ok | both_inf).all()), f"{name}: max err {err.nan_to_num(0).max().item():.3e}: {info}"


def _grads_close(got3, want3, dtype, info):
    a, r, floor = GRAD_TOL[dtype]
    for name, got, want in zip(("dq", "dk", "dv"), got3, want3):
        _close(name, got, want, a * want.abs().max().item() + floor, r, info)


def _cu(lengths):
    return torch.tensor([0] + list(torch.tensor(lengths).cumsum(0)), dtype=torch.int32)


def _case(rng):
    dtype = rng.choice([torch.float32, torch.bfloat16, torch.float16])
    D, H, B = rng.choice([32, 64, 128]), rng.choice([1, 2, 3]), rng.choice([1, 2])
    causal = rng.random() < 0.5
    kind = rng.choice(["block", "block", "ring", "ring_bwd", "fp8", "fp8", "fp8_ring", "varlen", "block_bwd", "block_bwd",
                       "varlen_bwd", "varlen_bwd", "zigzag", "zigzag", "fp8_qkv", "flags", "varlen_decode"])
    share, groups = rng.choice([0, 0, 1, 2, 2]), rng.choice([0, 0, 1, 2])
    _lib.tune("fwd_share", share)
    _lib.tune("fwd_groups", groups)
    _lib.tune("fwd32_split", rng.choice([0, 0, 1, 2]))
    _lib.tune("few_rows", rng.choice([0, 0, 1]))   # up to three unmasked query rows: the streaming kernel, or the MFMA kernels
    g = torch.Generator().manual_seed(rng.randrange(1 << 30))
    mk = lambda *shape, dt=None: torch.randn(shape, generator=g).to(dt or dtype)
    atol, rtol = OUT_TOL[dtype]
    if kind in ("fp8", "fp8_ring") and (dtype == torch.float32 or D == 32):
        return
    if kind == "fp8_qkv":  # e4m3 q as well: scores on the 8-bit matrix instruction, D = 128
        dt = rng.choice([torch.bfloat16, torch.float16])
        Sq, Sk = rng.choice([1, 3, 64, 100, 128, 256, 300, 513]), rng.choice([1, 64, 65, 128, 200, 513, 769])
        info = (kind, dt, B, H, Sq, Sk, causal, share, groups)
        qf, kf, vf = (mk(B, H, n_, 128, dt=torch.float32) for n_ in (Sq, Sk, Sk))
        (q8, qs), (k8, ks), (v8, vs) = (ops.quantize_fp8_per_head(t, "bhsd") for t in (qf, kf, vf))
        deq = lambda x8, sc: x8.double() * sc[:, :, None, None].double()
        want_o, want_l = O.attn_block(deq(q8, qs), deq(k8, ks), deq(v8, vs), None, causal)
        o, l = ops.flash_fwd(q8.to(DEV), k8.to(DEV), v8.to(DEV), None, causal, layout="bhsd", q_scale=qs, k_scale=ks, v_scale=vs, out_dtype=dt)
        _close("out", o, want_o, *OUT_TOL[dt], info)
        _close("lse", l, want_l, LSE_ATOL, 0, info)
        return
    if kind == "flags":  # one launch per rank behind arrival flags (all raised): 16-bit types, D = 64 or 128
        if dtype == torch.float32 or D == 32:
            return
        P, s = rng.choice([2, 3, 4, 5]), rng.choice([32, 64, 100, 128, 192, 260])
        info = (kind, dtype, B, H, P, s, D, causal, groups)
        q, k, v = (mk(B, P * s, H, D) for _ in range(3))
        want_o, want_l = O.full_attention(q, k, v, None, causal)
        flags = ops.RingFlags(P, torch.device(DEV))
        flags.set_all()
        o, l = ops.ring_fwd_flags(q.to(DEV), k.to(DEV), v.to(DEV), P, flags, None, causal)
        _close("out", o, want_o, atol, rtol, info)
        _close("lse", l, want_l, LSE_ATOL, 0, info)
        assert not flags.failed(), info
        return
    if kind == "block":
        Sq = rng.choice([1, 2, 3, 7, 64, 65, 127, 128, 129, 200, 256, 300, 513, 700])
        Sk = rng.choice([1, 3, 64, 65, 128, 130, 255, 256, 400, 769])
        split = rng.choice(["auto", "auto", 2, 3, 5])   # keys cut into chunks that run side by side (calls without a mask, 16-bit, D >= 64)
        info = (kind, dtype, B, H, Sq, Sk, D, causal, share, groups, split)
        q, k, v = mk(B, H, Sq, D), mk(B, H, Sk, D), mk(B, H, Sk, D)
        want_o, want_l = O.attn_block(q, k, v, None, causal)
        o, l = ops.flash_fwd(q.to(DEV), k.to(DEV), v.to(DEV), None, causal, layout="bhsd", split_kv=split)
        _close("out", o, want_o, atol, rtol, info)
        _close("lse", l, want_l, LSE_ATOL, 0, info)
    elif kind == "ring":
        P, s, fuse = rng.choice([2, 3, 4, 5]), rng.choice([32, 64, 100, 128, 192, 260]), rng.choice(["step", "rank", "all"])
        info = (kind, dtype, B, H, P, s, D, causal, fuse, share, groups)
        q, k, v = (mk(B, P * s, H, D) for _ in range(3))
        want_o, want_l = O.full_attention(q, k, v, None, causal)
        o, l = spa.ring.ring_flash_attn_forward(q.to(DEV), k.to(DEV), v.to(DEV), None, causal, P, fuse=fuse)
        _close("out", o, want_o, atol, rtol, info)
        _close("lse", l, want_l, LSE_ATOL, 0, info)
    elif kind == "zigzag":
        P, hc, fuse = rng.choice([2, 3, 4, 5]), rng.choice([8, 32, 50, 64, 96, 100, 128, 130]), rng.choice(["step", "rank", "all"])
        info = (kind, dtype, B, H, P, hc, D, fuse, share, groups)
        q, k, v = (mk(B, 2 * P * hc, H, D) for _ in range(3))
        idx = O.zigzag_order(2 * P * hc, P)
        want_o, want_l = O.full_attention(q, k, v, None, True)
        o, l = spa.ring.ring_flash_attn_forward(q[:, idx].to(DEV), k[:, idx].to(DEV), v[:, idx].to(DEV), None, True, P, fuse=fuse,
                                                sharding="zigzag")
        _close("out", o, want_o[:, idx], atol, rtol, info)
        _close("lse", l, want_l[:, :, idx], LSE_ATOL, 0, info)
    elif kind == "ring_bwd":
        S = rng.choice([2, 33, 64, 100, 128, 200, 257, 384])
        P = rng.choice([1, 1, 2, 4]) if S % 4 == 0 else 1
        info = (kind, dtype, B, H, S, D, causal, P)
        q, k, v, do = (mk(B, S, H, D) for _ in range(4))
        want = O.attn_backward_autograd(q, k, v, do, None, causal)
        xs = [t.to(DEV).requires_grad_(True) for t in (q, k, v)]
        spa.ring_flash_attn_func(*xs, causal=causal, ring_size=P).backward(do.to(DEV))
        _grads_close([x.grad for x in xs], want, dtype, info)
    elif kind == "block_bwd":
        Sq = rng.choice([2, 33, 64, 100, 128, 130, 257, 300])
        Sk = rng.choice([2, 40, 64, 128, 129, 200, 260, 384, 520])
        info = (kind, dtype, B, H, Sq, Sk, D, causal)
        q, do, k, v = mk(B, Sq, H, D), mk(B, Sq, H, D), mk(B, Sk, H, D), mk(B, Sk, H, D)
        want = O.attn_backward_autograd(q, k, v, do, None, causal)
        qd, kd, vd, dd = (t.to(DEV) for t in (q, k, v, do))
        o, l = ops.flash_fwd(qd, kd, vd, None, causal, layout="bshd")
        delta = ops.bwd_delta(o, dd, layout="bshd")
        poison = [torch.full(t.shape, float("nan"), dtype=dtype, device=DEV) for t in (q, k, v)]
        got = ops.flash_bwd_out(qd, kd, vd, dd, l, delta, None, causal, layout="bshd", dq=poison[0], dk=poison[1], dv=poison[2])
        _grads_close(got, want, dtype, info)
    elif kind == "varlen_bwd":
        ns = rng.choice([1, 2, 4])
        lq = [rng.choice([0, 1, 5, 64, 100, 129, 200]) for _ in range(ns)]
        lk = [rng.choice([0, 2, 40, 64, 130, 260]) for _ in range(ns)]
        if sum(lq) == 0 or sum(lk) == 0:
            return
        info = (kind, dtype, lq, lk, H, D, causal)
        q, do, k, v = mk(sum(lq), H, D), mk(sum(lq), H, D), mk(sum(lk), H, D), mk(sum(lk), H, D)
        xs = [t.to(DEV).requires_grad_(True) for t in (q, k, v)]
        spa.sp_aurora_varlen_func(*xs, _cu(lq).to(DEV), _cu(lk).to(DEV), causal=causal).backward(do.to(DEV))
        q0 = k0 = 0
        for a, b in zip(lq, lk):
            qs, ks = slice(q0, q0 + a), slice(k0, k0 + b)
            if a and b:
                want = O.attn_backward_autograd(q[None, qs], k[None, ks], v[None, ks], do[None, qs], None, causal)
                _grads_close((xs[0].grad[qs], xs[1].grad[ks], xs[2].grad[ks]), [w[0] for w in want], dtype, info)
            else:  # nothing attends, or nothing is attended to
                assert not (xs[0].grad[qs].any() or xs[1].grad[ks].any() or xs[2].grad[ks].any()), f"nonzero gradient: {info}"
            q0 += a
            k0 += b
    elif kind == "fp8":
        Sq, Sk = rng.choice([1, 64, 100, 128, 256, 300]), rng.choice([1, 64, 65, 128, 200, 513])
        info = (kind, dtype, B, H, Sq, Sk, D, causal, share, groups)
        q, kf, vf = mk(B, H, Sq, D), mk(B, H, Sk, D, dt=torch.float32), mk(B, H, Sk, D, dt=torch.float32)
        k8, ks = ops.quantize_fp8_per_head(kf, "bhsd")
        v8, vs = ops.quantize_fp8_per_head(vf, "bhsd")
        want_o, want_l = O.attn_block(q, k8.double() * ks[:, :, None, None].double(), v8.double() * vs[:, :, None, None].double(), None, causal)
        o, l = ops.flash_fwd(q.to(DEV), k8.to(DEV), v8.to(DEV), None, causal, layout="bhsd", k_scale=ks, v_scale=vs)
        _close("out", o, want_o, atol, rtol, info)
        _close("lse", l, want_l, LSE_ATOL, 0, info)
    elif kind == "fp8_ring":
        P, s, fuse = rng.choice([2, 3, 4]), rng.choice([64, 100, 128, 256, 260]), rng.choice(["step", "rank", "all"])
        info = (kind, dtype, B, H, P, s, D, causal, fuse, share, groups)
        q, kf, vf = mk(B, P * s, H, D), mk(B, P * s, H, D, dt=torch.float32), mk(B, P * s, H, D, dt=torch.float32)
        k8, ks = ops.quantize_fp8_per_head(kf, "bshd")
        v8, vs = ops.quantize_fp8_per_head(vf, "bshd")
        want_o, want_l = O.full_attention(q, k8.double() * ks[:, None, :, None].double(), v8.double() * vs[:, None, :, None].double(), None, causal)
        o, l = ops.ring_fwd(q.to(DEV), k8.to(DEV), v8.to(DEV), ring_size=P, causal=causal, rank=-1, fuse=fuse, k_scale=ks, v_scale=vs)
        _close("out", o, want_o, atol, rtol, info)
        _close("lse", l, want_l, LSE_ATOL, 0, info)
    elif kind == "varlen_decode":   # up to three query rows per sequence against caches of different lengths, no mask
        ns = rng.choice([1, 3, 6])
        lq = [rng.choice([0, 1, 1, 2, 3]) for _ in range(ns)]
        lk = [rng.choice([0, 1, 7, 64, 130, 515, 1100]) for _ in range(ns)]
        if sum(lq) == 0 or sum(lk) == 0:
            return
        info = (kind, dtype, lq, lk, H, D)
        q, k, v = mk(sum(lq), H, D), mk(sum(lk), H, D), mk(sum(lk), H, D)
        o, l = ops.flash_fwd_varlen(q.to(DEV), k.to(DEV), v.to(DEV), _cu(lq).to(DEV), _cu(lk).to(DEV), max(lq), max(lk), None, False)
        q0 = k0 = 0
        for a, b in zip(lq, lk):
            if a and b:
                wo, wl = O.full_attention(q[None, q0:q0 + a], k[None, k0:k0 + b], v[None, k0:k0 + b], None, False)
                _close("out", o[q0:q0 + a], wo[0], atol, rtol, info)
                _close("lse", l[:, q0:q0 + a], wl[0], LSE_ATOL, 0, info)
            elif a:
                assert not o[q0:q0 + a].any() and bool(torch.isneginf(l[:, q0:q0 + a]).all()), f"a sequence without keys: {info}"
            q0 += a
            k0 += b
    else:  # varlen forward, every sequence attending to itself
        lens = [rng.choice([1, 5, 64, 100, 129, 200]) for _ in range(rng.choice([1, 2, 4]))]
        info = (kind, dtype, lens, H, D, causal, share, groups)
        q, k, v = (mk(sum(lens), H, D) for _ in range(3))
        outs, lses, r0 = [], [], 0
        for ln in lens:
            o1, l1 = O.full_attention(q[None, r0:r0 + ln], k[None, r0:r0 + ln], v[None, r0:r0 + ln], None, causal)
            outs.append(o1[0])
            lses.append(l1[0])
            r0 += ln
        cu = _cu(lens).to(DEV)
        o, l = ops.flash_fwd_varlen(q.to(DEV), k.to(DEV), v.to(DEV), cu, cu, max(lens), max(lens), None, causal)
        _close("out", o, torch.cat(outs, 0), atol, rtol, info)
        _close("lse", l, torch.cat(lses, 1), LSE_ATOL, 0, info)


def test_fixed_seed_sweep_of_random_shapes_against_the_oracle():
    rng = random.Random(SEED)
    try:
        for _ in range(N_CASES):
            _case(rng)
        torch.cuda.synchronize()
    finally:
        _lib.tune("fwd_share", 0)
        _lib.tune("fwd_groups", 0)
        _lib.tune("fwd32_split", 0)
        _lib.tune("few_rows", 0)
