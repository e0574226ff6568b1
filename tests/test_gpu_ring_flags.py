"""One launch per rank for a ring whose KV chunks arrive while the launch runs (spa_ring_fwd_flags): with the flags
raised beforehand the result is that of the plain one-launch form, bit for bit; with a second stream filling the
receive buffer and raising the flags while the kernel runs it is still that result; with flags that never come every
wave gives up at its spin limit, the launch ends and the fault word says so."""
import time

import pytest
import torch

from conftest import rand_qkv
from oracle import attn_oracle as O
from sp_aurora_amd import ops
from test_gpu_parity import DEV, check_lse, check_out

pytestmark = pytest.mark.gpu


def independent_stream():
    """A stream whose work runs while a kernel on the current stream waits.  Streams share a few hardware queues; a
    producer queued behind the waiting kernel on the same queue would only run once that kernel has given up.  Probed
    with a tiny launch and a short spin limit: the flag of its second chunk is raised on the candidate stream."""
    q, k, v = (t.to(DEV) for t in rand_qkv((1, 256, 1, 64), 899, torch.bfloat16))
    for _ in range(8):
        cand = torch.cuda.Stream()
        flags = ops.RingFlags(2, q.device)
        flags.set(1)
        torch.cuda.synchronize()
        ops.ring_fwd_flags(q, k, v, 2, flags, None, True, rank=1, spin_limit=40000)
        flags.set(0, stream=cand)
        torch.cuda.synchronize()
        if not flags.failed():
            return cand
    pytest.skip("no stream on a hardware queue of its own")


@pytest.mark.parametrize("B,H,P,s,D,dtype,causal", [
    (1, 4, 4, 256, 128, torch.bfloat16, True),
    (2, 2, 3, 100, 64, torch.float16, True),
    (1, 2, 4, 64, 128, torch.bfloat16, False),     # one wave group per workgroup
    (1, 32, 8, 1024, 128, torch.bfloat16, True),   # benchmark config 3
])
def test_flags_raised_beforehand_give_the_one_launch_result(B, H, P, s, D, dtype, causal):
    q, k, v = (t.to(DEV) for t in rand_qkv((B, P * s, H, D), 800, dtype, 0.5))
    want_o, want_l = ops.ring_fwd(q, k, v, P, None, causal, fuse="rank")
    flags = ops.RingFlags(P, q.device)
    flags.set_all()
    out, lse = ops.ring_fwd_flags(q, k, v, P, flags, None, causal)
    torch.cuda.synchronize()
    assert not flags.failed()
    assert torch.equal(out, want_o) and torch.equal(lse, want_l)
    # a new round on the same flag array: nothing raised yet for the new epoch, a tiny spin limit -> every wave gives up
    flags.next_epoch()
    ops.ring_fwd_flags(q, k, v, P, flags, None, causal, spin_limit=4)
    torch.cuda.synchronize()
    assert flags.failed()


def test_chunks_that_arrive_while_the_launch_runs():
    """Rank P-1 of a causal ring: its own chunk is there, the others are copied into a poisoned receive buffer by a second
    stream, each followed by its flag, while the rank's launch is already running and waiting."""
    B, H, P, s, D, dtype = 1, 8, 4, 512, 128, torch.bfloat16
    r = P - 1
    q, k, v = (t.to(DEV) for t in rand_qkv((B, P * s, H, D), 801, dtype, 0.5))
    (qc, kc, vc) = (t.cpu() for t in (q, k, v))
    want_o, want_l = O.full_attention(qc, kc, vc, None, True)
    rows = slice(r * s, (r + 1) * s)
    kbuf, vbuf = torch.full_like(k, float("nan")), torch.full_like(v, float("nan"))
    kbuf[:, rows], vbuf[:, rows] = k[:, rows], v[:, rows]
    flags = ops.RingFlags(P, q.device)
    out = torch.zeros_like(q)
    lse = torch.zeros((B, H, P * s), dtype=torch.float32, device=DEV)
    comm = independent_stream()
    torch.cuda.synchronize()
    flags.set(r)                                     # the rank's own chunk
    ops.ring_fwd_flags(q, kbuf, vbuf, P, flags, None, True, rank=r, out=out, lse=lse, spin_limit=1 << 21)
    with torch.cuda.stream(comm):
        for c in range(r - 1, -1, -1):               # ring order: chunk r-1 lands first
            time.sleep(0.002)
            cs = slice(c * s, (c + 1) * s)
            kbuf[:, cs].copy_(k[:, cs])
            vbuf[:, cs].copy_(v[:, cs])
            flags.set(c, stream=comm)
    torch.cuda.synchronize()
    assert not flags.failed(), "a wave gave up waiting for a chunk"
    check_out(out[:, rows], want_o[:, rows], dtype)
    check_lse(lse[:, :, rows], want_l[:, :, rows])
    assert not out[:, :r * s].any()


def test_flag_entry_refuses_what_it_is_not_built_for():
    from sp_aurora_amd import _lib
    q, k, v = (t.to(DEV) for t in rand_qkv((1, 256, 2, 32), 802, torch.bfloat16))
    flags = ops.RingFlags(2, q.device)
    with pytest.raises(_lib.SpaError):   # head dim 32
        ops.ring_fwd_flags(q, k, v, 2, flags, None, True)
    q, k, v = (t.to(DEV) for t in rand_qkv((1, 256, 2, 64), 803, torch.float32))
    with pytest.raises(_lib.SpaError):   # fp32
        ops.ring_fwd_flags(q, k, v, 2, flags, None, True)
    qb, kb, vb = (t.bfloat16() for t in (q, k, v))
    pad = torch.zeros(kb.numel() + 64, dtype=torch.bfloat16, device=DEV)
    k_off = pad[32:32 + kb.numel()].view_as(kb).copy_(kb)      # 64 bytes off a line boundary
    with pytest.raises(_lib.SpaError):   # a cache line would hold bytes of two chunks
        ops.ring_fwd_flags(qb, k_off, vb, 2, flags, None, True)
    with pytest.raises(ValueError):      # one flag per chunk
        ops.ring_fwd_flags(q.bfloat16(), k.bfloat16(), v.bfloat16(), 4, flags, None, True)


@pytest.mark.parametrize("B,H,P,s,causal", [(1, 4, 4, 256, True), (2, 2, 3, 100, True), (1, 2, 2, 64, False), (1, 32, 8, 256, True)])
def test_e4m3_tensors_with_flags(B, H, P, s, causal):
    """spa_ring_fwd_flags_fp8qkv: flags raised beforehand give the bits of the e4m3 ring's one-launch-per-rank form; with a
    second stream filling a zeroed receive buffer while the last rank's launch waits, the rows are those of the oracle's
    attention on the dequantised tensors."""
    from test_gpu_fp8kv import quantised
    D, S = 128, P * s
    q8, qsc, q_deq = quantised((B, S, H, D), 840, "bshd", spread=1.2)
    k8, ksc, k_deq = quantised((B, S, H, D), 841, "bshd", spread=1.5)
    v8, vsc, v_deq = quantised((B, S, H, D), 842, "bshd", spread=0.7)
    q8, k8, v8 = q8.to(DEV), k8.to(DEV), v8.to(DEV)
    scales = dict(q_scale=qsc, k_scale=ksc, v_scale=vsc)
    want_o, want_l = ops.ring_fwd(q8, k8, v8, P, None, causal, fuse="rank", **scales)
    flags = ops.RingFlags(P, q8.device)
    flags.set_all()
    out, lse = ops.ring_fwd_flags(q8, k8, v8, P, flags, None, causal, **scales)
    torch.cuda.synchronize()
    assert not flags.failed()
    assert torch.equal(out, want_o) and torch.equal(lse, want_l)
    if not causal or (s * D) % 128:
        return
    # chunks that land while rank P - 1 runs (zeros before: e4m3 has no NaN-free poison that survives a wrong read unseen,
    # so the check is the comparison with the oracle)
    r = P - 1
    oracle_o, oracle_l = O.full_attention(q_deq, k_deq, v_deq, None, True)
    rows = slice(r * s, (r + 1) * s)
    kbuf, vbuf = torch.zeros_like(k8), torch.zeros_like(v8)
    kbuf[:, rows], vbuf[:, rows] = k8[:, rows], v8[:, rows]
    flags.next_epoch()
    out2 = torch.zeros((B, S, H, D), dtype=torch.bfloat16, device=DEV)
    lse2 = torch.zeros((B, H, S), dtype=torch.float32, device=DEV)
    comm = independent_stream()
    torch.cuda.synchronize()
    flags.set(r)
    ops.ring_fwd_flags(q8, kbuf, vbuf, P, flags, None, True, rank=r, out=out2, lse=lse2, spin_limit=1 << 21, **scales)
    with torch.cuda.stream(comm):
        for c in range(r - 1, -1, -1):
            time.sleep(0.002)
            cs = slice(c * s, (c + 1) * s)
            kbuf[:, cs].copy_(k8[:, cs])
            vbuf[:, cs].copy_(v8[:, cs])
            flags.set(c, stream=comm)
    torch.cuda.synchronize()
    assert not flags.failed(), "a wave gave up waiting for a chunk"
    check_out(out2[:, rows], oracle_o[:, rows], torch.bfloat16)
    check_lse(lse2[:, :, rows], oracle_l[:, :, rows])
