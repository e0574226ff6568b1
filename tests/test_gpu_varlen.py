"""GPU parity of attention over packed variable-length batches: every sequence of the packed
batch must come out as the oracle's attention of that sequence alone (forward, lse, gradients).
The sequence-length patterns of the reference's own test come first
(test/flash_attention/test_intel_ring_flash_attn_varlen.py:42-48,146)."""
import pytest
import torch

from conftest import rand
from oracle import attn_oracle as O
import sp_aurora_amd as spa
from sp_aurora_amd import ops
from test_gpu_parity import DEV, check_grad, check_lse, check_out

pytestmark = pytest.mark.gpu


def cu_of(lengths):
    return torch.tensor([0] + list(torch.tensor(lengths).cumsum(0)), dtype=torch.int32)


def per_sequence(q, k, v, lens_q, lens_k, causal):
    """Oracle attention of each sequence alone -> packed out [Tq,H,D], lse [H,Tq]."""
    outs, lses = [], []
    q0 = k0 = 0
    for lq, lk in zip(lens_q, lens_k):
        if lq == 0:
            k0 += lk
            continue
        if lk == 0:
            outs.append(torch.zeros(lq, q.shape[1], q.shape[2], dtype=torch.float64))
            lses.append(torch.full((q.shape[1], lq), float("-inf"), dtype=torch.float64))
        else:
            o, l = O.full_attention(q[None, q0:q0 + lq], k[None, k0:k0 + lk], v[None, k0:k0 + lk], None, causal)
            outs.append(o[0])
            lses.append(l[0])
        q0 += lq
        k0 += lk
    return torch.cat(outs, 0), torch.cat(lses, 1)


SELF_CASES = [
    # lengths, H, D, dtype, causal
    ([128, 256, 128], 8, 64, torch.float16, True),        # "Mixed lengths"
    ([100, 100, 100, 100], 8, 64, torch.float16, True),   # "Equal lengths"
    ([512], 8, 64, torch.float16, True),                  # "Single sequence"
    ([64, 128, 256, 512], 8, 64, torch.float16, True),    # "Increasing lengths"
    ([128, 256, 128, 192], 8, 64, torch.float16, True),   # the distributed test's batch
    ([1, 77, 300, 5, 129], 3, 128, torch.bfloat16, False),
    ([1, 77, 300, 5, 129], 3, 128, torch.bfloat16, True),
    ([33, 1, 64, 200], 2, 32, torch.bfloat16, True),
    ([40, 130, 7], 2, 64, torch.float32, True),
    ([40, 130, 7], 2, 128, torch.float32, False),
]


@pytest.mark.parametrize("lengths,H,D,dtype,causal", SELF_CASES)
def test_varlen_forward_and_backward_match_per_sequence_attention(lengths, H, D, dtype, causal):
    T = sum(lengths)
    q, k, v, dout = (rand((T, H, D), 400 + i, dtype) for i in range(4))
    want_out, want_lse = per_sequence(q, k, v, lengths, lengths, causal)
    cu = cu_of(lengths).to(DEV)
    xs = [t.to(DEV).requires_grad_(True) for t in (q, k, v)]
    out, lse, _ = spa.sp_aurora_varlen_func(*xs, cu, cu, max_seqlen=max(lengths), dropout_p=0.0, causal=causal,
                                            return_attn_probs=True)
    assert out.shape == (T, H, D) and out.dtype == dtype and lse.shape == (H, T)
    check_out(out, want_out, dtype)
    check_lse(lse, want_lse)
    out.backward(dout.to(DEV))
    s0 = 0
    for n in lengths:
        sl = slice(s0, s0 + n)
        want = O.attn_backward_autograd(q[None, sl], k[None, sl], v[None, sl], dout[None, sl], None, causal)
        for x, w, name in zip(xs, want, "qkv"):
            if n == 1 and name in "qk":
                # a single key: the softmax is constant, dq = dk = 0 exactly; rounding of P - 1 remains
                assert w.abs().max() < 1e-12 and x.grad[sl].abs().max() < 1e-5
                continue
            check_grad(x.grad[sl], w[0], dtype, f"d{name} of the sequence at {s0}")
        s0 += n


@pytest.mark.parametrize("causal", [False, True])
def test_varlen_with_different_query_and_key_lengths_and_empty_sequences(causal):
    lens_q = [50, 0, 130, 20, 64]
    lens_k = [70, 40, 0, 300, 10]
    H, D, dtype = 2, 64, torch.bfloat16
    q = rand((sum(lens_q), H, D), 410, dtype)
    k, v = rand((sum(lens_k), H, D), 411, dtype), rand((sum(lens_k), H, D), 412, dtype)
    dout = rand((sum(lens_q), H, D), 413, dtype)
    want_out, want_lse = per_sequence(q, k, v, lens_q, lens_k, causal)
    xs = [t.to(DEV).requires_grad_(True) for t in (q, k, v)]
    out, lse, _ = spa.sp_aurora_varlen_func(*xs, cu_of(lens_q).to(DEV), cu_of(lens_k).to(DEV), causal=causal,
                                            return_attn_probs=True)
    check_out(out, want_out, dtype)
    got_lse = lse.cpu().double()
    finite = torch.isfinite(want_lse)
    assert torch.equal(torch.isneginf(got_lse), torch.isneginf(want_lse))
    assert (got_lse[finite] - want_lse[finite]).abs().max() <= 1e-3
    out.backward(dout.to(DEV))
    q0 = k0 = 0
    for lq, lk in zip(lens_q, lens_k):
        qs, ks = slice(q0, q0 + lq), slice(k0, k0 + lk)
        if lq and lk:
            want = O.attn_backward_autograd(q[None, qs], k[None, ks], v[None, ks], dout[None, qs], None, causal)
            check_grad(xs[0].grad[qs], want[0][0], dtype, "dq")
            check_grad(xs[1].grad[ks], want[1][0], dtype, "dk")
            check_grad(xs[2].grad[ks], want[2][0], dtype, "dv")
        else:  # nothing attends, or nothing is attended to
            assert not xs[0].grad[qs].any() and not xs[1].grad[ks].any() and not xs[2].grad[ks].any()
        q0 += lq
        k0 += lk


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("D,causal", [(64, True), (128, False), (32, True)])
def test_varlen_backward_written_in_the_inputs_type_equals_accumulate_then_cast(D, causal, dtype):
    """spa_flash_bwd_varlen_out against spa_flash_bwd_varlen into zeroed fp32 accumulators followed
    by the cast, bit for bit, into buffers that start out poisoned: every row of every sequence must
    be written, with zeros where a sequence has no keys or keys that no query sees."""
    lens_q = [50, 0, 130, 20, 64, 300]
    lens_k = [70, 40, 0, 300, 10, 300]
    H = 2
    Tq, Tk = sum(lens_q), sum(lens_k)
    q, dout = (rand((Tq, H, D), 430 + i, dtype).to(DEV) for i in range(2))
    k, v = (rand((Tk, H, D), 432 + i, dtype).to(DEV) for i in range(2))
    cu_q, cu_k = cu_of(lens_q).to(DEV), cu_of(lens_k).to(DEV)
    out, lse = ops.flash_fwd_varlen(q, k, v, cu_q, cu_k, max(lens_q), max(lens_k), None, causal)
    delta = ops.bwd_delta(out.unsqueeze(0), dout.unsqueeze(0), layout="bshd")[0]
    acc = [torch.zeros(t.shape, dtype=torch.float32, device=DEV) for t in (q, k, v)]
    ops.flash_bwd_varlen(q, k, v, dout, lse, delta, *acc, cu_q, cu_k, max(lens_q), max(lens_k), None, causal)
    want = [a.to(dtype) for a in acc]
    # gradients written into the halves of packed buffers (row stride 2 H D) that hold a marker value
    pq = torch.full((Tq, 2, H, D), 7.0, dtype=dtype, device=DEV)
    pkv = torch.full((Tk, 2, H, D), 7.0, dtype=dtype, device=DEV)
    ops.flash_bwd_varlen_out(q, k, v, dout, lse, delta, cu_q, cu_k, max(lens_q), max(lens_k), None, causal,
                             dq=pq[:, 1], dk=pkv[:, 0], dv=pkv[:, 1])
    for gt, w, name in zip((pq[:, 1], pkv[:, 0], pkv[:, 1]), want, "qkv"):
        assert torch.equal(gt, w), f"d{name}"
    assert (pq[:, 0] == 7.0).all()
    with pytest.raises(TypeError):
        ops.flash_bwd_varlen_out(q, k, v, dout, lse, delta, cu_q, cu_k, max(lens_q), max(lens_k), None, causal,
                                 dq=torch.empty(q.shape, dtype=torch.float64, device=DEV))
    with pytest.raises(ValueError):
        ops.flash_bwd_varlen_out(q, k, v, dout, lse, delta, cu_q, cu_k, max(lens_q), max(lens_k), None, causal,
                                 dk=torch.empty_like(k[:1]))


DECODE_CASES = [
    # query rows per sequence, keys per sequence, H, D, dtype
    ([1, 1, 1, 1, 1], [700, 1, 33, 1300, 64], 4, 128, torch.bfloat16),     # one new token per sequence, ragged caches
    ([1, 3, 0, 2, 1], [100, 515, 40, 0, 257], 3, 64, torch.float16),       # a sequence without queries, one without keys
    ([2, 2, 2], [4096, 5, 130], 2, 128, torch.float16),
    ([3, 1], [70, 900], 5, 64, torch.bfloat16),
]


@pytest.mark.parametrize("lens_q,lens_k,H,D,dtype", DECODE_CASES)
def test_varlen_few_query_rows_against_ragged_caches(lens_q, lens_k, H, D, dtype):
    """Sequences of up to three query rows without a mask run on the kernel that streams K and V (spa_tune few_rows = 1:
    the matrix-instruction kernels); both against the oracle's attention of each sequence alone, bf16 / fp16 and e4m3 K/V."""
    from sp_aurora_amd import _lib
    Tq, Tk = sum(lens_q), sum(lens_k)
    q, k, v = rand((Tq, H, D), 470, dtype), rand((Tk, H, D), 471, dtype), rand((Tk, H, D), 472, dtype)
    want_out, want_lse = per_sequence(q, k, v, lens_q, lens_k, False)
    cq, ck = cu_of(lens_q).to(DEV), cu_of(lens_k).to(DEV)
    k8, ksc = ops.quantize_fp8_per_head(k[None].float())
    v8, vsc = ops.quantize_fp8_per_head(v[None].float())
    nseq = len(lens_q)
    ksc, vsc = ksc.expand(nseq, H).contiguous(), vsc.expand(nseq, H).contiguous()   # one scale per head for every sequence
    k_deq = (k8[0].float() * ksc[0][None, :, None]).to(dtype)
    v_deq = (v8[0].float() * vsc[0][None, :, None]).to(dtype)
    want8_out, want8_lse = per_sequence(q, k_deq, v_deq, lens_q, lens_k, False)

    def lse_ok(got_lse, want):   # (a sequence without keys: lse = -inf)
        got_lse, fin = got_lse.cpu().double(), torch.isfinite(want)
        assert torch.equal(torch.isneginf(got_lse), torch.isneginf(want))
        assert (got_lse[fin] - want[fin]).abs().max() <= 1e-3

    got = {}
    try:
        for knob in (0, 1):
            _lib.tune("few_rows", knob)
            out = torch.full((Tq, H, D), 7.0, dtype=dtype, device=DEV)
            lse = torch.full((H, Tq), 7.0, dtype=torch.float32, device=DEV)
            ops.flash_fwd_varlen(q.to(DEV), k.to(DEV), v.to(DEV), cq, ck, max(lens_q), max(lens_k), None, False, out=out, lse=lse)
            check_out(out, want_out, dtype, f"knob {knob}")
            lse_ok(lse, want_lse)
            got[knob] = lse
            o8, l8 = ops.flash_fwd_varlen(q.to(DEV), k8[0].to(DEV), v8[0].to(DEV), cq, ck, max(lens_q), max(lens_k), None, False,
                                          k_scale=ksc.to(DEV), v_scale=vsc.to(DEV))
            check_out(o8, want8_out, dtype, f"e4m3 knob {knob}")
            lse_ok(l8, want8_lse)
    finally:
        _lib.tune("few_rows", 0)
    both = torch.isfinite(got[0]) & torch.isfinite(got[1])
    assert torch.equal(torch.isfinite(got[0]), torch.isfinite(got[1])) and (got[0][both] - got[1][both]).abs().max().item() < 1e-4


def test_varlen_large_batch_matches_the_fixed_length_kernels():
    """Enough workgroups for the shared-buffer forward variant; equal lengths make the padded
    batch call a second opinion, the ragged tail a check that short sequences leave their
    neighbours' rows alone."""
    H, D, dtype = 16, 128, torch.bfloat16
    lengths = [1024] * 8 + [1000, 24]
    T = sum(lengths)
    q, k, v = (rand((T, H, D), 420 + i, dtype).to(DEV) for i in range(3))
    cu = cu_of(lengths).to(DEV)
    out, lse = ops.flash_fwd_varlen(q, k, v, cu, cu, 1024, 1024, None, True)
    ref_out, ref_lse = ops.flash_fwd(q[:8192].view(8, 1024, H, D), k[:8192].view(8, 1024, H, D),
                                     v[:8192].view(8, 1024, H, D), None, True)
    assert torch.equal(out[:8192].view(8, 1024, H, D), ref_out)
    assert torch.equal(lse[:, :8192].view(H, 8, 1024).transpose(0, 1), ref_lse)
    for s0, n in ((8192, 1000), (9192, 24)):
        o, l = ops.flash_fwd(q[None, s0:s0 + n], k[None, s0:s0 + n], v[None, s0:s0 + n], None, True)
        check_out(out[s0:s0 + n], o[0].cpu(), dtype)
        assert (lse[:, s0:s0 + n] - l[0]).abs().max() <= 1e-3


def test_varlen_lse_helpers_round_trip():
    """flatten_varlen_lse / unflatten_varlen_lse (sp_aurora/utils.py:150-169) against the packed lse."""
    lengths, H, D = [30, 64, 7], 2, 64
    T = sum(lengths)
    q, k, v = (rand((T, H, D), 430 + i, torch.bfloat16).to(DEV) for i in range(3))
    cu = cu_of(lengths).to(DEV)
    _, lse, _ = spa.sp_aurora_varlen_func(q, k, v, cu, cu, max_seqlen=64, causal=True, return_attn_probs=True)
    padded = spa.unflatten_varlen_lse(lse.t().unsqueeze(-1), cu, 64)     # [nseq, H, max]
    assert padded.shape == (3, H, 64)
    assert torch.equal(spa.flatten_varlen_lse(padded, cu), lse)


def test_varlen_offsets_are_read_on_the_host_once_per_array():
    """The first call with a cu_seqlens array validates it (a blocking device-to-host read); later calls
    with the same array, with max_seqlen given, must not synchronise with the device at all - and a changed
    array is looked at again."""
    lengths, H, D = [30, 64, 7], 2, 64
    T = sum(lengths)
    q, k, v = (rand((T, H, D), 440 + i, torch.bfloat16).to(DEV) for i in range(3))
    cu = cu_of(lengths).to(DEV)
    first = spa.sp_aurora_varlen_func(q, k, v, cu, cu, max_seqlen=64, causal=True)
    torch.cuda.synchronize()
    torch.cuda.set_sync_debug_mode("error")
    try:
        again = spa.sp_aurora_varlen_func(q, k, v, cu, cu, max_seqlen=64, causal=True)
        unchecked = spa.sp_aurora_varlen_func(q, k, v, cu.clone(), None, max_seqlen=64, causal=True, check_offsets=False)
    finally:
        torch.cuda.set_sync_debug_mode("default")
    assert torch.equal(first, again) and torch.equal(first, unchecked)
    cu[-1] = T - 1  # in place: same address, new version counter
    with pytest.raises(ValueError):
        spa.sp_aurora_varlen_func(q, k, v, cu, cu, max_seqlen=64, causal=True)


def test_varlen_backward_leaves_zeros_in_rows_of_no_sequence():
    """Direct callers of ops.flash_bwd_varlen_out may pass offsets that end before the tensors do: the
    gradients allocated by the wrapper are zero there (the kernels do not touch such rows)."""
    lengths, H, D, dtype = [40, 24], 2, 64, torch.bfloat16
    used, T = sum(lengths), sum(lengths) + 19
    q, k, v, dout = (rand((T, H, D), 450 + i, dtype).to(DEV) for i in range(4))
    cu = cu_of(lengths).to(DEV)
    out, lse = ops.flash_fwd_varlen(q, k, v, cu, cu, 40, 40, None, True, out=torch.zeros_like(q),
                                    lse=torch.zeros((H, T), dtype=torch.float32, device=DEV))
    delta = ops.bwd_delta(out.unsqueeze(0), dout.unsqueeze(0), layout="bshd")[0]
    junk = torch.full((64 << 20,), 1e30, dtype=torch.float32, device=DEV)  # what a recycled allocation may hold
    del junk
    dq, dk, dv = ops.flash_bwd_varlen_out(q, k, v, dout, lse, delta, cu, cu, 40, 40, None, True)
    for g in (dq, dk, dv):
        assert not g[used:].any() and g[:used].float().abs().max() > 0


@pytest.mark.parametrize("P,local_lengths,H,D,dtype,causal", [
    (2, [64, 128, 32], 2, 64, torch.bfloat16, True),
    (4, [32, 96, 64, 48], 8, 64, torch.float16, True),     # the distributed test's batch, every sequence cut in four
    (3, [50, 7, 130], 2, 128, torch.bfloat16, True),
    (2, [100, 40], 2, 64, torch.float32, True),
    (3, [20, 64], 1, 128, torch.bfloat16, False),
])
def test_ring_over_a_packed_batch_matches_per_sequence_attention(P, local_lengths, H, D, dtype, causal):
    """sp_aurora_varlen_func(ring_size=P): rank r holds slice r of every sequence.  Expected: the oracle's attention of
    every WHOLE sequence (P times the local length) alone, re-sliced into the ranks' shards; forward, lse, gradients."""
    T = sum(local_lengths)
    glob_q, glob_k, glob_v, glob_do = [], [], [], []
    want_o, want_l, want_g = [], [], []
    for i, l in enumerate(local_lengths):
        q, k, v, do = (rand((1, P * l, H, D), 460 + 10 * i + j, dtype) for j in range(4))
        o, ls = O.full_attention(q, k, v, None, causal)
        g = O.attn_backward_autograd(q, k, v, do, None, causal)
        glob_q.append(q[0]); glob_k.append(k[0]); glob_v.append(v[0]); glob_do.append(do[0])
        want_o.append(o[0]); want_l.append(ls[0]); want_g.append([x[0] for x in g])
    # shard r = slice r of every sequence, packed in sequence order; the shards stacked
    stack = lambda seqs: torch.cat([torch.cat([s_[r * l:(r + 1) * l] for s_, l in zip(seqs, local_lengths)], 0) for r in range(P)], 0)
    stack_l = lambda seqs: torch.cat([torch.cat([s_[:, r * l:(r + 1) * l] for s_, l in zip(seqs, local_lengths)], 1) for r in range(P)], 1)
    xs = [stack(t).to(DEV).requires_grad_(True) for t in (glob_q, glob_k, glob_v)]
    cu = cu_of(local_lengths).to(DEV)
    out, lse, _ = spa.sp_aurora_varlen_func(*xs, cu, cu, max_seqlen=max(local_lengths), causal=causal, return_attn_probs=True, ring_size=P)
    assert out.shape == (P * T, H, D) and lse.shape == (H, P * T)
    check_out(out, stack(want_o), dtype)
    check_lse(lse, stack_l(want_l))
    out.backward(stack(glob_do).to(DEV))
    for x, j, name in zip(xs, range(3), "qkv"):
        check_grad(x.grad, stack([g[j] for g in want_g]), dtype, "d" + name)
    # the three launch forms (per shard pair with separate merges; one launch per rank; one launch) agree with the oracle,
    # and a single rank writes its rows only
    from sp_aurora_amd import varlen as V
    det = [x.detach() for x in xs]
    for fuse in ("step", "rank", "all"):
        o2, l2 = V.ring_varlen_forward(*det, cu, max(local_lengths), None, causal, P, fuse=fuse)
        check_out(o2, stack(want_o), dtype, fuse)
        check_lse(l2, stack_l(want_l))
    if dtype != torch.float32:
        r = P - 1
        o3 = torch.full_like(det[0], 7.0)
        l3 = torch.full((H, P * T), 7.0, dtype=torch.float32, device=DEV)
        ops.ring_fwd_varlen(*det, cu, max(local_lengths), P, None, causal, rank=r, out=o3, lse=l3)
        assert torch.equal(o3[r * T:], o2[r * T:]) or (o3[r * T:].float() - o2[r * T:].float()).abs().max() < 2e-2
        assert (o3[:r * T] == 7.0).all() and (l3[:, :r * T] == 7.0).all()


@pytest.mark.parametrize("P,local_lengths,H,D,dtype", [
    (2, [64, 128], 2, 64, torch.bfloat16),
    (4, [32, 0, 96, 2], 2, 128, torch.float16),     # an empty sequence and one with a single row per half
    (3, [100, 36], 3, 32, torch.float32),
    (2, [130, 62, 8], 1, 64, torch.bfloat16),
])
def test_zigzag_ring_over_a_packed_batch(P, local_lengths, H, D, dtype):
    """zigzag_sp_aurora_varlen_func(ring_size=P): rank r holds half-slices r and 2P-1-r of every sequence.  Expected: the
    oracle's causal attention of every whole sequence alone, brought into the shards' order; forward, lse, gradients."""
    T = sum(local_lengths)
    seq_lens = [P * l for l in local_lengths]
    parts = {name: [] for name in ("q", "k", "v", "do", "o", "l", "dq", "dk", "dv")}
    for i, n in enumerate(seq_lens):
        q, k, v, do = (rand((1, n, H, D), 560 + 10 * i + j, dtype) for j in range(4))
        if n:
            o, ls = O.full_attention(q, k, v, None, True)
            g = O.attn_backward_autograd(q, k, v, do, None, True)
        else:
            o, ls, g = q.float(), torch.zeros((1, H, 0)), (q.float(), k.float(), v.float())
        for name, t in zip(("q", "k", "v", "do", "o", "dq", "dk", "dv"), (q, k, v, do, o, *g)):
            parts[name].append(t[0])
        parts["l"].append(ls[0])
    idx = spa.zigzag_varlen_order(seq_lens, P)
    nat = {name: torch.cat(ts, 1 if name == "l" else 0) for name, ts in parts.items()}
    xs = [nat[name][idx].to(DEV).requires_grad_(True) for name in "qkv"]
    cu = cu_of(local_lengths).to(DEV)
    out, lse, _ = spa.zigzag_sp_aurora_varlen_func(*xs, cu, cu, max_seqlen=max(local_lengths), causal=True, return_attn_probs=True,
                                                   ring_size=P)
    assert out.shape == (P * T, H, D) and lse.shape == (H, P * T)
    check_out(out, nat["o"][idx], dtype)
    check_lse(lse, nat["l"][:, idx])
    out.backward(nat["do"][idx].to(DEV))
    for x, name in zip(xs, "qkv"):
        check_grad(x.grad, nat["d" + name][idx], dtype, "d" + name)
    # without a mask the sharding does not matter: the contiguous ring's result on the same rows
    a = spa.zigzag_sp_aurora_varlen_func(*[x.detach() for x in xs], cu, cu, max_seqlen=max(local_lengths), causal=False, ring_size=P)
    b = spa.sp_aurora_varlen_func(*[x.detach() for x in xs], cu, cu, max_seqlen=max(local_lengths), causal=False, ring_size=P)
    assert torch.equal(a, b)
    # an odd share of a shard cannot be halved
    if T:
        bad = cu_of([T - 1, 1]).to(DEV)
        with pytest.raises(ValueError):
            spa.zigzag_sp_aurora_varlen_func(*[x.detach() for x in xs], bad, bad, max_seqlen=T, causal=True, ring_size=P)
