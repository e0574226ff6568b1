"""spa_ring_fwd_static — the ring forward for callers that cannot allocate — against spa_ring_fwd.

Both entry points run the same kernels; the only difference is where the earlier block results of a
rank live between step launches (the caller's workspace / the library's built-in buffer).  The
results must therefore be bit-identical, on two calls in a row, the second one smaller (the buffer
keeps the first call's contents).  Called through the C ABI directly.
"""
import ctypes

import pytest
import torch

from conftest import rand_qkv
from sp_aurora_amd import _lib

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
_DT = {torch.float32: _lib.SPA_F32, torch.bfloat16: _lib.SPA_BF16, torch.float16: _lib.SPA_F16}


def _call_pair(B, S, H, D, P, causal, dtype, seed, fuse, rank=-1):
    """(out, lse) of spa_ring_fwd with a caller workspace and of spa_ring_fwd_static."""
    lib = _lib.load()
    q, k, v = [t.to(DEV) for t in rand_qkv((B, S, H, D), seed, dtype)]
    st = _lib.strides3((S * H * D, D, H * D))
    nbytes = lib.spa_ring_fwd_workspace_bytes(B, H, S, D, P, _DT[dtype])
    assert 0 < nbytes <= lib.spa_static_scratch_bytes()
    ws = torch.empty((nbytes,), dtype=torch.uint8, device=DEV)
    res = []
    for static in (False, True):
        out = torch.full((B, S, H, D), float("nan"), dtype=dtype, device=DEV)
        lse = torch.full((B, H, S), float("nan"), dtype=torch.float32, device=DEV)
        torch.cuda.synchronize()
        stream = torch.cuda.current_stream().cuda_stream
        tail = (B, H, S, D, P, rank, st, st, st, st, D ** -0.5, 1 if causal else 0, _DT[dtype], fuse, stream)
        before = torch.cuda.memory_allocated()
        if static:
            rc = lib.spa_ring_fwd_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(), *tail)
        else:
            rc = lib.spa_ring_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(), ws.data_ptr(), *tail)
        assert rc == 0, lib.spa_last_error()
        assert torch.cuda.memory_allocated() == before
        torch.cuda.synchronize()
        res.append((out, lse))
    return res


def _same(a, b, rows=slice(None)):
    """Bit-identical, and every row the call is responsible for (`rows` of the sequence) written:
    the tensors start out as NaN."""
    (out_a, lse_a), (out_b, lse_b) = a, b
    for name, t in (("out", out_a[:, rows]), ("lse", lse_a[:, :, rows]), ("out (static)", out_b[:, rows]),
                    ("lse (static)", lse_b[:, :, rows])):
        n_nan = int(torch.isnan(t.float()).sum())
        assert n_nan == 0, f"{name}: {n_nan} NaN of {t.numel()}"
    bits = torch.int32 if out_a.dtype == torch.float32 else torch.int16
    assert torch.equal(out_a.view(bits), out_b.view(bits))
    assert torch.equal(lse_a.view(torch.int32), lse_b.view(torch.int32))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_static_scratch_matches_caller_workspace_twice_in_a_row(dtype):
    step = _lib.SPA_RING_PER_STEP
    # first call: the larger input; second call: a smaller one over the same (now dirty) buffer
    _same(*_call_pair(1, 2048, 8, 128, 4, True, dtype, 301, step))
    _same(*_call_pair(2, 384, 2, 64, 3, False, dtype, 302, step))
    # one rank only, and a fused schedule that needs no scratch at all
    _same(*_call_pair(1, 1024, 4, 128, 4, True, dtype, 303, step, rank=2), rows=slice(512, 768))
    _same(*_call_pair(1, 1024, 4, 128, 4, True, dtype, 304, _lib.SPA_RING_PER_RANK))


def test_static_scratch_rejects_sizes_beyond_the_buffer():
    lib = _lib.load()
    B, S, H, D, P = 1, 8192, 64, 128, 2   # one block output of a rank: 64 MiB
    assert lib.spa_ring_fwd_workspace_bytes(B, H, S, D, P, _lib.SPA_BF16) > lib.spa_static_scratch_bytes()
    x = torch.empty((16,), dtype=torch.bfloat16, device=DEV)   # never dereferenced: the size check comes first
    st = _lib.strides3((S * H * D, D, H * D))
    p = x.data_ptr()
    rc = lib.spa_ring_fwd_static(p, p, p, p, p, B, H, S, D, P, -1, st, st, st, st, 0.1, 1, _lib.SPA_BF16,
                                 _lib.SPA_RING_PER_STEP, None)
    assert rc == -1 and b"built-in buffer" in lib.spa_last_error()
    torch.cuda.synchronize()


def test_static_scratch_entry_under_graph_capture():
    """What the entry point is for: a per-step ring forward captured in a graph without any
    workspace tensor; every replay (eager work and synchronisations in between) must equal the
    eager result of spa_ring_fwd."""
    from sp_aurora_amd import ops
    B, S, H, D, P = 1, 1024, 4, 128, 4
    q, k, v = (t.to(DEV) for t in rand_qkv((B, S, H, D), 310, torch.bfloat16))
    want_out, want_lse = ops.ring_fwd(q, k, v, P, None, True, fuse="step")
    out = torch.empty_like(q)
    lse = torch.empty((B, H, S), dtype=torch.float32, device=DEV)
    run = lambda: ops.ring_fwd(q, k, v, P, None, True, out=out, lse=lse, fuse="step", static_scratch=True)
    run()  # the first call on a device looks the buffer's address up: outside the capture
    torch.cuda.synchronize()
    assert torch.equal(out, want_out) and torch.equal(lse, want_lse)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run()
    for rep in range(3):
        out.fill_(7)
        lse.fill_(7)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want_out) and torch.equal(lse, want_lse), f"replay {rep} differs"
        q.mul_(-1)
        torch.cuda.synchronize()
        q.mul_(-1)
