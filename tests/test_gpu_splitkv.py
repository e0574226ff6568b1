"""The block forward with the keys cut into chunks that run side by side (few query rows, many keys: a decode step
against a long cache): forced chunk counts and the library's own choice, against the oracle's attention and against the
same call without the split; ragged chunk sizes, e4m3 K/V, strided views, a caller's workspace."""
import pytest
import torch

from conftest import rand
from oracle import attn_oracle as O
from sp_aurora_amd import _lib, ops
from test_gpu_parity import DEV, check_lse, check_out

pytestmark = pytest.mark.gpu

CASES = [
    # B, H, Sq, Sk, D, dtype, nsplit
    (1, 32, 1, 8192, 128, torch.bfloat16, 8),       # one new token against a cache
    (2, 4, 17, 5000, 64, torch.float16, 5),         # chunks of 1024, the last one 904 keys
    (1, 8, 128, 4096, 128, torch.bfloat16, 4),
    (1, 2, 130, 1025, 64, torch.bfloat16, 8),       # two query tiles; 1025 keys: eight chunks of 256 would not do, 128-key chunks: 9 -> fewer planes
    (3, 1, 5, 700, 128, torch.float16, 2),          # the second chunk 316 keys
    (1, 2, 64, 200, 64, torch.bfloat16, 4),         # 200 keys: chunks of 128 -> two planes
    # up to four query rows: the kernel that streams K and V past them
    (2, 3, 1, 3000, 128, torch.float16, 6),         # chunks of 512, the last one 440 keys
    (1, 5, 2, 777, 64, torch.bfloat16, 3),          # chunks of 384: a wave's eight loads reach past the chunk's end
    (2, 2, 3, 1300, 128, torch.bfloat16, 1),        # one chunk: no workspace, written in place
    (1, 3, 4, 130, 64, torch.float16, 2),           # the second chunk two keys: three of its waves see none
    (1, 2, 4, 5, 128, torch.bfloat16, 1),           # five keys
]


@pytest.mark.parametrize("B,H,Sq,Sk,D,dtype,nsplit", CASES)
def test_key_split_matches_the_oracle_and_the_plain_call(B, H, Sq, Sk, D, dtype, nsplit):
    q, k, v = rand((B, Sq, H, D), 1000, dtype), rand((B, Sk, H, D), 1001, dtype), rand((B, Sk, H, D), 1002, dtype)
    want_o, want_l = O.full_attention(q, k, v, None, False)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    for scale in (None, -0.3):
        wo, wl = (want_o, want_l) if scale is None else O.full_attention(q, k, v, scale, False)
        out, lse = ops.flash_fwd(qd, kd, vd, scale, False, split_kv=nsplit)
        check_out(out, wo, dtype, f"split {nsplit} scale {scale}")
        check_lse(lse, wl)
    plain_o, plain_l = ops.flash_fwd(qd, kd, vd, None, False, split_kv=None)
    out, lse = ops.flash_fwd(qd, kd, vd, None, False, split_kv=nsplit)
    assert (lse - plain_l).abs().max().item() < 1e-4
    tol = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
    assert (out.float() - plain_o.float()).abs().max().item() <= tol * max(1.0, plain_o.float().abs().max().item())
    # a caller's workspace, poisoned; out / lse given; the operator layout
    ws = ops.flash_fwd_splitkv_workspace(qd, nsplit)
    ws.fill_(0xFF)
    o2 = torch.full_like(qd.transpose(1, 2), 7.0)
    l2 = torch.full((B, H, Sq), 7.0, dtype=torch.float32, device=DEV)
    ops.flash_fwd(qd.transpose(1, 2), kd.transpose(1, 2), vd.transpose(1, 2), None, False, layout="bhsd", out=o2, lse=l2, split_kv=nsplit,
                  workspace=ws)
    assert torch.equal(o2.transpose(1, 2), out) and torch.equal(l2, lse)


def test_key_split_with_e4m3_cache():
    B, H, Sq, Sk, D = 1, 8, 4, 6000, 128
    from test_gpu_fp8kv import quantised
    q = rand((B, Sq, H, D), 1010, torch.bfloat16)
    k8, ksc, k_deq = quantised((B, Sk, H, D), 1011, "bshd", spread=1.3)
    v8, vsc, v_deq = quantised((B, Sk, H, D), 1012, "bshd")
    want_o, want_l = O.full_attention(q, k_deq, v_deq, None, False)
    for nsplit in (3, 6, "auto"):
        out, lse = ops.flash_fwd(q.to(DEV), k8.to(DEV), v8.to(DEV), None, False, k_scale=ksc, v_scale=vsc, split_kv=nsplit)
        check_out(out, want_o, torch.bfloat16, f"e4m3 split {nsplit}")
        check_lse(lse, want_l)


@pytest.mark.parametrize("D,Sq", [(64, 1), (64, 4), (128, 2)])
def test_few_rows_with_e4m3_cache_against_the_mfma_kernel(D, Sq):
    """The streaming kernel and the MFMA kernel on the same chunks (spa_tune few_rows = 1 keeps the latter), e4m3 K/V."""
    B, H, Sk = 2, 3, 2500
    from test_gpu_fp8kv import quantised
    q = rand((B, Sq, H, D), 1030, torch.float16)
    k8, ksc, k_deq = quantised((B, Sk, H, D), 1031, "bshd", spread=1.2)
    v8, vsc, v_deq = quantised((B, Sk, H, D), 1032, "bshd")
    want_o, want_l = O.full_attention(q, k_deq, v_deq, 0.2, False)
    got = {}
    try:
        for knob in (0, 1):
            _lib.tune("few_rows", knob)
            for nsplit in (1, 4):
                out, lse = ops.flash_fwd(q.to(DEV), k8.to(DEV), v8.to(DEV), 0.2, False, k_scale=ksc, v_scale=vsc, split_kv=nsplit)
                check_out(out, want_o, torch.float16, f"e4m3 few rows knob {knob} split {nsplit}")
                check_lse(lse, want_l)
                got[knob, nsplit] = (out, lse)
    finally:
        _lib.tune("few_rows", 0)
    assert (got[0, 4][1] - got[1, 4][1]).abs().max().item() < 1e-4


def test_the_librarys_choice_and_what_is_refused():
    lib = _lib.load()
    sug = lambda B, H, Sq, Sk, D, mask=0, dt=_lib.SPA_BF16: lib.spa_flash_fwd_splitkv_suggest(B, H, Sq, Sk, D, mask, dt)
    assert sug(1, 32, 1, 32768, 128) > 1               # 32 workgroups on 256 CUs
    assert sug(1, 32, 8, 1024, 128) == 1 and sug(1, 32, 1, 512, 128) == 1   # too few keys to cut
    assert sug(1, 32, 8192, 8192, 128) == 1            # enough workgroups as it is
    assert sug(1, 32, 1, 32768, 128, mask=1) == 1      # causal
    assert sug(1, 32, 1, 32768, 32) == 1 and sug(1, 32, 1, 32768, 128, dt=_lib.SPA_F32) == 1
    q, k = rand((1, 2, 8, 64), 1020, torch.bfloat16).to(DEV), rand((1, 2, 4096, 64), 1021, torch.bfloat16).to(DEV)
    ws = ops.flash_fwd_splitkv_workspace(q, 4, layout="bhsd")
    st = lambda t: _lib.strides3((t.stride(0), t.stride(1), t.stride(2)))
    out, lse = torch.empty_like(q), torch.empty((1, 2, 8), dtype=torch.float32, device=DEV)
    args = (q.data_ptr(), k.data_ptr(), k.data_ptr(), out.data_ptr(), lse.data_ptr())
    tail = (st(q), st(k), st(k), st(out), 0.125, _lib.SPA_BF16, None)
    assert lib.spa_flash_fwd_splitkv(*args, None, 1, 2, 8, 4096, 64, 4, *tail) == -1 and b"workspace" in lib.spa_last_error()
    assert lib.spa_flash_fwd_splitkv(*args, ws.data_ptr(), 1, 2, 8, 4096, 64, 0, *tail) == -1
    assert lib.spa_flash_fwd_splitkv(*args, ws.data_ptr(), 1, 2, 8, 4096, 64, 4, *tail) == 0
    assert lib.spa_flash_fwd_splitkv(*args, None, 1, 2, 8, 4096, 64, 1, *tail) == 0    # one chunk: the plain call, no workspace
    torch.cuda.synchronize()
    with pytest.raises(ValueError):
        ops.flash_fwd(q, k, k, layout="bhsd", split_kv=8, workspace=ws)                # a workspace for four chunks


@pytest.mark.parametrize("Sq", [2, 4])   # the kernel that streams K and V; the matrix-instruction kernel
def test_key_split_replays_from_a_captured_graph(Sq):
    """Two launches and a caller's workspace, nothing allocated, no synchronisation: the call can be captured; every replay
    (with eager work in between and new values in the captured buffers) equals the eager result."""
    B, H, Sk, D, n = 1, 8, 4096, 128, 6
    q, k, v = (rand((B, s_, H, D), 1030 + i, torch.bfloat16).to(DEV) for i, s_ in enumerate((Sq, Sk, Sk)))
    ws = ops.flash_fwd_splitkv_workspace(q, n)
    out, lse = torch.empty_like(q), torch.empty((B, H, Sq), dtype=torch.float32, device=DEV)
    call = lambda: ops.flash_fwd(q, k, v, None, False, out=out, lse=lse, split_kv=n, workspace=ws)
    eager_out, eager_lse = (t.clone() for t in call())
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for rep in range(3):
        out.fill_(7)
        lse.fill_(7)
        ws.fill_(0xFF)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager_out) and torch.equal(lse, eager_lse), f"replay {rep} differs"
        k.mul_(-1)
        torch.cuda.synchronize()
        k.mul_(-1)
