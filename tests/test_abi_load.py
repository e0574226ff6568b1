"""CPU-side checks of the drop-in boundary: the library loads without a GPU, exports exactly
what include/sp_aurora_hip.h declares, and its argument checks answer with codes, not crashes."""
import ctypes
import os
import re

import pytest

from sp_aurora_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "sp_aurora_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(spa_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    assert declared_symbols() == sorted(_lib.SIGNATURES)


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(lib, name), name


def test_abi_version_and_error_string():
    lib = _lib.load()
    assert lib.spa_abi_version() == 1
    assert isinstance(lib.spa_last_error(), bytes)


def test_ring_workspace_sizes():
    """16-bit inputs: one slot per step but a rank's last (a block output in q's type and its fp32 lse, each a
    multiple of 256 bytes); fp32: the running output, one block's output and its lse."""
    lib = _lib.load()
    up = lambda n: (n + 255) // 256 * 256
    for B, H, S, D, P in [(1, 32, 8192, 128, 8), (2, 3, 600, 64, 3), (1, 1, 64, 32, 1), (2, 16, 32768, 128, 16)]:
        s = S // P
        for dt in (_lib.SPA_BF16, _lib.SPA_F16):
            assert lib.spa_ring_fwd_workspace_bytes(B, H, S, D, P, dt) == (P - 1) * (up(B * s * H * D * 2) + up(B * H * s * 4))
        assert lib.spa_ring_fwd_workspace_bytes(B, H, S, D, P, _lib.SPA_F32) == 2 * B * s * H * D * 4 + B * H * s * 4
    assert lib.spa_ring_fwd_workspace_bytes(1, 1, 100, 64, 3, _lib.SPA_BF16) == -1   # the ring must divide the sequence
    assert lib.spa_ring_fwd_workspace_bytes(1, 1, 64, 64, 2, 7) == -1                 # no such dtype


def _s3(*v):
    return _lib.strides3(v)


def test_bad_arguments_return_codes_without_touching_a_device():
    lib = _lib.load()
    st = _s3(64, 64, 64)
    # null pointers
    assert lib.spa_flash_fwd(None, None, None, None, None, 1, 1, 8, 8, 64, st, st, st, st, 1.0, 0, 1, None) == -1
    assert b"null" in lib.spa_last_error()
    p = ctypes.c_void_p(4096)  # aligned, never dereferenced: every check below fails before a launch
    # unsupported head dim
    assert lib.spa_flash_fwd(p, p, p, p, p, 1, 1, 8, 8, 48, st, st, st, st, 1.0, 0, 1, None) == -2
    # a scale that is not finite (any finite one is accepted, negative and zero included)
    assert lib.spa_flash_fwd(p, p, p, p, p, 1, 1, 8, 8, 64, st, st, st, st, float("nan"), 0, 1, None) == -1
    assert lib.spa_flash_fwd(p, p, p, p, p, 1, 1, 8, 8, 64, st, st, st, st, float("inf"), 0, 1, None) == -1
    # bad dtype / mask
    assert lib.spa_flash_fwd(p, p, p, p, p, 1, 1, 8, 8, 64, st, st, st, st, 1.0, 0, 7, None) == -1
    assert lib.spa_flash_fwd(p, p, p, p, p, 1, 1, 8, 8, 64, st, st, st, st, 1.0, 5, 1, None) == -1
    # misaligned pointer / stride
    assert lib.spa_flash_fwd(ctypes.c_void_p(4098), p, p, p, p, 1, 1, 8, 8, 64, st, st, st, st, 1.0, 0, 1, None) == -3
    assert lib.spa_flash_fwd(p, p, p, p, p, 1, 1, 8, 8, 64, _s3(63, 63, 63), st, st, st, 1.0, 0, 1, None) == -3
    # sizes
    assert lib.spa_flash_fwd(p, p, p, p, p, 1, 1, 0, 8, 64, st, st, st, st, 1.0, 0, 1, None) == -1
    # merge: head dim must be a power of two
    assert lib.spa_merge(p, p, p, p, 1, 1, 8, 24, st, st, 1, 0, None) == -2
    # relayout: heads not divisible, in place, bad pack
    assert lib.spa_relayout_s2h(p, ctypes.c_void_p(8192), 3, 1, 4, 8, 16, 1, 2, None) == -1
    assert lib.spa_relayout_s2h(p, p, 2, 1, 4, 8, 16, 1, 2, None) == -1
    assert lib.spa_relayout_h2s(p, ctypes.c_void_p(8192), 2, 1, 4, 8, 16, 4, 2, None) == -1
    # backward: unknown dtype code
    f = ctypes.c_void_p(4096)
    args = [f] * 9 + [1, 1, 8, 8, 64] + [st] * 7
    assert lib.spa_flash_bwd(*args, 1.0, 0, 9, None) == -1
    # e4m3 K/V: scales required, fp32 queries and head dim 32 unsupported, 8-byte alignment of k8 / v8
    a8 = [p, p, p, p, p, p, p, 1, 1, 8, 8, 64, st, st, st, st, 1.0, 0, 1, None]
    bad = list(a8); bad[3] = None
    assert lib.spa_flash_fwd_fp8kv(*bad) == -1 and b"scale" in lib.spa_last_error()
    bad = list(a8); bad[18] = 0
    assert lib.spa_flash_fwd_fp8kv(*bad) == -2
    bad = list(a8); bad[11] = 32
    assert lib.spa_flash_fwd_fp8kv(*bad) == -2
    bad = list(a8); bad[1] = ctypes.c_void_p(4100)
    assert lib.spa_flash_fwd_fp8kv(*bad) == -3
    bad = list(a8); bad[13] = _s3(60, 60, 60)
    assert lib.spa_flash_fwd_fp8kv(*bad) == -3
    # variable-length batches: (head, row) strides; the cu_seqlens arrays are never read on the host
    s2 = _lib.strides2((64, 64))
    ok = [p] * 7 + [2, 1, 16, 16, 8, 8, 64, s2, s2, s2, s2, 1.0, 1, 1, None]
    bad = list(ok); bad[5] = None  # cu_seqlens_q
    assert lib.spa_flash_fwd_varlen(*bad) == -1 and b"cu_seqlens" in lib.spa_last_error()
    bad = list(ok); bad[11] = 32  # longest sequence longer than the total
    assert lib.spa_flash_fwd_varlen(*bad) == -1
    bad = list(ok); bad[13] = 48  # head dim
    assert lib.spa_flash_fwd_varlen(*bad) == -2
    bad = list(ok); bad[5] = ctypes.c_void_p(4098)  # cu_seqlens alignment
    assert lib.spa_flash_fwd_varlen(*bad) == -3
    bad = list(ok); bad[14] = _lib.strides2((64, 63))  # row stride
    assert lib.spa_flash_fwd_varlen(*bad) == -3
    okb = [p] * 11 + [2, 1, 16, 16, 8, 8, 64] + [s2] * 7 + [1.0, 1, 1, None]
    bad = list(okb); bad[11] = 0  # no sequences
    assert lib.spa_flash_bwd_varlen(*bad) == -1
    bad = list(okb); bad[-2] = 9  # dtype
    assert lib.spa_flash_bwd_varlen(*bad) == -1
    # gradients written in the inputs' type: their rows are 16-byte aligned in that type
    bad = list(okb); bad[6] = None  # dq
    assert lib.spa_flash_bwd_varlen_out(*bad) == -1 and b"spa_flash_bwd_varlen_out" in lib.spa_last_error()
    bad = list(okb); bad[24] = _lib.strides2((64, 68))  # dv rows: 136 bytes in bf16
    assert lib.spa_flash_bwd_varlen_out(*bad) == -3
    assert lib.spa_flash_bwd_varlen(*bad) != -3  # 272 bytes as fp32 accumulators: aligned


def test_python_wrappers_refuse_cpu_tensors():
    import torch
    from sp_aurora_amd import ops
    q = torch.zeros(1, 8, 1, 64)
    with pytest.raises(ValueError, match="HIP device"):
        ops.flash_fwd(q, q, q)


def test_public_signatures_match_the_reference():
    """Argument names and defaults of sp_aurora/intel_ring_flash_attn.py:344-411 and
    sp_aurora/intel_ulysses_attn.py:501-513, plus the keyword-only ring_size extension."""
    import inspect
    import sp_aurora_amd as spa
    base = ["dropout_p", "softmax_scale", "causal", "window_size", "alibi_slopes", "deterministic",
            "return_attn_probs", "group"]
    for fn, head in ((spa.ring_flash_attn_func, ["q", "k", "v"]), (spa.ring_flash_attn_kvpacked_func, ["q", "kv"]),
                     (spa.ring_flash_attn_qkvpacked_func, ["qkv"])):
        sig = inspect.signature(fn)
        names = list(sig.parameters)
        assert names == head + base + ["ring_size", "sharding"]
        assert sig.parameters["ring_size"].kind is inspect.Parameter.KEYWORD_ONLY
        assert sig.parameters["dropout_p"].default == 0.0
        assert sig.parameters["causal"].default is False
        assert sig.parameters["window_size"].default == (-1, -1)
    assert spa.sp_aurora_func is spa.ring_flash_attn_func is spa.intel_ring_flash_attn_func
    assert spa.sp_aurora_kvpacked_func is spa.ring_flash_attn_kvpacked_func
    assert spa.sp_aurora_qkvpacked_func is spa.ring_flash_attn_qkvpacked_func
    assert list(inspect.signature(spa.ulysses_flash_attn_func).parameters) == ["q", "k", "v"] + base
    assert list(inspect.signature(spa.intel_all_to_all_4d).parameters) == ["input", "scatter_idx", "gather_idx", "group"]
    assert list(inspect.signature(spa.update_out_and_lse).parameters) == ["out", "lse", "block_out", "block_lse", "slice_"]
    fwd = list(inspect.signature(spa._flash_attn_forward).parameters)
    assert fwd[:9] == ["q", "k", "v", "dropout_p", "softmax_scale", "causal", "window_size", "alibi_slopes", "return_softmax"]


def test_unsupported_features_raise_before_any_launch():
    import torch
    import sp_aurora_amd as spa
    q = torch.zeros(1, 8, 1, 64)
    with pytest.raises(NotImplementedError):
        spa.ring_flash_attn_func(q, q, q, dropout_p=0.1)
    with pytest.raises(NotImplementedError):
        spa.ring_flash_attn_func(q, q, q, window_size=(4, 0))
    with pytest.raises(AssertionError):
        spa.ring_flash_attn_func(q, q, q, alibi_slopes=torch.zeros(1))
    with pytest.raises(NotImplementedError):
        spa.ring_flash_attn_func(q, q, q, group=object())
    cu = torch.tensor([0, 8], dtype=torch.int32)
    with pytest.raises(NotImplementedError):
        spa.sp_aurora_varlen_func(q[0], q[0], q[0], cu, cu, max_seqlen=8, dropout_p=0.1)
    with pytest.raises(ValueError, match="HIP device"):
        spa.sp_aurora_varlen_func(q[0], q[0], q[0], cu, cu, max_seqlen=8)


def test_backward_wrappers_check_shapes_before_any_launch():
    """The backward kernels index every tensor with q's and k's sizes; a mismatched call must be
    refused on the host (here with CPU tensors: the shape checks come before the device check)."""
    import torch
    from sp_aurora_amd import ops
    B, Sq, Sk, H, D = 1, 16, 24, 2, 64
    mk = lambda *shape, dt=torch.bfloat16: torch.zeros(shape, dtype=dt)
    good = dict(q=mk(B, Sq, H, D), k=mk(B, Sk, H, D), v=mk(B, Sk, H, D), dout=mk(B, Sq, H, D),
                lse=mk(B, H, Sq, dt=torch.float32), delta=mk(B, H, Sq, dt=torch.float32),
                dq_acc=mk(B, Sq, H, D, dt=torch.float32), dk_acc=mk(B, Sk, H, D, dt=torch.float32),
                dv_acc=mk(B, Sk, H, D, dt=torch.float32))
    with pytest.raises(ValueError, match="HIP device"):  # well-formed, but on the CPU
        ops.flash_bwd(**good)
    bad = {
        "v": mk(B, Sk + 8, H, D), "dout": mk(B, Sq + 8, H, D), "dq_acc": mk(B, Sq - 8, H, D, dt=torch.float32),
        "dk_acc": mk(B, Sk, H + 1, D, dt=torch.float32), "dv_acc": mk(B, Sq, H, D, dt=torch.float32),
        "lse": mk(B, H, Sq + 1, dt=torch.float32), "delta": mk(B, H + 1, Sq, dt=torch.float32),
        "k": mk(B, Sk, H, 2 * D),
    }
    for name, t in bad.items():
        with pytest.raises(ValueError, match="shape|must have|must be"):
            ops.flash_bwd(**{**good, name: t})
    with pytest.raises(TypeError):
        ops.flash_bwd(**{**good, "dout": mk(B, Sq, H, D, dt=torch.float16)})
    with pytest.raises(TypeError):
        ops.flash_bwd(**{**good, "lse": mk(B, H, Sq)})

    # packed variable-length batches
    Tq, Tk = 40, 48
    cu_q = torch.tensor([0, 16, 40], dtype=torch.int32)
    cu_k = torch.tensor([0, 24, 48], dtype=torch.int32)
    vgood = dict(q=mk(Tq, H, D), k=mk(Tk, H, D), v=mk(Tk, H, D), dout=mk(Tq, H, D),
                 lse=mk(H, Tq, dt=torch.float32), delta=mk(H, Tq, dt=torch.float32),
                 dq_acc=mk(Tq, H, D, dt=torch.float32), dk_acc=mk(Tk, H, D, dt=torch.float32),
                 dv_acc=mk(Tk, H, D, dt=torch.float32), cu_seqlens_q=cu_q, cu_seqlens_k=cu_k,
                 max_seqlen_q=24, max_seqlen_k=24)
    with pytest.raises(ValueError, match="HIP device"):
        ops.flash_bwd_varlen(**vgood)
    vbad = {"dout": mk(Tq + 1, H, D), "dk_acc": mk(Tk - 8, H, D, dt=torch.float32), "lse": mk(H, Tq + 4, dt=torch.float32),
            "v": mk(Tk, H + 1, D), "cu_seqlens_k": torch.tensor([0, 48], dtype=torch.int32)}
    for name, t in vbad.items():
        with pytest.raises(ValueError):
            ops.flash_bwd_varlen(**{**vgood, name: t})

    # the same tensors with the gradients written in q's dtype
    ogood = {k: v for k, v in good.items() if not k.endswith("_acc")}
    with pytest.raises(ValueError, match="HIP device"):
        ops.flash_bwd_out(**ogood)
    for name, t in (("dq", mk(B, Sq - 8, H, D)), ("dk", mk(B, Sk, H + 1, D)), ("dv", mk(B, Sk, H, D, dt=torch.float32)),
                    ("lse", mk(B, H, Sq + 1, dt=torch.float32))):
        with pytest.raises(ValueError):
            ops.flash_bwd_out(**{**ogood, name: t})
    vogood = {k: v for k, v in vgood.items() if not k.endswith("_acc")}
    with pytest.raises(ValueError, match="HIP device"):
        ops.flash_bwd_varlen_out(**vogood)
    for name, t in (("dq", mk(Tq + 1, H, D)), ("dk", mk(Tk - 8, H, D)), ("delta", mk(H, Tq + 4, dt=torch.float32))):
        with pytest.raises(ValueError):
            ops.flash_bwd_varlen_out(**{**vogood, name: t})
    with pytest.raises(TypeError):
        ops.flash_bwd_varlen_out(**{**vogood, "dv": mk(Tk, H, D, dt=torch.float32)})


def test_cu_seqlens_are_checked_on_the_host():
    import torch
    from sp_aurora_amd import ops
    ok = torch.tensor([0, 5, 5, 12], dtype=torch.int32)
    ops.check_cu_seqlens(ok, 12, 7, "cu")
    for cu, total, mx in [(torch.tensor([1, 5, 12]), 12, 12),      # does not start at 0
                          (torch.tensor([0, 7, 5, 12]), 12, 12),   # decreases
                          (ok, 16, 7),                             # does not end at the row count
                          (ok, 12, 6),                             # longest sequence above max_seqlen
                          (torch.tensor([0]), 0, 1)]:              # no sequence
        with pytest.raises(ValueError):
            ops.check_cu_seqlens(cu, total, mx, "cu")
    # the public function refuses a bad array before touching the device
    import sp_aurora_amd as spa
    q = torch.zeros((12, 2, 64), dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="ends at"):
        spa.sp_aurora_varlen_func(q, q, q, torch.tensor([0, 5, 10], dtype=torch.int32), max_seqlen=5)
    with pytest.raises(ValueError, match="exceeds"):
        spa.sp_aurora_varlen_func(q, q, q, torch.tensor([0, 5, 12], dtype=torch.int32), max_seqlen=5)


def test_recording_belongs_to_the_recording_thread():
    """ops.prepared() swaps a recorder in for the calling thread only: another thread that calls into
    the library meanwhile reaches the real library (here: a query that must run, not be recorded)."""
    import threading
    seen = {}
    with _lib.recording() as rec:
        assert _lib.load() is rec

        def other():
            lib = _lib.load()
            seen["is_recorder"] = lib is rec
            seen["version"] = lib.spa_abi_version()

        t = threading.Thread(target=other)
        t.start()
        t.join()
        # queries that launch nothing run as they are, also on the recording thread
        assert rec.spa_static_scratch_bytes() == 32 << 20
        buf = ctypes.create_string_buffer(8)
        assert rec.spa_device_info(buf, 0) == -1  # ran (and refused the zero-sized buffer) instead of being recorded
        assert rec.calls == []
    assert seen == {"is_recorder": False, "version": 1}
    assert not isinstance(_lib.load(), _lib._Recorder)


@pytest.mark.skipif(__import__("torch").cuda.is_available(), reason="passes pointers that must never reach a device")
def test_tensors_of_2_gib_and_more_per_head_pass_the_argument_checks():
    """K / V (and in the backward q / dout) of one (batch, head) may span 2 GiB and more: H = 64, D = 128, S = 262144
    in the public [B,S,H,D] layout is 4 GiB per head.  Without a device every check passes and the launch itself
    reports the missing device (-4); what stays refused says why (-2)."""
    lib = _lib.load()
    p = ctypes.c_void_p(4096)
    H, D, S = 64, 128, 262144
    st = _s3(S * H * D, D, H * D)
    assert lib.spa_flash_fwd(p, p, p, p, p, 1, H, S, S, D, st, st, st, st, 1.0, 1, 1, None) == -4
    assert b"device" in lib.spa_last_error()
    assert lib.spa_ring_fwd(p, p, p, p, p, p, 1, H, S, D, 16, -1, st, st, st, st, 1.0, 1, 1, 1, None) == -4
    assert lib.spa_flash_bwd_out(*([p] * 9 + [1, H, S, S, D] + [st] * 7), 1.0, 1, 1, None) == -4
    # e4m3 K/V (1 byte per element: 8 heads more), zigzag shards, and rows so far apart that 128 of them exceed 1 GiB
    st8 = _s3(2 * S * H * D, D, 2 * H * D)
    assert lib.spa_flash_fwd_fp8kv(p, p, p, p, p, p, p, 1, 2 * H, S, S, D, st, st8, st8, st, 1.0, 1, 1, None) == -2
    assert b"e4m3" in lib.spa_last_error()
    assert lib.spa_ring_fwd(p, p, p, p, p, p, 1, H, S, D, 16, -1, st, st, st, st, 1.0, 1, 1, 1 | 16, None) == -2
    assert b"zigzag" in lib.spa_last_error()
    far = _s3(0, D, 8 << 20)
    assert lib.spa_flash_fwd(p, p, p, p, p, 1, 1, 1024, 1024, D, st, far, far, st, 1.0, 0, 1, None) == -2
    assert b"1 GiB" in lib.spa_last_error()
