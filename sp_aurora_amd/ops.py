"""Tensor-level wrappers over the C ABI: torch is used for device memory and streams only.

Every function takes tensors in either the reference's public layout ``"bshd"``
([B,S,H,D], sp_aurora/intel_ring_flash_attn.py:399-435) or its operator layout
``"bhsd"`` ([B,H,S,D], sp_aurora/intel_flash_attn.py:56); both reach the same
kernels through (batch, head, seq) strides, so no transposes or copies are made.
"""
import torch

from . import _lib

_DT = {torch.float32: _lib.SPA_F32, torch.bfloat16: _lib.SPA_BF16, torch.float16: _lib.SPA_F16}


def _dtype_code(t):
    try:
        return _DT[t.dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {t.dtype}; expected float32, bfloat16 or float16") from None


def _bhs(t, layout):
    """(B, H, S, D) sizes and (batch, head, seq) element strides of a 4-D view."""
    if t.dim() != 4:
        raise ValueError(f"expected a 4-D tensor, got {tuple(t.shape)}")
    st = t.stride()
    if layout == "bshd":
        B, S, H, D = t.shape
        return (B, H, S, D), (st[0], st[2], st[1])
    if layout == "bhsd":
        B, H, S, D = t.shape
        return (B, H, S, D), (st[0], st[1], st[2])
    raise ValueError(f"layout must be 'bshd' or 'bhsd', got {layout!r}")


def _rows_ok(t, esz):
    return t.stride(-1) == 1 and t.data_ptr() % 16 == 0 and all((s * esz) % 16 == 0 for s in t.stride()[:-1])


def _prep(t):
    """A view the kernels can read as is, else a compact copy (inner stride 1, 16-byte rows)."""
    if not t.is_cuda:
        raise ValueError("sp_aurora_amd kernels need tensors on a HIP device (got a CPU tensor)")
    return t if _rows_ok(t, t.element_size()) else t.contiguous()


FP8 = torch.float8_e4m3fn  # OCP e4m3: the 8-bit K/V format of spa_flash_fwd_fp8kv


def _fp8_scales(k, v, k_scale, v_scale, n_lead, H):
    """Checks the (k8, v8, k_scale, v_scale) quadruple of an e4m3 K/V call; returns the scales as
    contiguous fp32 [n_lead, H] tensors on k's device."""
    if k.dtype != FP8 or v.dtype != FP8:
        raise TypeError("e4m3 K/V: k and v must both be torch.float8_e4m3fn")
    if k_scale is None or v_scale is None:
        raise ValueError("e4m3 K/V need k_scale and v_scale (fp32, one per (batch or sequence, head))")
    out = []
    for name, sc in (("k_scale", k_scale), ("v_scale", v_scale)):
        if tuple(sc.shape) != (n_lead, H):
            raise ValueError(f"{name} must have shape {(n_lead, H)}, got {tuple(sc.shape)}")
        out.append(sc.to(device=k.device, dtype=torch.float32).contiguous())
    return out


def quantize_fp8_per_head(x, layout="bshd"):
    """x [B,S,H,D] (or [B,H,S,D]) -> (x8 e4m3 of the same shape, scale fp32 [B,H]) with
    x ~= x8 * scale[b,h]: one absmax scale per (batch, head), 448 = the largest e4m3 value.
    A convenience for producing the inputs of the e4m3 K/V entry points (torch ops)."""
    dims = (1, 3) if layout == "bshd" else (2, 3)
    amax = x.detach().abs().amax(dim=dims, keepdim=True).float().clamp_min(1e-12)
    scale = amax / 448.0
    x8 = (x.float() / scale).clamp(-448.0, 448.0).to(FP8)
    return x8, scale.reshape(x.shape[0], -1).contiguous()


def _stream():
    return torch.cuda.current_stream().cuda_stream


class _Current:
    """Stands in for torch.cuda.device(d) when d is the current device already (the usual case):
    entering and leaving the real context costs several microseconds per call."""

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


_CURRENT = _Current()


def _on(device):
    idx = device.index
    if idx is None or idx == torch.cuda.current_device():
        return _CURRENT
    return torch.cuda.device(device)


def prepared(fn, *args, **kwargs):
    """Runs `fn(*args, **kwargs)` (any function of this module, or a composition of them) once in
    recording mode and returns (run, result): `run()` replays exactly the C calls `fn` made, with
    every argument already converted, and `result` is what `fn` returned (the tensors the calls
    write into).  For loops that issue the same call on the same buffers many times: a replay costs
    the ctypes call and the kernel launch, not the Python-side checks (about 11 -> 3 us of host time
    per call for a merge or a re-layout).
    The tensors must be kernel-ready as passed (no hidden .contiguous() copies: a copy made while
    recording would be the buffer the replays read), stay alive and keep their addresses; the stream
    is the one current while recording."""
    with _lib.recording() as rec:
        result = fn(*args, **kwargs)
    calls = tuple(rec.calls)
    keep = (args, kwargs, result)  # the recorded pointers refer to these

    def run():
        for cfn, cargs in calls:
            rc = cfn(*cargs)
            if rc:
                _lib.check(rc)
        return keep[2]

    return run, result


def flash_fwd(q, k, v, softmax_scale=None, causal=False, layout="bshd", out=None, lse=None, k_scale=None, v_scale=None,
              q_scale=None, out_dtype=torch.bfloat16, split_kv="auto", workspace=None):
    """Block attention forward -> (out like q, lse fp32 [B,H,Sq]).  Calls spa_flash_fwd, or
    spa_flash_fwd_fp8kv when k, v are torch.float8_e4m3fn (then k_scale, v_scale fp32 [B,H] give
    K = k * k_scale[b,h], V = v * v_scale[b,h]; q bf16 or fp16), or spa_flash_fwd_fp8qkv when q is
    torch.float8_e4m3fn as well (q_scale fp32 [B,H]; D = 128; out in `out_dtype`, bf16 or fp16): the scores
    then run on the 8-bit matrix instruction.
    split_kv: for calls without a mask whose few query rows would leave most CUs idle (a decode step against a long
    cache) the keys are cut into chunks that run side by side (spa_flash_fwd_splitkv[_fp8kv]): "auto" = as many as
    the library suggests, an int = that many, None or 1 = never.  The chunks' results wait in `workspace` (a uint8 tensor
    of flash_fwd_splitkv_workspace(...) bytes; allocated here when not given, except while the stream is being captured,
    where "auto" then does not split).  With up to three query rows and no mask the library runs a kernel that streams K and V
    past the rows instead of the matrix-instruction kernel, split or not."""
    lib = _lib.load()
    fp8 = k.dtype == FP8 or v.dtype == FP8
    if q.dtype == FP8:
        return _flash_fwd_fp8qkv(lib, q, k, v, softmax_scale, causal, layout, out, lse, q_scale, k_scale, v_scale, out_dtype)
    if fp8:
        q = _prep(q)
        k, v = [t if t.stride(-1) == 1 and all(s % 8 == 0 for s in t.stride()[:-1]) and t.data_ptr() % 8 == 0 else t.contiguous() for t in (k, v)]
        if not k.is_cuda or not v.is_cuda:
            raise ValueError("sp_aurora_amd kernels need tensors on a HIP device (got a CPU tensor)")
    else:
        q, k, v = _prep(q), _prep(k), _prep(v)
        if not (q.dtype == k.dtype == v.dtype):
            raise TypeError("q, k, v must share a dtype")
    (B, H, Sq, D), qs = _bhs(q, layout)
    (Bk, Hk, Sk, Dk), ks = _bhs(k, layout)
    (Bv, Hv, Sv, Dv), vs = _bhs(v, layout)
    if (Bk, Hk, Dk) != (B, H, D) or (Bv, Hv, Sv, Dv) != (Bk, Hk, Sk, Dk):
        raise ValueError(f"shape mismatch: q {tuple(q.shape)} k {tuple(k.shape)} v {tuple(v.shape)}")
    if softmax_scale is None:
        softmax_scale = D ** (-0.5)
    if out is None:
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    if lse is None:
        lse = torch.empty((B, H, Sq), dtype=torch.float32, device=q.device)
    _, os_ = _bhs(out, layout)
    nsplit = 1
    if split_kv is not None and split_kv != 1 and not causal and q.dtype in (torch.bfloat16, torch.float16) and D in (64, 128):
        if split_kv == "auto":
            nsplit = lib.spa_flash_fwd_splitkv_suggest(B, H, Sq, Sk, D, _lib.SPA_MASK_NONE, _dtype_code(q))
            if nsplit > 1 and workspace is None and q.is_cuda and torch.cuda.is_current_stream_capturing():
                nsplit = 1
        else:
            nsplit = int(split_kv)
            if nsplit < 1:
                raise ValueError(f"split_kv must be 'auto', None or a positive int, got {split_kv!r}")
    if nsplit > 1:
        need = lib.spa_flash_fwd_splitkv_workspace_bytes(B, H, Sq, D, nsplit, _dtype_code(q))
        if workspace is None:
            workspace = torch.empty((need,), dtype=torch.uint8, device=q.device)
        elif workspace.numel() * workspace.element_size() < need or workspace.device != q.device:
            raise ValueError(f"split_kv={nsplit}: the workspace must hold {need} bytes on q's device")
        stail = (workspace.data_ptr(), B, H, Sq, Sk, D, nsplit, _lib.strides3(qs), _lib.strides3(ks), _lib.strides3(vs), _lib.strides3(os_),
                 float(softmax_scale), _dtype_code(q), _stream())
        with _on(q.device):
            if fp8:
                ksc, vsc = _fp8_scales(k, v, k_scale, v_scale, B, H)
                _lib.check(lib.spa_flash_fwd_splitkv_fp8kv(q.data_ptr(), k.data_ptr(), v.data_ptr(), ksc.data_ptr(), vsc.data_ptr(),
                                                           out.data_ptr(), lse.data_ptr(), *stail))
            else:
                _lib.check(lib.spa_flash_fwd_splitkv(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(), *stail))
        return out, lse
    tail = (B, H, Sq, Sk, D, _lib.strides3(qs), _lib.strides3(ks), _lib.strides3(vs), _lib.strides3(os_),
            float(softmax_scale), _lib.SPA_MASK_CAUSAL if causal else _lib.SPA_MASK_NONE, _dtype_code(q), _stream())
    with _on(q.device):
        if fp8:
            ksc, vsc = _fp8_scales(k, v, k_scale, v_scale, B, H)
            _lib.check(lib.spa_flash_fwd_fp8kv(q.data_ptr(), k.data_ptr(), v.data_ptr(), ksc.data_ptr(), vsc.data_ptr(),
                                               out.data_ptr(), lse.data_ptr(), *tail))
        else:
            _lib.check(lib.spa_flash_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(), *tail))
    return out, lse


def flash_fwd_splitkv_workspace(q, nsplit, layout="bshd"):
    """Scratch tensor (uint8) for flash_fwd(..., split_kv=nsplit) on this q."""
    (B, H, Sq, D), _ = _bhs(q, layout)
    need = _lib.load().spa_flash_fwd_splitkv_workspace_bytes(B, H, Sq, D, int(nsplit), _dtype_code(q))
    if need < 0:
        raise ValueError("the key split is built for bf16 / fp16 queries")
    return torch.empty((need,), dtype=torch.uint8, device=q.device)


def _flash_fwd_fp8qkv(lib, q, k, v, softmax_scale, causal, layout, out, lse, q_scale, k_scale, v_scale, out_dtype):
    if k.dtype != FP8 or v.dtype != FP8:
        raise TypeError("e4m3 q goes with e4m3 k and v")
    if out_dtype not in (torch.bfloat16, torch.float16):
        raise TypeError("e4m3 q: out_dtype must be bfloat16 or float16")
    ok16 = lambda t: t.is_cuda and t.stride(-1) == 1 and t.data_ptr() % 16 == 0 and all(s % 16 == 0 for s in t.stride()[:-1])
    for name, t in (("q", q), ("k", k), ("v", v)):
        if not t.is_cuda:
            raise ValueError("sp_aurora_amd kernels need tensors on a HIP device (got a CPU tensor)")
    q, k, v = [t if ok16(t) else t.contiguous() for t in (q, k, v)]
    (B, H, Sq, D), qs = _bhs(q, layout)
    (Bk, Hk, Sk, Dk), ks = _bhs(k, layout)
    shp_v, vs = _bhs(v, layout)
    if (Bk, Hk, Dk) != (B, H, D) or shp_v != (Bk, Hk, Sk, Dk):
        raise ValueError(f"shape mismatch: q {tuple(q.shape)} k {tuple(k.shape)} v {tuple(v.shape)}")
    if q_scale is None or tuple(q_scale.shape) != (B, H):
        raise ValueError(f"e4m3 q needs q_scale (fp32 {(B, H)})")
    ksc, vsc = _fp8_scales(k, v, k_scale, v_scale, B, H)
    qsc = q_scale.to(device=q.device, dtype=torch.float32).contiguous()
    if softmax_scale is None:
        softmax_scale = D ** (-0.5)
    if out is None:
        out = torch.empty(q.shape, dtype=out_dtype, device=q.device)
    if lse is None:
        lse = torch.empty((B, H, Sq), dtype=torch.float32, device=q.device)
    _, os_ = _bhs(out, layout)
    with _on(q.device):
        _lib.check(lib.spa_flash_fwd_fp8qkv(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), qsc.data_ptr(), ksc.data_ptr(), vsc.data_ptr(), out.data_ptr(), lse.data_ptr(),
            B, H, Sq, Sk, D, _lib.strides3(qs), _lib.strides3(ks), _lib.strides3(vs), _lib.strides3(os_),
            float(softmax_scale), _lib.SPA_MASK_CAUSAL if causal else _lib.SPA_MASK_NONE, _dtype_code(out), _stream()))
    return out, lse


def ring_fwd_workspace(q, ring_size, layout="bshd", out_dtype=None):
    """Scratch tensor spa_ring_fwd needs for this q and ring size (uint8, 16-byte aligned); out_dtype: the type of
    the result when q is e4m3."""
    lib = _lib.load()
    (B, H, S, D), _ = _bhs(q, layout)
    nbytes = lib.spa_ring_fwd_workspace_bytes(B, H, S, D, int(ring_size), _DT[out_dtype] if q.dtype == FP8 else _dtype_code(q))
    if nbytes < 0:
        raise ValueError(f"ring_size={ring_size} must divide the sequence length {S}")
    return torch.empty((nbytes,), dtype=torch.uint8, device=q.device)


RING_FUSE = {"step": _lib.SPA_RING_PER_STEP, "rank": _lib.SPA_RING_PER_RANK, "all": _lib.SPA_RING_ALL_RANKS}


def ring_fwd(q, k, v, ring_size, softmax_scale=None, causal=False, rank=-1, layout="bshd", out=None, lse=None,
             workspace=None, fuse="rank", static_scratch=False, k_scale=None, v_scale=None, sharding="contiguous",
             q_scale=None, out_dtype=torch.bfloat16):
    """Simulated ring forward of one rank (or all, rank=-1) over the full-sequence q,k,v: one C call
    that enqueues the kernels in ring order.  Calls spa_ring_fwd.  `fuse`: "step" = one launch per
    (q chunk, kv chunk) pair, "rank" = one launch per rank walking its chunks, "all" = one launch.
    Returns (out like q, lse fp32 [B,H,S]); with rank >= 0 only that rank's rows are written.
    k, v may be torch.float8_e4m3fn with k_scale, v_scale fp32 [B,H] (spa_ring_fwd_fp8kv); q as well, with q_scale
    and the result's out_dtype (spa_ring_fwd_fp8qkv: D = 128, scores on the 8-bit matrix instruction).
    sharding="zigzag": the rows of q, k, v are in zigzag-sharded order (chunk r of the tensors holds
    half-chunks r and 2P-1-r of the sequence); out and lse come back in the same order.
    static_scratch=True calls spa_ring_fwd_static instead: no workspace tensor, the library's built-in
    32 MiB buffer holds a rank's earlier block results between step launches (for callers that must not allocate;
    calls that overlap on one device race)."""
    lib = _lib.load()
    fp8 = k.dtype == FP8 or v.dtype == FP8
    qk8 = q.dtype == FP8
    if qk8:
        if not fp8 or q_scale is None or out_dtype not in (torch.bfloat16, torch.float16):
            raise ValueError("e4m3 q goes with e4m3 k, v, a q_scale and out_dtype bfloat16 or float16")
        if not q.is_cuda:
            raise ValueError("sp_aurora_amd kernels need tensors on a HIP device (got a CPU tensor)")
        ok16 = lambda t: t.stride(-1) == 1 and t.data_ptr() % 16 == 0 and all(s % 16 == 0 for s in t.stride()[:-1])
        q = q if ok16(q) else q.contiguous()
        k = k if k.is_cuda and ok16(k) else k.contiguous()
    if fp8:
        if static_scratch:
            raise ValueError("static_scratch=True has no e4m3 K/V form")
        q = q if qk8 else _prep(q)
        k, v = [t if t.stride(-1) == 1 and all(s % 8 == 0 for s in t.stride()[:-1]) and t.data_ptr() % 8 == 0 else t.contiguous() for t in (k, v)]
        if not k.is_cuda or not v.is_cuda:
            raise ValueError("sp_aurora_amd kernels need tensors on a HIP device (got a CPU tensor)")
    else:
        q, k, v = _prep(q), _prep(k), _prep(v)
        if not (q.dtype == k.dtype == v.dtype):
            raise TypeError("q, k, v must share a dtype")
    (B, H, S, D), qs = _bhs(q, layout)
    shp_k, ks = _bhs(k, layout)
    shp_v, vs = _bhs(v, layout)
    if shp_k != (B, H, S, D) or shp_v != (B, H, S, D):
        raise ValueError(f"ring attention needs q, k, v of one shape, got {tuple(q.shape)} {tuple(k.shape)} {tuple(v.shape)}")
    if softmax_scale is None:
        softmax_scale = D ** (-0.5)
    if out is None:
        out = torch.empty(q.shape, dtype=out_dtype if qk8 else q.dtype, device=q.device)
    if lse is None:
        lse = torch.empty((B, H, S), dtype=torch.float32, device=q.device)
    if fuse not in RING_FUSE:
        raise ValueError(f"fuse must be one of {sorted(RING_FUSE)}, got {fuse!r}")
    if sharding not in ("contiguous", "zigzag"):
        raise ValueError(f"sharding must be 'contiguous' or 'zigzag', got {sharding!r}")
    if static_scratch and workspace is not None:
        raise ValueError("static_scratch=True takes no workspace")
    if workspace is None and not static_scratch and (fuse == "step" or q.dtype == torch.float32):
        workspace = ring_fwd_workspace(q, ring_size, layout, out.dtype)
    _, os_ = _bhs(out, layout)
    tail = (B, H, S, D, int(ring_size), int(rank),
            _lib.strides3(qs), _lib.strides3(ks), _lib.strides3(vs), _lib.strides3(os_),
            float(softmax_scale), _lib.SPA_MASK_CAUSAL if causal else _lib.SPA_MASK_NONE,
            _dtype_code(out), RING_FUSE[fuse] | (_lib.SPA_RING_ZIGZAG if sharding == "zigzag" else 0), _stream())
    with _on(q.device):
        if qk8:
            ksc, vsc = _fp8_scales(k, v, k_scale, v_scale, B, H)
            if tuple(q_scale.shape) != (B, H):
                raise ValueError(f"q_scale must have shape {(B, H)}, got {tuple(q_scale.shape)}")
            qsc = q_scale.to(device=q.device, dtype=torch.float32).contiguous()
            _lib.check(lib.spa_ring_fwd_fp8qkv(q.data_ptr(), k.data_ptr(), v.data_ptr(), qsc.data_ptr(), ksc.data_ptr(), vsc.data_ptr(),
                                               out.data_ptr(), lse.data_ptr(),
                                               workspace.data_ptr() if workspace is not None else None, *tail))
        elif fp8:
            ksc, vsc = _fp8_scales(k, v, k_scale, v_scale, B, H)
            _lib.check(lib.spa_ring_fwd_fp8kv(q.data_ptr(), k.data_ptr(), v.data_ptr(), ksc.data_ptr(), vsc.data_ptr(),
                                              out.data_ptr(), lse.data_ptr(),
                                              workspace.data_ptr() if workspace is not None else None, *tail))
        elif static_scratch:
            _lib.check(lib.spa_ring_fwd_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(), *tail))
        else:
            _lib.check(lib.spa_ring_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(),
                                        workspace.data_ptr() if workspace is not None else None, *tail))
    return out, lse


class RingFlags:
    """Arrival flags of a ring's KV chunks for ring_fwd_flags: uint32 flag per chunk and a fault word, on the device.
    `epoch` is what a flag must reach; next_epoch() starts a new round without clearing the array."""

    def __init__(self, ring_size, device):
        self.arrive = torch.zeros((int(ring_size),), dtype=torch.int32, device=device)
        self.fault = torch.zeros((1,), dtype=torch.int32, device=device)
        self.epoch = 1

    def next_epoch(self):
        self.epoch += 1
        return self.epoch

    def set(self, chunk, stream=None):
        """arrive[chunk] = epoch after everything enqueued so far on `stream` (default: the current one)."""
        st = _stream() if stream is None else stream.cuda_stream
        _lib.check(_lib.load().spa_ring_flag_set(self.arrive.data_ptr(), int(chunk), self.epoch, st))

    def set_all(self, stream=None):
        for c in range(self.arrive.numel()):
            self.set(c, stream)

    def failed(self):
        """True when some wave gave up waiting (reads the fault word: synchronises)."""
        return bool(self.fault.item())


def ring_fwd_flags(q, k, v, ring_size, flags, softmax_scale=None, causal=False, rank=-1, layout="bshd", out=None, lse=None,
                   spin_limit=1 << 20, q_scale=None, k_scale=None, v_scale=None, out_dtype=torch.bfloat16):
    """ring_fwd(fuse="rank") for chunks that arrive while the launch runs: a workgroup waits for flags.arrive[c] >=
    flags.epoch (bounded by spin_limit polls) before it touches chunk c.  Calls spa_ring_fwd_flags, or, for e4m3 q, k, v
    with their [B,H] scales (D = 128, result in out_dtype), spa_ring_fwd_flags_fp8qkv."""
    lib = _lib.load()
    fp8 = q.dtype == FP8
    if fp8:
        if k.dtype != FP8 or v.dtype != FP8 or q_scale is None or out_dtype not in (torch.bfloat16, torch.float16):
            raise ValueError("e4m3 q goes with e4m3 k, v, the three scales and out_dtype bfloat16 or float16")
        if not (q.is_cuda and k.is_cuda and v.is_cuda):
            raise ValueError("sp_aurora_amd kernels need tensors on a HIP device (got a CPU tensor)")
        ok16 = lambda t: t.stride(-1) == 1 and t.data_ptr() % 16 == 0 and all(s_ % 16 == 0 for s_ in t.stride()[:-1])
        q, k, v = (t if ok16(t) else t.contiguous() for t in (q, k, v))
    else:
        q, k, v = _prep(q), _prep(k), _prep(v)
        if not (q.dtype == k.dtype == v.dtype):
            raise TypeError("q, k, v must share a dtype")
    (B, H, S, D), qs = _bhs(q, layout)
    shp_k, ks = _bhs(k, layout)
    shp_v, vs = _bhs(v, layout)
    if shp_k != (B, H, S, D) or shp_v != (B, H, S, D):
        raise ValueError(f"ring attention needs q, k, v of one shape, got {tuple(q.shape)} {tuple(k.shape)} {tuple(v.shape)}")
    if flags.arrive.numel() != int(ring_size) or flags.arrive.device != q.device:
        raise ValueError("flags must hold one entry per chunk on q's device")
    if softmax_scale is None:
        softmax_scale = D ** (-0.5)
    if out is None:
        out = torch.empty(q.shape, dtype=out_dtype if fp8 else q.dtype, device=q.device)
    if lse is None:
        lse = torch.empty((B, H, S), dtype=torch.float32, device=q.device)
    _, os_ = _bhs(out, layout)
    tail = (flags.arrive.data_ptr(), flags.epoch, int(spin_limit), flags.fault.data_ptr(), B, H, S, D, int(ring_size), int(rank),
            _lib.strides3(qs), _lib.strides3(ks), _lib.strides3(vs), _lib.strides3(os_), float(softmax_scale),
            _lib.SPA_MASK_CAUSAL if causal else _lib.SPA_MASK_NONE, _dtype_code(out), _stream())
    with _on(q.device):
        if fp8:
            ksc, vsc = _fp8_scales(k, v, k_scale, v_scale, B, H)
            if tuple(q_scale.shape) != (B, H):
                raise ValueError(f"q_scale must have shape {(B, H)}, got {tuple(q_scale.shape)}")
            qsc = q_scale.to(device=q.device, dtype=torch.float32).contiguous()
            _lib.check(lib.spa_ring_fwd_flags_fp8qkv(q.data_ptr(), k.data_ptr(), v.data_ptr(), qsc.data_ptr(), ksc.data_ptr(), vsc.data_ptr(),
                                                     out.data_ptr(), lse.data_ptr(), *tail))
        else:
            _lib.check(lib.spa_ring_fwd_flags(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(), *tail))
    return out, lse


def merge(out_acc, lse_acc, blk_out, blk_lse, layout="bshd", init=False):
    """In-place merge of (blk_out, blk_lse) into fp32 (out_acc, lse_acc).  Calls spa_merge."""
    lib = _lib.load()
    blk_out = _prep(blk_out)
    (B, H, Sq, D), as_ = _bhs(out_acc, layout)
    shp, bs = _bhs(blk_out, layout)
    if shp != (B, H, Sq, D) or tuple(lse_acc.shape) != (B, H, Sq) or tuple(blk_lse.shape) != (B, H, Sq):
        raise ValueError("merge: shape mismatch")
    if out_acc.dtype != torch.float32 or lse_acc.dtype != torch.float32 or blk_lse.dtype != torch.float32:
        raise TypeError("merge: accumulators and lse must be float32")
    if not (lse_acc.is_contiguous() and blk_lse.is_contiguous() and _rows_ok(out_acc, 4)):
        raise ValueError("merge: lse tensors must be contiguous and out_acc 16-byte aligned")
    with _on(out_acc.device):
        _lib.check(lib.spa_merge(
            out_acc.data_ptr(), lse_acc.data_ptr(), blk_out.data_ptr(), blk_lse.data_ptr(),
            B, H, Sq, D, _lib.strides3(as_), _lib.strides3(bs), _dtype_code(blk_out),
            1 if init else 0, _stream()))
    return out_acc, lse_acc


def finalize(out_acc, dtype, layout="bshd", out=None):
    """out = out_acc.to(dtype) through spa_finalize."""
    lib = _lib.load()
    (B, H, Sq, D), as_ = _bhs(out_acc, layout)
    if out is None:
        out = torch.empty(out_acc.shape, dtype=dtype, device=out_acc.device)
    _, os_ = _bhs(out, layout)
    with _on(out_acc.device):
        _lib.check(lib.spa_finalize(out.data_ptr(), out_acc.data_ptr(), B, H, Sq, D,
                                    _lib.strides3(os_), _lib.strides3(as_), _dtype_code(out), _stream()))
    return out


def _relayout(x, P, s2h, out=None):
    """x: [P, B, s, (pack,) H, D] (s2h) or [P, B, P*s, (pack,) H/P, D] (h2s), contiguous."""
    lib = _lib.load()
    if x.dim() not in (5, 6):
        raise ValueError(f"expected [P,B,S,H,D] or [P,B,S,pack,H,D], got {tuple(x.shape)}")
    if not x.is_cuda:
        raise ValueError("sp_aurora_amd kernels need tensors on a HIP device (got a CPU tensor)")
    x = x.contiguous()
    pack = x.shape[3] if x.dim() == 6 else 1
    if x.shape[0] != P:
        raise ValueError(f"leading axis {x.shape[0]} != P={P}")
    B, S_in, H_in, D = x.shape[1], x.shape[2], x.shape[-2], x.shape[-1]
    if s2h:
        if H_in % P:
            raise ValueError(f"heads ({H_in}) not divisible by P={P}")
        s, H = S_in, H_in
        oshape = (P, B, P * s) + ((pack,) if x.dim() == 6 else ()) + (H // P, D)
    else:
        if S_in % P:
            raise ValueError(f"sequence ({S_in}) not divisible by P={P}")
        s, H = S_in // P, H_in * P
        oshape = (P, B, s) + ((pack,) if x.dim() == 6 else ()) + (H, D)
    if out is None:
        out = torch.empty(oshape, dtype=x.dtype, device=x.device)
    fn = lib.spa_relayout_s2h if s2h else lib.spa_relayout_h2s
    with _on(x.device):
        _lib.check(fn(x.data_ptr(), out.data_ptr(), P, B, s, H, D, pack, x.element_size(), _stream()))
    return out


def relayout_s2h(x, P, out=None):
    """Sequence-sharded [P][B,s,(pack,)H,D] -> head-sharded [P][B,P*s,(pack,)H/P,D]."""
    return _relayout(x, P, True, out)


def relayout_h2s(y, P, out=None):
    """Head-sharded [P][B,P*s,(pack,)H/P,D] -> sequence-sharded [P][B,s,(pack,)H,D]."""
    return _relayout(y, P, False, out)


def bwd_delta(out, dout, layout="bshd"):
    """delta = rowsum(dout * out), fp32 [B,H,Sq].  Calls spa_bwd_delta."""
    lib = _lib.load()
    out, dout = _prep(out), _prep(dout)
    (B, H, Sq, D), os_ = _bhs(out, layout)
    shp, ds = _bhs(dout, layout)
    if shp != (B, H, Sq, D) or out.dtype != dout.dtype:
        raise ValueError("bwd_delta: out and dout must match in shape and dtype")
    delta = torch.empty((B, H, Sq), dtype=torch.float32, device=out.device)
    with _on(out.device):
        _lib.check(lib.spa_bwd_delta(out.data_ptr(), dout.data_ptr(), delta.data_ptr(), B, H, Sq, D,
                                     _lib.strides3(os_), _lib.strides3(ds), _dtype_code(out), _stream()))
    return delta


def flash_bwd(q, k, v, dout, lse, delta, dq_acc, dk_acc, dv_acc, softmax_scale=None, causal=False,
              layout="bshd"):
    """Block-wise backward of one (q chunk, kv chunk) pair; adds into fp32 dq/dk/dv accumulators."""
    if not (q.dtype == k.dtype == v.dtype == dout.dtype):
        raise TypeError("flash_bwd: q, k, v, dout must share a dtype")
    (B, H, Sq, D), _ = _bhs(q, layout)
    shp_k, shp_v, shp_do = _bhs(k, layout)[0], _bhs(v, layout)[0], _bhs(dout, layout)[0]
    shp_dq, dqs = _bhs(dq_acc, layout)
    shp_dk, dks = _bhs(dk_acc, layout)
    shp_dv, dvs = _bhs(dv_acc, layout)
    Sk = shp_k[2]
    # the kernels index every tensor with these sizes: a mismatch would be an out-of-bounds access
    if shp_k != (B, H, Sk, D) or shp_v != shp_k:
        raise ValueError(f"flash_bwd: shape mismatch: q {tuple(q.shape)} k {tuple(k.shape)} v {tuple(v.shape)}")
    if shp_do != (B, H, Sq, D) or shp_dq != (B, H, Sq, D):
        raise ValueError(f"flash_bwd: dout {tuple(dout.shape)} and dq_acc {tuple(dq_acc.shape)} must have q's shape {tuple(q.shape)}")
    if shp_dk != shp_k or shp_dv != shp_k:
        raise ValueError(f"flash_bwd: dk_acc {tuple(dk_acc.shape)} and dv_acc {tuple(dv_acc.shape)} must have k's shape {tuple(k.shape)}")
    if tuple(lse.shape) != (B, H, Sq) or tuple(delta.shape) != (B, H, Sq):
        raise ValueError(f"flash_bwd: lse {tuple(lse.shape)} and delta {tuple(delta.shape)} must be [B,H,Sq] = {(B, H, Sq)}")
    if softmax_scale is None:
        softmax_scale = D ** (-0.5)
    for t in (dq_acc, dk_acc, dv_acc, lse, delta):
        if t.dtype != torch.float32:
            raise TypeError("flash_bwd: accumulators, lse and delta must be float32")
        if t.device != q.device:
            raise ValueError("flash_bwd: every tensor must live on q's device")
    if not (lse.is_contiguous() and delta.is_contiguous()):
        raise ValueError("flash_bwd: lse and delta must be contiguous [B,H,Sq]")
    lib = _lib.load()
    q, k, v, dout = _prep(q), _prep(k), _prep(v), _prep(dout)
    qs, ks, vs, dos = _bhs(q, layout)[1], _bhs(k, layout)[1], _bhs(v, layout)[1], _bhs(dout, layout)[1]
    if not (_rows_ok(dq_acc, 4) and _rows_ok(dk_acc, 4) and _rows_ok(dv_acc, 4)):
        raise ValueError("flash_bwd: accumulators need an inner stride of 1 and 16-byte aligned rows")
    with _on(q.device):
        _lib.check(lib.spa_flash_bwd(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), dout.data_ptr(), lse.data_ptr(), delta.data_ptr(),
            dq_acc.data_ptr(), dk_acc.data_ptr(), dv_acc.data_ptr(),
            B, H, Sq, Sk, D,
            _lib.strides3(qs), _lib.strides3(ks), _lib.strides3(vs), _lib.strides3(dos),
            _lib.strides3(dqs), _lib.strides3(dks), _lib.strides3(dvs),
            float(softmax_scale), _lib.SPA_MASK_CAUSAL if causal else _lib.SPA_MASK_NONE,
            _dtype_code(q), _stream()))
    return dq_acc, dk_acc, dv_acc


# ------------------------------------------------------------------ variable-length batches
def check_cu_seqlens(cu, total, max_seqlen, what):
    """One host-side look at a cu_seqlens array (a device-to-host read): offsets start at 0, never
    decrease, end at `total` rows, and no sequence is longer than `max_seqlen`.  The kernels trust
    these values when they index the packed tensors, so a bad array would be an out-of-bounds access."""
    c = cu.detach().to("cpu", torch.int64)
    if c.dim() != 1 or c.numel() < 2:
        raise ValueError(f"{what} must be a 1-D tensor of nseq + 1 offsets, got {tuple(cu.shape)}")
    lens = c[1:] - c[:-1]
    if int(c[0]) != 0 or bool((lens < 0).any()):
        raise ValueError(f"{what} must start at 0 and never decrease")
    if int(c[-1]) != int(total):
        raise ValueError(f"{what} ends at {int(c[-1])}, the packed tensor has {int(total)} rows")
    if int(lens.max()) > int(max_seqlen):
        raise ValueError(f"{what}: longest sequence {int(lens.max())} exceeds max_seqlen {int(max_seqlen)}")


# (address, version counter, length, device, total rows, max_seqlen) of cu_seqlens arrays that passed
# check_cu_seqlens: a training loop hands the same array to every layer, and one look is enough
_CU_CHECKED = {}


def check_cu_seqlens_once(cu, total, max_seqlen, what):
    """check_cu_seqlens, remembered per distinct array (same storage address, same version counter,
    same sizes), so that only the first call with an array pays the blocking device-to-host read.
    While the current stream is being captured nothing is read (a synchronous copy is illegal
    there): the caller of a captured region vouches for its offsets.  Returns True when the array
    is known to be good, False when the check was skipped."""
    key = (cu.data_ptr(), cu._version, cu.numel(), str(cu.device), int(total), int(max_seqlen))
    if key in _CU_CHECKED:
        return True
    if cu.is_cuda and torch.cuda.is_current_stream_capturing():
        return False
    check_cu_seqlens(cu, total, max_seqlen, what)
    if len(_CU_CHECKED) >= 256:
        _CU_CHECKED.clear()
    _CU_CHECKED[key] = True
    return True



def _thd(t, what):
    """(rows, H, D) sizes and (head, row) element strides of a packed 3-D tensor."""
    if t.dim() != 3:
        raise ValueError(f"{what}: expected a packed [total, H, D] tensor, got {tuple(t.shape)}")
    return tuple(t.shape), (t.stride(1), t.stride(0))


def _cu(cu, device, what):
    if cu.dim() != 1 or cu.numel() < 2:
        raise ValueError(f"{what} must be a 1-D tensor of nseq + 1 offsets, got {tuple(cu.shape)}")
    if cu.dtype != torch.int32 or cu.device != device or not cu.is_contiguous():
        cu = cu.to(device=device, dtype=torch.int32).contiguous()
    return cu


def flash_bwd_out(q, k, v, dout, lse, delta, softmax_scale=None, causal=False, layout="bshd", dq=None, dk=None, dv=None):
    """Backward that one call computes in full: returns (dq, dk, dv) in q's dtype, written by the kernels
    (no fp32 accumulators).  dq, dk, dv may be given (views of q's / k's shape and dtype).  Calls spa_flash_bwd_out."""
    if not (q.dtype == k.dtype == v.dtype == dout.dtype):
        raise TypeError("flash_bwd_out: q, k, v, dout must share a dtype")
    (B, H, Sq, D), _ = _bhs(q, layout)
    shp_k, shp_v, shp_do = _bhs(k, layout)[0], _bhs(v, layout)[0], _bhs(dout, layout)[0]
    Sk = shp_k[2]
    if shp_k != (B, H, Sk, D) or shp_v != shp_k or shp_do != (B, H, Sq, D):
        raise ValueError(f"flash_bwd_out: shape mismatch: q {tuple(q.shape)} k {tuple(k.shape)} v {tuple(v.shape)} dout {tuple(dout.shape)}")
    if tuple(lse.shape) != (B, H, Sq) or tuple(delta.shape) != (B, H, Sq):
        raise ValueError(f"flash_bwd_out: lse {tuple(lse.shape)} and delta {tuple(delta.shape)} must be [B,H,Sq] = {(B, H, Sq)}")
    for t in (lse, delta):
        if t.dtype != torch.float32 or not t.is_contiguous() or t.device != q.device:
            raise ValueError("flash_bwd_out: lse and delta must be contiguous float32 tensors on q's device")
    q, k, v, dout = _prep(q), _prep(k), _prep(v), _prep(dout)
    dq = torch.empty(q.shape, dtype=q.dtype, device=q.device) if dq is None else dq
    dk = torch.empty(k.shape, dtype=q.dtype, device=q.device) if dk is None else dk
    dv = torch.empty(v.shape, dtype=q.dtype, device=q.device) if dv is None else dv
    for g, like, name in ((dq, q, "dq"), (dk, k, "dk"), (dv, v, "dv")):
        # the kernels index the gradients with q's / k's sizes: a mismatch would be an out-of-bounds access
        if tuple(g.shape) != tuple(like.shape) or g.dtype != q.dtype or g.device != q.device or not _rows_ok(g, g.element_size()):
            raise ValueError(f"flash_bwd_out: {name} must have the shape, dtype and device of its input, inner stride 1 and 16-byte aligned rows")
    if softmax_scale is None:
        softmax_scale = D ** (-0.5)
    lib = _lib.load()
    qs, ks, vs, dos = _bhs(q, layout)[1], _bhs(k, layout)[1], _bhs(v, layout)[1], _bhs(dout, layout)[1]
    dqs, dks, dvs = _bhs(dq, layout)[1], _bhs(dk, layout)[1], _bhs(dv, layout)[1]
    with _on(q.device):
        _lib.check(lib.spa_flash_bwd_out(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), dout.data_ptr(), lse.data_ptr(), delta.data_ptr(),
            dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), B, H, Sq, Sk, D,
            _lib.strides3(qs), _lib.strides3(ks), _lib.strides3(vs), _lib.strides3(dos),
            _lib.strides3(dqs), _lib.strides3(dks), _lib.strides3(dvs),
            float(softmax_scale), _lib.SPA_MASK_CAUSAL if causal else _lib.SPA_MASK_NONE, _dtype_code(q), _stream()))
    return dq, dk, dv


def flash_fwd_varlen(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, softmax_scale=None,
                     causal=False, out=None, lse=None, k_scale=None, v_scale=None):
    """Attention inside each sequence of a packed batch: q [total_q,H,D], k,v [total_k,H,D],
    cu_seqlens_* int32 [nseq+1] on the device.  Returns (out like q, lse fp32 [H,total_q]).
    Calls spa_flash_fwd_varlen, or spa_flash_fwd_varlen_fp8kv when k, v are torch.float8_e4m3fn
    (k_scale, v_scale: fp32 [nseq, H])."""
    lib = _lib.load()
    fp8 = k.dtype == FP8 or v.dtype == FP8
    if fp8:
        q = _prep(q)
        k, v = [t if t.is_contiguous() else t.contiguous() for t in (k, v)]
        if not k.is_cuda or not v.is_cuda:
            raise ValueError("sp_aurora_amd kernels need tensors on a HIP device (got a CPU tensor)")
    else:
        q, k, v = _prep(q), _prep(k), _prep(v)
        if not (q.dtype == k.dtype == v.dtype):
            raise TypeError("q, k, v must share a dtype")
    (Tq, H, D), qs = _thd(q, "q")
    (Tk, Hk, Dk), ks = _thd(k, "k")
    shp_v, vs = _thd(v, "v")
    if (Hk, Dk) != (H, D) or shp_v != (Tk, Hk, Dk):
        raise ValueError(f"shape mismatch: q {tuple(q.shape)} k {tuple(k.shape)} v {tuple(v.shape)}")
    cu_q, cu_k = _cu(cu_seqlens_q, q.device, "cu_seqlens_q"), _cu(cu_seqlens_k, q.device, "cu_seqlens_k")
    if cu_q.numel() != cu_k.numel():
        raise ValueError("cu_seqlens_q and cu_seqlens_k must describe the same number of sequences")
    if softmax_scale is None:
        softmax_scale = D ** (-0.5)
    if out is None:
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    if lse is None:
        lse = torch.empty((H, Tq), dtype=torch.float32, device=q.device)
    _, os_ = _thd(out, "out")
    tail = (cu_q.data_ptr(), cu_k.data_ptr(), cu_q.numel() - 1, H, Tq, Tk, int(max_seqlen_q), int(max_seqlen_k), D,
            _lib.strides2(qs), _lib.strides2(ks), _lib.strides2(vs), _lib.strides2(os_),
            float(softmax_scale), _lib.SPA_MASK_CAUSAL if causal else _lib.SPA_MASK_NONE, _dtype_code(q), _stream())
    with _on(q.device):
        if fp8:
            ksc, vsc = _fp8_scales(k, v, k_scale, v_scale, cu_q.numel() - 1, H)
            _lib.check(lib.spa_flash_fwd_varlen_fp8kv(q.data_ptr(), k.data_ptr(), v.data_ptr(), ksc.data_ptr(), vsc.data_ptr(),
                                                      out.data_ptr(), lse.data_ptr(), *tail))
        else:
            _lib.check(lib.spa_flash_fwd_varlen(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(), *tail))
    return out, lse


def ring_fwd_varlen(q, k, v, cu_seqlens, max_seqlen, ring_size, softmax_scale=None, causal=False, rank=-1, fuse="rank", out=None,
                    lse=None):
    """Ring forward over a packed variable-length batch: q, k, v [P * T, H, D] = P stacked shards (rank r holds the r-th of
    P equal slices of every sequence), cu_seqlens int32 [nseq + 1] the layout of one shard of T rows.  One launch per
    rank (fuse="rank") or one for all ranks ("all").  Returns (out like q, lse fp32 [H, P * T]).  Calls spa_ring_fwd_varlen
    (bf16 / fp16)."""
    lib = _lib.load()
    q, k, v = _prep(q), _prep(k), _prep(v)
    if not (q.dtype == k.dtype == v.dtype):
        raise TypeError("q, k, v must share a dtype")
    (PT, H, D), qs = _thd(q, "q")
    shp_k, ks = _thd(k, "k")
    shp_v, vs = _thd(v, "v")
    P = int(ring_size)
    if shp_k != (PT, H, D) or shp_v != (PT, H, D) or P < 1 or PT % P:
        raise ValueError(f"ring over a packed batch: q, k, v of one shape whose rows ring_size={P} divides, got {tuple(q.shape)} "
                         f"{tuple(k.shape)} {tuple(v.shape)}")
    if fuse not in ("rank", "all"):
        raise ValueError(f"fuse must be 'rank' or 'all', got {fuse!r}")
    cu = _cu(cu_seqlens, q.device, "cu_seqlens")
    if softmax_scale is None:
        softmax_scale = D ** (-0.5)
    if out is None:
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    if lse is None:
        lse = torch.empty((H, PT), dtype=torch.float32, device=q.device)
    _, os_ = _thd(out, "out")
    with _on(q.device):
        _lib.check(lib.spa_ring_fwd_varlen(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(), cu.data_ptr(), cu.numel() - 1, H, PT // P,
            int(max_seqlen), D, P, int(rank), _lib.strides2(qs), _lib.strides2(ks), _lib.strides2(vs), _lib.strides2(os_),
            float(softmax_scale), _lib.SPA_MASK_CAUSAL if causal else _lib.SPA_MASK_NONE, _dtype_code(q), RING_FUSE[fuse], _stream()))
    return out, lse


def _flash_bwd_varlen(name, q, k, v, dout, lse, delta, dq, dk, dv, grad_dtype, cu_seqlens_q, cu_seqlens_k,
                      max_seqlen_q, max_seqlen_k, softmax_scale, causal):
    if not (q.dtype == k.dtype == v.dtype == dout.dtype):
        raise TypeError(f"{name}: q, k, v, dout must share a dtype")
    (Tq, H, D), _ = _thd(q, "q")
    shp_k, shp_v, shp_do = _thd(k, "k")[0], _thd(v, "v")[0], _thd(dout, "dout")[0]
    shp_dq, dqs = _thd(dq, "dq")
    shp_dk, dks = _thd(dk, "dk")
    shp_dv, dvs = _thd(dv, "dv")
    Tk = shp_k[0]
    # the kernels index the gradients with q's / k's sizes: a mismatch would be an out-of-bounds access
    if shp_k != (Tk, H, D) or shp_v != shp_k or shp_dk != shp_k or shp_dv != shp_k:
        raise ValueError(f"{name}: k {shp_k}, v {shp_v}, dk {shp_dk}, dv {shp_dv} must agree (heads and head dim as q {tuple(q.shape)})")
    if shp_do != (Tq, H, D) or shp_dq != (Tq, H, D):
        raise ValueError(f"{name}: dout {shp_do} and dq {shp_dq} must have q's shape {tuple(q.shape)}")
    for t in (lse, delta):
        if t.dtype != torch.float32:
            raise TypeError(f"{name}: lse and delta must be float32")
    for t in (dq, dk, dv):
        if t.dtype != grad_dtype:
            raise TypeError(f"{name}: dq, dk, dv must be {grad_dtype}")
    for t in (dq, dk, dv, lse, delta):
        if t.device != q.device:
            raise ValueError(f"{name}: every tensor must live on q's device")
    if tuple(lse.shape) != (H, Tq) or tuple(delta.shape) != (H, Tq) or not lse.is_contiguous() or not delta.is_contiguous():
        raise ValueError("lse and delta must be contiguous [H, total_q]")
    if cu_seqlens_q.numel() != cu_seqlens_k.numel():
        raise ValueError("cu_seqlens_q and cu_seqlens_k must describe the same number of sequences")
    lib = _lib.load()
    q, k, v, dout = _prep(q), _prep(k), _prep(v), _prep(dout)
    qs, ks, vs, dos = _thd(q, "q")[1], _thd(k, "k")[1], _thd(v, "v")[1], _thd(dout, "dout")[1]
    gsz = dq.element_size()
    if not (_rows_ok(dq, gsz) and _rows_ok(dk, gsz) and _rows_ok(dv, gsz)):
        raise ValueError(f"{name}: dq, dk, dv need an inner stride of 1 and 16-byte aligned rows")
    cu_q, cu_k = _cu(cu_seqlens_q, q.device, "cu_seqlens_q"), _cu(cu_seqlens_k, q.device, "cu_seqlens_k")
    if softmax_scale is None:
        softmax_scale = D ** (-0.5)
    with _on(q.device):
        _lib.check(getattr(lib, name)(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), dout.data_ptr(), lse.data_ptr(), delta.data_ptr(),
            dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), cu_q.data_ptr(), cu_k.data_ptr(),
            cu_q.numel() - 1, H, Tq, Tk, int(max_seqlen_q), int(max_seqlen_k), D,
            _lib.strides2(qs), _lib.strides2(ks), _lib.strides2(vs), _lib.strides2(dos), _lib.strides2(dqs),
            _lib.strides2(dks), _lib.strides2(dvs),
            float(softmax_scale), _lib.SPA_MASK_CAUSAL if causal else _lib.SPA_MASK_NONE, _dtype_code(q), _stream()))


def flash_bwd_varlen(q, k, v, dout, lse, delta, dq_acc, dk_acc, dv_acc, cu_seqlens_q, cu_seqlens_k, max_seqlen_q,
                     max_seqlen_k, softmax_scale=None, causal=False):
    """Backward of flash_fwd_varlen; adds into the fp32 accumulators dq [total_q,H,D], dk, dv
    [total_k,H,D].  lse, delta: fp32 [H,total_q].  Calls spa_flash_bwd_varlen."""
    _flash_bwd_varlen("spa_flash_bwd_varlen", q, k, v, dout, lse, delta, dq_acc, dk_acc, dv_acc, torch.float32,
                      cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, softmax_scale, causal)


def flash_bwd_varlen_out(q, k, v, dout, lse, delta, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
                         softmax_scale=None, causal=False, dq=None, dk=None, dv=None, rows_covered=False):
    """Backward of flash_fwd_varlen in one call: returns (dq, dk, dv) in q's dtype, written by the
    kernels (no fp32 accumulators).  The kernels write the rows of the sequences cu_seqlens names, up
    to max_seqlen each: a row of no sequence is not touched.  Gradients allocated here therefore start
    as zeros unless the caller vouches with rows_covered=True that the offsets end at the tensors' row
    counts and no sequence exceeds max_seqlen (what check_cu_seqlens establishes); tensors passed in
    as dq / dk / dv are the caller's to initialise.  Calls spa_flash_bwd_varlen_out."""
    alloc = torch.empty if rows_covered else torch.zeros
    dq = alloc(q.shape, dtype=q.dtype, device=q.device) if dq is None else dq
    dk = alloc(k.shape, dtype=q.dtype, device=q.device) if dk is None else dk
    dv = alloc(v.shape, dtype=q.dtype, device=q.device) if dv is None else dv
    _flash_bwd_varlen("spa_flash_bwd_varlen_out", q, k, v, dout, lse, delta, dq, dk, dv, q.dtype,
                      cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, softmax_scale, causal)
    return dq, dk, dv
