"""ctypes binding of libsp_aurora_hip.so — the only way this package reaches the GPU kernels.

The library must have been built (``python -m sp_aurora_amd.build``); there is no
fallback path: a missing library raises, it never degrades to torch ops.
"""
import ctypes
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libsp_aurora_hip.so")

SPA_F32, SPA_BF16, SPA_F16 = 0, 1, 2
SPA_MASK_NONE, SPA_MASK_CAUSAL = 0, 1
SPA_RING_PER_STEP, SPA_RING_PER_RANK, SPA_RING_ALL_RANKS = 0, 1, 2
SPA_RING_ZIGZAG = 16  # or-ed into `fuse`: the rows are in zigzag-sharded order

_I64x3 = ctypes.c_int64 * 3
_vp = ctypes.c_void_p
_i = ctypes.c_int
_f = ctypes.c_float
_s3 = ctypes.POINTER(ctypes.c_int64)

# name -> (restype, argtypes); mirrors include/sp_aurora_hip.h declaration by declaration
SIGNATURES = {
    "spa_abi_version": (_i, []),
    "spa_last_error": (ctypes.c_char_p, []),
    "spa_device_info": (_i, [ctypes.c_char_p, _i]),
    "spa_flash_fwd": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _s3, _s3, _s3, _s3, _f, _i, _i, _vp]),
    "spa_flash_fwd_fp8kv": (_i, [_vp] * 7 + [_i] * 5 + [_s3] * 4 + [_f, _i, _i, _vp]),
    "spa_flash_fwd_fp8qkv": (_i, [_vp] * 8 + [_i] * 5 + [_s3] * 4 + [_f, _i, _i, _vp]),
    "spa_flash_fwd_varlen_fp8kv": (_i, [_vp] * 9 + [_i] * 7 + [_s3] * 4 + [_f, _i, _i, _vp]),
    "spa_ring_fwd_fp8kv": (_i, [_vp] * 8 + [_i] * 6 + [_s3] * 4 + [_f, _i, _i, _i, _vp]),
    "spa_ring_fwd_fp8qkv": (_i, [_vp] * 9 + [_i] * 6 + [_s3] * 4 + [_f, _i, _i, _i, _vp]),
    "spa_ring_fwd_flags": (_i, [_vp] * 6 + [ctypes.c_uint32, ctypes.c_uint32, _vp] + [_i] * 6 + [_s3] * 4 + [_f, _i, _i, _vp]),
    "spa_ring_fwd_flags_fp8qkv": (_i, [_vp] * 9 + [ctypes.c_uint32, ctypes.c_uint32, _vp] + [_i] * 6 + [_s3] * 4 + [_f, _i, _i, _vp]),
    "spa_ring_flag_set": (_i, [_vp, _i, ctypes.c_uint32, _vp]),
    "spa_ring_fwd_workspace_bytes": (ctypes.c_int64, [_i, _i, _i, _i, _i, _i]),
    "spa_flash_fwd_splitkv_workspace_bytes": (ctypes.c_int64, [_i, _i, _i, _i, _i, _i]),
    "spa_flash_fwd_splitkv_suggest": (_i, [_i, _i, _i, _i, _i, _i, _i]),
    "spa_flash_fwd_splitkv": (_i, [_vp] * 6 + [_i] * 6 + [_s3] * 4 + [_f, _i, _vp]),
    "spa_flash_fwd_splitkv_fp8kv": (_i, [_vp] * 8 + [_i] * 6 + [_s3] * 4 + [_f, _i, _vp]),
    "spa_ring_fwd": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _s3, _s3, _s3, _s3, _f, _i, _i, _i, _vp]),
    "spa_static_scratch_bytes": (ctypes.c_int64, []),
    "spa_static_scratch_init": (_i, []),
    "spa_ring_fwd_static": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _s3, _s3, _s3, _s3, _f, _i, _i, _i, _vp]),
    "spa_tune": (_i, [_i, _i]),
    "spa_merge": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _s3, _s3, _i, _i, _vp]),
    "spa_finalize": (_i, [_vp, _vp, _i, _i, _i, _i, _s3, _s3, _i, _vp]),
    "spa_relayout_s2h": (_i, [_vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "spa_relayout_h2s": (_i, [_vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "spa_bwd_delta": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _s3, _s3, _i, _vp]),
    "spa_flash_bwd": (_i, [_vp] * 9 + [_i] * 5 + [_s3] * 7 + [_f, _i, _i, _vp]),
    "spa_flash_bwd_out": (_i, [_vp] * 9 + [_i] * 5 + [_s3] * 7 + [_f, _i, _i, _vp]),
    "spa_flash_fwd_varlen": (_i, [_vp] * 7 + [_i] * 7 + [_s3] * 4 + [_f, _i, _i, _vp]),
    "spa_ring_fwd_varlen": (_i, [_vp] * 6 + [_i] * 7 + [_s3] * 4 + [_f, _i, _i, _i, _vp]),
    "spa_flash_bwd_varlen": (_i, [_vp] * 11 + [_i] * 7 + [_s3] * 7 + [_f, _i, _i, _vp]),
    "spa_flash_bwd_varlen_out": (_i, [_vp] * 11 + [_i] * 7 + [_s3] * 7 + [_f, _i, _i, _vp]),
}

_lib = None


class SpaError(RuntimeError):
    """A negative return code from the C ABI; .code holds it."""

    def __init__(self, code, msg):
        super().__init__(f"[spa {code}] {msg}")
        self.code = code


# entry points that return an int but launch nothing: they run as they are while recording
_QUERIES = ("spa_abi_version", "spa_tune", "spa_device_info", "spa_static_scratch_init", "spa_flash_fwd_splitkv_suggest")


class _Recorder:
    """Stands in for the library while ops.prepared() records a call sequence: every spa_* call is
    stored with its arguments converted to ctypes objects once, and reports success."""

    def __init__(self, lib):
        self._lib = lib
        self.calls = []

    def __getattr__(self, name):
        fn = getattr(self._lib, name)
        if name not in SIGNATURES or fn.restype is not _i or name in _QUERIES:
            return fn  # queries run as they are

        def record(*args):
            if len(args) != len(fn.argtypes):
                raise TypeError(f"{name}: expected {len(fn.argtypes)} arguments, got {len(args)}")
            cargs = tuple(a if isinstance(a, ctypes.Array) else t(a) for a, t in zip(args, fn.argtypes))
            self.calls.append((fn, cargs))
            return 0

        return record


# the recorder of ops.prepared() belongs to the thread that records: other threads keep calling the library
_tls = threading.local()


def load():
    """Load the shared library once and attach the prototypes.  Raises if it was not built."""
    global _lib
    rec = getattr(_tls, "recorder", None)
    if rec is not None:
        return rec
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} not found: build it with `python -m sp_aurora_amd.build` "
            "(sp_aurora_amd has no non-HIP path)"
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    if lib.spa_abi_version() != 1:
        raise ImportError(f"{LIB_PATH}: ABI version {lib.spa_abi_version()} != 1")
    _lib = lib
    return lib


_STRIDE_CACHE = {}


def _strides(vals, n):
    """An int64[n] argument; the arrays are read-only for the library, so equal stride tuples share one."""
    key = tuple(vals)
    arr = _STRIDE_CACHE.get(key)
    if arr is None:
        if len(key) != n:
            raise ValueError(f"expected {n} strides, got {key}")
        if len(_STRIDE_CACHE) > 4096:
            _STRIDE_CACHE.clear()
        arr = _STRIDE_CACHE[key] = (ctypes.c_int64 * n)(*[int(v) for v in key])
    return arr


def strides3(vals):
    return _strides(vals, 3)


def strides2(vals):
    return _strides(vals, 2)


class recording:
    """Context manager: inside it, load() hands the calling thread a recorder instead of the library."""

    def __enter__(self):
        if getattr(_tls, "recorder", None) is not None:
            raise RuntimeError("recording() does not nest")
        lib = load()
        _tls.recorder = _Recorder(lib)
        return _tls.recorder

    def __exit__(self, *exc):
        _tls.recorder = None
        return False


def check(code):
    if code != 0:
        raise SpaError(code, load().spa_last_error().decode("utf-8", "replace"))


TUNE_KNOBS = {"fwd_groups": 0, "fwd_share": 1, "bwd_dq_waves": 2, "bwd_dkdv_form": 3, "fwd32_split": 4, "few_rows": 5}


def tune(knob, value):
    """Kernel-variant override for experiments and tests (spa_tune); value 0 = the library's choice."""
    check(load().spa_tune(TUNE_KNOBS[knob], int(value)))


def device_info():
    buf = ctypes.create_string_buffer(512)
    check(load().spa_device_info(buf, 512))
    return dict(kv.split("=", 1) for kv in buf.value.decode().split(";"))
