"""sp_aurora attention hot path on AMD Instinct MI355X (gfx950).

The package keeps the names sp_aurora exports for this path (sp_aurora/__init__.py:59-122)
so that `import sp_aurora_amd as sp_aurora` is a drop-in for: the block attention operator,
update_out_and_lse, the ring attention functions (documented in the reference's README as
sp_aurora_func / sp_aurora_kvpacked_func / sp_aurora_qkvpacked_func) and the Ulysses
re-layout and attention functions.  All compute runs in libsp_aurora_hip.so (hand-written
HIP kernels behind a C ABI, see include/sp_aurora_hip.h); importing the package without the
built library fails at the first call.
"""
from . import _lib, ops  # noqa: F401
from .flash_attn import (  # noqa: F401
    _flash_attn_backward,
    _flash_attn_forward,
    get_device_info,
    intel_flash_attn_backward,
    intel_flash_attn_forward,
    is_available,
)
from .layers import (  # noqa: F401
    HAS_FLASH_ATTN,
    HAS_LONG_CTX_ATTN,
    HAS_SPARSE_SAGE_ATTENTION,
    AttnType,
    LongContextAttention,
    UlyssesAttention,
    pytorch_attn_forward,
    pytorch_attn_func,
    ring_pytorch_attn_forward,
    ring_pytorch_attn_func,
    select_flash_attn_impl,
)
from .ring import (  # noqa: F401
    IntelRingFlashAttnFunc,
    RingFlashAttnFunc,
    intel_ring_flash_attn_func,
    intel_ring_flash_attn_kvpacked_func,
    intel_ring_flash_attn_qkvpacked_func,
    ring_flash_attn_backward,
    ring_flash_attn_forward,
    ring_flash_attn_forward_rank,
    ring_flash_attn_func,
    ring_flash_attn_kvpacked_func,
    ring_flash_attn_qkvpacked_func,
    sp_aurora_func,
    sp_aurora_kvpacked_func,
    sp_aurora_qkvpacked_func,
)
from .ulysses import (  # noqa: F401
    IntelSeqAllToAll4D,
    SeqAllToAll4D,
    SeqAllToAll5D,
    all_to_all_4D,
    all_to_all_5D,
    intel_all_to_all_4d,
    intel_ulysses_flash_attn_forward,
    intel_ulysses_flash_attn_func,
    intel_ulysses_flash_attn_kvpacked_func,
    intel_ulysses_flash_attn_qkvpacked_func,
    ulysses_flash_attn_func,
    ulysses_flash_attn_kvpacked_func,
    ulysses_flash_attn_qkvpacked_func,
)
from .utils import flatten_varlen_lse, unflatten_varlen_lse, update_out_and_lse  # noqa: F401
from .varlen import (VarlenFlashAttnFunc, ring_flash_attn_varlen_func, sp_aurora_varlen_func,  # noqa: F401
                     zigzag_sp_aurora_varlen_func, zigzag_varlen_order)

SeqAllToAll4D_v2 = SeqAllToAll4D  # sp_aurora/__init__.py:77

__version__ = "0.1.0"
