"""Block attention operator with the reference's names and argument meaning, over the HIP kernels.

Mirrors sp_aurora/intel_flash_attn.py (intel_flash_attn_forward :18-126,
intel_flash_attn_backward :129-157, aliases :161-168) and the plugin shim
sp_aurora/intel_flash_attn_sycl.py:40-144.  Tensors are in the operator layout
[batch, heads, seq, head_dim]; the result is (out like q, lse fp32 [batch, heads, seq_q]).
"""
import torch

from . import ops


def _check_unsupported(dropout_p, window_size, alibi_slopes, return_softmax=False):
    if alibi_slopes is not None:
        # the reference asserts the same in its autograd Function
        # (sp_aurora/intel_ring_flash_attn.py:295)
        raise AssertionError("alibi_slopes is not supported")
    if dropout_p and dropout_p > 0.0:
        raise NotImplementedError("dropout is not supported (the reference lists it as unsupported too)")
    if window_size is not None and tuple(window_size) != (-1, -1):
        raise NotImplementedError("sliding-window attention is not supported; pass window_size=(-1, -1)")
    if return_softmax:
        raise NotImplementedError("returning the attention matrix is not supported; the kernel never forms it")


def intel_flash_attn_forward(q, k, v, dropout_p=0.0, softmax_scale=None, causal=False,
                             window_size=(-1, -1), alibi_slopes=None, return_softmax=False, **kwargs):
    """out = softmax(q k^T * scale + mask) v and lse = logsumexp(...), one fused HIP kernel.

    q [B,H,Sq,D], k,v [B,H,Sk,D] (any strides with a contiguous head dim).  `causal` is the
    reference's top-left aligned mask (sp_aurora/intel_flash_attn.py:79-84).
    softmax_scale None -> D ** -0.5 (:46-47).  Returns (out [B,H,Sq,D] in q.dtype, lse fp32 [B,H,Sq]).

    Additive: k, v may be torch.float8_e4m3fn (a quantised KV cache) with keyword arguments
    k_scale, v_scale (fp32 [B,H]: K = k * k_scale[b,h], V = v * v_scale[b,h]); q stays bf16 / fp16, or is
    torch.float8_e4m3fn too with q_scale (fp32 [B,H]) and out_dtype (bf16 / fp16): D = 128, scores on the 8-bit
    matrix instruction.
    """
    _check_unsupported(dropout_p, window_size, alibi_slopes, return_softmax)
    return ops.flash_fwd(q, k, v, softmax_scale, bool(causal), layout="bhsd",
                         k_scale=kwargs.get("k_scale"), v_scale=kwargs.get("v_scale"), q_scale=kwargs.get("q_scale"),
                         out_dtype=kwargs.get("out_dtype", torch.bfloat16))


def intel_flash_attn_backward(dout, q, k, v, out, softmax_lse, dq=None, dk=None, dv=None, dropout_p=0.0,
                              softmax_scale=None, causal=False, window_size=(-1, -1), alibi_slopes=None,
                              deterministic=False, rng_state=None, **kwargs):
    """Gradients of the block operator given its saved (out, lse); operator layout [B,H,S,D].

    The reference's function of this name is an empty stub (sp_aurora/intel_flash_attn.py:129-157)
    and its ring backward re-runs autograd per block instead
    (sp_aurora/intel_ring_flash_attn.py:229-244); this one does the block-wise recompute
    with the given lse (spa_flash_bwd_out: no fp32 accumulators to zero, read back and cast).
    Writes into dq/dk/dv when given (flash-attn convention) and returns them.
    """
    _check_unsupported(dropout_p, window_size, alibi_slopes)
    delta = ops.bwd_delta(out, dout, layout="bhsd")
    lse = softmax_lse if softmax_lse.is_contiguous() else softmax_lse.contiguous()
    # one call computes the whole gradient of the block: the kernels write it in the inputs' type,
    # straight into dq / dk / dv when those are given in a form the kernels can write
    given = (dq, dk, dv)
    direct = [g if g is not None and g.dtype == q.dtype and g.shape == like.shape and ops._rows_ok(g, g.element_size()) else None
              for g, like in zip(given, (q, k, v))]
    res = ops.flash_bwd_out(q, k, v, dout, lse, delta, softmax_scale, bool(causal), layout="bhsd",
                            dq=direct[0], dk=direct[1], dv=direct[2])
    out_grads = []
    for got, dst, was_direct in zip(res, given, direct):
        if dst is not None and was_direct is None:
            dst.copy_(got)
            got = dst
        out_grads.append(got)
    return tuple(out_grads)


# the names the ring code imports (sp_aurora/intel_flash_attn.py:161-168)
_flash_attn_forward = intel_flash_attn_forward
_flash_attn_backward = intel_flash_attn_backward


def is_available():
    """True when the HIP library loads and a device is visible; mirrors is_sycl_available
    (sp_aurora/intel_flash_attn_sycl.py:147-149)."""
    try:
        from . import _lib
        _lib.load()
    except (ImportError, OSError):
        return False
    return torch.cuda.is_available()


def get_device_info():
    """Mirrors get_sycl_device_info (sp_aurora/intel_flash_attn_sycl.py:152-160)."""
    from . import _lib
    return _lib.device_info()
