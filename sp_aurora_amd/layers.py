"""The attention modules that sit on top of the ring and Ulysses functions, on one GPU.

Mirrors sp_aurora/ulysses/attn_layer.py (AttnType :23-35, select_flash_attn_impl :38-137,
UlyssesAttention :140-252) and sp_aurora/hybrid/long_ctx_attention.py (LongContextAttention
:19-260).  The reference's modules take one rank's shard and a process group; here one GPU
holds every rank's shard stacked on a leading axis ([W, B, s, H, D], rank w owns sequence
rows w*s .. (w+1)*s), and the degrees say how the W ranks split into Ulysses groups and ring
groups.  Ranks of one Ulysses group are neighbours (w = g*U + i), ranks of one ring group
share i: after the head-scatter / sequence-gather exchange inside each Ulysses group, rank
(g, i) holds rows g*U*s .. (g+1)*U*s of head slice i, and the ring over g walks those row
blocks in order.

Every attention implementation the reference can select maps to the same HIP kernels.
"""
from enum import Enum

import torch

from .flash_attn import _check_unsupported
from .ring import _no_multi_gpu, ring_flash_attn_func
from .ulysses import SeqAllToAll4D, ulysses_flash_attn_func

__all__ = ["AttnType", "select_flash_attn_impl", "UlyssesAttention", "LongContextAttention", "pytorch_attn_forward",
           "pytorch_attn_func", "ring_pytorch_attn_func", "ring_pytorch_attn_forward", "HAS_LONG_CTX_ATTN",
           "HAS_FLASH_ATTN", "HAS_SPARSE_SAGE_ATTENTION"]

# sp_aurora/globals.py:171-173
HAS_LONG_CTX_ATTN = True
HAS_FLASH_ATTN = True
HAS_SPARSE_SAGE_ATTENTION = False


class AttnType(str, Enum):
    """sp_aurora/ulysses/attn_layer.py:23-35 — kept so that callers' configuration still parses."""
    TORCH = "torch"
    INTEL_SYCL = "intel_sycl"
    INTEL_ONEDNN = "intel_onednn"
    FA = "flash_attn"
    FA3 = "flash_attn_3"


def _local_attention(q, k, v, dropout_p=0.0, softmax_scale=None, causal=False, window_size=(-1, -1),
                     softcap=0.0, alibi_slopes=None, deterministic=False, return_attn_probs=False):
    """Attention of [B,S,H,D] tensors on this GPU; with return_attn_probs also the fp32 lse
    [B,H,S] (the second value of the reference's functions, attn_layer.py:84-86,119-126)."""
    if softcap:
        raise NotImplementedError("softcap is not supported")
    res = ring_flash_attn_func(q, k, v, dropout_p, softmax_scale, causal, window_size, alibi_slopes,
                               deterministic, return_attn_probs, None, ring_size=1)
    return res[:2] if return_attn_probs else res


def pytorch_attn_forward(q, k, v, dropout_p=0.0, softmax_scale=None, causal=False, window_size=(-1, -1), softcap=0.0,
                         alibi_slopes=None, deterministic=False, return_attn_probs=False):
    """sp_aurora/kernels/attention.py:12-86 with its documented layout (batch, seq_len, num_heads,
    head_dim): -> (out, None).  The reference's second value is the materialised S x S probability
    matrix, which these kernels never form: return_attn_probs raises."""
    if return_attn_probs:
        raise NotImplementedError("the attention probabilities are not materialised")
    return _local_attention(q, k, v, dropout_p, softmax_scale, causal, window_size, softcap, alibi_slopes,
                            deterministic, False), None


def pytorch_attn_func(q, k, v, dropout_p=0.0, softmax_scale=None, causal=False, window_size=(-1, -1), softcap=0.0,
                      alibi_slopes=None, deterministic=False, return_attn_probs=False):
    """sp_aurora/kernels/attention.py:89-117: the output of pytorch_attn_forward."""
    return pytorch_attn_forward(q, k, v, dropout_p, softmax_scale, causal, window_size, softcap, alibi_slopes,
                                deterministic, return_attn_probs)[0]


def ring_pytorch_attn_func(q, k, v, dropout_p=0.0, softmax_scale=None, causal=False, window_size=(-1, -1),
                           alibi_slopes=None, deterministic=False, return_attn_probs=False, group=None, *, ring_size=1):
    """sp_aurora/ring_pytorch_attn.py:20-197, the reference's second ring implementation: the same
    result as ring_flash_attn_func, through the same kernels."""
    out = ring_flash_attn_func(q, k, v, dropout_p, softmax_scale, causal, window_size, alibi_slopes, deterministic,
                               return_attn_probs, group, ring_size=ring_size)
    return out[:2] if return_attn_probs else out


def ring_pytorch_attn_forward(q, k, v, dropout_p=0.0, softmax_scale=None, causal=False, window_size=(-1, -1),
                              alibi_slopes=None, deterministic=False, return_attn_probs=False, group=None, *,
                              ring_size=1):
    """sp_aurora/ring_pytorch_attn.py:200-226: -> (out, lse); the reference returns None for the lse
    unless return_attn_probs, this returns the fp32 [B,H,S] lse either way."""
    out, lse, _ = ring_flash_attn_func(q, k, v, dropout_p, softmax_scale, causal, window_size, alibi_slopes,
                                       deterministic, True, group, ring_size=ring_size)
    return out, lse


def select_flash_attn_impl(attn_type):
    """sp_aurora/ulysses/attn_layer.py:38-137: a callable (q, k, v, dropout_p, softmax_scale, causal,
    window_size, softcap, alibi_slopes, deterministic, return_attn_probs) -> out or (out, lse)."""
    AttnType(attn_type)  # raises ValueError for a name the reference does not know
    return _local_attention


class UlyssesAttention(torch.nn.Module):
    """sp_aurora/ulysses/attn_layer.py:140-252.  forward takes the rank-stacked [P,B,s,H,D]
    tensors of a Ulysses group (or one rank's [B,S,H,D], a world of one) and returns the
    output in the same layout."""

    def __init__(self, sequence_process_group=None, scatter_idx=2, gather_idx=1, use_sync=False,
                 attn_type=AttnType.TORCH):
        super().__init__()
        _no_multi_gpu(sequence_process_group)
        if (scatter_idx, gather_idx) != (2, 1):
            raise ValueError(f"Unsupported scatter_idx={scatter_idx}, gather_idx={gather_idx}")
        self.spg = sequence_process_group
        self.scatter_idx = scatter_idx
        self.gather_idx = gather_idx
        self.use_sync = use_sync
        self.attn_type = AttnType(attn_type)
        self.attn_fn = select_flash_attn_impl(self.attn_type)

    def forward(self, query, key, value, dropout_p=0.0, softmax_scale=None, causal=False,
                window_size=(-1, -1), softcap=0.0, alibi_slopes=None, deterministic=False,
                return_attn_probs=False, *args):
        if softcap:
            raise NotImplementedError("softcap is not supported")
        if query.dim() == 4:
            # world size 1 (attn_layer.py:203-215)
            return self.attn_fn(query, key, value, dropout_p, softmax_scale, causal, window_size, softcap,
                                alibi_slopes, deterministic, return_attn_probs)
        out = ulysses_flash_attn_func(query, key, value, dropout_p, softmax_scale, causal, window_size,
                                      alibi_slopes, deterministic, False, self.spg)
        if self.use_sync:
            torch.cuda.synchronize()
        return out


class LongContextAttention(torch.nn.Module):
    """Ulysses inside groups of `sp_ulysses_degree` neighbouring ranks, ring attention across
    `sp_ring_degree` such groups (sp_aurora/hybrid/long_ctx_attention.py:19-260).

    forward takes rank-stacked [W,B,s,H,D] tensors, W = sp_ulysses_degree * sp_ring_degree,
    and returns the output in the same layout.  With both degrees 1 the tensors may also be
    one rank's [B,S,H,D]."""

    def __init__(self, scatter_idx=2, gather_idx=1, sp_ulysses_degree=None, sp_ring_degree=None,
                 use_ulysses=True, use_ring=True, ulysses_pg=None, ring_pg=None, attn_type=AttnType.FA,
                 use_pack_qkv=False, use_sync=False):
        super().__init__()
        _no_multi_gpu(ulysses_pg)
        _no_multi_gpu(ring_pg)
        if (scatter_idx, gather_idx) != (2, 1):
            raise ValueError(f"Unsupported scatter_idx={scatter_idx}, gather_idx={gather_idx}")
        self.attn_type = AttnType(attn_type)
        self.sp_ulysses_degree = int(sp_ulysses_degree or 1)
        self.sp_ring_degree = int(sp_ring_degree or 1)
        if self.sp_ulysses_degree < 1 or self.sp_ring_degree < 1:
            raise ValueError("degrees must be positive")
        self.use_ulysses = bool(use_ulysses) and self.sp_ulysses_degree > 1
        self.use_ring = bool(use_ring) and self.sp_ring_degree > 1
        self.ulysses_pg = ulysses_pg
        self.ring_pg = ring_pg
        self.scatter_idx = scatter_idx
        self.gather_idx = gather_idx
        self.use_pack_qkv = use_pack_qkv
        self.use_sync = use_sync
        self.ulysses_attn = (UlyssesAttention(ulysses_pg, scatter_idx, gather_idx, use_sync, self.attn_type)
                             if self.use_ulysses else None)

    # ---- the exchange of one Ulysses group, and its inverse ----
    def _scatter_heads(self, tensors):
        """[U,B,s,H,D] each -> [U,B,U*s,H/U,D] each; packed = one exchange for all of them, the
        tensors side by side on the batch axis (long_ctx_attention.py:143-152)."""
        if self.use_pack_qkv and len(tensors) > 1:
            packed = SeqAllToAll4D.apply(self.ulysses_pg, torch.cat(tensors, dim=1), self.scatter_idx,
                                         self.gather_idx)
            return list(torch.chunk(packed, len(tensors), dim=1))
        return [SeqAllToAll4D.apply(self.ulysses_pg, t.contiguous(), self.scatter_idx, self.gather_idx)
                for t in tensors]

    def forward(self, query, key, value, dropout_p=0.0, softmax_scale=None, causal=False,
                window_size=(-1, -1), softcap=0.0, alibi_slopes=None, deterministic=False,
                return_attn_probs=False, joint_tensor_key_value=None):
        if softcap:
            raise NotImplementedError("softcap is not supported")
        _check_unsupported(dropout_p, window_size, alibi_slopes)
        if joint_tensor_key_value is not None:
            # [..., s, 2, H, D] (long_ctx_attention.py:136-138)
            key, value = joint_tensor_key_value.unbind(dim=-3)
        U = self.sp_ulysses_degree if self.use_ulysses else 1
        R = self.sp_ring_degree if self.use_ring else 1
        W = U * R
        if query.dim() == 4:
            if W != 1:
                raise ValueError(f"expected rank-stacked [{W},B,s,H,D] tensors, got {tuple(query.shape)}")
            return _local_attention(query, key, value, dropout_p, softmax_scale, causal, window_size, softcap,
                                    alibi_slopes, deterministic, False)
        if query.dim() != 5 or query.shape[0] != W:
            raise ValueError(f"expected rank-stacked [{W},B,s,H,D] tensors, got {tuple(query.shape)}")
        _, B, s, H, D = query.shape
        if H % U:
            raise ValueError(f"heads {H} must be divisible by the Ulysses degree {U}")
        if softmax_scale is None:
            softmax_scale = D ** (-0.5)

        if U == 1:
            # ring only (:198-213): the stacked shards are the ring's chunks
            if B == 1:
                full = lambda t: t.reshape(1, W * s, H, D)
            else:
                full = lambda t: t.transpose(0, 1).reshape(B, W * s, H, D)
            out = ring_flash_attn_func(full(query), full(key), full(value), dropout_p, softmax_scale, causal,
                                       window_size, alibi_slopes, deterministic, False, self.ring_pg, ring_size=R)
            out = out.view(B, W, s, H, D).transpose(0, 1)
            return out if B == 1 else out.contiguous()
        if R == 1:
            # Ulysses only (:216-229)
            return self.ulysses_attn(query, key, value, dropout_p, softmax_scale, causal, window_size, softcap,
                                     alibi_slopes, deterministic, False)

        # hybrid (:141-195): exchange inside each Ulysses group, ring across the groups
        h = H // U
        groups = [self._scatter_heads([t[g * U:(g + 1) * U] for t in (query, key, value)]) for g in range(R)]
        # [U,B,R*U*s,h,D]: head slice i of the whole sequence; the U slices fold into the batch
        ql, kl, vl = (torch.cat([groups[g][j] for g in range(R)], dim=2).view(U * B, W * s, h, D) for j in range(3))
        ol = ring_flash_attn_func(ql, kl, vl, dropout_p, softmax_scale, causal, window_size, alibi_slopes,
                                  deterministic, False, self.ring_pg, ring_size=R)
        ol = ol.view(U, B, R, U * s, h, D)
        outs = [SeqAllToAll4D.apply(self.ulysses_pg, ol[:, :, g].contiguous(), self.gather_idx, self.scatter_idx)
                for g in range(R)]
        if self.use_sync:
            torch.cuda.synchronize()
        return torch.cat(outs, dim=0)

    def get_sequence_parallel_degree(self):
        return self.sp_ulysses_degree * self.sp_ring_degree

    def get_ulysses_degree(self):
        return self.sp_ulysses_degree

    def get_ring_degree(self):
        return self.sp_ring_degree
