"""update_out_and_lse over the HIP merge kernel; mirrors sp_aurora/utils.py:47-147.

Shapes are the reference's: the block operator hands over block_out [B,H,S,D] and
block_lse [B,H,S]; the running accumulators are out fp32 [B,S,H,D] and lse fp32
[B,S,H,1] (utils.py:116-122).  Here lse is a transposed view of a contiguous
[B,H,S] buffer, which is what the kernel reads and writes.
"""
import inspect
from functools import cache

import torch

from . import ops

__all__ = ["update_out_and_lse", "get_default_args", "flatten_varlen_lse", "unflatten_varlen_lse"]


@cache
def _get_default_args(func):
    spec = inspect.getfullargspec(func)
    defaults = spec.defaults if spec.defaults is not None else ()
    padded = (None,) * (len(spec.args) - len(defaults)) + defaults
    args = dict(zip(spec.args, padded))
    if "softcap" in args:
        args["softcap"] = 0.0
    return args


def get_default_args(func):
    """Keyword defaults of `func` as a dict (sp_aurora/utils.py:28-44)."""
    if inspect.isfunction(func):
        return _get_default_args(func)
    return _get_default_args(func._init_fn)


def _lse_store(lse):
    """Contiguous [B,H,S] storage behind an lse given as [B,S,H,1] / [B,S,H] / [B,H,S]; and
    whether that storage aliases `lse` (so that an in-place kernel update is visible)."""
    base = lse.squeeze(-1).transpose(1, 2) if lse.dim() == 4 else lse
    if base.is_contiguous():
        return base, True
    return base.contiguous(), False


def update_out_and_lse(out, lse, block_out, block_lse, slice_=None):
    """Merge one block result into the running (out, lse); returns (out, lse).

    First call (out is None): out = float32 copy of block_out as [B,S,H,D], lse [B,S,H,1]
    (sp_aurora/utils.py:116-122).  Later calls: out <- out - sigmoid(block_lse - lse) *
    (out - block_out), lse <- lse - logsigmoid(lse - block_lse) (:103-104), computed by one
    kernel IN PLACE on the accumulators (the reference returns fresh tensors; the values are
    the same).  block_out may come in operator layout [B,H,S,D] or already as [B,S,H,D]; as in
    the reference (:133-137) it is taken as [B,H,S,D] when its dims 1,2 are those of out swapped.
    """
    if out is None:
        if slice_ is not None:
            raise RuntimeError("first update_out_and_lse should not pass slice_ args")
        if block_out.dim() != 4 or block_lse.dim() != 3:
            raise RuntimeError(f"expected block_out [B,H,S,D] and block_lse [B,H,S], got "
                               f"{tuple(block_out.shape)} and {tuple(block_lse.shape)}")
        B, H, S, D = block_out.shape
        out = torch.empty((B, S, H, D), dtype=torch.float32, device=block_out.device)
        store = torch.empty((B, H, S), dtype=torch.float32, device=block_out.device)
        ops.merge(out, store, block_out.transpose(1, 2), block_lse.contiguous().float(), layout="bshd", init=True)
        return out, store.transpose(1, 2).unsqueeze(-1)

    if slice_ is not None:
        s_out, s_lse = out[slice_], lse[slice_]
        n_out, n_lse = update_out_and_lse(s_out, s_lse, block_out, block_lse)
        if n_lse.data_ptr() != s_lse.data_ptr():
            lse[slice_] = n_lse
        if n_out.data_ptr() != s_out.data_ptr():
            out[slice_] = n_out
        return out, lse

    if block_out.shape[1] != out.shape[1] and block_out.shape[2] == out.shape[1]:
        block_out = block_out.transpose(1, 2)
    if out.shape != block_out.shape:
        raise RuntimeError(f"Shape mismatch after block_out transformation: out.shape={tuple(out.shape)}, "
                           f"block_out.shape={tuple(block_out.shape)}")
    B, S, H, D = out.shape
    if block_lse.dim() == 4:
        block_lse = block_lse.squeeze(-1)
    if tuple(block_lse.shape) != (B, H, S):
        if tuple(block_lse.shape) == (B, S, H):
            block_lse = block_lse.transpose(1, 2)
        else:
            raise RuntimeError(f"Shape mismatch after transformation: lse.shape={tuple(lse.shape)}, "
                               f"block_lse.shape={tuple(block_lse.shape)}")
    store, aliased = _lse_store(lse)
    if tuple(store.shape) != (B, H, S):
        raise RuntimeError(f"lse shape {tuple(lse.shape)} does not match out {tuple(out.shape)}")
    ops.merge(out, store, block_out, block_lse.contiguous().float(), layout="bshd", init=False)
    if aliased:
        return out, lse
    new = store.transpose(1, 2)
    return out, new.unsqueeze(-1) if lse.dim() == 4 else new


def flatten_varlen_lse(lse, cu_seqlens):
    """sp_aurora/utils.py:150-156."""
    parts = []
    for i in range(len(cu_seqlens) - 1):
        start, end = int(cu_seqlens[i]), int(cu_seqlens[i + 1])
        parts.append(lse[i, :, : end - start])
    return torch.cat(parts, dim=1)


def unflatten_varlen_lse(lse, cu_seqlens, max_seqlen: int):
    """sp_aurora/utils.py:159-169."""
    num_seq = len(cu_seqlens) - 1
    num_head = lse.shape[-2]
    new_lse = torch.empty((num_seq, max_seqlen, num_head, 1), dtype=torch.float32, device=lse.device)
    for i in range(num_seq):
        start, end = int(cu_seqlens[i]), int(cu_seqlens[i + 1])
        new_lse[i, : end - start] = lse[start:end]
    return new_lse.squeeze(dim=-1).transpose(1, 2).contiguous()
