"""Writes the committed fixtures tests/golden/*.npz from the CPU oracle.

The reference holds no golden vectors for this path (its tests build their expectations inline),
and its Python cannot be imported here (hard dependency on intel_extension_for_pytorch), so the
vectors come from oracle/attn_oracle.py in float64 — which tests/test_oracle.py pins against
brute force, closed forms and library routines.  Inputs are not stored: they are re-drawn from
the seed (conftest.rand_qkv) and checked against the stored SHA-256.

Run from the repo root:  python tests/golden/make_golden.py
"""
import hashlib
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from conftest import rand_qkv  # noqa: E402
from oracle import attn_oracle as O  # noqa: E402


def digest(*tensors):
    h = hashlib.sha256()
    for t in tensors:
        h.update(t.contiguous().view(torch.uint8).numpy().tobytes())
    return h.hexdigest()


# name -> (seed, dtype, shape [B,S,H,D], input scale, causal, ring size, softmax scale)
CASES = {
    # benchmark config 1: the reference's CPU-runnable case
    "cfg1_fp32_b1_s512_h8_d64": (0, torch.float32, (1, 512, 8, 64), 1.0, False, 1, 1.0 / 8.0),
    # known-answer procedure of test/flash_attention/test_flash_attention_simple.py:74-137
    "simple_fp32_b1_s64_h2_d32_causal": (42, torch.float32, (1, 64, 2, 32), 1.0, True, 1, None),
    # small ring cases in every dtype
    "ring4_bf16_b1_s256_h4_d64_causal": (7, torch.bfloat16, (1, 256, 4, 64), 1.0, True, 4, None),
    "ring2_fp16_b2_s128_h2_d128": (8, torch.float16, (2, 128, 2, 128), 1.0, False, 2, None),
    "ring4_fp32_b1_s96_h2_d32_causal": (9, torch.float32, (1, 96, 2, 32), 1.0, True, 4, None),
}


def main():
    for name, (seed, dtype, shape, in_scale, causal, P, scale) in CASES.items():
        q, k, v = rand_qkv(shape, seed, dtype, in_scale)
        out, lse = O.ring_forward(q, k, v, P, scale, causal, out_dtype=torch.float64)
        full, full_lse = O.full_attention(q, k, v, scale, causal)
        assert torch.allclose(out, full, atol=1e-12) and torch.allclose(lse, full_lse, atol=1e-12)
        path = os.path.join(HERE, name + ".npz")
        np.savez_compressed(path, out=out.to(torch.float32).numpy(), lse=lse.to(torch.float32).numpy(),
                            input_sha256=np.array(digest(q, k, v)))
        print(f"{name}: out {tuple(out.shape)} lse {tuple(lse.shape)} -> {os.path.getsize(path)} bytes")


if __name__ == "__main__":
    main()
