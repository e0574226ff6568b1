"""The fp32 forward for launches with few query rows (32-row workgroups whose eight waves share the key tiles and
combine through LDS): forced on and off through spa_tune, both forms against the oracle on the same inputs, and the
library's own choice at the benchmark's config 1."""
import pytest
import torch

from conftest import rand_qkv
from oracle import attn_oracle as O
from sp_aurora_amd import _lib, ops
from test_gpu_parity import DEV, check_lse, check_out

pytestmark = pytest.mark.gpu

CASES = [
    # B, H, Sq, Sk, D, causal
    (1, 8, 512, 512, 64, False),    # benchmark config 1
    (1, 8, 512, 512, 64, True),
    (2, 3, 100, 333, 64, False),    # ragged rows and keys
    (1, 2, 257, 257, 32, True),     # one row in the last tile
    (1, 1, 31, 1000, 32, False),    # fewer rows than a tile, more key tiles than waves
    (1, 2, 300, 70, 64, True),      # more rows than keys: the last tiles see every key
    (1, 1, 64, 17, 64, False),      # fewer key tiles than waves
]


@pytest.mark.parametrize("form", [1, 2])
@pytest.mark.parametrize("B,H,Sq,Sk,D,causal", CASES)
def test_both_fp32_forms_match_the_oracle(form, B, H, Sq, Sk, D, causal):
    g = torch.Generator().manual_seed(1234 + Sq + Sk)
    q = torch.randn((B, Sq, H, D), generator=g)
    k = torch.randn((B, Sk, H, D), generator=g)
    v = torch.randn((B, Sk, H, D), generator=g)
    want_o, want_l = O.full_attention(q, k, v, None, causal)
    _lib.tune("fwd32_split", form)
    try:
        for scale in (None, -0.2):
            out, lse = ops.flash_fwd(q.to(DEV), k.to(DEV), v.to(DEV), scale, causal, layout="bshd")
            if scale is None:
                check_out(out.cpu(), want_o, torch.float32, f"form {form}")
                check_lse(lse.cpu(), want_l)
            else:
                wo, wl = O.full_attention(q, k, v, scale, causal)
                check_out(out.cpu(), wo, torch.float32, f"form {form} negative scale")
                check_lse(lse.cpu(), wl)
    finally:
        _lib.tune("fwd32_split", 0)


def test_strided_views_and_the_librarys_choice():
    """config 1 as the packed tensor's views (the public qkv-packed call), no knob: the result is the oracle's; the two
    forms agree to rounding."""
    B, S, H, D = 1, 512, 8, 64
    (qkv,) = rand_qkv((B, S, 3, H, D), 77, torch.float32, n=1)
    q, k, v = (qkv[:, :, i] for i in range(3))
    want_o, want_l = O.full_attention(q, k, v, None, True)
    qd = qkv.to(DEV)
    res = {}
    for form in (0, 1, 2):
        _lib.tune("fwd32_split", form)
        try:
            res[form] = ops.flash_fwd(qd[:, :, 0], qd[:, :, 1], qd[:, :, 2], None, True, layout="bshd")
        finally:
            _lib.tune("fwd32_split", 0)
        check_out(res[form][0].cpu(), want_o, torch.float32, f"form {form}")
        check_lse(res[form][1].cpu(), want_l)
    assert torch.equal(res[0][0], res[2][0]), "32 workgroups of 128 rows on this device: the library takes the 32-row form"
    assert (res[1][0] - res[2][0]).abs().max().item() < 1e-5
