"""GPU parity of the attention modules (UlyssesAttention, LongContextAttention) against the
oracle's full attention: whatever way the ranks are split, every rank's rows of the result
must be the rows of attention over the whole sequence
(the reference's own criterion: test/test_ring_attention_full_accuracy.py:122-171,
test/verification/test_ulysses_fixed.py:165-344)."""
import pytest
import torch

from conftest import rand_qkv
from oracle import attn_oracle as O
import sp_aurora_amd as spa
from test_gpu_parity import DEV, check_grad, check_out

pytestmark = pytest.mark.gpu


def stack(t, W):
    """[B, W*s, H, D] -> rank-stacked [W, B, s, H, D] on the device."""
    return torch.stack(t.chunk(W, 1)).contiguous().to(DEV)


def unstack(t):
    return torch.cat(list(t), 1)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_ulysses_attention_module(causal, dtype):
    P, B, s, H, D = 4, 2, 48, 8, 64
    q, k, v = rand_qkv((B, P * s, H, D), 300, dtype)
    want, _ = O.full_attention(q, k, v, None, causal)
    layer = spa.UlyssesAttention(None, attn_type=spa.AttnType.TORCH)
    out = layer(stack(q, P), stack(k, P), stack(v, P), causal=causal)
    assert out.shape == (P, B, s, H, D) and out.dtype == dtype
    check_out(unstack(out), want, dtype)
    # a world of one: plain attention of the 4-D tensors, with the lse on request
    out1, lse1 = layer(q.to(DEV), k.to(DEV), v.to(DEV), causal=causal, return_attn_probs=True)
    check_out(out1, want, dtype)
    assert lse1.shape == (B, H, P * s) and lse1.dtype == torch.float32


@pytest.mark.parametrize("pack", [False, True])
@pytest.mark.parametrize("U,R", [(2, 2), (4, 2), (2, 3), (1, 4), (4, 1), (1, 1)])
@pytest.mark.parametrize("causal", [False, True])
def test_long_context_attention_equals_full_attention(U, R, causal, pack):
    W, B, s, H, D = U * R, 2, 40, 4, 64
    dtype = torch.bfloat16
    q, k, v = rand_qkv((B, W * s, H, D), 310 + U * 7 + R, dtype)
    want, _ = O.full_attention(q, k, v, None, causal)
    layer = spa.LongContextAttention(sp_ulysses_degree=U, sp_ring_degree=R, use_pack_qkv=pack)
    assert (layer.get_sequence_parallel_degree(), layer.get_ulysses_degree(), layer.get_ring_degree()) == (W, U, R)
    out = layer(stack(q, W), stack(k, W), stack(v, W), causal=causal)
    assert out.shape == (W, B, s, H, D) and out.dtype == dtype
    check_out(unstack(out), want, dtype)
    if W == 1:
        check_out(layer(q.to(DEV), k.to(DEV), v.to(DEV), causal=causal), want, dtype)
    # the joint key/value form
    kv = torch.stack([stack(k, W), stack(v, W)], dim=3)
    out2 = layer(stack(q, W), None, None, causal=causal, joint_tensor_key_value=kv)
    assert torch.equal(out2, out)


@pytest.mark.parametrize("U,R", [(2, 2), (1, 2), (2, 1)])
def test_long_context_attention_gradients(U, R):
    W, B, s, H, D = U * R, 1, 64, 4, 64
    dtype = torch.bfloat16
    q, k, v, dout = rand_qkv((B, W * s, H, D), 320, dtype, n=4)
    want = O.attn_backward_autograd(q, k, v, dout, None, True)
    xs = [stack(t, W).requires_grad_(True) for t in (q, k, v)]
    layer = spa.LongContextAttention(sp_ulysses_degree=U, sp_ring_degree=R)
    out = layer(*xs, causal=True)
    out.backward(stack(dout, W))
    for x, w, name in zip(xs, want, "qkv"):
        assert x.grad.shape == (W, B, s, H, D)
        check_grad(unstack(x.grad), w, dtype, "d" + name)


def test_layer_argument_contract():
    with pytest.raises(ValueError):
        spa.select_flash_attn_impl("no_such_kernel")
    assert spa.AttnType("flash_attn") is spa.AttnType.FA
    layer = spa.LongContextAttention(sp_ulysses_degree=2, sp_ring_degree=2, attn_type="flash_attn")
    q = torch.zeros(3, 1, 8, 4, 64, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        layer(q, q, q)  # 3 stacked ranks for a world of 4
    q = torch.zeros(4, 1, 8, 4, 64, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(NotImplementedError):
        layer(q, q, q, softcap=1.0)
    with pytest.raises(NotImplementedError):
        layer(q, q, q, dropout_p=0.1)
    with pytest.raises(ValueError):
        spa.LongContextAttention(sp_ulysses_degree=8, sp_ring_degree=1)(
            torch.zeros(8, 1, 8, 4, 64, device=DEV, dtype=torch.bfloat16), q, q)  # 4 heads over 8 ranks


def test_second_implementation_names_reach_the_same_kernels():
    """pytorch_attn_* (sp_aurora/kernels/attention.py) and ring_pytorch_attn_* (sp_aurora/ring_pytorch_attn.py)."""
    B, S, H, D = 2, 96, 4, 64
    q, k, v = rand_qkv((B, S, H, D), 330, torch.bfloat16)
    want, want_lse = O.full_attention(q, k, v, None, True)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    out, probs = spa.pytorch_attn_forward(qd, kd, vd, causal=True)
    assert probs is None
    check_out(out, want, torch.bfloat16)
    assert torch.equal(spa.pytorch_attn_func(qd, kd, vd, causal=True), out)
    out2, lse2 = spa.ring_pytorch_attn_forward(qd, kd, vd, causal=True, ring_size=3)
    check_out(out2, want, torch.bfloat16)
    assert (lse2.cpu().double() - want_lse).abs().max() <= 1e-3
    assert torch.equal(spa.ring_pytorch_attn_func(qd, kd, vd, causal=True, ring_size=3), out2)
    with pytest.raises(NotImplementedError):
        spa.pytorch_attn_forward(qd, kd, vd, return_attn_probs=True)
    assert spa.HAS_LONG_CTX_ATTN and spa.HAS_FLASH_ATTN and not spa.HAS_SPARSE_SAGE_ATTENTION
    assert spa.SeqAllToAll4D_v2 is spa.SeqAllToAll4D
