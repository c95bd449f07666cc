"""GPU parity of the thin adaptors over chunk_simple_gla, called exactly as the reference's modules call them:
lightning_attn2 / lightning_attn2_no_decay (linear_moe/sequence_modeling/lightning_attention/
lightning_attention.py:121-123) and chunk_linear_attn with its normaliser (basic_linear_attention.py:133)."""
import pytest
import torch

from oracle import naive
from tests.util import TOL, gen, max_abs_rel

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H", [16, 12])          # a power of two and the interleaved completion of the slopes
def test_lightning_attn2_fwd_bwd(cuda, dtype, H):
    """lightning_attn2(q, k, v, slope[H,1,1]) -> o only; [B,H,T,D]; no scale; forward and dq, dk, dv."""
    from linear_moe_amd.lightning import lightning_attn2
    B, T, K, V = 2, 200, 64, 128
    q, k = 0.3 * gen(3101, B, H, T, K, dtype=dtype), 0.3 * gen(3102, B, H, T, K, dtype=dtype)
    v, do = gen(3103, B, H, T, V, dtype=dtype), gen(3104, B, H, T, V, dtype=dtype)
    slope = naive.lightning_slopes(H).float().reshape(H, 1, 1)
    ref_in = [x.double().requires_grad_(True) for x in (q, k, v)]
    ref = naive.naive_lightning_attn2(*ref_in, slope)
    ref_g = torch.autograd.grad((ref * do.double()).sum(), ref_in)
    dev_in = [x.to(cuda).requires_grad_(True) for x in (q, k, v)]
    o = lightning_attn2(*dev_in, slope.to(cuda))
    assert isinstance(o, torch.Tensor) and o.shape == v.shape and o.dtype == dtype
    grads = torch.autograd.grad((o * do.to(cuda)).sum(), dev_in)
    torch.cuda.synchronize()
    assert max_abs_rel(o.detach().cpu(), ref.detach()) < TOL[dtype]
    for gd, gr, n in zip(grads, ref_g, "qkv"):
        assert max_abs_rel(gd.cpu(), gr) < TOL[dtype], n


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_lightning_attn2_no_decay(cuda, dtype):
    from linear_moe_amd.lightning import lightning_attn2_no_decay
    B, H, T, K, V = 1, 3, 130, 128, 64
    q, k = 0.3 * gen(3111, B, H, T, K, dtype=dtype), 0.3 * gen(3112, B, H, T, K, dtype=dtype)
    v = gen(3113, B, H, T, V, dtype=dtype)
    ref = torch.tril(q.double() @ k.double().transpose(-1, -2)) @ v.double()
    o = lightning_attn2_no_decay(q.to(cuda), k.to(cuda), v.to(cuda))
    torch.cuda.synchronize()
    assert isinstance(o, torch.Tensor)
    assert max_abs_rel(o.cpu(), ref) < TOL[dtype]


@pytest.mark.parametrize("scale", [None, 1.0])
@pytest.mark.parametrize("head_first", [True, False])
def test_linear_attn_normalised_default_scale(cuda, scale, head_first):
    """chunk_linear_attn(q, k, v, normalize=True) with the default scale K^-0.5, as BasicLinearAttention calls it
    with la_do_feature_map_norm: o_t = sum a_ts v_s / (sum a_ts + eps), a_ts = scale q_t.k_s, checked against the
    closed form written out here (not the oracle's expression) and against the oracle; forward and gradients."""
    from linear_moe_amd import chunk_linear_attn
    B, H, T, K, V = 2, 2, 150, 64, 64
    # positive features (the reference's feature maps are positive: elu+1, relu, ...), so the normaliser is not tiny
    q, k = gen(3201, B, H, T, K).abs() + 0.1, gen(3202, B, H, T, K).abs() + 0.1
    v, do = gen(3203, B, H, T, V), gen(3204, B, H, T, V)
    sc = K ** -0.5 if scale is None else scale
    ref_in = [x.double().requires_grad_(True) for x in (q, k, v)]
    A = torch.tril(sc * ref_in[0] @ ref_in[1].transpose(-1, -2))
    ref = (A @ ref_in[2]) / (A.sum(-1, keepdim=True) + 1e-10)
    ref_g = torch.autograd.grad((ref * do.double()).sum(), ref_in)
    o_or, _ = naive.naive_linear_attn(q, k, v, scale=scale, normalize=True)
    assert torch.allclose(o_or, ref.detach(), atol=1e-12)
    tf = (lambda x: x) if head_first else (lambda x: x.transpose(1, 2).contiguous())
    dev_in = [tf(x).to(cuda).requires_grad_(True) for x in (q, k, v)]
    o, ht = chunk_linear_attn(*dev_in, scale=scale, normalize=True, head_first=head_first)
    grads = torch.autograd.grad((o * tf(do).to(cuda)).sum(), dev_in)
    torch.cuda.synchronize()
    assert ht is None
    assert max_abs_rel(tf(o.detach().cpu()), ref.detach()) < 1e-5
    for gd, gr, n in zip(grads, ref_g, "qkv"):
        assert max_abs_rel(tf(gd.cpu()), gr) < 1e-5, n
