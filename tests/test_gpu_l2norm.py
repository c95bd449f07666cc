"""GPU parity of the row-wise L2 normalisation (HIP, through the C ABI) against the fp64 oracle."""
import pytest
import torch

from oracle import naive
from tests.util import TOL, gen, max_abs_rel

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("D", [64, 128, 256])
def test_l2norm_fwd_bwd(cuda, dtype, D):
    from linear_moe_amd import l2_norm
    x = gen(900 + D, 2, 37, 3, D, dtype=dtype)
    dy = gen(901 + D, 2, 37, 3, D, dtype=dtype)
    xr = x.double().requires_grad_(True)
    ref = naive.naive_l2_norm(xr, eps=1e-6)
    (ref * dy.double()).sum().backward()
    xd = x.to(cuda).requires_grad_(True)
    y = l2_norm(xd)
    (y * dy.to(cuda)).sum().backward()
    torch.cuda.synchronize()
    assert y.dtype == dtype and y.shape == x.shape
    assert max_abs_rel(y.detach().cpu(), ref.detach()) < TOL[dtype]
    assert max_abs_rel(xd.grad.cpu(), xr.grad) < TOL[dtype]


def test_l2norm_strided_input_and_eps(cuda):
    from linear_moe_amd import l2_norm
    x = gen(950, 4, 9, 128).to(cuda)
    xt = x.transpose(0, 1)                       # not contiguous
    y = l2_norm(xt, 0.25)
    ref = naive.naive_l2_norm(xt.cpu(), eps=0.25)
    assert max_abs_rel(y.cpu(), ref) < 1e-5
    with pytest.raises(ValueError):
        l2_norm(torch.zeros(3, 48, device=cuda))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gdn_with_qk_l2norm_in_kernel(cuda, dtype):
    """chunk_gated_delta_rule(use_qk_l2norm_in_kernel=True) = the op on normalised q, k, gradients included."""
    from linear_moe_amd import chunk_gated_delta_rule
    from tests.test_gpu_gdn import gdn_inputs
    from tests.util import oracle_grads
    B, T, H, K, V = 1, 130, 2, 128, 64
    q, k, v, g, beta = gdn_inputs(970, B, T, H, K, V, dtype, False, True)
    q, k = (q.float() * 3.0).to(dtype), (k.float() * 0.5).to(dtype)       # not normalised on entry
    ins = dict(q=q, k=k, v=v, g=g, beta=beta)
    do = gen(975, B, T, H, V, dtype=dtype)
    fn = lambda q, k, v, g, beta: naive.naive_recurrent_gated_delta_rule(
        q, k, v, g, beta, None, None, True, None, False, use_qk_l2norm_in_kernel=True)
    ref_o, _, ref = oracle_grads(fn, ins, do, None)
    dev = {n: x.to(cuda).requires_grad_(True) for n, x in ins.items()}
    o, _ = chunk_gated_delta_rule(dev['q'], dev['k'], dev['v'], dev['g'], dev['beta'], use_qk_l2norm_in_kernel=True)
    (o * do.to(cuda)).sum().backward()
    torch.cuda.synchronize()
    assert max_abs_rel(o.detach().cpu(), ref_o) < TOL[dtype]
    for n, r in ref.items():
        assert max_abs_rel(dev[n].grad.cpu(), r) < TOL[dtype], n
