"""GPU parity of the row-wise neighbours of the chunk ops (RMS norm with optional swish gate, SiLU + L2
norm; HIP, through the C ABI) against the fp64 oracle."""
import pytest
import torch

from oracle import naive
from tests.util import TOL, gen, max_abs_rel

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("D", [64, 128, 256])
@pytest.mark.parametrize("gated", [False, True])
def test_rms_norm_fwd_bwd(cuda, dtype, D, gated):
    from linear_moe_amd import rms_norm_fn, rms_norm_swish_gate
    x = gen(1100 + D, 2, 3, 41, D, dtype=dtype)
    w = (1.0 + 0.2 * gen(1101 + D, D)).to(dtype)
    gate = gen(1102 + D, 2, 3, 41, D, dtype=dtype) if gated else None
    dy = gen(1103 + D, 2, 3, 41, D, dtype=dtype)
    xr, wr = x.double().requires_grad_(True), w.double().requires_grad_(True)
    gr = gate.double().requires_grad_(True) if gated else None
    ref = naive.naive_rms_norm(xr, wr, gr, eps=1e-5)
    (ref * dy.double()).sum().backward()
    xd, wd = x.to(cuda).requires_grad_(True), w.to(cuda).requires_grad_(True)
    gd = gate.to(cuda).requires_grad_(True) if gated else None
    y = rms_norm_swish_gate(xd, gd, wd, eps=1e-5) if gated else rms_norm_fn(xd, wd, None, eps=1e-5)
    (y * dy.to(cuda)).sum().backward()
    torch.cuda.synchronize()
    assert y.dtype == dtype and y.shape == x.shape
    assert max_abs_rel(y.detach().cpu(), ref.detach()) < TOL[dtype]
    assert max_abs_rel(xd.grad.cpu(), xr.grad) < TOL[dtype]
    assert wd.grad.dtype == dtype
    assert max_abs_rel(wd.grad.cpu(), wr.grad) < TOL[dtype]
    if gated:
        assert max_abs_rel(gd.grad.cpu(), gr.grad) < TOL[dtype]


def test_rms_norm_module_and_many_rows(cuda):
    """The module with the reference's constructor; enough rows that every work-group loops and the
    weight gradient goes through many partial rows; run twice: bit-identical (fixed summation order)."""
    from linear_moe_amd import RMSNorm
    m = RMSNorm(128, eps=1e-5).to(cuda)
    with torch.no_grad():
        m.weight.copy_(1.0 + 0.1 * gen(1201, 128))
    x = gen(1202, 4, 16, 2048, 128)
    dy = gen(1203, 4, 16, 2048, 128)
    xr, wr = x.double().requires_grad_(True), m.weight.detach().cpu().double().requires_grad_(True)
    (naive.naive_rms_norm(xr, wr, None, eps=1e-5) * dy.double()).sum().backward()
    grads = []
    for _ in range(2):
        m.weight.grad = None
        xd = x.to(cuda).requires_grad_(True)
        (m(xd) * dy.to(cuda)).sum().backward()
        torch.cuda.synchronize()
        grads.append((xd.grad.clone(), m.weight.grad.clone()))
    assert max_abs_rel(grads[0][0].cpu(), xr.grad) < 1e-5
    assert max_abs_rel(grads[0][1].cpu(), wr.grad) < 1e-5
    assert torch.equal(grads[0][0], grads[1][0]) and torch.equal(grads[0][1], grads[1][1])
    no_affine = RMSNorm(64, elementwise_affine=False).to(cuda)
    xs = gen(1204, 5, 64)
    assert max_abs_rel(no_affine(xs.to(cuda)).cpu(), naive.naive_rms_norm(xs, eps=1e-5)) < 1e-5
    with pytest.raises(ValueError):
        RMSNorm(48).to(cuda)(torch.zeros(3, 48, device=cuda))
    assert m(torch.zeros(0, 128, device=cuda)).shape == (0, 128)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("D", [64, 128])
def test_silu_l2_norm_fwd_bwd(cuda, dtype, D):
    from linear_moe_amd import silu_l2_norm
    x = gen(1300 + D, 2, 37, 3, D, dtype=dtype)
    dy = gen(1301 + D, 2, 37, 3, D, dtype=dtype)
    xr = x.double().requires_grad_(True)
    ref = naive.naive_silu_l2_norm(xr, eps=1e-6)
    (ref * dy.double()).sum().backward()
    xd = x.to(cuda).requires_grad_(True)
    y = silu_l2_norm(xd)
    (y * dy.to(cuda)).sum().backward()
    torch.cuda.synchronize()
    assert max_abs_rel(y.detach().cpu(), ref.detach()) < TOL[dtype]
    assert max_abs_rel(xd.grad.cpu(), xr.grad) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H", [16, 12, 32])
def test_gdn_gates_fwd_bwd(cuda, dtype, H):
    """Gate construction of the gated delta rule with the reference's parameter laws (A ~ U(0, 16),
    dt log-uniform in [1e-3, 0.1] -> dt_bias = softplus^-1(dt)); enough rows for several partial rows."""
    import math
    from linear_moe_amd import gdn_gates
    B, T = 3, 1031
    a = 2.0 * gen(1400 + H, B, T, H, dtype=dtype)
    b = 2.0 * gen(1401 + H, B, T, H, dtype=dtype)
    gg = torch.Generator().manual_seed(1402 + H)
    A_log = torch.log(torch.rand(H, generator=gg) * 16 + 1e-3)
    dtv = torch.exp(torch.rand(H, generator=gg) * (math.log(0.1) - math.log(1e-3)) + math.log(1e-3)).clamp(min=1e-4)
    dt_bias = dtv + torch.log(-torch.expm1(-dtv))
    dg, dbeta = gen(1403 + H, B, T, H), gen(1404 + H, B, T, H, dtype=dtype)
    ar, br = a.double().requires_grad_(True), b.double().requires_grad_(True)
    Ar, Dr = A_log.double().requires_grad_(True), dt_bias.double().requires_grad_(True)
    g_ref, beta_ref = naive.naive_gdn_gates(ar, br, Ar, Dr)
    ((g_ref * dg.double()).sum() + (beta_ref * dbeta.double()).sum()).backward()
    ad, bd = a.to(cuda).requires_grad_(True), b.to(cuda).requires_grad_(True)
    Ad, Dd = A_log.to(cuda).requires_grad_(True), dt_bias.to(cuda).requires_grad_(True)
    g, beta = gdn_gates(ad, bd, Ad, Dd)
    ((g * dg.to(cuda)).sum() + (beta.float() * dbeta.to(cuda).float()).sum()).backward()
    torch.cuda.synchronize()
    assert g.dtype == torch.float32 and beta.dtype == dtype
    tol = TOL[dtype]
    assert max_abs_rel(g.detach().cpu(), g_ref.detach()) < (1e-5 if dtype == torch.float32 else tol)
    assert max_abs_rel(beta.detach().cpu(), beta_ref.detach()) < tol
    assert max_abs_rel(ad.grad.cpu(), ar.grad) < tol
    assert max_abs_rel(bd.grad.cpu(), br.grad) < tol
    assert max_abs_rel(Ad.grad.cpu(), Ar.grad) < tol
    assert max_abs_rel(Dd.grad.cpu(), Dr.grad) < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("clamp", [None, -0.05])
def test_gla_gate_fwd_bwd(cuda, dtype, clamp):
    from linear_moe_amd import gla_gate
    x = 3.0 * gen(1500, 2, 4, 133, 64, dtype=dtype)
    dy = gen(1501, 2, 4, 133, 64, dtype=dtype)
    xr = x.double().requires_grad_(True)
    ref = naive.naive_gla_gate(xr, 16.0, clamp)
    (ref * dy.double()).sum().backward()
    xd = x.to(cuda).requires_grad_(True)
    y = gla_gate(xd, 16.0, clamp)
    (y * dy.to(cuda)).sum().backward()
    torch.cuda.synchronize()
    assert y.dtype == dtype and (y <= 0).all()
    assert max_abs_rel(y.detach().cpu(), ref.detach()) < TOL[dtype]
    # elements that sit on the clamp within rounding may go either way: compare away from it
    far = (ref.detach() - (clamp if clamp is not None else -1e30)).abs() > 1e-3
    assert max_abs_rel((xd.grad.cpu() * far), (xr.grad * far)) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("D", [64, 128])
def test_gdn_qkv_prologue_fwd_bwd(cuda, dtype, D):
    """One pass over the fused projection [T, B, H 3 D] against split -> transpose -> SiLU -> L2 norm."""
    from linear_moe_amd import gdn_qkv_prologue
    T, B, H = 37, 3, 5
    qkv = gen(1300 + D, T, B, H * 3 * D, dtype=dtype)
    dq, dk, dv = (gen(1301 + D + i, B, T, H, D, dtype=dtype) for i in range(3))
    xr = qkv.double().requires_grad_(True)
    rq, rk, rv = naive.naive_gdn_qkv_prologue(xr, H, D)
    ((rq * dq.double()).sum() + (rk * dk.double()).sum() + (rv * dv.double()).sum()).backward()
    xd = qkv.to(cuda).requires_grad_(True)
    q, k, v = gdn_qkv_prologue(xd, H, D)
    ((q * dq.to(cuda)).sum() + (k * dk.to(cuda)).sum() + (v * dv.to(cuda)).sum()).backward()
    torch.cuda.synchronize()
    for got, ref in ((q, rq), (k, rk), (v, rv)):
        assert got.shape == (B, T, H, D) and got.dtype == dtype and got.is_contiguous()
        assert max_abs_rel(got.detach().cpu(), ref.detach()) < TOL[dtype]
    assert xd.grad.shape == qkv.shape
    assert max_abs_rel(xd.grad.cpu(), xr.grad) < TOL[dtype]
    # the same numbers as the three-kernel chain it replaces, to the rounding of the element type
    from linear_moe_amd import silu_l2_norm
    q3 = silu_l2_norm(xd.detach().view(T, B, H, 3 * D)[..., :D].transpose(0, 1).contiguous())
    assert max_abs_rel(q.detach().cpu(), q3.cpu()) < (1e-6 if dtype == torch.float32 else 8e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_swish_gate_relayout_fwd_bwd(cuda, dtype):
    from linear_moe_amd import swish_gate_relayout
    T, B, H, D = 29, 3, 3, 64
    o = gen(1400, B, T, H, D, dtype=dtype)
    gate = gen(1401, T, B, H * D, dtype=dtype)
    dy = gen(1402, T, B, H * D, dtype=dtype)
    orf, grf = o.double().requires_grad_(True), gate.double().requires_grad_(True)
    ref = naive.naive_swish_gate_relayout(orf, grf)
    (ref * dy.double()).sum().backward()
    od, gd = o.to(cuda).requires_grad_(True), gate.to(cuda).requires_grad_(True)
    y = swish_gate_relayout(od, gd)
    (y * dy.to(cuda)).sum().backward()
    torch.cuda.synchronize()
    assert y.shape == (T, B, H * D) and y.dtype == dtype
    assert max_abs_rel(y.detach().cpu(), ref.detach()) < TOL[dtype]
    assert max_abs_rel(od.grad.cpu(), orf.grad) < TOL[dtype]
    assert max_abs_rel(gd.grad.cpu(), grf.grad) < TOL[dtype]
