"""GPU parity of chunk_gated_delta_rule (HIP, through the C ABI) against the token-recurrence oracle."""
import pytest
import torch
import torch.nn.functional as F

from oracle import naive
from tests.util import TOL, gen, max_abs_rel

pytestmark = pytest.mark.gpu


def gdn_inputs(seed, B, T, H, K, V, dtype, head_first=False, strong_gate=False):
    """Inputs with the laws of the contract's gated-delta-rule configs."""
    shp = (B, H, T) if head_first else (B, T, H)
    q = F.normalize(gen(seed, *shp, K), dim=-1).to(dtype)
    k = F.normalize(gen(seed + 1, *shp, K), dim=-1).to(dtype)
    v = gen(seed + 2, *shp, V, dtype=dtype)
    beta = torch.sigmoid(gen(seed + 3, *shp)).to(dtype)
    gh = torch.Generator().manual_seed(seed + 4)
    if strong_gate:   # g = -exp(A_h) softplus(x + dt_bias_h), A_h ~ U(log 1, log 16)
        A = torch.rand(H, generator=gh) * torch.log(torch.tensor(16.0))
        dtb = torch.randn(H, generator=gh) * 0.1
    else:             # the reference's init: small decays
        A = torch.log(torch.rand(H, generator=gh) * 15 + 1)
        dtb = torch.full((H,), -4.0)
    x = gen(seed + 5, *shp)
    hdim = 1 if head_first else 2
    sh = [1, 1, 1]
    sh[hdim] = H
    g = -torch.exp(A).view(sh) * F.softplus(x + dtb.view(sh))
    return q, k, v, g.float(), beta


CASES = [
    # B, T, H, K, V, h0, head_first, strong
    (2, 200, 3, 128, 128, True, False, False),
    (1, 256, 2, 128, 128, False, False, True),
    (2, 130, 2, 64, 128, True, True, True),
    (1, 64, 2, 128, 64, True, False, False),
    (1, 5, 1, 64, 64, False, False, True),
    # the value head of expand_v = 2 (kernel instances of their own: one pass over q, k for all 256 columns)
    (2, 200, 2, 128, 256, True, False, False),
    (1, 130, 3, 128, 256, False, True, True),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", CASES)
def test_gdn_fwd(cuda, dtype, case):
    from linear_moe_amd import chunk_gated_delta_rule
    B, T, H, K, V, use_h0, head_first, strong = case
    q, k, v, g, beta = gdn_inputs(100, B, T, H, K, V, dtype, head_first, strong)
    h0 = gen(114, B, H, K, V) * 0.1 if use_h0 else None
    ref_o, ref_ht = naive.naive_recurrent_gated_delta_rule(q, k, v, g, beta, None, h0, True, None, head_first)
    dev = lambda x: None if x is None else x.to(cuda)
    o, ht = chunk_gated_delta_rule(dev(q), dev(k), dev(v), dev(g), dev(beta), None, dev(h0), True, None, head_first)
    torch.cuda.synchronize()
    assert o.dtype == dtype and o.shape == v.shape
    tol = TOL[dtype]
    assert max_abs_rel(o.cpu(), ref_o) < tol
    assert max_abs_rel(ht.cpu(), ref_ht) < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gdn_fwd_varlen(cuda, dtype):
    from linear_moe_amd import chunk_gated_delta_rule
    lens = [1, 64, 135, 70]
    cu = torch.tensor([0, 1, 65, 200, 270], dtype=torch.int32)
    T, H, K, V = sum(lens), 2, 128, 128
    q, k, v, g, beta = gdn_inputs(200, 1, T, H, K, V, dtype, False, True)
    h0 = gen(214, len(lens), H, K, V) * 0.1
    ref_o, ref_ht = naive.naive_recurrent_gated_delta_rule(q, k, v, g, beta, None, h0, True, cu, False)
    dev = lambda x: x.to(cuda)
    o, ht = chunk_gated_delta_rule(dev(q), dev(k), dev(v), dev(g), dev(beta), None, dev(h0), True, dev(cu), False)
    torch.cuda.synchronize()
    tol = TOL[dtype]
    assert max_abs_rel(o.cpu(), ref_o) < tol
    assert max_abs_rel(ht.cpu(), ref_ht) < tol


BWD_CASES = [
    # B, T, H, K, V, h0, head_first, strong
    (2, 200, 2, 128, 128, True, False, False),
    (1, 256, 2, 128, 128, False, False, True),
    (1, 130, 2, 64, 128, True, True, True),
    (1, 3, 1, 64, 64, True, False, False),
    # K = 64, V = 128 time-first over several chunks with a partial one: the shape on which a build of the
    # chunk-parallel backward that refreshed the lane index once per helper call (instead of once per item) gave
    # wrong dq, dk in fp32 -- kept as a fixed case (the random trials reach this shape only by chance of the seed)
    (2, 330, 3, 64, 128, True, False, False),
    (1, 200, 2, 128, 64, False, False, True),
    (2, 200, 2, 128, 256, True, False, False),
    (1, 330, 3, 128, 256, False, True, True),
    (1, 7, 1, 128, 256, True, False, False),
]


def _gdn_bwd_check(cuda, dtype, ins, do, dht, cu, head_first):
    from linear_moe_amd import chunk_gated_delta_rule
    from tests.util import oracle_grads
    fn = lambda q, k, v, g, beta, h0: naive.naive_recurrent_gated_delta_rule(
        q, k, v, g, beta, None, h0, True, cu, head_first)
    _, _, ref = oracle_grads(fn, ins, do, dht)
    dev = {n: (None if x is None else x.to(cuda).requires_grad_(True)) for n, x in ins.items()}
    o, ht = chunk_gated_delta_rule(dev['q'], dev['k'], dev['v'], dev['g'], dev['beta'], None, dev['h0'], True,
                                   None if cu is None else cu.to(cuda), head_first)
    ((o * do.to(cuda)).sum() + (ht * dht.to(cuda)).sum()).backward()
    torch.cuda.synchronize()
    for n, r in ref.items():
        err = max_abs_rel(dev[n].grad.cpu(), r)
        assert err < TOL[dtype], (n, err)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", BWD_CASES)
def test_gdn_bwd(cuda, dtype, case):
    B, T, H, K, V, use_h0, head_first, strong = case
    q, k, v, g, beta = gdn_inputs(300, B, T, H, K, V, dtype, head_first, strong)
    ins = dict(q=q, k=k, v=v, g=g, beta=beta, h0=gen(314, B, H, K, V) * 0.1 if use_h0 else None)
    shp = (B, H, T) if head_first else (B, T, H)
    _gdn_bwd_check(cuda, dtype, ins, gen(315, *shp, V, dtype=dtype), gen(316, B, H, K, V), None, head_first)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gdn_bwd_varlen(cuda, dtype):
    cu = torch.tensor([0, 1, 65, 200, 270], dtype=torch.int32)
    T, H, K, V, N = 270, 2, 128, 128, 4
    q, k, v, g, beta = gdn_inputs(400, 1, T, H, K, V, dtype, False, True)
    ins = dict(q=q, k=k, v=v, g=g, beta=beta, h0=gen(414, N, H, K, V) * 0.1)
    _gdn_bwd_check(cuda, dtype, ins, gen(415, 1, T, H, V, dtype=dtype), gen(416, N, H, K, V), cu, False)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gdn_bwd_varlen_wide_value_head(cuda, dtype):
    cu = torch.tensor([0, 64, 65, 200, 333], dtype=torch.int32)
    T, H, K, V, N = 333, 2, 128, 256, 4
    q, k, v, g, beta = gdn_inputs(420, 1, T, H, K, V, dtype, False, True)
    ins = dict(q=q, k=k, v=v, g=g, beta=beta, h0=gen(434, N, H, K, V) * 0.1)
    _gdn_bwd_check(cuda, dtype, ins, gen(435, 1, T, H, V, dtype=dtype), gen(436, N, H, K, V), cu, False)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gdn_wide_value_head_equals_its_two_halves(cuda, dtype):
    """V = 256 in one call against the two calls on 128 columns each that the op used to be cut into: the columns of v
    are independent, so o, the final state and dv agree bit for bit (the same slice kernels on the same operands);
    dq, dk, dg, dbeta are sums over all columns and agree to rounding (one sum over 256 columns against two rounded
    sums of 128)."""
    from linear_moe_amd import chunk_gated_delta_rule
    B, T, H, K, V = 2, 300, 3, 128, 256
    q, k, v, g, beta = gdn_inputs(440, B, T, H, K, V, dtype, False, True)
    h0, do, dht = gen(454, B, H, K, V) * 0.1, gen(455, B, T, H, V, dtype=dtype), gen(456, B, H, K, V)
    res = []
    for halves in (False, True):
        d = {n: x.to(cuda).requires_grad_(True) for n, x in dict(q=q, k=k, v=v, g=g, beta=beta, h0=h0).items()}
        if halves:
            parts = [chunk_gated_delta_rule(d['q'], d['k'], d['v'][..., c:c + 128], d['g'], d['beta'], K ** -0.5,
                                            d['h0'][..., c:c + 128], True) for c in (0, 128)]
            o, ht = torch.cat([p[0] for p in parts], -1), torch.cat([p[1] for p in parts], -1)
        else:
            o, ht = chunk_gated_delta_rule(d['q'], d['k'], d['v'], d['g'], d['beta'], None, d['h0'], True)
        ((o * do.to(cuda)).sum() + (ht * dht.to(cuda)).sum()).backward()
        res.append((o.detach(), ht.detach(), {n: x.grad for n, x in d.items()}))
    (o1, ht1, g1), (o2, ht2, g2) = res
    assert torch.equal(o1, o2) and torch.equal(ht1, ht2)
    assert torch.equal(g1['v'], g2['v']) and torch.equal(g1['h0'], g2['h0'])
    for n in ('q', 'k', 'g', 'beta'):
        assert max_abs_rel(g1[n].cpu(), g2[n].cpu()) < TOL[dtype], n


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", [(2, 200, 2, 128, 128, True), (1, 70, 2, 64, 128, False), (1, 130, 2, 128, 256, True)])
def test_delta_rule_fwd_bwd(cuda, dtype, case):
    """chunk_delta_rule as the reference calls it (deltanet.py:127-130): head-first, positional chunk size."""
    from linear_moe_amd import chunk_delta_rule
    from tests.util import oracle_grads
    B, T, H, K, V, use_h0 = case
    q, k, v, _, beta = gdn_inputs(500, B, T, H, K, V, dtype, True, False)
    ins = dict(q=q, k=k, v=v, beta=beta, h0=gen(514, B, H, K, V) * 0.1 if use_h0 else None)
    do, dht = gen(515, B, H, T, V, dtype=dtype), gen(516, B, H, K, V)
    fn = lambda q, k, v, beta, h0: naive.naive_recurrent_gated_delta_rule(q, k, v, None, beta, None, h0, True, None, True)
    ref_o, ref_ht, ref = oracle_grads(fn, ins, do, dht)
    dev = {n: (None if x is None else x.to(cuda).requires_grad_(True)) for n, x in ins.items()}
    o, ht = chunk_delta_rule(dev['q'], dev['k'], dev['v'], dev['beta'], 32, initial_state=dev['h0'],
                             output_final_state=True)
    ((o * do.to(cuda)).sum() + (ht * dht.to(cuda)).sum()).backward()
    torch.cuda.synchronize()
    tol = TOL[dtype]
    assert max_abs_rel(o.detach().cpu(), ref_o) < tol and max_abs_rel(ht.detach().cpu(), ref_ht) < tol
    for n, r in ref.items():
        err = max_abs_rel(dev[n].grad.cpu(), r)
        assert err < tol, (n, err)


def test_forward_only_call_equals_the_saving_call(cuda):
    """Without anything that requires a gradient, what only the backward reads (per-chunk states, v_new, Tinv) is
    neither allocated nor written (NULL through the C ABI): outputs and final state are bit-identical."""
    from linear_moe_amd import chunk_gated_delta_rule
    B, T, H, K, V = 2, 300, 3, 128, 128
    q, k, v, g, beta = (x.to(cuda) for x in gdn_inputs(4100, B, T, H, K, V, torch.bfloat16, False))
    h0 = (gen(4110, B, H, K, V) * 0.5).to(cuda)
    with torch.no_grad():
        o1, ht1 = chunk_gated_delta_rule(q, k, v, g, beta, None, h0, True, None, False)
    o2, ht2 = chunk_gated_delta_rule(q.clone().requires_grad_(True), k, v, g, beta, None, h0, True, None, False)
    torch.cuda.synchronize()
    assert torch.equal(o1, o2.detach()) and torch.equal(ht1, ht2.detach())
