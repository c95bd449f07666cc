"""Head dimensions the kernels are not instantiated for (anything but 64 and 128, and K = 128 with V = 256 for the
delta rule): the public ops pad and cut them into blocks of 128 / 64 columns, the delta rule with a key block of 128
also into value blocks of 256 (``linear_moe_amd/_host.py::by_head_dim_blocks``).  HIP through the C ABI against the
token-recurrence oracle on the whole head dimensions; e.g. ``expand_v = 2`` with a head dimension of 128 (V = 256,
``linear_moe/model/common_modules/linear_attention.py`` of the reference scales ``head_v_dim`` that way)."""
import pytest
import torch
import torch.nn.functional as F

from oracle import naive
from tests.util import TOL, gen, max_abs_rel, oracle_grads

pytestmark = pytest.mark.gpu


def _check(cuda, dtype, ins, do, dht, ref_fn, run):
    ref_o, ref_ht, ref = oracle_grads(ref_fn, ins, do, dht)
    dev = {n: (None if x is None else x.to(cuda).requires_grad_(True)) for n, x in ins.items()}
    o, ht = run(dev)
    ((o * do.to(cuda)).sum() + (ht * dht.to(cuda)).sum()).backward()
    torch.cuda.synchronize()
    tol = TOL[dtype]
    assert o.dtype == dtype and o.shape == ref_o.shape and ht.shape == ref_ht.shape
    assert max_abs_rel(o.detach().cpu(), ref_o) < tol
    assert max_abs_rel(ht.detach().cpu(), ref_ht) < tol
    for n, r in ref.items():
        err = max_abs_rel(dev[n].grad.cpu(), r)
        assert err < tol, (n, err)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("K,V", [(128, 256), (96, 192), (32, 48), (64, 80), (128, 320), (64, 256)])
def test_gated_delta_rule_other_head_dims(cuda, dtype, K, V):
    from linear_moe_amd import chunk_gated_delta_rule
    B, T, H = 2, 130, 2
    q = F.normalize(gen(1, B, T, H, K), dim=-1).to(dtype)
    k = F.normalize(gen(2, B, T, H, K), dim=-1).to(dtype)
    v = gen(3, B, T, H, V, dtype=dtype)
    g = -torch.rand(B, T, H, generator=torch.Generator().manual_seed(4))
    beta = torch.rand(B, T, H, generator=torch.Generator().manual_seed(5)).to(dtype)
    ins = dict(q=q, k=k, v=v, g=g, beta=beta, h0=gen(6, B, H, K, V) * 0.1)
    do, dht = gen(7, B, T, H, V, dtype=dtype), gen(8, B, H, K, V)
    _check(cuda, dtype, ins, do, dht,
           lambda q, k, v, g, beta, h0: naive.naive_recurrent_gated_delta_rule(q, k, v, g, beta, None, h0, True, None, False),
           lambda d: chunk_gated_delta_rule(d['q'], d['k'], d['v'], d['g'], d['beta'], None, d['h0'], True, None, False))


def test_gated_delta_rule_rejects_a_key_beyond_one_block(cuda):
    from linear_moe_amd import chunk_gated_delta_rule
    x = torch.zeros(1, 4, 1, 160, device=cuda, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="K <= 128"):
        chunk_gated_delta_rule(x, x, x[..., :64], torch.zeros(1, 4, 1, device=cuda), torch.zeros(1, 4, 1, device=cuda))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("K,V", [(192, 80), (48, 256), (256, 128)])
def test_gla_other_head_dims(cuda, dtype, K, V):
    from linear_moe_amd import chunk_gla
    B, H, T = 1, 2, 130
    q, k, v = gen(11, B, H, T, K, dtype=dtype), gen(12, B, H, T, K, dtype=dtype), gen(13, B, H, T, V, dtype=dtype)
    g = F.logsigmoid(gen(14, B, H, T, K)) / 16
    ins = dict(q=q, k=k, v=v, g=g, h0=gen(15, B, H, K, V) * 0.5)
    do, dht = gen(16, B, H, T, V, dtype=dtype), gen(17, B, H, K, V)
    _check(cuda, dtype, ins, do, dht,
           lambda q, k, v, g, h0: naive.naive_recurrent_gla(q, k, v, g, None, h0, True, None, True),
           lambda d: chunk_gla(d['q'], d['k'], d['v'], d['g'], None, d['h0'], True, None, True))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("K,V", [(160, 32), (16, 256)])
def test_simple_gla_other_head_dims_packed(cuda, dtype, K, V):
    from linear_moe_amd import chunk_simple_gla
    cu = torch.tensor([0, 70, 71, 200], dtype=torch.int32)
    T, H, N = 200, 2, 3
    q, k, v = gen(21, 1, T, H, K, dtype=dtype), gen(22, 1, T, H, K, dtype=dtype), gen(23, 1, T, H, V, dtype=dtype)
    g = F.logsigmoid(gen(24, 1, T, H))
    ins = dict(q=q, k=k, v=v, g=g, h0=gen(25, N, H, K, V) * 0.5)
    do, dht = gen(26, 1, T, H, V, dtype=dtype), gen(27, N, H, K, V)
    _check(cuda, dtype, ins, do, dht,
           lambda q, k, v, g, h0: naive.naive_recurrent_simple_gla(q, k, v, g, None, h0, True, cu, False),
           lambda d: chunk_simple_gla(d['q'], d['k'], d['v'], d['g'], None, d['h0'], True, cu.to(cuda), False))


def test_delta_rule_other_head_dims(cuda):
    from linear_moe_amd import chunk_delta_rule
    dtype = torch.bfloat16
    B, H, T, K, V = 1, 2, 100, 96, 256
    q = F.normalize(gen(31, B, H, T, K), dim=-1).to(dtype)
    k = F.normalize(gen(32, B, H, T, K), dim=-1).to(dtype)
    v = gen(33, B, H, T, V, dtype=dtype)
    beta = torch.rand(B, H, T, generator=torch.Generator().manual_seed(34)).to(dtype)
    ins = dict(q=q, k=k, v=v, beta=beta, h0=gen(35, B, H, K, V) * 0.1)
    do, dht = gen(36, B, H, T, V, dtype=dtype), gen(37, B, H, K, V)
    _check(cuda, dtype, ins, do, dht,
           lambda q, k, v, beta, h0: naive.naive_recurrent_gated_delta_rule(q, k, v, None, beta, None, h0, True, None, True),
           lambda d: chunk_delta_rule(d['q'], d['k'], d['v'], d['beta'], 64, None, d['h0'], True, None, True))
