"""GPU edge cases of the three chunk ops (HIP, through the C ABI): a packed batch that contains an empty
sequence, and a call with no tokens at all.  An empty sequence hands its initial state through unchanged
(final state = initial state, gradient of the initial state = gradient of the final state)."""
import pytest
import torch
import torch.nn.functional as F

from oracle import naive
from tests.util import TOL, gen, max_abs_rel, oracle_grads

pytestmark = pytest.mark.gpu

OPS = ["simple_gla", "gla", "gdn"]


def _inputs(op, T, H, K, V, dtype, seed):
    q, k = gen(seed, 1, T, H, K, dtype=dtype), F.normalize(gen(seed + 1, 1, T, H, K), dim=-1).to(dtype)
    v = gen(seed + 2, 1, T, H, V, dtype=dtype)
    ins = dict(q=q, k=k, v=v)
    if op == "gla":
        ins["g"] = F.logsigmoid(gen(seed + 3, 1, T, H, K)) / 4
    else:
        ins["g"] = F.logsigmoid(gen(seed + 3, 1, T, H))
    if op == "gdn":
        ins["beta"] = torch.sigmoid(gen(seed + 4, 1, T, H)).to(dtype)
    return ins


def _call(op, ins, h0, cu, ours):
    if ours:
        from linear_moe_amd import chunk_gated_delta_rule, chunk_gla, chunk_simple_gla
        if op == "simple_gla":
            return chunk_simple_gla(ins["q"], ins["k"], ins["v"], ins["g"], None, h0, True, cu, False)
        if op == "gla":
            return chunk_gla(ins["q"], ins["k"], ins["v"], ins["g"], None, h0, True, cu, False)
        return chunk_gated_delta_rule(ins["q"], ins["k"], ins["v"], ins["g"], ins["beta"], None, h0, True, cu, False)
    if op == "simple_gla":
        return naive.naive_recurrent_simple_gla(ins["q"], ins["k"], ins["v"], ins["g"], None, h0, True, cu, False)
    if op == "gla":
        return naive.naive_recurrent_gla(ins["q"], ins["k"], ins["v"], ins["g"], None, h0, True, cu, False)
    return naive.naive_recurrent_gated_delta_rule(ins["q"], ins["k"], ins["v"], ins["g"], ins["beta"], None, h0, True, cu, False)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("op", OPS)
def test_packed_batch_with_empty_sequences(cuda, op, dtype):
    cu = torch.tensor([0, 0, 70, 70, 200, 200], dtype=torch.int32)       # sequences 0, 2 and 4 are empty
    T, H, K, V, N = 200, 2, 64, 64, 5
    ins = _inputs(op, T, H, K, V, dtype, 3000)
    h0 = gen(3010, N, H, K, V) * 0.5
    do, dht = gen(3011, 1, T, H, V, dtype=dtype), gen(3012, N, H, K, V)
    names = list(ins)
    ref_in = dict(ins, h0=h0)
    fn = lambda **kw: _call(op, {n: kw[n] for n in names}, kw["h0"], cu, False)
    ref_o, ref_ht, ref = oracle_grads(fn, ref_in, do, dht)
    dev = {n: x.to(cuda).requires_grad_(True) for n, x in ref_in.items()}
    o, ht = _call(op, dev, dev["h0"], cu.to(cuda), True)
    ((o * do.to(cuda)).sum() + (ht * dht.to(cuda)).sum()).backward()
    torch.cuda.synchronize()
    tol = TOL[dtype]
    assert max_abs_rel(o.detach().cpu(), ref_o) < tol
    assert max_abs_rel(ht.detach().cpu(), ref_ht) < tol
    for e in (0, 2, 4):                                                   # handed through bit for bit
        assert torch.equal(ht[e].detach().cpu(), h0[e])
        assert torch.equal(dev["h0"].grad[e].cpu(), dht[e])
    for n, r in ref.items():
        assert max_abs_rel(dev[n].grad.cpu(), r) < tol, n


@pytest.mark.parametrize("op", OPS)
def test_no_tokens_at_all(cuda, op):
    dtype = torch.bfloat16
    B, T, H, K, V = 2, 0, 2, 64, 64
    q, k, v = (torch.zeros(B, T, H, D, dtype=dtype, device=cuda, requires_grad=True) for D in (K, K, V))
    ins = dict(q=q, k=k, v=v)
    ins["g"] = torch.zeros(B, T, H, K, device=cuda) if op == "gla" else torch.zeros(B, T, H, device=cuda)
    if op == "gdn":
        ins["beta"] = torch.zeros(B, T, H, dtype=dtype, device=cuda)
    h0 = (gen(3100, B, H, K, V) * 0.5).to(cuda).requires_grad_(True)
    dht = gen(3101, B, H, K, V).to(cuda)
    o, ht = _call(op, ins, h0, None, True)
    assert o.shape == (B, T, H, V)
    (ht * dht).sum().backward()
    torch.cuda.synchronize()
    assert torch.equal(ht.detach(), h0.detach())
    assert torch.equal(h0.grad, dht)
