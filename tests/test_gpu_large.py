"""Tensors of more than 2^31 elements (packed input, 17 sequences of 65536 tokens, H = 16, K = V = 128: 2.28 G
elements per tensor, about 80 GB on the GPU): the last sequence, whose rows lie beyond the 32-bit element range,
gives bit for bit what it gives as a call of its own -- outputs, final state and every gradient."""
import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("op", ["gdn", "gla", "simple_gla"])
def test_offsets_beyond_32_bits(cuda, op):
    import linear_moe_amd as L
    if torch.cuda.get_device_properties(0).total_memory < 150 * 2**30:
        pytest.skip("needs about 100 GB of GPU memory")
    N, Ls, H, K, V = 17, 65536, 16, 128, 128
    T = N * Ls
    assert T * H * K > 2**31
    g_ = torch.Generator(device=cuda).manual_seed(5)
    rn = lambda *s, dt=torch.bfloat16: torch.randn(*s, device=cuda, generator=g_, dtype=torch.float32).to(dt)
    q = F.normalize(rn(1, T, H, K, dt=torch.float32), dim=-1).bfloat16()
    k = F.normalize(rn(1, T, H, K, dt=torch.float32), dim=-1).bfloat16()
    v = rn(1, T, H, V)
    if op == "gla":
        g = (-torch.rand(1, T, H, K, device=cuda, generator=g_) * 0.1).bfloat16()
    else:
        g = -torch.rand(1, T, H, device=cuda, generator=g_) * 0.1
    beta = torch.sigmoid(rn(1, T, H, dt=torch.float32)).bfloat16()
    h0 = rn(N, H, K, V, dt=torch.float32) * 0.1
    do, dht = rn(1, T, H, V), rn(N, H, K, V, dt=torch.float32)
    cu = torch.arange(N + 1, dtype=torch.int32, device=cuda) * Ls

    def run(q, k, v, g, beta, h0, cu, do, dht):
        ins = [x.clone().requires_grad_(True) for x in ((q, k, v, g, beta, h0) if op == "gdn" else (q, k, v, g, h0))]
        if op == "gdn":
            o, ht = L.chunk_gated_delta_rule(*ins[:5], None, ins[5], True, cu, False)
        elif op == "gla":
            o, ht = L.chunk_gla(*ins[:4], None, ins[4], True, cu, False)
        else:
            o, ht = L.chunk_simple_gla(*ins[:4], None, ins[4], True, cu, False)
        return (o.detach(), ht.detach()) + tuple(torch.autograd.grad([o, ht], ins, [do, dht]))

    s = N - 1
    sl = slice(s * Ls, (s + 1) * Ls)
    cut = lambda x: x[:, sl].contiguous()
    small = run(cut(q), cut(k), cut(v), cut(g), cut(beta), h0[s:s + 1].contiguous(), None, cut(do), dht[s:s + 1].contiguous())
    big = run(q, k, v, g, beta, h0, cu, do, dht)
    torch.cuda.synchronize()
    per_seq = (1, len(big) - 1)                        # ht and dh0 are per sequence, the rest per token
    for i, (a, b) in enumerate(zip(big, small)):
        a = a[s:s + 1] if i in per_seq else a[:, sl]
        assert torch.equal(a, b), i
    del big, small
    torch.cuda.empty_cache()


def test_row_kernels_beyond_32_bits(cuda):
    """Row-wise neighbours on 2^24 + 1000 rows of 128 (2.15 G elements): the last rows equal a small call."""
    from linear_moe_amd import gla_gate, l2_norm, rms_norm_fn, silu_l2_norm
    if torch.cuda.get_device_properties(0).total_memory < 150 * 2**30:
        pytest.skip("needs about 40 GB of GPU memory")
    rows, D, tail = 2**24 + 1000, 128, 777
    assert rows * D > 2**31
    g_ = torch.Generator(device=cuda).manual_seed(6)
    x = torch.randn(rows, D, device=cuda, generator=g_, dtype=torch.float32).bfloat16()
    dy = torch.randn(tail, D, device=cuda, generator=g_, dtype=torch.float32).bfloat16()
    w = (1 + 0.1 * torch.randn(D, device=cuda, generator=g_)).bfloat16()
    fns = {"l2_norm": lambda t: l2_norm(t), "silu_l2_norm": lambda t: silu_l2_norm(t),
           "rms_norm": lambda t: rms_norm_fn(t, w, None, eps=1e-5), "gla_gate": lambda t: gla_gate(t, 16.0)}
    for name, fn in fns.items():
        xb = x.clone().requires_grad_(True)
        yb = fn(xb)
        dyb = torch.zeros_like(yb)
        dyb[-tail:] = dy
        (gb,) = torch.autograd.grad(yb, xb, dyb)
        xs = x[-tail:].clone().requires_grad_(True)
        ys = fn(xs)
        (gs,) = torch.autograd.grad(ys, xs, dy)
        torch.cuda.synchronize()
        assert torch.equal(yb[-tail:].detach(), ys.detach()), name
        assert torch.equal(gb[-tail:], gs), name
        del xb, yb, dyb, gb
        torch.cuda.empty_cache()


def test_gated_norm_and_layer_relayouts_beyond_32_bits(cuda):
    """The gated output norm and the two kernels that change the layout (the prologue [T, B, H 3D] -> q^, k^, silu(v) as
    [B, T, H, D]; the epilogue [B, T, H, D] x gate -> [T, B, H D]) on tensors beyond 2^31 elements: the first and the
    last rows / tokens give inside the large call the bits they give as a call of their own, forward and backward; the
    weight gradient of the norm, a sum over all rows, against the same sum formed with torch in pieces."""
    import linear_moe_amd as L
    if torch.cuda.get_device_properties(0).total_memory < 150 * 2**30:
        pytest.skip("needs about 60 GB of GPU memory")
    bf = torch.bfloat16
    D, R, n = 128, 2**24 + 1024, 512
    assert R * D > 2**31
    g_ = torch.Generator(device=cuda).manual_seed(7)
    rnd = lambda *s: torch.randn(*s, generator=g_, device=cuda, dtype=bf)

    def fwd_bwd(f, args, dy):
        leaves = [t.detach().clone().requires_grad_(True) for t in args]
        y = f(*leaves)
        return (y.detach(),) + torch.autograd.grad(y, leaves, dy)

    x, gate, dy = rnd(R, D), rnd(R, D), rnd(R, D)
    w = (1 + 0.1 * torch.randn(D, generator=g_, device=cuda)).to(bf)
    whole = fwd_bwd(lambda a, b: L.rms_norm_swish_gate(a, b, w), (x, gate), dy)
    for sl in (slice(0, n), slice(R - n, R)):
        part = fwd_bwd(lambda a, b: L.rms_norm_swish_gate(a, b, w), (x[sl], gate[sl]), dy[sl])
        torch.cuda.synchronize()
        for a, b in zip(whole, part):
            assert torch.equal(a[sl], b), sl
    del whole
    wl = w.clone().requires_grad_(True)
    (dw,) = torch.autograd.grad(L.rms_norm_swish_gate(x, gate, wl), [wl], dy)
    ref = torch.zeros(D, device=cuda, dtype=torch.float64)
    for r0 in range(0, R, 2**20):
        xs, gs, ds = (t[r0:r0 + 2**20].float() for t in (x, gate, dy))
        ref += (ds * gs * torch.sigmoid(gs) * xs * torch.rsqrt(xs.pow(2).mean(-1, keepdim=True) + 1e-5)).sum(0).double()
    err = float((dw.double() - ref).abs().max() / ref.abs().max())
    assert err < 2e-2, err                               # (dw is handed out in bfloat16)
    del x, gate, dy
    torch.cuda.empty_cache()

    T, B, H = 2**20 + 64, 3, 2                           # qkv: 2.4e9 elements; the last batch entry ends every tensor
    assert T * B * H * 3 * D > 2**31
    pro = lambda t: torch.cat(L.gdn_qkv_prologue(t, H, D), -1)
    qkv, dqkv = rnd(T, B, H * 3 * D), rnd(B, T, H, 3 * D)
    whole = fwd_bwd(pro, (qkv,), dqkv)
    for sl in (slice(0, 64), slice(T - 64, T)):
        part = fwd_bwd(pro, (qkv[sl],), dqkv[:, sl])
        torch.cuda.synchronize()
        assert torch.equal(whole[0][:, sl], part[0]) and torch.equal(whole[1][sl], part[1]), sl
    del whole, qkv, dqkv
    torch.cuda.empty_cache()

    T = 2**22 + 64                                       # [B, T, H D]: 3.2e9 elements
    o, og, dy = rnd(B, T, H, D), rnd(T, B, H * D), rnd(T, B, H * D)
    whole = fwd_bwd(L.swish_gate_relayout, (o, og), dy)
    for sl in (slice(0, 64), slice(T - 64, T)):
        part = fwd_bwd(L.swish_gate_relayout, (o[:, sl], og[sl]), dy[sl])
        torch.cuda.synchronize()
        assert torch.equal(whole[0][sl], part[0]) and torch.equal(whole[1][:, sl], part[1]), sl
        assert torch.equal(whole[2][sl], part[2]), sl
    del whole, o, og, dy
    torch.cuda.empty_cache()
