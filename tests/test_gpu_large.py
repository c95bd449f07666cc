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
