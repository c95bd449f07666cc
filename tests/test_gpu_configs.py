"""The five configurations of the contract at full size on the GPU.

Parity: the HIP result is compared with the CPU oracle on a slice the oracle finishes in
seconds (batch rows and heads are independent, so a slice of them is an exact sub-problem);
where gradients are needed at long T the float64 chunked restatement (pinned against the token
recurrence + autograd in tests/test_oracle_pins.py) is the checker.  On top of that, properties
that hold at any size are checked at the full size: state hand-off across a split that is not
a chunk multiple, and packed variable-length input == the dense op sequence by sequence.
Tolerances: fp32 max-abs error <= 1e-5 of max |ref|; bf16 <= 2e-2 of max |ref|.
"""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import chunked, naive
from tests.util import TOL, max_abs_rel

pytestmark = pytest.mark.gpu


def rn(gen, *shape):
    return torch.randn(*shape, generator=gen, dtype=torch.float32)


def test_config1_basic_linear_attention_fp32(cuda):
    from linear_moe_amd import chunk_linear_attn
    g_ = torch.Generator().manual_seed(1000)
    B, H, T, K = 1, 4, 512, 64
    q, k, v = rn(g_, B, H, T, K), rn(g_, B, H, T, K), rn(g_, B, H, T, K)
    ref, _ = naive.naive_recurrent_simple_gla(q, k, v, None, K ** -0.5)
    o, _ = chunk_linear_attn(q.to(cuda), k.to(cuda), v.to(cuda), normalize=False)
    assert o.dtype == torch.float32
    assert max_abs_rel(o.cpu(), ref) < 1e-5
    # elementwise relative error where the reference is not tiny
    big = ref.abs() > 1e-2 * ref.abs().max()
    assert ((o.cpu().double() - ref)[big].abs() / ref[big].abs()).max() < 1e-4


def test_config2_retention_bf16(cuda):
    from linear_moe_amd import chunk_retention, chunk_simple_gla
    g_ = torch.Generator().manual_seed(1001)
    B, H, T, K = 4, 16, 4096, 128
    q, k, v = (rn(g_, B, H, T, K).bfloat16() for _ in range(3))
    qd, kd, vd = q.to(cuda), k.to(cuda), v.to(cuda)
    o, ht = chunk_retention(qd, kd, vd, output_final_state=True)
    assert ht.shape == (B, H, K, K) and ht.dtype == torch.float32
    ref_o, ref_ht = naive.naive_retention(q[:1], k[:1], v[:1], output_final_state=True, dtype=torch.float32)
    assert max_abs_rel(o[:1].cpu(), ref_o) < TOL[torch.bfloat16]
    assert max_abs_rel(ht[:1].cpu(), ref_ht) < TOL[torch.bfloat16]
    # full size: split at a non-multiple of 64 and hand the state over
    T1 = 1000
    gh = torch.log1p(-torch.pow(2.0, -5.0 - torch.arange(H, dtype=torch.float32))).to(cuda)
    g = gh[None, :, None].expand(B, H, T)
    o1, h1 = chunk_simple_gla(qd[:, :, :T1], kd[:, :, :T1], vd[:, :, :T1], g[:, :, :T1], None, None, True)
    o2, h2 = chunk_simple_gla(qd[:, :, T1:], kd[:, :, T1:], vd[:, :, T1:], g[:, :, T1:], None, h1, True)
    assert max_abs_rel(torch.cat([o1, o2], 2), o) < TOL[torch.bfloat16]
    assert max_abs_rel(h2, ht) < TOL[torch.bfloat16]


def _check_grads(got, ref, tol):
    for n, r in ref.items():
        err = max_abs_rel(got[n], r)
        assert err < tol, (n, err)


def test_config3_gla_fwd_bwd_bf16(cuda):
    from linear_moe_amd import chunk_gla
    g_ = torch.Generator().manual_seed(1002)
    B, H, T, K, V = 8, 16, 2048, 64, 128
    q, k = rn(g_, B, H, T, K).bfloat16(), rn(g_, B, H, T, K).bfloat16()
    v = rn(g_, B, H, T, V).bfloat16()
    g = (F.logsigmoid(rn(g_, B, H, T, K)) / 16).bfloat16()
    do = rn(g_, B, H, T, V).bfloat16()
    h0 = torch.zeros(B, H, K, V)
    d = {n: x.to(cuda).requires_grad_(True) for n, x in dict(q=q, k=k, v=v, g=g, h0=h0).items()}
    o, _ = chunk_gla(d['q'], d['k'], d['v'], d['g'], None, d['h0'], False)
    (o * do.to(cuda)).sum().backward()
    torch.cuda.synchronize()
    # checker: float64 chunked restatement on batch row 0, heads 0..3
    s = (slice(0, 1), slice(0, 4))
    ro, _, (dq, dk, dv, dg, _, dh0) = chunked.chunk_fwd_bwd(
        'gla', q[s], k[s], v[s], g[s], None, None, h0[s], do[s], None, dtype=torch.float64)
    tol = TOL[torch.bfloat16]
    assert max_abs_rel(o[s].detach().cpu(), ro) < tol
    _check_grads({n: d[n].grad[s].cpu() for n in d}, dict(q=dq, k=dk, v=dv, g=dg, h0=dh0), tol)


def gdn_laws(g_, B, T, H, K, V):
    q = F.normalize(rn(g_, B, T, H, K), dim=-1).bfloat16()
    k = F.normalize(rn(g_, B, T, H, K), dim=-1).bfloat16()
    v = rn(g_, B, T, H, V).bfloat16()
    beta = torch.sigmoid(rn(g_, B, T, H)).bfloat16()
    A = torch.rand(H, generator=g_) * math.log(16.0)
    dtb = rn(g_, H) * 0.1
    g = -torch.exp(A)[None, None] * F.softplus(rn(g_, B, T, H) + dtb[None, None])
    do = rn(g_, B, T, H, V).bfloat16()
    return q, k, v, g, beta, do


def test_config4_gated_delta_rule_fwd_bwd_bf16(cuda):
    from linear_moe_amd import chunk_gated_delta_rule
    g_ = torch.Generator().manual_seed(1003)
    B, T, H, K, V = 4, 8192, 16, 128, 128
    q, k, v, g, beta, do = gdn_laws(g_, B, T, H, K, V)
    d = {n: x.to(cuda).requires_grad_(True) for n, x in dict(q=q, k=k, v=v, g=g, beta=beta).items()}
    o, _ = chunk_gated_delta_rule(d['q'], d['k'], d['v'], d['g'], d['beta'], head_first=False)
    (o * do.to(cuda)).sum().backward()
    torch.cuda.synchronize()
    hf = lambda x: x[:1, :, :4].transpose(1, 2)          # batch row 0, heads 0..3, head-first
    ro, _, (dq, dk, dv, dg, dbeta, _) = chunked.chunk_fwd_bwd(
        'gdn', hf(q), hf(k), hf(v), hf(g), hf(beta), None, None, hf(do), None, dtype=torch.float64)
    # the chunked checker itself against the token recurrence, forward, on the same slice
    no, _ = naive.naive_recurrent_gated_delta_rule(hf(q), hf(k), hf(v), hf(g), hf(beta), head_first=True,
                                                   dtype=torch.float32)
    assert max_abs_rel(no, ro) < 1e-4
    tol = TOL[torch.bfloat16]
    assert max_abs_rel(hf(o.detach().cpu()), ro) < tol
    _check_grads({n: hf(d[n].grad.cpu()) for n in d}, dict(q=dq, k=dk, v=dv, g=dg, beta=dbeta), tol)


def lognormal_lengths(g_, n, total):
    raw = torch.exp(8.0 + torch.randn(n, generator=g_))
    lens = torch.clamp((raw / raw.sum() * total).floor().long(), min=1)
    lens[lens.argmax()] += total - lens.sum()
    return lens


def test_config5_varlen_gated_delta_rule_fwd_bwd_bf16(cuda):
    from linear_moe_amd import chunk_gated_delta_rule
    g_ = torch.Generator().manual_seed(1004)
    N, Ttot, H, K, V = 16, 65536, 32, 128, 128
    lens = lognormal_lengths(g_, N, Ttot)
    cu = torch.zeros(N + 1, dtype=torch.int32)
    cu[1:] = lens.cumsum(0)
    assert int(cu[-1]) == Ttot
    q, k, v, g, beta, do = gdn_laws(g_, 1, Ttot, H, K, V)
    h0 = rn(g_, N, H, K, V) * 0.1
    dht = rn(g_, N, H, K, V)
    d = {n: x.to(cuda).requires_grad_(True) for n, x in dict(q=q, k=k, v=v, g=g, beta=beta, h0=h0).items()}
    o, ht = chunk_gated_delta_rule(d['q'], d['k'], d['v'], d['g'], d['beta'], None, d['h0'], True, cu.to(cuda), False)
    ((o * do.to(cuda)).sum() + (ht * dht.to(cuda)).sum()).backward()
    torch.cuda.synchronize()
    tol = TOL[torch.bfloat16]
    # checker: float64 chunked restatement, heads 0..1, the 5 shortest and the longest sequence
    order = lens.argsort()
    picks = order[:5].tolist() + [order[-1].item()]
    hs_ = slice(0, 2)
    for n in picks:
        s, e = int(cu[n]), int(cu[n + 1])
        hf = lambda x: x[:, s:e, hs_].transpose(1, 2)
        ro, rht, (dq, dk, dv, dg, dbeta, dh0) = chunked.chunk_fwd_bwd(
            'gdn', hf(q), hf(k), hf(v), hf(g), hf(beta), None, h0[n:n + 1, hs_], hf(do), dht[n:n + 1, hs_],
            dtype=torch.float64)
        assert max_abs_rel(hf(o.detach().cpu()), ro) < tol, n
        assert max_abs_rel(ht[n:n + 1, hs_].detach().cpu(), rht) < tol, n
        got = {m: hf(d[m].grad.cpu()) for m in ('q', 'k', 'v', 'g', 'beta')}
        got['h0'] = d['h0'].grad[n:n + 1, hs_].cpu()
        _check_grads(got, dict(q=dq, k=dk, v=dv, g=dg, beta=dbeta, h0=dh0), tol)
    # full size property: packed call == dense call of the same op, sequence by sequence
    for n in (order[0].item(), order[N // 2].item(), order[-1].item()):
        s, e = int(cu[n]), int(cu[n + 1])
        with torch.no_grad():
            on, hn = chunk_gated_delta_rule(d['q'][:, s:e], d['k'][:, s:e], d['v'][:, s:e], d['g'][:, s:e],
                                            d['beta'][:, s:e], None, d['h0'][n:n + 1], True, None, False)
        assert max_abs_rel(on, o[:, s:e].detach()) < 1e-6 and max_abs_rel(hn, ht[n:n + 1].detach()) < 1e-6
