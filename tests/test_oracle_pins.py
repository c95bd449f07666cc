"""Pins of the CPU oracle (oracle/naive.py, oracle/chunked.py).

The reference ships no test or golden vector for this path (its arithmetic lives in the absent
flash-linear-attention submodule), so the oracle is pinned by what the mathematics fixes:
closed forms, special cases that reduce to library routines, hand-unrolled tiny cases,
invariants, finite differences, and the independent torch routines shipped with
``transformers`` for the gated delta rule.  Each check is chosen so that a plausible slip (a
dropped decay, a transposed operand, an off-by-one in the gate's position) breaks it.
"""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import chunked, naive

D = torch.float64


def rnd(seed, *shape):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=D)


# ----------------------------- closed forms -------------------------------- #
def test_simple_gla_no_gate_is_masked_attention():
    q, k, v = rnd(1, 2, 3, 37, 8), rnd(2, 2, 3, 37, 8), rnd(3, 2, 3, 37, 5)
    o, ht = naive.naive_recurrent_simple_gla(q, k, v, None, 0.3, None, True)
    ref = 0.3 * torch.tril(q @ k.transpose(-1, -2)) @ v
    assert torch.allclose(o, ref, atol=1e-12)
    assert torch.allclose(ht, k.transpose(-1, -2) @ v, atol=1e-12)


def test_default_scale_is_rsqrt_k():
    q, k, v = rnd(1, 1, 1, 9, 16), rnd(2, 1, 1, 9, 16), rnd(3, 1, 1, 9, 4)
    o, _ = naive.naive_recurrent_simple_gla(q, k, v)
    assert torch.allclose(o, 0.25 * torch.tril(q @ k.transpose(-1, -2)) @ v, atol=1e-12)


def test_linear_attn_normalised_closed_form_and_by_hand():
    """normalize=True: o_t = sum_{s<=t} a_ts v_s / (sum_{s<=t} a_ts + eps), a_ts = scale q_t.k_s -- the scale sits in
    the numerator AND in the normaliser (a normaliser built from the unscaled q is off by 1/scale)."""
    q, k, v = rnd(11, 2, 3, 41, 8).abs(), rnd(12, 2, 3, 41, 8).abs(), rnd(13, 2, 3, 41, 5)
    for scale, eps in ((None, 1e-10), (1.0, 1e-10), (0.37, 1e-10), (0.37, 0.5)):
        o, ht = naive.naive_linear_attn(q, k, v, scale=scale, output_final_state=True, normalize=True, eps=eps)
        sc = 8 ** -0.5 if scale is None else scale
        A = torch.tril(sc * q @ k.transpose(-1, -2))
        assert torch.allclose(o, (A @ v) / (A.sum(-1, keepdim=True) + eps), atol=1e-12)
        assert torch.allclose(ht, k.transpose(-1, -2) @ v, atol=1e-12)          # the state is not normalised
        o_tf, _ = naive.naive_linear_attn(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), scale=scale,
                                          normalize=True, head_first=False, eps=eps)
        assert torch.allclose(o_tf.transpose(1, 2), o, atol=1e-12)
    # by hand, T = 2, K = V = 1, scale 1/2, eps = 1 (large on purpose: it shows where the scale sits):
    # a00 = .5*2*5 = 5, a10 = .5*3*5 = 7.5, a11 = .5*3*7 = 10.5;  o0 = 5*11/(5+1),  o1 = (7.5*11 + 10.5*13)/(18+1)
    t = lambda *x: torch.tensor(x, dtype=D).reshape(1, 1, 2, 1)
    o, _ = naive.naive_linear_attn(t(2, 3), t(5, 7), t(11, 13), scale=0.5, normalize=True, eps=1.0)
    assert torch.allclose(o.flatten(), torch.tensor([55 / 6, 219 / 19], dtype=D), atol=1e-13)
    # Based end to end: Taylor features, scale 1 -> weights 1 + s + s^2/2 with s = q.k / sqrt(D)
    Dh = 4
    q, k, v = 0.5 * rnd(14, 1, 2, 23, Dh), 0.5 * rnd(15, 1, 2, 23, Dh), rnd(16, 1, 2, 23, 3)
    o, _ = naive.naive_linear_attn(naive.naive_taylor_feature_map(q), naive.naive_taylor_feature_map(k), v, scale=1.0,
                                   normalize=True)
    x = q @ k.transpose(-1, -2) / Dh ** 0.5
    W = torch.tril(1 + x + x * x / 2)
    assert torch.allclose(o, (W @ v) / (W.sum(-1, keepdim=True) + 1e-10), atol=1e-12)


def test_retention_closed_form():
    B, H, T = 1, 4, 50
    q, k, v = rnd(4, B, H, T, 8), rnd(5, B, H, T, 8), rnd(6, B, H, T, 6)
    o, _ = naive.naive_retention(q, k, v, scale=1.0)
    gam = 1 - torch.pow(torch.tensor(2.0, dtype=D), -5.0 - torch.arange(H, dtype=D))
    idx = torch.arange(T)
    dist = (idx[:, None] - idx[None, :]).clamp_min(0).to(D)
    Dm = torch.tril(gam[:, None, None] ** dist)
    ref = ((q @ k.transpose(-1, -2)) * Dm[None]) @ v
    assert torch.allclose(o, ref, atol=1e-12)
    # value of the first head's decay: 1 - 2^-5
    assert math.isclose(math.exp(naive.retention_log_decay(4)[0].item()), 1 - 2 ** -5, rel_tol=1e-14)


def test_lightning_slopes_and_closed_form():
    s8 = naive.lightning_slopes(8)
    assert torch.allclose(s8, torch.tensor([2.0 ** -(i + 1) for i in range(8)], dtype=D))
    s16 = naive.lightning_slopes(16)
    assert torch.allclose(s16, torch.tensor([2.0 ** (-(i + 1) / 2) for i in range(16)], dtype=D))
    assert len(naive.lightning_slopes(12)) == 12          # non power of two: interleaved completion
    B, H, T = 1, 8, 20
    q, k, v = rnd(7, B, H, T, 4), rnd(8, B, H, T, 4), rnd(9, B, H, T, 4)
    o = naive.naive_lightning_attn2(q, k, v, s8.reshape(H, 1, 1))
    idx = torch.arange(T)
    dist = (idx[:, None] - idx[None, :]).clamp_min(0).to(D)
    Dm = torch.tril(torch.exp(-s8[:, None, None] * dist))
    assert torch.allclose(o, ((q @ k.transpose(-1, -2)) * Dm[None]) @ v, atol=1e-12)


def test_scalars_by_hand():
    # K = V = 1, T = 3, everything written out
    q = torch.tensor([2.0, -1.0, 0.5], dtype=D).view(1, 1, 3, 1)
    k = torch.tensor([1.0, 3.0, -2.0], dtype=D).view(1, 1, 3, 1)
    v = torch.tensor([0.5, 1.0, 4.0], dtype=D).view(1, 1, 3, 1)
    g = torch.tensor([-0.1, -0.2, -0.3], dtype=D).view(1, 1, 3)
    h0 = torch.tensor([[[[0.7]]]], dtype=D)
    e = math.exp
    s1 = e(-0.1) * 0.7 + 1.0 * 0.5
    s2 = e(-0.2) * s1 + 3.0 * 1.0
    s3 = e(-0.3) * s2 + (-2.0) * 4.0
    o, ht = naive.naive_recurrent_simple_gla(q, k, v, g, 1.0, h0, True)
    assert torch.allclose(o.flatten(), torch.tensor([2 * s1, -s2, 0.5 * s3], dtype=D), atol=1e-14)
    assert math.isclose(ht.item(), s3, rel_tol=1e-14)
    # gated delta rule on the same numbers, beta = (0.5, 1, 0.25)
    beta = torch.tensor([0.5, 1.0, 0.25], dtype=D).view(1, 1, 3)
    t1 = e(-0.1) * 0.7
    d1 = t1 + 1.0 * 0.5 * (0.5 - 1.0 * t1)
    t2 = e(-0.2) * d1
    d2 = t2 + 3.0 * 1.0 * (1.0 - 3.0 * t2)
    t3 = e(-0.3) * d2
    d3 = t3 + (-2.0) * 0.25 * (4.0 - (-2.0) * t3)
    o, ht = naive.naive_recurrent_gated_delta_rule(q, k, v, g, beta, 1.0, h0, True, head_first=True)
    assert torch.allclose(o.flatten(), torch.tensor([2 * d1, -d2, 0.5 * d3], dtype=D), atol=1e-14)
    assert math.isclose(ht.item(), d3, rel_tol=1e-14)


def test_gla_channel_constant_gate_equals_simple_gla():
    q, k, v = rnd(10, 2, 2, 33, 8), rnd(11, 2, 2, 33, 8), rnd(12, 2, 2, 33, 6)
    g = F.logsigmoid(rnd(13, 2, 2, 33))
    h0 = rnd(14, 2, 2, 8, 6)
    o1, h1 = naive.naive_recurrent_simple_gla(q, k, v, g, None, h0, True)
    o2, h2 = naive.naive_recurrent_gla(q, k, v, g[..., None].expand(-1, -1, -1, 8), None, h0, True)
    assert torch.allclose(o1, o2, atol=1e-12) and torch.allclose(h1, h2, atol=1e-12)


def test_gla_per_channel_decay_closed_form():
    # o_t = scale sum_{s<=t} sum_k q_tk k_sk exp(sum_{s<r<=t} g_rk) v_s
    B, H, T, K, V = 1, 1, 6, 3, 2
    q, k, v = rnd(15, B, H, T, K), rnd(16, B, H, T, K), rnd(17, B, H, T, V)
    g = F.logsigmoid(rnd(18, B, H, T, K))
    o, _ = naive.naive_recurrent_gla(q, k, v, g, 1.0)
    cs = g.cumsum(2)
    ref = torch.zeros(B, H, T, V, dtype=D)
    for t in range(T):
        for s in range(t + 1):
            wgt = (q[0, 0, t] * k[0, 0, s] * torch.exp(cs[0, 0, t] - cs[0, 0, s])).sum()
            ref[0, 0, t] += wgt * v[0, 0, s]
    assert torch.allclose(o, ref, atol=1e-12)


def test_gdn_beta_zero_only_decays_initial_state():
    B, H, T, K, V = 1, 2, 20, 4, 3
    q, k, v = rnd(19, B, T, H, K), rnd(20, B, T, H, K), rnd(21, B, T, H, V)
    g = F.logsigmoid(rnd(22, B, T, H))
    h0 = rnd(23, B, H, K, V)
    o, ht = naive.naive_recurrent_gated_delta_rule(q, k, v, g, torch.zeros(B, T, H, dtype=D), 1.0, h0, True)
    dec = torch.exp(g.cumsum(1))                                    # [B,T,H]
    ref = torch.einsum('bthk,bhkv->bthv', q, h0) * dec[..., None]
    assert torch.allclose(o, ref, atol=1e-12)
    assert torch.allclose(ht, h0 * dec[:, -1, :, None, None], atol=1e-12)


def test_gdn_orthonormal_keys_store_values_exactly():
    # distinct orthonormal keys, beta = 1, no decay: the state maps k_i to v_i
    K = V = T = 8
    k = torch.linalg.qr(rnd(24, K, K))[0].view(1, T, 1, K)
    v = rnd(25, 1, T, 1, V)
    z = torch.zeros(1, T, 1, dtype=D)
    o, ht = naive.naive_recurrent_gated_delta_rule(k, k, v, z, torch.ones(1, T, 1, dtype=D), 1.0, None, True)
    assert torch.allclose(torch.einsum('bthk,bhkv->bthv', k, ht), v, atol=1e-12)
    assert torch.allclose(o, v, atol=1e-12)          # querying with k_t right after writing v_t


def test_gdn_matches_transformers_torch_routines():
    tr = pytest.importorskip("transformers.models.qwen3_next.modeling_qwen3_next")
    B, T, H, K, V = 2, 150, 3, 16, 24
    q = F.normalize(rnd(26, B, T, H, K), dim=-1)
    k = F.normalize(rnd(27, B, T, H, K), dim=-1)
    v, beta = rnd(28, B, T, H, V), torch.sigmoid(rnd(29, B, T, H))
    g = -torch.rand(B, T, H, generator=torch.Generator().manual_seed(30), dtype=D)
    h0 = rnd(31, B, H, K, V) * 0.3
    o, ht = naive.naive_recurrent_gated_delta_rule(q, k, v, g, beta, None, h0, True)
    f = lambda x: x.float()
    o1, h1 = tr.torch_recurrent_gated_delta_rule(f(q), f(k), f(v), f(g), f(beta), f(h0), True)
    o2, h2 = tr.torch_chunk_gated_delta_rule(f(q), f(k), f(v), f(g), f(beta), 64, f(h0), True)
    for oo, hh in ((o1, h1), (o2, h2)):
        assert (oo.double() - o).abs().max() < 2e-5 * o.abs().max().clamp_min(1)
        assert (hh.double() - ht).abs().max() < 2e-5 * ht.abs().max().clamp_min(1)


# ------------------------------- invariants -------------------------------- #
def _ops():
    B, H, T, K, V = 2, 2, 90, 8, 6
    q, k, v = rnd(40, B, H, T, K), rnd(41, B, H, T, K), rnd(42, B, H, T, V)
    gs, gv = F.logsigmoid(rnd(43, B, H, T)), F.logsigmoid(rnd(44, B, H, T, K))
    beta = torch.sigmoid(rnd(45, B, H, T))
    kn = F.normalize(k, dim=-1)
    return {
        'simple_gla': lambda q_, k_, v_, h0, sl: naive.naive_recurrent_simple_gla(q_, k_, v_, gs[:, :, sl], None, h0, True),
        'gla': lambda q_, k_, v_, h0, sl: naive.naive_recurrent_gla(q_, k_, v_, gv[:, :, sl], None, h0, True),
        'gdn': lambda q_, k_, v_, h0, sl: naive.naive_recurrent_gated_delta_rule(
            q_, F.normalize(k_, dim=-1), v_, gs[:, :, sl], beta[:, :, sl], None, h0, True, head_first=True),
    }, (q, k, v)


@pytest.mark.parametrize("op", ['simple_gla', 'gla', 'gdn'])
def test_state_handoff_and_linearity(op):
    ops, (q, k, v) = _ops()
    f = ops[op]
    T, T1 = q.shape[2], 37
    full = slice(0, T)
    o, ht = f(q, k, v, None, full)
    o1, h1 = f(q[:, :, :T1], k[:, :, :T1], v[:, :, :T1], None, slice(0, T1))
    o2, h2 = f(q[:, :, T1:], k[:, :, T1:], v[:, :, T1:], h1, slice(T1, T))
    assert torch.allclose(torch.cat([o1, o2], 2), o, atol=1e-11)
    assert torch.allclose(h2, ht, atol=1e-11)
    # linear in v (zero initial state)
    oa, _ = f(q, k, 2.5 * v, None, full)
    assert torch.allclose(oa, 2.5 * o, atol=1e-10)


def test_varlen_equals_per_sequence_and_time_first_equals_head_first():
    T, H, K, V = 60, 2, 8, 6
    cu = torch.tensor([0, 7, 8, 40, 60])
    q, k, v = rnd(50, 1, T, H, K), F.normalize(rnd(51, 1, T, H, K), dim=-1), rnd(52, 1, T, H, V)
    g, beta = F.logsigmoid(rnd(53, 1, T, H)), torch.sigmoid(rnd(54, 1, T, H))
    h0 = rnd(55, 4, H, K, V)
    o, ht = naive.naive_recurrent_gated_delta_rule(q, k, v, g, beta, None, h0, True, cu)
    for n in range(4):
        s, e = int(cu[n]), int(cu[n + 1])
        on, hn = naive.naive_recurrent_gated_delta_rule(q[:, s:e], k[:, s:e], v[:, s:e], g[:, s:e], beta[:, s:e],
                                                        None, h0[n:n + 1], True)
        assert torch.allclose(o[:, s:e], on, atol=1e-12) and torch.allclose(ht[n:n + 1], hn, atol=1e-12)
    tp = lambda x: x.transpose(1, 2)
    oh, hh = naive.naive_recurrent_gated_delta_rule(tp(q), tp(k), tp(v), tp(g), tp(beta), None, h0[:1], True,
                                                    head_first=True)
    ot, ht_ = naive.naive_recurrent_gated_delta_rule(q, k, v, g, beta, None, h0[:1], True)
    assert torch.allclose(tp(oh), ot, atol=1e-12) and torch.allclose(hh, ht_, atol=1e-12)


# ---------------------- gradients: finite differences ---------------------- #
@pytest.mark.parametrize("op", ['simple_gla', 'gla', 'gdn'])
def test_oracle_gradcheck(op):
    B, H, T, K, V = 1, 1, 5, 3, 2
    q, k, v = rnd(60, B, H, T, K), rnd(61, B, H, T, K), rnd(62, B, H, T, V)
    h0 = rnd(63, B, H, K, V)
    if op == 'simple_gla':
        g = F.logsigmoid(rnd(64, B, H, T))
        f = lambda q, k, v, g, h0: naive.naive_recurrent_simple_gla(q, k, v, g, None, h0, True)
        args = (q, k, v, g, h0)
    elif op == 'gla':
        g = F.logsigmoid(rnd(64, B, H, T, K))
        f = lambda q, k, v, g, h0: naive.naive_recurrent_gla(q, k, v, g, None, h0, True)
        args = (q, k, v, g, h0)
    else:
        g, beta = F.logsigmoid(rnd(64, B, H, T)), torch.sigmoid(rnd(65, B, H, T))
        f = lambda q, k, v, g, beta, h0: naive.naive_recurrent_gated_delta_rule(q, k, v, g, beta, None, h0, True,
                                                                              head_first=True)
        args = (q, k, v, g, beta, h0)
    args = tuple(a.clone().requires_grad_(True) for a in args)
    assert torch.autograd.gradcheck(f, args, eps=1e-6, atol=1e-6)


# ------------------ chunked restatement vs token recurrence ---------------- #
@pytest.mark.parametrize("op", ['simple_gla', 'gla', 'gdn'])
@pytest.mark.parametrize("C", [16, 32, 64])
def test_chunked_matches_naive_and_autograd(op, C):
    B, H, T, K, V = 2, 2, 150, 8, 12
    q, k, v = rnd(70, B, H, T, K), rnd(71, B, H, T, K), rnd(72, B, H, T, V)
    if op == 'gdn':
        q, k = F.normalize(q, dim=-1), F.normalize(k, dim=-1)
    g = F.logsigmoid(rnd(73, B, H, T, K)) if op == 'gla' else F.logsigmoid(rnd(73, B, H, T))
    beta = torch.sigmoid(rnd(74, B, H, T)) if op == 'gdn' else None
    h0, do, dht = rnd(75, B, H, K, V) * 0.3, rnd(76, B, H, T, V), rnd(77, B, H, K, V)
    leaves = [x.clone().requires_grad_(True) for x in (q, k, v, g, h0)] + ([beta.clone().requires_grad_(True)] if op == 'gdn' else [])
    if op == 'simple_gla':
        o, ht = naive.naive_recurrent_simple_gla(*leaves[:4], None, leaves[4], True)
    elif op == 'gla':
        o, ht = naive.naive_recurrent_gla(*leaves[:4], None, leaves[4], True)
    else:
        o, ht = naive.naive_recurrent_gated_delta_rule(*leaves[:4], leaves[5], None, leaves[4], True, head_first=True)
    grads = torch.autograd.grad((o * do).sum() + (ht * dht).sum(), leaves)
    o2, ht2, (dq, dk, dv, dg, dbeta, dh0) = chunked.chunk_fwd_bwd(op, q, k, v, g, beta, None, h0, do, dht, C=C, dtype=D)
    assert torch.allclose(o2, o, atol=1e-10) and torch.allclose(ht2, ht, atol=1e-10)
    mine = [dq, dk, dv, dg, dh0] + ([dbeta] if op == 'gdn' else [])
    for a, b in zip(grads, mine):
        assert torch.allclose(a, b, atol=1e-9 * max(1.0, a.abs().max().item()))


def test_wy_backward_through_dZ_equals_the_w_u_form_and_autograd():
    """The form of the gated delta rule's backward that the HIP kernels compute (everything through
    dZ = T^T dv_new: no product with T in the chunk-parallel part, no w in the state recurrence) against the
    w / u form and against autograd through the token recurrence, in fp64 on a case with a partial last chunk, an
    initial state and a gradient of the final state."""
    B, H, T, K, V = 1, 2, 200, 16, 24
    q, k = rnd(81, B, H, T, K), F.normalize(rnd(82, B, H, T, K), dim=-1)
    v, do = rnd(83, B, H, T, V), rnd(86, B, H, T, V)
    g, beta = -torch.rand(B, H, T, dtype=torch.float64, generator=torch.Generator().manual_seed(84)) * 0.5, torch.sigmoid(rnd(85, B, H, T))
    h0, dht = rnd(87, B, H, K, V) * 0.1, rnd(88, B, H, K, V)
    _, _, saved = chunked.chunk_forward('gdn', q, k, v, g, beta, None, h0, 64, torch.float64)
    a = chunked.chunk_backward('gdn', q, k, v, g, beta, None, h0, do, dht, saved, 64, torch.float64)
    b = chunked.chunk_backward('gdn', q, k, v, g, beta, None, h0, do, dht, saved, 64, torch.float64, solve_form=True)
    leaves = [x.clone().requires_grad_(True) for x in (q, k, v, g, beta, h0)]
    o, ht = naive.naive_recurrent_gated_delta_rule(*leaves[:5], None, leaves[5], True, None, True)
    ref = torch.autograd.grad((o * do).sum() + (ht * dht).sum(), leaves)
    for x, y, r in zip(a, b, ref):
        assert (x - y).abs().max() < 1e-12 * max(1.0, r.abs().max().item())
        assert (y - r).abs().max() < 1e-11 * max(1.0, r.abs().max().item())


def test_gate_gradient_identity():
    # dg_t = sum_{s>=t} (q_s.dq_s - k_s.dk_s) + <S_T, dht>   (simple_gla)
    B, H, T, K, V = 1, 2, 40, 4, 3
    q, k, v = (x.requires_grad_(True) for x in (rnd(80, B, H, T, K), rnd(81, B, H, T, K), rnd(82, B, H, T, V)))
    g = F.logsigmoid(rnd(83, B, H, T)).requires_grad_(True)
    do, dht = rnd(84, B, H, T, V), rnd(85, B, H, K, V)
    o, ht = naive.naive_recurrent_simple_gla(q, k, v, g, None, None, True)
    dq, dk, dg = torch.autograd.grad((o * do).sum() + (ht * dht).sum(), (q, k, g))
    x = (q * dq).sum(-1) - (k * dk).sum(-1)
    ref = x.flip(2).cumsum(2).flip(2) + (ht * dht).sum((-1, -2))[..., None]
    assert torch.allclose(dg, ref, atol=1e-10)


def test_l2_norm_pins():
    """naive_l2_norm: library routine for eps = 0, hand-computed values that place eps inside the square
    root, scale invariance, and the backward formula of the reference kernel (l2norm.py:64-95)."""
    import torch.nn.functional as F
    x = rnd(7001, 5, 3, 16).double()
    assert torch.allclose(naive.naive_l2_norm(x, eps=0.0), F.normalize(x, dim=-1, eps=0.0), atol=1e-14)
    v = torch.tensor([[3.0, 4.0]], dtype=torch.float64)
    assert torch.allclose(naive.naive_l2_norm(v, eps=0.0), torch.tensor([[0.6, 0.8]], dtype=torch.float64))
    assert torch.allclose(naive.naive_l2_norm(v, eps=11.0), v / 6.0)                 # sqrt(25 + 11) = 6
    assert torch.equal(naive.naive_l2_norm(torch.zeros(2, 4)), torch.zeros(2, 4, dtype=torch.float64))
    big = x * 1e3
    assert torch.allclose(naive.naive_l2_norm(big), naive.naive_l2_norm(2.5 * big), atol=1e-9)
    xr = x.clone().requires_grad_(True)
    dy = rnd(7002, 5, 3, 16).double()
    (naive.naive_l2_norm(xr, eps=1e-6) * dy).sum().backward()
    var = (x * x).sum(-1, keepdim=True)
    rstd = 1.0 / torch.sqrt(var + 1e-6)
    want = dy * rstd - (dy * x).sum(-1, keepdim=True) * (1.0 / (var + 1e-6)) * rstd * x
    assert torch.allclose(xr.grad, want, atol=1e-12)


def test_rms_norm_pins():
    """naive_rms_norm: torch's own rms_norm and F.silu (independent library routines), hand-computed
    values that place eps inside the square root and use the mean (not the sum) of squares, and the
    backward formulas of the reference kernel (layernorm.py:266-286: wdy = w dy, c1 = mean(x^ wdy),
    dx = (wdy - x^ c1) rstd, dw = sum dy x^) against autograd through the oracle."""
    import torch.nn.functional as F
    x = rnd(7101, 4, 3, 16).double()
    w = rnd(7102, 16).double()
    gate = rnd(7103, 4, 3, 16).double()
    assert torch.allclose(naive.naive_rms_norm(x, w, None, eps=1e-5), F.rms_norm(x, (16,), w, 1e-5), atol=1e-13)
    assert torch.allclose(naive.naive_rms_norm(x, w, gate, eps=1e-5), F.rms_norm(x, (16,), w, 1e-5) * F.silu(gate), atol=1e-13)
    v = torch.tensor([[3.0, 4.0]], dtype=torch.float64)                      # mean of squares 12.5
    assert torch.allclose(naive.naive_rms_norm(v, eps=0.0), v / 12.5 ** 0.5)
    assert torch.allclose(naive.naive_rms_norm(v, eps=3.5), v / 4.0)          # sqrt(12.5 + 3.5) = 4
    xr, wr = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    dy = rnd(7104, 4, 3, 16).double()
    (naive.naive_rms_norm(xr, wr, None, eps=1e-5) * dy).sum().backward()
    rstd = 1.0 / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-5)
    xhat, wdy = x * rstd, w * dy
    c1 = (xhat * wdy).mean(-1, keepdim=True)
    assert torch.allclose(xr.grad, (wdy - xhat * c1) * rstd, atol=1e-12)
    assert torch.allclose(wr.grad, (dy * xhat).sum((0, 1)), atol=1e-12)


def test_silu_l2_norm_pins():
    import torch.nn.functional as F
    x = rnd(7201, 3, 5, 16).double()
    assert torch.allclose(naive.naive_silu_l2_norm(x, eps=0.0), F.normalize(F.silu(x), dim=-1, eps=0.0), atol=1e-14)
    assert torch.allclose(naive.naive_silu_l2_norm(x, eps=1e-6), naive.naive_l2_norm(F.silu(x), eps=1e-6), atol=1e-15)


def test_mixer_prologue_and_epilogue_layouts_by_hand():
    """Which element goes where: qkv [T, B, H, 3 D] holds q | k | v per head; outputs are [B, T, H, D]; the
    epilogue multiplies o[b, t] with the gate row [t, b].  Checked element by element against the formulas."""
    T, B, H, D = 3, 2, 2, 4
    qkv = torch.arange(T * B * H * 3 * D, dtype=torch.float64).reshape(T, B, H * 3 * D) / 50 - 1.0
    q, k, v = naive.naive_gdn_qkv_prologue(qkv, H, D, eps=1e-6)
    assert q.shape == k.shape == v.shape == (B, T, H, D)
    silu = lambda x: x / (1 + torch.exp(-x))
    for (t, b, h) in [(0, 0, 0), (2, 1, 1), (1, 0, 1)]:
        row = qkv[t, b, h * 3 * D:(h + 1) * 3 * D]
        sq, sk = silu(row[:D]), silu(row[D:2 * D])
        assert torch.allclose(q[b, t, h], sq / torch.sqrt((sq * sq).sum() + 1e-6), atol=1e-14)
        assert torch.allclose(k[b, t, h], sk / torch.sqrt((sk * sk).sum() + 1e-6), atol=1e-14)
        assert torch.allclose(v[b, t, h], silu(row[2 * D:]), atol=1e-14)
    o = torch.randn(B, T, H, D, dtype=torch.float64)
    gate = torch.randn(T, B, H * D, dtype=torch.float64)
    y = naive.naive_swish_gate_relayout(o, gate)
    assert y.shape == (T, B, H * D)
    assert torch.allclose(y[2, 1, D + 1], o[1, 2, 1, 1] * silu(gate[2, 1, D + 1]), atol=1e-14)
    assert torch.allclose(y[0, 1, 3], o[1, 0, 0, 3] * silu(gate[0, 1, 3]), atol=1e-14)


def test_gate_construction_pins():
    """Hand-computed values: softplus(0) = log 2, sigmoid(0) = 1/2, logsigmoid(0) = -log 2; the limits
    softplus(z) -> z and logsigmoid(z) -> z; the clamp; g <= 0 always."""
    import math
    z = torch.zeros(1, 2, dtype=torch.float64)
    A_log = torch.tensor([0.0, math.log(3.0)], dtype=torch.float64)
    g, beta = naive.naive_gdn_gates(z, z, A_log, torch.zeros(2, dtype=torch.float64))
    assert torch.allclose(g, torch.tensor([[-math.log(2.0), -3.0 * math.log(2.0)]], dtype=torch.float64))
    assert torch.allclose(beta, torch.full((1, 2), 0.5, dtype=torch.float64))
    big = torch.full((1, 2), 40.0, dtype=torch.float64)
    g2, _ = naive.naive_gdn_gates(big, z, A_log, torch.ones(2, dtype=torch.float64))
    assert torch.allclose(g2, torch.tensor([[-41.0, -123.0]], dtype=torch.float64))
    assert (naive.naive_gdn_gates(rnd(7301, 5, 2).double(), z, A_log, torch.zeros(2, dtype=torch.float64))[0] <= 0).all()
    x = torch.tensor([0.0, -50.0, 50.0, -1.0], dtype=torch.float64)
    y = naive.naive_gla_gate(x, 16.0)
    assert torch.allclose(y[:3], torch.tensor([-math.log(2.0) / 16, -50.0 / 16, 0.0], dtype=torch.float64), atol=1e-15)
    assert torch.allclose(y[3], torch.tensor(-math.log1p(math.e) / 16, dtype=torch.float64))
    assert torch.equal(naive.naive_gla_gate(x, 16.0, clamp_min=-1.0)[1], torch.tensor(-1.0, dtype=torch.float64))


def test_hgrn2_gate_pins():
    """k + exp(g) = 1 always (k = 1 - G, g = log G); f = 0 gives k = 1/2, g = -log 2; a lower bound of 1 closes
    the gate (k = 0, g = 0) and of 0 changes nothing; G >= lb."""
    import math
    f = rnd(7401, 3, 5, 8).double() * 3
    k, g = naive.naive_hgrn2_gates(f)
    assert torch.allclose(k + g.exp(), torch.ones_like(k), atol=1e-15)
    k0, g0 = naive.naive_hgrn2_gates(torch.zeros(1, 8, dtype=torch.float64))
    assert torch.allclose(k0, torch.full((1, 8), 0.5, dtype=torch.float64)) and torch.allclose(g0, torch.full((1, 8), -math.log(2.0), dtype=torch.float64))
    lb = torch.tensor([0.0, 1.0, 0.25, 0.5, 0.0, 1.0, 0.75, 0.1], dtype=torch.float64)
    kl, gl = naive.naive_hgrn2_gates(f, lb)
    assert torch.allclose(kl + gl.exp(), torch.ones_like(kl), atol=1e-15)
    assert torch.equal(kl[..., 1], torch.zeros_like(kl[..., 1])) and torch.equal(gl[..., 5], torch.zeros_like(gl[..., 5]))
    assert torch.allclose(kl[..., 0], k[..., 0]) and torch.allclose(gl[..., 4], g[..., 4])
    assert (gl.exp() >= lb - 1e-15).all()
    # f -> -inf with lb = 0.25: G -> 0.25
    kk, gg = naive.naive_hgrn2_gates(torch.full((1, 8), -60.0, dtype=torch.float64), lb)
    assert torch.allclose(gg[0, 2], torch.tensor(math.log(0.25), dtype=torch.float64))


def test_feature_map_pins():
    """Kernel identities the maps are built for: Taylor phi(q).phi(k) = 1 + s + s^2/2, s = q.k/sqrt(D); ReBased
    (no norm, gamma = 1) phi(q).phi(k) = (q.k)^2/D.  Feature order against torch.triu_indices, the indexing the
    reference uses (feature_map.py:24-30), and feature counts 1 + D + D(D+1)/2 and D(D+1)/2."""
    D = 16
    q, k = rnd(7501, 2, 3, 7, D).double(), rnd(7502, 2, 3, 7, D).double()
    s = (q * k).sum(-1) / D ** 0.5
    pq, pk = naive.naive_taylor_feature_map(q), naive.naive_taylor_feature_map(k)
    assert pq.shape[-1] == 1 + D + D * (D + 1) // 2 == 153
    assert torch.allclose((pq * pk).sum(-1), 1 + s + s * s / 2, atol=1e-12)
    one = torch.ones(D, dtype=torch.float64)
    rq = naive.naive_rebased_feature_map(q, one, None, normalize=False)
    rk = naive.naive_rebased_feature_map(k, one, None, normalize=False)
    assert rq.shape[-1] == D * (D + 1) // 2 == 136
    assert torch.allclose((rq * rk).sum(-1), (q * k).sum(-1) ** 2 / D, atol=1e-12)
    # order: [diag | off] for ReBased, [1 | x | diag | off] for Taylor, off in triu_indices(D, D, 1) order
    z = torch.einsum("...i,...j->...ij", q, q)
    iu = torch.triu_indices(D, D, 1)
    ar = torch.arange(D)
    assert torch.allclose(rq[..., :D], z[..., ar, ar] * D ** -0.5) and torch.allclose(rq[..., D:], z[..., iu[0], iu[1]] * (2.0 / D) ** 0.5)
    assert torch.allclose(pq[..., 1 + D:1 + 2 * D], z[..., ar, ar] / (2.0 * D) ** 0.5)
    assert torch.allclose(pq[..., 1 + 2 * D:], z[..., iu[0], iu[1]] / D ** 0.5)
    assert torch.allclose(pq[..., 1:1 + D], q / D ** 0.25) and torch.equal(pq[..., 0], torch.ones_like(pq[..., 0]))
    # the norm in front of the ReBased map is torch's layer norm with eps 1e-6
    ga, be = 1 + 0.1 * rnd(7503, D).double(), 0.1 * rnd(7504, D).double()
    ln = F.layer_norm(q, (D,), ga, be, 1e-6)
    assert torch.allclose(naive.naive_rebased_feature_map(q, ga, be), naive.naive_rebased_feature_map(ln, None, None, normalize=False), atol=1e-13)


def test_slice_transitions_compose():
    """Sequence-parallel composition: running slices from the state the transitions of lower slices give equals
    the whole sequence (ungated, scalar and per-channel gates: S_out = decay S_in + M; delta rule: S_out = P S_in
    + M with P the final state of the v = 0 recurrence started from the identity)."""
    B, H, T, K, V = 1, 2, 24, 4, 3
    q, k, v = rnd(7601, B, H, T, K).double(), F.normalize(rnd(7602, B, H, T, K).double(), dim=-1), rnd(7603, B, H, T, V).double()
    g = F.logsigmoid(rnd(7604, B, H, T).double())
    gk = F.logsigmoid(rnd(7605, B, H, T, K).double())
    beta = torch.sigmoid(rnd(7606, B, H, T).double())
    cuts = [0, 5, 16, 24]
    zero = torch.zeros(B, H, K, V, dtype=torch.float64)
    eye = torch.eye(K, dtype=torch.float64).expand(B, H, K, K)
    sl = lambda x, a, b: x[:, :, a:b]
    cases = {
        "scalar": (lambda a, b, h0: naive.naive_recurrent_simple_gla(sl(q, a, b), sl(k, a, b), sl(v, a, b), sl(g, a, b), 1.0, h0, True),
                   lambda a, b: sl(g, a, b).sum(2).exp()[..., None, None]),
        "channel": (lambda a, b, h0: naive.naive_recurrent_gla(sl(q, a, b), sl(k, a, b), sl(v, a, b), sl(gk, a, b), 1.0, h0, True),
                    lambda a, b: sl(gk, a, b).sum(2).exp()[..., None]),
    }
    for name, (run, decay) in cases.items():
        full, _ = run(0, T, zero)
        state, outs = zero, []
        for a, b in zip(cuts[:-1], cuts[1:]):
            outs.append(run(a, b, state)[0])
            state = decay(a, b) * state + run(a, b, zero)[1]
        assert torch.allclose(torch.cat(outs, 2), full, atol=1e-12), name
    rung = lambda a, b, h0, vv: naive.naive_recurrent_gated_delta_rule(sl(q, a, b), sl(k, a, b), vv, sl(g, a, b), sl(beta, a, b), 1.0, h0, True, head_first=True)
    full, _ = rung(0, T, zero, v)
    state, outs = zero, []
    for a, b in zip(cuts[:-1], cuts[1:]):
        outs.append(rung(a, b, state, sl(v, a, b))[0])
        P = rung(a, b, eye, torch.zeros(B, H, b - a, K, dtype=torch.float64))[1]
        state = P @ state + rung(a, b, zero, sl(v, a, b))[1]
    assert torch.allclose(torch.cat(outs, 2), full, atol=1e-12)


def test_mom_routing_pins():
    """oracle/mom.py (transform / reconstruct of mom_linear_attention.py:15-120): hand-written expectations
    for a tiny routing (time order, truncation keeps the LAST tokens, zeros on the LEFT), and the properties
    that a wrong side / index would break: every kept (token, choice) appears exactly once; with weights that
    sum to one, no truncation and the identity in place of the op, reconstruct(transform(x)) = x."""
    from oracle import mom
    x = torch.arange(1.0, 5.0).view(1, 4, 1) * torch.ones(1, 4, 8)             # token t carries the value t + 1
    sel = torch.tensor([[[0], [1], [0], [0]]])
    pad, max_len, kept = mom.transform(x, sel, 2, capacity=1.0)
    assert max_len == 3 and pad.shape == (2, 1, 4, 8)
    assert pad[0, 0, :, 0].tolist() == [0.0, 1.0, 3.0, 4.0]                    # memory 0: tokens 0, 2, 3, right-aligned
    assert pad[1, 0, :, 0].tolist() == [0.0, 0.0, 0.0, 2.0]                    # memory 1: token 1
    pad, max_len, kept = mom.transform(x, sel, 2, capacity=0.5)                # capacity_len 2: token 0 is dropped
    assert max_len == 2 and pad[0, 0, :, 0].tolist() == [3.0, 4.0] and pad[1, 0, :, 0].tolist() == [0.0, 2.0]
    assert kept[0][0] == [(2, 0), (3, 0)] and kept[0][1] == [(1, 0)]
    w = torch.ones(1, 4, 1)
    rec = mom.reconstruct(pad, kept, w)
    assert rec[0, :, 0].tolist() == [0.0, 2.0, 3.0, 4.0]                       # the dropped token gets nothing
    # random routing, topk = 2
    g = torch.Generator().manual_seed(7401)
    B, S, E, topk, D = 2, 23, 4, 2, 8
    scores = torch.rand(B, S, E, generator=g)
    wts, sel = torch.topk(scores, topk, dim=-1)
    wts = wts / wts.sum(-1, keepdim=True)
    xr = torch.randn(B, S, D, generator=g, dtype=torch.float64)
    pad, max_len, kept = mom.transform(xr, sel, E, capacity=1.0)
    seen = sorted((b, t, k) for b in range(B) for e in range(E) for (t, k) in kept[b][e])
    assert seen == sorted((b, t, k) for b in range(B) for t in range(S) for k in range(topk))
    for b in range(B):
        for e in range(E):
            assert kept[b][e] == sorted(kept[b][e]) and all(int(sel[b, t, k]) == e for t, k in kept[b][e])
    assert torch.allclose(mom.reconstruct(pad, kept, wts.double()), xr, atol=1e-12)


def test_fp32_gate_scan_alone_costs_a_third_of_the_fp32_bar_at_strength_3():
    """Why the fp32 GPU tests allow 2.5e-5 instead of 1e-5 for the strongest gates (3 x logsigmoid, |b| up to ~180
    inside a chunk): the cumulative gate of a chunk is an fp32 running sum in the kernels (and in fla).  Here
    everything is exact (fp64 token recurrence) except that sum: the gates are replaced by the differences of their
    fp32 running sums, chunk by chunk.  At strength 3 that alone moves the outputs and dq by 1e-6 .. 1e-5 of their
    size; at strength 0.3 by less than 1e-6."""
    import torch.nn.functional as F
    from tests.util import max_abs_rel

    def rounded_gates(g, chunk=64):
        B, T, H = g.shape
        out = torch.empty(B, T, H, dtype=torch.float64)
        for c0 in range(0, T, chunk):
            gc = g[:, c0:c0 + chunk].float()
            b32 = torch.zeros(B, H, dtype=torch.float32)
            prev = torch.zeros(B, H, dtype=torch.float64)
            for i in range(gc.shape[1]):
                b32 = b32 + gc[:, i]
                out[:, c0 + i] = b32.double() - prev
                prev = b32.double()
        return out

    def worst(strength):
        w = 0.0
        for seed in range(3):
            gen_ = torch.Generator().manual_seed(seed)
            B, T, H, K, V = 2, 257, 2, 64, 64
            rn = lambda *s: torch.randn(*s, generator=gen_, dtype=torch.float64)
            q, k, v, do = rn(B, T, H, K), F.normalize(rn(B, T, H, K), dim=-1), rn(B, T, H, V), rn(B, T, H, V)
            g = (F.logsigmoid(torch.randn(B, T, H, generator=gen_)) * strength).float().double()

            def run(gg):
                ql = q.clone().requires_grad_(True)
                o, _ = naive.naive_recurrent_simple_gla(ql, k, v, gg, None, None, False, None, False)
                (dq,) = torch.autograd.grad((o * do).sum(), [ql])
                return o.detach(), dq
            (o0, dq0), (o1, dq1) = run(g), run(rounded_gates(g))
            w = max(w, max_abs_rel(o1, o0), max_abs_rel(dq1, dq0))
        return w

    strong, weak = worst(3.0), worst(0.3)
    assert 1e-6 < strong < 1e-5, strong
    assert weak < 1e-6, weak
