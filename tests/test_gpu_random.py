"""GPU parity on randomly drawn problems (fixed seeds): op, dtype, head dims, layout, packed lengths incl. empty
and one-token sequences, initial / final state, gate dtype and gate strength are drawn per trial and the HIP
result (outputs and every gradient, through the C ABI) is compared with the fp64 token recurrence."""
import random

import pytest
import torch
import torch.nn.functional as F

from oracle import naive

pytestmark = pytest.mark.gpu


def _rel(x, r, floor=0.0):
    return float((x.double() - r.double()).abs().max() / max(float(r.double().abs().max()), floor, 1e-30))


def _trial(seed, trial, cuda):
    import linear_moe_amd as L
    rnd = random.Random(seed * 1000 + trial)
    g_ = torch.Generator().manual_seed(seed * 100000 + trial)
    gen = lambda *s: torch.randn(*s, generator=g_)
    op = rnd.choice(['sgla', 'sgla_nog', 'gla', 'gdn', 'delta'])
    dtype = rnd.choice([torch.float32, torch.bfloat16])
    K, V, H = rnd.choice([64, 128]), rnd.choice([64, 128]), rnd.choice([1, 2, 3])
    varlen = rnd.random() < 0.4
    hf = (not varlen) and rnd.random() < 0.5
    use_h0, want_ht = rnd.random() < 0.6, rnd.random() < 0.7
    if varlen:
        N = rnd.randint(1, 4)
        lens = [rnd.choice([0, 1, 5, 63, 64, 65, 100, 130, 200]) for _ in range(N)]
        if sum(lens) == 0:
            lens[0] = 7
        T, B = sum(lens), 1
        cu = torch.tensor([0] + [int(x) for x in torch.tensor(lens).cumsum(0)], dtype=torch.int32)
    else:
        N = B = rnd.choice([1, 2])
        T = rnd.choice([1, 2, 17, 64, 65, 127, 128, 129, 191, 257])
        cu, lens = None, None
    shp = (B, H, T) if hf else (B, T, H)
    q, k, v = gen(*shp, K), F.normalize(gen(*shp, K), dim=-1), gen(*shp, V)
    strength = rnd.choice([0.05, 0.3, 1.0, 3.0])
    g = F.logsigmoid(gen(*shp, K) if op == 'gla' else gen(*shp)) * strength
    beta = torch.sigmoid(gen(*shp))
    h0 = gen(N, H, K, V) * 0.5 if use_h0 else None
    do, dht = gen(*shp, V), gen(N, H, K, V)
    gdt = torch.float32 if (dtype == torch.float32 or rnd.random() < 0.5) else torch.bfloat16
    ins = dict(q=q.to(dtype), k=k.to(dtype), v=v.to(dtype))
    if op in ('sgla', 'gdn'):
        ins['g'] = g
    if op == 'gla':
        ins['g'] = g.to(gdt)
    if op in ('gdn', 'delta'):
        ins['beta'] = beta.to(dtype)
    if h0 is not None:
        ins['h0'] = h0

    def run(ours, t):
        h, c = t.get('h0'), (cu if (not ours or cu is None) else cu.to(cuda))
        if op in ('sgla', 'sgla_nog'):
            f = L.chunk_simple_gla if ours else naive.naive_recurrent_simple_gla
            return f(t['q'], t['k'], t['v'], t.get('g'), None, h, want_ht, c, hf)
        if op == 'gla':
            f = L.chunk_gla if ours else naive.naive_recurrent_gla
            return f(t['q'], t['k'], t['v'], t['g'], None, h, want_ht, c, hf)
        if not ours:
            return naive.naive_recurrent_gated_delta_rule(t['q'], t['k'], t['v'], t.get('g'), t['beta'], None, h, want_ht, c, hf)
        if op == 'gdn':
            return L.chunk_gated_delta_rule(t['q'], t['k'], t['v'], t['g'], t['beta'], None, h, want_ht, c, hf)
        return L.chunk_delta_rule(t['q'], t['k'], t['v'], t['beta'], 64, None, h, want_ht, c, hf)

    rl = {n: x.detach().double().requires_grad_(True) for n, x in ins.items()}
    ro, rht = run(False, rl)
    loss = (ro * do.to(dtype).double()).sum() + ((rht * dht.double()).sum() if want_ht else 0)
    rg = torch.autograd.grad(loss, list(rl.values()))
    dl = {n: x.to(cuda).requires_grad_(True) for n, x in ins.items()}
    o, ht = run(True, dl)
    loss = (o * do.to(dtype).to(cuda)).sum() + ((ht * dht.to(cuda)).sum() if want_ht else 0)
    gg = torch.autograd.grad(loss, list(dl.values()))
    torch.cuda.synchronize()
    # fp32 with the strongest gates (3 x logsigmoid: |b| up to ~180 inside a chunk): 2.5e-5 instead of 1e-5.  The
    # cumulative gate of a chunk is an fp32 sum here as in fla; its rounding alone, with everything else exact, costs
    # up to 3e-6 of the outputs and 6e-6 of dg at this strength (tests/test_oracle_pins.py::
    # test_fp32_gate_scan_alone_costs_a_third_of_the_fp32_bar_at_strength_3), and the kernels measure 8e-6 on the
    # outputs and 1.2e-5 on dg over the three ops
    tol = 2e-2 if dtype == torch.bfloat16 else (1e-5 if strength <= 1.0 else 2.5e-5)
    what = f"seed {seed} trial {trial}: op={op} {dtype} K={K} V={V} H={H} T={T} B={B} lens={lens} head_first={hf} " \
           f"h0={use_h0} ht={want_ht} g={gdt} x{strength}"
    assert _rel(o.detach().cpu(), ro.detach()) < tol, what
    if want_ht:
        assert _rel(ht.detach().cpu(), rht.detach()) < tol, what
    grads = dict(zip(rl, zip(gg, rg)))
    for n, (a, b) in grads.items():
        # dg is a difference of terms of the size of q.dq (a sum over the K channels of a token): where it vanishes
        # identically (no state ahead of a one-token sequence) the error is measured against those terms
        floor = float((grads['q'][1] * rl['q'].detach()).sum(-1).abs().max()) if n == 'g' else 0.0
        assert _rel(a.cpu(), b, floor) < tol, (what, n)


@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6])
def test_random_problems(cuda, seed):
    for trial in range(60):
        _trial(seed, trial, cuda)
