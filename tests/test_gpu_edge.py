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


def test_delta_rule_without_tokens_hands_the_state_through(cuda):
    """chunk_delta_rule with T = 0: the final state is the initial state (zeros without one), never uninitialised."""
    from linear_moe_amd import chunk_delta_rule
    B, H, K, V = 2, 2, 64, 128
    q, k, v = (torch.zeros(B, H, 0, D, dtype=torch.bfloat16, device=cuda) for D in (K, K, V))
    beta = torch.zeros(B, H, 0, dtype=torch.bfloat16, device=cuda)
    h0 = (gen(3110, B, H, K, V) * 0.5).to(cuda).requires_grad_(True)
    dht = gen(3111, B, H, K, V).to(cuda)
    o, ht = chunk_delta_rule(q, k, v, beta, 64, None, h0, True)
    assert o.shape == (B, H, 0, V)
    (ht * dht).sum().backward()
    assert torch.equal(ht.detach(), h0.detach()) and torch.equal(h0.grad, dht)
    _, ht = chunk_delta_rule(q, k, v, beta, 64, None, None, True)
    assert torch.equal(ht, torch.zeros(B, H, K, V, device=cuda))


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


@pytest.mark.parametrize("packed", [False, True])
def test_forward_and_backward_can_be_captured_in_a_graph(cuda, packed):
    """The library allocates nothing and launches only on the stream it is given, so a forward + backward of the
    gated delta rule can be captured into a HIP graph; every replay (with eager work between the replays)
    reproduces the eager results bit for bit.  Packed input too: the chunk tables of offsets on the device are built
    on the device, inside the capture."""
    from linear_moe_amd import _host
    from linear_moe_amd.gated_delta_rule import GDNCall
    B, T, H, K, V = (1, 600, 2, 128, 128) if packed else (2, 300, 2, 128, 128)
    dt = torch.bfloat16
    q, k = gen(3200, B, T, H, K, dtype=dt).to(cuda), F.normalize(gen(3201, B, T, H, K), dim=-1).to(dt).to(cuda)
    v, do = gen(3202, B, T, H, V, dtype=dt).to(cuda), gen(3203, B, T, H, V, dtype=dt).to(cuda)
    g, beta = F.logsigmoid(gen(3204, B, T, H)).to(cuda), torch.sigmoid(gen(3205, B, T, H)).to(dt).to(cuda)
    cu = torch.tensor([0, 70, 70, 333, 600], dtype=torch.int32, device=cuda) if packed else None
    N = 4 if packed else B
    h0 = (0.1 * gen(3206, N, H, K, V)).to(cuda) if packed else None
    dht = gen(3207, N, H, K, V).to(cuda) if packed else None
    call = GDNCall(keep=True)

    def step():
        o, ht = call.forward(q, k, v, g, beta, None, h0, packed, cu, False)
        return (o,) + ((ht,) if packed else ()) + tuple(x for x in call.backward(do, dht) if x is not None)

    ref = [x.clone() for x in step()]
    if packed:                                          # the plan is cached now: no call below builds one
        n_plans = len(_host._PLAN_CACHE)
        assert any(e[0] is cu for e in _host._PLAN_CACHE)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    for _ in range(3):
        for x in outs:
            x.zero_()                                   # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert all(torch.equal(a, b) for a, b in zip(outs, ref))
    if packed:
        assert len(_host._PLAN_CACHE) == n_plans        # a capture neither reads nor fills the cache


@pytest.mark.parametrize("op", OPS)
def test_offsets_on_the_device_give_the_bits_of_offsets_on_the_host(cuda, op):
    """Offsets handed over on the device are never read back: the chunk tables are built there, sized for an upper
    bound of the chunk count, with the true count on the device for the kernels.  Same call with the offsets as a host
    tensor (validated, exact tables): the same bits, outputs, states and every gradient."""
    lens = [70, 0, 300, 1, 64, 129]
    T, N, H, K, V = sum(lens), len(lens), 3, 64, 128
    ins = {n: x.to(cuda) for n, x in _inputs(op, T, H, K, V, torch.bfloat16, 3500).items()}
    h0 = (gen(3510, N, H, K, V) * 0.1).to(cuda)
    do, dht = gen(3511, 1, T, H, V, dtype=torch.bfloat16).to(cuda), gen(3512, N, H, K, V).to(cuda)
    cu_host = torch.tensor([0] + lens, dtype=torch.int32).cumsum(0).to(torch.int32)
    names = list(ins)

    def run(cu):
        leaves = {n: x.clone().requires_grad_(True) for n, x in dict(ins, h0=h0).items()}
        o, ht = _call(op, leaves, leaves["h0"], cu, True)
        grads = torch.autograd.grad([o, ht], [leaves[n] for n in names + ["h0"]], [do, dht])
        return (o.detach(), ht.detach()) + tuple(grads)

    from linear_moe_amd import _host
    on_dev = run(cu_host.to(cuda))
    on_host = run(cu_host)
    torch.cuda.synchronize()
    plan = _host.prepare_cu_seqlens(cu_host.to(cuda), T)
    assert plan.nt_dev is not None and int(plan.nt_dev) == sum((x + 63) // 64 for x in lens) < plan.NT
    for a, b in zip(on_dev, on_host):
        assert torch.equal(a, b)


def test_a_captured_packed_step_follows_the_offsets_it_finds_at_replay(cuda):
    """A forward + backward on packed input captured with its offsets in a static device buffer: the chunk tables are
    part of the graph, so after new offsets (other lengths, another number of chunks) were copied into the buffer a
    replay gives what an eager call on those offsets gives, bit for bit."""
    from linear_moe_amd.gated_delta_rule import GDNCall
    T, H, K, V, dt = 640, 2, 128, 128, torch.bfloat16
    q, k = gen(3600, 1, T, H, K, dtype=dt).to(cuda), F.normalize(gen(3601, 1, T, H, K), dim=-1).to(dt).to(cuda)
    v, do = gen(3602, 1, T, H, V, dtype=dt).to(cuda), gen(3603, 1, T, H, V, dtype=dt).to(cuda)
    g, beta = F.logsigmoid(gen(3604, 1, T, H)).to(cuda), torch.sigmoid(gen(3605, 1, T, H)).to(dt).to(cuda)
    offsets = [[0, 70, 70, 333, 640], [0, 1, 200, 639, 640], [0, 128, 256, 384, 640]]      # 11, 12 and 10 chunks
    h0, dht = (0.1 * gen(3606, 4, H, K, V)).to(cuda), gen(3607, 4, H, K, V).to(cuda)

    def step(call, cu):
        o, ht = call.forward(q, k, v, g, beta, None, h0, True, cu, False)
        return (o, ht) + tuple(x for x in call.backward(do, dht) if x is not None)

    refs = [[x.clone() for x in step(GDNCall(keep=True), torch.tensor(o_, dtype=torch.int32, device=cuda))] for o_ in offsets]
    cu = torch.tensor(offsets[0], dtype=torch.int32, device=cuda)
    call = GDNCall(keep=True)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(call, cu)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step(call, cu)
    for i in (0, 1, 2, 1, 0):
        cu.copy_(torch.tensor(offsets[i], dtype=torch.int32))
        for x in outs:
            x.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for a, b in zip(outs, refs[i]):
            assert torch.equal(a, b), i


@pytest.mark.parametrize("op", OPS)
def test_strided_views_need_no_copy_and_give_the_same(cuda, op):
    """q, k, v as slices of one fused projection output [B, T, H, K + K + V] (row stride larger than the row), the
    head-first call on transposed views of the same memory, and do as a strided view: bit for bit what contiguous
    tensors give (the C ABI takes element strides; nothing is copied for 16-byte aligned rows)."""
    dtype = torch.bfloat16
    B, T, H, K, V = 2, 150, 2, 64, 128
    ins = _inputs(op, T, H, K, V, dtype, 3300)
    ins = {n: (x.expand(B, *x.shape[1:]).clone() if x.shape[0] == 1 else x) for n, x in ins.items()}
    ins = {n: x + 0.01 * torch.arange(B, dtype=x.dtype).view(B, *([1] * (x.dim() - 1))) for n, x in ins.items()}
    fused = torch.cat([ins["q"], ins["k"], ins["v"]], dim=-1).to(cuda)          # [B, T, H, 2K + V]
    views = dict(q=fused[..., :K], k=fused[..., K:2 * K], v=fused[..., 2 * K:])
    assert not views["q"].is_contiguous()
    do_wide = gen(3310, B, T, H, 2 * V, dtype=dtype).to(cuda)
    do = do_wide[..., V:]

    def run(q, k, v, do, head_first):
        t = dict(ins)
        leaves = dict(q=q.detach().requires_grad_(True), k=k.detach().requires_grad_(True), v=v.detach().requires_grad_(True))
        for n in ("g", "beta"):
            if n in t:
                x = t[n].to(cuda)
                leaves[n] = (x.transpose(1, 2) if head_first else x).detach().requires_grad_(True)
        from linear_moe_amd import chunk_gated_delta_rule, chunk_gla, chunk_simple_gla
        if op == "simple_gla":
            o, _ = chunk_simple_gla(leaves["q"], leaves["k"], leaves["v"], leaves["g"], None, None, False, None, head_first)
        elif op == "gla":
            o, _ = chunk_gla(leaves["q"], leaves["k"], leaves["v"], leaves["g"], None, None, False, None, head_first)
        else:
            o, _ = chunk_gated_delta_rule(leaves["q"], leaves["k"], leaves["v"], leaves["g"], leaves["beta"], None, None,
                                          False, None, head_first)
        grads = torch.autograd.grad(o, [leaves["q"], leaves["k"], leaves["v"]], do)
        return [o.detach()] + list(grads)

    ref = run(views["q"].contiguous(), views["k"].contiguous(), views["v"].contiguous(), do.contiguous(), False)
    got = run(views["q"], views["k"], views["v"], do, False)
    torch.cuda.synchronize()
    for a, b in zip(got, ref):
        assert torch.equal(a, b)
    tr = lambda x: x.transpose(1, 2)                                             # [B, H, T, D] views, not contiguous
    got_hf = run(tr(views["q"]), tr(views["k"]), tr(views["v"]), tr(do), True)
    torch.cuda.synchronize()
    for a, b in zip(got_hf, ref):
        assert torch.equal(tr(a), b)


@pytest.mark.parametrize("op", OPS)
def test_a_sequence_gives_the_same_bits_alone_and_inside_a_large_packed_batch(cuda, op):
    """The sequential passes carry 64 V columns per work-group when sequences x heads alone fill the GPU and 32
    otherwise: a choice of the launch that must not show in the results.  One sequence out of 17 x 16 heads
    (wide slices) against the same sequence as a call of its own (narrow slices), outputs and all gradients."""
    N, Ls, H, K, V = 17, 200, 16, 128, 128
    T = N * Ls
    ins = {n: x.to(cuda) for n, x in _inputs(op, T, H, K, V, torch.bfloat16, 3300).items()}
    h0 = (gen(3310, N, H, K, V) * 0.1).to(cuda)
    do, dht = gen(3311, 1, T, H, V, dtype=torch.bfloat16).to(cuda), gen(3312, N, H, K, V).to(cuda)
    cu = (torch.arange(N + 1, dtype=torch.int32) * Ls).to(cuda)
    names = list(ins)

    def run(ins, h0, cu, do, dht):
        leaves = {n: x.clone().requires_grad_(True) for n, x in dict(ins, h0=h0).items()}
        o, ht = _call(op, leaves, leaves["h0"], cu, True)
        grads = torch.autograd.grad([o, ht], [leaves[n] for n in names + ["h0"]], [do, dht])
        return (o.detach(), ht.detach()) + tuple(grads)

    s = N - 1
    sl = slice(s * Ls, (s + 1) * Ls)
    cut = lambda x: x[:, sl].contiguous()
    alone = run({n: cut(x) for n, x in ins.items()}, h0[s:s + 1].contiguous(), None, cut(do), dht[s:s + 1].contiguous())
    packed = run(ins, h0, cu, do, dht)
    torch.cuda.synchronize()
    per_seq = (1, len(packed) - 1)                     # ht and dh0 are per sequence, the rest per token
    labels = ["o", "ht"] + ["d" + n for n in names] + ["dh0"]
    for i, (a, b) in enumerate(zip(packed, alone)):
        a = a[s:s + 1] if i in per_seq else a[:, sl]
        assert torch.equal(a, b), labels[i]


@pytest.mark.parametrize("op", OPS)
def test_the_order_in_which_the_passes_take_the_sequences_does_not_show(cuda, op):
    """The plan of a packed batch of unequal lengths lists the sequences longest first and the sequential passes take
    them in that order (their work-groups are dispatched by index): which work-group computes a sequence must not
    change what it computes.  Same call with the order as planned and with the order taken away: the same bits."""
    from linear_moe_amd import _host
    lens = [70, 300, 1, 64, 129, 500, 33]
    T, N, H, K, V = sum(lens), len(lens), 5, 64, 128
    ins = {n: x.to(cuda) for n, x in _inputs(op, T, H, K, V, torch.bfloat16, 3400).items()}
    h0 = (gen(3410, N, H, K, V) * 0.1).to(cuda)
    do, dht = gen(3411, 1, T, H, V, dtype=torch.bfloat16).to(cuda), gen(3412, N, H, K, V).to(cuda)
    cu = torch.tensor([0] + lens, dtype=torch.int32).cumsum(0).to(torch.int32).to(cuda)
    names = list(ins)

    def run():
        leaves = {n: x.clone().requires_grad_(True) for n, x in dict(ins, h0=h0).items()}
        o, ht = _call(op, leaves, leaves["h0"], cu, True)
        grads = torch.autograd.grad([o, ht], [leaves[n] for n in names + ["h0"]], [do, dht])
        return (o.detach(), ht.detach()) + tuple(grads)

    plan = _host.prepare_cu_seqlens(cu, T)
    order = plan.seq_order
    assert order is not None and order.tolist()[:2] == [5, 1]
    try:
        planned = run()
        plan.seq_order = None
        as_given = run()
    finally:
        plan.seq_order = order
    torch.cuda.synchronize()
    for a, b in zip(planned, as_given):
        assert torch.equal(a, b)


@pytest.mark.parametrize("op", OPS)
def test_saved_tensors_belong_to_autograd(cuda, op):
    """What a call keeps for its backward (inputs, per-chunk states, the other intermediates) is handed to autograd:
    it is freed when the node's backward has run, although the output -- and with it the node -- is still alive; an
    input modified in place between forward and backward is an error, not a wrong gradient; a second backward works
    with retain_graph and is refused without."""
    T, H, K, V = 4096, 4, 128, 128
    ins = {n: x.to(cuda) for n, x in _inputs(op, T, H, K, V, torch.bfloat16, 3700).items()}
    do = gen(3711, 1, T, H, V, dtype=torch.bfloat16).to(cuda)
    names = list(ins)

    def forward():
        leaves = {n: x.clone().requires_grad_(True) for n, x in ins.items()}
        work = {n: x * 1 for n, x in leaves.items()}                 # (not leaves: they may be written in place)
        o, _ = _call(op, work, None, None, True)
        return leaves, work, o

    torch.cuda.synchronize()
    m0 = torch.cuda.memory_allocated()
    leaves, work, o = forward()
    m1 = torch.cuda.memory_allocated()
    g1 = torch.autograd.grad(o, [leaves[n] for n in names], do, retain_graph=True)
    g2 = torch.autograd.grad(o, [leaves[n] for n in names], do)
    for a, b in zip(g1, g2):
        assert torch.equal(a, b)
    with pytest.raises(RuntimeError):
        torch.autograd.grad(o, [leaves[n] for n in names], do)       # freed by the backward before
    held = sum(x.numel() * x.element_size() for x in list(leaves.values()) + list(g1) + list(g2)) \
        + o.numel() * o.element_size()
    del work
    torch.cuda.synchronize()
    m2 = torch.cuda.memory_allocated()
    states = (T // 64) * H * K * V * 2                               # the per-chunk states alone
    assert m1 - m0 > held - sum(x.numel() * x.element_size() for x in list(g1) + list(g2)) + states
    assert m2 - m0 <= held + (1 << 20), (m2 - m0, held)

    leaves, work, o = forward()
    work["k"].add_(1)
    with pytest.raises(RuntimeError, match="modified by an inplace operation"):
        torch.autograd.grad(o, [leaves[n] for n in names], do)
