"""GPU parity of the mixture-of-memories routing (pack / combine through the C ABI) against the CPU
restatement of the reference's transform / reconstruct, and equivalence of the packed variable-length
flow with the reference's pad-to-capacity flow around the gated delta rule."""
import pytest
import torch
import torch.nn.functional as F

from oracle import mom, naive
from tests.util import TOL, gen, max_abs_rel

pytestmark = pytest.mark.gpu


def routing(seed, B, S, E, topk):
    g = torch.Generator().manual_seed(seed)
    wts, sel = torch.topk(torch.softmax(torch.randn(B, S, E, generator=g), -1), topk, dim=-1)
    return wts / wts.sum(-1, keepdim=True), sel


@pytest.mark.parametrize("capacity", [None, 1.0, 0.3])
def test_plan_matches_the_reference_routing(cuda, capacity):
    from linear_moe_amd import mom_plan
    B, S, E, topk = 3, 37, 4, 2
    _, sel = routing(3001, B, S, E, topk)
    plan = mom_plan(sel.to(cuda), E, capacity)
    _, max_len, kept = mom.transform(torch.zeros(B, S, 8), sel, E, float(topk) if capacity is None else capacity)
    assert plan.max_len == max_len
    cu = plan.cu_seqlens.cpu().tolist()
    tok, ch = plan.src_token.cpu().tolist(), plan.src_choice.cpu().tolist()
    for e in range(E):
        assert int(plan.mem_offsets[e]) == cu[e * B]
        for b in range(B):
            seq = e * B + b
            got = [(tok[r] - b * S, ch[r] % topk) for r in range(cu[seq], cu[seq + 1])]
            assert all(tok[r] // S == b for r in range(cu[seq], cu[seq + 1]))
            assert got == kept[b][e]
    row_of = plan.row_of.cpu().view(B, S, topk)
    kept_set = {(b, t, k) for b in range(B) for e in range(E) for (t, k) in kept[b][e]}
    for b in range(B):
        for t in range(S):
            for k in range(topk):
                assert (int(row_of[b, t, k]) >= 0) == ((b, t, k) in kept_set)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("capacity", [None, 0.4])
def test_pack_and_combine_fwd_bwd(cuda, dtype, capacity):
    from linear_moe_amd import mom_combine, mom_pack, mom_plan
    B, S, E, topk, D = 2, 53, 3, 2, 72
    wts, sel = routing(3101, B, S, E, topk)
    plan = mom_plan(sel.to(cuda), E, capacity)
    x = gen(3102, B, S, D, dtype=dtype)
    # pack: rows in memory-major order = the reference's padded tensor without its padding
    pad, max_len, kept = mom.transform(x.double(), sel, E, float(topk) if capacity is None else capacity)
    want_rows = torch.cat([pad[e, b, pad.shape[2] - len(kept[b][e]):] for e in range(E) for b in range(B)], 0)
    xd = x.to(cuda).requires_grad_(True)
    xp = mom_pack(xd, plan)
    assert xp.shape == (plan.T_total, D) and torch.equal(xp.detach().cpu().double(), want_rows)
    dxp = gen(3103, plan.T_total, D, dtype=dtype)
    (xp * dxp.to(cuda)).sum().backward()
    ref_dx = torch.zeros(B * S, D, dtype=torch.float64)
    ref_dx.index_add_(0, plan.src_token.cpu().long(), dxp.double())
    assert max_abs_rel(xd.grad.cpu().view(B * S, D), ref_dx) < TOL[dtype]
    # combine against reconstruct: y rows -> right-aligned padded [E, B, L, D]
    y = gen(3104, plan.T_total, D, dtype=dtype)
    L = max(max_len, 1)
    cu = plan.cu_seqlens.cpu().tolist()
    yr = y.double().requires_grad_(True)
    wr = wts.double().requires_grad_(True)
    ypad = torch.zeros(E, B, L, D, dtype=torch.float64)
    pieces = {}
    for e in range(E):
        for b in range(B):
            n = cu[e * B + b + 1] - cu[e * B + b]
            pieces[(e, b)] = n
    ypad = torch.stack([torch.stack([torch.cat([torch.zeros(L - pieces[(e, b)], D, dtype=torch.float64),
                                                yr[cu[e * B + b]:cu[e * B + b + 1]]], 0) for b in range(B)], 0)
                        for e in range(E)], 0)
    ref = mom.reconstruct(ypad, kept, wr)
    dout = gen(3105, B, S, D, dtype=dtype)
    (ref * dout.double()).sum().backward()
    yd, wd = y.to(cuda).requires_grad_(True), wts.to(dtype).to(cuda).requires_grad_(True)
    out = mom_combine(yd, plan, wd)
    (out * dout.to(cuda)).sum().backward()
    torch.cuda.synchronize()
    assert max_abs_rel(out.detach().cpu(), ref.detach()) < TOL[dtype]
    assert max_abs_rel(yd.grad.cpu(), yr.grad) < TOL[dtype]
    assert max_abs_rel(wd.grad.cpu(), wr.grad) < TOL[dtype]


@pytest.mark.parametrize("capacity", [1.0, 0.5])
def test_packed_flow_equals_the_padded_flow_around_the_gated_delta_rule(cuda, capacity):
    """Reference flow: transform -> op per memory on the padded [B, capacity_len] batch -> reconstruct.
    Packed flow: mom_pack -> ONE cu_seqlens call -> mom_combine.  Left padding (zero q, k, v) leaves the
    state untouched whatever its gate is, so both compute the same function."""
    from linear_moe_amd import chunk_gated_delta_rule, mom_combine, mom_pack, mom_plan
    B, S, E, topk, H, K, V = 2, 150, 3, 2, 2, 64, 64
    wts, sel = routing(3201, B, S, E, topk)
    # per-token inputs of the op as functions of the token (stand-ins for the per-memory projections)
    q = F.normalize(gen(3202, B, S, H * K).view(B, S, H, K), dim=-1).reshape(B, S, H * K)
    k = F.normalize(gen(3203, B, S, H * K).view(B, S, H, K), dim=-1).reshape(B, S, H * K)
    v = gen(3204, B, S, H * V)
    g = -F.softplus(gen(3205, B, S, H)) * 0.3
    beta = torch.sigmoid(gen(3206, B, S, H))
    gb = torch.cat([g, beta, torch.zeros(B, S, 8 - 2 * H)], -1)           # rows of 8 for the routing kernels
    # reference flow on the CPU (fp64)
    outs = []
    kept = None
    padded = {}
    for name, t in dict(q=q, k=k, v=v, gb=gb).items():
        padded[name], max_len, kept = mom.transform(t.double(), sel, E, capacity)
    L = padded["q"].shape[2]
    ys = []
    for e in range(E):
        qe, ke = padded["q"][e].view(B, L, H, K), padded["k"][e].view(B, L, H, K)
        ve = padded["v"][e].view(B, L, H, V)
        ge, be = padded["gb"][e][..., :H].clone(), padded["gb"][e][..., H:2 * H].clone()
        lens = torch.tensor([[len(kept[b][e])] for b in range(B)])
        is_pad = torch.arange(L).view(1, L) < (L - lens)
        ge[is_pad] = -1.0                                                  # any gate on a padded position
        be[is_pad] = 0.5
        oe, _ = naive.naive_recurrent_gated_delta_rule(qe, ke, ve, ge, be, None, None, False, None, False)
        ys.append(oe.reshape(B, L, H * V))
    ref = mom.reconstruct(torch.stack(ys, 0), kept, wts.double())
    # packed flow on the GPU (fp32)
    plan = mom_plan(sel.to(cuda), E, capacity)
    d = lambda t: t.to(cuda)
    qp, kp, vp, gbp = (mom_pack(d(t), plan) for t in (q, k, v, gb))
    T = plan.T_total
    o, _ = chunk_gated_delta_rule(qp.view(1, T, H, K), kp.view(1, T, H, K), vp.view(1, T, H, V),
                                  gbp[:, :H].contiguous().view(1, T, H), gbp[:, H:2 * H].contiguous().view(1, T, H),
                                  cu_seqlens=plan.cu_seqlens)
    out = mom_combine(o.reshape(T, H * V), plan, d(wts))
    torch.cuda.synchronize()
    assert out.shape == (B, S, H * V)
    assert max_abs_rel(out.cpu(), ref) < 1e-5


def test_routing_to_result_captures_into_a_graph_and_follows_new_routing_at_replay(cuda):
    """Without a capacity nothing of the routing is read on the host: plan, pack, the packed op and combine are
    device work only, so the whole path from the selected memories to the mixed result captures into a HIP graph, and
    a replay after other routing was copied into the captured buffers gives what an eager run on that routing gives."""
    from linear_moe_amd import chunk_gated_delta_rule, mom_combine, mom_pack, mom_plan
    B, S, E, topk, H, K, V = 2, 150, 3, 2, 2, 64, 64
    d = lambda t: t.to(cuda)
    q = d(F.normalize(gen(3302, B, S, H * K).view(B, S, H, K), dim=-1).reshape(B, S, H * K))
    k = d(F.normalize(gen(3303, B, S, H * K).view(B, S, H, K), dim=-1).reshape(B, S, H * K))
    v = d(gen(3304, B, S, H * V))
    gb = d(torch.cat([-F.softplus(gen(3305, B, S, H)) * 0.3, torch.sigmoid(gen(3306, B, S, H)), torch.zeros(B, S, 8 - 2 * H)], -1))
    routings = [routing(3310 + i, B, S, E, topk) for i in range(3)]
    sel, wts = d(routings[0][1]).clone(), d(routings[0][0]).clone()

    def run(sel, wts):
        plan = mom_plan(sel, E)
        T = plan.T_total
        assert T == B * S * topk
        qp, kp, vp, gbp = (mom_pack(t, plan) for t in (q, k, v, gb))
        o, _ = chunk_gated_delta_rule(qp.view(1, T, H, K), kp.view(1, T, H, K), vp.view(1, T, H, V),
                                      gbp[:, :H].contiguous().view(1, T, H), gbp[:, H:2 * H].contiguous().view(1, T, H),
                                      cu_seqlens=plan.cu_seqlens)
        return mom_combine(o.reshape(T, H * V), plan, wts)

    refs = [run(d(s_), d(w_)).clone() for (w_, s_) in routings]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run(sel, wts)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = run(sel, wts)
    for i in (0, 1, 2, 0):
        sel.copy_(d(routings[i][1]))
        wts.copy_(d(routings[i][0]))
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, refs[i]), i
