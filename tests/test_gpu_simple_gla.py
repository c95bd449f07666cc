"""GPU parity of chunk_simple_gla (HIP, through the C ABI) against the token-recurrence oracle."""
import ctypes as C

import pytest
import torch
import torch.nn.functional as F

from oracle import naive
from tests.util import TOL, gen, max_abs_rel

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kd", [64, 128])
def test_toolkit_selftest(cuda, dtype, kd):
    from linear_moe_amd import _lib
    lib = _lib.load()
    A = gen(1, 64, kd, dtype=dtype).to(cuda)
    B = gen(2, 64, kd, dtype=dtype).to(cuda)
    Cm = torch.empty(64, 64, device=cuda)
    Ct = torch.empty(kd, kd, device=cuda)
    rc = lib.lmoe_selftest_gemm(_lib.LMOE_F32 if dtype == torch.float32 else _lib.LMOE_BF16, kd,
                                A.data_ptr(), B.data_ptr(), Cm.data_ptr(), Ct.data_ptr(),
                                C.c_void_p(torch.cuda.current_stream().cuda_stream))
    _lib.check(rc, "selftest")
    torch.cuda.synchronize()
    assert max_abs_rel(Cm, A.double() @ B.double().T) < 1e-5
    assert max_abs_rel(Ct, A.double().T @ B.double()) < 1e-5


CASES = [
    # B, H, T, K, V, gate, h0, head_first
    (1, 4, 512, 64, 64, False, False, True),      # contract config 1 (basic linear attention)
    (2, 3, 200, 128, 128, True, True, True),      # T not a multiple of 64, state in/out
    (2, 2, 130, 64, 128, True, True, False),
    (1, 2, 64, 128, 64, True, False, False),
    (1, 1, 1, 64, 64, True, True, True),          # single token
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", CASES)
def test_simple_gla_fwd(cuda, dtype, case):
    from linear_moe_amd import chunk_simple_gla
    B, H, T, K, V, gate, use_h0, head_first = case
    shp = (B, H, T) if head_first else (B, T, H)
    q, k = gen(10, *shp, K, dtype=dtype), gen(11, *shp, K, dtype=dtype)
    v = gen(12, *shp, V, dtype=dtype)
    g = torch.nn.functional.logsigmoid(gen(13, *shp)) if gate else None
    h0 = gen(14, B, H, K, V) * 0.5 if use_h0 else None
    ref_o, ref_ht = naive.naive_recurrent_simple_gla(q, k, v, g, None, h0, True, None, head_first)
    o, ht = chunk_simple_gla(q.to(cuda), k.to(cuda), v.to(cuda), None if g is None else g.to(cuda),
                             None, None if h0 is None else h0.to(cuda), True, None, head_first)
    torch.cuda.synchronize()
    assert o.dtype == dtype and o.shape == v.shape and ht.dtype == torch.float32
    tol = TOL[dtype]
    assert max_abs_rel(o.cpu(), ref_o) < tol
    assert max_abs_rel(ht.cpu(), ref_ht) < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_simple_gla_fwd_varlen(cuda, dtype):
    from linear_moe_amd import chunk_simple_gla
    lens = [1, 64, 135, 70]
    cu = torch.tensor([0, 1, 65, 200, 270], dtype=torch.int32)
    T, H, K, V = sum(lens), 2, 64, 128
    q, k, v = gen(20, 1, T, H, K, dtype=dtype), gen(21, 1, T, H, K, dtype=dtype), gen(22, 1, T, H, V, dtype=dtype)
    g = torch.nn.functional.logsigmoid(gen(23, 1, T, H))
    h0 = gen(24, len(lens), H, K, V) * 0.5
    ref_o, ref_ht = naive.naive_recurrent_simple_gla(q, k, v, g, None, h0, True, cu, False)
    o, ht = chunk_simple_gla(q.to(cuda), k.to(cuda), v.to(cuda), g.to(cuda), None, h0.to(cuda), True,
                             cu.to(cuda), False)
    torch.cuda.synchronize()
    tol = TOL[dtype]
    assert max_abs_rel(o.cpu(), ref_o) < tol
    assert max_abs_rel(ht.cpu(), ref_ht) < tol


BWD_CASES = [
    # B, H, T, K, V, gate, h0, head_first
    (2, 3, 200, 128, 128, True, True, True),
    (2, 2, 130, 64, 128, True, True, False),
    (1, 2, 256, 128, 64, False, False, True),
    (1, 1, 3, 64, 64, True, True, True),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", BWD_CASES)
def test_simple_gla_bwd(cuda, dtype, case):
    from linear_moe_amd import chunk_simple_gla
    from tests.util import oracle_grads
    B, H, T, K, V, gate, use_h0, head_first = case
    shp = (B, H, T) if head_first else (B, T, H)
    ins = dict(q=gen(30, *shp, K, dtype=dtype), k=gen(31, *shp, K, dtype=dtype), v=gen(32, *shp, V, dtype=dtype),
               g=torch.nn.functional.logsigmoid(gen(33, *shp)) if gate else None,
               h0=gen(34, B, H, K, V) * 0.5 if use_h0 else None)
    do, dht = gen(35, *shp, V, dtype=dtype), gen(36, B, H, K, V)
    fn = lambda q, k, v, g, h0: naive.naive_recurrent_simple_gla(q, k, v, g, None, h0, True, None, head_first)
    _, _, ref = oracle_grads(fn, ins, do, dht)
    dev = {n: (None if x is None else x.to(cuda).requires_grad_(True)) for n, x in ins.items()}
    o, ht = chunk_simple_gla(dev['q'], dev['k'], dev['v'], dev['g'], None, dev['h0'], True, None, head_first)
    ((o * do.to(cuda)).sum() + (ht * dht.to(cuda)).sum()).backward()
    torch.cuda.synchronize()
    tol = TOL[dtype]
    for n, r in ref.items():
        assert max_abs_rel(dev[n].grad.cpu(), r) < tol, n


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_simple_gla_bwd_varlen(cuda, dtype):
    from linear_moe_amd import chunk_simple_gla
    from tests.util import oracle_grads
    cu = torch.tensor([0, 1, 65, 200, 270], dtype=torch.int32)
    T, H, K, V, N = 270, 2, 64, 128, 4
    ins = dict(q=gen(40, 1, T, H, K, dtype=dtype), k=gen(41, 1, T, H, K, dtype=dtype),
               v=gen(42, 1, T, H, V, dtype=dtype), g=torch.nn.functional.logsigmoid(gen(43, 1, T, H)),
               h0=gen(44, N, H, K, V) * 0.5)
    do, dht = gen(45, 1, T, H, V, dtype=dtype), gen(46, N, H, K, V)
    fn = lambda q, k, v, g, h0: naive.naive_recurrent_simple_gla(q, k, v, g, None, h0, True, cu, False)
    _, _, ref = oracle_grads(fn, ins, do, dht)
    dev = {n: x.to(cuda).requires_grad_(True) for n, x in ins.items()}
    o, ht = chunk_simple_gla(dev['q'], dev['k'], dev['v'], dev['g'], None, dev['h0'], True, cu.to(cuda), False)
    ((o * do.to(cuda)).sum() + (ht * dht.to(cuda)).sum()).backward()
    torch.cuda.synchronize()
    for n, r in ref.items():
        assert max_abs_rel(dev[n].grad.cpu(), r) < TOL[dtype], n


def test_forward_only_call_equals_the_saving_call(cuda):
    """Without anything that requires a gradient the per-chunk states are not written (hs = NULL through the C ABI):
    outputs and final state are bit-identical to those of the call that saves them for a backward."""
    from linear_moe_amd import chunk_simple_gla
    B, H, T, K, V = 2, 3, 300, 128, 64
    q, k, v = (gen(4000 + i, B, H, T, D, dtype=torch.bfloat16).to(cuda) for i, D in enumerate((K, K, V)))
    g = F.logsigmoid(gen(4003, B, H, T)).to(cuda)
    h0 = (gen(4004, B, H, K, V) * 0.5).to(cuda)
    with torch.no_grad():
        o1, ht1 = chunk_simple_gla(q, k, v, g, None, h0, True)
    o2, ht2 = chunk_simple_gla(q.clone().requires_grad_(True), k, v, g, None, h0, True)
    torch.cuda.synchronize()
    assert torch.equal(o1, o2.detach()) and torch.equal(ht1, ht2.detach())


@pytest.mark.parametrize("K", [64, 128])
def test_simple_gla_does_not_depend_on_the_width_of_the_v_slices(cuda, K):
    """Both state passes take 64-wide V slices when there are enough (sequence, head) pairs to fill the chip with them
    and 32-wide ones otherwise: a batch of 64 copies of a problem (wide) gives, row for row, the bits of the problem
    alone (narrow) - outputs, final state and every gradient."""
    from linear_moe_amd import chunk_simple_gla
    B, H, T, V = 1, 4, 200, 128
    q, k, v = gen(50, B, T, H, K).bfloat16(), gen(51, B, T, H, K).bfloat16(), gen(52, B, T, H, V).bfloat16()
    g = torch.nn.functional.logsigmoid(gen(53, B, T, H))
    h0, do, dht = gen(54, B, H, K, V) * 0.5, gen(55, B, T, H, V).bfloat16(), gen(56, B, H, K, V)

    def run(rep):
        ins = [x.to(cuda).repeat(rep, *([1] * (x.dim() - 1))).requires_grad_(True) for x in (q, k, v, g, h0)]
        o, ht = chunk_simple_gla(ins[0], ins[1], ins[2], ins[3], None, ins[4], True, None, False)
        grads = torch.autograd.grad([o, ht], ins, [do.to(cuda).repeat(rep, 1, 1, 1), dht.to(cuda).repeat(rep, 1, 1, 1)])
        return [o, ht] + list(grads)

    one, many = run(1), run(64)
    torch.cuda.synchronize()
    for a, b in zip(one, many):
        assert torch.equal(a[0], b[0]) and torch.equal(a[0], b[63])
    with torch.no_grad():          # the forward-only instance (no per-chunk states written) of the wide pass
        o, ht = chunk_simple_gla(*[x.to(cuda).repeat(64, *([1] * (x.dim() - 1))) for x in (q, k, v, g)], None,
                                 h0.to(cuda).repeat(64, 1, 1, 1), True, None, False)
    assert torch.equal(o[63], one[0][0]) and torch.equal(ht[63], one[1][0])


@pytest.mark.parametrize("B,H,T,K,V,varlen", [(2, 3, 200, 128, 128, False), (1, 4, 64, 64, 64, False),
                                              (2, 2, 130, 64, 128, False), (1, 2, 333, 128, 64, False),
                                              (1, 4, 700, 128, 128, True)])
def test_dv_of_the_fused_backward_kernel_equals_the_kernel_of_its_own(cuda, B, H, T, K, V, varlen):
    """With 2-byte elements dv is formed by the kernel that forms dq and dk, from the tiles that kernel holds anyway,
    as transposed products; the chunk-parallel dv kernel (what the fp32 path runs, still reachable as a stage) forms
    the same sums in the same order: bit for bit the same dv, partial chunks and packed sequences included."""
    from linear_moe_amd import _lib
    from linear_moe_amd.simple_gla import SimpleGLACall
    lib = _lib.load()
    q, k = gen(70, B, T, H, K).bfloat16().to(cuda), gen(71, B, T, H, K).bfloat16().to(cuda)
    v, do = gen(72, B, T, H, V).bfloat16().to(cuda), gen(73, B, T, H, V).bfloat16().to(cuda)
    g = F.logsigmoid(gen(74, B, T, H)).to(cuda)
    cu = torch.tensor([0, 100, 101, 450, 700], device=cuda, dtype=torch.int32) if varlen else None
    N = 4 if varlen else B
    h0, dht = (gen(75, N, H, K, V) * 0.3).to(cuda), gen(76, N, H, K, V).to(cuda)
    call = SimpleGLACall(keep=True)
    call.forward(q, k, v, g, None, h0, True, cu, False)
    dq, dk, dv, dg, dh0 = call.backward(do, dht)
    torch.cuda.synchronize()
    fused = dv.clone()
    assert fused.abs().max() > 0
    dv.zero_()
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    _lib.check(lib.lmoe_launch_stage(C.byref(call.bwd_args), call.OP, 3, st), "dv stage")      # 3: the dv kernel
    torch.cuda.synchronize()
    assert torch.equal(fused, dv)
