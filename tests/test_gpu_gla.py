"""GPU parity of chunk_gla (HIP, through the C ABI) against the token-recurrence oracle."""
import pytest
import torch
import torch.nn.functional as F

from oracle import naive
from tests.util import TOL, gen, max_abs_rel, oracle_grads

pytestmark = pytest.mark.gpu

CASES = [
    # B, H, T, K, V, h0, head_first, g dtype fp32?, normalizer
    (2, 2, 200, 64, 128, True, True, False, 16.0),     # the reference's gate: logsigmoid / 16
    (1, 2, 130, 128, 128, True, False, True, 1.0),     # HGRN2-style gate: logsigmoid in fp32
    (1, 2, 64, 128, 64, False, True, True, 0.25),      # strong decay (4 * logsigmoid)
    (1, 1, 3, 64, 64, True, True, False, 16.0),
    # decay over 16 tokens far beyond what the diagonal blocks may factor through a reference gate: every
    # diagonal block takes the per-pair path (the case above mixes both, the first two factor all of them)
    (1, 2, 130, 64, 128, True, True, True, 0.1),
]


def gla_inputs(seed, B, H, T, K, V, dtype, head_first, g_fp32, normalizer):
    shp = (B, H, T) if head_first else (B, T, H)
    q, k, v = gen(seed, *shp, K, dtype=dtype), gen(seed + 1, *shp, K, dtype=dtype), gen(seed + 2, *shp, V, dtype=dtype)
    g = F.logsigmoid(gen(seed + 3, *shp, K)) / normalizer
    g = g if (g_fp32 or dtype == torch.float32) else g.to(dtype)
    return q, k, v, g


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", CASES)
def test_gla_fwd_bwd(cuda, dtype, case):
    from linear_moe_amd import chunk_gla
    B, H, T, K, V, use_h0, head_first, g_fp32, normalizer = case
    q, k, v, g = gla_inputs(500, B, H, T, K, V, dtype, head_first, g_fp32, normalizer)
    ins = dict(q=q, k=k, v=v, g=g, h0=gen(514, B, H, K, V) * 0.5 if use_h0 else None)
    shp = (B, H, T) if head_first else (B, T, H)
    do, dht = gen(515, *shp, V, dtype=dtype), gen(516, B, H, K, V)
    fn = lambda q, k, v, g, h0: naive.naive_recurrent_gla(q, k, v, g, None, h0, True, None, head_first)
    ref_o, ref_ht, ref = oracle_grads(fn, ins, do, dht)
    dev = {n: (None if x is None else x.to(cuda).requires_grad_(True)) for n, x in ins.items()}
    o, ht = chunk_gla(dev['q'], dev['k'], dev['v'], dev['g'], None, dev['h0'], True, None, head_first)
    ((o * do.to(cuda)).sum() + (ht * dht.to(cuda)).sum()).backward()
    torch.cuda.synchronize()
    tol = TOL[dtype]
    assert o.dtype == dtype and dev['g'].grad.dtype == g.dtype
    assert max_abs_rel(o.detach().cpu(), ref_o) < tol
    assert max_abs_rel(ht.detach().cpu(), ref_ht) < tol
    for n, r in ref.items():
        err = max_abs_rel(dev[n].grad.cpu(), r)
        assert err < tol, (n, err)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gla_varlen(cuda, dtype):
    from linear_moe_amd import chunk_gla
    cu = torch.tensor([0, 1, 65, 200, 270], dtype=torch.int32)
    T, H, K, V, N = 270, 2, 64, 128, 4
    q, k, v, g = gla_inputs(600, 1, H, T, K, V, dtype, False, True, 16.0)
    ins = dict(q=q, k=k, v=v, g=g, h0=gen(614, N, H, K, V) * 0.5)
    do, dht = gen(615, 1, T, H, V, dtype=dtype), gen(616, N, H, K, V)
    fn = lambda q, k, v, g, h0: naive.naive_recurrent_gla(q, k, v, g, None, h0, True, cu, False)
    ref_o, ref_ht, ref = oracle_grads(fn, ins, do, dht)
    dev = {n: x.to(cuda).requires_grad_(True) for n, x in ins.items()}
    o, ht = chunk_gla(dev['q'], dev['k'], dev['v'], dev['g'], None, dev['h0'], True, cu.to(cuda), False)
    ((o * do.to(cuda)).sum() + (ht * dht.to(cuda)).sum()).backward()
    torch.cuda.synchronize()
    tol = TOL[dtype]
    assert max_abs_rel(o.detach().cpu(), ref_o) < tol
    assert max_abs_rel(ht.detach().cpu(), ref_ht) < tol
    for n, r in ref.items():
        err = max_abs_rel(dev[n].grad.cpu(), r)
        assert err < tol, (n, err)


def test_gla_results_do_not_depend_on_the_width_of_the_v_slices(cuda):
    """The state passes take 64-wide V slices when there are enough (sequence, head) pairs to fill the chip with them
    and 32-wide ones otherwise: a batch of 64 copies of a problem (wide) gives, row for row, the bits of the problem
    alone (narrow)."""
    from linear_moe_amd import chunk_gla
    B, H, T, K, V = 1, 4, 200, 64, 128
    q, k, v = gen(40, B, T, H, K).bfloat16(), gen(41, B, T, H, K).bfloat16(), gen(42, B, T, H, V).bfloat16()
    g = (F.logsigmoid(gen(43, B, T, H, K)) / 4).bfloat16()
    h0, do, dht = gen(44, B, H, K, V) * 0.5, gen(45, B, T, H, V).bfloat16(), gen(46, B, H, K, V)

    def run(rep):
        ins = [x.to(cuda).repeat(rep, *([1] * (x.dim() - 1))).requires_grad_(True) for x in (q, k, v, g, h0)]
        o, ht = chunk_gla(ins[0], ins[1], ins[2], ins[3], None, ins[4], True, None, False)
        grads = torch.autograd.grad([o, ht], ins, [do.to(cuda).repeat(rep, 1, 1, 1), dht.to(cuda).repeat(rep, 1, 1, 1)])
        return [o, ht] + list(grads)

    one, many = run(1), run(64)
    torch.cuda.synchronize()
    for a, b in zip(one, many):
        assert torch.equal(a[0], b[0]) and torch.equal(a[0], b[63])


@pytest.mark.parametrize("B,H,T,K,V,varlen,gdt", [(2, 3, 200, 128, 128, False, torch.float32),
                                                  (1, 4, 64, 64, 64, False, torch.bfloat16),
                                                  (2, 2, 130, 64, 128, False, torch.bfloat16),
                                                  (1, 2, 333, 128, 64, False, torch.float32),
                                                  (1, 4, 700, 64, 128, True, torch.bfloat16)])
def test_gla_dv_of_the_fused_backward_kernel_equals_the_kernel_of_its_own(cuda, B, H, T, K, V, varlen, gdt):
    """With 2-byte elements dv is formed by the kernel that forms dq, dk and dg, from the do and dS' slices it stages
    anyway; the chunk-parallel dv kernel (what the fp32 path runs, still reachable as a stage) forms the same products
    in the same order: bit for bit the same dv, partial chunks and packed sequences included."""
    import ctypes as C
    from linear_moe_amd import _lib
    from linear_moe_amd.gla import GLACall
    lib = _lib.load()
    q, k = gen(80, B, T, H, K).bfloat16().to(cuda), gen(81, B, T, H, K).bfloat16().to(cuda)
    v, do = gen(82, B, T, H, V).bfloat16().to(cuda), gen(83, B, T, H, V).bfloat16().to(cuda)
    g = (F.logsigmoid(gen(84, B, T, H, K)) / 16).to(gdt).to(cuda)
    cu = torch.tensor([0, 100, 101, 450, 700], device=cuda, dtype=torch.int32) if varlen else None
    N = 4 if varlen else B
    h0, dht = (gen(85, N, H, K, V) * 0.3).to(cuda), gen(86, N, H, K, V).to(cuda)
    call = GLACall(keep=True)
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


@pytest.mark.parametrize("B,H,T,K,V,varlen", [(2, 3, 200, 64, 128, False), (1, 4, 64, 64, 64, False),
                                              (64, 4, 130, 64, 128, False), (1, 4, 700, 64, 128, True),
                                              (2, 3, 200, 128, 128, False), (1, 2, 333, 128, 64, False),
                                              (1, 4, 700, 128, 128, True)])
def test_gla_output_of_the_fused_forward_pass_equals_the_output_kernel(cuda, B, H, T, K, V, varlen):
    """With 2-byte elements the forward state pass forms the output as well (three teams, one barrier per chunk, the
    state never read back); the chunk-parallel output kernel (what the fp32 path runs, still reachable as a stage)
    forms the same products in the same order from the per-chunk states the pass has saved: bit for bit the same o —
    narrow and wide V slices (the batch of 64), partial chunks, packed sequences."""
    import ctypes as C
    from linear_moe_amd import _lib
    from linear_moe_amd.gla import GLACall
    lib = _lib.load()
    q, k = gen(90, B, T, H, K).bfloat16().to(cuda), gen(91, B, T, H, K).bfloat16().to(cuda)
    v = gen(92, B, T, H, V).bfloat16().to(cuda)
    g = (F.logsigmoid(gen(93, B, T, H, K)) / 16).bfloat16().to(cuda)
    cu = torch.tensor([0, 100, 101, 450, 700], device=cuda, dtype=torch.int32) if varlen else None
    N = 4 if varlen else B
    h0 = (gen(94, N, H, K, V) * 0.3).to(cuda)
    call = GLACall(keep=True)
    o, ht = call.forward(q, k, v, g, None, h0, True, cu, False)
    torch.cuda.synchronize()
    fused = o.clone()
    assert fused.abs().max() > 0
    o.zero_()
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    _lib.check(lib.lmoe_launch_stage(C.byref(call.fwd_args), call.OP, 2, st), "output stage")   # 2: the output kernel
    torch.cuda.synchronize()
    assert torch.equal(fused, o)


def test_gla_forward_only_call_equals_the_saving_call(cuda):
    """Nothing requires a gradient: the per-chunk states are neither allocated nor written (bf16: the state pass forms
    the output itself); the output and the final state are those of the call that saves them."""
    from linear_moe_amd import chunk_gla
    B, H, T, K, V = 2, 4, 300, 64, 128
    q, k = gen(95, B, T, H, K).bfloat16().to(cuda), gen(96, B, T, H, K).bfloat16().to(cuda)
    v = gen(97, B, T, H, V).bfloat16().to(cuda)
    g = (F.logsigmoid(gen(98, B, T, H, K)) / 16).bfloat16().to(cuda)
    h0 = (gen(99, B, H, K, V) * 0.3).to(cuda)
    with torch.no_grad():
        o1, ht1 = chunk_gla(q, k, v, g, None, h0, True, None, False)
    o2, ht2 = chunk_gla(q.clone().requires_grad_(True), k, v, g, None, h0, True, None, False)
    torch.cuda.synchronize()
    assert torch.equal(o1, o2.detach()) and torch.equal(ht1, ht2.detach())
