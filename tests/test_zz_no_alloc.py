"""The allocation-free backward of the RMS norm (lmoe_rmsnorm_bwd_noalloc: partial rows of dw in a scratch array the
library holds in static device memory) against lmoe_rmsnorm_bwd with a caller-allocated workspace, through the C ABI:
the same kernels on the same grid, so dx, dgate and dw must agree bit for bit -- on two calls in a row, the second
with a smaller input (its partial rows are a prefix of what the first call left in the shared array)."""
import ctypes as C

import pytest
import torch

from tests.util import gen

pytestmark = pytest.mark.gpu


def _both(lib, _lib, cuda, rows, D, dtype, with_gate, seed):
    dt = _lib.LMOE_F32 if dtype == torch.float32 else _lib.LMOE_BF16
    x, dy = gen(seed, rows, D, dtype=dtype).to(cuda), gen(seed + 1, rows, D, dtype=dtype).to(cuda)
    w = (1 + 0.1 * gen(seed + 2, D)).to(dtype).to(cuda)
    gate = gen(seed + 3, rows, D, dtype=dtype).to(cuda) if with_gate else None
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    p = lambda t: None if t is None else t.data_ptr()
    nparts = lib.lmoe_rmsnorm_partials(rows, D, dt)
    assert nparts > 0
    part = torch.empty(nparts, D, dtype=torch.float32, device=cuda)
    out = []
    for noalloc in (False, True):
        dx = torch.full_like(x, float("nan"))
        dgate = torch.full_like(x, float("nan")) if with_gate else None
        dw = torch.full((D,), float("nan"), dtype=torch.float32, device=cuda)
        if noalloc:
            rc = lib.lmoe_rmsnorm_bwd_noalloc(p(x), p(w), p(gate), p(dy), p(dx), p(dgate), p(dw), rows, D, dt, 1e-5, st)
        else:
            rc = lib.lmoe_rmsnorm_bwd(p(x), p(w), p(gate), p(dy), p(dx), p(dgate), p(part), p(dw), rows, D, dt, 1e-5, st)
        _lib.check(rc, "rmsnorm backward")
        torch.cuda.synchronize()
        out.append((dx, dgate, dw))
    (dx0, dg0, dw0), (dx1, dg1, dw1) = out
    assert torch.isfinite(dw1).all() and torch.isfinite(dx1.float()).all()
    assert torch.equal(dx0, dx1) and torch.equal(dw0, dw1)
    if with_gate:
        assert torch.equal(dg0, dg1)
    # and the numbers are the right ones (fp64 autograd through the formula)
    xr, wr = x.double().cpu().requires_grad_(True), w.double().cpu().requires_grad_(True)
    y = xr * torch.rsqrt((xr * xr).mean(-1, keepdim=True) + 1e-5) * wr
    if with_gate:
        gr = gate.double().cpu()
        y = y * gr * torch.sigmoid(gr)
    y.backward(dy.double().cpu())
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert ((dw1.cpu().double() - wr.grad).abs().max() / wr.grad.abs().max()).item() < tol
    assert ((dx1.cpu().double() - xr.grad).abs().max() / xr.grad.abs().max()).item() < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm_bwd_noalloc_matches_the_workspace_entry_point(cuda, dtype):
    from linear_moe_amd import _lib
    lib = _lib.load()
    # large first (the full grid: every partial row of the scratch is written), then smaller inputs and other widths
    _both(lib, _lib, cuda, 70000, 128, dtype, True, 4100)
    _both(lib, _lib, cuda, 301, 128, dtype, True, 4110)
    _both(lib, _lib, cuda, 5, 256, dtype, False, 4120)
    _both(lib, _lib, cuda, 1000, 64, dtype, False, 4130)


def test_rmsnorm_bwd_noalloc_rejects_bad_arguments(cuda):
    from linear_moe_amd import _lib
    lib = _lib.load()
    x = torch.zeros(4, 128, dtype=torch.bfloat16, device=cuda)
    dw = torch.zeros(128, dtype=torch.float32, device=cuda)
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.lmoe_rmsnorm_bwd_noalloc(x.data_ptr(), None, None, x.data_ptr(), x.data_ptr(), None, None, 4, 128,
                                      _lib.LMOE_BF16, 1e-5, st)
    assert rc < 0 and b"dw" in lib.lmoe_last_error()
    rc = lib.lmoe_rmsnorm_bwd_noalloc(x.data_ptr(), None, None, x.data_ptr(), x.data_ptr(), None, dw.data_ptr(), 4, 96,
                                      _lib.LMOE_BF16, 1e-5, st)
    assert rc < 0


def test_rmsnorm_bwd_noalloc_inside_a_graph_capture(cuda):
    """What the entry point is for: a caller under HIP graph capture.  The address of the scratch array is looked up on
    the first call on a device, which is host work that does not belong into a capture: one eager call (any size)
    resolves it, the captured call then only launches.  Replays, with eager work and another eager call of the entry
    point on a smaller input between them, reproduce the workspace entry point bit for bit."""
    from linear_moe_amd import _lib
    lib = _lib.load()
    rows, D, dt = 3000, 128, _lib.LMOE_BF16
    x, dy, gate = (gen(4200 + i, rows, D, dtype=torch.bfloat16).to(cuda) for i in range(3))
    w = (1 + 0.1 * gen(4203, D)).to(torch.bfloat16).to(cuda)
    p = lambda t: t.data_ptr()
    part = torch.empty(lib.lmoe_rmsnorm_partials(rows, D, dt), D, dtype=torch.float32, device=cuda)
    ref = [torch.empty_like(x), torch.empty_like(x), torch.empty(D, dtype=torch.float32, device=cuda)]
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    _lib.check(lib.lmoe_rmsnorm_bwd(p(x), p(w), p(gate), p(dy), p(ref[0]), p(ref[1]), p(part), p(ref[2]), rows, D, dt, 1e-5, st), "ref")
    out = [torch.empty_like(x), torch.empty_like(x), torch.empty(D, dtype=torch.float32, device=cuda)]
    small = [torch.empty(7, D, dtype=torch.bfloat16, device=cuda), torch.empty(D, dtype=torch.float32, device=cuda)]

    def call(stream, n, dx, dgate, dw):
        _lib.check(lib.lmoe_rmsnorm_bwd_noalloc(p(x), p(w), p(gate), p(dy), p(dx), p(dgate), p(dw), n, D, dt, 1e-5,
                                                C.c_void_p(stream.cuda_stream)), "noalloc")

    call(torch.cuda.current_stream(), 7, small[0], small[0], small[1])       # resolves the scratch address, eagerly
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(torch.cuda.current_stream(), rows, *out)
    for _ in range(3):
        for t in out:
            t.zero_()
        call(torch.cuda.current_stream(), 7, small[0], small[0], small[1])   # shares the array: overwrites a prefix of it
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert all(torch.equal(a, b) for a, b in zip(out, ref))
