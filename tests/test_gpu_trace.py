"""The traced instances of the two forward sequential passes (profiling support, include/lmoe.h): they compute
what the plain instances compute, bit for bit, and their time stamps are ordered the way the kernels' barriers
order the teams."""
import ctypes as C

import pytest
import torch

pytestmark = pytest.mark.gpu


def _ordered(t, nch, marks, bits=64):
    """stamps of one slot: marks in the given order rise within a chunk, and from chunk to chunk (bits = 32: the
    stamps are the low 32 bits of the clock, differences are taken modulo 2^32)"""
    t = t[:nch]
    assert (t[:, marks] > 0).all()

    def later(b, a):
        d = b - a
        if bits == 32:
            d = ((d + 2 ** 31) % 2 ** 32) - 2 ** 31
        return (d >= 0).all()

    for a, b in zip(marks, marks[1:]):
        assert later(t[:, b], t[:, a]), (a, b)
    assert later(t[1:, marks[0]], t[:-1, marks[-1]])


def test_traced_simple_gla_forward_is_the_forward_and_its_stamps_are_ordered():
    from linear_moe_amd import _lib
    from linear_moe_amd.simple_gla import SimpleGLACall
    lib = _lib.load()
    torch.manual_seed(11)
    dev = torch.device("cuda:0")
    B, H, T, K = 2, 4, 1000, 128
    q, k, v = (torch.randn(B, T, H, K, device=dev, dtype=torch.bfloat16) for _ in range(3))
    g = -torch.rand(B, T, H, device=dev) * 0.1
    call = SimpleGLACall(keep=True)
    o, ht = call.forward(q, k * K ** -0.5, v, g, None, None, True, None, False, save=False)
    o_ref, ht_ref = o.clone(), ht.clone()
    o.zero_(), ht.zero_()
    tr = torch.zeros(3 * 24 * 8, dtype=torch.int64, device=dev)
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    _lib.check(lib.lmoe_trace_simple_gla_fwd(C.byref(call.fwd_args), tr.data_ptr(), 3, st), "trace")
    torch.cuda.synchronize()
    assert torch.equal(o, o_ref) and torch.equal(ht, ht_ref)
    t = tr.cpu().view(3, 24, 8)
    nch = (T + 63) // 64
    _ordered(t[0], nch - 1, [0, 1, 5, 6, 2, 3], bits=32)      # (the last chunk has no next one to prepare)
    _ordered(t[1], nch, [0, 1, 5, 2, 4], bits=32)
    _ordered(t[2], nch, [0, 1, 5, 2, 4, 6], bits=32)
    assert (t[:, nch:] == 0).all()
    # the teams meet at the barrier: nobody leaves the barrier of a chunk before everybody has arrived at it
    d = t[:, None, :nch, 1] - t[None, :, :nch, 0]              # leave of team i minus arrival of team j, modulo 2^32
    assert ((((d + 2 ** 31) % 2 ** 32) - 2 ** 31) >= 0).all()
    # instances that do not exist are refused, not run
    call2 = SimpleGLACall(keep=True)
    call2.forward(q, k, v, g, None, None, False, None, False, save=True)
    assert lib.lmoe_trace_simple_gla_fwd(C.byref(call2.fwd_args), tr.data_ptr(), 3, st) == -24
    assert lib.lmoe_trace_simple_gla_fwd(C.byref(call.fwd_args), tr.data_ptr(), 10 ** 6, st) == -24


def test_traced_gdn_forward_is_the_forward_and_its_stamps_are_ordered():
    import torch.nn.functional as F
    from linear_moe_amd import _lib
    from linear_moe_amd.gated_delta_rule import GDNCall
    lib = _lib.load()
    torch.manual_seed(12)
    dev = torch.device("cuda:0")
    B, H, T, K = 2, 4, 1000, 128
    q, k = (F.normalize(torch.randn(B, T, H, K, device=dev), dim=-1).bfloat16() for _ in range(2))
    v = torch.randn(B, T, H, K, device=dev, dtype=torch.bfloat16)
    g = -torch.rand(B, T, H, device=dev) * 0.1
    beta = torch.rand(B, T, H, device=dev).bfloat16()
    call = GDNCall(keep=True)
    o, ht = call.forward(q, k, v, g, beta, None, None, True, None, False)
    o_ref, ht_ref = o.clone(), ht.clone()
    o.zero_(), ht.zero_()
    tr = torch.zeros(4 * 128 * 8, dtype=torch.int64, device=dev)
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    _lib.check(lib.lmoe_trace_gdn_state_fwd(C.byref(call.fwd_args), tr.data_ptr(), 3, st), "trace")
    torch.cuda.synchronize()
    assert torch.equal(o, o_ref) and torch.equal(ht, ht_ref)
    t = tr.cpu().view(4, 128, 8)
    nch = (T + 63) // 64
    for slot in range(4):
        _ordered(t[slot], nch, [0, 1, 2, 3])
    assert (t[:, :nch, 3].min(0).values >= t[:, :nch, 2].max(0).values).all()
