"""CPU-only checks of the host side: the C ABI library loads and exports what include/lmoe.h
declares, the ctypes mirror of lmoe_args has the C layout, the chunk tables of packed input are
right, and invalid calls are rejected before anything is launched."""
import ctypes as C
import os
import re
import subprocess
import sys
import tempfile

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "lmoe.h")


def declared_functions():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return re.findall(r"^\s*(?:const\s+char\s*\*|int64_t|int)\s+(lmoe_\w+)\s*\(", src, flags=re.M)


def test_library_exports_every_declared_symbol():
    from linear_moe_amd import _lib
    lib = _lib.load()
    names = declared_functions()
    assert set(names) == set(_lib.ENTRY_POINTS), (names, _lib.ENTRY_POINTS)
    for n in names:
        assert getattr(lib, n) is not None
    assert lib.lmoe_version() >= 100


def test_ctypes_struct_matches_c_layout():
    from linear_moe_amd import _lib
    fields = [f[0] for f in _lib.Args._fields_]
    prog = ['#include <stdio.h>', '#include <stddef.h>', f'#include "{HEADER}"', 'int main(void){',
            'printf("%zu\\n", sizeof(lmoe_args));']
    prog += [f'printf("%zu\\n", offsetof(lmoe_args, {f}));' for f in fields]
    prog += ['return 0;}']
    with tempfile.TemporaryDirectory() as d:
        src, exe = os.path.join(d, "t.c"), os.path.join(d, "t")
        open(src, "w").write("\n".join(prog))
        subprocess.check_call(["gcc", "-o", exe, src])
        out = [int(x) for x in subprocess.check_output([exe]).split()]
    assert out[0] == C.sizeof(_lib.Args)
    for f, off in zip(fields, out[1:]):
        assert getattr(_lib.Args, f).offset == off, f


def test_invalid_arguments_are_rejected_without_a_launch():
    from linear_moe_amd import _lib
    lib = _lib.load()
    for name in _lib.ENTRY_POINTS[2:8]:
        assert getattr(lib, name)(None, None) == -1
        assert b"null argument block" in lib.lmoe_last_error()
    a = _lib.Args()
    a.dtype, a.K, a.V, a.H = 7, 64, 64, 1
    assert lib.lmoe_chunk_simple_gla_fwd(C.byref(a), None) == -2
    a.dtype, a.K = _lib.LMOE_BF16, 48
    assert lib.lmoe_chunk_simple_gla_fwd(C.byref(a), None) == -3
    assert b"K=48" in lib.lmoe_last_error()
    a.K, a.B, a.N = 64, 2, 1                       # dense input must have N == B
    assert lib.lmoe_chunk_gla_fwd(C.byref(a), None) == -6
    a.N = 2                                        # q, k, v null
    assert lib.lmoe_chunk_gated_delta_rule_fwd(C.byref(a), None) == -7
    with pytest.raises(ValueError):
        _lib.check(-7, "x")
    assert lib.lmoe_selftest_gemm(0, 64, None, None, None, None, None) == -1


def test_gated_delta_rule_needs_w_and_u_only_where_the_state_pass_reads_them():
    """2-byte elements with a Tinv buffer: the state pass forms w, u itself, they may be NULL.  4-byte elements, or no
    Tinv: they are required.  A call without chunks validates and returns before any launch (no GPU needed)."""
    from linear_moe_amd import _lib
    lib = _lib.load()
    fake = 0x1000                                  # never dereferenced: NT == 0

    def args(dtype, tinv, wu):
        a = _lib.Args()
        a.dtype, a.B, a.T, a.H, a.K, a.V, a.N, a.NT = dtype, 1, 0, 1, 64, 64, 1, 0
        a.scale, a.gate, a.g_dtype, a.beta_dtype = 1.0, 1, _lib.LMOE_F32, dtype
        for n in ("q", "k", "v", "g", "beta", "o"):
            setattr(a, n, _lib.Tensor4(fake, 0, 64, 64))
        a.pmat = a.gcum = fake
        a.tinv = fake if tinv else None
        if wu:
            a.w = a.u = _lib.Tensor4(fake, 0, 64, 64)
        return a

    for dtype in (_lib.LMOE_BF16, _lib.LMOE_F32):
        for tinv in (False, True):
            for wu in (False, True):
                a = args(dtype, tinv, wu)
                rc = lib.lmoe_chunk_gated_delta_rule_fwd(C.byref(a), None)
                needed = dtype == _lib.LMOE_F32 or not tinv
                assert rc == (-11 if needed and not wu else 0), (dtype, tinv, wu)
                if rc:
                    assert b"w and u must not be null" in lib.lmoe_last_error()


def test_chunk_count_and_row_alignment_are_checked_before_any_launch():
    """The kernels derive every address from B, T, NT and the strides: a chunk count that does not belong to B and T
    (dense) or exceeds the bound ceil(T / 64) + N (packed), and rows that are not 16-byte aligned, are refused."""
    from linear_moe_amd import _lib
    lib = _lib.load()
    fake = 0x1000                                  # never dereferenced: every call below is refused

    def args(**kw):
        a = _lib.Args()
        a.dtype, a.B, a.T, a.H, a.K, a.V, a.N, a.NT = _lib.LMOE_BF16, 2, 130, 1, 64, 64, 2, 6
        a.scale, a.gate = 1.0, _lib.GATE_NONE
        for n in ("q", "k", "v", "o"):
            setattr(a, n, _lib.Tensor4(fake, 130 * 64, 64, 64))
        for n, x in kw.items():
            setattr(a, n, x)
        return a

    for nt in (5, 7, 0):
        assert lib.lmoe_chunk_simple_gla_fwd(C.byref(args(NT=nt)), None) == -4
        assert b"has 6 chunks" in lib.lmoe_last_error()
    packed = dict(B=1, T=260, N=3, cu_seqlens=fake, chunk_map=fake, seq_chunk0=fake)
    assert lib.lmoe_chunk_simple_gla_fwd(C.byref(args(NT=9, **packed)), None) == -4     # at most 5 + 3
    assert b"at most 8 chunks" in lib.lmoe_last_error()
    for bad in (_lib.Tensor4(fake + 2, 130 * 64, 64, 64), _lib.Tensor4(fake, 130 * 64, 68, 64),
                _lib.Tensor4(fake, 130 * 64 + 4, 64, 64), _lib.Tensor4(fake, 130 * 64, 64, 60)):
        for name in ("q", "k", "v", "o"):
            assert lib.lmoe_chunk_simple_gla_fwd(C.byref(args(**{name: bad})), None) == -9, name
    f32 = args(dtype=_lib.LMOE_F32, v=_lib.Tensor4(fake, 130 * 64, 68, 64))            # 4 elements are 16 bytes
    assert lib.lmoe_chunk_simple_gla_bwd(C.byref(f32), None) == -11                     # (passes on to the next check)


def test_options_outside_flas_signature_are_validated_before_any_launch():
    """V = 256 belongs to the gated delta rule alone (2-byte calls then need tinv); normalize belongs to ungated 2-byte
    calls of chunk_simple_gla and names the buffers it needs; v_act needs 2-byte elements and tinv.  Calls without
    chunks validate and return before any launch (no GPU needed)."""
    from linear_moe_amd import _lib
    lib = _lib.load()
    fake = 0x1000                                  # never dereferenced: NT == 0

    def args(dtype, K=128, V=128):
        a = _lib.Args()
        a.dtype, a.B, a.T, a.H, a.K, a.V, a.N, a.NT = dtype, 1, 0, 1, K, V, 1, 0
        a.scale, a.gate, a.g_dtype, a.beta_dtype = 1.0, _lib.GATE_SCALAR, _lib.LMOE_F32, dtype
        for n in ("q", "k", "v", "g", "beta", "o", "w", "u"):
            setattr(a, n, _lib.Tensor4(fake, 0, 64, 64))
        a.pmat = a.gcum = a.tinv = fake
        return a

    a = args(_lib.LMOE_BF16, V=256)
    assert lib.lmoe_chunk_gated_delta_rule_fwd(C.byref(a), None) == 0
    assert lib.lmoe_chunk_simple_gla_fwd(C.byref(a), None) == -3 and b"V=256" in lib.lmoe_last_error()
    a.tinv = None
    assert lib.lmoe_chunk_gated_delta_rule_fwd(C.byref(a), None) == -11 and b"needs tinv" in lib.lmoe_last_error()
    assert lib.lmoe_chunk_gated_delta_rule_fwd(C.byref(args(_lib.LMOE_F32, V=256)), None) == 0
    assert lib.lmoe_chunk_gated_delta_rule_fwd(C.byref(args(_lib.LMOE_BF16, K=64, V=256)), None) == -3
    # v_act
    a = args(_lib.LMOE_BF16)
    a.v_act = 1
    assert lib.lmoe_chunk_gated_delta_rule_fwd(C.byref(a), None) == 0
    a.dtype = a.beta_dtype = _lib.LMOE_F32
    assert lib.lmoe_chunk_gated_delta_rule_fwd(C.byref(a), None) == -15 and b"v_act" in lib.lmoe_last_error()
    # q_raw / k_raw (backward): both or neither, 2-byte elements, V <= 128
    def bwd_args(dtype, V=128):
        b = args(dtype, V=V)
        b.hs = b.dhs = fake
        b.vnew.ptr = b.dvnew.ptr = fake
        b.d_o = b.dq = b.dk = b.dv = b.dg = b.dbeta = _lib.Tensor4(fake, 0, 64, 64)
        return b
    b = bwd_args(_lib.LMOE_BF16)
    assert lib.lmoe_chunk_gated_delta_rule_bwd(C.byref(b), None) == 0
    b.q_raw = _lib.Tensor4(fake, 0, 64, 64)
    assert lib.lmoe_chunk_gated_delta_rule_bwd(C.byref(b), None) == -11 and b"go together" in lib.lmoe_last_error()
    b.k_raw = _lib.Tensor4(fake, 0, 64, 64)
    assert lib.lmoe_chunk_gated_delta_rule_bwd(C.byref(b), None) == 0
    for bad in (bwd_args(_lib.LMOE_F32), bwd_args(_lib.LMOE_BF16, V=256)):
        bad.q_raw = bad.k_raw = _lib.Tensor4(fake, 0, 64, 64)
        assert lib.lmoe_chunk_gated_delta_rule_bwd(C.byref(bad), None) == -15
    # normalize
    a = args(_lib.LMOE_BF16)
    a.gate, a.normalize, a.norm_eps = _lib.GATE_NONE, 1, 1e-10
    assert lib.lmoe_chunk_simple_gla_fwd(C.byref(a), None) == -11 and b"den" in lib.lmoe_last_error()
    a.den = _lib.Tensor4(fake, 0, 1, 1)
    assert lib.lmoe_chunk_simple_gla_fwd(C.byref(a), None) == 0          # forward only: hs NULL, zs not needed
    a.hs = fake
    assert lib.lmoe_chunk_simple_gla_fwd(C.byref(a), None) == -11 and b"zs" in lib.lmoe_last_error()
    a.zs = fake
    assert lib.lmoe_chunk_simple_gla_fwd(C.byref(a), None) == 0
    a.gate = _lib.GATE_SCALAR
    assert lib.lmoe_chunk_simple_gla_fwd(C.byref(a), None) == -15 and b"LMOE_GATE_NONE" in lib.lmoe_last_error()
    a.gate, a.dtype = _lib.GATE_NONE, _lib.LMOE_F32
    assert lib.lmoe_chunk_simple_gla_fwd(C.byref(a), None) == -15 and b"2-byte" in lib.lmoe_last_error()
    a.dtype = _lib.LMOE_BF16
    a.dhs = fake
    a.d_o = a.dq = a.dk = a.dv = _lib.Tensor4(fake, 0, 64, 64)
    assert lib.lmoe_chunk_simple_gla_bwd(C.byref(a), None) == -11 and b"norm_ws" in lib.lmoe_last_error()
    a.norm_ws = fake
    assert lib.lmoe_chunk_simple_gla_bwd(C.byref(a), None) == 0
    a.normalize = 2                                # den as a second output: the backward wants its gradient
    assert lib.lmoe_chunk_simple_gla_fwd(C.byref(a), None) == 0
    assert lib.lmoe_chunk_simple_gla_bwd(C.byref(a), None) == -11 and b"dden" in lib.lmoe_last_error()
    a.dden = _lib.Tensor4(fake, 0, 1, 1)
    assert lib.lmoe_chunk_simple_gla_bwd(C.byref(a), None) == 0
    a.normalize = 3
    assert lib.lmoe_chunk_simple_gla_fwd(C.byref(a), None) == -15


def test_chunk_gla_forward_needs_hs_only_where_an_output_kernel_reads_it():
    """2-byte elements: the forward state pass forms the output itself and hs, which only the backward reads, may be
    NULL (a forward-only call).  4-byte elements hand the states to their output kernel through hs: required.  A
    call without chunks validates and returns before any launch (no GPU needed)."""
    from linear_moe_amd import _lib
    lib = _lib.load()
    fake = 0x1000                                  # never dereferenced: NT == 0
    for dtype in (_lib.LMOE_BF16, _lib.LMOE_F32):
        for with_hs in (False, True):
            a = _lib.Args()
            a.dtype, a.B, a.T, a.H, a.K, a.V, a.N, a.NT = dtype, 1, 0, 1, 64, 64, 1, 0
            a.scale, a.gate, a.g_dtype = 1.0, _lib.GATE_VECTOR, _lib.LMOE_F32
            for n in ("q", "k", "v", "g", "o"):
                setattr(a, n, _lib.Tensor4(fake, 0, 64, 64))
            a.amat = a.qe = a.ke = a.gcum = fake
            a.hs = fake if with_hs else None
            rc = lib.lmoe_chunk_gla_fwd(C.byref(a), None)
            assert rc == (-11 if dtype == _lib.LMOE_F32 and not with_hs else 0), (dtype, with_hs)
            if rc:
                assert b"hs must not be null" in lib.lmoe_last_error()
            if not with_hs:                        # the backward always needs it
                a.dhs = fake
                a.d_o = a.dq = a.dk = a.dv = a.dg = _lib.Tensor4(fake, 0, 64, 64)
                assert lib.lmoe_chunk_gla_bwd(C.byref(a), None) == -11


def test_workspace_bytes_matches_the_buffers_the_host_layer_allocates():
    from linear_moe_amd import _lib
    lib = _lib.load()
    B, T, H, K, V = 2, 200, 3, 64, 128
    NT = B * ((T + 63) // 64)
    for dtype, s in ((_lib.LMOE_BF16, 2), (_lib.LMOE_F32, 4)):
        states, tiles, rk, rv = NT * H * K * V, NT * H * 64 * 64, B * T * H * K, B * T * H * V
        bv = NT * H * 64 * V          # vnew / dvnew: whole chunks in the library's blocked layout [NT,H,V/32,64,32]
        want = {(0, 0): states, (0, 1): states, (1, 0): states + tiles + 2 * NT * H * 64 * K, (1, 1): states,
                (2, 0): states + 2 * tiles + bv + (rk + rv if s == 4 else 0), (2, 1): states + bv}
        for (op, part), n in want.items():
            extra = NT * H * 5 * 64 * 4 if (op, part) == (2, 0) else 0      # fp32 gate table of the delta rule
            extra = NT * H * K * 4 if (op, part) == (1, 0) else extra       # fp32 chunk decays of chunk_gla
            assert lib.lmoe_workspace_bytes(op, dtype, part, B, T, H, K, V, NT) == n * s + extra
    assert lib.lmoe_workspace_bytes(5, 0, 0, B, T, H, K, V, NT) == -21
    assert lib.lmoe_workspace_bytes(0, 9, 0, B, T, H, K, V, NT) == -2
    assert lib.lmoe_workspace_bytes(0, 0, 2, B, T, H, K, V, NT) == -22
    assert lib.lmoe_workspace_bytes(0, 0, 0, B, -1, H, K, V, NT) == -4


def test_seq_plan_tables():
    from linear_moe_amd._host import SeqPlan
    p = SeqPlan(3, 130, None, "cpu")
    assert (p.N, p.NT) == (3, 9) and p.cu is None
    cu = torch.tensor([0, 1, 65, 200, 270, 270], dtype=torch.int64)
    p = SeqPlan(1, 270, cu, "cpu")
    assert p.N == 5 and p.NT == 1 + 1 + 3 + 2 + 0
    assert p.seq_chunk0.tolist() == [0, 1, 2, 5, 7, 7]
    assert p.chunk_map.tolist() == [[0, 0], [1, 0], [2, 0], [2, 1], [2, 2], [3, 0], [3, 1]]
    assert p.cu.dtype == torch.int32
    # the order in which the sequential passes take the sequences: by number of chunks, longest first, ties as given
    assert p.seq_order.dtype == torch.int32 and p.seq_order.tolist() == [2, 3, 0, 1, 4]
    assert SeqPlan(1, 256, torch.tensor([0, 64, 128, 256 - 64, 256]), "cpu").seq_order is None      # equal lengths
    for bad in ([1, 5, 270], [0, 50, 40, 270], [0, 100]):
        with pytest.raises(ValueError):
            SeqPlan(1, 270, torch.tensor(bad), "cpu")


def test_tables_built_without_reading_the_offsets_equal_the_validated_ones():
    """The table builder for offsets that stay on the device (run here on CPU tensors: it is made of torch operations
    only, none of which needs a value on the host) against the host path: the first NT rows of chunk_map, the first
    chunks, the count and the order agree; the rows past the count belong to no sequence."""
    from linear_moe_amd._host import SeqPlan
    for lens in ([5, 64, 0, 200, 1, 65], [64, 64], [1], [0, 0, 130]):
        T = sum(lens)
        cu = torch.tensor([0] + lens).cumsum(0).to(torch.int32)
        exact = SeqPlan(1, T, cu, "cpu")
        dev = SeqPlan.__new__(SeqPlan)
        dev.seq_order = None
        dev._build_on_device(T, cu)
        nt = int(dev.nt_dev)
        assert nt == exact.NT <= dev.NT == (T + 63) // 64 + len(lens)
        assert torch.equal(dev.chunk_map[:nt], exact.chunk_map) and torch.equal(dev.seq_chunk0, exact.seq_chunk0)
        assert (dev.chunk_map[nt:, 0] == len(lens)).all()
        assert dev.chunk_map.dtype == dev.seq_chunk0.dtype == dev.nt_dev.dtype == torch.int32
        if exact.seq_order is not None:
            assert torch.equal(dev.seq_order, exact.seq_order)


def test_seq_plan_is_built_once_per_cu_seqlens_tensor():
    """The chunk tables of a packed batch are built on the first call that sees its cu_seqlens tensor; later calls with
    the same tensor (the other layers, the backward, every step that reuses the batch) take them from the cache without
    touching the offsets -- no host read, hence no synchronisation.  An in-place change or another tensor with equal
    contents makes a new plan."""
    from linear_moe_amd import _host
    _host._PLAN_CACHE.clear()
    cu = torch.tensor([0, 1, 65, 200], dtype=torch.int32)
    p1 = _host.seq_plan(1, 200, cu, "cpu")
    assert _host.seq_plan(1, 200, cu, "cpu") is p1
    other = cu.clone()
    p2 = _host.seq_plan(1, 200, other, "cpu")
    assert p2 is not p1 and p2.chunk_map.tolist() == p1.chunk_map.tolist()
    assert _host.seq_plan(1, 200, cu, "cpu") is p1                 # still cached behind the newer entry
    cu[1] = 2                                                      # in-place change: the version counter moves
    p3 = _host.seq_plan(1, 200, cu, "cpu")
    assert p3 is not p1 and p3.cu.tolist() == [0, 2, 65, 200]
    for i in range(_host._PLAN_CACHE_SIZE + 3):                    # bounded
        _host.seq_plan(1, 200, torch.tensor([0, 100 + i, 200]), "cpu")
    assert len(_host._PLAN_CACHE) == _host._PLAN_CACHE_SIZE
    assert _host.prepare_cu_seqlens(other, 200, "cpu").NT == 1 + 1 + 3
    with pytest.raises(ValueError):
        _host.seq_plan(1, 201, other, "cpu")                       # another T: validated afresh
    # a write that the version counter does not see: offsets on the host are compared on a hit, the stale entry goes
    p4 = _host.seq_plan(1, 200, other, "cpu")
    other.data[1] = 3
    p5 = _host.seq_plan(1, 200, other, "cpu")
    assert p5 is not p4 and p5.cu.tolist() == [0, 3, 65, 200]
    assert _host.seq_plan(1, 200, other, "cpu") is p5


def test_python_layer_validates_before_launch():
    import linear_moe_amd as L
    q = torch.zeros(1, 2, 8, 64)
    with pytest.raises(RuntimeError, match="GPU only"):
        L.chunk_simple_gla(q, q, q)
    from linear_moe_amd._host import _check_inputs
    qc = torch.zeros(1, 2, 8, 64, device="meta")

    class Fake:  # shape / dtype / is_cuda carrier: validation must not touch data
        def __init__(self, t, dt=torch.bfloat16):
            self.shape, self.dtype, self.is_cuda, self._t = t.shape, dt, True, t

        def dim(self):
            return self._t.dim()

    f = Fake(qc)
    assert _check_inputs(f, f, f, True, None) == (1, 8, 2, 64, 64)
    with pytest.raises(ValueError, match="unsupported"):
        g = Fake(torch.zeros(1, 2, 8, 48, device="meta"))
        _check_inputs(g, g, g, True, None)
    with pytest.raises(ValueError, match="head_first=False"):
        _check_inputs(f, f, f, True, torch.tensor([0, 8]))
    with pytest.raises(ValueError, match="batch size 1"):
        g = Fake(torch.zeros(2, 8, 2, 64, device="meta"))
        _check_inputs(g, g, g, False, torch.tensor([0, 8]))
    with pytest.raises(ValueError, match="dtype"):
        g = Fake(qc, torch.float16)
        _check_inputs(g, g, g, True, None)


REFERENCE_PKG = "/root/reference/linear_moe"

# the import lines of the reference as of this writing; used where the reference is not mounted
_KNOWN_IMPORTS = {
    "fla.ops.gla": ["chunk_gla", "fused_chunk_gla", "fused_recurrent_gla"],
    "fla.ops.gated_delta_rule": ["chunk_gated_delta_rule", "fused_recurrent_gated_delta_rule"],
    "fla.ops.delta_rule": ["chunk_delta_rule", "fused_chunk_delta_rule", "fused_recurrent_delta_rule"],
    "fla.ops.linear_attn": ["chunk_linear_attn", "fused_chunk_linear_attn", "fused_recurrent_linear_attn"],
    "fla.ops.retention": ["chunk_retention", "fused_chunk_retention", "fused_recurrent_retention",
                          "parallel_retention"],
    "fla.ops.based": ["parallel_based"], "fla.ops.rebased": ["parallel_rebased"],
    "fla.ops.rwkv6": ["chunk_rwkv6", "fused_recurrent_rwkv6"],
    "fla.ops.rwkv7": ["chunk_rwkv7", "fused_recurrent_rwkv7"],
    "fla.ops.rotary": ["apply_rotary"], "fla.modules.rotary": ["RotaryEmbedding"],
    "fla.modules.l2norm": ["l2_norm"],
    "lightning_attn.ops.triton": ["lightning_attn2", "lightning_attn2_no_decay"],
}


def _reference_imports():
    """{module: sorted names} of every ``from fla... import`` / ``from lightning_attn... import`` statement in the
    reference's package, read from the source text with ``ast`` (nothing of the reference is imported or run)."""
    import ast
    found = {}
    for dirpath, _, files in os.walk(REFERENCE_PKG):
        for f in files:
            if not f.endswith(".py"):
                continue
            try:
                tree = ast.parse(open(os.path.join(dirpath, f), encoding="utf-8", errors="replace").read())
            except SyntaxError:
                continue
            for node in ast.walk(tree):
                if isinstance(node, ast.ImportFrom) and node.module and node.level == 0 and \
                        node.module.split(".")[0] in ("fla", "lightning_attn"):
                    found.setdefault(node.module, set()).update(a.name for a in node.names)
                elif isinstance(node, ast.Import):
                    for a in node.names:
                        if a.name.split(".")[0] in ("fla", "lightning_attn"):
                            found.setdefault(a.name, set())
    return {m: sorted(n) for m, n in found.items()}


def test_fla_shim_resolves_every_name_the_reference_imports():
    """A fresh interpreter with only the shim directory on its path (as the reference's launcher sets
    PYTHONPATH=$FLA_PATH) resolves every ``fla`` / ``lightning_attn`` import statement found in the reference's
    sources (collected at test time where the reference is mounted; the recorded list otherwise, and the two
    must agree), plus ``fla.ops.simple_gla``."""
    shim = os.path.join(ROOT, "linear_moe_amd", "fla_shim")
    imports = dict(_KNOWN_IMPORTS)
    if os.path.isdir(REFERENCE_PKG):
        scanned = _reference_imports()
        assert scanned, "no fla import found in the reference: the scan is broken"
        assert scanned == {m: sorted(n) for m, n in _KNOWN_IMPORTS.items()}, \
            "the reference imports names the recorded list does not hold (or the reverse)"
        imports = scanned
    lines = [f"from {m} import {', '.join(n)}" if n else f"import {m}" for m, n in sorted(imports.items())]
    code = "\n".join(lines) + (
        "\nfrom fla.ops.simple_gla import chunk_simple_gla\n"
        "from fla.modules.l2norm import l2_norm\n"
        "from fla.ops.gated_delta_rule import chunk_gated_delta_rule\n"
        "from fla.ops.rotary import apply_rotary\n"
        "from fla.ops.rwkv6 import chunk_rwkv6\n"
        "import linear_moe_amd, torch\n"
        "assert chunk_gated_delta_rule is linear_moe_amd.chunk_gated_delta_rule\n"
        "assert l2_norm is linear_moe_amd.l2_norm\n"
        "for fn in (apply_rotary, chunk_rwkv6):\n"
        "    try:\n"
        "        fn()\n"
        "    except NotImplementedError:\n"
        "        pass\n"
        "    else:\n"
        "        raise SystemExit('a name off the path must raise when called')\n"
        "print('ok')\n")
    env = {k: v for k, v in os.environ.items() if k != "PYTHONPATH"}
    env["PYTHONPATH"] = shim
    out = subprocess.check_output([sys.executable, "-c", code], env=env, cwd=tempfile.gettempdir())
    assert out.strip() == b"ok"


def test_head_dim_blocks_plan():
    from linear_moe_amd._host import dim_blocks
    assert dim_blocks(64) == [(0, 64, 64)] and dim_blocks(128) == [(0, 128, 128)]
    assert dim_blocks(16) == [(0, 16, 64)] and dim_blocks(96) == [(0, 96, 128)]
    assert dim_blocks(256) == [(0, 128, 128), (128, 256, 128)]
    assert dim_blocks(192) == [(0, 128, 128), (128, 192, 64)]
    for d in range(1, 400):
        b = dim_blocks(d)
        assert b[0][0] == 0 and b[-1][1] == d and all(x[1] == y[0] for x, y in zip(b, b[1:]))
        assert all(w in (64, 128) and 0 < d1 - d0 <= w for d0, d1, w in b)
    with pytest.raises(ValueError):
        dim_blocks(0)


@pytest.mark.parametrize("op,K,V", [("gla", 160, 80), ("gla", 48, 256), ("gdn", 96, 256), ("gdn", 32, 48)])
def test_ops_on_other_head_dims_are_the_op_on_padded_blocks(op, K, V):
    """The pad / cut / add logic around the kernels, with the fp64 token recurrence standing in for the kernels (on
    the block sizes the kernels take, asserted): outputs, final state and every gradient equal the recurrence on
    the whole head dimensions."""
    from oracle import naive
    from linear_moe_amd._host import by_head_dim_blocks
    from tests.util import gen
    B, T, H = 2, 9, 2
    dd = torch.float64
    q, k = gen(1, B, T, H, K, dtype=dd), gen(2, B, T, H, K, dtype=dd)
    v, h0 = gen(3, B, T, H, V, dtype=dd), gen(4, B, H, K, V, dtype=dd) * 0.3
    if op == "gdn":
        k = torch.nn.functional.normalize(k, dim=-1)
    gk = torch.nn.functional.logsigmoid(gen(5, B, T, H, K, dtype=dd)) if op == "gla" else None
    g = -torch.rand(B, T, H, generator=torch.Generator().manual_seed(6), dtype=dd)
    beta = torch.rand(B, T, H, generator=torch.Generator().manual_seed(7), dtype=dd)
    scale = K ** -0.5
    seen = []

    def core(q_, k_, v_, g_, h_):
        seen.append((q_.shape[-1], v_.shape[-1]))
        if op == "gla":
            return naive.naive_recurrent_gla(q_, k_, v_, g_, scale, h_, True, None, False)
        return naive.naive_recurrent_gated_delta_rule(q_, k_, v_, g, beta, scale, h_, True, None, False)

    leaves = [x.clone().requires_grad_(True) for x in (q, k, v, h0)] + ([gk.clone().requires_grad_(True)] if op == "gla" else [])
    o, ht = by_head_dim_blocks(core, leaves[0], leaves[1], leaves[2], leaves[4] if op == "gla" else None, leaves[3], True,
                               op == "gla", op)
    assert all(kk in (64, 128) and vv in (64, 128) for kk, vv in seen)
    ref_leaves = [x.clone().requires_grad_(True) for x in (q, k, v, h0)] + ([gk.clone().requires_grad_(True)] if op == "gla" else [])
    if op == "gla":
        ro, rht = naive.naive_recurrent_gla(ref_leaves[0], ref_leaves[1], ref_leaves[2], ref_leaves[4], scale, ref_leaves[3], True, None, False)
    else:
        ro, rht = naive.naive_recurrent_gated_delta_rule(ref_leaves[0], ref_leaves[1], ref_leaves[2], g, beta, scale, ref_leaves[3], True, None, False)
    assert o.shape == ro.shape and ht.shape == rht.shape
    assert torch.allclose(o, ro, atol=1e-10) and torch.allclose(ht, rht, atol=1e-10)
    do, dht = gen(8, *o.shape, dtype=dd), gen(9, *ht.shape, dtype=dd)
    gr = torch.autograd.grad((o * do).sum() + (ht * dht).sum(), leaves)
    rr = torch.autograd.grad((ro * do).sum() + (rht * dht).sum(), ref_leaves)
    for a, b in zip(gr, rr):
        assert torch.allclose(a, b, atol=1e-9)
    if op == "gdn":
        with pytest.raises(ValueError, match="one block"):
            by_head_dim_blocks(core, torch.zeros(1, 2, 1, 160), torch.zeros(1, 2, 1, 160), v[:1, :2, :1], None, None, False, False, op)
