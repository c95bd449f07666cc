"""ctypes binding of ``liblmoe_hip.so`` (C ABI declared in ``include/lmoe.h``).

The library is the only compute path of this package: when it is missing every op raises
``RuntimeError`` -- there is no eager or CPU fallback.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liblmoe_hip.so")

LMOE_BF16, LMOE_F32 = 0, 1
GATE_NONE, GATE_SCALAR, GATE_VECTOR = 0, 1, 2
CHUNK = 64


class Tensor4(C.Structure):
    """``lmoe_tensor``: x[b][t][h][d] at ptr + b*sb + t*st + h*sh + d (element strides)."""
    _fields_ = [("ptr", C.c_void_p), ("sb", C.c_int64), ("st", C.c_int64), ("sh", C.c_int64)]


class Args(C.Structure):
    """``lmoe_args`` -- field order must match include/lmoe.h."""
    _fields_ = [
        ("dtype", C.c_int32), ("g_dtype", C.c_int32), ("beta_dtype", C.c_int32), ("gate", C.c_int32),
        ("B", C.c_int32), ("T", C.c_int32), ("H", C.c_int32), ("K", C.c_int32), ("V", C.c_int32),
        ("N", C.c_int32), ("NT", C.c_int32), ("scale", C.c_float),
        ("cu_seqlens", C.c_void_p), ("chunk_map", C.c_void_p), ("seq_chunk0", C.c_void_p),
        ("q", Tensor4), ("k", Tensor4), ("v", Tensor4), ("g", Tensor4), ("beta", Tensor4),
        ("h0", C.c_void_p),
        ("o", Tensor4), ("ht", C.c_void_p),
        ("hs", C.c_void_p), ("vnew", Tensor4), ("w", Tensor4), ("u", Tensor4),
        ("tinv", C.c_void_p), ("amat", C.c_void_p), ("pmat", C.c_void_p), ("gcum", C.c_void_p),
        ("qe", C.c_void_p), ("ke", C.c_void_p),
        ("d_o", Tensor4), ("dht", C.c_void_p),
        ("dq", Tensor4), ("dk", Tensor4), ("dv", Tensor4), ("dg", Tensor4), ("dbeta", Tensor4),
        ("dh0", C.c_void_p),
        ("dhs", C.c_void_p), ("dvnew", Tensor4),
        ("seq_order", C.c_void_p),
        ("nt_dev", C.c_void_p),
        ("normalize", C.c_int32), ("norm_eps", C.c_float), ("den", Tensor4), ("zs", C.c_void_p),
        ("norm_ws", C.c_void_p), ("v_act", C.c_int32), ("dden", Tensor4),
        ("q_raw", Tensor4), ("k_raw", Tensor4), ("qk_eps", C.c_float),
    ]


ENTRY_POINTS = (
    "lmoe_version", "lmoe_last_error",
    "lmoe_chunk_simple_gla_fwd", "lmoe_chunk_simple_gla_bwd",
    "lmoe_chunk_gla_fwd", "lmoe_chunk_gla_bwd",
    "lmoe_chunk_gated_delta_rule_fwd", "lmoe_chunk_gated_delta_rule_bwd",
    "lmoe_launch_stage", "lmoe_selftest_gemm", "lmoe_workspace_bytes", "lmoe_l2norm_fwd", "lmoe_l2norm_bwd",
    "lmoe_silu_l2norm_fwd", "lmoe_silu_l2norm_bwd", "lmoe_gdn_qkv_prologue_fwd", "lmoe_gdn_qkv_prologue_bwd",
    "lmoe_swish_gate_relayout_fwd", "lmoe_swish_gate_relayout_bwd", "lmoe_rmsnorm_partials", "lmoe_rmsnorm_fwd", "lmoe_rmsnorm_bwd", "lmoe_rmsnorm_bwd_noalloc",
    "lmoe_gdn_gates_partials", "lmoe_gdn_gates_fwd", "lmoe_gdn_gates_bwd", "lmoe_gla_gate_fwd", "lmoe_gla_gate_bwd",
    "lmoe_hgrn2_gate_fwd", "lmoe_hgrn2_gate_bwd", "lmoe_quad_featmap_features", "lmoe_quad_featmap_fwd",
    "lmoe_quad_featmap_bwd",
    "lmoe_fused_recurrent_fwd", "lmoe_trace_gdn_state_fwd", "lmoe_trace_simple_gla_fwd", "lmoe_mom_gather", "lmoe_mom_combine", "lmoe_mom_rowdot",
)

_lib = None


def load() -> C.CDLL:
    """Load the HIP library (once).  Raises RuntimeError when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
            "(or __graft_entry__.build()).  This package has no fallback path.")
    lib = C.CDLL(LIB_PATH)
    lib.lmoe_version.restype = C.c_int
    lib.lmoe_last_error.restype = C.c_char_p
    for name in ENTRY_POINTS[2:8]:
        fn = getattr(lib, name)
        fn.argtypes = [C.POINTER(Args), C.c_void_p]
        fn.restype = C.c_int
    lib.lmoe_launch_stage.argtypes = [C.POINTER(Args), C.c_int32, C.c_int32, C.c_void_p]
    lib.lmoe_launch_stage.restype = C.c_int
    lib.lmoe_selftest_gemm.argtypes = [C.c_int32, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                       C.c_void_p]
    lib.lmoe_selftest_gemm.restype = C.c_int
    lib.lmoe_l2norm_fwd.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_int32, C.c_float, C.c_void_p]
    lib.lmoe_l2norm_fwd.restype = C.c_int
    lib.lmoe_l2norm_bwd.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_int32, C.c_float,
                                    C.c_void_p]
    lib.lmoe_l2norm_bwd.restype = C.c_int
    lib.lmoe_silu_l2norm_fwd.argtypes = lib.lmoe_l2norm_fwd.argtypes
    lib.lmoe_silu_l2norm_fwd.restype = C.c_int
    lib.lmoe_silu_l2norm_bwd.argtypes = lib.lmoe_l2norm_bwd.argtypes
    lib.lmoe_silu_l2norm_bwd.restype = C.c_int
    lib.lmoe_gdn_qkv_prologue_fwd.argtypes = [C.c_void_p] * 4 + [C.c_int32] * 5 + [C.c_float, C.c_void_p]
    lib.lmoe_gdn_qkv_prologue_fwd.restype = C.c_int
    lib.lmoe_gdn_qkv_prologue_bwd.argtypes = [C.c_void_p] * 5 + [C.c_int32] * 5 + [C.c_float, C.c_void_p]
    lib.lmoe_gdn_qkv_prologue_bwd.restype = C.c_int
    lib.lmoe_swish_gate_relayout_fwd.argtypes = [C.c_void_p] * 3 + [C.c_int32] * 4 + [C.c_void_p]
    lib.lmoe_swish_gate_relayout_fwd.restype = C.c_int
    lib.lmoe_swish_gate_relayout_bwd.argtypes = [C.c_void_p] * 5 + [C.c_int32] * 4 + [C.c_void_p]
    lib.lmoe_swish_gate_relayout_bwd.restype = C.c_int
    lib.lmoe_rmsnorm_partials.argtypes = [C.c_int64, C.c_int32, C.c_int32]
    lib.lmoe_rmsnorm_partials.restype = C.c_int32
    lib.lmoe_rmsnorm_fwd.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int32,
                                     C.c_int32, C.c_float, C.c_void_p]
    lib.lmoe_rmsnorm_fwd.restype = C.c_int
    lib.lmoe_rmsnorm_bwd.argtypes = [C.c_void_p] * 8 + [C.c_int64, C.c_int32, C.c_int32, C.c_float, C.c_void_p]
    lib.lmoe_rmsnorm_bwd.restype = C.c_int
    lib.lmoe_rmsnorm_bwd_noalloc.argtypes = [C.c_void_p] * 7 + [C.c_int64, C.c_int32, C.c_int32, C.c_float, C.c_void_p]
    lib.lmoe_rmsnorm_bwd_noalloc.restype = C.c_int
    lib.lmoe_gdn_gates_partials.argtypes = [C.c_int64, C.c_int32]
    lib.lmoe_gdn_gates_partials.restype = C.c_int
    lib.lmoe_gdn_gates_fwd.argtypes = [C.c_void_p] * 6 + [C.c_int64, C.c_int32, C.c_int32, C.c_void_p]
    lib.lmoe_gdn_gates_fwd.restype = C.c_int
    lib.lmoe_gdn_gates_bwd.argtypes = [C.c_void_p] * 10 + [C.c_int64, C.c_int32, C.c_int32, C.c_void_p]
    lib.lmoe_gdn_gates_bwd.restype = C.c_int
    lib.lmoe_gla_gate_fwd.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_float, C.c_float, C.c_void_p]
    lib.lmoe_gla_gate_fwd.restype = C.c_int
    lib.lmoe_gla_gate_bwd.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_float, C.c_float,
                                      C.c_void_p]
    lib.lmoe_gla_gate_bwd.restype = C.c_int
    lib.lmoe_hgrn2_gate_fwd.argtypes = [C.c_void_p] * 4 + [C.c_int64, C.c_int32, C.c_int32, C.c_void_p]
    lib.lmoe_hgrn2_gate_fwd.restype = C.c_int
    lib.lmoe_hgrn2_gate_bwd.argtypes = [C.c_void_p] * 5 + [C.c_int64, C.c_int32, C.c_int32, C.c_void_p]
    lib.lmoe_hgrn2_gate_bwd.restype = C.c_int
    lib.lmoe_quad_featmap_features.argtypes = [C.c_int32, C.c_float, C.c_float]
    lib.lmoe_quad_featmap_features.restype = C.c_int
    lib.lmoe_quad_featmap_fwd.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_int32] + [C.c_float] * 4 + [
        C.c_int32, C.c_void_p]
    lib.lmoe_quad_featmap_fwd.restype = C.c_int
    lib.lmoe_quad_featmap_bwd.argtypes = [C.c_void_p] * 3 + [C.c_int64, C.c_int32, C.c_int32] + [C.c_float] * 4 + [
        C.c_int32, C.c_void_p]
    lib.lmoe_quad_featmap_bwd.restype = C.c_int
    lib.lmoe_fused_recurrent_fwd.argtypes = [C.POINTER(Args), C.c_int32, C.c_void_p]
    lib.lmoe_fused_recurrent_fwd.restype = C.c_int
    lib.lmoe_trace_gdn_state_fwd.argtypes = [C.POINTER(Args), C.c_void_p, C.c_int32, C.c_void_p]
    lib.lmoe_trace_gdn_state_fwd.restype = C.c_int
    lib.lmoe_trace_simple_gla_fwd.argtypes = [C.POINTER(Args), C.c_void_p, C.c_int32, C.c_void_p]
    lib.lmoe_trace_simple_gla_fwd.restype = C.c_int
    lib.lmoe_mom_gather.argtypes = [C.c_void_p] * 4 + [C.c_int64, C.c_int32, C.c_int32, C.c_void_p]
    lib.lmoe_mom_gather.restype = C.c_int
    for fn in (lib.lmoe_mom_combine, lib.lmoe_mom_rowdot):
        fn.argtypes = [C.c_void_p] * 4 + [C.c_int64, C.c_int32, C.c_int32, C.c_int32, C.c_void_p]
        fn.restype = C.c_int
    lib.lmoe_workspace_bytes.argtypes = [C.c_int32] * 9
    lib.lmoe_workspace_bytes.restype = C.c_int64
    _lib = lib
    return lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().lmoe_last_error().decode()
        if rc < 0:
            raise ValueError(f"{what}: {msg} (code {rc})")
        raise RuntimeError(f"{what}: {msg} (hipError {rc})")
