"""Token-by-token (``fused_recurrent_*``) forward of the ops on MI355X, for decoding and short sequences.

The reference selects these callables with ``la_mode='fused_recurrent'``
(``linear_moe/sequence_modeling/gated_deltanet/gated_deltanet.py:72-73``, ``gla/gla.py:58-59``,
``deltanet/deltanet.py:81-82``, ``basic_linear_attention/basic_linear_attention.py:99-100``).  Same
signatures and results as the chunk ops.  The recurrent kernel keeps the state in registers and saves
nothing, so it serves calls that need no gradient (generation); a call that does need one runs the
chunk kernels, which compute the same function.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Tuple

import torch

from . import _lib
from ._host import seq_plan, _aligned, _check_inputs, _desc, _state_check, base_args, ptr, stream_ptr
from .delta_rule import chunk_delta_rule
from .gated_delta_rule import chunk_gated_delta_rule
from .gla import chunk_gla
from .l2norm import l2_norm
from .simple_gla import chunk_simple_gla

_OP_SIMPLE, _OP_GLA, _OP_GDN = 0, 1, 2


def _needs_grad(*xs) -> bool:
    return torch.is_grad_enabled() and any(x is not None and torch.is_tensor(x) and x.requires_grad for x in xs)


def _sdt(x: torch.Tensor) -> int:
    return _lib.LMOE_F32 if x.dtype == torch.float32 else _lib.LMOE_BF16


def _recurrent(op, q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens, head_first):
    lib = _lib.load()
    dims = _check_inputs(q, k, v, head_first, cu_seqlens)
    B, T, H, K, V = dims
    q, k, v = _aligned(q.detach()), _aligned(k.detach()), _aligned(v.detach())
    plan = seq_plan(B, T, cu_seqlens, q.device)
    a = base_args(q, k, v, head_first, scale, plan, dims)
    tok = (B, H, T) if head_first else (B, T, H)
    a.gate = _lib.GATE_NONE
    if g is not None:
        g = g.detach()
        if g.dtype not in (torch.float32, torch.bfloat16):
            g = g.float()
        if op == _OP_GLA:
            if g.shape != q.shape:
                raise ValueError(f"g must have the shape of q, got {tuple(g.shape)}")
            g = _aligned(g)
            a.gate = _lib.GATE_VECTOR
        else:
            if tuple(g.shape) != tok:
                raise ValueError(f"g must have shape {tok}, got {tuple(g.shape)}")
            a.gate = _lib.GATE_SCALAR
        a.g, a.g_dtype = _desc(g, head_first), _sdt(g)
    elif op == _OP_GLA:
        raise ValueError("fused_recurrent_gla needs the gate g")
    if op == _OP_GDN:
        if beta is None or tuple(beta.shape) != tok:
            raise ValueError(f"beta must have shape {tok}")
        beta = beta.detach()
        if beta.dtype not in (torch.float32, torch.bfloat16):
            beta = beta.float()
        a.beta, a.beta_dtype = _desc(beta, head_first), _sdt(beta)
    h0 = _state_check(initial_state, plan.N, H, K, V, "initial_state")
    a.h0 = ptr(h0)
    o = torch.empty_like(v)
    ht = torch.empty(plan.N, H, K, V, dtype=torch.float32, device=q.device) if output_final_state else None
    a.o, a.ht = _desc(o, head_first), ptr(ht)
    _lib.check(lib.lmoe_fused_recurrent_fwd(C.byref(a), op, stream_ptr()), "fused_recurrent forward")
    return o, ht


def fused_recurrent_simple_gla(q, k, v, g=None, scale: Optional[float] = None, initial_state=None,
                               output_final_state: bool = False, cu_seqlens=None, head_first: bool = True
                               ) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    if _needs_grad(q, k, v, g, initial_state):
        return chunk_simple_gla(q, k, v, g, scale, initial_state, output_final_state, cu_seqlens, head_first)
    return _recurrent(_OP_SIMPLE, q, k, v, g, None, scale, initial_state, output_final_state, cu_seqlens, head_first)


def fused_recurrent_gla(q, k, v, gk=None, scale: Optional[float] = None, initial_state=None,
                        output_final_state: bool = False, cu_seqlens=None, head_first: bool = True
                        ) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    if _needs_grad(q, k, v, gk, initial_state):
        return chunk_gla(q, k, v, gk, scale, initial_state, output_final_state, cu_seqlens, head_first)
    return _recurrent(_OP_GLA, q, k, v, gk, None, scale, initial_state, output_final_state, cu_seqlens, head_first)


def fused_recurrent_gated_delta_rule(q, k, v, g, beta, scale: Optional[float] = None, initial_state=None,
                                     output_final_state: bool = False, cu_seqlens=None, head_first: bool = False,
                                     use_qk_l2norm_in_kernel: bool = False
                                     ) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    if _needs_grad(q, k, v, g, beta, initial_state):
        return chunk_gated_delta_rule(q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens,
                                      head_first, use_qk_l2norm_in_kernel)
    if use_qk_l2norm_in_kernel:
        q, k = l2_norm(q.detach()), l2_norm(k.detach())
    return _recurrent(_OP_GDN, q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens, head_first)


def fused_recurrent_delta_rule(q, k, v, beta, scale: Optional[float] = None, initial_state=None,
                               output_final_state: bool = False, cu_seqlens=None, head_first: bool = True
                               ) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    if _needs_grad(q, k, v, beta, initial_state):
        return chunk_delta_rule(q, k, v, beta, 64, scale, initial_state, output_final_state, cu_seqlens, head_first)
    return _recurrent(_OP_GDN, q, k, v, None, beta, scale, initial_state, output_final_state, cu_seqlens, head_first)
