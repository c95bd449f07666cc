"""``chunk_gla`` on MI355X: S_t = diag(e^{g_t}) S_{t-1} + k_t^T v_t, o_t = scale q_t S_t with
per-channel log-decays g_t in R^K.

Keeps flash-linear-attention's call signature as the reference uses it at
``linear_moe/sequence_modeling/gla/gla.py:94`` (``chunk_gla(q, k, v, gk)``, ``[B,H,T,D]``) and
``linear_moe/sequence_modeling/hgrn2/hgrn2.py:76``.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Tuple

import torch

from . import _lib
from ._host import (HEAD_DIMS, seq_plan, _aligned, _check_inputs, _desc, _state_check, base_args, by_head_dim_blocks,
                    no_tokens, ptr, stash, stream_ptr, unstash)


class GLACall:
    """One call of the op: owns the argument blocks and every buffer the kernels touch
    (shared by the autograd function and the benchmark harness)."""

    OP = 1  # LMOE_OP_GLA

    def __init__(self, keep: bool = False):
        self.keep = keep

    def _gate(self, a, g, head_first):
        a.gate = _lib.GATE_VECTOR
        a.g = _desc(g, head_first)
        a.g_dtype = _lib.LMOE_F32 if g.dtype == torch.float32 else _lib.LMOE_BF16

    def forward(self, q, k, v, g, scale, initial_state, output_final_state, cu_seqlens, head_first, save=True):
        """save=False: a forward-only call (nothing requires a gradient): the per-chunk states are not written where
        the state pass forms the output itself (bf16); the fp32 path's output kernel reads them."""
        lib = _lib.load()
        dims = _check_inputs(q, k, v, head_first, cu_seqlens)
        B, T, H, K, V = dims
        if g is None or tuple(g.shape) != tuple(q.shape):
            raise ValueError(f"g must have the shape of q {tuple(q.shape)}")
        # fp32 operands take an fp32 gate; bf16 operands take the gate as bf16 or fp32
        if q.dtype == torch.float32 or g.dtype not in (torch.float32, torch.bfloat16):
            g = g.float()
        q, k, v, g = _aligned(q), _aligned(k), _aligned(v), _aligned(g)
        plan = seq_plan(B, T, cu_seqlens, q.device)
        h0 = _state_check(initial_state, plan.N, H, K, V, "initial_state")
        a = base_args(q, k, v, head_first, scale, plan, dims)
        self._gate(a, g, head_first)
        a.h0 = ptr(h0)
        dev, dt = q.device, q.dtype
        o = torch.empty_like(v)
        ht = torch.empty(plan.N, H, K, V, dtype=torch.float32, device=dev) if output_final_state else None
        fused = dt == torch.bfloat16
        hs = torch.empty(max(plan.NT, 1), H, K, V, dtype=dt, device=dev) if (save or not fused) else None
        amat = torch.empty(max(plan.NT, 1), H, 64, 64, dtype=dt, device=dev)
        # gated operands of the state passes (q e^b, k e^{b_C - b}, e^{b_C}), formed once per chunk
        qe = torch.empty(max(plan.NT, 1), H, 64, K, dtype=dt, device=dev)
        ke = torch.empty_like(qe)
        gdec = torch.empty(max(plan.NT, 1), H, K, dtype=torch.float32, device=dev)
        a.o, a.ht, a.hs, a.amat = _desc(o, head_first), ptr(ht), ptr(hs), amat.data_ptr()
        a.qe, a.ke, a.gcum = qe.data_ptr(), ke.data_ptr(), gdec.data_ptr()
        _lib.check(lib.lmoe_chunk_gla_fwd(C.byref(a), stream_ptr()), "chunk_gla forward")
        self.saved = (q, k, v, g, h0, hs, amat, qe, ke, gdec)
        self.fwd_args, self.fwd_keep = a, ((o, ht) if self.keep else None)
        self.plan, self.dims, self.head_first, self.scale = plan, dims, head_first, scale
        self.has_h0 = initial_state is not None
        return o, ht

    def backward(self, do, dht):
        lib = _lib.load()
        q, k, v, g, h0, hs, amat, qe, ke, gdec = self.saved
        plan, dims, head_first = self.plan, self.dims, self.head_first
        do = _aligned(do)
        a = base_args(q, k, v, head_first, self.scale, plan, dims)
        self._gate(a, g, head_first)
        a.h0, a.hs, a.amat = ptr(h0), hs.data_ptr(), amat.data_ptr()
        a.qe, a.ke, a.gcum = qe.data_ptr(), ke.data_ptr(), gdec.data_ptr()
        a.d_o = _desc(do, head_first)
        dht = None if dht is None else dht.float().contiguous()
        a.dht = ptr(dht)
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        a.dq, a.dk, a.dv = _desc(dq, head_first), _desc(dk, head_first), _desc(dv, head_first)
        dg = torch.empty(g.shape, dtype=g.dtype, device=q.device)      # written in the dtype of g by the kernel
        a.dg = _desc(dg, head_first)
        dh0 = torch.empty_like(h0) if self.has_h0 else None
        a.dh0 = ptr(dh0)
        dhs = torch.empty_like(hs)
        a.dhs = dhs.data_ptr()
        _lib.check(lib.lmoe_chunk_gla_bwd(C.byref(a), stream_ptr()), "chunk_gla backward")
        self.bwd_args = a
        self.bwd_keep = (do, dht, dq, dk, dv, dg, dh0, dhs) if self.keep else None
        return dq, dk, dv, dg, dh0


class _ChunkGLA(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, g, scale, initial_state, output_final_state, cu_seqlens, head_first):
        call = GLACall()
        o, ht = call.forward(q, k, v, g, scale, initial_state, output_final_state, cu_seqlens, head_first,
                             save=any(ctx.needs_input_grad))
        ctx.call, ctx.g_dtype = call, g.dtype
        stash(ctx, call)
        return o, ht

    @staticmethod
    def backward(ctx, do, dht):
        unstash(ctx, ctx.call)
        try:
            dq, dk, dv, dg, dh0 = ctx.call.backward(do, dht)
        finally:
            ctx.call.saved = None
        return dq, dk, dv, dg.to(ctx.g_dtype), None, dh0, None, None, None


def chunk_gla(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: torch.Tensor,
    scale: Optional[float] = None,
    initial_state: Optional[torch.Tensor] = None,
    output_final_state: bool = False,
    cu_seqlens: Optional[torch.Tensor] = None,
    head_first: bool = True,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """q, k, g: ``[B,H,T,K]``, v: ``[B,H,T,V]`` (``[B,T,H,*]`` with ``head_first=False``); g is the
    per-channel log-space decay.  Returns ``(o, final_state)``."""
    if q.dim() == 4 and v.dim() == 4 and (q.shape[-1] not in HEAD_DIMS or v.shape[-1] not in HEAD_DIMS):
        if g is None or g.shape != q.shape:
            raise ValueError("chunk_gla: g must have the shape of q")
        sc = q.shape[-1] ** -0.5 if scale is None else scale          # of the whole key, not of a block
        return by_head_dim_blocks(
            lambda q_, k_, v_, g_, h0: chunk_gla(q_, k_, v_, g_, sc, h0, output_final_state, cu_seqlens, head_first),
            q, k, v, g, initial_state, output_final_state, True, "chunk_gla")
    r = no_tokens(q, k, v, head_first, cu_seqlens, initial_state, output_final_state)
    if r is not None:
        return r
    return _ChunkGLA.apply(q, k, v, g, scale, initial_state, output_final_state, cu_seqlens, head_first)
