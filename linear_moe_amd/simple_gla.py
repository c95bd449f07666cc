"""``chunk_simple_gla`` on MI355X: S_t = e^{g_t} S_{t-1} + k_t^T v_t, o_t = scale q_t S_t.

Keeps flash-linear-attention's call signature; it is the op behind the reference's
``chunk_retention`` (``linear_moe/sequence_modeling/retention/retention.py:91``),
``chunk_linear_attn`` (``.../basic_linear_attention/basic_linear_attention.py:133``) and
``lightning_attn2`` (``.../lightning_attention/lightning_attention.py:121-123``).
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Tuple

import torch

from . import _lib
from ._host import (HEAD_DIMS, seq_plan, _aligned, _check_inputs, _desc, _state_check, base_args, by_head_dim_blocks,
                    no_tokens, ptr, stash, stream_ptr, unstash)


class SimpleGLACall:
    """One call of the op: owns the argument blocks and every buffer the kernels touch
    (shared by the autograd function and the benchmark harness)."""

    OP = 0  # LMOE_OP_SIMPLE_GLA

    def __init__(self, keep: bool = False):
        # keep=True (benchmark harness) also pins outputs and gradients so that the argument
        # blocks stay valid for lmoe_launch_stage; the autograd path must not (reference cycle)
        self.keep = keep

    def forward(self, q, k, v, g, scale, initial_state, output_final_state, cu_seqlens, head_first, save=True,
                norm_eps=None, emit_den=False):
        """save=False: a forward-only call (nothing requires a gradient): the per-chunk states are not written.
        norm_eps: the output leaves the kernels divided by ``scale q_t . sum_{s<=t} k_s + norm_eps`` (ungated calls
        on 2-byte elements: ``can_normalize``).  emit_den (instead of norm_eps): the output stays undivided and
        ``scale q_t . sum_{s<=t} k_s`` is kept in ``self.den`` for the caller (who adds those of several key blocks
        before dividing); ``backward`` then takes the gradient of den beside that of o."""
        ctx = self
        lib = _lib.load()
        dims = _check_inputs(q, k, v, head_first, cu_seqlens)
        B, T, H, K, V = dims
        q, k, v = _aligned(q), _aligned(k), _aligned(v)
        plan = seq_plan(B, T, cu_seqlens, q.device)
        if g is not None:
            want = (B, H, T) if head_first else (B, T, H)
            if tuple(g.shape) != want:
                raise ValueError(f"g must have shape {want}, got {tuple(g.shape)}")
            if g.dtype not in (torch.float32, torch.bfloat16):
                g = g.float()
        h0 = _state_check(initial_state, plan.N, H, K, V, "initial_state")
        a = base_args(q, k, v, head_first, scale, plan, dims)
        a.gate = _lib.GATE_NONE if g is None else _lib.GATE_SCALAR
        if g is not None:
            a.g = _desc(g, head_first)
            a.g_dtype = _lib.LMOE_F32 if g.dtype == torch.float32 else _lib.LMOE_BF16
        a.h0 = ptr(h0)
        o = torch.empty_like(v)
        ht = torch.empty(plan.N, H, K, V, dtype=torch.float32, device=q.device) if output_final_state else None
        hs = torch.empty(max(plan.NT, 1), H, K, V, dtype=q.dtype, device=q.device) if save else None
        a.o = _desc(o, head_first)
        a.ht = ptr(ht)
        a.hs = ptr(hs)
        den = zs = None
        if emit_den:
            norm_eps = 0.0
        if norm_eps is not None:
            if g is not None or q.dtype != torch.bfloat16:
                raise ValueError("the normalised output exists for ungated calls on bfloat16")
            den = torch.empty((B, H, T) if head_first else (B, T, H), dtype=torch.float32, device=q.device)
            zs = torch.empty(max(plan.NT, 1), H, K, dtype=torch.float32, device=q.device) if save else None
            a.normalize, a.norm_eps, a.den, a.zs = (2 if emit_den else 1), norm_eps, _desc(den, head_first), ptr(zs)
        _lib.check(lib.lmoe_chunk_simple_gla_fwd(C.byref(a), stream_ptr()), "chunk_simple_gla forward")
        # (emit_den: den belongs to the caller, the backward does not read it)
        ctx.saved = (q, k, v, g, h0, hs, None if emit_den else den, zs)
        ctx.norm_eps = norm_eps
        ctx.emit_den, self.den = emit_den, (den if emit_den else None)
        ctx.fwd_args, ctx.fwd_keep = a, ((o, ht) if self.keep else None)
        ctx.plan, ctx.dims, ctx.head_first, ctx.scale = plan, dims, head_first, scale
        ctx.has_h0 = initial_state is not None
        return o, ht

    def backward(self, do, dht, o=None, dden=None):
        """o: the output of the forward call, for a call with norm_eps (handed in by the caller, who holds it: this
        object must not, it would close a reference cycle through the autograd graph).  dden: the gradient of den,
        for a call with emit_den (None: zero)."""
        ctx = self
        lib = _lib.load()
        q, k, v, g, h0, hs, den, zs = ctx.saved
        plan, dims, head_first = ctx.plan, ctx.dims, ctx.head_first
        B, T, H, K, V = dims
        do = _aligned(do)
        a = base_args(q, k, v, head_first, ctx.scale, plan, dims)
        a.gate = _lib.GATE_NONE if g is None else _lib.GATE_SCALAR
        if g is not None:
            a.g = _desc(g, head_first)
            a.g_dtype = _lib.LMOE_F32 if g.dtype == torch.float32 else _lib.LMOE_BF16
        a.h0 = ptr(h0)
        a.hs = hs.data_ptr()
        a.d_o = _desc(do, head_first)
        dht = None if dht is None else dht.float().contiguous()
        a.dht = ptr(dht)
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        a.dq, a.dk, a.dv = _desc(dq, head_first), _desc(dk, head_first), _desc(dv, head_first)
        dg = None
        if g is not None:
            dg = torch.empty(g.shape, dtype=torch.float32, device=q.device)
            a.dg = _desc(dg, head_first)
        dh0 = torch.empty_like(h0) if ctx.has_h0 else None
        a.dh0 = ptr(dh0)
        dhs = torch.empty_like(hs)
        a.dhs = dhs.data_ptr()
        norm_ws = None
        if ctx.norm_eps is not None:
            norm_eps = ctx.norm_eps
            norm_ws = torch.empty(max(plan.NT, 1), H, V // 32, 64 + K, dtype=torch.float32, device=q.device)
            a.norm_eps, a.zs, a.norm_ws = norm_eps, zs.data_ptr(), norm_ws.data_ptr()
            if ctx.emit_den:
                shape = (B, H, T) if head_first else (B, T, H)
                dden = torch.zeros(shape, dtype=torch.float32, device=q.device) if dden is None else dden.float().contiguous()
                a.normalize, a.dden = 2, _desc(dden, head_first)
            else:
                o = _aligned(o)
                a.normalize, a.den, a.o = 1, _desc(den, head_first), _desc(o, head_first)
        _lib.check(lib.lmoe_chunk_simple_gla_bwd(C.byref(a), stream_ptr()), "chunk_simple_gla backward")
        ctx.bwd_args = a
        ctx.bwd_keep = (do, dht, dq, dk, dv, dg, dh0, dhs, norm_ws, o, dden) if self.keep else None
        if dg is not None and dg.dtype != g.dtype:
            dg = dg.to(g.dtype)
        return dq, dk, dv, dg, dh0


class _ChunkSimpleGLA(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, g, scale, initial_state, output_final_state, cu_seqlens, head_first, norm_eps=None):
        call = SimpleGLACall()
        o, ht = call.forward(q, k, v, g, scale, initial_state, output_final_state, cu_seqlens, head_first,
                             save=any(ctx.needs_input_grad), norm_eps=norm_eps)
        ctx.call = call
        stash(ctx, call, o if norm_eps is not None else None)    # (the backward of the normalisation reads the output)
        return o, ht

    @staticmethod
    def backward(ctx, do, dht):
        (o,) = unstash(ctx, ctx.call)
        try:
            dq, dk, dv, dg, dh0 = ctx.call.backward(do, dht, o)
        finally:
            ctx.call.saved = None
        return dq, dk, dv, dg, None, dh0, None, None, None, None


class _ChunkSimpleGLAWithDen(torch.autograd.Function):
    """The ungated op with den = scale q_t . sum_{s<=t} k_s as a second output (nothing divided)."""

    @staticmethod
    def forward(ctx, q, k, v, scale, initial_state, output_final_state, cu_seqlens, head_first):
        call = SimpleGLACall()
        o, ht = call.forward(q, k, v, None, scale, initial_state, output_final_state, cu_seqlens, head_first,
                             save=any(ctx.needs_input_grad), emit_den=True)
        ctx.call = call
        den, call.den = call.den, None
        stash(ctx, call)
        return o, den, ht

    @staticmethod
    def backward(ctx, do, dden, dht):
        unstash(ctx, ctx.call)
        try:
            if do is None:
                v = ctx.call.saved[2]
                do = torch.zeros(v.shape, dtype=v.dtype, device=v.device)
            dq, dk, dv, _, dh0 = ctx.call.backward(do, dht, None, dden)
        finally:
            ctx.call.saved = None
        return dq, dk, dv, None, dh0, None, None, None


def chunk_simple_gla_with_den(q, k, v, scale=None, initial_state=None, output_final_state=False, cu_seqlens=None,
                              head_first=True):
    """The ungated op and, beside its (undivided) output, ``den_t = scale q_t . sum_{s<=t} k_s`` (fp32, ``[B,H,T]`` /
    ``[B,T,H]``): for ``chunk_linear_attn(normalize=True)`` over several key blocks, where the divisor is the sum of
    the blocks' den.  Differentiable in both outputs.  Returns ``(o, den, final_state)``."""
    if not can_normalize(q, v):
        raise ValueError("chunk_simple_gla_with_den: bfloat16 q, k, v with head dimensions of 64 or 128")
    return _ChunkSimpleGLAWithDen.apply(q, k, v, scale, initial_state, output_final_state, cu_seqlens, head_first)


def can_normalize(q, v, g=None) -> bool:
    """Whether ``chunk_simple_gla_normalized`` takes this call: ungated, bfloat16, head dimensions of 64 or 128."""
    return (g is None and q.dim() == 4 and v.dim() == 4 and q.dtype == torch.bfloat16
            and q.shape[-1] in HEAD_DIMS and v.shape[-1] in HEAD_DIMS)


def chunk_simple_gla_normalized(q, k, v, scale=None, initial_state=None, output_final_state=False, cu_seqlens=None,
                                head_first=True, eps: float = 1e-10):
    """The ungated op with the normaliser of ``fla.ops.linear_attn.chunk_linear_attn(normalize=True)`` inside the
    kernels: ``o_t = scale q_t S_t / (scale q_t . sum_{s<=t} k_s + eps)`` -- the sum of the keys is carried beside the
    state as one more column, nothing passes through memory between the op and the division, and the backward folds
    the gradient of the divisor into the sums it forms anyway.  ``initial_state`` seeds S only: the sum of the keys
    starts inside the call.  Returns ``(o, final_state)``."""
    if not can_normalize(q, v):
        raise ValueError("chunk_simple_gla_normalized: bfloat16 q, k, v with head dimensions of 64 or 128")
    r = no_tokens(q, k, v, head_first, cu_seqlens, initial_state, output_final_state)
    if r is not None:
        return r
    return _ChunkSimpleGLA.apply(q, k, v, None, scale, initial_state, output_final_state, cu_seqlens, head_first,
                                 float(eps))


def chunk_simple_gla(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: Optional[torch.Tensor] = None,
    scale: Optional[float] = None,
    initial_state: Optional[torch.Tensor] = None,
    output_final_state: bool = False,
    cu_seqlens: Optional[torch.Tensor] = None,
    head_first: bool = True,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """q, k: ``[B,H,T,K]``, v: ``[B,H,T,V]`` (``[B,T,H,*]`` with ``head_first=False``);
    g: ``[B,H,T]`` log-space decay or None.  Returns ``(o, final_state)`` with ``o`` shaped like
    ``v`` and ``final_state`` fp32 ``[N,H,K,V]`` or None.  K, V of 64 or 128 run as they are; any other size is
    padded / cut into such blocks (``_host.by_head_dim_blocks``)."""
    if q.dim() == 4 and v.dim() == 4 and (q.shape[-1] not in HEAD_DIMS or v.shape[-1] not in HEAD_DIMS):
        sc = q.shape[-1] ** -0.5 if scale is None else scale          # of the whole key, not of a block
        return by_head_dim_blocks(
            lambda q_, k_, v_, _g, h0: chunk_simple_gla(q_, k_, v_, g, sc, h0, output_final_state, cu_seqlens, head_first),
            q, k, v, None, initial_state, output_final_state, True, "chunk_simple_gla")
    r = no_tokens(q, k, v, head_first, cu_seqlens, initial_state, output_final_state)
    if r is not None:
        return r
    return _ChunkSimpleGLA.apply(q, k, v, g, scale, initial_state, output_final_state, cu_seqlens, head_first)
