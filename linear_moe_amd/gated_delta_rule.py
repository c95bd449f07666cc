"""``chunk_gated_delta_rule`` on MI355X.

  S~_t = e^{g_t} S_{t-1};  S_t = S~_t + k_t^T beta_t (v_t - k_t S~_t);  o_t = scale q_t S_t

Keeps flash-linear-attention's call signature as the reference uses it at
``linear_moe/sequence_modeling/gated_deltanet/gated_deltanet.py:112``:
``chunk_gated_delta_rule(q, k, v, g, beta, head_first=False)`` with q, k, v ``[B,T,H,D]`` and
g, beta ``[B,T,H]``.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Tuple

import torch

from . import _lib
from .l2norm import l2_norm
from ._host import (HEAD_DIMS, WIDE_V, seq_plan, _aligned, _check_inputs, _desc, _state_check, base_args, by_head_dim_blocks,
                    no_tokens, ptr, stash, stream_ptr, unstash)


def _scalar_dt(x: torch.Tensor) -> int:
    return _lib.LMOE_F32 if x.dtype == torch.float32 else _lib.LMOE_BF16


class GDNCall:
    """One call of the op: owns the argument blocks and every buffer the kernels touch.
    The autograd function and the benchmark harness (per-kernel timing through
    ``lmoe_launch_stage``) both drive the kernels through this object."""

    OP = 2  # LMOE_OP_GATED_DELTA_RULE

    def __init__(self, keep: bool = False):
        # keep=True (benchmark harness) also pins outputs and gradients so that the argument
        # blocks stay valid for lmoe_launch_stage; the autograd path must not (reference cycle)
        self.keep = keep

    def forward(self, q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens, head_first, save=True,
                v_act=False):
        """save=False: a forward-only call (nothing requires a gradient): what only the backward reads (the
        per-chunk states, v_new, Tinv) is neither allocated nor written.
        v_act: v is the argument of the SiLU in front of the op (bfloat16 only): the kernels apply it where they
        read v, and ``backward`` returns the gradient with respect to that argument."""
        ctx = self
        lib = _lib.load()
        dims = _check_inputs(q, k, v, head_first, cu_seqlens, wide_v=True)
        B, T, H, K, V = dims
        q, k, v = _aligned(q), _aligned(k), _aligned(v)
        plan = seq_plan(B, T, cu_seqlens, q.device)
        want = (B, H, T) if head_first else (B, T, H)
        if beta is None or tuple(beta.shape) != want:
            raise ValueError(f"beta must have shape {want}")
        if g is not None and tuple(g.shape) != want:
            raise ValueError(f"g must have shape {want}, got {tuple(g.shape)}")
        if g is not None and g.dtype not in (torch.float32, torch.bfloat16):
            g = g.float()
        if beta.dtype not in (torch.float32, torch.bfloat16):
            beta = beta.float()
        h0 = _state_check(initial_state, plan.N, H, K, V, "initial_state")
        a = base_args(q, k, v, head_first, scale, plan, dims)
        a.gate = _lib.GATE_NONE if g is None else _lib.GATE_SCALAR
        if g is not None:
            a.g, a.g_dtype = _desc(g, head_first), _scalar_dt(g)
        a.beta, a.beta_dtype = _desc(beta, head_first), _scalar_dt(beta)
        a.h0 = ptr(h0)
        dev, dt = q.device, q.dtype
        # (v_act: v is a block of a wider tensor; o is a tensor of its own)
        o = torch.empty(v.shape, dtype=dt, device=dev) if v_act else torch.empty_like(v)
        ht = torch.empty(plan.N, H, K, V, dtype=torch.float32, device=dev) if output_final_state else None
        hs = torch.empty(max(plan.NT, 1), H, K, V, dtype=dt, device=dev) if save else None
        # always: the backward reads it, and the forward state pass forms w from it (8 KB per chunk and head)
        tinv = torch.empty(max(plan.NT, 1), H, 64, 64, dtype=dt, device=dev)
        # P: the bf16 forward pass forms it on the chip and stores it only for the backward
        pmat = torch.empty(max(plan.NT, 1), H, 64, 64, dtype=dt, device=dev) if (save or dt == torch.float32) else None
        gcum = torch.empty(max(plan.NT, 1), H, 5, 64, dtype=torch.float32, device=dev)
        # w, u: the bf16 state passes form them on the chip from tinv; only the fp32 forward pass reads them
        w = torch.empty(B, T, H, K, dtype=dt, device=dev) if dt == torch.float32 else None
        u = torch.empty(B, T, H, V, dtype=dt, device=dev) if dt == torch.float32 else None
        # library-side layout [chunk, head, 32-column slice, token in chunk, column] (see include/lmoe.h)
        vnew = torch.empty(max(plan.NT, 1), H, V // 32, 64, 32, dtype=dt, device=dev) if save else None
        a.o, a.ht, a.hs, a.tinv = _desc(o, head_first), ptr(ht), ptr(hs), ptr(tinv)
        a.pmat, a.gcum = ptr(pmat), gcum.data_ptr()
        a.w, a.u = _desc(w, False), _desc(u, False)
        a.vnew.ptr = ptr(vnew)
        if v_act and dt != torch.bfloat16:
            raise ValueError("v_act exists for bfloat16")
        a.v_act = int(bool(v_act))
        ctx.v_act = bool(v_act)
        _lib.check(lib.lmoe_chunk_gated_delta_rule_fwd(C.byref(a), stream_ptr()), "chunk_gated_delta_rule forward")
        ctx.saved = (q, k, v, g, beta, h0, hs, tinv, pmat, gcum, vnew)
        ctx.fwd_args, ctx.fwd_keep = a, ((o, ht, w, u) if self.keep else None)
        ctx.plan, ctx.dims, ctx.head_first, ctx.scale = plan, dims, head_first, scale
        ctx.has_h0 = initial_state is not None
        return o, ht

    def backward(self, do, dht, dv_out=None, dq_out=None, dk_out=None, qk_raw=None, qk_eps=1e-6):
        """dv_out, dq_out, dk_out: where the gradients go (tensors of the shapes of v, q, k, any strides the kernels
        take: e.g. the blocks of the gradient of a fused projection); default: new tensors.  qk_raw = (q_raw, k_raw)
        (bfloat16): q and k of the forward were l2norm(silu(.)) of these rows (eps qk_eps inside the root), and dq,
        dk are returned with respect to them."""
        ctx = self
        lib = _lib.load()
        q, k, v, g, beta, h0, hs, tinv, pmat, gcum, vnew = ctx.saved
        plan, dims, head_first = ctx.plan, ctx.dims, ctx.head_first
        B, T, H, K, V = dims
        do = _aligned(do)
        a = base_args(q, k, v, head_first, ctx.scale, plan, dims)
        a.gate = _lib.GATE_NONE if g is None else _lib.GATE_SCALAR
        if g is not None:
            a.g, a.g_dtype = _desc(g, head_first), _scalar_dt(g)
        a.beta, a.beta_dtype = _desc(beta, head_first), _scalar_dt(beta)
        a.h0, a.hs, a.tinv, a.pmat = ptr(h0), hs.data_ptr(), tinv.data_ptr(), pmat.data_ptr()
        a.gcum = gcum.data_ptr()
        a.vnew.ptr = vnew.data_ptr()
        a.d_o = _desc(do, head_first)
        dht = None if dht is None else dht.float().contiguous()
        a.dht = ptr(dht)
        dev, dt = q.device, q.dtype
        dq = torch.empty_like(q) if dq_out is None else dq_out
        dk = torch.empty_like(k) if dk_out is None else dk_out
        dv = torch.empty_like(v) if dv_out is None else dv_out
        for n, t, like in (("dq_out", dq, q), ("dk_out", dk, k), ("dv_out", dv, v)):
            if t.shape != like.shape or t.dtype != dt or _aligned(t) is not t:
                raise ValueError(f"{n} must have the shape and dtype of its input, 16-byte aligned rows, a contiguous "
                                 "last dimension")
        a.dq, a.dk, a.dv = _desc(dq, head_first), _desc(dk, head_first), _desc(dv, head_first)
        a.v_act = int(ctx.v_act)
        if qk_raw is not None:
            q_raw, k_raw = qk_raw
            if dt != torch.bfloat16:
                raise ValueError("qk_raw exists for bfloat16")
            for t, like in ((q_raw, q), (k_raw, k)):
                if t.shape != like.shape or t.dtype != dt or _aligned(t) is not t:
                    raise ValueError("qk_raw: the shapes and dtype of q, k, 16-byte aligned rows, a contiguous last dimension")
            a.q_raw, a.k_raw, a.qk_eps = _desc(q_raw, head_first), _desc(k_raw, head_first), float(qk_eps)
        dg = torch.empty(beta.shape, dtype=torch.float32, device=dev)
        dbeta = torch.empty(beta.shape, dtype=torch.float32, device=dev)
        a.dg, a.dbeta = _desc(dg, head_first), _desc(dbeta, head_first)
        dh0 = torch.empty_like(h0) if ctx.has_h0 else None
        a.dh0 = ptr(dh0)
        dhs = torch.empty_like(hs)
        dvnew = torch.empty_like(vnew)
        a.dhs = dhs.data_ptr()
        a.dvnew.ptr = dvnew.data_ptr()
        _lib.check(lib.lmoe_chunk_gated_delta_rule_bwd(C.byref(a), stream_ptr()), "chunk_gated_delta_rule backward")
        ctx.bwd_args = a
        ctx.bwd_keep = (do, dht, dq, dk, dv, dg, dbeta, dh0, dhs, dvnew, qk_raw) if self.keep else None
        dg = None if g is None else dg.to(g.dtype)
        return dq, dk, dv, dg, dbeta.to(beta.dtype), dh0


class _ChunkGatedDeltaRule(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens, head_first):
        call = GDNCall()
        o, ht = call.forward(q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens, head_first,
                             save=any(ctx.needs_input_grad))
        ctx.call = call
        stash(ctx, call)
        return o, ht

    @staticmethod
    def backward(ctx, do, dht):
        unstash(ctx, ctx.call)
        try:
            dq, dk, dv, dg, dbeta, dh0 = ctx.call.backward(do, dht)
        finally:
            ctx.call.saved = None
        return dq, dk, dv, dg, dbeta, None, dh0, None, None, None


def chunk_gated_delta_rule(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: torch.Tensor,
    beta: torch.Tensor,
    scale: Optional[float] = None,
    initial_state: Optional[torch.Tensor] = None,
    output_final_state: bool = False,
    cu_seqlens: Optional[torch.Tensor] = None,
    head_first: bool = False,
    use_qk_l2norm_in_kernel: bool = False,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """q, k: ``[B,T,H,K]``, v: ``[B,T,H,V]``, g (log-space decay) and beta: ``[B,T,H]``
    (``[B,H,T,*]`` with ``head_first=True``).  Returns ``(o, final_state)``.  K, V of 64 or 128 and K = 128 with
    V = 256 (``expand_v = 2``) run as they are; a smaller K is zero-padded, any other V is cut into blocks of
    256 (K > 64) / 128 / 64 columns (``_host.by_head_dim_blocks``).

    ``use_qk_l2norm_in_kernel=True`` gives the results of fla's flag, not its fusion: q and k go through the ``l2_norm``
    kernel (one read and one write of each, forward and backward) in front of the op, the op's kernels do not
    normalise.  A caller that holds the fused projection of the mixer gets q^, k^ and silu(v) in one pass from
    ``layer_io.gdn_qkv_prologue`` instead."""
    if use_qk_l2norm_in_kernel:
        q = l2_norm(q)
        k = l2_norm(k)
    if q.dim() == 4 and v.dim() == 4 and (q.shape[-1] not in HEAD_DIMS or v.shape[-1] not in HEAD_DIMS) \
            and (q.shape[-1], v.shape[-1]) != WIDE_V:
        # e.g. K = 96 (padded to 128), V = 320 (a block of 256 and one of 64 columns)
        sc = q.shape[-1] ** -0.5 if scale is None else scale          # of the whole key, not of the padded one
        return by_head_dim_blocks(
            lambda q_, k_, v_, _g, h0: chunk_gated_delta_rule(q_, k_, v_, g, beta, sc, h0, output_final_state,
                                                              cu_seqlens, head_first),
            q, k, v, None, initial_state, output_final_state, False, "chunk_gated_delta_rule", wide_v=True)
    r = no_tokens(q, k, v, head_first, cu_seqlens, initial_state, output_final_state, wide_v=True)
    if r is not None:
        return r
    return _ChunkGatedDeltaRule.apply(q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens,
                                      head_first)
