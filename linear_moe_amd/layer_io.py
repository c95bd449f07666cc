"""The gated-delta-rule token mixer's prologue and epilogue around the chunk op, one pass each on MI355X.

``gdn_qkv_prologue`` stands where the reference splits its fused projection into q, k, v
(``linear_moe/sequence_modeling/linear_attention.py:159-163``), moves them to ``[B, T, H, D]``, applies SiLU to all
three and the L2 norm to q and k (``gated_deltanet/gated_deltanet.py:99, 101, 105-106``): three strided copies, an
elementwise kernel and two row kernels become one kernel that reads the projection once and writes the three tensors
the op reads.  ``swish_gate_relayout`` stands where the op's output goes back to ``[T, B, H D]``
(``gated_deltanet.py:114``) and is multiplied by ``swish(o_gate)`` (``linear_attention.py:255``).
"""
from __future__ import annotations

import torch

from . import _lib
from ._host import stash, stream_ptr, unstash


def _dt(x):
    if not x.is_cuda:
        raise RuntimeError("linear_moe_amd ops are GPU only (no CPU fallback)")
    if x.dtype not in (torch.bfloat16, torch.float32):
        raise ValueError(f"dtype {x.dtype} unsupported (bfloat16 or float32)")
    return _lib.LMOE_F32 if x.dtype == torch.float32 else _lib.LMOE_BF16


class _QKVPrologue(torch.autograd.Function):
    @staticmethod
    def forward(ctx, qkv, H, D, eps):
        dt = _dt(qkv)
        if qkv.dim() != 3 and qkv.dim() != 4:
            raise ValueError("gdn_qkv_prologue: qkv must be [T, B, H * 3 * D] or [T, B, H, 3 * D]")
        T, B = qkv.shape[0], qkv.shape[1]
        if qkv.numel() != T * B * H * 3 * D:
            raise ValueError(f"gdn_qkv_prologue: {tuple(qkv.shape)} is not [T, B, {H} heads x 3 x {D}]")
        if D not in (64, 128):
            raise ValueError(f"gdn_qkv_prologue: head dimension {D} unsupported (64 or 128)")
        lib = _lib.load()
        x = qkv.contiguous()
        q, k, v = (torch.empty(B, T, H, D, dtype=qkv.dtype, device=qkv.device) for _ in range(3))
        _lib.check(lib.lmoe_gdn_qkv_prologue_fwd(x.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), T, B, H, D, dt, eps,
                                                 stream_ptr()), "gdn_qkv_prologue")
        ctx.save_for_backward(x)
        ctx.dims, ctx.eps, ctx.dt, ctx.shape = (T, B, H, D), eps, dt, qkv.shape
        return q, k, v

    @staticmethod
    def backward(ctx, dq, dk, dv):
        (x,) = ctx.saved_tensors
        T, B, H, D = ctx.dims
        lib = _lib.load()
        dq, dk, dv = (torch.zeros(B, T, H, D, dtype=x.dtype, device=x.device) if g is None else g.contiguous()
                      for g in (dq, dk, dv))
        dx = torch.empty_like(x)
        _lib.check(lib.lmoe_gdn_qkv_prologue_bwd(x.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), dx.data_ptr(),
                                                 T, B, H, D, ctx.dt, ctx.eps, stream_ptr()), "gdn_qkv_prologue backward")
        return dx.view(ctx.shape), None, None, None


class _GDNMixerCore(torch.autograd.Function):
    """Prologue and op as one node of the graph, so that the gradient of the projection is one buffer that the op's
    backward (v block) and the prologue's backward (q and k blocks) fill in place."""

    @staticmethod
    def forward(ctx, qkv, g, beta, H, D, eps, scale):
        from .gated_delta_rule import GDNCall
        dt = _dt(qkv)
        if dt != _lib.LMOE_BF16:
            raise ValueError("gdn_mixer_core: bfloat16 only (the op applies SiLU to v in its 2-byte kernels)")
        T, B = qkv.shape[0], qkv.shape[1]
        if qkv.dim() not in (3, 4) or qkv.numel() != T * B * H * 3 * D:
            raise ValueError(f"gdn_mixer_core: {tuple(qkv.shape)} is not [T, B, {H} heads x 3 x {D}]")
        if D not in (64, 128):
            raise ValueError(f"gdn_mixer_core: head dimension {D} unsupported (64 or 128)")
        lib = _lib.load()
        x = qkv.contiguous()
        q, k = (torch.empty(B, T, H, D, dtype=qkv.dtype, device=qkv.device) for _ in range(2))
        _lib.check(lib.lmoe_gdn_qkv_prologue_fwd(x.data_ptr(), q.data_ptr(), k.data_ptr(), None, T, B, H, D, dt, eps,
                                                 stream_ptr()), "gdn_mixer_core prologue")
        v = x.view(T, B, H, 3 * D)[..., 2 * D:].transpose(0, 1)            # [B, T, H, D], strided: the op reads it in place
        call = GDNCall()
        o, _ = call.forward(q, k, v, g, beta, scale, None, False, None, False,
                            save=any(ctx.needs_input_grad[:3]), v_act=True)
        ctx.call = call
        stash(ctx, call, x)
        ctx.dims, ctx.eps, ctx.dt, ctx.shape = (T, B, H, D), eps, dt, qkv.shape
        return o

    @staticmethod
    def backward(ctx, do):
        T, B, H, D = ctx.dims
        (x,) = unstash(ctx, ctx.call)
        # the op writes all three blocks of the projection's gradient itself: dv as silu'(v) times its dv, dq and dk
        # through the backward of the L2 norm and of SiLU, applied to its dq, dk tiles on their way out, from the raw
        # rows of the projection
        dx = torch.empty_like(x)
        blocks = lambda t: [t.view(T, B, H, 3 * D)[..., i * D:(i + 1) * D].transpose(0, 1) for i in range(3)]
        dxq, dxk, dxv = blocks(dx)
        xq, xk, _ = blocks(x)
        try:
            _, _, _, dg, dbeta, _ = ctx.call.backward(do, None, dv_out=dxv, dq_out=dxq, dk_out=dxk, qk_raw=(xq, xk),
                                                      qk_eps=ctx.eps)
        finally:
            ctx.call.saved = None
        return dx.view(ctx.shape), dg, dbeta, None, None, None, None


def gdn_mixer_core(qkv: torch.Tensor, g: torch.Tensor, beta: torch.Tensor, num_heads: int, head_dim: int,
                   eps: float = 1e-6, scale=None) -> torch.Tensor:
    """``gdn_qkv_prologue`` and ``chunk_gated_delta_rule(..., head_first=False)`` in one call (bfloat16): q^ and k^ are
    written as by the prologue, v is never written -- the op reads the v block of ``qkv`` in place and applies SiLU
    where it stages it.  The backward is the op's alone: it writes ``silu'(v)`` times its dv straight into the v block
    of the projection's gradient and sends its dq, dk through the backward of the L2 norm and of SiLU on their way
    into the q and k blocks (no pass of the prologue's own).  ``g``, ``beta``: ``[B, T, H]``.
    Returns o ``[B, T, H, D]``, the bits of the two-call path."""
    return _GDNMixerCore.apply(qkv, g, beta, num_heads, head_dim, eps, scale)


def gdn_qkv_prologue(qkv: torch.Tensor, num_heads: int, head_dim: int, eps: float = 1e-6):
    """``qkv`` ``[T, B, H * 3 D]`` (per head q | k | v) -> ``l2norm(silu(q))``, ``l2norm(silu(k))``, ``silu(v)``,
    each ``[B, T, H, D]`` contiguous: the inputs of ``chunk_gated_delta_rule(..., head_first=False)``."""
    return _QKVPrologue.apply(qkv, num_heads, head_dim, eps)


class _SwishGateRelayout(torch.autograd.Function):
    @staticmethod
    def forward(ctx, o, gate):
        dt = _dt(o)
        if o.dim() != 4:
            raise ValueError("swish_gate_relayout: o must be [B, T, H, D]")
        B, T, H, D = o.shape
        W = H * D
        if gate.dtype != o.dtype or gate.numel() != o.numel() or gate.shape[0] != T or gate.shape[1] != B:
            raise ValueError(f"swish_gate_relayout: gate must be [T, B, H * D] = [{T}, {B}, {W}] in the dtype of o")
        if W % 8:
            raise ValueError("swish_gate_relayout: H * D must be a multiple of 8")
        lib = _lib.load()
        oc, gc = o.contiguous(), gate.contiguous()
        y = torch.empty(T, B, W, dtype=o.dtype, device=o.device)
        _lib.check(lib.lmoe_swish_gate_relayout_fwd(oc.data_ptr(), gc.data_ptr(), y.data_ptr(), T, B, W, dt, stream_ptr()),
                   "swish_gate_relayout")
        ctx.save_for_backward(oc, gc)
        ctx.dims, ctx.dt, ctx.gshape = (T, B, W), dt, gate.shape
        return y

    @staticmethod
    def backward(ctx, dy):
        oc, gc = ctx.saved_tensors
        T, B, W = ctx.dims
        lib = _lib.load()
        dyc = dy.contiguous()
        do, dgate = torch.empty_like(oc), torch.empty_like(gc)
        _lib.check(lib.lmoe_swish_gate_relayout_bwd(oc.data_ptr(), gc.data_ptr(), dyc.data_ptr(), do.data_ptr(),
                                                    dgate.data_ptr(), T, B, W, ctx.dt, stream_ptr()),
                   "swish_gate_relayout backward")
        return do, dgate.view(ctx.gshape)


def swish_gate_relayout(o: torch.Tensor, o_gate: torch.Tensor) -> torch.Tensor:
    """``o`` ``[B, T, H, D]`` (the op's output), ``o_gate`` ``[T, B, H D]`` -> ``[T, B, H D]``:
    ``rearrange(o, 'b n h d -> n b (h d)') * swish(o_gate)``."""
    return _SwishGateRelayout.apply(o, o_gate)
