"""RMS norm of the op's output rows on MI355X, optionally fused with the swish output gate.

Stands where the reference's token mixers normalise the output of the chunk op,
``self.la_output_norm(output)`` with ``RMSNorm(head_v_dim)``
(``linear_moe/sequence_modeling/gla/gla.py:95``, ``retention/retention.py:92``; module
``linear_moe/model/common_modules/layernorm.py:626-666`` -> ``rms_norm_fn`` ``:515-537``), and, with
``gate``, where ``LinearAttention.forward`` multiplies by ``swish(o_gate)``
(``linear_moe/sequence_modeling/linear_attention.py:255``): one pass over the rows instead of two.
"""
from __future__ import annotations

import torch
from torch import nn

from . import _lib
from ._host import stream_ptr

_DIMS = (64, 128, 256)


class _RMSNorm(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, gate, eps):
        if not x.is_cuda:
            raise RuntimeError("linear_moe_amd ops are GPU only (no CPU fallback)")
        if x.dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"rms_norm: dtype {x.dtype} unsupported (bfloat16 or float32)")
        D = x.shape[-1]
        if D not in _DIMS:
            raise ValueError(f"rms_norm: last dimension {D} unsupported {_DIMS}")
        if weight is not None and (weight.shape != (D,) or not weight.is_cuda):
            raise ValueError(f"rms_norm: weight must be a GPU tensor of shape ({D},)")
        if gate is not None and (gate.shape != x.shape or gate.dtype != x.dtype):
            raise ValueError("rms_norm: gate must have the shape and dtype of x")
        lib = _lib.load()
        xc = x.contiguous()
        wc = None if weight is None else weight.detach().to(x.dtype).contiguous()
        gc = None if gate is None else gate.contiguous()
        y = torch.empty_like(xc)
        dt = _lib.LMOE_F32 if x.dtype == torch.float32 else _lib.LMOE_BF16
        rows = xc.numel() // D
        if rows:
            _lib.check(lib.lmoe_rmsnorm_fwd(xc.data_ptr(), None if wc is None else wc.data_ptr(),
                                            None if gc is None else gc.data_ptr(), y.data_ptr(), None, rows, D, dt, eps,
                                            stream_ptr()), "rms_norm")
        ctx.save_for_backward(xc, wc, gc)
        ctx.eps, ctx.dt, ctx.wdtype = eps, dt, None if weight is None else weight.dtype
        return y

    @staticmethod
    def backward(ctx, dy):
        xc, wc, gc = ctx.saved_tensors
        lib = _lib.load()
        D = xc.shape[-1]
        rows = xc.numel() // D
        dyc = dy.contiguous()
        dx = torch.empty_like(xc)
        dgate = None if gc is None else torch.empty_like(gc)
        dw = None
        if wc is not None and ctx.needs_input_grad[1]:
            dw = torch.zeros(D, dtype=torch.float32, device=xc.device)
        if rows:
            part = None
            if dw is not None:
                part = torch.empty(lib.lmoe_rmsnorm_partials(rows, D, ctx.dt), D, dtype=torch.float32, device=xc.device)
            _lib.check(lib.lmoe_rmsnorm_bwd(xc.data_ptr(), None if wc is None else wc.data_ptr(),
                                            None if gc is None else gc.data_ptr(), dyc.data_ptr(), dx.data_ptr(),
                                            None if dgate is None else dgate.data_ptr(),
                                            None if part is None else part.data_ptr(),
                                            None if dw is None else dw.data_ptr(), rows, D, ctx.dt, ctx.eps, stream_ptr()),
                       "rms_norm backward")
        return dx, (None if dw is None else dw.to(ctx.wdtype)), dgate, None


def rms_norm_fn(x, weight, bias=None, residual=None, eps: float = 1e-6, prenorm: bool = False,
                residual_in_fp32: bool = False):
    """Signature of the reference's ``rms_norm_fn`` (layernorm.py:515-537).  The options its token
    mixers never use on this path (bias, residual, prenorm) are rejected rather than emulated."""
    if bias is not None or residual is not None or prenorm:
        raise NotImplementedError("rms_norm_fn: bias / residual / prenorm are outside the output-norm path")
    return _RMSNorm.apply(x, weight, None, eps)


def rms_norm_swish_gate(x, gate, weight=None, eps: float = 1e-5):
    """``rms_norm(x) * weight * gate * sigmoid(gate)`` in one pass (forward and backward)."""
    return _RMSNorm.apply(x, weight, gate, eps)


class RMSNorm(nn.Module):
    """Constructor and forward of the reference's ``RMSNorm`` (layernorm.py:626-666)."""

    def __init__(self, hidden_size: int, elementwise_affine: bool = True, bias: bool = False, eps: float = 1e-5):
        super().__init__()
        if bias:
            raise NotImplementedError("RMSNorm: bias is outside the output-norm path")
        self.hidden_size, self.elementwise_affine, self.eps = hidden_size, elementwise_affine, eps
        self.register_parameter("weight", None)
        self.register_parameter("bias", None)
        if elementwise_affine:
            self.weight = nn.Parameter(torch.ones(hidden_size))

    def forward(self, x, residual=None, prenorm=False, residual_in_fp32=False):
        return rms_norm_fn(x, self.weight, self.bias, residual=residual, eps=self.eps, prenorm=prenorm,
                           residual_in_fp32=residual_in_fp32)
