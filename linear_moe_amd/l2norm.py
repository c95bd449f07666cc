"""Row-wise L2 normalisation on MI355X: ``y = x / sqrt(sum x^2 + eps)`` over the last dimension.

Stands where the reference's token mixers call ``l2_norm_fn`` on q and k
(``linear_moe/model/common_modules/l2norm.py:172-201``, used at
``linear_moe/sequence_modeling/gated_deltanet/gated_deltanet.py:105-106``) and where
flash-linear-attention's ``use_qk_l2norm_in_kernel`` normalises them in front of its kernels.
"""
from __future__ import annotations

import torch

from . import _lib
from ._host import stream_ptr

_DIMS = (64, 128, 256)


class _L2Norm(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, eps, silu=False):
        if not x.is_cuda:
            raise RuntimeError("linear_moe_amd ops are GPU only (no CPU fallback)")
        if x.dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"l2_norm: dtype {x.dtype} unsupported (bfloat16 or float32)")
        D = x.shape[-1]
        if D not in _DIMS:
            raise ValueError(f"l2_norm: last dimension {D} unsupported {_DIMS}")
        lib = _lib.load()
        xc = x.contiguous()
        y = torch.empty_like(xc)
        dt = _lib.LMOE_F32 if x.dtype == torch.float32 else _lib.LMOE_BF16
        fwd = lib.lmoe_silu_l2norm_fwd if silu else lib.lmoe_l2norm_fwd
        _lib.check(fwd(xc.data_ptr(), y.data_ptr(), xc.numel() // D, D, dt, eps, stream_ptr()), "l2_norm")
        ctx.save_for_backward(xc)
        ctx.eps, ctx.dt, ctx.silu = eps, dt, silu
        return y

    @staticmethod
    def backward(ctx, dy):
        (xc,) = ctx.saved_tensors
        lib = _lib.load()
        D = xc.shape[-1]
        dyc = dy.contiguous()
        dx = torch.empty_like(xc)
        bwd = lib.lmoe_silu_l2norm_bwd if ctx.silu else lib.lmoe_l2norm_bwd
        _lib.check(bwd(xc.data_ptr(), dyc.data_ptr(), dx.data_ptr(), xc.numel() // D, D, ctx.dt, ctx.eps, stream_ptr()),
                   "l2_norm backward")
        return dx, None, None


def l2_norm(x: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    return _L2Norm.apply(x, eps)


def silu_l2_norm(x: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """``l2_norm(silu(x))`` in one pass: what the reference does to q and k of the gated delta rule in two
    (``linear_moe/sequence_modeling/gated_deltanet/gated_deltanet.py:101`` then ``:105-106``)."""
    return _L2Norm.apply(x, eps, True)


l2_norm_fn = l2_norm
