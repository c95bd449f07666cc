"""Quadratic feature maps of Based and ReBased on MI355X, written straight into the key blocks the chunk
kernels take.

The reference expands q and k of head dimension D into ``1 + D + D(D+1)/2`` (Based, ``TaylorFeatureMap``,
``linear_moe/model/common_modules/feature_map.py:190-203``) or ``D(D+1)/2`` (ReBased, ``RebasedFeatureMap``,
``:206-246``) features and calls ``chunk_linear_attn(q, k, v, normalize=True, scale=1)``
(``linear_moe/sequence_modeling/based/based.py:68-69``, ``.../rebased/rebased.py:72-76``).  The feature count
(153 / 136 for D = 16) is no head dimension of the kernels, and linear attention without decay is a sum over
key blocks, so the maps here return a :class:`KeyBlocks`: the features zero-padded to a multiple of 64 and split
into contiguous blocks of 128 (the last one possibly 64) columns, which ``chunk_linear_attn`` sums over.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import _lib
from ._host import stream_ptr


class KeyBlocks(tuple):
    """Tuple of contiguous ``[..., T, width]`` tensors (widths 128, ..., 128, then 128 or 64) that together hold
    ``features`` feature columns followed by zero padding."""

    features: int

    def __new__(cls, blocks, features):
        self = super().__new__(cls, blocks)
        self.features = features
        return self

    def dense(self) -> torch.Tensor:
        """The unpadded ``[..., T, features]`` tensor (a copy; for tests and for callers that want fla's layout)."""
        return torch.cat(tuple(self), dim=-1)[..., :self.features]


def _widths(Kp: int):
    w = [128] * (Kp // 128)
    if Kp % 128:
        w.append(64)
    return w


class _QuadFeatureMap(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, c0, c1, cd, co):
        if not x.is_cuda:
            raise RuntimeError("linear_moe_amd ops are GPU only (no CPU fallback)")
        if x.dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"feature map: dtype {x.dtype} unsupported (bfloat16 or float32)")
        D = x.shape[-1]
        if D not in (8, 16, 32):
            raise ValueError(f"feature map: head dimension {D} unsupported (8, 16 or 32)")
        lib = _lib.load()
        xc = x.contiguous()
        rows = xc.numel() // D
        F = lib.lmoe_quad_featmap_features(D, c0, c1)
        Kp = -(-F // 64) * 64
        dt = _lib.LMOE_F32 if x.dtype == torch.float32 else _lib.LMOE_BF16
        buf = torch.empty(rows * Kp, dtype=x.dtype, device=x.device)
        _lib.check(lib.lmoe_quad_featmap_fwd(xc.data_ptr(), buf.data_ptr(), rows, D, Kp, c0, c1, cd, co, dt, stream_ptr()),
                   "quad_feature_map")
        ctx.save_for_backward(xc)
        ctx.args = (D, Kp, c0, c1, cd, co, dt)
        blocks, off = [], 0
        for w in _widths(Kp):
            blocks.append(buf[off:off + rows * w].view(*x.shape[:-1], w))
            off += rows * w
        ctx.nblocks = len(blocks)
        return tuple(blocks)

    @staticmethod
    def backward(ctx, *dblocks):
        (xc,) = ctx.saved_tensors
        D, Kp, c0, c1, cd, co, dt = ctx.args
        lib = _lib.load()
        rows = xc.numel() // D
        dy = torch.empty(rows * Kp, dtype=xc.dtype, device=xc.device)
        off = 0
        for w, d in zip(_widths(Kp), dblocks):
            part = dy[off:off + rows * w].view(*xc.shape[:-1], w)
            if d is None:
                part.zero_()
            else:
                part.copy_(d)
            off += rows * w
        dx = torch.empty_like(xc)
        _lib.check(lib.lmoe_quad_featmap_bwd(xc.data_ptr(), dy.data_ptr(), dx.data_ptr(), rows, D, Kp, c0, c1, cd, co, dt,
                                             stream_ptr()), "quad_feature_map backward")
        return dx, None, None, None, None


def quad_feature_map(x: torch.Tensor, c0: float, c1: float, cd: float, co: float) -> KeyBlocks:
    """``[c0 | c1 x_i | cd x_i^2 | co x_i x_j (i < j)]`` over the last dimension of x as key blocks."""
    D = x.shape[-1]
    feats = (1 if c0 else 0) + (D if c1 else 0) + D * (D + 1) // 2
    return KeyBlocks(_QuadFeatureMap.apply(x, float(c0), float(c1), float(cd), float(co)), feats)


def taylor_feature_map(x: torch.Tensor) -> KeyBlocks:
    """Based: ``phi(q) . phi(k) = 1 + s + s^2 / 2`` with ``s = q . k / sqrt(D)``."""
    D = x.shape[-1]
    return quad_feature_map(x, 1.0, D ** -0.25, (2.0 * D) ** -0.5, D ** -0.5)


def rebased_feature_map(x: torch.Tensor, gamma: Optional[torch.Tensor] = None, beta: Optional[torch.Tensor] = None,
                        normalize: bool = True, eps: float = 1e-6) -> KeyBlocks:
    """ReBased: ``phi(q) . phi(k) = (q' . k')^2 / D`` for ``x' = gamma * norm(x) + beta``.  The D-wide layer norm /
    affine in front is torch's (``feature_map.py:229-240``); the expansion is the kernel."""
    D = x.shape[-1]
    if normalize:
        x = torch.nn.functional.layer_norm(x, (D,), gamma, beta, eps)
    elif gamma is not None and beta is not None:
        x = torch.addcmul(beta, x, gamma)
    elif gamma is not None:
        x = x * gamma
    else:
        raise RuntimeError("rebased_feature_map: needs normalize=True or gamma")
    return quad_feature_map(x, 0.0, 0.0, D ** -0.5, (2.0 / D) ** 0.5)
