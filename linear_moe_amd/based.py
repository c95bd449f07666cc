"""``parallel_based`` / ``parallel_rebased``: causal attention with the polynomial weights ``1 + s + s^2/2``
(Based) and ``s^2`` (ReBased), ``s = scale * q . k``, evaluated as linear attention over the quadratic feature
maps (the weights are exactly ``phi(q) . phi(k)``), i.e. through ``chunk_linear_attn`` over key blocks.

Called by the reference as ``parallel_based(q, k, v, True, True)``
(``linear_moe/sequence_modeling/based/based.py:72``) and ``parallel_rebased(q, k, v, eps, True, True)``
(``linear_moe/sequence_modeling/rebased/rebased.py:79``), q, k ``[B, H, T, D]`` with D <= 128 there; here D in
{8, 16, 32} (the feature count grows as D^2 / 2).  The normaliser's epsilon is the one argument / default of
these calls; what fla's kernels do beyond the formula above is not checkable offline.
"""
from __future__ import annotations

import torch

from .feature_map import quad_feature_map
from .linear_attn import chunk_linear_attn


def _poly_attn(q, k, v, c0, c1, c2, scale, use_normalize, eps):
    # weights c0 + c1 s + c2 s^2 with s = scale q.k:  phi = [sqrt(c0) | sqrt(c1 scale) x | sqrt(c2) scale x_i^2 |
    # sqrt(2 c2) scale x_i x_j]
    fm = lambda x: quad_feature_map(x, c0 ** 0.5, (c1 * scale) ** 0.5, c2 ** 0.5 * scale, (2.0 * c2) ** 0.5 * scale)
    qb, kb = fm(q), fm(k)
    # (the normaliser is one more value column inside the kernels: chunk_linear_attn)
    o, _ = chunk_linear_attn(qb, kb, v, scale=1.0, normalize=use_normalize, _eps=eps)
    return o.to(v.dtype)


def parallel_based(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, use_scale: bool = True,
                   use_normalize: bool = True, eps: float = 1e-6) -> torch.Tensor:
    scale = q.shape[-1] ** -0.5 if use_scale else 1.0
    return _poly_attn(q, k, v, 1.0, 1.0, 0.5, scale, use_normalize, eps)


def parallel_rebased(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, eps: float = 1e-5, use_scale: bool = True,
                     use_normalize: bool = True) -> torch.Tensor:
    scale = q.shape[-1] ** -0.5 if use_scale else 1.0
    return _poly_attn(q, k, v, 0.0, 0.0, 1.0, scale, use_normalize, eps)
