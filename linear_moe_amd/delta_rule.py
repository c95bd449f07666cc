"""``chunk_delta_rule`` on MI355X: the gated delta rule without decay.

  S_t = S_{t-1} + k_t^T beta_t (v_t - k_t S_{t-1});  o_t = scale q_t S_t

Keeps the call the reference makes at ``linear_moe/sequence_modeling/deltanet/deltanet.py:127-130``:
``chunk_delta_rule(q, k, v, beta, chunk_size)`` with q, k, v ``[B,H,T,D]`` and beta ``[B,H,T]``.
The result does not depend on the chunk length, so the kernels keep their 64-token chunks whatever
``BT`` names.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from ._host import HEAD_DIMS, WIDE_V, by_head_dim_blocks, no_tokens
from .gated_delta_rule import _ChunkGatedDeltaRule


def chunk_delta_rule(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    beta: torch.Tensor,
    BT: int = 64,
    scale: Optional[float] = None,
    initial_state: Optional[torch.Tensor] = None,
    output_final_state: bool = False,
    cu_seqlens: Optional[torch.Tensor] = None,
    head_first: bool = True,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    if BT not in (16, 32, 64):
        raise ValueError(f"chunk size must be 16, 32 or 64, got {BT}")
    if q.dim() == 4 and v.dim() == 4 and (q.shape[-1] not in HEAD_DIMS or v.shape[-1] not in HEAD_DIMS) \
            and (q.shape[-1], v.shape[-1]) != WIDE_V:
        sc = q.shape[-1] ** -0.5 if scale is None else scale
        return by_head_dim_blocks(
            lambda q_, k_, v_, _g, h0: chunk_delta_rule(q_, k_, v_, beta, BT, sc, h0, output_final_state, cu_seqlens,
                                                        head_first),
            q, k, v, None, initial_state, output_final_state, False, "chunk_delta_rule", wide_v=True)
    r = no_tokens(q, k, v, head_first, cu_seqlens, initial_state, output_final_state, wide_v=True)
    if r is not None:
        return r
    return _ChunkGatedDeltaRule.apply(q, k, v, None, beta, scale, initial_state, output_final_state, cu_seqlens,
                                      head_first)
