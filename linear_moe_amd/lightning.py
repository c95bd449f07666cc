"""``lightning_attn2`` / ``lightning_attn2_no_decay``: o_i = sum_{j<=i} e^{-s_h (i-j)} (q_i . k_j) v_j.
The same recurrence as chunk_simple_gla with g = -s_h and scale 1; called by the reference at
``linear_moe/sequence_modeling/lightning_attention/lightning_attention.py:121-123`` with
``[B,H,T,D]`` inputs and slopes ``[H,1,1]``; returns ``o`` only."""
from __future__ import annotations

import torch

from .simple_gla import chunk_simple_gla


def lightning_attn2(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, s: torch.Tensor) -> torch.Tensor:
    B, H, T = q.shape[:3]
    g = (-s.reshape(1, H, 1).float()).expand(B, H, T)
    o, _ = chunk_simple_gla(q, k, v, g, 1.0, None, False, None, True)
    return o


def lightning_attn2_no_decay(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    o, _ = chunk_simple_gla(q, k, v, None, 1.0, None, False, None, True)
    return o
