"""``chunk_retention``: chunk_simple_gla with the fixed per-head decay g_h = log(1 - 2^(-5-h)).
Called by the reference at ``linear_moe/sequence_modeling/retention/retention.py:91``."""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from .simple_gla import chunk_simple_gla


_DECAY = {}


def retention_log_decay(H: int, device=None) -> torch.Tensor:
    """log(1 - 2^(-5-h)) for h < H, fp32 (formed once per head count and device, then reused: the call itself
    then launches nothing but the op)."""
    key = (H, str(device))
    if key not in _DECAY:
        h = torch.arange(H, dtype=torch.float64)
        _DECAY[key] = torch.log1p(-torch.pow(2.0, -5.0 - h)).float().to(device)
    return _DECAY[key]


def chunk_retention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    scale: Optional[float] = None,
    initial_state: Optional[torch.Tensor] = None,
    output_final_state: bool = False,
    cu_seqlens: Optional[torch.Tensor] = None,
    head_first: bool = True,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    if head_first:
        B, H, T = q.shape[:3]
        g = retention_log_decay(H, q.device)[None, :, None].expand(B, H, T)
    else:
        B, T, H = q.shape[:3]
        g = retention_log_decay(H, q.device)[None, None, :].expand(B, T, H)
    return chunk_simple_gla(q, k, v, g, scale, initial_state, output_final_state, cu_seqlens, head_first)
