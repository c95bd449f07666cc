"""``chunk_linear_attn``: chunk_simple_gla without decay, optionally normalised by
q . cumsum(k).  Called by the reference at
``linear_moe/sequence_modeling/basic_linear_attention/basic_linear_attention.py:133`` and, with
``normalize=True, scale=1``, by ``.../based/based.py:69`` and ``.../rebased/rebased.py:76``."""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from .simple_gla import chunk_simple_gla


def chunk_linear_attn(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    scale: Optional[float] = None,
    initial_state: Optional[torch.Tensor] = None,
    output_final_state: bool = False,
    normalize: bool = True,
    head_first: bool = True,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    o, ht = chunk_simple_gla(q, k, v, None, scale, initial_state, output_final_state, None, head_first)
    if normalize:
        tdim = 2 if head_first else 1
        z = (q * k.cumsum(tdim)).sum(-1, keepdim=True) + 1e-10
        o = o / z
    return o, ht
