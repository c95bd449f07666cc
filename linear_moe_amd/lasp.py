"""One GPU's share of sequence-parallel linear attention (LASP-2): the transition of a T-slice and how transitions
of lower slices combine into a slice's initial state.

The reference splits T over the context-parallel ranks; each rank forms the memory of its slice with zero
initial state (``prepare_m``), all-gathers the memories, sums those of lower ranks into its initial state ``KV``
and finishes its slice from there (``linear_moe/sequence_modeling/lasp2/lasp2_without_mask_triton_op.py:688-710``;
backward with the suffix sum of ``dKV``, ``:728-749``).  Its kernels cover the ungated case only.  Here the same
scheme is stated for the three chunk ops through their own ``initial_state`` / ``output_final_state`` arguments
(and their gradients ``dh0`` / ``dht``):

    ungated / scalar gate / per-channel gate:   S_out = decay * S_in + M      decay = 1, e^{sum g} [B,H], e^{sum g} [B,H,K]
    (gated) delta rule:                         S_out = P S_in + M            P [B,H,K,K]

``M`` is the final state of the slice run from a zero state; ``P`` is the final state of the same recurrence with
``v = 0`` run from the identity (the recurrence is linear in the state, column by column).  Everything here is
differentiable, so gradients reach lower slices through ``initial_state`` exactly as the reference's backward
exchange carries them.  The exchange itself (one all-gather of the transitions per direction) is the caller's:
this module holds no communication.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Sequence

import torch

from .gated_delta_rule import chunk_gated_delta_rule
from .gla import chunk_gla
from .simple_gla import chunk_simple_gla


@dataclass
class SliceTransition:
    """``S_out = decay (*) S_in + memory``; decay None (identity), [B,H], [B,H,K] or a matrix [B,H,K,K]."""
    memory: torch.Tensor                    # [B, H, K, V] fp32
    decay: Optional[torch.Tensor] = None

    def apply(self, state: Optional[torch.Tensor]) -> torch.Tensor:
        if state is None:
            return self.memory
        d = self.decay
        if d is None:
            return state + self.memory
        if d.dim() == 2:
            return d[..., None, None] * state + self.memory
        if d.dim() == 3:
            return d[..., None] * state + self.memory
        return torch.matmul(d, state) + self.memory


def combine_transitions(lower: Sequence[SliceTransition]) -> Optional[torch.Tensor]:
    """Initial state of a slice from the transitions of all lower slices, in order (None for the first slice)."""
    state = None
    for t in lower:
        state = t.apply(state)
    return state


def _tdim(head_first):
    return 2 if head_first else 1


def simple_gla_transition(k, v, g=None, head_first=True) -> SliceTransition:
    """Transition of one slice of chunk_simple_gla / chunk_linear_attn / chunk_retention."""
    _, m = chunk_simple_gla(k, k, v, g, 1.0, None, True, None, head_first)
    decay = None if g is None else g.float().sum(_tdim(head_first)).exp()
    return SliceTransition(m, decay)


def gla_transition(k, v, g, head_first=True) -> SliceTransition:
    """Transition of one slice of chunk_gla (g per key channel)."""
    _, m = chunk_gla(k, k, v, g, 1.0, None, True, None, head_first)
    return SliceTransition(m, g.float().sum(_tdim(head_first)).exp())


def gated_delta_rule_transition(k, v, g, beta, head_first=False) -> SliceTransition:
    """Transition of one slice of chunk_gated_delta_rule (g = None: the delta rule)."""
    if g is None:
        g = torch.zeros(beta.shape, dtype=torch.float32, device=beta.device)
    _, m = chunk_gated_delta_rule(k, k, v, g, beta, 1.0, None, True, None, head_first)
    K = k.shape[-1]
    B, H = (k.shape[0], k.shape[1]) if head_first else (k.shape[0], k.shape[2])
    eye = torch.eye(K, dtype=torch.float32, device=k.device).expand(B, H, K, K).contiguous()
    _, p = chunk_gated_delta_rule(k, k, torch.zeros_like(k), g, beta, 1.0, eye, True, None, head_first)
    return SliceTransition(m, p)
