"""CPU restatement of the reference's mixture-of-memories routing, for tests only.

TEST INFRASTRUCTURE: nothing in ``linear_moe_amd/`` imports this module.

``transform`` pads the tokens routed to every (memory, batch row) to a common capacity and
``reconstruct`` scatters the per-memory results back and mixes them with the routing weights
(linear_moe/sequence_modeling/mom_linear_attention.py:15-77 and :79-120).  Both are restated here
with explicit loops over (batch row, memory), which is what the reference's index arithmetic
computes: per (b, e) the routed tokens in time order, truncated to the LAST ``max_len`` of them,
left-padded with zeros to ``capacity_len = ceil(seq_len * capacity)`` (mom_linear_attention.py:57:
``ceil(s / topk * capacity)`` with ``s`` already multiplied by ``topk`` at :26-27).

The reference sorts with ``argsort`` on the key ``batch * (max_expert + 1) + expert`` (:40-43) and relies
on the sort keeping the time order inside equal keys; the restatement makes that order explicit.
"""
from __future__ import annotations

import math
from typing import List, Tuple

import torch


def routed_tokens(selected: torch.Tensor, num_memories: int) -> List[List[List[Tuple[int, int]]]]:
    """routed[b][e] = [(t, k), ...] in time order: token t of batch row b chose memory e as its k-th choice."""
    B, S, topk = selected.shape
    routed = [[[] for _ in range(num_memories)] for _ in range(B)]
    for b in range(B):
        for t in range(S):
            for k in range(topk):
                routed[b][int(selected[b, t, k])].append((t, k))
    return routed


def transform(x: torch.Tensor, selected: torch.Tensor, num_memories: int, capacity: float):
    """x [B, S, D], selected [B, S, topk] -> (padded [E, B, capacity_len, D], max_len, kept) where
    kept[b][e] lists the (t, k) that survive the truncation (mom_linear_attention.py:15-77)."""
    B, S, D = x.shape
    routed = routed_tokens(selected, num_memories)
    capacity_len = math.ceil(S * capacity)
    longest = max(len(routed[b][e]) for b in range(B) for e in range(num_memories))
    max_len = min(longest, capacity_len)
    out = torch.zeros(num_memories, B, capacity_len, D, dtype=x.dtype)
    kept = [[None] * num_memories for _ in range(B)]
    for b in range(B):
        for e in range(num_memories):
            toks = routed[b][e][-max_len:] if max_len > 0 else []
            kept[b][e] = toks
            for j, (t, _) in enumerate(toks):
                out[e, b, capacity_len - len(toks) + j] = x[b, t]        # left padding (:70-72)
    return out, max_len, kept


def reconstruct(y: torch.Tensor, kept, routing_weights: torch.Tensor) -> torch.Tensor:
    """y [E, B, L, ...] with every kept sequence right-aligned in L -> [B, S, ...]:
    out[b, t] = sum_k w[b, t, k] * y[e(b,t,k), b, slot]; dropped tokens contribute nothing
    (mom_linear_attention.py:79-120)."""
    E, B, L = y.shape[:3]
    S = routing_weights.shape[1]
    out = torch.zeros((B, S) + tuple(y.shape[3:]), dtype=y.dtype)
    for b in range(B):
        for e in range(E):
            toks = kept[b][e]
            for j, (t, k) in enumerate(toks):
                out[b, t] = out[b, t] + routing_weights[b, t, k].to(y.dtype) * y[e, b, L - len(toks) + j]
    return out
