"""Mixture-of-memories routing on MI355X: pack the routed tokens of all memories into one variable-length
batch, run the op once, combine the results per token.

The reference pads the tokens routed to every (memory, batch row) to a common capacity
(``transform``, ``linear_moe/sequence_modeling/mom_linear_attention.py:15-77``), calls the op once per
memory (``:369-409``) and scatters the results back (``reconstruct``, ``:79-120``).  Left padding with
zero tokens does not change a linear-attention state, so the same function is computed by one
``cu_seqlens`` call over the packed tokens: no padded rows, one launch for all memories.

    plan = mom_plan(selected_memories, num_memories, capacity)     # index tables (device)
    xp   = mom_pack(hidden, plan)                                  # [T_total, D]; rows of memory m:
                                                                   #   plan.mem_offsets[m] : plan.mem_offsets[m + 1]
    ... per-memory projections on those row ranges, then one op call with cu_seqlens = plan.cu_seqlens ...
    out  = mom_combine(op_output_rows, plan, routing_weights)      # [B, S, D']

Sequences are ordered memory-major: sequence ``m * B + b`` holds the tokens of batch row ``b`` routed to
memory ``m``, in time order, truncated to the last ``max_len`` of them exactly as the reference truncates.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional

import torch

from . import _lib
from ._host import stream_ptr


@dataclass
class MomPlan:
    B: int
    S: int
    topk: int
    num_memories: int
    T_total: int
    src_token: torch.Tensor     # [T_total] int32: flat token index b * S + t of every packed row
    src_choice: torch.Tensor    # [T_total] int32: flat (token, k) index of every packed row
    row_of: torch.Tensor        # [B * S, topk] int32: packed row of every (token, k), -1 if dropped
    cu_seqlens: torch.Tensor    # [num_memories * B + 1] int32 (device)
    max_len_dev: torch.Tensor   # 0-dim int64 (device): tokens kept per sequence at most
    mem_offsets_dev: torch.Tensor   # [num_memories + 1] int64 (device): row range of every memory

    # the two figures a caller may want on the host are read back only when asked for
    @property
    def max_len(self) -> int:
        return int(self.max_len_dev)

    @property
    def mem_offsets(self) -> torch.Tensor:
        return self.mem_offsets_dev.to("cpu")


def mom_plan(selected_memories: torch.Tensor, num_memories: int, capacity: Optional[float] = None,
             check: bool = False) -> MomPlan:
    """Index tables for ``selected_memories`` [B, S, topk] (as ``torch.topk`` returns them,
    mom_linear_attention.py:288).  ``capacity``: the reference's capacity factor; ``None`` keeps every token.

    Built by device operations only (stable sort by (memory, batch row), counts, prefix sums, scatters), as the
    reference builds its tables on the device (mom_linear_attention.py:28-66).  Without a capacity nothing is read
    back to the host: every routed token is kept, ``T_total = B * S * topk`` is known up front, and pack -> op ->
    combine can run inside a HIP graph capture with the plan in it.  With a capacity the number of surviving rows is
    the one device-to-host read of the call.  ``check`` validates the memory indices (two more reads)."""
    if selected_memories.dim() != 3:
        raise ValueError("selected_memories must be [B, S, topk]")
    B, S, topk = selected_memories.shape
    dev = selected_memories.device
    sel = selected_memories.reshape(-1).to(torch.int64)                        # flat (b, t, k)
    if check and sel.numel() and (int(sel.min()) < 0 or int(sel.max()) >= num_memories):
        raise ValueError("selected_memories out of range")
    n = sel.numel()
    flat = torch.arange(n, device=dev)
    b_of = flat // (S * topk)
    key = sel * B + b_of                                                       # memory-major sequences
    order = torch.argsort(key, stable=True)                                    # time order inside a sequence
    lens = torch.zeros(num_memories * B, dtype=torch.int64, device=dev).scatter_add_(0, key, torch.ones_like(key))
    longest = lens.max() if lens.numel() else torch.zeros((), dtype=torch.int64, device=dev)
    row_of = torch.full((n,), -1, dtype=torch.int32, device=dev)
    cu = torch.zeros(num_memories * B + 1, dtype=torch.int64, device=dev)
    if capacity is None:
        max_len_dev = longest
        cu[1:] = torch.cumsum(lens, 0)
        rows, T_total = order, n                                               # every (token, k), sorted
    else:
        max_len_dev = torch.clamp(longest, max=math.ceil(S * capacity))
        starts = torch.cumsum(lens, 0) - lens
        skey = key[order]
        pos = flat - starts[skey]                                              # position inside its sequence
        keep = pos >= (lens[skey] - max_len_dev)                               # the last max_len survive
        cu[1:] = torch.cumsum(torch.minimum(lens, max_len_dev), 0)
        rows = order[keep]                                                     # (the one read: how many survive)
        T_total = int(rows.numel())
    row_of[rows] = torch.arange(T_total, dtype=torch.int32, device=dev)
    return MomPlan(B, S, topk, num_memories, T_total, (rows // topk).to(torch.int32).contiguous(),
                   rows.to(torch.int32).contiguous(), row_of.view(B * S, topk).contiguous(),
                   cu.to(torch.int32).contiguous(), max_len_dev, cu[::B].contiguous())


def _dt(t):
    if t.dtype not in (torch.bfloat16, torch.float32):
        raise ValueError(f"dtype {t.dtype} unsupported (bfloat16 or float32)")
    return _lib.LMOE_F32 if t.dtype == torch.float32 else _lib.LMOE_BF16


def _rows(x: torch.Tensor, n: int, what: str) -> torch.Tensor:
    if not x.is_cuda:
        raise RuntimeError("linear_moe_amd ops are GPU only (no CPU fallback)")
    x2 = x.reshape(n, -1).contiguous()
    if x2.shape[1] % 8:
        raise ValueError(f"{what}: row length {x2.shape[1]} must be a multiple of 8")
    return x2


class _Pack(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, plan):
        lib = _lib.load()
        x2 = _rows(x, plan.B * plan.S, "mom_pack")
        D = x2.shape[1]
        out = torch.empty(plan.T_total, D, dtype=x.dtype, device=x.device)
        _lib.check(lib.lmoe_mom_gather(x2.data_ptr(), plan.src_token.data_ptr(), None, out.data_ptr(), plan.T_total, D,
                                       _dt(x), stream_ptr()), "mom_pack")
        ctx.plan, ctx.shape = plan, x.shape
        return out

    @staticmethod
    def backward(ctx, dout):
        lib = _lib.load()
        plan = ctx.plan
        d2 = dout.contiguous()
        D = d2.shape[1]
        dx = torch.empty(plan.B * plan.S, D, dtype=dout.dtype, device=dout.device)
        _lib.check(lib.lmoe_mom_combine(d2.data_ptr(), plan.row_of.data_ptr(), None, dx.data_ptr(), plan.B * plan.S,
                                        plan.topk, D, _dt(dout), stream_ptr()), "mom_pack backward")
        return dx.view(ctx.shape), None


class _Combine(torch.autograd.Function):
    @staticmethod
    def forward(ctx, y, w, plan):
        lib = _lib.load()
        y2 = _rows(y, plan.T_total, "mom_combine")
        D = y2.shape[1]
        w2 = w.reshape(plan.B * plan.S, plan.topk).to(y.dtype).contiguous()
        out = torch.empty(plan.B * plan.S, D, dtype=y.dtype, device=y.device)
        _lib.check(lib.lmoe_mom_combine(y2.data_ptr(), plan.row_of.data_ptr(), w2.data_ptr(), out.data_ptr(),
                                        plan.B * plan.S, plan.topk, D, _dt(y), stream_ptr()), "mom_combine")
        ctx.save_for_backward(y2, w2)
        ctx.plan, ctx.yshape, ctx.wshape, ctx.wdtype = plan, y.shape, w.shape, w.dtype
        return out.view((plan.B, plan.S) + tuple(y.shape[1:]))

    @staticmethod
    def backward(ctx, dout):
        lib = _lib.load()
        y2, w2 = ctx.saved_tensors
        plan = ctx.plan
        D = y2.shape[1]
        g = dout.reshape(plan.B * plan.S, D).contiguous()
        # dy[row] = w[choice(row)] * dout[token(row)];  dw[t][k] = <dout[t], y[row_of[t][k]]>
        scale = w2.reshape(-1)[plan.src_choice.long()].contiguous()
        dy = torch.empty_like(y2)
        _lib.check(lib.lmoe_mom_gather(g.data_ptr(), plan.src_token.data_ptr(), scale.data_ptr(), dy.data_ptr(),
                                       plan.T_total, D, _dt(y2), stream_ptr()), "mom_combine backward")
        dw = torch.empty_like(w2)
        _lib.check(lib.lmoe_mom_rowdot(y2.data_ptr(), plan.row_of.data_ptr(), g.data_ptr(), dw.data_ptr(),
                                       plan.B * plan.S, plan.topk, D, _dt(y2), stream_ptr()), "mom_combine backward")
        return dy.view(ctx.yshape), dw.view(ctx.wshape).to(ctx.wdtype), None


def mom_pack(x: torch.Tensor, plan: MomPlan) -> torch.Tensor:
    """x [B, S, D] -> packed rows [T_total, D] (memory-major sequences, see the module docstring)."""
    if x.shape[0] != plan.B or x.shape[1] != plan.S:
        raise ValueError("mom_pack: x must be [B, S, ...] of the plan")
    return _Pack.apply(x, plan)


def mom_combine(y: torch.Tensor, plan: MomPlan, routing_weights: torch.Tensor) -> torch.Tensor:
    """y [T_total, ...] (the op's output rows), routing_weights [B, S, topk] -> [B, S, ...]:
    ``out[b, t] = sum_k w[b, t, k] * y[row of (b, t, k)]``; tokens dropped by the capacity contribute nothing."""
    if y.shape[0] != plan.T_total:
        raise ValueError("mom_combine: y must have T_total rows")
    return _Combine.apply(y, routing_weights, plan)
