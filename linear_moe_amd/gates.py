"""Gate construction in front of the chunk ops on MI355X (one elementwise pass each, forward and backward).

``gdn_gates``: ``beta = sigmoid(b)``, ``g = -exp(A_log) * softplus(a + dt_bias)`` (fp32), what
``LinearAttention.forward`` of the reference forms for the gated delta rule
(``linear_moe/sequence_modeling/linear_attention.py:153-154``; parameters ``:92-113``).
``gla_gate``: ``logsigmoid(x) / normalizer`` with the optional lower clamp of
``linear_moe/sequence_modeling/gla/gla.py:85, :90-91``.
``hgrn2_gates``: ``k = 1 - sigmoid(f)``, ``g = logsigmoid(f)`` (fp32), optionally with a lower bound
(``linear_moe/sequence_modeling/linear_rnn.py:327-335``), in front of ``chunk_gla(q, k, i, g)``.
"""
from __future__ import annotations

import math

import torch

from . import _lib
from ._host import stream_ptr


def _dt(t):
    if t.dtype not in (torch.bfloat16, torch.float32):
        raise ValueError(f"dtype {t.dtype} unsupported (bfloat16 or float32)")
    return _lib.LMOE_F32 if t.dtype == torch.float32 else _lib.LMOE_BF16


class _GdnGates(torch.autograd.Function):
    @staticmethod
    def forward(ctx, a, b, A_log, dt_bias):
        if not a.is_cuda:
            raise RuntimeError("linear_moe_amd ops are GPU only (no CPU fallback)")
        if a.shape != b.shape or a.dtype != b.dtype:
            raise ValueError("gdn_gates: a and b must agree in shape and dtype")
        H = a.shape[-1]
        if A_log.shape != (H,) or dt_bias.shape != (H,):
            raise ValueError(f"gdn_gates: A_log and dt_bias must have shape ({H},)")
        lib = _lib.load()
        ac, bc = a.contiguous(), b.contiguous()
        Af, Bf = A_log.detach().float().contiguous(), dt_bias.detach().float().contiguous()
        g = torch.empty(a.shape, dtype=torch.float32, device=a.device)
        beta = torch.empty_like(bc)
        rows = ac.numel() // H
        _lib.check(lib.lmoe_gdn_gates_fwd(ac.data_ptr(), bc.data_ptr(), Af.data_ptr(), Bf.data_ptr(), g.data_ptr(),
                                          beta.data_ptr(), rows, H, _dt(a), stream_ptr()), "gdn_gates")
        ctx.save_for_backward(ac, bc, Af, Bf)
        ctx.pdt = (A_log.dtype, dt_bias.dtype)
        return g, beta

    @staticmethod
    def backward(ctx, dg, dbeta):
        ac, bc, Af, Bf = ctx.saved_tensors
        lib = _lib.load()
        H = ac.shape[-1]
        rows = ac.numel() // H
        dgc = (torch.zeros_like(ac, dtype=torch.float32) if dg is None else dg.float().contiguous())
        dbc = (torch.zeros_like(bc) if dbeta is None else dbeta.to(bc.dtype).contiguous())
        da, db = torch.empty_like(ac), torch.empty_like(bc)
        dpar = torch.zeros(2, H, dtype=torch.float32, device=ac.device)
        if rows:
            part = torch.empty(lib.lmoe_gdn_gates_partials(rows, H), 2, H, dtype=torch.float32, device=ac.device)
            _lib.check(lib.lmoe_gdn_gates_bwd(ac.data_ptr(), bc.data_ptr(), Af.data_ptr(), Bf.data_ptr(), dgc.data_ptr(),
                                              dbc.data_ptr(), da.data_ptr(), db.data_ptr(), part.data_ptr(),
                                              dpar.data_ptr(), rows, H, _dt(ac), stream_ptr()), "gdn_gates backward")
        return da, db, dpar[0].to(ctx.pdt[0]), dpar[1].to(ctx.pdt[1])


def gdn_gates(a: torch.Tensor, b: torch.Tensor, A_log: torch.Tensor, dt_bias: torch.Tensor):
    """(g, beta) for a, b of shape [..., H]: g fp32, beta in the dtype of b."""
    return _GdnGates.apply(a, b, A_log, dt_bias)


class _GlaGate(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, normalizer, clamp_min):
        if not x.is_cuda:
            raise RuntimeError("linear_moe_amd ops are GPU only (no CPU fallback)")
        if x.numel() % 8:
            raise ValueError("gla_gate: the element count must be a multiple of 8")
        lib = _lib.load()
        xc = x.contiguous()
        y = torch.empty_like(xc)
        cm = -math.inf if clamp_min is None else float(clamp_min)
        _lib.check(lib.lmoe_gla_gate_fwd(xc.data_ptr(), y.data_ptr(), xc.numel(), _dt(x), float(normalizer), cm,
                                         stream_ptr()), "gla_gate")
        ctx.save_for_backward(xc)
        ctx.args = (float(normalizer), cm)
        return y

    @staticmethod
    def backward(ctx, dy):
        (xc,) = ctx.saved_tensors
        lib = _lib.load()
        dyc = dy.contiguous()
        dx = torch.empty_like(xc)
        _lib.check(lib.lmoe_gla_gate_bwd(xc.data_ptr(), dyc.data_ptr(), dx.data_ptr(), xc.numel(), _dt(xc), ctx.args[0],
                                         ctx.args[1], stream_ptr()), "gla_gate backward")
        return dx, None, None


def gla_gate(x: torch.Tensor, normalizer: float = 16.0, clamp_min=None) -> torch.Tensor:
    """``max(logsigmoid(x) / normalizer, clamp_min)`` in the dtype of x."""
    return _GlaGate.apply(x, normalizer, clamp_min)


class _Hgrn2Gates(torch.autograd.Function):
    @staticmethod
    def forward(ctx, f, lower_bound):
        if not f.is_cuda:
            raise RuntimeError("linear_moe_amd ops are GPU only (no CPU fallback)")
        D = f.shape[-1]
        if D % 8:
            raise ValueError("hgrn2_gates: the last dimension must be a multiple of 8")
        lb = None
        if lower_bound is not None:
            if lower_bound.shape != (D,):
                raise ValueError(f"hgrn2_gates: lower_bound must have shape ({D},)")
            lb = lower_bound.detach().float().contiguous()
        lib = _lib.load()
        fc = f.contiguous()
        k = torch.empty_like(fc)
        g = torch.empty(fc.shape, dtype=torch.float32, device=f.device)
        _lib.check(lib.lmoe_hgrn2_gate_fwd(fc.data_ptr(), None if lb is None else lb.data_ptr(), k.data_ptr(), g.data_ptr(),
                                           fc.numel(), D, _dt(f), stream_ptr()), "hgrn2_gates")
        ctx.save_for_backward(fc, lb)
        return k, g

    @staticmethod
    def backward(ctx, dk, dg):
        fc, lb = ctx.saved_tensors
        lib = _lib.load()
        dkc = torch.zeros_like(fc) if dk is None else dk.to(fc.dtype).contiguous()
        dgc = torch.zeros_like(fc, dtype=torch.float32) if dg is None else dg.float().contiguous()
        df = torch.empty_like(fc)
        _lib.check(lib.lmoe_hgrn2_gate_bwd(fc.data_ptr(), None if lb is None else lb.data_ptr(), dkc.data_ptr(),
                                           dgc.data_ptr(), df.data_ptr(), fc.numel(), fc.shape[-1], _dt(fc), stream_ptr()),
                   "hgrn2_gates backward")
        return df, None


def hgrn2_gates(f: torch.Tensor, lower_bound: torch.Tensor = None):
    """(k, g) for the forget projection f of shape [..., D]: k in the dtype of f, g fp32.  ``lower_bound`` ([D]) is
    taken as a constant (no gradient flows to it)."""
    if lower_bound is not None and lower_bound.requires_grad:
        raise NotImplementedError("hgrn2_gates: no gradient for lower_bound; pass lower_bound.detach()")
    return _Hgrn2Gates.apply(f, lower_bound)
