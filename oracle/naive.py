"""CPU oracle: token-by-token recurrences for the chunked linear-attention path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this file; it
is the checker used by ``tests/``, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py``.

The reference (OpenSparseLLMs/Linear-MoE) does not hold this arithmetic itself:
its token mixers call the third-party package flash-linear-attention ("fla",
pinned snapshot 2025-03-03 by ``examples/linear_moe_qwen2/run_pretrain_qwen.sh:8``;
the submodule directory is empty in the checkout).  The functions below restate
fla's published ``naive_recurrent_*`` recurrences, anchored on the reference's
call sites:

* ``linear_moe/sequence_modeling/gated_deltanet/gated_deltanet.py:112``
  ``chunk_gated_delta_rule(q, k, v, g, beta, head_first=False)``
* ``linear_moe/sequence_modeling/gla/gla.py:94``  ``chunk_gla(q, k, v, gk)``
* ``linear_moe/sequence_modeling/retention/retention.py:91`` ``chunk_retention(q, k, v)``
* ``linear_moe/sequence_modeling/basic_linear_attention/basic_linear_attention.py:133``
  ``chunk_linear_attn(q, k, v, normalize=...)``
* ``linear_moe/sequence_modeling/lightning_attention/lightning_attention.py:121-123``
  ``lightning_attn2(q, k, v, slope)``

Parity status: the reference ships no test, golden vector or fixture for this
path, so these recurrences are pinned by mathematics instead (closed forms,
special cases that reduce to ``tril(QK^T)V``, hand-unrolled tiny cases, linearity
and state hand-off invariants, finite-difference gradients, and the independent
``transformers`` torch routine for the gated delta rule) in
``tests/test_oracle_pins.py``.  What only an import of fla could pin -- its
exact low-precision rounding points and the epsilon of ``normalize=True`` --
is "parity unpinned" and documented as such in the tests.

All functions are differentiable through ``torch.autograd`` and compute in the
dtype given by ``dtype`` (float64 by default).
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

Tensor = torch.Tensor


def _to_head_first(x: Tensor, head_first: bool) -> Tensor:
    # [B,T,H,...] -> [B,H,T,...]
    return x if head_first else x.transpose(1, 2)


def _seq_ranges(cu_seqlens, B: int, T: int):
    if cu_seqlens is None:
        return None
    cu = [int(c) for c in cu_seqlens]
    return list(zip(cu[:-1], cu[1:]))


def _run_varlen(core, tensors, initial_state, output_final_state, cu_seqlens):
    """Apply ``core`` (head-first dense op on [1,H,T,..]) to every packed sequence."""
    outs, finals = [], []
    for n, (s, e) in enumerate(_seq_ranges(cu_seqlens, 1, 0)):
        sl = [None if t is None else t[:, :, s:e] for t in tensors]
        h0 = None if initial_state is None else initial_state[n:n + 1]
        o, ht = core(*sl, h0)
        outs.append(o)
        finals.append(ht)
    o = torch.cat(outs, dim=2)
    ht = torch.cat(finals, dim=0) if output_final_state else None
    return o, ht


# --------------------------------------------------------------------------- #
# simple_gla: S_t = e^{g_t} S_{t-1} + k_t^T v_t ; o_t = scale q_t S_t
# (g scalar per token and head; g=None means no decay)
# --------------------------------------------------------------------------- #
def naive_recurrent_simple_gla(
    q: Tensor, k: Tensor, v: Tensor, g: Optional[Tensor] = None,
    scale: Optional[float] = None, initial_state: Optional[Tensor] = None,
    output_final_state: bool = False, cu_seqlens=None, head_first: bool = True,
    dtype=torch.float64,
) -> Tuple[Tensor, Optional[Tensor]]:
    out_dtype = v.dtype
    q, k, v = (_to_head_first(x, head_first).to(dtype) for x in (q, k, v))
    g = None if g is None else _to_head_first(g, head_first).to(dtype)
    K = q.shape[-1]
    scale = K ** -0.5 if scale is None else scale
    h0 = None if initial_state is None else initial_state.to(dtype)

    def core(q, k, v, g, h0):
        B, H, T, _ = q.shape
        V = v.shape[-1]
        S = q.new_zeros(B, H, K, V) if h0 is None else h0
        o = []
        for t in range(T):
            if g is not None:
                S = S * g[:, :, t].exp()[..., None, None]
            S = S + k[:, :, t, :, None] * v[:, :, t, None, :]
            o.append(torch.einsum('bhk,bhkv->bhv', q[:, :, t], S) * scale)
        o = torch.stack(o, dim=2) if T > 0 else q.new_zeros(B, H, 0, V)
        return o, S

    if cu_seqlens is not None:
        o, ht = _run_varlen(core, (q, k, v, g), h0, output_final_state, cu_seqlens)
    else:
        o, ht = core(q, k, v, g, h0)
        ht = ht if output_final_state else None
    o = _to_head_first(o, head_first)  # transpose back when time-first
    return o, ht


# --------------------------------------------------------------------------- #
# gla: S_t = diag(e^{g_t}) S_{t-1} + k_t^T v_t ; o_t = scale q_t S_t  (g_t in R^K)
# --------------------------------------------------------------------------- #
def naive_recurrent_gla(
    q: Tensor, k: Tensor, v: Tensor, g: Tensor,
    scale: Optional[float] = None, initial_state: Optional[Tensor] = None,
    output_final_state: bool = False, cu_seqlens=None, head_first: bool = True,
    dtype=torch.float64,
) -> Tuple[Tensor, Optional[Tensor]]:
    q, k, v, g = (_to_head_first(x, head_first).to(dtype) for x in (q, k, v, g))
    K = q.shape[-1]
    scale = K ** -0.5 if scale is None else scale
    h0 = None if initial_state is None else initial_state.to(dtype)

    def core(q, k, v, g, h0):
        B, H, T, _ = q.shape
        V = v.shape[-1]
        S = q.new_zeros(B, H, K, V) if h0 is None else h0
        o = []
        for t in range(T):
            S = S * g[:, :, t].exp()[..., None]
            S = S + k[:, :, t, :, None] * v[:, :, t, None, :]
            o.append(torch.einsum('bhk,bhkv->bhv', q[:, :, t], S) * scale)
        o = torch.stack(o, dim=2) if T > 0 else q.new_zeros(B, H, 0, V)
        return o, S

    if cu_seqlens is not None:
        o, ht = _run_varlen(core, (q, k, v, g), h0, output_final_state, cu_seqlens)
    else:
        o, ht = core(q, k, v, g, h0)
        ht = ht if output_final_state else None
    return _to_head_first(o, head_first), ht


# --------------------------------------------------------------------------- #
# gated delta rule:
#   S~_t = e^{g_t} S_{t-1};  r_t = v_t - k_t S~_t;  S_t = S~_t + k_t^T (beta_t r_t)
#   o_t = scale q_t S_t
# --------------------------------------------------------------------------- #
def naive_recurrent_gated_delta_rule(
    q: Tensor, k: Tensor, v: Tensor, g: Optional[Tensor], beta: Tensor,
    scale: Optional[float] = None, initial_state: Optional[Tensor] = None,
    output_final_state: bool = False, cu_seqlens=None, head_first: bool = False,
    use_qk_l2norm_in_kernel: bool = False, dtype=torch.float64,
) -> Tuple[Tensor, Optional[Tensor]]:
    q, k, v, beta = (_to_head_first(x, head_first).to(dtype) for x in (q, k, v, beta))
    g = None if g is None else _to_head_first(g, head_first).to(dtype)
    if use_qk_l2norm_in_kernel:
        # linear_moe/model/common_modules/l2norm.py:22-45 (eps 1e-6 inside the rsqrt)
        q = q * torch.rsqrt((q * q).sum(-1, keepdim=True) + 1e-6)
        k = k * torch.rsqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    K = q.shape[-1]
    scale = K ** -0.5 if scale is None else scale
    h0 = None if initial_state is None else initial_state.to(dtype)

    def core(q, k, v, g, beta, h0):
        B, H, T, _ = q.shape
        V = v.shape[-1]
        S = q.new_zeros(B, H, K, V) if h0 is None else h0
        o = []
        for t in range(T):
            if g is not None:
                S = S * g[:, :, t].exp()[..., None, None]
            r = v[:, :, t] - torch.einsum('bhk,bhkv->bhv', k[:, :, t], S)
            S = S + k[:, :, t, :, None] * (beta[:, :, t, None] * r)[:, :, None, :]
            o.append(torch.einsum('bhk,bhkv->bhv', q[:, :, t], S) * scale)
        o = torch.stack(o, dim=2) if T > 0 else q.new_zeros(B, H, 0, V)
        return o, S

    if cu_seqlens is not None:
        o, ht = _run_varlen(core, (q, k, v, g, beta), h0, output_final_state, cu_seqlens)
    else:
        o, ht = core(q, k, v, g, beta, h0)
        ht = ht if output_final_state else None
    return _to_head_first(o, head_first), ht


# --------------------------------------------------------------------------- #
# adaptors the reference's modules call (same recurrences, fixed gates)
# --------------------------------------------------------------------------- #
def retention_log_decay(H: int, dtype=torch.float64) -> Tensor:
    """g_h = log(1 - 2^(-5-h)) -- the per-head decay chunk_retention applies."""
    h = torch.arange(H, dtype=dtype)
    return torch.log1p(-torch.pow(torch.tensor(2.0, dtype=dtype), -5.0 - h))


def naive_retention(q, k, v, scale=None, initial_state=None, output_final_state=False,
                    cu_seqlens=None, head_first=True, dtype=torch.float64):
    H = q.shape[1] if head_first else q.shape[2]
    T = q.shape[2] if head_first else q.shape[1]
    gh = retention_log_decay(H, dtype)
    g = gh[None, :, None].expand(q.shape[0], H, T) if head_first else gh[None, None, :].expand(q.shape[0], T, H)
    return naive_recurrent_simple_gla(q, k, v, g, scale, initial_state, output_final_state,
                                      cu_seqlens, head_first, dtype)


def naive_linear_attn(q, k, v, scale=None, initial_state=None, output_final_state=False,
                      normalize=True, head_first=True, dtype=torch.float64, eps=1e-10):
    """chunk_linear_attn: simple_gla with g=None; normalize divides o by (scale q) . cumsum(k) + eps, i.e.
    o_t = sum_{s<=t} a_ts v_s / (sum_{s<=t} a_ts + eps) with a_ts = scale q_t . k_s: the scale cancels up to eps
    (call sites: basic_linear_attention.py:133 with the default scale, based.py:69 / rebased.py:76 with scale 1).

    The value of eps is recalled from fla (not checkable offline): parity unpinned for that constant only; the
    formula is pinned by its closed form and a hand-worked case in tests/test_oracle_pins.py.
    """
    o, ht = naive_recurrent_simple_gla(q, k, v, None, scale, initial_state, output_final_state,
                                       None, head_first, dtype)
    if normalize:
        qh, kh = (_to_head_first(x, head_first).to(dtype) for x in (q, k))
        sc = q.shape[-1] ** -0.5 if scale is None else scale
        z = sc * (qh * kh.cumsum(2)).sum(-1, keepdim=True) + eps
        o = _to_head_first(_to_head_first(o, head_first) / z, head_first)
    return o, ht


def lightning_slopes(H: int, dtype=torch.float64) -> Tensor:
    """ALiBi-style slopes, linear_moe/sequence_modeling/lightning_attention/lightning_attention.py:79-105."""
    def pow2(n):
        start = 2 ** (-(2 ** -(math.log2(n) - 3)))
        return [start * start ** i for i in range(n)]

    def slopes(n):
        if math.log2(n).is_integer():
            return pow2(n)
        c = 2 ** math.floor(math.log2(n))
        return pow2(c) + slopes(2 * c)[0::2][: n - c]

    return torch.tensor(slopes(H), dtype=dtype)


def naive_lightning_attn2(q, k, v, s, dtype=torch.float64):
    """o_i = sum_{j<=i} e^{-s_h (i-j)} (q_i . k_j) v_j  (head-first, no scale)."""
    B, H, T, _ = q.shape
    g = (-s.reshape(1, H, 1).to(dtype)).expand(B, H, T)
    o, _ = naive_recurrent_simple_gla(q, k, v, g, 1.0, None, False, None, True, dtype)
    return o


def naive_l2_norm(x: Tensor, eps: float = 1e-6, dtype=torch.float64) -> Tensor:
    """y = x / sqrt(sum x^2 + eps) over the last dimension
    (linear_moe/model/common_modules/l2norm.py:22-45: eps sits inside the square root; the backward
    kernel :64-95 is the derivative of exactly this expression, so autograd through it is the oracle
    of the gradient too)."""
    x = x.to(dtype)
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + eps)


def naive_rms_norm(x: Tensor, weight: Tensor = None, gate: Tensor = None, eps: float = 1e-5, dtype=torch.float64) -> Tensor:
    """y = x / sqrt(mean(x^2) + eps) * weight [* gate * sigmoid(gate)] over the last dimension
    (linear_moe/model/common_modules/layernorm.py:113-127 with IS_RMS_NORM: var = sum(x^2) / N,
    rstd = 1 / sqrt(var + eps), y = x * rstd * w; the gate product is linear_attention.py:255,
    ``o * swish(o_gate)``).  Autograd through this expression is the oracle of the backward."""
    x = x.to(dtype)
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    if weight is not None:
        y = y * weight.to(dtype)
    if gate is not None:
        g = gate.to(dtype)
        y = y * g * torch.sigmoid(g)
    return y


def naive_silu_l2_norm(x: Tensor, eps: float = 1e-6, dtype=torch.float64) -> Tensor:
    """l2_norm(silu(x)) (gated_deltanet.py:101 then :105-106)."""
    x = x.to(dtype)
    return naive_l2_norm(x * torch.sigmoid(x), eps, dtype)


def naive_gdn_qkv_prologue(qkv: Tensor, H: int, D: int, eps: float = 1e-6, dtype=torch.float64):
    """The gated-delta-rule mixer between its fused projection and the op, step by step as the reference does it:
    view [T, B, H, 3 D] and split into q, k, v (linear_moe/sequence_modeling/linear_attention.py:159-163),
    'n b h d -> b n h d' (gated_deltanet/gated_deltanet.py:99), SiLU on all three (:101), l2 norm of q and k
    (:105-106).  Returns q, k, v, each [B, T, H, D]."""
    T, B = qkv.shape[0], qkv.shape[1]
    q, k, v = torch.split(qkv.to(dtype).reshape(T, B, H, 3 * D), [D, D, D], dim=3)
    q, k, v = (x.transpose(0, 1) for x in (q, k, v))
    return naive_silu_l2_norm(q, eps, dtype), naive_silu_l2_norm(k, eps, dtype), v * torch.sigmoid(v)


def naive_swish_gate_relayout(o: Tensor, o_gate: Tensor, dtype=torch.float64) -> Tensor:
    """'b n h d -> n b (h d)' (gated_deltanet.py:114), then o * swish(o_gate) (linear_attention.py:255)."""
    B, T, H, D = o.shape
    g = o_gate.to(dtype).reshape(T, B, H * D)
    return o.to(dtype).transpose(0, 1).reshape(T, B, H * D) * (g * torch.sigmoid(g))


def naive_gdn_gates(a: Tensor, b: Tensor, A_log: Tensor, dt_bias: Tensor, dtype=torch.float64):
    """(g, beta) of the gated delta rule (linear_moe/sequence_modeling/linear_attention.py:153-154):
    beta = sigmoid(b), g = -exp(A_log) * softplus(a + dt_bias)."""
    import torch.nn.functional as F
    g = -torch.exp(A_log.to(dtype)) * F.softplus(a.to(dtype) + dt_bias.to(dtype))
    return g, torch.sigmoid(b.to(dtype))


def naive_gla_gate(x: Tensor, normalizer: float = 16.0, clamp_min=None, dtype=torch.float64) -> Tensor:
    """gk of chunk_gla (linear_moe/sequence_modeling/gla/gla.py:85, :90-91)."""
    import torch.nn.functional as F
    y = F.logsigmoid(x.to(dtype)) / normalizer
    return y if clamp_min is None else torch.clamp_min(y, clamp_min)


def naive_hgrn2_gates(f: Tensor, lower_bound: Tensor = None, dtype=torch.float64):
    """(k, g) of HGRN2 (linear_moe/sequence_modeling/linear_rnn.py:327-335): without a lower bound
    k = 1 - sigmoid(f), g = logsigmoid(f); with one G = lb + (1 - lb) sigmoid(f), k = 1 - G, g = log G."""
    import torch.nn.functional as F
    f = f.to(dtype)
    if lower_bound is None:
        return 1 - torch.sigmoid(f), F.logsigmoid(f)
    G = lower_bound.to(dtype) + (1 - lower_bound.to(dtype)) * torch.sigmoid(f)
    return 1 - G, torch.log(G)


def _pair_products(x: Tensor):
    """(off-diagonal x_i x_j for i < j in row-major order of the strict upper triangle, diagonal x_i^2):
    ``flatten_diag_outer_product_off1(x, x)`` of linear_moe/model/common_modules/feature_map.py:24-30, as loops."""
    D = x.shape[-1]
    off = [x[..., i] * x[..., j] for i in range(D) for j in range(i + 1, D)]
    diag = [x[..., i] * x[..., i] for i in range(D)]
    return torch.stack(off, dim=-1), torch.stack(diag, dim=-1)


def naive_taylor_feature_map(x: Tensor, dtype=torch.float64) -> Tensor:
    """TaylorFeatureMap of Based (feature_map.py:190-203): [1 | x / D^(1/4) | x_i^2 / sqrt(2 D) | x_i x_j / sqrt(D)]."""
    x = x.to(dtype)
    D = x.shape[-1]
    off, diag = _pair_products(x)
    rd = math.sqrt(D)
    return torch.cat([torch.ones_like(x[..., :1]), x / math.sqrt(rd), diag / (rd * math.sqrt(2.0)), off / rd], dim=-1)


def naive_rebased_feature_map(x: Tensor, gamma: Tensor = None, beta: Tensor = None, normalize: bool = True,
                              eps: float = 1e-6, dtype=torch.float64) -> Tensor:
    """RebasedFeatureMap with flatten=True (feature_map.py:206-246; its layer norm has eps 1e-6, layernorm.py:474):
    x' = gamma * norm(x) + beta, then [x'_i^2 / sqrt(D) | x'_i x'_j sqrt(2 / D)]."""
    x = x.to(dtype)
    D = x.shape[-1]
    if normalize:
        mu = x.mean(-1, keepdim=True)
        var = ((x - mu) ** 2).mean(-1, keepdim=True)
        x = (x - mu) / torch.sqrt(var + eps)
    if gamma is not None:
        x = x * gamma.to(dtype)
    if beta is not None:
        x = x + beta.to(dtype)
    off, diag = _pair_products(x)
    return torch.cat([diag * D ** -0.5, off * (2.0 / D) ** 0.5], dim=-1)
