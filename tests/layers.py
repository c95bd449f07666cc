"""The reference's token-mixer layer around the chunk ops, restated as plain ``nn.Module``s on the kernels of
``linear_moe_amd`` (no Megatron): the order of operations of ``LinearAttention.forward``
(linear_moe/sequence_modeling/linear_attention.py:146-163 projections, gates and the q/k/v split; :232-256 the
core module, ``o * swish(o_gate)`` and the output projection) with the core modules ``GatedDeltaNet.forward``
(gated_deltanet/gated_deltanet.py:99-114) and ``GLA.forward`` (gla/gla.py:82-97).  Inputs are ``[T, B, hidden]`` as in
the reference.  ``oracle_forward`` of each layer is the same chain on the fp64 oracle functions."""
import torch
import torch.nn.functional as F
from torch import nn

from oracle import naive


class GatedDeltaNetLayer(nn.Module):
    def __init__(self, hidden: int, heads: int, head_dim: int, seed: int = 0):
        super().__init__()
        g = torch.Generator().manual_seed(seed)
        H, D = heads, head_dim
        self.H, self.D = H, D
        w = lambda o, i: nn.Parameter(torch.randn(o, i, generator=g) * i ** -0.5)
        self.qkv_proj, self.o_gate_proj, self.o_proj = w(3 * H * D, hidden), w(H * D, hidden), w(hidden, H * D)
        self.beta_proj, self.a_proj = w(H, hidden), w(H, hidden)
        # parameter laws of linear_attention.py:93-110
        self.A_log = nn.Parameter(torch.log(torch.rand(H, generator=g) * 15 + 1))
        dt = torch.exp(torch.rand(H, generator=g) * (torch.log(torch.tensor(0.1)) - torch.log(torch.tensor(0.001)))
                       + torch.log(torch.tensor(0.001))).clamp_min(1e-4)
        self.dt_bias = nn.Parameter(dt + torch.log(-torch.expm1(-dt)))

    def _split(self, x):
        T, B, _ = x.shape
        qkv = F.linear(x, self.qkv_proj.to(x.dtype)).view(T, B, self.H, 3 * self.D)
        return torch.split(qkv, [self.D, self.D, self.D], dim=3)          # each [T, B, H, D] (a strided view)

    def forward(self, x, fused: bool = True, core: bool = False):
        """fused: the one-pass prologue / epilogue kernels; otherwise the chain of copies, row kernels and eager
        elementwise ops they replace (same numbers to the rounding of the element type).  core (with fused, bfloat16):
        prologue and op as one call that never writes silu(v) (``gdn_mixer_core``)."""
        import linear_moe_amd as L
        T, B, _ = x.shape
        o_gate = F.linear(x, self.o_gate_proj.to(x.dtype))
        xt = x.transpose(0, 1)                                             # [B, T, hidden]
        gk, beta = L.gdn_gates(F.linear(xt, self.a_proj.to(x.dtype)), F.linear(xt, self.beta_proj.to(x.dtype)),
                               self.A_log, self.dt_bias)                   # [B, T, H]: fp32 log-decay, beta
        if fused and core:
            o = L.gdn_mixer_core(F.linear(x, self.qkv_proj.to(x.dtype)), gk, beta, self.H, self.D)
            return F.linear(L.swish_gate_relayout(o, o_gate), self.o_proj.to(x.dtype))
        if fused:
            q, k, v = L.gdn_qkv_prologue(F.linear(x, self.qkv_proj.to(x.dtype)), self.H, self.D)
        else:
            q, k, v = self._split(x)
            q, k, v = (t.transpose(0, 1).contiguous() for t in (q, k, v))  # [B, T, H, D]
            q, k, v = L.silu_l2_norm(q), L.silu_l2_norm(k), F.silu(v)
        o, _ = L.chunk_gated_delta_rule(q, k, v, gk, beta, head_first=False)
        if fused:
            o = L.swish_gate_relayout(o, o_gate)
        else:
            o = o.transpose(0, 1).reshape(T, B, self.H * self.D)           # 'b n h d -> n b (h d)'
            o = o * F.silu(o_gate)
        return F.linear(o, self.o_proj.to(x.dtype))

    def oracle_forward(self, x):
        T, B, _ = x.shape
        P = lambda p: p.double()
        qkv = (x @ P(self.qkv_proj).T).view(T, B, self.H, 3 * self.D)
        q, k, v = torch.split(qkv, [self.D, self.D, self.D], dim=3)
        o_gate = x @ P(self.o_gate_proj).T
        xt = x.transpose(0, 1)
        gk, beta = naive.naive_gdn_gates(xt @ P(self.a_proj).T, xt @ P(self.beta_proj).T, P(self.A_log), P(self.dt_bias))
        q, k, v = (t.transpose(0, 1) for t in (q, k, v))
        q, k, v = naive.naive_silu_l2_norm(q), naive.naive_silu_l2_norm(k), F.silu(v)
        o, _ = naive.naive_recurrent_gated_delta_rule(q, k, v, gk, beta, None, None, False, None, False)
        o = o.transpose(0, 1).reshape(T, B, self.H * self.D)
        o = o * F.silu(o_gate)
        return o @ P(self.o_proj).T


class GLALayer(nn.Module):
    def __init__(self, hidden: int, heads: int, head_dim: int, low_rank: int = 16, seed: int = 0, eps: float = 1e-5):
        super().__init__()
        g = torch.Generator().manual_seed(seed)
        H, D = heads, head_dim
        self.H, self.D, self.eps = H, D, eps
        w = lambda o, i: nn.Parameter(torch.randn(o, i, generator=g) * i ** -0.5)
        self.qkv_proj, self.o_gate_proj, self.o_proj = w(3 * H * D, hidden), w(H * D, hidden), w(hidden, H * D)
        # GLAGate: low-rank two-layer map with a bias (gla/gla_gate.py:22-23)
        self.gk_down, self.gk_up, self.gk_bias = w(low_rank, hidden), w(H * D, low_rank), nn.Parameter(torch.zeros(H * D))
        self.norm_weight = nn.Parameter(1 + 0.1 * torch.randn(D, generator=g))

    def forward(self, x):
        import linear_moe_amd as L
        T, B, _ = x.shape
        dt = x.dtype
        qkv = F.linear(x, self.qkv_proj.to(dt)).view(T, B, self.H, 3 * self.D)
        q, k, v = torch.split(qkv, [self.D, self.D, self.D], dim=3)
        o_gate = F.linear(x, self.o_gate_proj.to(dt))
        gk = F.linear(F.linear(x, self.gk_down.to(dt)), self.gk_up.to(dt), self.gk_bias.to(dt))
        q, k, v = (t.permute(1, 2, 0, 3).contiguous() for t in (q, k, v))            # 'n b h d -> b h n d'
        gk = gk.view(T, B, self.H, self.D).permute(1, 2, 0, 3).contiguous()
        gk = L.gla_gate(gk, 16.0)                                                     # logsigmoid / normalizer
        q, k = F.silu(q), F.silu(k)                                                   # swish feature map
        o, _ = L.chunk_gla(q, k, v, gk)
        o = o.permute(2, 0, 1, 3).contiguous()                                        # 'b h n d -> n b h d'
        # output RMS norm over head_v_dim (gla.py:95) and o * swish(o_gate) (linear_attention.py:255) in one pass
        o = L.rms_norm_swish_gate(o, o_gate.view(T, B, self.H, self.D), self.norm_weight.to(dt), self.eps)
        return F.linear(o.reshape(T, B, self.H * self.D), self.o_proj.to(dt))

    def oracle_forward(self, x):
        T, B, _ = x.shape
        P = lambda p: p.double()
        qkv = (x @ P(self.qkv_proj).T).view(T, B, self.H, 3 * self.D)
        q, k, v = torch.split(qkv, [self.D, self.D, self.D], dim=3)
        o_gate = x @ P(self.o_gate_proj).T
        gk = (x @ P(self.gk_down).T) @ P(self.gk_up).T + P(self.gk_bias)
        q, k, v = (t.permute(1, 2, 0, 3) for t in (q, k, v))
        gk = naive.naive_gla_gate(gk.view(T, B, self.H, self.D).permute(1, 2, 0, 3), 16.0)
        q, k = F.silu(q), F.silu(k)
        o, _ = naive.naive_recurrent_gla(q, k, v, gk, None, None, False, None, True)
        o = naive.naive_rms_norm(o, P(self.norm_weight), None, self.eps)
        o = o.permute(2, 0, 1, 3).reshape(T, B, self.H * self.D)
        o = o * F.silu(o_gate)
        return o @ P(self.o_proj).T


class _CoreBase(nn.Module):
    """Shared by the three core modules below: q, k, v arrive as [T, B, H, D] (what LinearAttention.forward hands
    to ``core_linear_attention``, linear_attention.py:248-252), go to 'b h n d', and the result returns as
    'n b (h d)' behind an RMS norm over head_v_dim."""

    def __init__(self, heads: int, head_dim: int, seed: int, eps: float = 1e-5):
        super().__init__()
        g = torch.Generator().manual_seed(seed)
        self.H, self.D, self.eps = heads, head_dim, eps
        self.norm_weight = nn.Parameter(1 + 0.1 * torch.randn(head_dim, generator=g))

    @staticmethod
    def _in(x):
        return x.permute(1, 2, 0, 3)                                                  # 'n b h d -> b h n d'

    def _out(self, o, norm):
        o = norm(o)
        T = o.shape[2]
        return o.permute(2, 0, 1, 3).reshape(T, o.shape[0], self.H * self.D)          # 'b h n d -> n b (h d)'


class RetentionCore(_CoreBase):
    """Retention.forward (retention/retention.py:78-96): feature map (swish) on q, k, chunk_retention, RMSNorm."""

    def forward(self, q, k, v):
        import linear_moe_amd as L
        q, k, v = (self._in(x).contiguous() for x in (q, k, v))
        q, k = F.silu(q), F.silu(k)
        o, _ = L.chunk_retention(q, k, v)
        return self._out(o, lambda x: L.rms_norm_fn(x, self.norm_weight.to(x.dtype), None, eps=self.eps))

    def oracle_forward(self, q, k, v):
        q, k, v = (self._in(x) for x in (q, k, v))
        o, _ = naive.naive_retention(F.silu(q), F.silu(k), v)
        return self._out(o, lambda x: naive.naive_rms_norm(x, self.norm_weight.double(), None, self.eps))


class BasicLinearAttentionCore(_CoreBase):
    """BasicLinearAttention.forward (basic_linear_attention/basic_linear_attention.py:114-138) with the 'elu' feature
    map (:75-79), la_norm_q / la_norm_k (:127-130) and chunk_linear_attn(normalize=la_do_feature_map_norm) at its
    default scale (:133)."""

    def __init__(self, heads, head_dim, seed, normalize=True, norm_qk=True):
        super().__init__(heads, head_dim, seed)
        self.normalize, self.norm_qk = normalize, norm_qk

    def _maps(self, q, k):
        q, k = F.elu(q) + 1, F.elu(k) + 1
        if self.norm_qk:
            q, k = q / (q.sum(-1, True) + 1e-4), k / (k.sum(-1, True) + 1e-4)
        return q, k

    def forward(self, q, k, v):
        import linear_moe_amd as L
        q, k, v = (self._in(x).contiguous() for x in (q, k, v))
        q, k = self._maps(q, k)
        o, _ = L.chunk_linear_attn(q, k, v, normalize=self.normalize)
        return self._out(o, lambda x: L.rms_norm_fn(x, self.norm_weight.to(x.dtype), None, eps=self.eps))

    def oracle_forward(self, q, k, v):
        q, k, v = (self._in(x) for x in (q, k, v))
        q, k = self._maps(q, k)
        o, _ = naive.naive_linear_attn(q, k, v, normalize=self.normalize)
        return self._out(o, lambda x: naive.naive_rms_norm(x, self.norm_weight.double(), None, self.eps))


class LightningCore(_CoreBase):
    """LightningAttention.forward (lightning_attention/lightning_attention.py:108-126) on tensor-parallel rank `rank` of
    `tp`: the slopes of all `heads * tp` heads (:79-105), chunked per rank as :54-61 does, feature map (swish) on q, k,
    lightning_attn2(q, k, v, slope_rate), RMSNorm."""

    def __init__(self, heads, head_dim, seed, tp=1, rank=0):
        super().__init__(heads, head_dim, seed)
        slopes = naive.lightning_slopes(heads * tp).reshape(heads * tp, 1, 1)
        self.register_buffer("slope_rate", torch.chunk(slopes, tp, 0)[rank].float())

    def forward(self, q, k, v):
        import linear_moe_amd as L
        q, k, v = (self._in(x).contiguous() for x in (q, k, v))
        o = L.lightning_attn2(F.silu(q), F.silu(k), v, self.slope_rate)
        return self._out(o, lambda x: L.rms_norm_fn(x, self.norm_weight.to(x.dtype), None, eps=self.eps))

    def oracle_forward(self, q, k, v):
        q, k, v = (self._in(x) for x in (q, k, v))
        o = naive.naive_lightning_attn2(F.silu(q), F.silu(k), v, self.slope_rate.double())
        return self._out(o, lambda x: naive.naive_rms_norm(x, self.norm_weight.double(), None, self.eps))
