"""The token-mixer layer composed end to end on the GPU kernels, in the reference's order of operations
(tests/layers.py: LinearAttention.forward around GatedDeltaNet.forward / GLA.forward), forward and every gradient
(hidden states and all parameters) against the same chain of fp64 oracle functions."""
import pytest
import torch
import torch.nn.functional as F

from oracle import naive
from tests.layers import GatedDeltaNetLayer, GLALayer
from tests.util import TOL, gen, max_abs_rel

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind", ["gated_deltanet", "gla"])
def test_layer_matches_the_oracle_chain(cuda, kind, dtype):
    hidden, H, D, T, B = 256, 2, 128, 200, 2
    layer = (GatedDeltaNetLayer if kind == "gated_deltanet" else GLALayer)(hidden, H, D, seed=5)
    x = gen(5100, T, B, hidden)
    dy = gen(5101, T, B, hidden)
    # oracle: fp64 on the CPU, on the parameters and inputs as the device sees them (rounded to dtype once)
    ref_layer = (GatedDeltaNetLayer if kind == "gated_deltanet" else GLALayer)(hidden, H, D, seed=5)
    if dtype == torch.bfloat16:
        with torch.no_grad():
            for p in ref_layer.parameters():
                if p.dim() == 2 or p is getattr(ref_layer, "gk_bias", None) or p is getattr(ref_layer, "norm_weight", None):
                    p.copy_(p.to(dtype).float())            # the projections run in dtype; A_log, dt_bias stay fp32
    xr = x.to(dtype).double().requires_grad_(True)
    yr = ref_layer.oracle_forward(xr)
    ref_params = dict(ref_layer.named_parameters())
    ref_grads = torch.autograd.grad((yr * dy.double()).sum(), [xr] + list(ref_params.values()))
    layer = layer.to(cuda)
    xd = x.to(dtype).to(cuda).requires_grad_(True)
    y = layer(xd)
    assert y.shape == (T, B, hidden) and y.dtype == dtype
    grads = torch.autograd.grad((y * dy.to(dtype).to(cuda)).sum(), [xd] + list(layer.parameters()))
    torch.cuda.synchronize()
    # the bars of the ops themselves (measured over three seeds: fp32 <= 3.8e-6, bf16 <= 9.7e-3, A_log / dt_bias 1.7e-2)
    tol = TOL[dtype]
    assert max_abs_rel(y.detach().cpu(), yr.detach()) < tol
    names = ["x"] + list(ref_params)
    for n, gd, gr in zip(names, grads, ref_grads):
        # A_log, dt_bias: H numbers, each the sum of B*T signed per-token terms that cancel to a fraction of their
        # absolute sum; the rounding of every term (in bf16: dg comes through bf16 q, k, v) does not cancel with it:
        # 4e-5 / 4e-2 for these two (measured: fp32 up to 2.2e-5, bf16 1.7e-2); everything else at the bars of the ops
        t = (4 if dtype == torch.float32 else 2) * tol if n in ("A_log", "dt_bias") else tol
        err = max_abs_rel(gd.cpu(), gr)
        assert err < t, (n, err)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gdn_layer_fused_prologue_epilogue_equals_the_unfused_chain(cuda, dtype):
    """The one-pass prologue / epilogue kernels against the chain of copies, row kernels and eager ops they replace:
    the same layer output and hidden-state gradient to the rounding of the element type."""
    hidden, H, D, T, B = 256, 2, 128, 130, 2
    layer = GatedDeltaNetLayer(hidden, H, D, seed=6).to(cuda)
    x = gen(5200, T, B, hidden).to(dtype).to(cuda)
    dy = gen(5201, T, B, hidden).to(dtype).to(cuda)
    outs = []
    for fused in (True, False):
        xd = x.clone().requires_grad_(True)
        y = layer(xd, fused=fused)
        (gx,) = torch.autograd.grad((y * dy).sum(), [xd])
        outs.append((y.detach(), gx))
    torch.cuda.synchronize()
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    assert max_abs_rel(outs[0][0].cpu(), outs[1][0].cpu()) < tol
    assert max_abs_rel(outs[0][1].cpu(), outs[1][1].cpu()) < tol


@pytest.mark.parametrize("D,T,B,H", [(128, 200, 2, 3), (64, 200, 2, 3), (128, 1, 1, 1), (64, 65, 3, 2), (128, 64, 1, 2)])
def test_gdn_mixer_core_equals_prologue_then_op(cuda, D, T, B, H):
    """gdn_mixer_core (q^, k^ written, silu(v) applied where the op stages v, dv written straight into the v block of
    the projection's gradient) against gdn_qkv_prologue followed by chunk_gated_delta_rule: the same output bit for
    bit (the same q^, k^ and the same rounded silu(v) reach the same kernels), the same dg, dbeta and q / k blocks of
    the projection's gradient bit for bit, its v block to the rounding of the element type (one rounding of
    beta dZ silu'(v) instead of two)."""
    import linear_moe_amd as L
    bf = torch.bfloat16
    qkv = gen(5250, T, B, H * 3 * D).to(bf).to(cuda)
    g = (-torch.rand(B, T, H, generator=torch.Generator().manual_seed(5251)) * 0.2).to(cuda)
    beta = torch.rand(B, T, H, generator=torch.Generator().manual_seed(5252)).to(bf).to(cuda)
    do = gen(5253, B, T, H, D).to(bf).to(cuda)
    res = []
    for core in (True, False):
        leaves = [t.clone().requires_grad_(True) for t in (qkv, g, beta)]
        if core:
            o = L.gdn_mixer_core(*leaves, H, D)
        else:
            q, k, v = L.gdn_qkv_prologue(leaves[0], H, D)
            o, _ = L.chunk_gated_delta_rule(q, k, v, leaves[1], leaves[2], head_first=False)
        res.append((o.detach(), torch.autograd.grad((o * do).sum(), leaves)))
    torch.cuda.synchronize()
    (o1, g1), (o2, g2) = res
    assert o1.is_contiguous() and torch.equal(o1, o2)
    assert torch.equal(g1[1], g2[1]) and torch.equal(g1[2], g2[2])
    d1, d2 = (x.view(T, B, H, 3 * D) for x in (g1[0], g2[0]))
    assert torch.equal(d1[..., :2 * D], d2[..., :2 * D])
    assert max_abs_rel(d1[..., 2 * D:].float().cpu(), d2[..., 2 * D:].float().cpu()) < 1e-2
    # and against the oracle chain in fp64: silu'(v) times the gradient of the op with respect to silu(v)
    x64 = qkv.double().cpu().view(T, B, H, 3 * D).requires_grad_(True)
    q, k, v = (t.transpose(0, 1) for t in torch.split(x64, [D, D, D], dim=3))
    oo, _ = naive.naive_recurrent_gated_delta_rule(naive.naive_silu_l2_norm(q), naive.naive_silu_l2_norm(k), F.silu(v),
                                                   g.double().cpu(), beta.double().cpu(), None, None, False, None, False)
    (gx,) = torch.autograd.grad((oo * do.double().cpu()).sum(), [x64])
    assert max_abs_rel(o1.cpu(), oo.detach()) < TOL[bf]
    assert max_abs_rel(d1.cpu(), gx) < 4e-2


def test_gdn_layer_with_the_mixer_core(cuda):
    """The composed layer through gdn_mixer_core against the layer through prologue + op (bfloat16)."""
    hidden, H, D, T, B = 256, 2, 128, 130, 2
    layer = GatedDeltaNetLayer(hidden, H, D, seed=6).to(cuda)
    x = gen(5200, T, B, hidden).to(torch.bfloat16).to(cuda)
    dy = gen(5201, T, B, hidden).to(torch.bfloat16).to(cuda)
    outs = []
    for core in (True, False):
        xd = x.clone().requires_grad_(True)
        y = layer(xd, fused=True, core=core)
        outs.append((y.detach(), torch.autograd.grad((y * dy).sum(), [xd] + list(layer.parameters()))))
    torch.cuda.synchronize()
    assert torch.equal(outs[0][0], outs[1][0])
    for a, b in zip(outs[0][1], outs[1][1]):
        assert max_abs_rel(a.float().cpu(), b.float().cpu()) < 1e-2


CORES = {
    "retention": lambda: __import__("tests.layers", fromlist=["x"]).RetentionCore(4, 64, seed=7),
    "basic_normalized": lambda: __import__("tests.layers", fromlist=["x"]).BasicLinearAttentionCore(3, 64, seed=8),
    "basic_plain": lambda: __import__("tests.layers", fromlist=["x"]).BasicLinearAttentionCore(3, 64, seed=8, normalize=False, norm_qk=False),
    "lightning_tp2_rank1": lambda: __import__("tests.layers", fromlist=["x"]).LightningCore(6, 128, seed=9, tp=2, rank=1),
}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind", list(CORES))
def test_core_modules_of_the_other_dispatch_branches(cuda, kind, dtype):
    """The core modules LinearAttention.forward dispatches to besides the gated delta rule and GLA
    (linear_attention.py:218-252): Retention, BasicLinearAttention (with and without the feature-map normalisation and
    the normaliser of chunk_linear_attn at its default scale), LightningAttention with the slopes of one tensor-parallel
    rank -- each in the reference's order of operations on the GPU kernels, output and dq, dk, dv and the norm weight
    against the same chain of fp64 oracle functions."""
    core = CORES[kind]()
    T, B, H, D = 150, 2, core.H, core.D
    q, k, v = (gen(5300 + i, T, B, H, D).to(dtype) for i in range(3))
    dy = gen(5303, T, B, H * D).to(dtype)
    ref_core = CORES[kind]()
    if dtype == torch.bfloat16:
        with torch.no_grad():
            ref_core.norm_weight.copy_(ref_core.norm_weight.to(dtype).float())
    lr = [x.double().requires_grad_(True) for x in (q, k, v)]
    yr = ref_core.oracle_forward(*lr)
    gr = torch.autograd.grad((yr * dy.double()).sum(), lr + [ref_core.norm_weight])
    core = core.to(cuda)
    ld = [x.to(cuda).requires_grad_(True) for x in (q, k, v)]
    y = core(*ld)
    assert y.shape == (T, B, H * D) and y.dtype == dtype
    gd = torch.autograd.grad((y * dy.to(cuda)).sum(), ld + [core.norm_weight])
    torch.cuda.synchronize()
    # the bars of the ops; lightning attention in bf16: twice that (its slopes reach e^-8 per token on the last heads,
    # the outputs of those heads are sums of a few tokens, and the rounding of q and k to bf16 is 3.6e-2 of dq, dk)
    tol = 2 * TOL[dtype] if (kind.startswith("lightning") and dtype == torch.bfloat16) else TOL[dtype]
    errs = {"y": max_abs_rel(y.detach().cpu(), yr.detach())}
    for n, a, b in zip(("dq", "dk", "dv", "dw"), gd, gr):
        errs[n] = max_abs_rel(a.cpu(), b)
    print(kind, dtype, {n: f"{e:.1e}" for n, e in errs.items()})
    for n, e in errs.items():
        assert e < tol, (n, e)
