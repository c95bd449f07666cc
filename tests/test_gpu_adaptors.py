"""GPU parity of the thin adaptors over chunk_simple_gla, called exactly as the reference's modules call them:
lightning_attn2 / lightning_attn2_no_decay (linear_moe/sequence_modeling/lightning_attention/
lightning_attention.py:121-123) and chunk_linear_attn with its normaliser (basic_linear_attention.py:133)."""
import pytest
import torch

from oracle import naive
from tests.util import TOL, gen, max_abs_rel

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H", [16, 12])          # a power of two and the interleaved completion of the slopes
def test_lightning_attn2_fwd_bwd(cuda, dtype, H):
    """lightning_attn2(q, k, v, slope[H,1,1]) -> o only; [B,H,T,D]; no scale; forward and dq, dk, dv."""
    from linear_moe_amd.lightning import lightning_attn2
    B, T, K, V = 2, 200, 64, 128
    q, k = 0.3 * gen(3101, B, H, T, K, dtype=dtype), 0.3 * gen(3102, B, H, T, K, dtype=dtype)
    v, do = gen(3103, B, H, T, V, dtype=dtype), gen(3104, B, H, T, V, dtype=dtype)
    slope = naive.lightning_slopes(H).float().reshape(H, 1, 1)
    ref_in = [x.double().requires_grad_(True) for x in (q, k, v)]
    ref = naive.naive_lightning_attn2(*ref_in, slope)
    ref_g = torch.autograd.grad((ref * do.double()).sum(), ref_in)
    dev_in = [x.to(cuda).requires_grad_(True) for x in (q, k, v)]
    o = lightning_attn2(*dev_in, slope.to(cuda))
    assert isinstance(o, torch.Tensor) and o.shape == v.shape and o.dtype == dtype
    grads = torch.autograd.grad((o * do.to(cuda)).sum(), dev_in)
    torch.cuda.synchronize()
    assert max_abs_rel(o.detach().cpu(), ref.detach()) < TOL[dtype]
    for gd, gr, n in zip(grads, ref_g, "qkv"):
        assert max_abs_rel(gd.cpu(), gr) < TOL[dtype], n


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_lightning_attn2_no_decay(cuda, dtype):
    from linear_moe_amd.lightning import lightning_attn2_no_decay
    B, H, T, K, V = 1, 3, 130, 128, 64
    q, k = 0.3 * gen(3111, B, H, T, K, dtype=dtype), 0.3 * gen(3112, B, H, T, K, dtype=dtype)
    v = gen(3113, B, H, T, V, dtype=dtype)
    ref = torch.tril(q.double() @ k.double().transpose(-1, -2)) @ v.double()
    o = lightning_attn2_no_decay(q.to(cuda), k.to(cuda), v.to(cuda))
    torch.cuda.synchronize()
    assert isinstance(o, torch.Tensor)
    assert max_abs_rel(o.cpu(), ref) < TOL[dtype]


@pytest.mark.parametrize("scale", [None, 1.0])
@pytest.mark.parametrize("head_first", [True, False])
def test_linear_attn_normalised_default_scale(cuda, scale, head_first):
    """chunk_linear_attn(q, k, v, normalize=True) with the default scale K^-0.5, as BasicLinearAttention calls it
    with la_do_feature_map_norm: o_t = sum a_ts v_s / (sum a_ts + eps), a_ts = scale q_t.k_s, checked against the
    closed form written out here (not the oracle's expression) and against the oracle; forward and gradients."""
    from linear_moe_amd import chunk_linear_attn
    B, H, T, K, V = 2, 2, 150, 64, 64
    # positive features (the reference's feature maps are positive: elu+1, relu, ...), so the normaliser is not tiny
    q, k = gen(3201, B, H, T, K).abs() + 0.1, gen(3202, B, H, T, K).abs() + 0.1
    v, do = gen(3203, B, H, T, V), gen(3204, B, H, T, V)
    sc = K ** -0.5 if scale is None else scale
    ref_in = [x.double().requires_grad_(True) for x in (q, k, v)]
    A = torch.tril(sc * ref_in[0] @ ref_in[1].transpose(-1, -2))
    ref = (A @ ref_in[2]) / (A.sum(-1, keepdim=True) + 1e-10)
    ref_g = torch.autograd.grad((ref * do.double()).sum(), ref_in)
    o_or, _ = naive.naive_linear_attn(q, k, v, scale=scale, normalize=True)
    assert torch.allclose(o_or, ref.detach(), atol=1e-12)
    tf = (lambda x: x) if head_first else (lambda x: x.transpose(1, 2).contiguous())
    dev_in = [tf(x).to(cuda).requires_grad_(True) for x in (q, k, v)]
    o, ht = chunk_linear_attn(*dev_in, scale=scale, normalize=True, head_first=head_first)
    grads = torch.autograd.grad((o * tf(do).to(cuda)).sum(), dev_in)
    torch.cuda.synchronize()
    assert ht is None
    assert max_abs_rel(tf(o.detach().cpu()), ref.detach()) < 1e-5
    for gd, gr, n in zip(grads, ref_g, "qkv"):
        assert max_abs_rel(tf(gd.cpu()), gr) < 1e-5, n


def _normalised_closed_form(q, k, v, h0, do, dht, sc, lens=None, eps=1e-10):
    """fp64: o_t = (sum_s a_ts v_s + sc q_t h0) / (sum_s a_ts + eps), a_ts = sc q_t.k_s [s <= t]; [B,H,T,*] inputs
    (lens: the sequences packed along T of a batch of one).  Returns o, final state and their gradients."""
    ins = [x.double().requires_grad_(True) for x in (q, k, v, h0)]
    qd, kd, vd, hd = ins
    T = q.shape[2]
    bounds = [0, T] if lens is None else [0] + list(torch.tensor(lens).cumsum(0))
    os_, hts = [], []
    for n in range(len(bounds) - 1):
        a0, a1 = int(bounds[n]), int(bounds[n + 1])
        hn = hd if lens is None else hd[n:n + 1]
        A = torch.tril(sc * qd[:, :, a0:a1] @ kd[:, :, a0:a1].transpose(-1, -2))
        os_.append((A @ vd[:, :, a0:a1] + sc * qd[:, :, a0:a1] @ hn) / (A.sum(-1, keepdim=True) + eps))
        hts.append(hn + kd[:, :, a0:a1].transpose(-1, -2) @ vd[:, :, a0:a1])
    o, ht = torch.cat(os_, 2), torch.cat(hts, 0)
    grads = torch.autograd.grad((o * do.double()).sum() + (ht * dht.double()).sum(), ins)
    return o.detach(), ht.detach(), grads


@pytest.mark.parametrize("head_first", [True, False])
@pytest.mark.parametrize("shape", [(2, 3, 333, 64, 64), (2, 2, 200, 128, 128), (1, 3, 130, 64, 128), (1, 2, 70, 128, 64),
                                   (4, 32, 130, 128, 128), (8, 32, 65, 64, 64), (1, 2, 100, 96, 80), (1, 2, 66, 32, 16)])
def test_linear_attn_normalised_inside_the_kernels(cuda, shape, head_first):
    """bfloat16 with one key block: the kernels carry the sum of the keys beside the state and divide before they
    store; the backward folds the gradient of the divisor into its own sums.  Against the closed form in fp64 on the
    same bf16 inputs, output, final state and every gradient (shapes five and six run the 64-column slices of the
    state passes, the others the 32-column ones; the last two have head dimensions the host pads)."""
    from linear_moe_amd import chunk_linear_attn
    B, H, T, K, V = shape
    bf = torch.bfloat16
    q, k = (gen(3301, B, H, T, K).abs() + 0.1).to(bf), (gen(3302, B, H, T, K).abs() + 0.1).to(bf)
    v, do = gen(3303, B, H, T, V, dtype=bf), gen(3304, B, H, T, V, dtype=bf)
    h0, dht = gen(3305, B, H, K, V) * 0.5, gen(3306, B, H, K, V)
    sc = K ** -0.5
    ref_o, ref_ht, ref_g = _normalised_closed_form(q, k, v, h0, do, dht, sc)
    tf = (lambda x: x) if head_first else (lambda x: x.transpose(1, 2).contiguous())
    dev_in = [tf(x).to(cuda).requires_grad_(True) for x in (q, k, v)] + [h0.to(cuda).requires_grad_(True)]
    o, ht = chunk_linear_attn(*dev_in[:3], initial_state=dev_in[3], output_final_state=True, normalize=True,
                              head_first=head_first)
    grads = torch.autograd.grad((o * tf(do).to(cuda)).sum() + (ht * dht.to(cuda)).sum(), dev_in)
    torch.cuda.synchronize()
    assert o.dtype == bf
    assert max_abs_rel(tf(o.detach().cpu()), ref_o) < TOL[bf]
    assert max_abs_rel(ht.detach().cpu(), ref_ht) < TOL[bf]
    for gd, gr, n in zip(grads, ref_g, ("q", "k", "v", "h0")):
        gd = gd.cpu() if n == "h0" else tf(gd.cpu())
        assert max_abs_rel(gd, gr) < TOL[bf], n


def test_normalised_op_on_packed_sequences_and_forward_only(cuda):
    """The normalised op on sequences packed along T (the sum of the keys starts anew in every sequence), and a
    forward-only call (nothing saved) giving the bits of the saving one."""
    from linear_moe_amd.simple_gla import chunk_simple_gla_normalized
    lens, H, K, V = [70, 1, 129, 64], 2, 128, 128
    T, N, bf = sum(lens), len(lens), torch.bfloat16
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    q, k = (gen(3401, 1, H, T, K).abs() + 0.1).to(bf), (gen(3402, 1, H, T, K).abs() + 0.1).to(bf)
    v, do = gen(3403, 1, H, T, V, dtype=bf), gen(3404, 1, H, T, V, dtype=bf)
    h0, dht = gen(3405, N, H, K, V) * 0.5, gen(3406, N, H, K, V)
    ref_o, ref_ht, ref_g = _normalised_closed_form(q, k, v, h0, do, dht, K ** -0.5, lens)
    tf = lambda x: x.transpose(1, 2).contiguous()
    dev_in = [tf(x).to(cuda).requires_grad_(True) for x in (q, k, v)] + [h0.to(cuda).requires_grad_(True)]
    o, ht = chunk_simple_gla_normalized(*dev_in[:3], None, dev_in[3], True, cu.to(cuda), False)
    grads = torch.autograd.grad((o * tf(do).to(cuda)).sum() + (ht * dht.to(cuda)).sum(), dev_in)
    with torch.no_grad():
        o2, ht2 = chunk_simple_gla_normalized(*dev_in[:3], None, dev_in[3], True, cu.to(cuda), False)
    torch.cuda.synchronize()
    assert torch.equal(o2, o.detach()) and torch.equal(ht2, ht.detach())
    assert max_abs_rel(tf(o.detach().cpu()), ref_o) < TOL[bf]
    assert max_abs_rel(ht.detach().cpu(), ref_ht) < TOL[bf]
    for gd, gr, n in zip(grads, ref_g, ("q", "k", "v", "h0")):
        gd = gd.cpu() if n == "h0" else tf(gd.cpu())
        assert max_abs_rel(gd, gr) < TOL[bf], n


@pytest.mark.parametrize("shape", [(2, 2, 200, 128, 128), (8, 32, 70, 64, 64)])
def test_op_with_den_as_a_second_output(cuda, shape):
    """chunk_simple_gla_with_den: o undivided and den = scale q . cumsum(k) beside it, each with a gradient of its own
    (what chunk_linear_attn(normalize=True) over several key blocks is built from), against the closed form in fp64."""
    from linear_moe_amd.simple_gla import chunk_simple_gla_with_den
    B, H, T, K, V = shape
    bf = torch.bfloat16
    q, k = (gen(3501, B, H, T, K).abs() + 0.1).to(bf), (gen(3502, B, H, T, K).abs() + 0.1).to(bf)
    v, do = gen(3503, B, H, T, V, dtype=bf), gen(3504, B, H, T, V, dtype=bf)
    dd = gen(3505, B, H, T)
    sc = K ** -0.5
    ins = [x.double().requires_grad_(True) for x in (q, k, v)]
    A = torch.tril(sc * ins[0] @ ins[1].transpose(-1, -2))
    ref_o, ref_den = A @ ins[2], A.sum(-1)
    ref_g = torch.autograd.grad((ref_o * do.double()).sum() + (ref_den * dd.double()).sum(), ins)
    dev_in = [x.to(cuda).requires_grad_(True) for x in (q, k, v)]
    o, den, ht = chunk_simple_gla_with_den(*dev_in)
    grads = torch.autograd.grad((o * do.to(cuda)).sum() + (den * dd.to(cuda)).sum(), dev_in)
    torch.cuda.synchronize()
    assert ht is None and den.dtype == torch.float32 and den.shape == (B, H, T)
    assert max_abs_rel(o.detach().cpu(), ref_o.detach()) < TOL[bf]
    assert max_abs_rel(den.detach().cpu(), ref_den.detach()) < TOL[bf]
    for gd, gr, n in zip(grads, ref_g, "qkv"):
        assert max_abs_rel(gd.cpu(), gr) < TOL[bf], n
    # den alone (o unused): the gradient of o is zero
    dev_in = [x.to(cuda).requires_grad_(True) for x in (q, k, v)]
    _, den, _ = chunk_simple_gla_with_den(*dev_in)
    gq, gk = torch.autograd.grad((den * dd.to(cuda)).sum(), dev_in[:2])
    rq, rk = torch.autograd.grad((torch.tril(sc * ins[0] @ ins[1].transpose(-1, -2)).sum(-1) * dd.double()).sum(), ins[:2])
    assert max_abs_rel(gq.cpu(), rq) < TOL[bf] and max_abs_rel(gk.cpu(), rk) < TOL[bf]
