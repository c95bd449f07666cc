"""GPU parity of the token-by-token (fused_recurrent_*) forward, through the C ABI, against the fp64
recurrences: decoding steps (T = 1 with state hand-off), short and chunk-crossing sequences, packed input."""
import pytest
import torch
import torch.nn.functional as F

from oracle import naive
from tests.test_gpu_gdn import gdn_inputs
from tests.util import TOL, gen, max_abs_rel

pytestmark = pytest.mark.gpu

# T <= 4 tokens per sequence take the decoding-step kernel, longer ones the token-block kernel
SHAPES = [(2, 1, 3, 64, 128), (2, 3, 2, 128, 128), (1, 4, 3, 64, 64), (1, 7, 2, 128, 64), (2, 70, 2, 128, 128),
          (1, 130, 2, 64, 64)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("gated", [True, False])
def test_recurrent_gated_delta_rule(cuda, dtype, shape, gated):
    from linear_moe_amd import fused_recurrent_delta_rule, fused_recurrent_gated_delta_rule
    B, T, H, K, V = shape
    q, k, v, g, beta = gdn_inputs(2100 + T, B, T, H, K, V, dtype, False, True)
    h0 = 0.3 * gen(2107, B, H, K, V)
    ref_o, ref_ht = naive.naive_recurrent_gated_delta_rule(q, k, v, g if gated else None, beta, None, h0, True, None, False)
    d = lambda x: x.to(cuda)
    if gated:
        o, ht = fused_recurrent_gated_delta_rule(d(q), d(k), d(v), d(g), d(beta), initial_state=d(h0),
                                                 output_final_state=True)
    else:
        hf = lambda x: x.transpose(1, 2)
        o, ht = fused_recurrent_delta_rule(hf(d(q)), hf(d(k)), hf(d(v)), hf(d(beta)), initial_state=d(h0),
                                           output_final_state=True)
        o = o.transpose(1, 2)
    torch.cuda.synchronize()
    assert o.dtype == dtype and ht.dtype == torch.float32
    assert max_abs_rel(o.cpu(), ref_o) < TOL[dtype]
    assert max_abs_rel(ht.cpu(), ref_ht) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("gate", ["none", "scalar", "vector"])
def test_recurrent_simple_gla_and_gla(cuda, dtype, shape, gate):
    from linear_moe_amd import fused_recurrent_gla, fused_recurrent_simple_gla
    B, T, H, K, V = shape
    q, k = gen(2200 + T, B, H, T, K, dtype=dtype), gen(2201 + T, B, H, T, K, dtype=dtype)
    v = gen(2202 + T, B, H, T, V, dtype=dtype)
    h0 = 0.3 * gen(2203, B, H, K, V)
    d = lambda x: x.to(cuda)
    if gate == "vector":
        g = (F.logsigmoid(gen(2204 + T, B, H, T, K)) / 4).to(dtype)
        ref_o, ref_ht = naive.naive_recurrent_gla(q, k, v, g, None, h0, True)
        o, ht = fused_recurrent_gla(d(q), d(k), d(v), d(g), initial_state=d(h0), output_final_state=True)
    else:
        g = F.logsigmoid(gen(2205 + T, B, H, T)) / 4 if gate == "scalar" else None
        ref_o, ref_ht = naive.naive_recurrent_simple_gla(q, k, v, g, None, h0, True)
        o, ht = fused_recurrent_simple_gla(d(q), d(k), d(v), None if g is None else d(g), initial_state=d(h0),
                                           output_final_state=True)
    torch.cuda.synchronize()
    assert max_abs_rel(o.cpu(), ref_o) < TOL[dtype]
    assert max_abs_rel(ht.cpu(), ref_ht) < TOL[dtype]


def test_recurrent_decode_steps_continue_a_chunked_prefill(cuda):
    """Prefill with the chunk kernels, then decode token by token through h0 / ht: the same outputs
    as one pass over the whole sequence."""
    from linear_moe_amd import chunk_gated_delta_rule, fused_recurrent_gated_delta_rule
    B, T, H, K, V = 2, 100, 2, 128, 128
    q, k, v, g, beta = (x.to(cuda) for x in gdn_inputs(2300, B, T + 3, H, K, V, torch.float32, False, True))
    full_o, full_ht = chunk_gated_delta_rule(q, k, v, g, beta, output_final_state=True)
    o, st = chunk_gated_delta_rule(q[:, :T], k[:, :T], v[:, :T], g[:, :T], beta[:, :T], output_final_state=True)
    outs = [o]
    for t in range(T, T + 3):
        s = slice(t, t + 1)
        o1, st = fused_recurrent_gated_delta_rule(q[:, s], k[:, s], v[:, s], g[:, s], beta[:, s], initial_state=st,
                                                  output_final_state=True)
        outs.append(o1)
    torch.cuda.synchronize()
    assert max_abs_rel(torch.cat(outs, 1).cpu(), full_o.cpu()) < 1e-5
    assert max_abs_rel(st.cpu(), full_ht.cpu()) < 1e-5


def test_recurrent_packed_input_and_grad_route(cuda):
    from linear_moe_amd import fused_recurrent_gated_delta_rule
    H, K, V = 2, 64, 64
    lens = [1, 64, 135, 5]
    T = sum(lens)
    cu = torch.tensor([0, 1, 65, 200, 205], dtype=torch.int32)
    q, k, v, g, beta = gdn_inputs(2400, 1, T, H, K, V, torch.float32, False, True)
    h0 = 0.2 * gen(2401, len(lens), H, K, V)
    ref_o, ref_ht = naive.naive_recurrent_gated_delta_rule(q, k, v, g, beta, None, h0, True, cu, False)
    d = lambda x: x.to(cuda)
    o, ht = fused_recurrent_gated_delta_rule(d(q), d(k), d(v), d(g), d(beta), initial_state=d(h0),
                                             output_final_state=True, cu_seqlens=d(cu))
    assert max_abs_rel(o.cpu(), ref_o) < 1e-5 and max_abs_rel(ht.cpu(), ref_ht) < 1e-5
    # a call that needs a gradient runs the chunk kernels (same function, differentiable)
    qd = d(q).requires_grad_(True)
    o2, _ = fused_recurrent_gated_delta_rule(qd, d(k), d(v), d(g), d(beta), cu_seqlens=d(cu))
    o2.sum().backward()
    assert qd.grad is not None and max_abs_rel(o2.detach().cpu(), naive.naive_recurrent_gated_delta_rule(
        q, k, v, g, beta, None, None, False, cu, False)[0]) < 1e-5
