"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py).
CPU: the oracles still reproduce them (token recurrence in fp64, chunked restatement in fp32).
GPU: the HIP kernels reproduce them through the C ABI, in fp32 (1e-5) and bf16 (2e-2)."""
import os

import numpy as np
import pytest
import torch

from oracle import chunked, naive
from tests.util import TOL, max_abs_rel

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
FILES = {"simple_gla_dense": "simple_gla", "gla_dense": "gla", "gdn_dense": "gdn", "gdn_varlen": "gdn"}


def load(name):
    z = np.load(os.path.join(GOLD, name + ".npz"), allow_pickle=False)
    return {k: torch.from_numpy(z[k]) for k in z.files}


def run_naive(op, d, dtype=torch.float64):
    cu = d.get("cu_seqlens")
    a = (d["in_q"], d["in_k"], d["in_v"], d["in_g"])
    if op == "simple_gla":
        return naive.naive_recurrent_simple_gla(*a, None, d["in_h0"], True, cu, False, dtype)
    if op == "gla":
        return naive.naive_recurrent_gla(*a, None, d["in_h0"], True, cu, False, dtype)
    return naive.naive_recurrent_gated_delta_rule(*a, d["in_beta"], None, d["in_h0"], True, cu, False, dtype=dtype)


@pytest.mark.parametrize("name", list(FILES))
def test_oracle_reproduces_golden(name):
    d = load(name)
    o, ht = run_naive(FILES[name], d)
    assert max_abs_rel(o, d["out_o"]) < 1e-6 and max_abs_rel(ht, d["out_ht"]) < 1e-6


@pytest.mark.parametrize("name", ["simple_gla_dense", "gla_dense", "gdn_dense"])
def test_chunked_port_reproduces_golden(name):
    d, op = load(name), FILES[name]
    tp = lambda x: x.transpose(1, 2).contiguous()
    beta = tp(d["in_beta"]) if op == "gdn" else None
    o, ht, (dq, dk, dv, dg, dbeta, dh0) = chunked.chunk_fwd_bwd(
        op, tp(d["in_q"]), tp(d["in_k"]), tp(d["in_v"]), tp(d["in_g"]), beta, None, d["in_h0"], tp(d["in_do"]),
        d["in_dht"], dtype=torch.float32)
    got = dict(out_o=tp(o), out_ht=ht, grad_q=tp(dq), grad_k=tp(dk), grad_v=tp(dv), grad_g=tp(dg), grad_h0=dh0)
    if op == "gdn":
        got["grad_beta"] = tp(dbeta)
    for k, x in got.items():
        assert max_abs_rel(x, d[k]) < 2e-4, k


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", list(FILES))
def test_hip_reproduces_golden(cuda, name, dtype):
    import linear_moe_amd as L
    d, op = load(name), FILES[name]
    cu = d.get("cu_seqlens")
    dev = {}
    for n in ("q", "k", "v", "g", "beta", "h0"):
        if "in_" + n in d:
            x = d["in_" + n]
            # inputs are bf16-representable, so both dtypes see identical numbers
            x = x.to(dtype) if n in ("q", "k", "v", "beta") or (n == "g" and op == "gla") else x
            dev[n] = x.to(cuda).requires_grad_(True)
    cud = None if cu is None else cu.to(cuda)
    if op == "simple_gla":
        o, ht = L.chunk_simple_gla(dev["q"], dev["k"], dev["v"], dev["g"], None, dev["h0"], True, cud, False)
    elif op == "gla":
        o, ht = L.chunk_gla(dev["q"], dev["k"], dev["v"], dev["g"], None, dev["h0"], True, cud, False)
    else:
        o, ht = L.chunk_gated_delta_rule(dev["q"], dev["k"], dev["v"], dev["g"], dev["beta"], None, dev["h0"], True,
                                         cud, False)
    ((o * d["in_do"].to(dtype).to(cuda)).sum() + (ht * d["in_dht"].to(cuda)).sum()).backward()
    torch.cuda.synchronize()
    tol = TOL[dtype]
    assert max_abs_rel(o.detach().cpu(), d["out_o"]) < tol
    assert max_abs_rel(ht.detach().cpu(), d["out_ht"]) < tol
    for n, x in dev.items():
        err = max_abs_rel(x.grad.cpu(), d["grad_" + n])
        assert err < tol, (n, err)
