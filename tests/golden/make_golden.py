#!/usr/bin/env python3
"""Writes the golden fixtures tests/golden/*.npz from the float64 token-recurrence oracle
(oracle/naive.py) and torch.autograd.  The reference holds no vectors for this path, so these
are the build's own known-answer files: small seeded cases (one full and one partial chunk,
initial state in, final state out, one packed variable-length case) with outputs and all
gradients, stored as float32.  Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch
import torch.nn.functional as F

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import naive  # noqa: E402

OUT = os.path.dirname(os.path.abspath(__file__))


def rnd(seed, *shape):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float32)


def case(op, seed, B, T, H, K, V, cu=None):
    """Time-first [B,T,H,*] inputs, rounded to bf16-representable values so that the bf16 and
    the fp32 kernels consume bit-identical numbers."""
    r16 = lambda x: x.to(torch.bfloat16).to(torch.float32)
    q, k, v = r16(rnd(seed, B, T, H, K)), r16(rnd(seed + 1, B, T, H, K)), r16(rnd(seed + 2, B, T, H, V))
    N = B if cu is None else len(cu) - 1
    h0 = rnd(seed + 3, N, H, K, V) * 0.3
    do, dht = r16(rnd(seed + 4, B, T, H, V)), rnd(seed + 5, N, H, K, V)
    ins = dict(q=q, k=k, v=v, h0=h0)
    if op == 'gla':
        ins['g'] = r16(F.logsigmoid(rnd(seed + 6, B, T, H, K)) / 4)
    else:
        ins['g'] = F.logsigmoid(rnd(seed + 6, B, T, H))
    if op == 'gdn':
        ins['q'], ins['k'] = r16(F.normalize(q, dim=-1)), r16(F.normalize(k, dim=-1))
        ins['beta'] = r16(torch.sigmoid(rnd(seed + 7, B, T, H)))
    leaves = {n: x.double().requires_grad_(True) for n, x in ins.items()}
    cut = None if cu is None else torch.tensor(cu)
    if op == 'simple_gla':
        o, ht = naive.naive_recurrent_simple_gla(leaves['q'], leaves['k'], leaves['v'], leaves['g'], None,
                                                 leaves['h0'], True, cut, False)
    elif op == 'gla':
        o, ht = naive.naive_recurrent_gla(leaves['q'], leaves['k'], leaves['v'], leaves['g'], None, leaves['h0'],
                                          True, cut, False)
    else:
        o, ht = naive.naive_recurrent_gated_delta_rule(leaves['q'], leaves['k'], leaves['v'], leaves['g'],
                                                       leaves['beta'], None, leaves['h0'], True, cut, False)
    grads = torch.autograd.grad((o * do.double()).sum() + (ht * dht.double()).sum(), list(leaves.values()))
    out = {f"in_{n}": x.numpy() for n, x in ins.items()}
    out.update(in_do=do.numpy(), in_dht=dht.numpy(), out_o=o.detach().float().numpy(),
               out_ht=ht.detach().float().numpy())
    out.update({f"grad_{n}": gx.float().numpy() for n, gx in zip(leaves.keys(), grads)})
    if cu is not None:
        out['cu_seqlens'] = np.asarray(cu, dtype=np.int32)
    return out


def main():
    specs = [
        ('simple_gla_dense', 'simple_gla', 11, 1, 70, 1, 64, 64, None),
        ('gla_dense', 'gla', 21, 1, 70, 1, 64, 64, None),
        ('gdn_dense', 'gdn', 31, 1, 70, 1, 64, 64, None),
        ('gdn_varlen', 'gdn', 41, 1, 75, 1, 64, 64, [0, 1, 66, 75]),
    ]
    for name, op, seed, B, T, H, K, V, cu in specs:
        np.savez(os.path.join(OUT, name + '.npz'), **case(op, seed, B, T, H, K, V, cu))
        print('wrote', name)


if __name__ == '__main__':
    main()
