"""Shared helpers of the parity tests: seeded inputs and the two error measures used."""
import math

import torch


def max_abs_rel(x: torch.Tensor, ref: torch.Tensor) -> float:
    """max|x - ref| / max|ref|  -- the bf16 tolerance of the contract is 2e-2 on this measure."""
    ref = ref.double()
    return ((x.double() - ref).abs().max() / ref.abs().max().clamp_min(1e-30)).item()


def rms_rel(x: torch.Tensor, ref: torch.Tensor) -> float:
    ref = ref.double()
    return ((x.double() - ref).pow(2).mean().sqrt() / ref.pow(2).mean().sqrt().clamp_min(1e-30)).item()


def gen(seed: int, *shape, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=torch.float32).to(dtype)


TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2}


def oracle_grads(fn, inputs, do, dht):
    """Gradients of sum(o*do) + sum(ht*dht) through an oracle function, in float64.
    ``inputs``: dict name -> tensor or None; returns (o, ht, dict name -> grad)."""
    leaves = {k: v.detach().double().requires_grad_(True) for k, v in inputs.items() if v is not None}
    o, ht = fn(**{k: leaves.get(k) for k in inputs})
    loss = (o * do.double()).sum()
    if dht is not None:
        loss = loss + (ht * dht.double()).sum()
    grads = torch.autograd.grad(loss, list(leaves.values()))
    return o.detach(), ht.detach(), dict(zip(leaves.keys(), grads))
