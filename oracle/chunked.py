"""CPU oracle, chunked form (C = 64) with a hand-written backward.

TEST INFRASTRUCTURE ONLY (checker + the timed ``cpu_baseline`` of ``bench.py``);
the shipped package never imports it.

This file restates, in plain torch on the CPU, the *chunk* algorithms that
flash-linear-attention's ``chunk_simple_gla`` / ``chunk_gla`` /
``chunk_gated_delta_rule`` implement (the functions the reference calls at
``linear_moe/sequence_modeling/gla/gla.py:94``,
``.../retention/retention.py:91``,
``.../basic_linear_attention/basic_linear_attention.py:133`` and
``.../gated_deltanet/gated_deltanet.py:112``).  It has the same pass structure
as the HIP kernels (chunk-parallel preparation, sequential state pass,
chunk-parallel output; reverse state pass and chunk-parallel gradient pass), so
each kernel can be checked stage by stage.  It is itself pinned against
``oracle/naive.py`` (token recurrences) and ``torch.autograd`` in
``tests/test_oracle_pins.py``.

Layout inside this file: head-first ``[B, H, T, D]``; ``T`` is padded to a
multiple of the chunk with zero tokens (zero q,k,v,beta and zero log-decay leave
the state untouched).
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn.functional as F

Tensor = torch.Tensor
CHUNK = 64


def _pad_t(x: Tensor, C: int) -> Tensor:
    T = x.shape[2]
    pad = (-T) % C
    if pad == 0:
        return x
    if x.dim() == 3:
        return F.pad(x, (0, pad))
    return F.pad(x, (0, 0, 0, pad))


def _chunks(x: Tensor, C: int) -> Tensor:
    # [B,H,T,...] -> [B,H,NT,C,...]
    B, H, T = x.shape[:3]
    return x.reshape(B, H, T // C, C, *x.shape[3:])


def _tril(C, dtype, diag=0):
    return torch.tril(torch.ones(C, C, dtype=dtype), diagonal=diag)


# --------------------------------------------------------------------------- #
# forward
# --------------------------------------------------------------------------- #
def _gate_terms(g: Optional[Tensor], B, H, NT, C, K, dtype, vector: bool):
    """Chunk-local inclusive cumsum b and the derived decay factors."""
    if g is None:
        b = torch.zeros(B, H, NT, C, dtype=dtype)
    else:
        b = g.cumsum(3)
    bC = b[:, :, :, -1:]                      # [..,1] or [..,1,K]
    return b, bC


def chunk_forward(op: str, q, k, v, g=None, beta=None, scale=None, h0=None, C: int = CHUNK,
                  dtype=torch.float32):
    """Returns (o [B,H,T,V], final state [B,H,K,V], saved dict for the backward)."""
    assert op in ('simple_gla', 'gla', 'gdn')
    B, H, T, K = q.shape
    V = v.shape[-1]
    scale = K ** -0.5 if scale is None else scale
    q, k, v = (_pad_t(x.to(dtype), C) for x in (q, k, v))
    g = None if g is None else _pad_t(g.to(dtype), C)
    beta = None if beta is None else _pad_t(beta.to(dtype), C)
    Tp = q.shape[2]
    NT = Tp // C
    qc, kc, vc = _chunks(q, C), _chunks(k, C), _chunks(v, C)
    gc = None if g is None else _chunks(g, C)
    vector = op == 'gla'
    b, bC = _gate_terms(gc, B, H, NT, C, K, dtype, vector)
    mask_d = _tril(C, dtype)          # i >= j
    mask_s = _tril(C, dtype, -1)      # i >  j

    if vector:
        e_b = b.exp()                                   # [B,H,NT,C,K]
        e_d = (bC - b).exp()                            # [B,H,NT,C,K]
        decay = bC.exp().squeeze(3)                     # [B,H,NT,K]
        # A_ij = sum_k q_ik k_jk e^{b_ik - b_jk}, i >= j (exponent formed per pair: <= 0)
        diff = b[:, :, :, :, None, :] - b[:, :, :, None, :, :]          # [..,C,C,K]
        diff = diff * mask_d[:, :, None]                                # zero the masked part
        P = torch.einsum('bhnik,bhnjk,bhnijk->bhnij', qc, kc, diff.exp()) * mask_d
    else:
        e_b = b.exp()[..., None]                        # [B,H,NT,C,1]
        e_d = (bC - b).exp()[..., None]
        decay = bC.exp().squeeze(3)                     # [B,H,NT]
        Gam = ((b[..., :, None] - b[..., None, :]) * mask_d).exp() * mask_d
        P = (qc @ kc.transpose(-1, -2)) * Gam

    saved = dict(b=b)
    if op == 'gdn':
        bc = _chunks(beta, C)[..., None]
        k_b, v_b = kc * bc, vc * bc
        Gam_s = Gam * mask_s
        M = k_b @ kc.transpose(-1, -2)
        L = M * Gam_s
        eye = torch.eye(C, dtype=dtype)
        # T = (I + L)^-1 by forward substitution (unit lower triangular)
        Tm = torch.linalg.solve_triangular(eye + L, eye.expand_as(L).contiguous(), upper=False)
        k_bg = k_b * e_b
        u = Tm @ v_b
        w = Tm @ k_bg
        saved.update(Tm=Tm, w=w, u=u)

    S = torch.zeros(B, H, K, V, dtype=dtype) if h0 is None else h0.to(dtype)
    hs, vnew = [], []
    k_d = kc * e_d
    for c in range(NT):
        hs.append(S)
        if op == 'gdn':
            vn = u[:, :, c] - w[:, :, c] @ S
        else:
            vn = vc[:, :, c]
        vnew.append(vn)
        dec = decay[:, :, c]
        dec = dec[..., None] if vector else dec[..., None, None]
        S = S * dec + k_d[:, :, c].transpose(-1, -2) @ vn
    hs = torch.stack(hs, 2) if NT else torch.zeros(B, H, 0, K, V, dtype=dtype)       # [B,H,NT,K,V]
    vnew = torch.stack(vnew, 2) if NT else torch.zeros(B, H, 0, C, V, dtype=dtype)   # [B,H,NT,C,V]
    o = scale * ((qc * e_b) @ hs + P @ vnew)
    o = o.reshape(B, H, Tp, V)[:, :, :T]
    saved.update(hs=hs, vnew=vnew, P=P, ht=S)
    return o, S, saved


# --------------------------------------------------------------------------- #
# backward (manual, per chunk)
# --------------------------------------------------------------------------- #
def chunk_backward(op: str, q, k, v, g, beta, scale, h0, do, dht, saved, C: int = CHUNK,
                   dtype=torch.float32, solve_form: bool = False):
    """Manual backward.  Returns dq, dk, dv, dg, dbeta, dh0 (entries None where not applicable).

    ``solve_form`` (gated delta rule): the backward of the WY form written through dZ = T^T dv_new, the gradient
    with respect to Z = beta (v - e^b k S) (v_new = T Z solves (I + L) v_new = Z): dv = beta dZ,
    d(k beta e^b) = -dZ S^T, dL = -strictlower(dZ v_new^T), and the state recurrence subtracts (k beta e^b)^T dZ.
    It is what the HIP kernels compute; the default is the w / u form (dT = du v_b^T + dw k_bg^T,
    dL = -T^T dT T^T), which fla's kernels follow.  Both are pinned against autograd and against each other in
    tests/test_oracle_pins.py."""
    B, H, T, K = q.shape
    V = v.shape[-1]
    scale = K ** -0.5 if scale is None else scale
    q, k, v, do = (_pad_t(x.to(dtype), C) for x in (q, k, v, do))
    beta = None if beta is None else _pad_t(beta.to(dtype), C)
    Tp = q.shape[2]
    NT = Tp // C
    qc, kc, vc, doc = _chunks(q, C), _chunks(k, C), _chunks(v, C), _chunks(do, C)
    vector = op == 'gla'
    b, hs, vnew = saved['b'], saved['hs'], saved['vnew']
    bC = b[:, :, :, -1:]
    mask_d = _tril(C, dtype)
    mask_s = _tril(C, dtype, -1)
    if vector:
        e_b, e_d, decay = b.exp(), (bC - b).exp(), bC.exp().squeeze(3)
        diff = (b[:, :, :, :, None, :] - b[:, :, :, None, :, :]) * mask_d[:, :, None]
        Gam_k = diff.exp() * mask_d[:, :, None]          # [..,C,C,K]
        P = torch.einsum('bhnik,bhnjk,bhnijk->bhnij', qc, kc, Gam_k)
    else:
        e_b, e_d, decay = b.exp()[..., None], (bC - b).exp()[..., None], bC.exp().squeeze(3)
        Gam = ((b[..., :, None] - b[..., None, :]) * mask_d).exp() * mask_d
        QK = qc @ kc.transpose(-1, -2)
        P = QK * Gam
    k_d = kc * e_d
    q_g = qc * e_b

    # ---- chunk-parallel: local part of dv_new ---------------------------------
    dv_loc = scale * (P.transpose(-1, -2) @ doc)
    # ---- reverse state pass ---------------------------------------------------
    dS = torch.zeros(B, H, K, V, dtype=dtype) if dht is None else dht.to(dtype)
    dhs = [None] * NT            # gradient w.r.t. the state at the END of chunk c
    dvn = [None] * NT
    if op == 'gdn':
        w = saved['w']
    for c in reversed(range(NT)):
        dhs[c] = dS
        dvn[c] = dv_loc[:, :, c] + k_d[:, :, c] @ dS
        dec = decay[:, :, c]
        dec = dec[..., None] if vector else dec[..., None, None]
        dS_new = scale * (q_g[:, :, c].transpose(-1, -2) @ doc[:, :, c]) + dec * dS
        if op == 'gdn' and solve_form:
            dz_c = saved['Tm'][:, :, c].transpose(-1, -2) @ dvn[c]
            kbg_c = kc[:, :, c] * _chunks(beta, C)[:, :, c][..., None] * e_b[:, :, c]
            dS_new = dS_new - kbg_c.transpose(-1, -2) @ dz_c
        elif op == 'gdn':
            dS_new = dS_new - w[:, :, c].transpose(-1, -2) @ dvn[c]
        dS = dS_new
    dh0 = dS
    if NT:
        dhs = torch.stack(dhs, 2)
        dvn = torch.stack(dvn, 2)
    else:
        dhs = torch.zeros(B, H, 0, K, V, dtype=dtype)
        dvn = torch.zeros(B, H, 0, C, V, dtype=dtype)

    # ---- chunk-parallel gradient pass -----------------------------------------
    dP = scale * (doc @ vnew.transpose(-1, -2)) * mask_d
    dq_inter = scale * (doc @ hs.transpose(-1, -2)) * e_b
    dk_d = vnew @ dhs.transpose(-1, -2)                     # grad w.r.t. k_d
    hdh = (hs * dhs).sum(-1) if vector else (hs * dhs).sum((-1, -2))   # <S, dS'> (per K row for gla)
    if vector:
        dq = dq_inter + torch.einsum('bhnij,bhnjk,bhnijk->bhnik', dP, kc, Gam_k)
        dk = dk_d * e_d + torch.einsum('bhnij,bhnik,bhnijk->bhnjk', dP, qc, Gam_k)
        db = qc * dq - kc * dk                               # [..,C,K]
        last = (dk_d * k_d).sum(3) + decay * hdh             # [B,H,NT,K]
        db[:, :, :, -1] = db[:, :, :, -1] + last
        dg = db.flip(3).cumsum(3).flip(3)
        dv = dvn
        dbeta = None
    elif op == 'simple_gla':
        dPG = dP * Gam
        dq = dq_inter + dPG @ kc
        dk = dk_d * e_d + dPG.transpose(-1, -2) @ qc
        db = (qc * dq).sum(-1) - (kc * dk).sum(-1)           # [..,C]
        last = (dk_d * k_d).sum((-1, -2)) + decay * hdh
        db[..., -1] = db[..., -1] + last
        dg = db.flip(3).cumsum(3).flip(3)
        dv = dvn
        dbeta = None
    else:  # gdn
        Tm, u = saved['Tm'], saved['u']
        bc = _chunks(beta, C)[..., None]
        k_b, v_b = kc * bc, vc * bc
        k_bg = k_b * e_b
        Gam_s = Gam * mask_s
        M = k_b @ kc.transpose(-1, -2)
        dPG = dP * Gam
        dq = dq_inter + dPG @ kc
        dk = dk_d * e_d + dPG.transpose(-1, -2) @ qc
        if solve_form:
            dZ = Tm.transpose(-1, -2) @ dvn
            dv_b = dZ
            dk_bg = -(dZ @ hs.transpose(-1, -2))
            dL = -(dZ @ vnew.transpose(-1, -2)) * mask_s
        else:
            dw = -(dvn @ hs.transpose(-1, -2))
            du = dvn
            dT = du @ v_b.transpose(-1, -2) + dw @ k_bg.transpose(-1, -2)
            dv_b = Tm.transpose(-1, -2) @ du
            dk_bg = Tm.transpose(-1, -2) @ dw
            dL = -(Tm.transpose(-1, -2) @ dT @ Tm.transpose(-1, -2)) * mask_s
        dM = dL * Gam_s
        dk_b = dM @ kc + dk_bg * e_b
        dk = dk + dM.transpose(-1, -2) @ k_b + dk_b * bc
        dbeta = (dk_b * kc).sum(-1) + (dv_b * vc).sum(-1)
        dv = dv_b * bc
        dG = dP * P + dL * M * Gam_s          # dP already masked; P = QK*Gam
        db = (dq_inter * qc).sum(-1) + dG.sum(-1) - dG.sum(-2) \
            - (dk_d * k_d).sum(-1) + (dk_bg * k_bg).sum(-1)
        last = (dk_d * k_d).sum((-1, -2)) + decay * hdh
        db[..., -1] = db[..., -1] + last
        dg = db.flip(3).cumsum(3).flip(3)

    def unchunk(x):
        return x.reshape(B, H, Tp, *x.shape[4:])[:, :, :T]

    dq, dk, dv, dg = unchunk(dq), unchunk(dk), unchunk(dv), unchunk(dg)
    dbeta = None if dbeta is None else unchunk(dbeta)
    return dq, dk, dv, dg, dbeta, dh0


def chunk_fwd_bwd(op, q, k, v, g, beta, scale, h0, do, dht, C: int = CHUNK, dtype=torch.float32):
    """One forward + manual backward; what the ``cpu_baseline`` leg times."""
    o, ht, saved = chunk_forward(op, q, k, v, g, beta, scale, h0, C, dtype)
    grads = chunk_backward(op, q, k, v, g, beta, scale, h0, do, dht, saved, C, dtype)
    return o, ht, grads
