"""``chunk_linear_attn``: chunk_simple_gla without decay, optionally normalised by
q . cumsum(k).  Called by the reference at
``linear_moe/sequence_modeling/basic_linear_attention/basic_linear_attention.py:133`` and, with
``normalize=True, scale=1``, by ``.../based/based.py:69`` and ``.../rebased/rebased.py:76``.

The key dimension may be any size: without decay the op is a sum over key blocks, so q and k are taken either as
tensors (split here into blocks of 128 / 64 columns, zero-padded) or as the key blocks the feature maps of
``feature_map.py`` write directly."""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from .simple_gla import can_normalize, chunk_simple_gla, chunk_simple_gla_normalized, chunk_simple_gla_with_den


def chunk_linear_attn(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    scale: Optional[float] = None,
    initial_state: Optional[torch.Tensor] = None,
    output_final_state: bool = False,
    normalize: bool = True,
    head_first: bool = True,
    _eps: float = 1e-10,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """``_eps`` (not part of fla's signature): the epsilon of the normaliser, for the callers in this package whose
    reference functions carry their own (``based.py``)."""
    qb, kb = _key_blocks(q), _key_blocks(k)
    if [b.shape for b in qb] != [b.shape for b in kb]:
        raise ValueError("chunk_linear_attn: q and k must agree in shape")
    K = sum(b.shape[-1] for b in qb)          # padded key dimension
    if scale is None:
        scale = (q.features if hasattr(q, "features") else q.shape[-1]) ** -0.5
    if initial_state is not None and initial_state.shape[-2] != K:
        if initial_state.shape[-2] > K:
            raise ValueError(f"chunk_linear_attn: initial_state has {initial_state.shape[-2]} key rows, q has {K}")
        initial_state = torch.nn.functional.pad(initial_state, (0, 0, 0, K - initial_state.shape[-2]))
    # The normaliser z_i = scale sum_{j<=i} q_i . k_j is the op itself with one more value column of ones (fla
    # normalises with q * scale, so the scale cancels in o up to the epsilon): it is formed inside the kernels, in
    # the fp32 state, instead of by a cumulative sum over k in HBM.
    V = v.shape[-1]
    if normalize and V <= 128 and v.dim() == 4 and v.dtype == torch.bfloat16:
        # bfloat16: the kernels carry the column themselves (a value head that is not 64 or 128 wide is zero-padded to
        # the next of the two: zero columns stay zero).  One key block: they also divide before they store.  Several
        # (the feature maps of Based / ReBased): the divisor is the sum over the blocks, so every block hands out its
        # den beside its undivided output and the division follows the two sums.
        Vp = 64 if V <= 64 else 128
        pad = torch.nn.functional.pad
        vp = v if Vp == V else pad(v, (0, Vp - V))
        h0 = initial_state if (initial_state is None or Vp == V) else pad(initial_state, (0, Vp - V))
        feats = q.features if hasattr(q, "features") else q.shape[-1]
        if all(can_normalize(qi, vp) for qi in qb):
            if len(qb) == 1:
                o, ht = chunk_simple_gla_normalized(qb[0], kb[0], vp, scale, h0, output_final_state, None, head_first, _eps)
            else:
                o, den, hts, k0 = None, None, [], 0
                for qi, ki in zip(qb, kb):
                    w = qi.shape[-1]
                    h0i = None if h0 is None else h0[..., k0:k0 + w, :].contiguous()
                    oi, di, hi = chunk_simple_gla_with_den(qi, ki, vp, scale, h0i, output_final_state, None, head_first)
                    o = oi.float() if o is None else o + oi.float()
                    den = di if den is None else den + di
                    hts.append(hi)
                    k0 += w
                o = (o / (den.unsqueeze(-1) + _eps)).to(v.dtype)
                ht = torch.cat(hts, dim=-2) if output_final_state else None
            if ht is not None and (ht.shape[-2] != feats or Vp != V):
                ht = ht[..., :feats, :V]
            return (o if Vp == V else o[..., :V]), ht
    # otherwise (fp32, several key blocks, other head dimensions) the column is appended here: chunk_simple_gla cuts
    # the V + 1 columns into the blocks the kernels take; the carried state has no normaliser column (the sum starts
    # inside the call).
    if normalize:
        v = torch.cat([v, v.new_ones(*v.shape[:-1], 1)], dim=-1)
        if initial_state is not None:
            initial_state = torch.nn.functional.pad(initial_state, (0, 1))
    o, hts, k0 = None, [], 0
    for qi, ki in zip(qb, kb):
        w = qi.shape[-1]
        h0 = None if initial_state is None else initial_state[..., k0:k0 + w, :].contiguous()
        oi, hi = chunk_simple_gla(qi, ki, v, None, scale, h0, output_final_state, None, head_first)
        if len(qb) > 1:
            oi = oi.float()
        o = oi if o is None else o + oi
        hts.append(hi)
        k0 += w
    if normalize:
        o = o.float()
        o = o[..., :V] / (o[..., V:] + _eps)
    o = o.to(v.dtype)
    ht = None
    if output_final_state:
        ht = hts[0] if len(hts) == 1 else torch.cat(hts, dim=-2)
        feats = q.features if hasattr(q, "features") else q.shape[-1]
        if feats != K:
            ht = ht[..., :feats, :]
        if normalize:
            ht = ht[..., :V]
    return o, ht


def _key_blocks(x):
    """x as a list of contiguous key blocks of 128 / 64 columns (zero-padded)."""
    if isinstance(x, (tuple, list)):
        return list(x)
    K = x.shape[-1]
    if K in (64, 128):
        return [x]
    Kp = -(-K // 64) * 64
    if Kp != K:
        x = torch.nn.functional.pad(x, (0, Kp - K))
    out, k0 = [], 0
    while k0 < Kp:
        w = 128 if Kp - k0 >= 128 else 64
        out.append(x[..., k0:k0 + w].contiguous())
        k0 += w
    return out
