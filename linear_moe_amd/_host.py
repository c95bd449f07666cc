"""Host-side plumbing shared by the chunk ops: argument validation, stride descriptors,
the chunk table of packed (cu_seqlens) input and the ``lmoe_args`` block of the C ABI.

Argument meaning follows flash-linear-attention's chunk ops as the reference calls them
(``linear_moe/sequence_modeling/gla/gla.py:94``, ``.../retention/retention.py:91``,
``.../gated_deltanet/gated_deltanet.py:112``): ``head_first=True`` means ``[B,H,T,D]``,
otherwise ``[B,T,H,D]``; ``scale=None`` means ``K ** -0.5``; states are fp32 ``[N,H,K,V]``.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Tuple

import torch

from . import _lib
from ._lib import Args, Tensor4, CHUNK

_DT = {torch.bfloat16: _lib.LMOE_BF16, torch.float32: _lib.LMOE_F32}


def _check_inputs(q, k, v, head_first: bool, cu_seqlens, wide_v: bool = False) -> Tuple[int, int, int, int, int]:
    """wide_v: the op also has kernels for K = 128 with V = 256 (the gated delta rule)."""
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise ValueError("q, k, v must be 4-dimensional")
    if not (q.is_cuda and k.is_cuda and v.is_cuda):
        raise RuntimeError("linear_moe_amd ops run on the GPU only (HIP kernels; there is no CPU path)")
    if q.dtype not in _DT or k.dtype != q.dtype or v.dtype != q.dtype:
        raise ValueError(f"q, k, v must share dtype bfloat16 or float32, got {q.dtype}, {k.dtype}, {v.dtype}")
    if q.shape != k.shape or q.shape[:3] != v.shape[:3]:
        raise ValueError(f"shape mismatch: q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)}")
    if head_first:
        B, H, T, K = q.shape
    else:
        B, T, H, K = q.shape
    V = v.shape[-1]
    if (K not in HEAD_DIMS or V not in HEAD_DIMS) and not (wide_v and (K, V) == WIDE_V):
        raise ValueError(f"head dims K={K}, V={V} unsupported: the kernels take K and V of 64 or 128 "
                         "(the public ops pad and split other sizes before they get here)")
    if cu_seqlens is not None:
        if head_first:
            raise ValueError("cu_seqlens requires head_first=False ([1, T, H, D] packed input)")
        if B != 1:
            raise ValueError(f"cu_seqlens requires batch size 1 (packed input), got B={B}")
    return B, T, H, K, V


HEAD_DIMS = (64, 128)      # what the kernels are instantiated for
WIDE_V = (128, 256)        # and, for the gated delta rule, this (K, V) as well


def dim_blocks(D: int, widest: int = 128):
    """D columns as the blocks the kernels take: ``[(start, stop, width)]`` with width 64, 128 or (``widest=256``)
    256 (the last block zero-padded up to its width)."""
    if D < 1:
        raise ValueError(f"head dimension must be positive, got {D}")
    out, d0 = [], 0
    while D - d0 > widest:
        out.append((d0, d0 + widest, widest))
        d0 += widest
    out.append((d0, D, 64 if D - d0 <= 64 else 128 if D - d0 <= 128 else 256))
    return out


def by_head_dim_blocks(core, q, k, v, gk, initial_state, output_final_state: bool, sum_over_k: bool, name: str,
                       wide_v: bool = False):
    """An op on head dimensions the kernels are not instantiated for, as calls on blocks of 128 / 64 columns.

    The columns of v (and of the state) are independent in all three ops, so V is cut into blocks and the outputs
    are concatenated; a short block is zero-padded (zero columns of v give zero columns of o and of the state).
    K: zero columns of q and k change nothing, so a short K is padded; ``sum_over_k`` ops (no delta rule: the op is
    a sum over key blocks) also take K > 128 as several blocks whose outputs are added in fp32.  ``core(q, k, v, gk,
    h0) -> (o, ht)`` runs the op on supported dimensions (``gk``: the per-channel gate of chunk_gla or None).
    Everything around ``core`` is differentiable torch code.  Each V block repeats the work that depends on q, k
    only (for the delta rule the WY preparation): the supported dimensions are the fast path.  ``wide_v``: with a key
    of more than 64 columns (one block of 128) the op takes value blocks of 256 columns."""
    pad = torch.nn.functional.pad
    K, V = q.shape[-1], v.shape[-1]
    kb = dim_blocks(K)
    vb = dim_blocks(V, 256 if wide_v and len(kb) == 1 and kb[0][2] == 128 else 128)
    if len(kb) > 1 and not sum_over_k:
        raise ValueError(f"{name}: K={K} unsupported: the delta rule needs the whole key in one block (K <= 128)")
    if initial_state is not None and tuple(initial_state.shape[-2:]) != (K, V):
        raise ValueError(f"{name}: initial_state must end in [{K}, {V}], got {tuple(initial_state.shape)}")
    cut = lambda x, d0, d1, w: pad(x[..., d0:d1], (0, w - (d1 - d0))).contiguous()
    qs = [(cut(q, k0, k1, w), cut(k, k0, k1, w), None if gk is None else cut(gk, k0, k1, w)) for k0, k1, w in kb]
    o_cols, ht_cols = [], []
    for v0, v1, vw in vb:
        v_ = cut(v, v0, v1, vw)
        o_v, ht_rows = None, []
        for (k0, k1, kw), (q_, k_, g_) in zip(kb, qs):
            h0 = None
            if initial_state is not None:
                h0 = pad(initial_state[..., k0:k1, v0:v1], (0, vw - (v1 - v0), 0, kw - (k1 - k0))).contiguous()
            o_, ht_ = core(q_, k_, v_, g_, h0)
            if len(kb) > 1:
                o_ = o_.to(torch.promote_types(o_.dtype, torch.float32))
            o_v = o_ if o_v is None else o_v + o_
            if output_final_state:
                ht_rows.append(ht_[..., :k1 - k0, :v1 - v0])
        o_cols.append(o_v[..., :v1 - v0].to(v.dtype))
        if output_final_state:
            ht_cols.append(ht_rows[0] if len(ht_rows) == 1 else torch.cat(ht_rows, dim=-2))
    o = o_cols[0] if len(o_cols) == 1 else torch.cat(o_cols, dim=-1)
    ht = None
    if output_final_state:
        ht = ht_cols[0] if len(ht_cols) == 1 else torch.cat(ht_cols, dim=-1)
    return o, ht


def no_tokens(q, k, v, head_first: bool, cu_seqlens, initial_state, output_final_state: bool, wide_v: bool = False):
    """The call without any token (T = 0, or a batch of zero rows): nothing to launch.  Returns None when there
    are tokens, else ``(o, final_state)``: an empty o and the initial state handed through (so that its gradient
    is the gradient of the final state), zeros without one."""
    B, T, H, K, V = _check_inputs(q, k, v, head_first, cu_seqlens, wide_v)
    if B * T > 0:
        return None
    N = B if cu_seqlens is None else cu_seqlens.numel() - 1
    _state_check(initial_state, N, H, K, V, "initial_state")
    o = torch.empty_like(v)
    if not output_final_state:
        return o, None
    if initial_state is None:
        return o, torch.zeros(N, H, K, V, dtype=torch.float32, device=q.device)
    return o, initial_state.float() + 0


def _desc(x: Optional[torch.Tensor], head_first: bool) -> Tensor4:
    """Stride descriptor of a [B,H,T,(D)] or [B,T,H,(D)] tensor."""
    if x is None:
        return Tensor4(None, 0, 0, 0)
    if head_first:
        sb, sh, st = x.stride(0), x.stride(1), x.stride(2)
    else:
        sb, st, sh = x.stride(0), x.stride(1), x.stride(2)
    return Tensor4(x.data_ptr(), sb, st, sh)


def _aligned(x: torch.Tensor) -> torch.Tensor:
    """Return x (or a contiguous copy) such that rows are 16-byte aligned and last dim contiguous."""
    if x.dim() == 4:
        vec = 16 // x.element_size()
        ok = x.stride(3) == 1 and x.data_ptr() % 16 == 0 and all(x.stride(i) % vec == 0 for i in range(3))
        return x if ok else x.contiguous()
    return x


class SeqPlan:
    """Chunk bookkeeping of one call: number of sequences / chunks and, for packed input,
    the device tables the kernels index with.  Build through ``seq_plan`` (cached).

    Offsets on the host (a CPU ``cu_seqlens``) are validated and give exact tables.  Offsets on the device are never
    read back: the tables are built there by a handful of small device operations, sized for the upper bound
    ``NT <= ceil(T / 64) + N`` of the chunk count (every sequence ends in at most one partial chunk), with the true
    count in ``nt_dev`` for the kernels; nothing synchronises with the host, so the build can run inside a HIP
    graph capture and a replay follows the offsets the buffer holds at that time.  Device offsets are trusted
    (start at 0, non-decreasing, last <= T), as fla trusts them."""

    def __init__(self, B: int, T: int, cu_seqlens: Optional[torch.Tensor], device):
        self.cu = None
        self.chunk_map = None
        self.seq_chunk0 = None
        self.seq_order = None
        self.nt_dev = None
        self.host_offsets = None
        if cu_seqlens is None:
            self.N = B
            self.NT = B * ((T + CHUNK - 1) // CHUNK)
            return
        if cu_seqlens.dim() != 1 or cu_seqlens.numel() < 2:
            raise ValueError("cu_seqlens must be a 1-D tensor of N+1 offsets")
        if cu_seqlens.is_cuda:
            self._build_on_device(T, cu_seqlens)
            return
        cu_host = cu_seqlens.detach().to("cpu", torch.int64)
        self.host_offsets = cu_host.clone()      # what the tables were built from (compared on a cache hit)
        lens = cu_host[1:] - cu_host[:-1]
        if int(cu_host[0]) != 0 or int(cu_host[-1]) != T or bool((lens < 0).any()):
            raise ValueError("cu_seqlens must start at 0, be non-decreasing and end at T")
        self.N = int(lens.numel())
        nch = (lens + CHUNK - 1) // CHUNK
        c0 = torch.zeros(self.N + 1, dtype=torch.int64)
        c0[1:] = torch.cumsum(nch, 0)
        self.NT = int(c0[-1])
        seq_of = torch.repeat_interleave(torch.arange(self.N), nch)
        local = torch.arange(self.NT) - c0[:-1][seq_of]
        cmap = torch.stack([seq_of, local], 1).to(torch.int32).contiguous()
        self.cu = cu_host.to(torch.int32).to(device)
        self.chunk_map = cmap.to(device)
        self.seq_chunk0 = c0.to(torch.int32).to(device)
        # the sequential passes take the longest sequences first (their work-groups are dispatched in index order): a
        # batch of unequal lengths then does not end on a long sequence that started late
        if self.N > 1 and int(nch.max()) != int(nch.min()):
            self.seq_order = torch.argsort(nch, descending=True, stable=True).to(torch.int32).to(device)

    def _build_on_device(self, T: int, cu_seqlens: torch.Tensor):
        dev = cu_seqlens.device
        N = cu_seqlens.numel() - 1
        nt_max = (T + CHUNK - 1) // CHUNK + N
        cu = cu_seqlens.detach().to(torch.int64)
        nch = (cu[1:] - cu[:-1] + (CHUNK - 1)) // CHUNK                        # chunks per sequence
        c0 = torch.cat([cu.new_zeros(1), torch.cumsum(nch, 0)])                 # [N + 1] first chunk of every sequence
        # rows past the true count belong to a sequence "N" that no kernel ever visits
        counts = torch.cat([nch, nt_max - c0[-1:]])
        seq_of = torch.repeat_interleave(torch.arange(N + 1, device=dev), counts, output_size=nt_max)
        local = torch.arange(nt_max, device=dev) - torch.cat([c0, c0[-1:]])[seq_of]
        self.N, self.NT = N, nt_max
        self.cu = cu.to(torch.int32).contiguous()
        self.chunk_map = torch.stack([seq_of, local], 1).to(torch.int32).contiguous()
        self.seq_chunk0 = c0.to(torch.int32).contiguous()
        self.nt_dev = c0[-1:].to(torch.int32).contiguous()
        if N > 1:
            self.seq_order = torch.argsort(nch, descending=True, stable=True).to(torch.int32).contiguous()


# Plans of the cu_seqlens tensors seen last, newest first.  An entry holds the tensor itself (so its address cannot be
# reused by another tensor while the entry lives) and its version counter (an in-place change through torch makes a new
# plan).  One packed batch is used by the forward and the backward of every layer: only the first of those calls
# builds the tables.  A write that torch does not see (another library writing into the buffer, ``.data`` tricks) leaves
# a stale entry behind: ``forget_cu_seqlens`` drops it.  While a HIP graph is being captured nothing is taken from or
# put into the cache: the tables of device offsets are built inside the capture, so that a replay follows the offsets
# the buffer holds when it runs.
_PLAN_CACHE: list = []
_PLAN_CACHE_SIZE = 8


def seq_plan(B: int, T: int, cu_seqlens: Optional[torch.Tensor], device) -> SeqPlan:
    if cu_seqlens is None:
        return SeqPlan(B, T, None, device)
    if cu_seqlens.is_cuda and torch.cuda.is_current_stream_capturing():
        return SeqPlan(B, T, cu_seqlens, device)
    for i, (cu, version, t, dev, plan) in enumerate(_PLAN_CACHE):
        if cu is cu_seqlens and version == cu_seqlens._version and t == T and dev == device:
            # offsets on the host cost nothing to compare: a write the version counter did not see is caught here
            if not cu_seqlens.is_cuda and not torch.equal(plan.host_offsets, cu_seqlens.detach().to(torch.int64)):
                del _PLAN_CACHE[i]
                break
            if i:
                _PLAN_CACHE.insert(0, _PLAN_CACHE.pop(i))
            return plan
    plan = SeqPlan(B, T, cu_seqlens, device)
    _PLAN_CACHE.insert(0, (cu_seqlens, cu_seqlens._version, T, device, plan))
    del _PLAN_CACHE[_PLAN_CACHE_SIZE:]
    return plan


def prepare_cu_seqlens(cu_seqlens: torch.Tensor, T: int, device=None) -> SeqPlan:
    """Build (and cache) the chunk tables of a packed batch ahead of its first use, off the critical path of a step.
    ``T`` is the total number of tokens (``cu_seqlens[-1]``; for offsets on the device: the number of rows of the
    packed tensors, which may exceed it)."""
    if device is None:
        device = cu_seqlens.device if cu_seqlens.is_cuda else torch.device("cuda", torch.cuda.current_device())
    return seq_plan(1, T, cu_seqlens, device)


def forget_cu_seqlens(cu_seqlens: Optional[torch.Tensor] = None) -> None:
    """Drop the cached chunk tables of ``cu_seqlens`` (of every tensor when None): to be called after the offsets were
    changed by a write that torch's version counter does not see."""
    if cu_seqlens is None:
        _PLAN_CACHE.clear()
    else:
        _PLAN_CACHE[:] = [e for e in _PLAN_CACHE if e[0] is not cu_seqlens]


def _state_check(x: Optional[torch.Tensor], N, H, K, V, name: str) -> Optional[torch.Tensor]:
    if x is None:
        return None
    if tuple(x.shape) != (N, H, K, V):
        raise ValueError(f"{name} must have shape [N,H,K,V] = {(N, H, K, V)}, got {tuple(x.shape)}")
    return x.detach().to(torch.float32).contiguous()


def base_args(q, k, v, head_first: bool, scale: Optional[float], plan: SeqPlan, dims) -> Args:
    B, T, H, K, V = dims
    if not (q.device == k.device == v.device) or q.device.index != torch.cuda.current_device():
        # (the kernels go to the current stream of the current device: one process per GPU, as the launchers run it)
        raise RuntimeError(f"q, k, v must live on the current device cuda:{torch.cuda.current_device()}, got "
                           f"{q.device}, {k.device}, {v.device}")
    a = Args()
    a.dtype = _DT[q.dtype]
    a.B, a.T, a.H, a.K, a.V = B, T, H, K, V
    a.N, a.NT = plan.N, plan.NT
    a.scale = float(K ** -0.5 if scale is None else scale)
    if plan.cu is not None:
        a.cu_seqlens = plan.cu.data_ptr()
        a.chunk_map = plan.chunk_map.data_ptr()
        a.seq_chunk0 = plan.seq_chunk0.data_ptr()
        a.seq_order = ptr(plan.seq_order)
        a.nt_dev = ptr(plan.nt_dev)
    a.q, a.k, a.v = _desc(q, head_first), _desc(k, head_first), _desc(v, head_first)
    return a


def token_major(B: int, T: int, H: int, D: int, dtype, device) -> torch.Tensor:
    """Internal per-token buffer [B, T, H, D] (time-first, contiguous)."""
    return torch.empty(B, T, H, D, dtype=dtype, device=device)


def stash(ctx, call, *extra) -> None:
    """Hands the tensors ``call`` keeps for its backward (``call.saved``) and ``extra`` over to autograd
    (``ctx.save_for_backward``).  Autograd then frees them as soon as the node's backward has run -- the per-chunk
    states of a layer go while the backward sweep passes the layer, not when the whole graph dies --, notices an
    input that was modified in place between forward and backward, and saved-tensor hooks see them."""
    ctx.n_stashed = len(call.saved)
    ctx.save_for_backward(*call.saved, *extra)
    call.saved = None


def unstash(ctx, call):
    """Gives ``call`` its tensors back for one backward; returns the ``extra`` of ``stash``."""
    t = ctx.saved_tensors
    call.saved = tuple(t[:ctx.n_stashed])
    return t[ctx.n_stashed:]


def stream_ptr() -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def ptr(x: Optional[torch.Tensor]):
    return None if x is None else x.data_ptr()
