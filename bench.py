#!/usr/bin/env python3
"""Headline benchmark: chunk_gated_delta_rule forward + backward on one MI355X.

Workload (the configuration the metric is quoted on): B=4, H=16, T=8192,
K=V=128, bf16; q,k ~ N(0,1) L2-normalised, v ~ N(0,1), beta = sigmoid(N(0,1)),
g = -exp(A_h) softplus(x + dt_bias_h), dO ~ N(0,1).  A "step" is one forward + one backward of
the op over that batch with all inputs resident in HBM.

Prints ONE JSON line: tokens/s of the whole step, the roofline record of the dominant kernel
(timed live with HIP events on the launch stream through ``lmoe_launch_stage``) and the CPU
baseline (the chunked torch restatement in ``oracle/`` timed on this host's cores).
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_MFMA_BF16 = 2.5e15   # dense bf16 MFMA, FLOP/s (MI355X published)
PEAK_MFMA_F32 = 157.3e12  # dense fp32 MFMA, FLOP/s (MI355X published)
PEAK_HBM = 8.0e12         # B/s
CH = 64

STAGE_NAMES = {0: "k_gdn_wy_fwd", 1: "k_gdn_state_fwd_reg", 4: "k_gdn_state_bwd", 5: "k_gdn_bwd_chunk"}

# HBM bytes per launch on this workload, from two rocprofv3 --pmc runs of this file (FETCH_SIZE, then
# WRITE_SIZE, KiB per dispatch), each scaled by what the same counter reads for the 256 MiB device
# copy that main() issues first (FETCH_SIZE reads half of the bytes fetched, WRITE_SIZE all of the
# bytes written).  Summary and commands: profiles/gdn_fwd_bwd_cfg4_hbm_traffic.md.
# The figures belong to the kernel sources they were measured on: TRAFFIC_SOURCES_SHA16 is the digest of those
# sources (kernel_sources_sha16()) at that time, and a build whose sources differ reports traffic = null
# rather than a stale number.
CALIB_COPY_BYTES = 256 << 20
MEASURED_TRAFFIC = {"k_gdn_wy_fwd": 237242548, "k_gdn_state_fwd_reg": 1120530337, "k_gdn_state_bwd": 945957881,
                    "k_gdn_bwd_chunk": 1825838726}
TRAFFIC_SOURCES_SHA16 = "741aeabd45d2fd45"
TRAFFIC_SOURCES = ("lmoe_common.hpp", "lmoe_seq.hpp", "lmoe_gdn_wy.hpp", "lmoe_gdn_state.hpp", "lmoe_gdn_state_reg.hpp", "lmoe_gdn_bwd_chunk.hpp",
                   "lmoe_gdn_fwd.hip", "lmoe_gdn_state.hip", "lmoe_gdn_bwd.hip")


# HBM bytes per call of the other contract configurations (bench.py --other-configs), same counters and scaling,
# summed over the kernels of the call; key = configuration number
OTHER_TRAFFIC = {"1": 2232824, "2": 272914694, "3": 1279660547, "5": 16651376487, "6": 1444943222, "7": 6580301476,
                 "8": 1510793999}
OTHER_TRAFFIC_SHA16 = "9a2741ef41ed699f"


def all_sources_sha16():
    """Digest of every kernel source of the library (what OTHER_TRAFFIC was counted on; lmoe_api.hip, which holds
    validation and dispatch but no kernel, is left out)."""
    import glob
    import hashlib
    h = hashlib.sha256()
    d = os.path.join(ROOT, "linear_moe_amd", "csrc")
    for path in sorted(glob.glob(os.path.join(d, "*.hpp")) + glob.glob(os.path.join(d, "*.hip"))):
        if os.path.basename(path) == "lmoe_api.hip":
            continue
        with open(path, "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def kernel_sources_sha16():
    """Digest of the sources of the four gated-delta-rule kernels (what MEASURED_TRAFFIC was counted on)."""
    import hashlib
    h = hashlib.sha256()
    for name in TRAFFIC_SOURCES:
        with open(os.path.join(ROOT, "linear_moe_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def gdn_inputs(B, T, H, K, V, seed, dtype, device):
    """Contract laws of the gated-delta-rule configs (CPU generator, then copied to the GPU)."""
    import torch
    import torch.nn.functional as F
    g_ = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g_, dtype=torch.float32)
    q = F.normalize(rn(B, T, H, K), dim=-1)
    k = F.normalize(rn(B, T, H, K), dim=-1)
    v = rn(B, T, H, V)
    beta = torch.sigmoid(rn(B, T, H))
    A = torch.rand(H, generator=g_) * math.log(16.0)          # A_h ~ U(log 1, log 16)
    dt_bias = rn(H) * 0.1
    g = -torch.exp(A)[None, None, :] * F.softplus(rn(B, T, H) + dt_bias[None, None, :])
    do = rn(B, T, H, V)
    dev = lambda x, dt: x.to(dt).to(device)
    return dict(q=dev(q, dtype), k=dev(k, dtype), v=dev(v, dtype), g=dev(g, torch.float32),
                beta=dev(beta, dtype), do=dev(do, dtype))


def stage_model(stage, K, V, s=2):
    """Algorithmic (flops, bytes) of one kernel per chunk and head: every product counted once on
    full 64-token tiles, multiply-add = 2 flops; every input read once, every output written once."""
    c = CH
    kv, ck, cv, cc = K * V, c * K, c * V, c * c
    lean = s == 2     # 2-byte elements: w = Tinv (k beta e^b), u = Tinv (v beta) are formed inside the state passes
    if stage == 0:   # k k^T(, q k^T), triangular inverse(, w, u) | r k,g,beta(,q,v)  w Tinv,gate table(,P,w,u)
        if lean:     # (the table has five fp32 rows; g is read as fp32)
            return 2 * cc * K + (2 / 3) * c ** 3, ck * s + cc * s + c * (20 + 4 + s)
        return 6 * cc * K + 2 * cc * V + (2 / 3) * c ** 3, (2 * ck + cv) * s + (ck + cv) * s + 2 * cc * s + c * (20 + 4 + s)
    if stage == 1:   # k S, Tinv Z, q S, q k^T, P v_new, k^T v_new | r q,k,Tinv,v,table (q,k,w,u,P,table)  w v_new,hs,o,P
        if lean:
            return 6 * c * kv + 4 * cc * V + 2 * cc * K, (2 * ck + cv + cc) * s + (2 * cv + kv + cc) * s + 20 * c
        return 6 * c * kv + 2 * cc * V, (3 * ck + cv + cc) * s + (2 * cv + kv) * s + 8 * c
    if stage == 4:   # k dS', P^T do, q^T do, Tinv^T dv_new, (k beta e^b)^T dZ | r q,k,Tinv,do,P,table  w dZ,dhs
        return 6 * c * kv + 4 * cc * V, (2 * ck + cv + 2 * cc) * s + (cv + kv) * s + 12 * c
    if stage == 5:   # do v'^T, dZ v'^T, do S^T, dZ S^T, v' dS'^T, G k, G^T q, dM k, dM^T k_b
        #              | r do,v',dZ,v,hs,dhs,q,k,g,beta  w dq,dk,dv,dbeta,dg
        return (4 * cc * V + 6 * c * kv + 8 * cc * K,
                (4 * cv + 2 * kv + 2 * ck) * s + (2 * ck + cv) * s + c * (4 + s + 8))
    raise ValueError(stage)


def time_stages(call, lib, reps):
    """Average duration (seconds) of every kernel, measured with events on the launch stream."""
    import torch
    from linear_moe_amd import _lib
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = {}
    for stage in (0, 1, 4, 5):         # stages 2, 3 (separate output / dv kernels) are not part of this op
        a = call.fwd_args if stage <= 2 else call.bwd_args
        n_warm = max(2, reps // 2)
        n_timed = max(1, reps - n_warm)
        for _ in range(n_warm):
            _lib.check(lib.lmoe_launch_stage(C.byref(a), call.OP, stage, st), "stage")
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n_timed):
            lib.lmoe_launch_stage(C.byref(a), call.OP, stage, st)
        e1.record()
        e1.synchronize()
        out[stage] = e0.elapsed_time(e1) * 1e-3 / n_timed
    return out


def cpu_baseline(B, T, H, K, V, seed, min_seconds=10.0):
    """The chunked torch restatement (oracle/chunked.py), forward + manual backward, fp32, on the
    host cores: whole passes over the full workload until at least ``min_seconds`` have elapsed."""
    import torch
    from oracle import chunked
    x = gdn_inputs(B, T, H, K, V, seed, torch.float32, "cpu")
    hf = {n: t.transpose(1, 2).contiguous() for n, t in x.items()}
    small = {n: t[:1, :2, :256].contiguous() for n, t in hf.items()}
    chunked.chunk_fwd_bwd("gdn", small["q"], small["k"], small["v"], small["g"], small["beta"], None, None,
                          small["do"], None)
    passes, t0 = 0, time.perf_counter()
    with torch.no_grad():
        while True:
            chunked.chunk_fwd_bwd("gdn", hf["q"], hf["k"], hf["v"], hf["g"], hf["beta"], None, None, hf["do"], None)
            passes += 1
            dt = time.perf_counter() - t0
            if dt >= min_seconds or passes >= 20:
                break
    return {"value": passes * B * T / dt, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{passes} passes over the full workload (B={B}, T={T}, H={H}, K=V={K}), fp32 chunked "
                      f"torch port, {dt:.1f} s"}


def neighbours(lib, rows, D, dev, reps):
    """Row-wise kernels around the op on `rows` x D bf16 (the q / k / o rows of the headline workload):
    seconds per launch from events on the launch stream, and algorithmic GB/s (every operand read
    once, every result written once) against the HBM peak."""
    import torch
    from linear_moe_amd import _lib
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    mk = lambda: torch.randn(rows, D, device=dev, dtype=torch.bfloat16)
    x, dy, gate, out, out2 = mk(), mk(), mk(), mk(), mk()
    w = torch.ones(D, device=dev, dtype=torch.bfloat16)
    part = torch.empty(lib.lmoe_rmsnorm_partials(rows, D, _lib.LMOE_BF16), D, device=dev, dtype=torch.float32)
    dw = torch.empty(D, device=dev, dtype=torch.float32)
    p = lambda t: C.c_void_p(t.data_ptr())
    bf = _lib.LMOE_BF16
    cases = {   # name: (launch, tensors of rows x D moved)
        "l2norm_fwd": (lambda: lib.lmoe_l2norm_fwd(p(x), p(out), rows, D, bf, 1e-6, st), 2),
        "l2norm_bwd": (lambda: lib.lmoe_l2norm_bwd(p(x), p(dy), p(out), rows, D, bf, 1e-6, st), 3),
        "silu_l2norm_fwd": (lambda: lib.lmoe_silu_l2norm_fwd(p(x), p(out), rows, D, bf, 1e-6, st), 2),
        "silu_l2norm_bwd": (lambda: lib.lmoe_silu_l2norm_bwd(p(x), p(dy), p(out), rows, D, bf, 1e-6, st), 3),
        "rmsnorm_fwd": (lambda: lib.lmoe_rmsnorm_fwd(p(x), p(w), None, p(out), None, rows, D, bf, 1e-5, st), 2),
        "rmsnorm_bwd": (lambda: lib.lmoe_rmsnorm_bwd(p(x), p(w), None, p(dy), p(out), None, p(part), p(dw), rows, D, bf,
                                                     1e-5, st), 3),
        "rmsnorm_gate_fwd": (lambda: lib.lmoe_rmsnorm_fwd(p(x), p(w), p(gate), p(out), None, rows, D, bf, 1e-5, st), 3),
        "rmsnorm_gate_bwd": (lambda: lib.lmoe_rmsnorm_bwd(p(x), p(w), p(gate), p(dy), p(out), p(out2), p(part), p(dw),
                                                          rows, D, bf, 1e-5, st), 5),
    }
    # gate construction: gated delta rule on [B*T][H] (a, b bf16 -> g fp32, beta bf16), chunk_gla on the
    # gate tensor of contract config 3 ([8,16,2048,64] bf16)
    Hh = 16
    grows = rows // Hh
    ga, gb = (torch.randn(grows, Hh, device=dev, dtype=torch.bfloat16) for _ in range(2))
    gA, gD = torch.zeros(Hh, device=dev), torch.zeros(Hh, device=dev)
    gg, gdg = torch.empty(grows, Hh, device=dev), torch.randn(grows, Hh, device=dev)
    gbeta, gda, gdb = (torch.empty(grows, Hh, device=dev, dtype=torch.bfloat16) for _ in range(3))
    gpart = torch.empty(lib.lmoe_gdn_gates_partials(grows, Hh), 2, Hh, device=dev)
    gdpar = torch.empty(2, Hh, device=dev)
    ngla = 8 * 16 * 2048 * 64
    extra = {   # name: (launch, bytes moved)
        "gdn_gates_fwd": (lambda: lib.lmoe_gdn_gates_fwd(p(ga), p(gb), p(gA), p(gD), p(gg), p(gbeta), grows, Hh, bf, st),
                          grows * Hh * (2 + 2 + 4 + 2)),
        "gdn_gates_bwd": (lambda: lib.lmoe_gdn_gates_bwd(p(ga), p(gb), p(gA), p(gD), p(gdg), p(gbeta), p(gda), p(gdb),
                                                         p(gpart), p(gdpar), grows, Hh, bf, st),
                          grows * Hh * (2 + 2 + 4 + 2 + 2 + 2)),
        "gla_gate_fwd": (lambda: lib.lmoe_gla_gate_fwd(p(x), p(out), ngla, bf, 16.0, float("-inf"), st), ngla * 4),
        "gla_gate_bwd": (lambda: lib.lmoe_gla_gate_bwd(p(x), p(dy), p(out), ngla, bf, 16.0, float("-inf"), st), ngla * 6),
    }
    # one decoding step of the gated delta rule (token-by-token kernel): 256 sequences, H = 16, K = V = 128,
    # fp32 state read and written once
    from linear_moe_amd._host import SeqPlan, _desc, base_args
    Nd, Hd = 256, 16
    dq, dk, dv, do_ = (torch.randn(Nd, 1, Hd, D, device=dev, dtype=torch.bfloat16) for _ in range(4))
    dgt = -torch.rand(Nd, 1, Hd, device=dev)
    dbt = torch.rand(Nd, 1, Hd, device=dev, dtype=torch.bfloat16)
    dh0 = torch.randn(Nd, Hd, D, D, device=dev) * 0.1
    dht = torch.empty_like(dh0)
    da = base_args(dq, dk, dv, False, None, SeqPlan(Nd, 1, None, dev), (Nd, 1, Hd, D, D))
    da.gate, da.g, da.g_dtype = _lib.GATE_SCALAR, _desc(dgt, False), _lib.LMOE_F32
    da.beta, da.beta_dtype = _desc(dbt, False), bf
    da.h0, da.ht, da.o = dh0.data_ptr(), dht.data_ptr(), _desc(do_, False)
    extra["gdn_decode_step_256seq"] = (lambda: lib.lmoe_fused_recurrent_fwd(C.byref(da), 2, st),
                                       2 * dh0.numel() * 4 + 4 * Nd * Hd * D * 2)
    # mixture-of-memories routing: B = 4, S = 8192, hidden 2048, 4 memories, top-2 -> 65536 packed rows
    from linear_moe_amd import mom_plan
    mB, mS, mE, mk, mD = 4, 8192, 4, 2, 2048
    msel = torch.topk(torch.rand(mB, mS, mE, device=dev), mk, dim=-1)[1]
    plan = mom_plan(msel, mE)
    mx = torch.randn(mB * mS, mD, device=dev, dtype=torch.bfloat16)
    mxp = torch.empty(plan.T_total, mD, device=dev, dtype=torch.bfloat16)
    mw = torch.rand(mB * mS, mk, device=dev, dtype=torch.bfloat16)
    mo = torch.empty_like(mx)
    extra["mom_pack"] = (lambda: lib.lmoe_mom_gather(p(mx), p(plan.src_token), None, p(mxp), plan.T_total, mD, bf, st),
                         (mx.numel() + mxp.numel()) * 2)
    extra["mom_combine"] = (lambda: lib.lmoe_mom_combine(p(mxp), p(plan.row_of), p(mw), p(mo), mB * mS, mk, mD, bf, st),
                            (mxp.numel() + mo.numel()) * 2)
    # HGRN2 gates on the forget projection of contract config 3's shape (bf16 in, k bf16 + g fp32 out), and the
    # Taylor feature map of Based on [8,16,2048] rows of D = 16 -> 153 features in 192 padded columns
    hk, hg, hdg = torch.empty(ngla, device=dev, dtype=torch.bfloat16), torch.empty(ngla, device=dev), torch.randn(ngla, device=dev)
    extra["hgrn2_gates_fwd"] = (lambda: lib.lmoe_hgrn2_gate_fwd(p(x), None, p(hk), p(hg), ngla, 64, bf, st), ngla * (2 + 2 + 4))
    extra["hgrn2_gates_bwd"] = (lambda: lib.lmoe_hgrn2_gate_bwd(p(x), None, p(dy), p(hdg), p(out), ngla, 64, bf, st),
                                ngla * (2 + 2 + 4 + 2))
    frows, fD, fKp = 8 * 16 * 2048, 16, 192
    fx, fdx = (torch.randn(frows, fD, device=dev, dtype=torch.bfloat16) for _ in range(2))
    fy = torch.randn(frows * fKp, device=dev, dtype=torch.bfloat16)
    fc = (1.0, fD ** -0.25, (2.0 * fD) ** -0.5, fD ** -0.5)
    extra["taylor_featmap_fwd"] = (lambda: lib.lmoe_quad_featmap_fwd(p(fx), p(fy), frows, fD, fKp, *fc, bf, st),
                                   frows * (fD + fKp) * 2)
    extra["taylor_featmap_bwd"] = (lambda: lib.lmoe_quad_featmap_bwd(p(fx), p(fy), p(fdx), frows, fD, fKp, *fc, bf, st),
                                   frows * (2 * fD + fKp) * 2)
    # prologue / epilogue of the gated-delta-rule mixer on the headline shape (rows = B T H): the fused projection
    # [T, B, H, 3 D] in, q^, k^, silu(v) out; o x swish(gate) with the change of layout
    pB, pH = 4, 16
    pT = rows // (pB * pH)
    pqkv, pdqkv = (torch.randn(pT, pB, pH * 3 * D, device=dev, dtype=torch.bfloat16) for _ in range(2))
    extra["gdn_qkv_prologue_fwd"] = (lambda: lib.lmoe_gdn_qkv_prologue_fwd(p(pqkv), p(x), p(dy), p(gate), pT, pB, pH, D, bf, 1e-6, st),
                                     6 * rows * D * 2)
    extra["gdn_qkv_prologue_bwd"] = (lambda: lib.lmoe_gdn_qkv_prologue_bwd(p(pqkv), p(x), p(dy), p(gate), p(pdqkv), pT, pB, pH, D, bf,
                                                                           1e-6, st), 9 * rows * D * 2)
    extra["swish_gate_relayout_fwd"] = (lambda: lib.lmoe_swish_gate_relayout_fwd(p(x), p(gate), p(out), pT, pB, pH * D, bf, st),
                                        3 * rows * D * 2)
    extra["swish_gate_relayout_bwd"] = (lambda: lib.lmoe_swish_gate_relayout_bwd(p(x), p(gate), p(dy), p(out), p(out2), pT, pB,
                                                                                 pH * D, bf, st), 5 * rows * D * 2)
    res = {}
    cases = {n: (f, k * rows * D * 2) for n, (f, k) in cases.items()}
    cases.update(extra)
    for name, (launch, nbytes) in cases.items():
        for _ in range(3):
            _lib.check(launch(), name)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            launch()
        e1.record()
        e1.synchronize()
        sec = e0.elapsed_time(e1) * 1e-3 / reps
        res[name] = {"us": round(sec * 1e6, 1), "bytes": nbytes, "GB/s": round(nbytes / sec / 1e9, 1),
                     "frac_hbm_peak": round(nbytes / sec / PEAK_HBM, 3)}
    return {"metric": "row-wise neighbour kernels, algorithmic GB/s", "unit": "GB/s", "dtype": "bf16",
            "config": {"workload": f"{rows} rows x {D} bf16 (q / k / o rows of B=4 H=16 T=8192)"}, "kernels": res}


def trace_state_fwd(lib, x, dims, work_group=16):
    """Per-phase breakdown of one chunk period of the forward sequential pass (k_gdn_state_fwd_reg) on the headline
    workload: the traced instance of the kernel records the shader clock where each team of the traced work-group
    arrives at and leaves the two barriers of a chunk and at a few points in between
    (lmoe_trace_gdn_state_fwd, include/lmoe.h).  Returns averages over the middle chunks of the sequence, in cycles
    after the release of barrier 1 of the same chunk (negative: before it, i.e. in the previous chunk's phase 2)."""
    import torch
    from linear_moe_amd import _lib
    from linear_moe_amd.gated_delta_rule import GDNCall
    B, T, H, K, V = dims
    call = GDNCall(keep=True)
    call.forward(x["q"], x["k"], x["v"], x["g"], x["beta"], None, None, False, None, False)
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    slots, chunks, marks = 4, 128, 8
    tr = torch.zeros(slots * chunks * marks, dtype=torch.int64, device=x["q"].device)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for _ in range(3):
        _lib.check(lib.lmoe_trace_gdn_state_fwd(C.byref(call.fwd_args), tr.data_ptr(), work_group, st), "trace")
    e0.record()
    _lib.check(lib.lmoe_trace_gdn_state_fwd(C.byref(call.fwd_args), tr.data_ptr(), work_group, st), "trace")
    e1.record()
    e1.synchronize()
    traced_us = e0.elapsed_time(e1) * 1e3
    t = tr.cpu().view(slots, chunks, marks).double()
    nch = min(chunks, (T + CH - 1) // CH)
    c0, c1 = nch // 4, nch - nch // 4
    ref = t[0, c0:c1, 1]                                          # the consumer leaves barrier 1
    period = float((t[0, c0 + 1:c1 + 1, 1] - t[0, c0:c1, 1]).mean())
    names = {0: {0: "arrives_b1", 1: "leaves_b1", 5: "kS_formed", 2: "arrives_b2_vnew_written", 3: "leaves_b2",
                 6: "state_updated", 4: "state_written"},
             1: {0: "arrives_b1", 1: "leaves_b1", 2: "arrives_b2_qS_formed", 3: "leaves_b2", 4: "o_written"},
             2: {0: "arrives_b1", 1: "leaves_b1", 6: "k_staged", 2: "arrives_b2_P_formed", 3: "leaves_b2",
                 4: "stores_issued", 5: "loads_issued"},
             3: {0: "arrives_b1", 1: "leaves_b1", 2: "arrives_b2_loads_issued", 3: "leaves_b2", 4: "tiles_staged"}}
    teams = {0: "consumer_wave", 1: "helper_wave", 2: "loader_team_1", 3: "loader_team_2"}
    out = {}
    for s_, nm in teams.items():
        out[nm] = {}
        for m, label in names[s_].items():
            d = float((t[s_, c0:c1, m] - ref).mean())
            if m == 0:
                d += period                                      # arrival at barrier 1 of the NEXT chunk
                label = "arrives_next_b1"
            out[nm][label] = round(d)
    return {"metric": "k_gdn_state_fwd_reg: shader-clock cycles after barrier 1 of a chunk, per team (traced build)",
            "unit": "cycles", "work_group": work_group, "chunks_averaged": [c0, c1], "period_cycles": round(period),
            "traced_kernel_us": round(traced_us, 1), "cycles_per_us": round(period * nch / traced_us, 1),
            "teams": out}


def trace_simple_gla_fwd(lib, dev, work_group=16):
    """The same breakdown for the forward pass of chunk_simple_gla (k_state_fwd_b) on contract configuration 2
    (retention, forward-only, B=4 H=16 T=4096 K=V=128 bf16): lmoe_trace_simple_gla_fwd, include/lmoe.h."""
    import torch
    from linear_moe_amd import _lib
    from linear_moe_amd.retention import retention_log_decay
    from linear_moe_amd.simple_gla import SimpleGLACall
    B, H, T, K = 4, 16, 4096, 128
    q, k, v = (torch.randn(B, H, T, K, device=dev, dtype=torch.bfloat16) for _ in range(3))
    g = retention_log_decay(H, dev)[None, :, None].expand(B, H, T)
    call = SimpleGLACall(keep=True)
    call.forward(q, k, v, g, None, None, True, None, True, save=False)
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    slots, chunks, marks = 3, 24, 8
    tr = torch.zeros(slots * chunks * marks, dtype=torch.int64, device=dev)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for _ in range(3):
        _lib.check(lib.lmoe_trace_simple_gla_fwd(C.byref(call.fwd_args), tr.data_ptr(), work_group, st), "trace")
    e0.record()
    _lib.check(lib.lmoe_trace_simple_gla_fwd(C.byref(call.fwd_args), tr.data_ptr(), work_group, st), "trace")
    e1.record()
    e1.synchronize()
    traced_us = e0.elapsed_time(e1) * 1e3
    t = tr.cpu().view(slots, chunks, marks).double()
    nall = (T + CH - 1) // CH
    nch = min(chunks, nall)
    c0, c1 = nch // 4, nch - nch // 4
    wrap = lambda d: ((d + 2.0 ** 31) % 2.0 ** 32) - 2.0 ** 31     # the stamps are the low 32 bits of the clock
    ref = t[0, c0:c1, 1]
    period = float(wrap(t[0, c0 + 1:c1 + 1, 1] - t[0, c0:c1, 1]).mean())
    names = {0: {0: "arrives_barrier", 1: "leaves_barrier", 5: "state_updated", 6: "state_copied", 2: "next_P_below_diagonal_formed",
                 3: "next_operands_read"},
             1: {0: "arrives_barrier", 1: "leaves_barrier", 5: "loads_issued", 2: "staged", 4: "hs_stored"},
             2: {0: "arrives_barrier", 1: "leaves_barrier", 5: "qS_issued", 2: "Pv_done", 4: "rows_stored",
                 6: "next_P_diagonal_formed_next_operands_read"}}
    teams = {0: "consumer_wave", 1: "loader_wave", 2: "output_wave"}
    out = {}
    for s_, nm in teams.items():
        out[nm] = {}
        for m, label in names[s_].items():
            d = float(wrap(t[s_, c0:c1, m] - ref).mean())
            if m == 0:
                d += period
                label = "arrives_next_barrier"
            out[nm][label] = round(d)
    return {"metric": "k_state_fwd_b: shader-clock cycles after the barrier of a chunk, per team (traced build)",
            "unit": "cycles", "config": {"workload": "retention fwd bf16 B=4 H=16 T=4096 K=V=128"},
            "work_group": work_group, "chunks_averaged": [c0, c1], "period_cycles": round(period),
            "traced_kernel_us": round(traced_us, 1), "cycles_per_us": round(period * nall / traced_us, 1),
            "teams": out}


def layer_bench(dev, steps, warmup):
    """The token-mixer path of the reference's gated-delta-rule layer between its projections (GEMMs left out):
    q / k / v split, layout change, SiLU, L2 norm, gate construction, the chunk op, layout change back and
    o * swish(o_gate) (linear_moe/sequence_modeling/linear_attention.py:153-163, 255 around
    gated_deltanet/gated_deltanet.py:99-114), forward + backward on the headline shape.  `unfused` is the chain of
    strided copies, row kernels and eager elementwise ops; `fused` the one-pass prologue / epilogue kernels;
    `mixer_core` prologue and op as one call (the op applies SiLU to v where it reads the projection)."""
    import torch
    import torch.nn.functional as F
    import linear_moe_amd as L
    B, T, H, D = 4, 8192, 16, 128
    g_ = torch.Generator().manual_seed(1004)
    rn = lambda *s: torch.randn(*s, generator=g_, dtype=torch.float32)
    bf = lambda x: x.to(torch.bfloat16).to(dev).requires_grad_(True)
    qkv, o_gate = bf(rn(T, B, H * 3 * D)), bf(rn(T, B, H * D))
    a, b = bf(rn(B, T, H)), bf(rn(B, T, H))
    A_log = torch.log(torch.rand(H, generator=g_) * 15 + 1).to(dev).requires_grad_(True)
    dt_bias = (rn(H) * 0.1).to(dev).requires_grad_(True)
    dy = rn(T, B, H * D).to(torch.bfloat16).to(dev)
    leaves = [qkv, o_gate, a, b, A_log, dt_bias]

    def mixer(fused, core=False):
        gk, beta = L.gdn_gates(a, b, A_log, dt_bias)
        if core:       # prologue and op in one call: silu(v) never written, dv written into the projection's gradient
            return L.swish_gate_relayout(L.gdn_mixer_core(qkv, gk, beta, H, D), o_gate)
        if fused:
            q, k, v = L.gdn_qkv_prologue(qkv, H, D)
        else:
            q, k, v = torch.split(qkv.view(T, B, H, 3 * D), [D, D, D], dim=3)
            q, k, v = (t.transpose(0, 1).contiguous() for t in (q, k, v))
            q, k, v = L.silu_l2_norm(q), L.silu_l2_norm(k), F.silu(v)
        o, _ = L.chunk_gated_delta_rule(q, k, v, gk, beta, head_first=False)
        if fused:
            return L.swish_gate_relayout(o, o_gate)
        return o.transpose(0, 1).reshape(T, B, H * D) * F.silu(o_gate)

    def step(fused, core=False):
        torch.autograd.grad([mixer(fused, core)], leaves, [dy])

    # the op alone on inputs of the same laws as the headline (what the layer's neighbours are compared with)
    x = gdn_inputs(B, T, H, D, D, 1004, torch.bfloat16, dev)
    ol = [x[n].requires_grad_(True) for n in ("q", "k", "v", "g", "beta")]

    def step_op():
        o, _ = L.chunk_gated_delta_rule(*ol, None, None, False, None, False)
        torch.autograd.grad([o], ol, [x["do"]])

    def timed(fn):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps

    for fn in (step_op, lambda: step(False), lambda: step(True), lambda: step(True, True)):   # everything warm first
        timed(fn)
    t_op = timed(step_op)
    t_un = timed(lambda: step(False))
    t_fu = timed(lambda: step(True))
    t_co = timed(lambda: step(True, True))
    t_un2 = timed(lambda: step(False))
    t_fu2 = timed(lambda: step(True))
    t_co2 = timed(lambda: step(True, True))
    t_un, t_fu, t_co = min(t_un, t_un2), min(t_fu, t_fu2), min(t_co, t_co2)
    return {"metric": "gated-delta-rule token mixer between its projections, fwd+bwd, ms", "unit": "ms",
            "config": {"workload": "B=4 T=8192 H=16 D=128 bf16: split, layout, SiLU, L2 norm, gates, chunk op, layout, swish gate"},
            "steps": steps, "warmup": warmup, "op_alone_ms": t_op * 1e3,
            "unfused_ms": t_un * 1e3, "fused_ms": t_fu * 1e3, "mixer_core_ms": t_co * 1e3,
            "neighbours_unfused_ms": (t_un - t_op) * 1e3, "neighbours_fused_ms": (t_fu - t_op) * 1e3,
            "neighbours_mixer_core_ms": (t_co - t_op) * 1e3,
            "neighbours_share_unfused": (t_un - t_op) / t_un, "neighbours_share_fused": (t_fu - t_op) / t_fu,
            "neighbours_share_mixer_core": (t_co - t_op) / t_co,
            "tokens_per_s_fused": B * T / t_fu, "tokens_per_s_mixer_core": B * T / t_co}


def other_configs(dev, steps, warmup, comparisons=True):
    """The four contract configurations beside the headline one, and the forward + backward of chunk_simple_gla on
    the shape of configuration 2, through the Python entry points (inputs of the contract's laws, drawn on the GPU:
    this leg times, the parity tests check): ms per call, tokens/s and the algorithmic bytes (every input read once,
    every output written once) against the HBM peak."""
    import torch
    import torch.nn.functional as F
    import linear_moe_amd as L

    def timed(fn):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps

    rn = lambda *s, dt=torch.bfloat16: torch.randn(*s, device=dev, dtype=dt)
    res = {}
    # 1: basic linear attention forward, fp32
    B, H, T, K = 1, 4, 512, 64
    q, k, v = (rn(B, H, T, K, dt=torch.float32) for _ in range(3))
    with torch.no_grad():
        sec = timed(lambda: L.chunk_linear_attn(q, k, v, normalize=False))
    sg_flops = lambda K, V: 2 * CH * K + 2 * CH * V + 4 * K * V       # per token and head, forward: q k^T, P v, q S, k^T v
    res["1 linear_attn fwd fp32 B=1 H=4 T=512 K=V=64"] = (sec, B * T, B * T * H * (2 * K + 2 * K) * 4,
                                                          B * T * H * sg_flops(K, K), PEAK_MFMA_F32)
    # 2: retention forward, bf16
    B, H, T, K = 4, 16, 4096, 128
    q, k, v = (rn(B, H, T, K) for _ in range(3))
    with torch.no_grad():
        sec = timed(lambda: L.chunk_retention(q, k, v, output_final_state=True))
    res["2 retention fwd bf16 B=4 H=16 T=4096 K=V=128"] = (sec, B * T, B * T * H * ((2 * K + 2 * K) * 2 + 4),
                                                           B * T * H * sg_flops(K, K), PEAK_MFMA_BF16)
    # 3: chunk_gla forward + backward, bf16
    B, H, T, K, V = 8, 16, 2048, 64, 128
    q, k = (rn(B, H, T, K).requires_grad_(True) for _ in range(2))
    v = rn(B, H, T, V).requires_grad_(True)
    g = (F.logsigmoid(rn(B, H, T, K, dt=torch.float32)) / 16).bfloat16().requires_grad_(True)
    do = rn(B, H, T, V)

    def f3():    # autograd.grad: no accumulation into .grad, which would be timed with the op
        o, _ = L.chunk_gla(q, k, v, g)
        torch.autograd.grad([o], [q, k, v, g], [do])
    sec = timed(f3)
    res["3 chunk_gla fwd+bwd bf16 B=8 H=16 T=2048 K=64 V=128"] = (sec, B * T, B * T * H * (9 * K + 5 * V) * 2,
                                                                  3 * B * T * H * sg_flops(K, V), PEAK_MFMA_BF16)
    # 5: packed gated delta rule forward + backward, 16 sequences of log-normal lengths, 65536 tokens
    N, Tt, H, K, V = 16, 65536, 32, 128, 128
    gen = torch.Generator().manual_seed(1005)
    raw = torch.exp(8 + torch.randn(N, generator=gen))
    lens = torch.clamp((raw / raw.sum() * Tt).floor().long(), min=1)
    lens[lens.argmax()] += Tt - lens.sum()
    cu = torch.zeros(N + 1, dtype=torch.int32)
    cu[1:] = lens.cumsum(0)
    cu = cu.to(dev)
    q = F.normalize(rn(1, Tt, H, K, dt=torch.float32), dim=-1).bfloat16().requires_grad_(True)
    k = F.normalize(rn(1, Tt, H, K, dt=torch.float32), dim=-1).bfloat16().requires_grad_(True)
    v = rn(1, Tt, H, V).requires_grad_(True)
    beta = torch.rand(1, Tt, H, device=dev).bfloat16().requires_grad_(True)
    g = (-torch.rand(1, Tt, H, device=dev)).requires_grad_(True)
    h0 = (rn(N, H, K, V, dt=torch.float32) * 0.1).requires_grad_(True)
    do, dht = rn(1, Tt, H, V), rn(N, H, K, V, dt=torch.float32)

    def f5():
        o, ht = L.chunk_gated_delta_rule(q, k, v, g, beta, None, h0, True, cu, False)
        torch.autograd.grad([o, ht], [q, k, v, g, beta, h0], [do, dht])
    sec = timed(f5)
    res["5 packed gated_delta_rule fwd+bwd bf16 16 seqs 65536 tokens H=32 K=V=128"] = (
        sec, Tt, Tt * H * ((6 * K + 5 * V) * 2 + 3 * 2 + 12) + 4 * N * H * K * V * 4,
        3 * Tt * H * (6 * CH * K + 4 * CH * V + 6 * K * V + (2 / 3) * CH * CH), PEAK_MFMA_BF16)
    # 6 (not a contract configuration): the shape of configuration 2 with its backward, the training step of the
    # chunk_simple_gla family (retention, lightning attention, basic linear attention); per-token log-decays
    B, H, T, K = 4, 16, 4096, 128
    q, k, v = (rn(B, T, H, K).requires_grad_(True) for _ in range(3))
    g = (-torch.rand(B, T, H, device=dev) * 0.1).requires_grad_(True)
    do = rn(B, T, H, K)

    def f6():
        o, _ = L.chunk_simple_gla(q, k, v, g, head_first=False)
        torch.autograd.grad([o], [q, k, v, g], [do])
    sec = timed(f6)
    res["6 simple_gla fwd+bwd bf16 B=4 H=16 T=4096 K=V=128"] = (sec, B * T, B * T * H * ((6 * K + 5 * K) * 2 + 12),
                                                                3 * B * T * H * sg_flops(K, K), PEAK_MFMA_BF16)
    # 7 (not a contract configuration): the headline shape with a value head of 256 columns (expand_v = 2), in one
    # call (kernel instances for K = 128, V = 256) and as the two calls on 128 columns each that it would otherwise
    # be cut into (each repeats the WY preparation and the reads of q, k; dq, dk, dg, dbeta are added afterwards)
    B, T, H, K, V = 4, 8192, 16, 128, 256
    q = F.normalize(rn(B, T, H, K, dt=torch.float32), dim=-1).bfloat16().requires_grad_(True)
    k = F.normalize(rn(B, T, H, K, dt=torch.float32), dim=-1).bfloat16().requires_grad_(True)
    v = rn(B, T, H, V).requires_grad_(True)
    beta = torch.rand(B, T, H, device=dev).bfloat16().requires_grad_(True)
    g = (-torch.rand(B, T, H, device=dev) * 0.1).requires_grad_(True)
    do = rn(B, T, H, V)

    def f7():
        o, _ = L.chunk_gated_delta_rule(q, k, v, g, beta)
        torch.autograd.grad([o], [q, k, v, g, beta], [do])

    def f7_halves():
        o = torch.cat([L.chunk_gated_delta_rule(q, k, v[..., c:c + 128], g, beta, K ** -0.5)[0] for c in (0, 128)], -1)
        torch.autograd.grad([o], [q, k, v, g, beta], [do])
    sec = timed(f7)
    # (comparisons=False: a profile of the command then holds one problem per kernel instance)
    extras = {"7": {"as_two_calls_on_128_columns_ms": round(timed(f7_halves) * 1e3, 4)}} if comparisons else {}
    res["7 gated_delta_rule fwd+bwd bf16 B=4 T=8192 H=16 K=128 V=256"] = (
        sec, B * T, B * T * H * ((6 * K + 5 * V) * 2 + 3 * 2 + 12),
        3 * B * T * H * (6 * CH * K + 4 * CH * V + 6 * K * V + (2 / 3) * CH * CH), PEAK_MFMA_BF16)
    # 8 (not a contract configuration): chunk_linear_attn with its normaliser (the default of the reference's
    # BasicLinearAttention), forward + backward on the shape of configuration 2, beside the same call without it
    B, H, T, K = 4, 16, 4096, 128
    q, k = (torch.rand(B, H, T, K, device=dev).bfloat16().requires_grad_(True) for _ in range(2))
    v = rn(B, H, T, K).requires_grad_(True)
    do = rn(B, H, T, K)

    def f8(normalize):
        o, _ = L.chunk_linear_attn(q, k, v, normalize=normalize)
        torch.autograd.grad([o], [q, k, v], [do])
    sec = timed(lambda: f8(True))
    if comparisons:
        extras["8"] = {"without_normaliser_ms": round(timed(lambda: f8(False)) * 1e3, 4)}
    res["8 linear_attn normalize=True fwd+bwd bf16 B=4 H=16 T=4096 K=V=128"] = (
        sec, B * T, B * T * H * ((6 * K + 5 * K) * 2), 3 * B * T * H * sg_flops(K, K), PEAK_MFMA_BF16)
    # one roofline record per configuration, for the whole call on its minimal traffic (every input read once, every
    # output written once): all five are bound by HBM on that count (arithmetic intensity below peak flops / peak
    # bytes).  `traffic` = HBM bytes per call summed over its kernels, from the FETCH_SIZE / WRITE_SIZE counters
    # (OTHER_TRAFFIC, measured on the sources OTHER_TRAFFIC_SHA16 names; null when the sources have changed since)
    fresh = all_sources_sha16() == OTHER_TRAFFIC_SHA16
    out = {}
    for n, (sec, tok, nb, fl, peak_f) in res.items():
        out[n] = {"ms": round(sec * 1e3, 4), "tokens_per_s": round(tok / sec), "algorithmic_bytes": nb,
                  "algorithmic_flops": round(fl), "frac_hbm_peak": round(nb / sec / PEAK_HBM, 4),
                  "roofline": {"bound": "hbm", "achieved": round(nb / sec / 1e9, 1), "peak": PEAK_HBM / 1e9,
                               "unit": "GB/s", "frac": round(nb / sec / PEAK_HBM, 4),
                               "mfma_frac": round(fl / sec / peak_f, 4),
                               "traffic": OTHER_TRAFFIC.get(n[0]) if fresh else None}}
        out[n].update(extras.get(n[0], {}))
    return {"metric": "contract configurations 1, 2, 3, 5, the training step on the shape of 2 (6) and the headline "
                      "shape with V = 256 (7), chunk_linear_attn with its normaliser (8): ms per call, tokens/s", "unit": "ms", "steps": steps,
            "warmup": warmup, "data": "synthetic", "configs": out}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--settle-steps", type=int, default=-1,
                    help="steps that have run before the reported pass starts its own --warmup (default, and minimum: "
                         "warmup + steps, i.e. the reported pass is the second of two identical ones; the first is "
                         "always in the record as ms_per_step_first_pass)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--stage-reps", type=int, default=40)
    ap.add_argument("--neighbours", action="store_true",
                    help="instead of the headline step: the row-wise kernels around the op (L2 norm, SiLU + L2 norm, "
                         "RMS norm with and without the swish gate) on the rows of the same workload, one JSON line")
    ap.add_argument("--trace-state-fwd", action="store_true",
                    help="instead of the headline step: the per-phase breakdown of one chunk period of the forward "
                         "sequential pass on the headline workload, one JSON line")
    ap.add_argument("--trace-simple-gla-fwd", action="store_true",
                    help="instead of the headline step: the same breakdown for the forward pass of chunk_simple_gla "
                         "on contract configuration 2, one JSON line")
    ap.add_argument("--layer", action="store_true",
                    help="instead of the headline step: the token-mixer path of the gated-delta-rule layer between its "
                         "projections (no GEMMs), with and without the one-pass prologue / epilogue kernels, one JSON line")
    ap.add_argument("--other-configs", action="store_true",
                    help="instead of the headline step: contract configurations 1, 2, 3 and 5, the training step on the "
                         "shape of 2, V = 256 and the normalised linear attention, one JSON line")
    ap.add_argument("--skip-comparisons", action="store_true",
                    help="with --other-configs: leave out the legs that run the same problems through the slower paths "
                         "(V = 256 as two calls, linear attention without its normaliser), so that a profile of the "
                         "command holds one problem per kernel instance")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the op shards over batch and heads without "
              "communication); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from linear_moe_amd import _lib
    from linear_moe_amd.gated_delta_rule import GDNCall
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    lib = _lib.load()
    dev = torch.device("cuda:0")
    B, T, H, K, V, seed = 4, 8192, 16, 128, 128, 1004
    # known-size device copy: the yardstick for the FETCH_SIZE / WRITE_SIZE counters under rocprofv3
    src = torch.empty(CALIB_COPY_BYTES, dtype=torch.uint8, device=dev).fill_(1)
    dst = torch.empty_like(src)
    dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst

    if args.neighbours:
        print(json.dumps(neighbours(lib, B * T * H, K, dev, args.stage_reps)))
        return
    if args.other_configs:
        print(json.dumps(other_configs(dev, args.steps, args.warmup, not args.skip_comparisons)))
        return
    if args.layer:
        print(json.dumps(layer_bench(dev, args.steps, args.warmup)))
        return
    if args.trace_simple_gla_fwd:
        print(json.dumps(trace_simple_gla_fwd(lib, dev)))
        return
    x = gdn_inputs(B, T, H, K, V, seed, torch.bfloat16, dev)
    if args.trace_state_fwd:
        print(json.dumps(trace_state_fwd(lib, x, (B, T, H, K, V))))
        return

    from linear_moe_amd import chunk_gated_delta_rule

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / args.steps

    # the step as a user of the library runs it: the public entry point under autograd (its allocations, the
    # autograd bookkeeping and the casts of the gradients to the input dtypes are inside the timed region)
    leaves = [x[n].requires_grad_(True) for n in ("q", "k", "v", "g", "beta")]

    def step_public():
        o, _ = chunk_gated_delta_rule(*leaves, None, None, False, None, False)
        torch.autograd.grad([o], leaves, [x["do"]])

    # the same kernels driven through the call object (no autograd): what the per-kernel timing uses
    call = GDNCall(keep=True)
    xd = {n: t.detach() for n, t in x.items()}

    def step_direct():
        call.forward(xd["q"], xd["k"], xd["v"], xd["g"], xd["beta"], None, None, False, None, False)
        call.backward(xd["do"], None)

    # What runs first after start-up is slow: the first 25 or so steps on a GPU that has been idle (even for 0.2 s),
    # on memory the allocator has just obtained, take up to 8 % longer than every later one (measured: step by
    # step the time falls from 1.3x to 1.0x over about 30 steps, and rises again after a pause or after
    # torch.cuda.empty_cache(); single kernels and whole steps alike).  The op lives inside long training runs, so
    # `value` is the steady-state figure, under one fixed definition: pass 1 = `warmup` untimed steps, then exactly
    # `steps` timed ones (ms_per_step_first_pass: what the flags ask for, literally); then `settle_steps` more
    # untimed steps where that flag asks for more than pass 1 already ran; then pass 2 = `warmup` untimed + `steps`
    # timed steps again, which is `value`.  warmup_effective = untimed + timed steps that ran before the reported
    # region started.
    dt_first = timed(step_public)
    settle_extra = max(0, args.settle_steps - (args.warmup + args.steps)) if args.settle_steps >= 0 else 0
    for _ in range(settle_extra):
        step_public()
    dt = timed(step_public)
    warmup_effective = 2 * args.warmup + args.steps + settle_extra
    dt_direct = timed(step_direct)
    # beside the headline: per-step statistics (an event pair per step), forward and backward on their own, and the
    # step with the caches flushed in front of it (512 MiB written between steps: twice the memory-side cache), all
    # through the call object, after everything above has run
    def per_step(fn, flush=None):
        ms = []
        for _ in range(args.steps):
            if flush is not None:
                flush.add_(1)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            fn()
            e1.record()
            e1.synchronize()
            ms.append(e0.elapsed_time(e1))
        ms.sort()
        return {"median": ms[len(ms) // 2], "min": ms[0], "max": ms[-1]}

    def fwd_only():
        call.forward(xd["q"], xd["k"], xd["v"], xd["g"], xd["beta"], None, None, False, None, False)

    def bwd_only():
        call.backward(xd["do"], None)
    fwd_only()
    stats = {"step": per_step(step_direct), "fwd": per_step(fwd_only), "bwd": per_step(bwd_only),
             "step_caches_flushed": per_step(step_direct, torch.zeros(512 << 20, dtype=torch.uint8, device=dev))}
    stages = time_stages(call, lib, args.stage_reps)

    tokens = B * T
    # whole-op algorithmic work per token and head: fwd 6CK+4CV+6KV+(2/3)C^2 flops, x3 for fwd+bwd;
    # bytes: every input read once, every output written once
    f_tok = 3 * (6 * CH * K + 4 * CH * V + 6 * K * V + (2 / 3) * CH * CH)
    b_tok = (6 * K + 5 * V) * 2 + 3 * 2 + 12
    flops, bytes_ = f_tok * tokens * H, b_tok * tokens * H

    dom = max(stages, key=stages.get)
    f_c, b_c = stage_model(dom, K, V)
    units = (B * T // CH) * H
    ai = f_c / b_c
    if ai >= PEAK_MFMA_BF16 / PEAK_HBM:
        roof = {"bound": "mfma", "achieved": f_c * units / stages[dom] / 1e12, "peak": PEAK_MFMA_BF16 / 1e12,
                "unit": "TFLOP/s"}
    else:
        roof = {"bound": "hbm", "achieved": b_c * units / stages[dom] / 1e9, "peak": PEAK_HBM / 1e9, "unit": "GB/s"}
    roof["frac"] = roof["achieved"] / roof["peak"]
    # the same roofline for the whole op on its minimal traffic (every input read once, every output written once):
    # `frac` above is the dominant kernel on ITS bytes, which include intermediates the pipeline writes and re-reads
    roof["frac_whole_op"] = bytes_ / dt / PEAK_HBM
    roof["mfma_frac_whole_op"] = flops / dt / PEAK_MFMA_BF16
    fresh = kernel_sources_sha16() == TRAFFIC_SOURCES_SHA16
    roof["traffic"] = MEASURED_TRAFFIC.get(STAGE_NAMES[dom]) if fresh else None
    if not fresh:
        roof["traffic_note"] = "kernel sources changed since the counters were read: not re-measured"
    roof["kernel"] = STAGE_NAMES[dom]
    roof["kernel_us"] = stages[dom] * 1e6
    roof["flops_per_launch"] = f_c * units
    roof["bytes_per_launch"] = b_c * units

    rec = {
        "metric": "chunk GDN fwd+bwd tokens/s @T=8k,H=16,D=128 bf16; % bf16 MFMA peak",
        "value": tokens / dt, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": dt * 1e3, "ms_per_step_call_object": dt_direct * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "ms_per_step_first_pass": dt_first * 1e3, "value_first_pass": tokens / dt_first,
        "warmup_effective": warmup_effective,
        "order": "pass 1 = warmup untimed + steps timed (ms_per_step_first_pass: GPU just woken up, memory just "
                 "allocated); value / ms_per_step = pass 2 of the same shape, run right behind it (steady state; "
                 "warmup_effective steps ran before its timed region)",
        "config": {"workload": "chunk_gated_delta_rule fwd+bwd B=4 H=16 T=8192 K=V=128 (contract config 4 of 5)",
                   "B": B, "T": T, "H": H, "K": K, "V": V, "chunk": CH,
                   "settle_steps": args.warmup + args.steps + settle_extra},
        "mfma_frac": flops / dt / PEAK_MFMA_BF16, "mfma_frac_first_pass": flops / dt_first / PEAK_MFMA_BF16,
        "hbm_frac_algorithmic": bytes_ / dt / PEAK_HBM,
        "tflops": flops / dt / 1e12,
        "kernels_us": {STAGE_NAMES[s]: round(t * 1e6, 1) for s, t in stages.items()},
        "kernels_sum_ms": sum(stages.values()) * 1e3,
        "ms_per_step_stats": {k: {n: round(v, 4) for n, v in d.items()} for k, d in stats.items()},
        "roofline": roof,
    }
    if not args.no_cpu:
        rec["cpu_baseline"] = cpu_baseline(B, T, H, K, V, seed)
    print(json.dumps(rec))


if __name__ == "__main__":
    main()
