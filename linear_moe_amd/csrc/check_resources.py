#!/usr/bin/env python3
"""Build-time guard of the register-steered kernels.

The hot kernels of the gated delta rule and the forward pass and the fused backward kernel of chunk_simple_gla rely on the compiler keeping their working set in registers (explicit
steering: refreshed lane indices, pinned sums, fenced products).  A compiler or source change that makes one of them
spill, or lowers the number of waves it runs with, costs a large factor in speed without failing any test.  This
script reads the per-kernel resource reports that ``-Rpass-analysis=kernel-resource-usage`` wrote at compile time
(``<unit>.remarks``) and fails the build when an instance for 2-byte elements (the performance path) of a guarded
kernel uses scratch memory, spills vector registers, or falls below its minimum occupancy.  4-byte instances are the
parity path and are only reported.

usage: check_resources.py unit.remarks [...]
"""
import re
import sys

# kernel -> minimum waves per SIMD of its 2-byte instances (what the launch shape was tuned for: the sequential
# passes and the chunk-parallel backward run one work-group of 12 waves per CU = 3 waves per SIMD; the WY
# preparation two or three work-groups of 4 waves)
GUARDED = {
    "k_state_fwd_b": 3,
    "k_gdn_state_fwd": 3,
    "k_gdn_state_fwd_reg": 3,
    "k_gdn_state_bwd": 3,
    "k_gdn_bwd_chunk": 3,
    "k_gdn_wy_fwd": 2,
    "k_gla_fwd_fused": 3,
    "k_bwd_dqkv": 2,          # one work-group of 8 waves per CU; its first version spilled loop-invariant lane arithmetic
}
FIELDS = {"ScratchSize [bytes/lane]": "scratch", "VGPRs Spill": "vspill", "Occupancy [waves/SIMD]": "occ",
          "VGPRs": "vgpr", "AGPRs": "agpr", "LDS Size [bytes/block]": "lds"}


def parse(path):
    kernels, cur = {}, None
    for line in open(path, errors="replace"):
        m = re.search(r"remark:\s+(.*?)\s*\[-Rpass-analysis", line)
        if not m:
            continue
        body = m.group(1)
        if body.startswith("Function Name:"):
            cur = body.split(":", 1)[1].strip()
            kernels[cur] = {}
        elif cur is not None and ":" in body:
            key, val = body.rsplit(":", 1)
            if key.strip() in FIELDS:
                try:
                    kernels[cur][FIELDS[key.strip()]] = int(val)
                except ValueError:
                    pass
    return kernels


def main(paths):
    bad, seen = [], {k: 0 for k in GUARDED}
    for path in paths:
        for name, r in parse(path).items():
            for kern, min_occ in GUARDED.items():
                # Itanium mangling: <len><name>I<template args>; DF16b = __bf16
                if f"{len(kern)}{kern}I" not in name:
                    continue
                two_byte = f"{kern}IDF16b" in name or kern.endswith("_reg")     # the _reg kernels exist for bf16 only
                line = (f"{kern:<18} {'bf16' if two_byte else 'fp32'} vgpr {r.get('vgpr', -1):3d} agpr {r.get('agpr', -1):3d} "
                        f"scratch {r.get('scratch', -1):4d} B  vgpr-spill {r.get('vspill', -1):3d}  waves/SIMD {r.get('occ', -1)}  "
                        f"lds {r.get('lds', -1)}  {name}")
                if not two_byte:
                    continue
                seen[kern] += 1
                if r.get("scratch", 1) != 0 or r.get("vspill", 1) != 0 or r.get("occ", 0) < min_occ:
                    bad.append(line)
    missing = [k for k, n in seen.items() if n == 0]
    if missing:
        print("check_resources: no resource report found for", ", ".join(missing), file=sys.stderr)
        return 1
    if bad:
        print("check_resources: 2-byte instances of guarded kernels spill or lost occupancy "
              "(needed: scratch 0, vgpr-spill 0, waves/SIMD >= " + str(GUARDED) + "):", file=sys.stderr)
        for b in bad:
            print("  " + b, file=sys.stderr)
        return 1
    print(f"check_resources: {sum(seen.values())} bf16 instances of {len(GUARDED)} guarded kernels: no scratch, no spills, "
          "occupancy as tuned")
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
