#!/usr/bin/env python3
"""Instructions per time step of a kernel's main loops, by class, from the compiler's assembly of these
sources (a development aid for the kernels that are bound by instruction issue on one wave).

    hipcc --offload-arch=gfx950 -O3 -std=c++17 -Xclang -target-feature -Xclang -packed-fp32-ops \\
          -I include -I recurrent-fwp_amd/csrc -mllvm -amdgpu-mfma-vgpr-form -S --cuda-device-only \\
          recurrent-fwp_amd/csrc/fwp_rec_reg.hip -o rec.s
    python3 recurrent-fwp_amd/csrc/isa_budget.py rec.s 'k_rec_fwd_regILi32ELi2ELi1ELi2E' 16

The third argument is the number of time steps one iteration of the loops covers (the tile length: the tile
loops are unrolled).  Every loop that does not overlap a larger one is listed, largest first: a kernel whose
waves have different roles has one loop per role.  Branches that are rarely taken (the exact softmax maximum)
are counted as if they always were."""
import collections
import re
import sys


def classify(op, line):
    dpp = "row_" in line or "quad_perm" in line or "dpp" in op
    if op.startswith("v_mfma"):
        return "MFMA"
    if op.startswith(("v_fmac", "v_fma", "v_pk_fma")):
        return "multiply-add" + (", operand through DPP" if dpp else "")
    if op.startswith("v_"):
        if op.startswith(("v_exp", "v_rcp", "v_log", "v_sqrt", "v_rsq")):
            return "exp / reciprocal"
        if op.startswith(("v_readlane", "v_readfirstlane", "v_writelane", "v_permlane")):
            return "lane read / row swap"
        if dpp:
            return "other vector through DPP (reductions, moves)"
        if op.startswith(("v_cmp", "v_cndmask")):
            return "compare / select"
        if op.startswith("v_mov"):
            return "vector move"
        if op.startswith(("v_mul_f32", "v_add_f32", "v_sub", "v_max_f32", "v_min_f32")):
            return "multiply or add"
        return "other vector (addresses, conversions)"
    if op.startswith("ds_"):
        return "LDS " + ("bpermute" if "permute" in op else "read" if "read" in op or "load" in op else "write")
    if op.startswith(("global_", "buffer_", "flat_")):
        return "vector memory"
    if op.startswith("s_waitcnt"):
        return "s_waitcnt"
    if op.startswith("s_nop"):
        return "s_nop (wait states)"
    if op.startswith("s_barrier"):
        return "s_barrier"
    return "scalar / branch"


def main():
    path, symbol, per = sys.argv[1], sys.argv[2], int(sys.argv[3])
    lines = open(path).read().split("\n")
    start = next(i for i, l in enumerate(lines) if re.match(r"^_Z\S+:", l) and symbol in l)
    end = next(i for i in range(start + 1, len(lines)) if lines[i].startswith(".Lfunc_end"))
    body = lines[start:end + 1]
    labels = {m.group(1): i for i, l in enumerate(body) for m in [re.match(r"^(\.LBB\d+_\d+):", l)] if m}
    loops = []
    for i, l in enumerate(body):
        m = re.match(r"\s+s_c?branch\w*\s+(\.LBB\d+_\d+)", l)
        if m and labels.get(m.group(1), i) < i:
            loops.append((i - labels[m.group(1)], labels[m.group(1)], i))
    loops.sort(reverse=True)
    chosen = []
    for n, a, b in loops:
        if all(b < ca or a > cb for _, ca, cb in chosen):
            chosen.append((n, a, b))
    print(f"{symbol}: {len(chosen)} loops that do not overlap")
    for n, a, b in chosen:
        cat = collections.Counter()
        for l in body[a:b + 1]:
            m = re.match(r"\s+([a-z_0-9]+)", l)
            if m and not l.strip().startswith((";", ".")):
                cat[classify(m.group(1), l)] += 1
        total = sum(cat.values())
        if total < 20 * per:
            continue
        print(f"\nloop of {total} instructions = {total / per:.1f} per step ({per} steps per iteration)")
        for c, k in sorted(cat.items(), key=lambda x: -x[1]):
            print(f"  {c:46s} {k / per:6.1f}")


if __name__ == "__main__":
    main()
