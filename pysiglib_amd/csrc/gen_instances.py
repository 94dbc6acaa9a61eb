"""Generates the tree-kernel instance files and their registry.

For every (dtype, dimension D, degree N) in the table below this script picks
the lane partition (TAIL = depth of the register-resident subtree, K = letters
per lane at the first subtree level) with a small instruction-count model under
a register budget, and writes

    gen/inst_<nn>.hip   explicit instantiations + a KernelEntry array
    gen/registry.cpp    the list of all arrays

D = 0 denotes the run-time-dimension kernel (TAIL = 1), instantiated for every
degree 2..MAX_GENERIC_N; it serves every shape that has no specialised entry.

Usage: python gen_instances.py [--out gen] [--files 24]
"""
import argparse
import os

MAX_GENERIC_N = 16
GENERIC_K = 4
# Shapes beyond the specialised table: run-time-dimension kernels with more letters per lane (the chain work of a lane
# is shared by more top-level updates), (D, K) per direction and degree range; D = -1 is the wide layout (one letter
# group of one path per wave, the group's increments arriving through scalar loads), D = 0 the packed one.  Measured on
# MI355X before the table grew (d = 41 .. 80 at degree 4, 21 .. 32 at degree 5, 9 .. 16 at degree 6, 6 .. 8 at degree 7, 5 .. 6 at degree 8,
# 4 at degree 9 and 10): the wide layout wins wherever it applies except in the backward of 4 channels; forward K 8 up
# to 8 channels, K 32 where 32 divides the channel count (single precision), else K 16; backward K 8 up to 8 channels, 16 up to 32, 32
# beyond; the packed K 16 backward is kept for single precision at 9 .. 15 channels.
MANY_CHANNELS_MAX_N = 10
def many_channels(direction, N):
    if N <= 5:
        return ((-1, 16), (-1, 32)) if direction == "fwd" else ((0, 16), (-1, 16), (-1, 32))
    if N <= 8:
        return ((-1, 8), (-1, 16)) if direction == "fwd" else ((0, 16), (-1, 8), (-1, 16))
    return ((-1, 8),) if direction == "fwd" else ()

# value budgets (signature values held per lane); backward holds state + adjoint
BUDGET = {("f64", "fwd"): 100, ("f64", "bwd"): 60, ("f32", "fwd"): 170, ("f32", "bwd"): 100}

# hand-tuned overrides: (dtype, D, N, dir) -> (TAIL, K)
OVERRIDES = {
    # measured on MI355X (kernel ms at the benchmark workloads, see profiles/)
    ("f32", 5, 7, "fwd"): (4, 1),
    ("f64", 3, 12, "fwd"): (5, 1),      # 24.1 ms; (4, 3) 25.3, (3, 3) and (4, 1) 31.7
    ("f32", 17, 4, "fwd"): (2, 6),      # staged 0.66 ms; (1, 17) direct 0.96, (2, 9) staged 0.79, (2, 3) staged 0.91
    # the per-level Horner values of a 12-letter chain leave no room for a depth-4 subtree (256 paths of 200 steps)
    ("f64", 2, 15, "bwd"): (3, 2),      # 9.4 ms; (4, 2) 13.6, (2, 2) 16.1
    ("f64", 2, 16, "bwd"): (3, 2),      # 29.0 ms; (4, 2) 58.3, (2, 2) 42.2, (5, 2) 85.8
}


# which twin (scalar-load or LDS-staged increments) a shape launches: 0 the general rules at run time, 1 always
# staged, 2 never staged, 3 staged only when the launch leaves SIMDs under-filled.  Measured on MI355X.
STAGE_POLICY = {
    ("f32", 5, 7, "fwd"): 1,
    ("f32", 17, 4, "fwd"): 1,
    ("f64", 3, 12, "fwd"): 2,
}

# Partitions and feeds found by a sweep on MI355X (every partition within the register budget whose lane count and
# letter waste are reasonable, both feeds, at a throughput workload: batch ~3e7 / d^N paths of 128 points): entries
# that beat the model's choice by at least 12 %.  "staged": 1 always, 3 only when the launch is under-filled.
# "ms": kernel time of the model's choice and of the entry.  Hand entries above take precedence.
_TUNED = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tuned_partitions.json")
if os.path.exists(_TUNED):
    import json
    with open(_TUNED) as _f:
        for _k, _v in json.load(_f).items():
            _dt, _d, _n, _dir = _k.split(",")
            _key = (_dt, int(_d), int(_n), _dir)
            if _key not in OVERRIDES:
                OVERRIDES[_key] = tuple(_v["partition"])
                STAGE_POLICY[_key] = int(_v["staged"])

# additional partitions compiled next to the default one (selectable through
# cusig_amd_force_partition; used for tuning sweeps): (dtype, D, N, dir) -> [(TAIL, K), ...]
EXTRA = {
}
# tuning sweeps: SIGAMD_EXTRA_PARTITIONS names a JSON file {"f32,17,4,fwd": [[2, 6], [2, 9]], ...} of more of them
if os.environ.get("SIGAMD_EXTRA_PARTITIONS"):
    import json
    with open(os.environ["SIGAMD_EXTRA_PARTITIONS"]) as _f:
        for _k, _v in json.load(_f).items():
            _dt, _d, _n, _dir = _k.split(",")
            EXTRA[(_dt, int(_d), int(_n), _dir)] = [tuple(x) for x in _v]


def rows_sweep_wins(dtype, D, N):
    """Backward shapes that the by-row reverse sweep (sig_rows.hip) serves faster than a compiled instance would: measured
    on MI355X at 48 .. 128 channels, degrees 3 and 4: 1.1-4x in single precision, 1-2.3x in double precision up to 64
    channels and 4-12x beyond (at 40 channels the instances still win at degree 4, by 1.4-2x)."""
    return 3 <= N <= 8 and D >= 48


def spec_shapes():
    """(D, N) pairs that get specialised kernels."""
    caps = {2: 16, 3: 14, 4: 10, 5: 9, 6: 8, 7: 7, 8: 7}
    caps.update({d: 5 for d in range(9, 21)})
    caps.update({d: 6 for d in range(9, 13)})
    caps.update({d: 4 for d in range(21, 49)})
    caps.update({d: 5 for d in range(21, 25)})
    caps.update({d: 3 for d in range(49, 129)})
    out = []
    for d, nmax in sorted(caps.items()):
        for n in range(2, nmax + 1):
            if n == 2 and d >= 18:
                continue        # degree 2 of that many channels always runs in closed form on the matrix cores
            out.append((d, n))
    return out


def fwd_cost(D, N, tail, K):
    """VALU instructions per lane per step of the forward sweep."""
    m = N - tail
    cost = m  # increment gathers along the prefix
    for t in range(1, N + 1):
        if t == 1:
            cost += 1
        elif t <= m:
            cost += 1 + 2 * (t - 2) + 1
        else:
            cost += 1 + 2 * (m - 1)
            depth = t - m
            nodes = K
            for e in range(1, depth + 1):
                if e == depth:
                    cost += nodes
                else:
                    cost += nodes + nodes // (K if e == 1 else D) + nodes  # child U + parent scale (approx)
                nodes *= D
    return cost


def lead_lag_mode(D, staged):
    """Lead-lag twin of a staged forward instance: 1 (time channel last, D odd), 2 (no time channel, D even), 0 none.
    At least two raw channels, and narrow enough for the skipped half to matter less than the compile time."""
    if not staged or D < 4 or D > 40:
        return 0
    return 1 if D % 2 else 2


def lead_lag_mode_bwd(T, D, tail, staged):
    """Lead-lag twin of a backward instance.  Staged instances as in the forward; scalar-fed ones where they are the
    faster choice for lead-lag paths (double precision from 14 channels on, single precision beyond the staged range)
    and the subtree has a level below the lane's own letters for the mask to act on."""
    if staged:
        return lead_lag_mode(D, True)
    if tail < 2 or D > 40 or D < (14 if T == "double" else 32):
        return 0
    return 1 if D % 2 else 2


def choose(D, N, dtype, direction):
    key = (dtype, D, N, direction)
    if key in OVERRIDES:
        return OVERRIDES[key]
    # Beyond the dimensions the tuning sweeps covered, measured on MI355X at d = 80, 100, 128 (degree 3) and d = 36, 40
    # (degree 4) against the model's choice: forward 1.5-5x (35-50 TFLOP/s f32, 23-25 f64 at degree 3; 60 / 23 at degree
    # 4), backward 1.3-2x (10-12 TFLOP/s f32 at degree 3, 45-52 f32 / 11 f64 at degree 4).
    if N == 3 and D > 64:
        if direction == "fwd":
            return (1, -(-D // 4) if D <= 100 else 13)      # four letter groups without a stub
        if dtype == "f32":
            return (2, 2) if D <= 100 else (2, 1)
    if N == 4 and D > 32:
        if direction == "fwd":
            return (1, D) if dtype == "f32" else (1, D // 2 if D <= 40 else (D + 1) // 2)     # beyond 40: two groups also for odd D
        # f64 beyond 40 channels: three letters per lane no longer fit the registers (d = 48: 65.8 ms, two letters 19.5;
        # d = 44: 23.7 / 14.8; d = 41: 13.0 / 13.2)
        return (2, 2) if dtype == "f64" and D > 40 else (2, 3)
    if dtype == "f64" and direction == "fwd" and D >= 24 and N == 3:
        # measured on MI355X (d = 24, 32, 48 at degree 3): the f64 forward runs 1.1-1.8x faster with one subtree level
        # per lane and all (or half of) the letters than with the two-level subtrees the model picks
        return (1, D if D <= 32 else (D + 1) // 2)
    budget = BUDGET[(dtype, direction)]
    best = None
    for tail in range(1, N):
        for K in range(1, D + 1):
            vals = (N - tail) + K * (D ** tail - 1) // (D - 1)
            if vals > budget:
                continue
            ng = -(-D // K)
            lanes = ng * D ** (N - tail)
            total = lanes * fwd_cost(D, N, tail, K)
            cand = (total, -lanes, tail, K)
            if best is None or cand < best:
                best = cand
    if best is None:
        return (1, 1)
    return (best[2], best[3])


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--out", default=os.path.join(os.path.dirname(os.path.abspath(__file__)), "gen"))
    ap.add_argument("--files", type=int, default=24)
    ap.add_argument("--quick", action="store_true", help="small table (fast builds while developing)")
    args = ap.parse_args()
    os.makedirs(args.out, exist_ok=True)

    insts = []  # (T, D, N, tail, K, dir)
    shapes = spec_shapes()
    if args.quick:
        shapes = [(2, 2), (2, 3), (2, 4), (3, 2), (3, 3), (3, 4), (4, 3), (5, 3), (10, 5), (5, 7), (3, 12), (17, 4)]
    for dtype in ("f64", "f32"):
        T = "double" if dtype == "f64" else "float"
        for (D, N) in shapes:
            for direction in ("fwd", "bwd"):
                if direction == "bwd" and rows_sweep_wins(dtype, D, N):
                    continue
                tail, K = choose(D, N, dtype, direction)
                parts = [(tail, K, 1)] + [(tl, kk, 0) for (tl, kk) in EXTRA.get((dtype, D, N, direction), [])
                                          if (tl, kk) != (tail, K)]
                for (tl, kk, pref) in parts:
                    insts.append((T, D, N, tl, kk, direction, pref, 0))
                    # wide layout: also the LDS-staged variant (the backward gains nothing from it beyond ~13 channels)
                    if D ** (N - tl) >= 48 and D <= (64 if direction == "fwd" else 31):
                        insts.append((T, D, N, tl, kk, direction, pref, 1))
        for N in range(2, MAX_GENERIC_N + 1):
            for direction in ("fwd", "bwd"):
                insts.append((T, 0, N, 1, GENERIC_K, direction, 1, 0))
                if N <= MANY_CHANNELS_MAX_N:
                    for (dd, kk) in many_channels(direction, N):
                        insts.append((T, dd, N, 1, kk, direction, 0, 0))

    # balance files by a rough compile-cost estimate
    def weight(i):
        T, D, N, tail, K, direction, pref, zl = i
        w = K * (max(D, 1) ** tail) + N * N
        return w * (3 if direction == "bwd" else 1)
    insts.sort(key=weight, reverse=True)
    buckets = [[] for _ in range(args.files)]
    loads = [0] * args.files
    for i in insts:
        j = loads.index(min(loads))
        buckets[j].append(i)
        loads[j] += weight(i)

    for old in os.listdir(args.out):
        if old.startswith("inst_") or old == "registry.cpp":
            os.remove(os.path.join(args.out, old))

    for fi, bucket in enumerate(buckets):
        lines = ["// generated by gen_instances.py -- do not edit", '#include "../sig_launch.h"', "",
                 "namespace sigamd {", ""]
        # explicit kernel instantiations (seen by the device and the host pass)
        for (T, D, N, tail, K, direction, pref, zl) in bucket:
            zs = "true" if zl else "false"
            if direction == "fwd":
                lines.append("template __global__ void tree_fwd_kernel<%s, %d, %d, %d, %d, %s>(const %s*, %s*, int64_t, "
                             "int64_t, int, int64_t, int, int, int64_t, int*, int);" % (T, D, N, tail, K, zs, T, T))
                if lead_lag_mode(D, zl):
                    lines.append("template __global__ void tree_fwd_kernel<%s, %d, %d, %d, %d, true, %d>(const %s*, %s*, int64_t, "
                                 "int64_t, int, int64_t, int, int, int64_t, int*, int);" % (T, D, N, tail, K, lead_lag_mode(D, zl), T, T))
            else:
                lines.append("template __global__ void tree_bwd_kernel<%s, %d, %d, %d, %d, %s>(const %s*, const %s*, "
                             "const %s*, %s*, int64_t, int64_t, int, int64_t, int, int, int, int64_t, int);" % (T, D, N, tail, K, zs, T, T, T, T))
                if lead_lag_mode_bwd(T, D, tail, zl):
                    lines.append("template __global__ void tree_bwd_kernel<%s, %d, %d, %d, %d, %s, %d>(const %s*, const %s*, "
                                 "const %s*, %s*, int64_t, int64_t, int, int64_t, int, int, int, int64_t, int);"
                                 % (T, D, N, tail, K, zs, lead_lag_mode_bwd(T, D, tail, zl), T, T, T, T))
        lines.append("")
        lines.append("#if !defined(__HIP_DEVICE_COMPILE__)   // the launcher table is host data")
        lines.append("static const KernelEntry kEntries_%02d[] = {" % fi)
        for (T, D, N, tail, K, direction, pref, zl) in bucket:
            is64 = 1 if T == "double" else 0
            zs = "true" if zl else "false"
            pol = STAGE_POLICY.get(("f64" if is64 else "f32", D, N, direction), 0)
            if N == 4 and D > 32 and direction == "fwd":
                pol = 2         # measured at d = 36, 40: one subtree level with all letters runs 1.7x faster scalar-fed
            name = "%s_%s_d%s_n%d_t%d_k%d%s" % (direction, "f64" if is64 else "f32", "0w" if D < 0 else str(D), N, tail, K,
                                                "_lds" if zl else "")
            if direction == "fwd":
                ll = lead_lag_mode(D, zl)
                ll_fn = ("&launch_tree_fwd<%s, %d, %d, %d, %d, true, %d>" % (T, D, N, tail, K, ll)) if ll else "nullptr"
                lines.append('    {%d, %d, %d, %d, %d, %d, &launch_tree_fwd<%s, %d, %d, %d, %d, %s>, nullptr, "%s", %d, &fwd_waves_per_simd<%s, %d, %d, %d, %d, %s>, %d, %s},'
                             % (is64, D, N, tail, K, zl, T, D, N, tail, K, zs, name, pref, T, D, N, tail, K, zs, pol, ll_fn))
            else:
                ll = lead_lag_mode_bwd(T, D, tail, zl)
                ll_fn = ("&launch_tree_bwd<%s, %d, %d, %d, %d, %s, %d>" % (T, D, N, tail, K, zs, ll)) if ll else "nullptr"
                lines.append('    {%d, %d, %d, %d, %d, %d, nullptr, &launch_tree_bwd<%s, %d, %d, %d, %d, %s>, "%s", %d, &bwd_waves_per_simd<%s, %d, %d, %d, %d, %s>, %d, nullptr, %s},'
                             % (is64, D, N, tail, K, zl, T, D, N, tail, K, zs, name, pref, T, D, N, tail, K, zs, pol, ll_fn))
        lines.append("};")
        lines.append("extern const EntryList kList_%02d = {kEntries_%02d, %d};" % (fi, fi, len(bucket)))
        lines.append("#endif")
        lines += ["", "}  // namespace sigamd", ""]
        with open(os.path.join(args.out, "inst_%02d.hip" % fi), "w") as fh:
            fh.write("\n".join(lines))

    reg = ["// generated by gen_instances.py -- do not edit", '#include "../sig_registry.h"', "", "namespace sigamd {", ""]
    for fi in range(args.files):
        reg.append("extern const EntryList kList_%02d;" % fi)
    reg.append("")
    reg.append("const EntryList* all_entry_lists(int* n_lists)")
    reg.append("{")
    reg.append("    static const EntryList lists[] = {%s};" % ", ".join("kList_%02d" % fi for fi in range(args.files)))
    reg.append("    *n_lists = %d;" % args.files)
    reg.append("    return lists;")
    reg.append("}")
    reg += ["", "}  // namespace sigamd", ""]
    with open(os.path.join(args.out, "registry.cpp"), "w") as fh:
        fh.write("\n".join(reg))
    print("wrote %d instances into %d files under %s" % (len(insts), args.files, args.out))
    for (T, D, N, tail, K, direction, pref, zl) in sorted(insts, key=lambda i: (i[0], i[1], i[2], i[5])):
        if (D, N) in ((10, 5), (5, 7), (3, 12), (17, 4)) and not zl:
            print("  ", T, D, N, direction, "tail", tail, "K", K, "default" if pref else "extra")


if __name__ == "__main__":
    main()
