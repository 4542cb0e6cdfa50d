"""Design-space exploration of (ps, wpb, dist) for the aggregation kernel on one GPU.

Counterpart of the reference's 5_MGG_DSE_*.py / bench_MGG_DSE_dist_ps.py / bench_MGG_DSE_dist_wpb.py, which sweep
dist x ps (wpb fixed) and dist x wpb (ps fixed) and tabulate the aggregation time.  Here the sweep runs in one
process on synthetic graphs of the benchmark shapes:

    python -m mgg_osdi23_amd.dse --workload share [--dim 16] [--iters 20] [--out table.json]
    python -m mgg_osdi23_amd.dse --workload whole --dim 16

Prints ps x wpb (dist = 1) and dist x ps (wpb = 8) tables in ms, GB/s of algorithmic traffic, and the best setting.

    python -m mgg_osdi23_amd.dse --workload whole --dim 44 --ld 48 --mode wd      # wpb x dist at ps 16, everything else by rule
    python -m mgg_osdi23_amd.dse --workload sparse --dim 64 --gin --mode core     # dense-core size sweep, best of a few wpb x dist

    python -m mgg_osdi23_amd.dse --mode heldout                                   # rules and cost model on graphs they never saw

`--mode wd`: the wpb x dist table at ps 16 with the order and the dense core left to the library (its rules and cost
model), and the time of the all-by-rule call beside the table's best.  `--mode core`: the aggregation time against the
size of the dense core (no counterpart in the reference), with the entries of the built plans (useful, padded, left to
the gather kernel) -- the data the library's cost model was fitted to -- and the size the model picks.
"""
from __future__ import annotations

import argparse
import json
import sys

import numpy as np

from . import host


# Graph families none of the library's rules or cost-model constants were fitted on (those came from sweeps on the three
# benchmark graphs "share", "whole" and "sparse" below): other generators, other skews, other sizes, other mean degrees.
#   name: (generator, generator arguments, ranks, row width, row pitch)
HELD_OUT = {
    "er32": ("er", dict(num_nodes=1_000_000, avg_degree=32.0, seed=101), 1, 64, 64),
    "er200": ("er", dict(num_nodes=500_000, avg_degree=200.0, seed=102), 1, 16, 16),
    "rmat45": ("rmat", dict(scale=20, num_nodes=1_000_000, num_draws=40_000_000, a=0.45, b=0.22, c=0.22, seed=103), 1, 41, 48),
    "rmat65": ("rmat", dict(scale=19, num_nodes=500_000, num_draws=60_000_000, a=0.65, b=0.15, c=0.15, seed=104), 1, 16, 16),
    "rmat57w64": ("rmat", dict(scale=20, num_nodes=1_000_000, num_draws=100_000_000, a=0.57, b=0.19, c=0.19, seed=105), 1, 64, 64),
    "share2": ("rmat", dict(scale=21, num_nodes=2_000_000, num_draws=30_000_000, a=0.57, b=0.19, c=0.19, seed=106, scramble=True), 2, 16, 16),
    # further batches: each was measured with the rules as they then stood, and what it showed went into them
    "rmat50w32": ("rmat", dict(scale=20, num_nodes=750_000, num_draws=50_000_000, a=0.50, b=0.20, c=0.20, seed=107), 1, 32, 32),
    "er64": ("er", dict(num_nodes=750_000, avg_degree=64.0, seed=108), 1, 41, 48),
    "rmat60w64": ("rmat", dict(scale=21, num_nodes=2_000_000, num_draws=80_000_000, a=0.60, b=0.17, c=0.17, seed=109), 1, 64, 64),
    "rmat57w24": ("rmat", dict(scale=19, num_nodes=400_000, num_draws=120_000_000, a=0.57, b=0.19, c=0.19, seed=110), 1, 24, 24),
    "rmat55w16": ("rmat", dict(scale=21, num_nodes=1_500_000, num_draws=60_000_000, a=0.55, b=0.20, c=0.20, seed=111), 1, 16, 16),
    "rmat62w41": ("rmat", dict(scale=20, num_nodes=600_000, num_draws=90_000_000, a=0.62, b=0.16, c=0.16, seed=112), 1, 41, 48),
    "er24w64": ("er", dict(num_nodes=2_000_000, avg_degree=24.0, seed=113), 1, 64, 64),
    "rmat48w64": ("rmat", dict(scale=19, num_nodes=300_000, num_draws=100_000_000, a=0.48, b=0.21, c=0.21, seed=114), 1, 64, 64),
    # the last four have only ever been measured with the rules as they are now
    "rmat52w48": ("rmat", dict(scale=20, num_nodes=900_000, num_draws=70_000_000, a=0.52, b=0.20, c=0.20, seed=115), 1, 48, 48),
    "rmat63w64": ("rmat", dict(scale=20, num_nodes=700_000, num_draws=110_000_000, a=0.63, b=0.15, c=0.17, seed=116), 1, 64, 64),
    "rmat58w20": ("rmat", dict(scale=21, num_nodes=1_800_000, num_draws=90_000_000, a=0.58, b=0.18, c=0.18, seed=117), 1, 20, 20),
    "rmat46w16": ("rmat", dict(scale=19, num_nodes=350_000, num_draws=140_000_000, a=0.46, b=0.22, c=0.22, seed=118), 1, 16, 16),
    # narrow rows beside a dense core in row-major order: made to check a candidate rule (2 rounds per wavefront there);
    # the graphs of width 20, here and above, set its lower bound; rmat56w24 and rmat59w28 agreed with it and moved nothing
    "rmat54w28": ("rmat", dict(scale=20, num_nodes=600_000, num_draws=80_000_000, a=0.54, b=0.20, c=0.20, seed=119), 1, 28, 28),
    "rmat61w12": ("rmat", dict(scale=21, num_nodes=1_200_000, num_draws=70_000_000, a=0.61, b=0.16, c=0.16, seed=120), 1, 12, 12),
    "rmat49w32": ("rmat", dict(scale=19, num_nodes=450_000, num_draws=110_000_000, a=0.49, b=0.21, c=0.21, seed=121), 1, 32, 32),
    "rmat56w24": ("rmat", dict(scale=21, num_nodes=1_600_000, num_draws=85_000_000, a=0.56, b=0.19, c=0.19, seed=122), 1, 24, 24),
    "rmat53w20": ("rmat", dict(scale=19, num_nodes=500_000, num_draws=65_000_000, a=0.53, b=0.20, c=0.20, seed=123), 1, 20, 20),
    "rmat59w28": ("rmat", dict(scale=20, num_nodes=1_000_000, num_draws=75_000_000, a=0.59, b=0.18, c=0.18, seed=124), 1, 28, 28),
}


def build_held_out(name: str, shrink: int = 0):
    """One of the HELD_OUT graphs as a workload dict (see build_workload); shrink divides nodes and edges by 2^k."""
    import torch
    gen, kw, ranks, dim, ld = HELD_OUT[name]
    kw = dict(kw)
    if gen == "er":
        kw["num_nodes"] >>= shrink
        V = kw["num_nodes"]
        ptr, col = host.gen_er(**kw)
    else:
        kw["num_nodes"] >>= shrink
        kw["num_draws"] >>= shrink
        kw["scale"] -= shrink
        V = kw["num_nodes"]
        if ranks > 1:
            npp, lb, ub = host.range_partition(V, ranks, 0)
            kw.update(row_lo=lb, row_hi=ub)
        ptr, col = host.gen_rmat(**kw)
    npp, lb, ub = host.range_partition(V, ranks, 0)
    if ranks > 1:
        lp, rp, lc, rc = host.split_CSR(ptr, col, lb, ub)
    else:
        lp, lc, rp, rc = ptr, col, np.zeros(V + 1, np.int32), np.zeros(0, np.int32)
    rows_tbl = ranks * npp
    x = np.zeros((rows_tbl, ld), np.float32)
    x[:, :dim] = host.fill_normal((rows_tbl, dim), seed=11)
    t = lambda a: torch.from_numpy(a).cuda() if len(a) else torch.zeros(1, dtype=torch.int32, device="cuda")
    w = dict(lb=lb, ub=ub, npp=npp, nnz=len(lc) + len(rc), rows=ub - lb, dim=dim, ld=ld, xr=torch.from_numpy(x).cuda(),
             xl=torch.from_numpy(np.ascontiguousarray(x[lb:ub])).cuda(), ptr_l=t(lp), col_l=t(lc), ptr_r=t(rp), col_r=t(rc),
             host=dict(ptr_l=lp, col_l=lc, ptr_r=rp, col_r=rc, x=x))
    w["out"] = torch.empty(ub - lb, ld, device="cuda")
    w["bytes"] = w["nnz"] * (4 + dim * 4) + w["rows"] * dim * 4 + (w["rows"] + 1) * 4 * (2 if len(rc) else 1)
    return w


def tune(w, gin=False):
    """The library's own search on a workload -> (knobs, ms)."""
    return host.tune_np_div(w["out"], w["xl"], w["ptr_l"], w["col_l"], w["ptr_r"], w["col_r"], w["lb"], w["ub"], w["dim"], w["npp"], 16,
                            input_remote=w["xr"], ld_in=w["ld"], ld_out=w["ld"], gin_eps=0.0 if gin else None)


def held_out_table(args):
    """Rules and cost model against measurement on the HELD_OUT graphs: by rule (every knob left at 0), the best cell of the
    wpb x dist table (order and core by rule), the library's search (ps x order x core size x wpb x dist), and the dense-core
    size the cost model predicts against the best of a sweep of sizes.  Prints one markdown table."""
    import torch
    rows = []
    for name in (args.only.split(",") if args.only else HELD_OUT):
        w = build_held_out(name, args.shrink)
        med = lambda wpb=0, dist=0, **kw: sorted(time_setting(w, 16, wpb, dist, args.iters, **kw) for _ in range(3))[1]
        for _ in range(3):
            time_setting(w, 16, 0, 0, args.iters, core_rows=0)
        rule = med(core_rows=0)
        rule_kernel = host.last_agg_kernel()
        grid = min((med(wpb=wpb, dist=d, core_rows=0), wpb, d) for wpb in (2, 4, 8, 16) for d in (1, 2, 4, 8, 16))
        host.forget(w["ptr_l"])  # the search must not find the rule's plans warm and its own cold
        knobs, _ = tune(w)
        searched = med(core_rows=0)  # the zeros now mean the searched setting
        host.forget(w["ptr_l"])
        import re
        m = re.search(r"core=(\d+)", rule_kernel)
        predicted = int(m.group(1)) if m else -1
        best_core = (rule if predicted < 0 else 1e30, -1)
        if not len(w["host"]["col_r"]):
            for K in (-1, 8192, 16384, 24576, 32768, 40960, 49152, 65536, 81920, 98304):
                if K > w["rows"] // 2:
                    continue
                cells = [(med(wpb=a, dist=b, core_rows=K), a, b) for a, b in ((4, 4), (4, 16), (8, 4), (8, 16))]
                print("  core %6d: " % K + "  ".join("wpb %d dist %2d %.4f" % (a, b, ms) for ms, a, b in cells) + "   by rule %.4f" % med(core_rows=K), flush=True)
                best_core = min(best_core, (min(cells)[0], K))
                host.forget(w["ptr_l"])
            at_predicted = min(med(wpb=a, dist=b, core_rows=predicted) for a, b in ((4, 4), (4, 16), (8, 4), (8, 16))) if predicted > 0 else best_core[0]
        else:
            at_predicted = best_core[0]
        rows.append((name, w["rows"], w["nnz"], w["dim"], rule, grid, searched, knobs, predicted, best_core, at_predicted, rule_kernel))
        print("%s: rule %.4f ms [%s]; best wpb x dist cell %.4f (wpb %d dist %d); searched %.4f %s; core predicted %d, best of sweep %d (%.4f ms, "
              "at the predicted size %.4f)" % (name, rule, rule_kernel, grid[0], grid[1], grid[2], searched, knobs, predicted, best_core[1],
                                               best_core[0], at_predicted), flush=True)
        host.release_cached()
        del w
        torch.cuda.empty_cache()
    print("\n| graph | rows | nnz | width | by rule (ms) | best wpb x dist cell | rule / cell | searched (ms) | rule / searched | core: predicted | "
          "core: best of sweep | predicted / best (ms ratio) |")
    print("|---|---|---|---|---|---|---|---|---|---|---|---|")
    for name, r, nnz, dim, rule, grid, searched, knobs, predicted, best_core, at_predicted, _k in rows:
        print("| %s | %d | %d | %d | %.4f | %.4f (wpb %d, dist %d) | %.3f | %.4f | %.3f | %d | %d | %.3f |" %
              (name, r, nnz, dim, rule, grid[0], grid[1], grid[2], rule / grid[0], searched, rule / searched, predicted, best_core[1],
               at_predicted / best_core[0]))


def build_workload(name: str, dim: int, small: bool, ld: int = 0, compact: bool = False):
    import torch
    ld = ld or dim
    if name == "share":
        scale, V, draws, num_gpus = (22, 4_194_304, 52_000_000, 8) if not small else (16, 65_536, 800_000, 8)
        npp, lb, ub = host.range_partition(V, num_gpus, 0)
        ptr, col = host.gen_rmat(scale, V, draws, seed=7, scramble=True, row_lo=lb, row_hi=ub)
        lp, rp, lc, rc = host.split_CSR(ptr, col, lb, ub)
        rows_tbl = num_gpus * npp
    else:
        if name == "sparse":  # 2.45 M nodes, ~123 M nnz (avg degree ~50): the GIN benchmark's graph
            scale, V, draws, seed = (22, 2_450_000, 64_000_000, 3) if not small else (16, 50_000, 1_300_000, 3)
        else:                 # 233 K nodes, ~228 M nnz (avg degree ~980): the GCN benchmark's graph
            scale, V, draws, seed = (18, 233_000, 216_000_000, 42) if not small else (14, 16_000, 1_500_000, 42)
        ptr, col = host.gen_rmat(scale, V, draws, seed=seed)
        npp, lb, ub = V, 0, V
        lp, lc = ptr, col
        rp, rc = np.zeros(V + 1, np.int32), np.zeros(0, np.int32)
        rows_tbl = V
    x = np.zeros((rows_tbl, ld), np.float32)
    x[:, :dim] = host.fill_normal((rows_tbl, dim), seed=11)
    dev = "cuda"
    t = lambda a: torch.from_numpy(a).to(dev) if len(a) else torch.zeros(1, dtype=torch.int32, device=dev)
    w = dict(lb=lb, ub=ub, npp=npp, nnz=len(lc) + len(rc), rows=ub - lb, dim=dim, ld=ld,
             xr=torch.from_numpy(x).to(dev), xl=torch.from_numpy(np.ascontiguousarray(x[lb:ub])).to(dev),
             ptr_l=t(lp), col_l=t(lc), ptr_r=t(rp), col_r=t(rc))
    if compact and len(rc):  # the remote rows staged compactly: one row per distinct remote id, most referenced first
        rcc, ids = host.compact_remote_device(w["col_r"], len(rc))
        w["col_r"], w["xr"] = rcc, w["xr"][ids.long()].contiguous()
    w["out"] = torch.empty(ub - lb, ld, device=dev)
    w["bytes"] = w["nnz"] * (4 + dim * 4) + w["rows"] * dim * 4 + (w["rows"] + 1) * 4 * (2 if len(rc) else 1)
    return w


def time_setting(w, ps, wpb, dist, iters, core_rows=-1, col_block_rows=0, gin=False):
    import torch

    def call():
        if gin:
            host.mgg_GIN_np_div(w["out"], w["xl"], w["ptr_l"], w["col_l"], w["ptr_r"], w["col_r"], w["lb"], w["ub"], w["dim"],
                                w["npp"], 0, ps, wpb, dist, 0.0, input_remote=w["xr"], ld_in=w["ld"], ld_out=w["ld"],
                                col_block_rows=col_block_rows, core_rows=core_rows)
        else:
            host.mgg_SAG_np_div(w["out"], w["xl"], w["ptr_l"], w["col_l"], w["ptr_r"], w["col_r"], w["lb"], w["ub"], w["dim"],
                                w["npp"], 0, ps, wpb, dist, input_remote=w["xr"], ld_in=w["ld"], ld_out=w["ld"],
                                col_block_rows=col_block_rows, core_rows=core_rows)

    call()
    call()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        call()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters


def sweep_wpb_dist(w, args):
    """wpb x dist at ps 16; order and dense core by the library's rules and cost model."""
    time_setting(w, 16, 0, 0, 4 * args.iters, core_rows=0, gin=args.gin)  # plans built, clocks up
    rule = time_setting(w, 16, 0, 0, args.iters, core_rows=0, gin=args.gin)
    print("everything by rule: %.4f ms   [%s]" % (rule, host.last_agg_kernel()))
    wpbs, dists = [2, 4, 8, 16], [1, 2, 4, 8, 16]
    print("\nms, ps = 16            " + "".join("dist=%-6d" % x for x in dists))
    best = (1e30, None)
    for wpb in wpbs:
        row = [time_setting(w, 16, wpb, d, args.iters, core_rows=0, gin=args.gin) for d in dists]
        best = min(best, min((ms, (wpb, d)) for ms, d in zip(row, dists)))
        print("wpb=%-3d               " % wpb + "".join("%-11.4f" % x for x in row))
        sys.stdout.flush()
    print("\nbest: wpb=%d dist=%d  %.4f ms; by rule / best = %.3f" % (best[1][0], best[1][1], best[0], rule / best[0]))


def sweep_core(w, args):
    """Aggregation time against the dense-core size (best of a few wpb x dist), with the plan's entry counts."""
    import ctypes as C
    time_setting(w, 16, 0, 0, 4 * args.iters, core_rows=0, gin=args.gin)  # plans built, clocks up
    rule = time_setting(w, 16, 0, 0, args.iters, core_rows=0, gin=args.gin)
    print("everything by rule: %.4f ms   [%s]" % (rule, host.last_agg_kernel()))
    print("\ncore rows | ms (best) | wpb dist | edges in the core | list entries with padding | edges left to the gather kernel")
    best = (1e30, None)
    for K in (-1, 8192, 16384, 24576, 32768, 36864, 40960, 49152, 57344, 61440, 65536, 73728, 81920, 98304):
        if K > w["rows"] // 2:
            continue
        sz = [0] * 5
        if K > 0:
            s5 = (C.c_int64 * 5)()
            host._check(host.lib().mggx_core_layout_device(host._dptr(w["ptr_l"]), host._dptr(w["col_l"]), w["rows"], w["lb"], K, s5, None, None,
                                                           None, None, None, None))
            sz = list(s5)
        row = min((time_setting(w, 16, wpb, d, args.iters, core_rows=K, gin=args.gin), wpb, d)
                  for wpb, d in ((4, 2), (4, 4), (4, 8), (4, 16), (8, 2), (8, 8), (16, 2)))
        best = min(best, (row[0], K))
        print("%9d | %9.4f | %3d %4d | %17d | %25d | %d" % (K, row[0], row[1], row[2], sz[4], sz[2], sz[3] if K > 0 else w["nnz"]))
        sys.stdout.flush()
    print("\nbest: %d rows, %.4f ms; by rule / best = %.3f" % (best[1], best[0], rule / best[0]))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default="share", choices=["share", "whole", "sparse"])
    ap.add_argument("--dim", type=int, default=16)
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--small", action="store_true")
    ap.add_argument("--out", default="")
    ap.add_argument("--mode", default="ps", choices=["ps", "wd", "core", "heldout"], help="ps: the reference's ps x wpb and dist x ps tables; "
                    "wd: wpb x dist at ps 16 with order and dense core by rule; core: dense-core size sweep; heldout: rules and cost "
                    "model against measurement on graph families they were not fitted on")
    ap.add_argument("--only", default="", help="--mode heldout: comma-separated names out of " + ", ".join(HELD_OUT))
    ap.add_argument("--shrink", type=int, default=0, help="--mode heldout: divide nodes and edges by 2^k")
    ap.add_argument("--ld", type=int, default=0, help="row pitch of the tables in floats (default: dim)")
    ap.add_argument("--gin", action="store_true", help="aggregate with the GIN self term")
    ap.add_argument("--compact-remote", action="store_true", help="share: stage the remote rows compactly")
    args = ap.parse_args()
    import torch
    torch.cuda.set_device(0)
    host.init(0)
    host.use_torch_stream()
    if args.mode == "heldout":
        return held_out_table(args)
    w = build_workload(args.workload, args.dim, args.small, args.ld, args.compact_remote)
    print("workload %s: rows=%d nnz=%d dim=%d algorithmic bytes=%d" % (args.workload, w["rows"], w["nnz"], args.dim, w["bytes"]))
    if args.mode == "wd":
        return sweep_wpb_dist(w, args)
    if args.mode == "core":
        return sweep_core(w, args)
    res = {"workload": args.workload, "dim": args.dim, "rows": w["rows"], "nnz": w["nnz"], "bytes": w["bytes"], "ps_wpb": {},
           "dist_ps": {}}
    best = (1e30, None)
    pss, wpbs, dists = [1, 2, 4, 8, 16, 32], [1, 2, 4, 8, 16], [1, 2, 4, 8, 16]
    print("\nms, dist = 1           " + "".join("wpb=%-7d" % x for x in wpbs))
    for ps in pss:
        row = []
        for wpb in wpbs:
            ms = time_setting(w, ps, wpb, 1, args.iters)
            host.release_cached() if False else None
            res["ps_wpb"]["%d,%d" % (ps, wpb)] = ms
            best = min(best, (ms, (ps, wpb, 1)))
            row.append(ms)
        print("ps=%-3d                " % ps + "".join("%-11.4f" % x for x in row))
        sys.stdout.flush()
    print("\nms, wpb = 8            " + "".join("ps=%-8d" % x for x in pss))
    for dist in dists:
        row = []
        for ps in pss:
            ms = time_setting(w, ps, 8, dist, args.iters)
            res["dist_ps"]["%d,%d" % (dist, ps)] = ms
            best = min(best, (ms, (ps, 8, dist)))
            row.append(ms)
        print("dist=%-3d              " % dist + "".join("%-11.4f" % x for x in row))
        sys.stdout.flush()
    ms, (ps, wpb, dist) = best
    res["best"] = {"ps": ps, "wpb": wpb, "dist": dist, "ms": ms, "gbps": w["bytes"] / (ms * 1e-3) / 1e9}
    print("\nbest: ps=%d wpb=%d dist=%d  %.4f ms  %.1f GB/s algorithmic" % (ps, wpb, dist, ms, res["best"]["gbps"]))
    if args.out:
        with open(args.out, "w") as f:
            json.dump(res, f, indent=1)


if __name__ == "__main__":
    main()
