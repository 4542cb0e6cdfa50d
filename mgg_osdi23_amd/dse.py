"""Design-space exploration of (ps, wpb, dist) for the aggregation kernel on one GPU.

Counterpart of the reference's 5_MGG_DSE_*.py / bench_MGG_DSE_dist_ps.py / bench_MGG_DSE_dist_wpb.py, which sweep
dist x ps (wpb fixed) and dist x wpb (ps fixed) and tabulate the aggregation time.  Here the sweep runs in one
process on synthetic graphs of the benchmark shapes:

    python -m mgg_osdi23_amd.dse --workload share [--dim 16] [--iters 20] [--out table.json]
    python -m mgg_osdi23_amd.dse --workload whole --dim 16

Prints ps x wpb (dist = 1) and dist x ps (wpb = 8) tables in ms, GB/s of algorithmic traffic, and the best setting.
"""
from __future__ import annotations

import argparse
import json
import sys

import numpy as np

from . import host


def build_workload(name: str, dim: int, small: bool):
    import torch
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
    x = host.fill_normal((rows_tbl, dim), seed=11)
    dev = "cuda"
    t = lambda a: torch.from_numpy(a).to(dev) if len(a) else torch.zeros(1, dtype=torch.int32, device=dev)
    w = dict(lb=lb, ub=ub, npp=npp, nnz=len(lc) + len(rc), rows=ub - lb, dim=dim,
             xr=torch.from_numpy(x).to(dev), xl=torch.from_numpy(np.ascontiguousarray(x[lb:ub])).to(dev),
             ptr_l=t(lp), col_l=t(lc), ptr_r=t(rp), col_r=t(rc))
    w["out"] = torch.empty(ub - lb, dim, device=dev)
    w["bytes"] = w["nnz"] * (4 + dim * 4) + w["rows"] * dim * 4 + (w["rows"] + 1) * 4 * (2 if len(rc) else 1)
    return w


def time_setting(w, ps, wpb, dist, iters):
    import torch

    def call():
        host.mgg_SAG_np_div(w["out"], w["xl"], w["ptr_l"], w["col_l"], w["ptr_r"], w["col_r"], w["lb"], w["ub"], w["dim"],
                            w["npp"], 0, ps, wpb, dist, input_remote=w["xr"])

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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default="share", choices=["share", "whole", "sparse"])
    ap.add_argument("--dim", type=int, default=16)
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--small", action="store_true")
    ap.add_argument("--out", default="")
    args = ap.parse_args()
    import torch
    torch.cuda.set_device(0)
    host.init(0)
    host.use_torch_stream()
    w = build_workload(args.workload, args.dim, args.small)
    print("workload %s: rows=%d nnz=%d dim=%d algorithmic bytes=%d" % (args.workload, w["rows"], w["nnz"], args.dim, w["bytes"]))
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
