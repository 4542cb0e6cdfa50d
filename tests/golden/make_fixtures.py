#!/usr/bin/env python3
"""Writes tests/golden/np_arrays.json from the REFERENCE's own host code.

The arrays come from oracle/_ref/libmgg_ref.so, i.e. from split_CSR<int> and
build_part<int> compiled out of the reference's neighbor_utils.cuh (see
oracle/build_ref.sh).  Run it where the reference tree is mounted:

    make -C oracle && python tests/golden/make_fixtures.py

Inputs are built here with numpy's PCG64 (seeded) or written out by hand, and
are stored in the fixture next to the outputs, so reading the fixture needs
neither the reference nor a generator.  Large cases store SHA-256 digests and
the first/last 64 entries of each array instead of the whole array.
"""
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
from oracle import orc  # noqa: E402


def digest(a):
    a = np.ascontiguousarray(a, dtype=np.int32)
    return {"n": int(a.size), "sha256": hashlib.sha256(a.tobytes()).hexdigest(), "head": a[:64].tolist(),
            "tail": a[-64:].tolist()}


def random_csr(rng, n, avg_deg, empty_frac=0.0, hub=0):
    deg = rng.poisson(avg_deg, n)
    deg[rng.random(n) < empty_frac] = 0
    if hub:
        deg[rng.integers(0, n)] = hub
    ptr = np.zeros(n + 1, np.int32)
    ptr[1:] = np.cumsum(deg)
    col = rng.integers(0, n, int(ptr[-1])).astype(np.int32)
    return ptr, col


def mtx_other():
    """tests/golden/mtx_other.json: assemble_csr_matrix, assemble_simetric_csr_matrix, getBandwidth and printMatrix of the
    reference's csr_formatter.h on small hand-written and seeded files (the file text is stored with the outputs)."""
    import tempfile
    files = [
        ("hand_sorted", "%%MatrixMarket matrix coordinate real general\n% a comment\n4 4 7\n1 1 1.5\n1 3 2\n2 2 3\n3 1 4\n3 4 5.25\n4 2 6\n4 4 7\n"),
        ("hand_gap_rows", "5 5 6\n1 2 1\n1 5 2\n3 1 3\n3 3 4\n5 4 5\n5 5 6\n"),
        ("hand_lower_triangle", "%%MatrixMarket matrix coordinate real symmetric\n4 4 6\n1 1 10\n2 1 20\n3 2 30\n4 1 40\n4 3 50\n4 4 60\n"),
    ]
    rng = np.random.default_rng(99)
    n = 9
    ent = sorted({(int(r), int(c)) for r, c in zip(rng.integers(1, n + 1, 30), rng.integers(1, n + 1, 30))})
    files.append(("seeded_9", "%d %d %d\n" % (n, n, len(ent)) + "".join("%d %d %g\n" % (r, c, 0.5 * (i + 1)) for i, (r, c) in enumerate(ent))))
    cases = []
    with tempfile.TemporaryDirectory() as d:
        for name, text in files:
            path = os.path.join(d, name + ".mtx")
            with open(path, "w") as f:
                f.write(text)
            rec = {"name": name, "file": text}
            for tag, sym in (("old", 0), ("sym", 1)):
                r = orc.ref_mtx_load_other(path, sym)
                rec[tag] = {"row_ptr": r["row_ptr"].tolist(), "col_ind": r["col_ind"].tolist(), "val": r["val"].tolist(),
                            "bandwidth": r["bandwidth"], "text": r["text"]}
            cases.append(rec)
    with open(os.path.join(HERE, "mtx_other.json"), "w") as f:
        json.dump({"note": "outputs of the reference's assemble_csr_matrix / assemble_simetric_csr_matrix / getBandwidth / printMatrix "
                           "(csr_formatter.h:31-109, 146-183); printMatrix on the result with row_ptr[0] = 1", "cases": cases}, f, indent=1)


def main():
    assert orc.have_ref(), "oracle/_ref/libmgg_ref.so is missing: run `make -C oracle` with the reference mounted"
    cases = []
    hand = [
        ("survey_probe", [0, 3, 3, 8, 9], [0, 1, 3, 0, 1, 2, 3, 2, 1]),
        ("last_row_empty", [0, 3, 3, 8, 8], [0, 1, 3, 0, 1, 2, 3, 2]),
        ("first_rows_empty", [0, 0, 0, 4, 6], [3, 2, 1, 0, 0, 3]),
        ("all_empty", [0, 0, 0, 0], []),
        ("single_row", [0, 5], [0, 0, 0, 0, 0]),
        ("degree_multiple_of_ps", [0, 4, 8, 16], [0, 1, 2, 0, 1, 2, 0, 1, 2, 0, 1, 2, 0, 1, 2, 0]),
    ]
    for name, ptr, col in hand:
        cases.append((name, np.array(ptr, np.int32), np.array(col, np.int32)))
    rng = np.random.default_rng(20231)
    cases.append(("random_64", *random_csr(rng, 64, 5.0, 0.2)))
    cases.append(("random_200_hub", *random_csr(rng, 200, 3.0, 0.3, hub=150)))
    cases.append(("random_256_dense", *random_csr(rng, 256, 20.0)))

    out = {"note": "outputs of the reference's split_CSR<int> / build_part<int> (neighbor_utils.cuh:381-460)", "small": [],
           "large": []}
    for name, ptr, col in cases:
        n = len(ptr) - 1
        entry = {"name": name, "ptr": ptr.tolist(), "col": col.tolist(), "split": [], "parts": []}
        for num_gpus in (1, 2, 3):
            for pe in range(num_gpus):
                npp = (n + num_gpus - 1) // num_gpus
                lb = npp * pe
                ub = min(lb + npp, n)
                if ub < lb:
                    continue
                lp, rp, lc, rc = orc.ref_split_csr(ptr, col, lb, ub)
                entry["split"].append({"lb": lb, "ub": ub, "local_ptr": lp.tolist(), "remote_ptr": rp.tolist(),
                                       "local_col": lc.tolist(), "remote_col": rc.tolist()})
        for ps in (1, 2, 3, 4, 16, 65536):
            pp, p2n, n2p = orc.ref_build_part(ptr, n, ps)
            entry["parts"].append({"ps": ps, "partPtr": pp.tolist(), "part2Node": p2n.tolist(), "node2Part": n2p.tolist()})
        out["small"].append(entry)

    # a 4096-node graph in the style of the first benchmark configuration (numpy-generated so the fixture does not
    # depend on this repository's own generator): digests only
    rng = np.random.default_rng(4096)
    ptr, col = random_csr(rng, 4096, 17.0)
    big = {"name": "random_4096", "seed": 4096, "avg_deg": 17.0, "ptr": digest(ptr), "col": digest(col), "split": [],
           "parts": []}
    for num_gpus, pe in ((1, 0), (8, 0), (8, 5)):
        npp = (4096 + num_gpus - 1) // num_gpus
        lb, ub = npp * pe, min(npp * pe + npp, 4096)
        lp, rp, lc, rc = orc.ref_split_csr(ptr, col, lb, ub)
        rec = {"lb": lb, "ub": ub, "local_ptr": digest(lp), "remote_ptr": digest(rp), "local_col": digest(lc),
               "remote_col": digest(rc), "parts": []}
        for ps in (1, 16, 32):
            pl = orc.ref_build_part(lp, ub - lb, ps)
            pr = orc.ref_build_part(rp, ub - lb, ps)
            rec["parts"].append({"ps": ps, "local": [digest(x) for x in pl], "remote": [digest(x) for x in pr]})
        big["split"].append(rec)
    out["large"].append(big)

    # the graph of the first benchmark configuration itself: Erdos-Renyi, 4096 nodes, average degree 16, self loops,
    # seed 0, from the library's generator (its digests pin the generator too); nGPU = 1 and rank 0 of 8, ps = 16
    from mgg_osdi23_amd import host
    ptr, col = host.gen_er(4096, 16.0, seed=0)
    cfg = {"name": "config1_er_4096", "generator": "gen_er", "num_nodes": 4096, "avg_deg": 16.0, "seed": 0, "ptr": digest(ptr),
           "col": digest(col), "split": [], "parts": []}
    for num_gpus, pe in ((1, 0), (8, 0)):
        npp = (4096 + num_gpus - 1) // num_gpus
        lb, ub = npp * pe, min(npp * pe + npp, 4096)
        lp, rp, lc, rc = orc.ref_split_csr(ptr, col, lb, ub)
        rec = {"lb": lb, "ub": ub, "local_ptr": digest(lp), "remote_ptr": digest(rp), "local_col": digest(lc),
               "remote_col": digest(rc), "parts": []}
        pl = orc.ref_build_part(lp, ub - lb, 16)
        pr = orc.ref_build_part(rp, ub - lb, 16)
        rec["parts"].append({"ps": 16, "local": [digest(x) for x in pl], "remote": [digest(x) for x in pr]})
        cfg["split"].append(rec)
    out["large"].append(cfg)

    # SAG_ref (utils.cuh:71-86) on a small seeded case, floats stored exactly as hex
    rng = np.random.default_rng(7)
    ptr, col = random_csr(rng, 40, 4.0, 0.1)
    x = rng.standard_normal((40, 5)).astype(np.float32)
    y = orc.ref_sag_ref(x, ptr, col)
    out["sag_ref"] = {"ptr": ptr.tolist(), "col": col.tolist(), "x_hex": x.tobytes().hex(), "y_hex": y.tobytes().hex(),
                      "shape": [40, 5]}

    mtx_other()

    with open(os.path.join(HERE, "np_arrays.json"), "w") as f:
        json.dump(out, f, separators=(",", ":"))
    print("wrote", os.path.join(HERE, "np_arrays.json"))


if __name__ == "__main__":
    main()
