"""Host-only parts of the C++ layer (include/mgg/*.h) that no harness program instantiates: the generic branches of
split_CSR<T> / build_part<T> (T = long, long long) and csr_formatter.h's older loaders, getBandwidth and printMatrix.
A small C++ program is compiled against the public headers and its output compared with the reference's own host code
(oracle/_ref, where present) and with fixtures that code produced (tests/golden/)."""
import json
import os
import subprocess

import numpy as np
import pytest

from oracle import orc

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
GOLDEN = os.path.join(HERE, "golden")


@pytest.fixture(scope="module")
def exe(tmp_path_factory):
    out = str(tmp_path_factory.mktemp("cpp") / "host_layer_check")
    pkg = os.path.join(ROOT, "mgg_osdi23_amd")
    subprocess.run(["g++", "-O1", "-std=c++17", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"),
                    os.path.join(HERE, "cpp", "host_layer_check.cpp"), "-o", out, "-L", pkg, "-lmggx", "-Wl,-rpath," + pkg], check=True)
    return out


def parse(stdout):
    arrays, texts, cur = {}, {}, None
    for line in stdout.splitlines():
        if line.endswith("_text_begin"):
            cur = line[: -len("_text_begin")]
            texts[cur] = ""
        elif line.endswith("_text_end"):
            cur = None
        elif cur is not None:
            texts[cur] += line + "\n"
        elif ": " in line or line.endswith(":"):
            name, _, rest = line.partition(":")
            if " " in name or "," in name:  # build_part's own log line
                continue
            arrays[name] = np.array([float(x) for x in rest.split()], np.float64)
    return arrays, texts


def test_split_and_build_part_for_64_bit_ids(exe, tmp_path):
    """split_CSR<long> / build_part<long> of the header against the reference's int outputs in the fixture (same numbers,
    wider type), against the int instantiation (which goes through the library), and against the reference's own
    split_CSR<long> / build_part<long> where oracle/_ref is built."""
    with open(os.path.join(GOLDEN, "np_arrays.json")) as f:
        gold = json.load(f)
    checked = 0
    for case in gold["small"]:
        ptr, col = case["ptr"], case["col"]
        parts_by_ps = {p["ps"]: p for p in case["parts"]}
        for sp in case["split"]:
            lb, ub = sp["lb"], sp["ub"]
            for ps in (3, 16):
                path = tmp_path / "in.txt"
                path.write_text("%d %d %d %d %d\n%s\n%s\n" % (len(ptr), len(col), lb, ub, ps, " ".join(map(str, ptr)), " ".join(map(str, col))))
                r = subprocess.run([exe, "split", str(path)], capture_output=True, text=True, check=True)
                got, _ = parse(r.stdout)
                for tag in ("long", "longlong", "int"):
                    for k in ("local_ptr", "remote_ptr", "local_col", "remote_col"):
                        assert np.array_equal(got["%s_%s" % (tag, k)], np.array(sp[k], np.float64)), (case["name"], tag, k)
                    for k in ("partPtr", "part2Node", "node2Part"):
                        assert np.array_equal(got["long_" + k], got["%s_%s" % (tag, k)]), (case["name"], tag, k)
                if lb == 0 and ub == len(ptr) - 1:  # the fixture's build_part cases are on the whole CSR = its own local half
                    if not sp["remote_col"]:
                        for k in ("partPtr", "part2Node", "node2Part"):
                            assert np.array_equal(got["long_" + k], np.array(parts_by_ps[ps][k], np.float64)), (case["name"], k)
                if orc.have_ref():
                    ref_s = orc.ref_split_csr_long(ptr, col, lb, ub)
                    for k, a in zip(("local_ptr", "remote_ptr", "local_col", "remote_col"), ref_s):
                        assert np.array_equal(got["long_" + k], a.astype(np.float64)), (case["name"], k)
                    ref_p = orc.ref_build_part_long(ref_s[0], ub - lb, ps)
                    for k, a in zip(("partPtr", "part2Node", "node2Part"), ref_p):
                        assert np.array_equal(got["long_" + k], a.astype(np.float64)), (case["name"], k)
                checked += 1
    assert checked >= 50


def test_older_mtx_loaders_bandwidth_and_print(exe, tmp_path):
    """assemble_csr_matrix, assemble_simetric_csr_matrix, getBandwidth, printMatrix against the fixture the reference's
    csr_formatter.h produced, and live against it where oracle/_ref is built."""
    with open(os.path.join(GOLDEN, "mtx_other.json")) as f:
        gold = json.load(f)
    for case in gold["cases"]:
        path = tmp_path / (case["name"] + ".mtx")
        path.write_text(case["file"])
        r = subprocess.run([exe, "mtx", str(path)], capture_output=True, text=True, check=True)
        got, texts = parse(r.stdout)
        wants = [case]
        if orc.have_ref():
            wants.append({"old": _live(str(path), 0), "sym": _live(str(path), 1)})
        for want in wants:
            for tag in ("old", "sym"):
                w = want[tag]
                assert np.array_equal(got[tag + "_row_ptr"], np.array(w["row_ptr"], np.float64)), (case["name"], tag)
                assert np.array_equal(got[tag + "_col_ind"], np.array(w["col_ind"], np.float64)), (case["name"], tag)
                assert np.allclose(got[tag + "_val"], np.array(w["val"], np.float64), rtol=1e-5, atol=0), (case["name"], tag)
                assert int(got[tag + "_bandwidth"][0]) == w["bandwidth"], (case["name"], tag)
                assert texts[tag] == w["text"], (case["name"], tag)


def _live(path, sym):
    d = orc.ref_mtx_load_other(path, sym)
    return {"row_ptr": d["row_ptr"].tolist(), "col_ind": d["col_ind"].tolist(), "val": d["val"].tolist(), "bandwidth": d["bandwidth"],
            "text": d["text"]}
