"""CPU tests of the integer/host part of the path: range partition, local/remote split, neighbor-partition arrays,
graph files.  Three implementations are compared bit for bit on every case:
  golden   arrays produced by the reference's own split_CSR/build_part (tests/golden/np_arrays.json)
  oracle   the C restatement (oracle/mgg_oracle.c)
  library  libmggx's host functions (the product)
and, where oracle/_ref was built in this container, the reference's code is called live as well.
"""
import hashlib
import json
import os

import numpy as np
import pytest

from mgg_osdi23_amd import host
from oracle import orc

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "np_arrays.json")
needs_ref = pytest.mark.skipif(not orc.have_ref(), reason="oracle/_ref not built (reference tree absent)")


@pytest.fixture(scope="module")
def golden():
    with open(GOLDEN) as f:
        return json.load(f)


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a, dtype=np.int32).tobytes()).hexdigest()


def same(a, b):
    a, b = np.asarray(a, np.int32), np.asarray(b, np.int32)
    return a.shape == b.shape and np.array_equal(a, b)


def random_csr(rng, n, avg_deg, empty_frac=0.0, hub=0):
    deg = rng.poisson(avg_deg, n)
    deg[rng.random(n) < empty_frac] = 0
    if hub:
        deg[rng.integers(0, n)] = hub
    ptr = np.zeros(n + 1, np.int32)
    ptr[1:] = np.cumsum(deg)
    col = rng.integers(0, n, int(ptr[-1])).astype(np.int32)
    return ptr, col


# --------------------------------------------------------------------------- golden vectors
def test_split_csr_matches_reference_golden(golden):
    for case in golden["small"]:
        ptr, col = np.array(case["ptr"], np.int32), np.array(case["col"], np.int32)
        for rec in case["split"]:
            want = [rec["local_ptr"], rec["remote_ptr"], rec["local_col"], rec["remote_col"]]
            for impl in (orc.split_csr, host.split_CSR):
                got = impl(ptr, col, rec["lb"], rec["ub"])
                for g, w in zip(got, want):
                    assert same(g, w), (case["name"], rec["lb"], rec["ub"], impl.__module__)


def test_build_part_matches_reference_golden(golden):
    for case in golden["small"]:
        ptr = np.array(case["ptr"], np.int32)
        n = len(ptr) - 1
        for rec in case["parts"]:
            want = [rec["partPtr"], rec["part2Node"], rec["node2Part"]]
            for impl in (orc.build_part, host.build_part):
                got = impl(ptr, n, rec["ps"])
                for g, w, name in zip(got, want, ("partPtr", "part2Node", "node2Part")):
                    assert same(g, w), (case["name"], rec["ps"], name, impl.__module__)


@pytest.mark.parametrize("which", [0, 1])
def test_large_case_digests(golden, which):
    """4096-node cases as SHA-256 digests of every array the reference's split_CSR / build_part produced: a numpy-generated
    graph, and the first benchmark configuration's own graph (Erdos-Renyi, average degree 16, seed 0, nGPU = 1 and 8)."""
    big = golden["large"][which]
    if big.get("generator") == "gen_er":
        ptr, col = host.gen_er(big["num_nodes"], big["avg_deg"], seed=big["seed"])
    else:
        rng = np.random.default_rng(big["seed"])
        ptr, col = random_csr(rng, 4096, big["avg_deg"])
    assert sha(ptr) == big["ptr"]["sha256"] and sha(col) == big["col"]["sha256"], "fixture input regenerated differently"
    for rec in big["split"]:
        for impl in (orc.split_csr, host.split_CSR):
            lp, rp, lc, rc = impl(ptr, col, rec["lb"], rec["ub"])
            for got, key in ((lp, "local_ptr"), (rp, "remote_ptr"), (lc, "local_col"), (rc, "remote_col")):
                assert sha(got) == rec[key]["sha256"] and got[:64].tolist() == rec[key]["head"], key
            for prec in rec["parts"]:
                for bp in (orc.build_part, host.build_part):
                    for side, indptr in (("local", lp), ("remote", rp)):
                        got3 = bp(indptr, rec["ub"] - rec["lb"], prec["ps"])
                        for g, w in zip(got3, prec[side]):
                            assert g.size == w["n"] and sha(g) == w["sha256"] and g[-64:].tolist() == w["tail"]


def test_sag_ref_golden(golden):
    rec = golden["sag_ref"]
    x = np.frombuffer(bytes.fromhex(rec["x_hex"]), np.float32).reshape(rec["shape"])
    y = np.frombuffer(bytes.fromhex(rec["y_hex"]), np.float32).reshape(rec["shape"])
    got = orc.sag_ref(x, np.array(rec["ptr"], np.int32), np.array(rec["col"], np.int32))
    assert np.array_equal(got, y)  # same serial order -> bit-exact


# --------------------------------------------------------------------------- live reference (this container only)
@needs_ref
@pytest.mark.parametrize("seed", range(6))
def test_against_live_reference(seed):
    rng = np.random.default_rng(seed)
    n = int(rng.integers(1, 400))
    ptr, col = random_csr(rng, n, float(rng.uniform(0.5, 12)), float(rng.uniform(0, 0.5)), hub=int(rng.integers(0, 300)))
    for num_gpus in (1, 2, 5):
        for pe in range(num_gpus):
            npp, lb, ub = orc.range_partition(n, num_gpus, pe)
            if ub < lb:
                continue
            want = orc.ref_split_csr(ptr, col, lb, ub)
            for impl in (orc.split_csr, host.split_CSR):
                assert all(same(g, w) for g, w in zip(impl(ptr, col, lb, ub), want))
            for ps in (1, 3, 16, 1 << 20):
                for indptr in (want[0], want[1]):
                    w3 = orc.ref_build_part(indptr, ub - lb, ps)
                    for impl in (orc.build_part, host.build_part):
                        assert all(same(g, w) for g, w in zip(impl(indptr, ub - lb, ps), w3)), (seed, num_gpus, pe, ps)
    x = rng.standard_normal((n, 3)).astype(np.float32)
    assert np.array_equal(orc.sag_ref(x, ptr, col), orc.ref_sag_ref(x, ptr, col))


# --------------------------------------------------------------------------- invariants (hold for any input)
@pytest.mark.parametrize("seed", range(4))
def test_split_and_part_invariants(seed):
    rng = np.random.default_rng(100 + seed)
    n = 500
    ptr, col = random_csr(rng, n, 9.0, 0.2, hub=700)
    npp, lb, ub = host.range_partition(n, 4, seed % 4)
    lp, rp, lc, rc = host.split_CSR(ptr, col, lb, ub)
    # per-row counts add up; merging local and remote in order gives back the row
    assert np.array_equal(np.diff(lp) + np.diff(rp), np.diff(ptr[lb:ub + 1]))
    assert np.all((lc >= lb) & (lc < ub)) and np.all((rc < lb) | (rc >= ub))
    for r in range(ub - lb):
        row = col[ptr[lb + r]:ptr[lb + r + 1]]
        assert np.array_equal(row[(row >= lb) & (row < ub)], lc[lp[r]:lp[r + 1]])
        assert np.array_equal(row[(row < lb) | (row >= ub)], rc[rp[r]:rp[r + 1]])
    for ps in (1, 4, 16):
        pp, p2n, n2p = host.build_part(lp, ub - lb, ps, compat=False)
        deg = np.diff(lp)
        assert len(p2n) == int(np.sum((deg + ps - 1) // ps))
        assert np.all(np.diff(p2n) >= 0) and np.all(np.diff(pp) > 0) and pp[-1] == lp[-1]
        assert np.all(np.diff(pp) <= ps)
        assert np.array_equal(n2p[:-1], np.concatenate([[0], np.cumsum((deg + ps - 1) // ps)])) and n2p[-1] == n2p[-2]
        # every partition stays inside its row
        assert np.all(pp[:-1] >= lp[p2n]) and np.all(pp[1:] <= lp[p2n + 1])


def test_build_part_terminal_entry_quirk():
    """The reference writes partPtr[numParts] only while visiting the last node: it stays 0 when that node is
    isolated.  compat=True reproduces it, compat=False writes the real end."""
    ptr = np.array([0, 3, 3, 8, 8], np.int32)
    pp, p2n, n2p = host.build_part(ptr, 4, 2, compat=True)
    assert pp.tolist() == [0, 2, 3, 5, 7, 0] and p2n.tolist() == [0, 0, 2, 2, 2] and n2p.tolist() == [0, 2, 2, 5, 5, 5]
    assert host.build_part(ptr, 4, 2, compat=False)[0].tolist() == [0, 2, 3, 5, 7, 8]
    assert orc.build_part(ptr, 4, 2)[0].tolist() == [0, 2, 3, 5, 7, 0]


def test_range_partition_closed_form():
    for V in (0, 1, 7, 8, 9, 4096, 233000, 4194304):
        for n in (1, 2, 3, 8):
            covered = 0
            for pe in range(n):
                npp, lb, ub = host.range_partition(V, n, pe)
                assert (npp, lb, ub) == orc.range_partition(V, n, pe)
                assert npp == -(-V // n) and lb == npp * pe and ub == min(lb + npp, V)
                covered += max(0, ub - lb)
            assert covered == V


def test_bad_arguments_are_reported_not_fatal():
    with pytest.raises(host.MggxError):
        host.range_partition(10, 0, 0)
    with pytest.raises(host.MggxError):
        host.build_part(np.array([0, 1], np.int32), 1, 0)
    with pytest.raises(host.MggxError):
        host.split_CSR(np.array([0, 2, 1], np.int32), np.array([0, 0], np.int32), 0, 2)  # decreasing row pointer


# --------------------------------------------------------------------------- graph files
def test_binary_graph_round_trip(tmp_path):
    rng = np.random.default_rng(3)
    ptr, col = random_csr(rng, 300, 6.0, 0.1)
    w = rng.integers(1, 100, len(col)).astype(np.int32)
    files = [str(tmp_path / n) for n in ("g_beg_pos.bin", "g_csr.bin", "g_weight.bin")]
    host.graph_write(*files, ptr, col, w)
    # on-disk layout of the reference's format: int64, int64, int32
    assert os.path.getsize(files[0]) == 8 * (len(ptr)) and os.path.getsize(files[1]) == 8 * len(col)
    assert os.path.getsize(files[2]) == 4 * len(col)
    assert np.array_equal(np.fromfile(files[0], np.int64), ptr) and np.array_equal(np.fromfile(files[1], np.int64), col)
    for loader in (host.graph_read, orc.graph_load) + ((orc.ref_graph_load,) if orc.have_ref() else ()):
        b, c, ww = loader(*files)
        assert same(b, ptr) and same(c, col) and same(ww, w), loader
    with pytest.raises(host.MggxError):
        host.graph_read(str(tmp_path / "missing.bin"), files[1], files[2])
    with open(files[1], "ab") as f:
        f.write(b"\0" * 8)  # csr file no longer matches the edge count
    with pytest.raises(host.MggxError):
        host.graph_read(*files)


def test_mtx_loader(tmp_path):
    p = tmp_path / "g.mtx"
    p.write_text("%%MatrixMarket matrix coordinate real general\n% comment\n5 5 7\n1 2 1.0\n1 5 1.0\n2 1 0.5\n4 4 1\n"
                 "4 1 2\n5 3 1\n5 2 1e0\n")
    want_ptr, want_col = [0, 2, 3, 3, 5, 7], [1, 4, 0, 3, 0, 2, 1]
    for loader in (host.mtx_read, orc.mtx_load) + ((orc.ref_mtx_load,) if orc.have_ref() else ()):
        rp, ci = loader(str(p))
        assert rp.tolist() == want_ptr and ci.tolist() == want_col, loader
    with pytest.raises(host.MggxError):
        host.mtx_read(str(tmp_path / "none.mtx"))


def test_edgelist_to_bin_converter(tmp_path):
    """.mtx / 0-based edge list -> binary triple, read back by all loaders; file order is kept inside a row."""
    mtx = tmp_path / "g.mtx"
    mtx.write_text("%%MatrixMarket matrix coordinate pattern general\n6 6 7\n3 1\n1 4 1.0\n3 6\n1 2\n6 6\n3 2\n5 1\n")
    V, E = host.edgelist_to_bin(str(mtx), str(tmp_path / "g"), is_mtx=True)
    assert (V, E) == (6, 7)
    want_ptr, want_col = [0, 2, 2, 5, 5, 6, 7], [3, 1, 0, 5, 1, 0, 5]
    files = [str(tmp_path / ("g" + s)) for s in ("_beg_pos.bin", "_csr.bin", "_weight.bin")]
    for loader in (host.graph_read, orc.graph_load) + ((orc.ref_graph_load,) if orc.have_ref() else ()):
        b, c, w = loader(*files)
        assert b.tolist() == want_ptr and c.tolist() == want_col and w.tolist() == [1] * 7
    el = tmp_path / "g0.txt"
    el.write_text("2 0\n0 3\n2 5\n0 1\n5 5\n2 1\n4 0\n")  # the same graph, already 0-based (dataset/0_to_base_zero.py output)
    assert host.edgelist_to_bin(str(el), str(tmp_path / "h")) == (6, 7)
    b, c, _ = host.graph_read(*[str(tmp_path / ("h" + s)) for s in ("_beg_pos.bin", "_csr.bin", "_weight.bin")])
    assert b.tolist() == want_ptr and c.tolist() == want_col
    with pytest.raises(host.MggxError):
        host.edgelist_to_bin(str(tmp_path / "missing.txt"), str(tmp_path / "x"))
    # a size line beyond int32 node ids is an error code, not a crash or a truncated count
    huge = tmp_path / "huge.mtx"
    huge.write_text("%%MatrixMarket matrix coordinate pattern general\n4000000000 4000000000 1\n1 2\n")
    with pytest.raises(host.MggxError, match="int32"):
        host.edgelist_to_bin(str(huge), str(tmp_path / "y"), is_mtx=True)


# --------------------------------------------------------------------------- generators
def test_generators_are_deterministic_and_well_formed():
    for gen in (lambda: host.gen_er(2000, 10.0, seed=4), lambda: host.gen_rmat(11, 1800, 30000, seed=4, threads=3),
                lambda: host.gen_rmat(11, 1800, 30000, seed=4, scramble=True, threads=2)):
        ptr, col = gen()
        ptr2, col2 = gen()
        assert np.array_equal(ptr, ptr2) and np.array_equal(col, col2)
        n = len(ptr) - 1
        assert ptr[0] == 0 and ptr[-1] == len(col) and np.all(np.diff(ptr) >= 1)  # self loop in every row
        for r in range(0, n, 97):
            row = col[ptr[r]:ptr[r + 1]]
            assert np.all(np.diff(row) > 0) and r in row  # sorted, duplicate-free, has its self loop
        # symmetric
        import scipy.sparse as sp
        A = sp.csr_matrix((np.ones(len(col), np.int8), col, ptr), shape=(n, n))
        assert (A != A.T).nnz == 0
    # thread count does not change the graph; a share is the matching row slice of the whole graph
    a = host.gen_rmat(11, 1800, 30000, seed=9, threads=1)
    b = host.gen_rmat(11, 1800, 30000, seed=9, threads=4)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
    sp_, sc_ = host.gen_rmat(11, 1800, 30000, seed=9, row_lo=450, row_hi=900)
    assert np.array_equal(sc_, a[1][a[0][450]:a[0][900]]) and np.array_equal(sp_, a[0][450:901] - a[0][450])
    x = host.fill_normal((200000,), seed=1)
    assert abs(float(x.mean())) < 0.01 and abs(float(x.std()) - 1.0) < 0.01
    u = host.fill_uniform((100000,), -1.0, 1.0, seed=2)
    assert u.min() >= -1.0 and u.max() < 1.0 and abs(float(u.mean())) < 0.01


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_compact_remote_staging_order(seed):
    """The distinct remote ids, most referenced first (ties by ascending id), and the rewritten column array:
    checked against numpy's unique/argsort and by the round trip fetch_ids[compact] == remote_col."""
    rng = np.random.default_rng(seed)
    V = 5000
    ptr, col = host.gen_rmat(13, V, 60_000, seed=seed, scramble=bool(seed % 2))
    npp, lb, ub = host.range_partition(V, 4, seed % 4)
    _, rp, _, rc = host.split_CSR(ptr, col, lb, ub)
    compact, ids = host.compact_remote(rc)
    assert np.array_equal(ids[compact], rc)
    uniq, cnt = np.unique(rc, return_counts=True)
    order = np.argsort(-cnt, kind="stable")       # ties keep ascending id
    assert np.array_equal(ids, uniq[order])
    assert not np.any((ids >= lb) & (ids < ub))   # remote ids only
    # degenerate inputs
    c0, i0 = host.compact_remote(np.zeros(0, np.int32))
    assert len(c0) == 0 and len(i0) == 0
    c1, i1 = host.compact_remote(np.array([7, 7, 7], np.int32))
    assert c1.tolist() == [0, 0, 0] and i1.tolist() == [7]
    with pytest.raises(host.MggxError):
        host.compact_remote(np.array([3, -1], np.int32))


def _first_from(mask, k):
    """The lowest set bit of a 16-bit mask when looking from bit k upwards, cyclically; -1 if the mask is empty."""
    if mask == 0:
        return -1
    m = ((mask >> k) | (mask << (16 - k))) & 0xFFFF
    return ((m & -m).bit_length() - 1 + k) & 15


def _bank_order(lists, P, tile):
    """16 lists of tile offsets in edge order (the lanes of a group) and the block's length P -> [P][16] as the library
    stores the block (see test_dense_core_layout)."""
    if P > 256:   # longer than the library re-orders: edge order, padding on the first zero column
        return np.array([[e[p] if p < len(e) else tile for e in lists] for p in range(P)], np.int64)
    q = [[[x for x in e if x % 16 == r] for r in range(16)] for e in lists]
    left = [len(e) for e in lists]
    out = np.zeros((P, 16), np.int64)
    for p in range(P):
        used, r = 0, [-1] * 16
        for first in (True, False):
            for i in range(16):
                slack = P - p - left[i]
                if left[i] == 0 or (slack == 0) != first:
                    continue
                have = sum(1 << k for k in range(16) if q[i][k])
                rr = _first_from(have & ~used, (i + p) % 16)
                if rr < 0 and slack == 0:
                    rr = _first_from(have, (i + p) % 16)
                r[i] = rr
                if rr >= 0:
                    used |= 1 << rr
        free = [k for k in range(16) if not (used >> k) & 1]
        npad = 0
        for i in range(16):
            if r[i] >= 0:
                out[p, i] = q[i][r[i]].pop(0)
                left[i] -= 1
            else:
                out[p, i] = tile + (free[npad] if npad < len(free) else npad % 16)
                npad += 1
    return out


@pytest.mark.parametrize("lb,core_rows,tile", [(0, 1024, 256), (0, 1700, 256), (300, 512, 64)])
def test_dense_core_layout(lb, core_rows, tile):
    """The core x core block as index lists plus the remaining CSR, against numpy: ranks by degree (ties by id), every
    core edge exactly once in the list of its (slice, tile) block at the right tile offset, the block in bank order (the
    16 lanes of a group placed together, position by position: lanes without padding left to spend first, then the
    others, each in lane order; a lane takes its first remaining entry, looking from residue (lane + p) mod 16 upwards,
    whose residue mod 16 is not taken at this position, else spends a padding slot, else repeats a residue; padding
    slots point at the zero columns tile + r for the residues r still free, in turn), everything else left in the CSR
    in its order."""
    V = 4000
    ptr, col = host.gen_rmat(12, V, 120_000, seed=4)
    col = (col + lb).astype(np.int32)  # a share whose rows start at lb: ids are global
    L = host.core_layout(ptr, col, lb, core_rows, tile)
    core = L["core"]
    assert core == core_rows // 512 * 512 and L["ntiles"] == core // tile
    deg = np.diff(ptr)
    order = np.argsort(-deg, kind="stable")[:core]
    assert np.array_equal(L["order"], order)
    rank = np.full(V, -1, np.int32)
    rank[order] = np.arange(core)
    assert np.array_equal(L["rank"], rank)
    rows = np.repeat(np.arange(V), deg)
    in_core = (rank[rows] >= 0) & (rank[col - lb] >= 0)
    assert L["core_nnz"] == int(in_core.sum())
    # the remainder
    keep = ~in_core
    assert np.array_equal(L["rem_col"], col[keep])
    rp = np.zeros(V + 1, np.int64)
    np.add.at(rp, rows[keep] + 1, 1)
    assert np.array_equal(L["rem_ptr"], np.cumsum(rp))
    # the lists
    ntiles, off, idx = L["ntiles"], L["blk_off"].astype(np.int64), L["idx"]
    assert len(off) == core // 64 * ntiles + 1 and len(idx) == off[-1] * 256 and np.all(np.diff(off) >= 0)
    seen = 0
    for grp in (list(range(0, core // 16, 5)) + [core // 16 - 1]):   # groups of 16 lanes: ranks 16 grp .. 16 grp + 15
        nbs = []
        for i in range(16 * grp, 16 * grp + 16):
            v = order[i]
            nb = rank[col[ptr[v]:ptr[v + 1]] - lb]
            nbs.append(nb[nb >= 0])
        g, l0 = grp // 4, 16 * (grp % 4)
        for t in range(ntiles):
            want = [[int(x) for x in nb[nb // tile == t] % tile] for nb in nbs]
            b0, b1 = off[g * ntiles + t], off[g * ntiles + t + 1]
            got = idx[b0 * 256:b1 * 256].reshape(-1, 64, 4).transpose(0, 2, 1).reshape(-1, 64)[:, l0:l0 + 16]   # [position][lane]
            assert max(len(w) for w in want) <= len(got)
            assert np.array_equal(got, _bank_order(want, len(got), tile))
            seen += sum(len(w) for w in want)
    assert seen > 0
    # every block is as long as its longest list, rounded up to 4
    cnt = np.zeros((core, ntiles), np.int64)
    rc, cc = rank[rows[in_core]], rank[col[in_core] - lb]
    np.add.at(cnt, (rc, cc // tile), 1)
    width = (cnt.reshape(core // 64, 64, ntiles).max(axis=1) + 3) // 4
    assert np.array_equal(np.diff(off), width.reshape(-1))


def test_dense_core_layout_rejects_what_it_cannot_hold():
    ptr, col = host.gen_rmat(10, 900, 9000, seed=1)
    with pytest.raises(host.MggxError):
        host.core_layout(ptr, col, 0, 400, 256)        # less than one 512-row unit
    with pytest.raises(host.MggxError):
        host.core_layout(ptr, col, 5, 512, 256)        # ids below lb
    with pytest.raises(host.MggxError):
        host.core_layout(ptr, col, 0, 512, 100)        # tile not a multiple of 64
