"""GPU parity tests: the HIP path, called through the C ABI, against the CPU oracle.

Tolerances (fp32): |gpu - oracle_f64| <= 1e-5 * sum|terms| per element; closed
forms (all-ones inputs, one-hot inputs) must be bit-exact.
"""
import numpy as np
import pytest

from oracle import orc
from tests.util import BF16_TOL, FP32_TOL, assert_close_to_oracle, share_of, sym_norm_scale, to_dev

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True, params=["auto", "wide"])
def addressing(request, gpu):
    """Every case runs with both gather addressing schemes (32-bit buffer offsets where they apply, and 64-bit)."""
    gpu.set_gather_addressing(1 if request.param == "wide" else 0)
    yield request.param
    gpu.set_gather_addressing(0)


def run_agg(host, sh, x_local, x_remote, dim, ps, wpb, dist, *, gin=False, eps=0.0, accumulate_into=None,
            ld_in=0, ld_out=0, row_scale_out=None, relu=False):
    import torch
    R = sh["ub"] - sh["lb"]
    ldo = ld_out or dim
    if accumulate_into is not None:
        out = to_dev(accumulate_into)
    else:
        out = torch.full((max(R, 1), ldo), 7.5, dtype=torch.float32, device="cuda")[:R]  # poison: must be overwritten
    d = dict(ptr_l=to_dev(sh["ptr_l"]), col_l=to_dev(sh["col_l"]) if len(sh["col_l"]) else torch.zeros(1, dtype=torch.int32, device="cuda"),
             ptr_r=to_dev(sh["ptr_r"]), col_r=to_dev(sh["col_r"]) if len(sh["col_r"]) else torch.zeros(1, dtype=torch.int32, device="cuda"))
    rs = to_dev(row_scale_out) if row_scale_out is not None else None
    if gin:
        host.mgg_GIN_np_div(out, x_local, d["ptr_l"], d["col_l"], d["ptr_r"], d["col_r"], sh["lb"], sh["ub"], dim,
                            sh["npp"], 0, ps, wpb, dist, eps, input_remote=x_remote, ld_in=ld_in, ld_out=ld_out)
    else:
        host.mgg_SAG_np_div(out, x_local, d["ptr_l"], d["col_l"], d["ptr_r"], d["col_r"], sh["lb"], sh["ub"], dim,
                            sh["npp"], 0, ps, wpb, dist, input_remote=x_remote, accumulate=accumulate_into is not None,
                            ld_in=ld_in, ld_out=ld_out, row_scale_out=rs, relu=relu)
    host.sync()
    return out.cpu().numpy()


def oracle_agg(sh, xl, xr, dim, **kw):
    want = orc.sag_np_div(xl, xr, sh["ptr_l"], sh["col_l"], sh["ptr_r"], sh["col_r"], sh["lb"], sh["ub"], dim, sh["npp"], **kw)
    rows = np.arange(sh["ub"] - sh["lb"], dtype=np.int32)
    kw2 = {k: v for k, v in kw.items() if k in ("flags", "eps", "rs_in", "rs_out")}
    kw2["flags"] = kw2.get("flags", 0) & ~orc.ACCUMULATE
    mag = orc.sag_np_div_rows(rows, xl, xr, sh["ptr_l"], sh["col_l"], sh["ptr_r"], sh["col_r"], sh["lb"], sh["ub"], dim,
                              sh["npp"], abs_sum=True, **kw2)
    return want, mag


@pytest.fixture(scope="module")
def er_graph():
    from mgg_osdi23_amd import host
    return host.gen_er(4096, 16.0, seed=0)


@pytest.fixture(scope="module")
def rmat_graph():
    from mgg_osdi23_amd import host
    V = 6000
    ptr, col = host.gen_rmat(13, V, 220_000, seed=5)
    return V, ptr, col


# --------------------------------------------------------------------------- config 1
@pytest.mark.parametrize("num_gpus,pe", [(1, 0), (8, 0), (8, 3), (8, 7)])
def test_config1_er_sum_aggregation(gpu, er_graph, num_gpus, pe):
    """4096-node Erdos-Renyi graph, avg degree 16, self loops, fp32 dim 16 ~U[-1,1] seed 0, ps=16:
    plain sum and D^-1/2 A D^-1/2 weighting; whole graph and an 8-way share with local/remote tables."""
    ptr, col = er_graph
    V, dim = 4096, 16
    x = gpu.fill_uniform((V, dim), -1.0, 1.0, seed=0)
    sh = share_of(ptr, col, V, num_gpus, pe)
    xl = x[sh["lb"]:sh["ub"]]
    got = run_agg(gpu, sh, to_dev(xl), to_dev(x), dim, 16, 4, 1)
    want, mag = oracle_agg(sh, xl, x, dim)
    assert_close_to_oracle(got, want, mag, FP32_TOL, "plain sum")
    # symmetric normalisation: pre-scaled table, post-scaled rows
    s = sym_norm_scale(ptr)
    xs = (x * s[:, None]).astype(np.float32)
    got = run_agg(gpu, sh, to_dev(xs[sh["lb"]:sh["ub"]]), to_dev(xs), dim, 16, 4, 1, row_scale_out=s[sh["lb"]:sh["ub"]])
    want, mag = oracle_agg(sh, xl, x, dim, rs_in=s, rs_out=s[sh["lb"]:sh["ub"]])
    assert_close_to_oracle(got, want, mag, FP32_TOL, "sym-norm")


# --------------------------------------------------------------------------- closed forms (bit-exact)
@pytest.mark.parametrize("dim", [16, 41, 64])
def test_all_ones_gives_degree_exactly(gpu, rmat_graph, dim):
    V, ptr, col = rmat_graph
    sh = share_of(ptr, col, V, 4, 1)
    ones = np.ones((V, dim), np.float32)
    got = run_agg(gpu, sh, to_dev(ones[sh["lb"]:sh["ub"]]), to_dev(ones), dim, 16, 8, 2)
    deg = (np.diff(sh["ptr_l"]) + np.diff(sh["ptr_r"])).astype(np.float32)
    assert np.array_equal(got, np.repeat(deg[:, None], dim, 1))
    got = run_agg(gpu, sh, to_dev(ones[sh["lb"]:sh["ub"]]), to_dev(ones), dim, 16, 8, 2, gin=True, eps=0.5)
    assert np.array_equal(got, np.repeat((deg + 1.5)[:, None], dim, 1))


def test_one_hot_gives_adjacency_rows_exactly(gpu):
    ptr, col = gpu.gen_rmat(7, 100, 700, seed=11)
    V = 100
    eye = np.zeros((V, 128), np.float32)
    eye[np.arange(V), np.arange(V)] = 1.0
    sh = share_of(ptr, col, V, 2, 1)
    got = run_agg(gpu, sh, to_dev(eye[sh["lb"]:sh["ub"]]), to_dev(eye), 128, 4, 2, 1)
    A = np.zeros((sh["ub"] - sh["lb"], 128), np.float32)
    for r in range(sh["lb"], sh["ub"]):
        for e in range(ptr[r], ptr[r + 1]):
            A[r - sh["lb"], col[e]] += 1.0
    assert np.array_equal(got, A)


# --------------------------------------------------------------------------- knob independence
@pytest.mark.parametrize("ps", [1, 2, 4, 8, 16, 32, 65536])
@pytest.mark.parametrize("wpb,dist", [(1, 1), (2, 4), (4, 1), (8, 1), (8, 16), (16, 2)])
def test_knobs_change_speed_not_result(gpu, rmat_graph, ps, wpb, dist):
    V, ptr, col = rmat_graph
    dim = 16
    x = gpu.fill_normal((V, dim), seed=2)
    sh = share_of(ptr, col, V, 4, 0)  # rank 0 owns the hubs of an unscrambled RMAT graph
    xl = x[sh["lb"]:sh["ub"]]
    got = run_agg(gpu, sh, to_dev(xl), to_dev(x), dim, ps, wpb, dist)
    want, mag = oracle_agg(sh, xl, x, dim)
    assert_close_to_oracle(got, want, mag, FP32_TOL, "ps=%d wpb=%d dist=%d" % (ps, wpb, dist))


@pytest.mark.parametrize("dim", [16, 64])
def test_library_chosen_knobs(gpu, rmat_graph, dim):
    """wpb = 0 / dist = 0 let the library pick the launch geometry; the result obeys the same tolerance."""
    V, ptr, col = rmat_graph
    x = gpu.fill_normal((V, dim), seed=77)
    sh = share_of(ptr, col, V, 2, 0)
    xl = x[sh["lb"]:sh["ub"]]
    got = run_agg(gpu, sh, to_dev(xl), to_dev(x), dim, 16, 0, 0)
    want, mag = oracle_agg(sh, xl, x, dim)
    assert_close_to_oracle(got, want, mag, FP32_TOL, "auto knobs")


@pytest.mark.parametrize("dim,gin", [(16, False), (64, True), (41, False)])
def test_search_of_wpb_and_dist(gpu, rmat_graph, dim, gin):
    """The one-call search over wpb x dist: leaves a correct result in the output, returns a pair from its grid, and
    a later call with wpb = dist = 0 on the same CSR tensors runs with that pair (bit-identical to naming it)."""
    import torch
    V, ptr, col = rmat_graph
    x = gpu.fill_normal((V, dim), seed=78)
    sh = share_of(ptr, col, V, 2, 0)
    xl = np.ascontiguousarray(x[sh["lb"]:sh["ub"]])
    R = sh["ub"] - sh["lb"]
    d = [to_dev(sh[k]) if len(sh[k]) else torch.zeros(1, dtype=torch.int32, device="cuda") for k in ("ptr_l", "col_l", "ptr_r", "col_r")]
    d_xl, d_x = to_dev(xl), to_dev(x)
    out = torch.full((R, dim), 7.5, device="cuda")
    kn, ms = gpu.tune_np_div(out, d_xl, d[0], d[1], d[2], d[3], sh["lb"], sh["ub"], dim, sh["npp"], 16, input_remote=d_x,
                             gin_eps=0.25 if gin else None)
    wpb, dist = kn["wpb"], kn["dist"]
    assert kn["ps"] == 16 and wpb in (4, 8, 16) and dist in (1, 2, 4, 8, 16) and ms > 0 and kn["col_block_rows"] == -1
    kw = dict(flags=orc.GIN, eps=0.25) if gin else {}
    want, mag = oracle_agg(sh, xl, x, dim, **kw)
    assert_close_to_oracle(out.cpu().numpy(), want, mag, FP32_TOL, "result left by the search")
    call = (lambda o, w, t: gpu.mgg_GIN_np_div(o, d_xl, d[0], d[1], d[2], d[3], sh["lb"], sh["ub"], dim, sh["npp"], 0, 16, w, t, 0.25,
                                                input_remote=d_x)) if gin else \
           (lambda o, w, t: gpu.mgg_SAG_np_div(o, d_xl, d[0], d[1], d[2], d[3], sh["lb"], sh["ub"], dim, sh["npp"], 0, 16, w, t,
                                                input_remote=d_x))
    auto, named = torch.empty_like(out), torch.empty_like(out)
    call(auto, 0, 0)
    assert "block=%d" % (64 * wpb) in gpu.last_agg_kernel()
    call(named, wpb, dist)
    gpu.sync()
    assert torch.equal(auto, named)
    with pytest.raises(gpu.MggxError):  # repeated runs would add up
        o = gpu._AggOpts()
        o.flags = gpu.AGG_ACCUMULATE
        import ctypes as C
        gpu._check(gpu.lib().mggx_sag_np_div_tune(gpu._dptr(out), gpu._dptr(d_xl), gpu._dptr(d_x), gpu._dptr(d[0]), gpu._dptr(d[1]),
                                                  gpu._dptr(d[2]), gpu._dptr(d[3]), sh["lb"], sh["ub"], dim, sh["npp"], 16,
                                                  C.byref(o), None, None))


@pytest.mark.parametrize("dim,block_rows,flags", [(16, 100, "plain"), (44, 64, "scale"), (41, 37, "gin"), (8, 300, "acc_relu"),
                                                  (64, 128, "plain"),
                                                  # 2 to 8 blocks: the finishing kernel takes all blocks of a row in one batch
                                                  (16, 3000, "scale"), (12, 2000, "plain"), (41, 1200, "plain"), (16, 1000, "scale"),
                                                  (24, 860, "acc_relu"), (44, 750, "gin")])
def test_column_blocked_order(gpu, rmat_graph, dim, block_rows, flags):
    """The column-blocked partition order (whole graph, rows sorted by neighbor id): same sums as the plain order and
    the oracle, with every epilogue; unsorted rows fall back to the plain order silently."""
    import torch
    V, ptr, col = rmat_graph
    x = gpu.fill_normal((V, dim), seed=91)
    sh = share_of(ptr, col, V, 1, 0)
    d_ptr, d_col = to_dev(ptr), to_dev(col)
    z, zc = torch.zeros(V + 1, dtype=torch.int32, device="cuda"), torch.zeros(1, dtype=torch.int32, device="cuda")
    d_x = to_dev(x)
    s = gpu.fill_uniform((V,), 0.5, 2.0, seed=92)
    base = gpu.fill_normal((V, dim), seed=93)

    def run(blk, ps, wpb, dist):
        out = to_dev(base.copy()) if flags == "acc_relu" else torch.full((V, dim), 7.5, device="cuda")
        if flags == "gin":
            gpu.mgg_GIN_np_div(out, d_x, d_ptr, d_col, z, zc, 0, V, dim, V, 0, ps, wpb, dist, 0.5, col_block_rows=blk)
        else:
            gpu.mgg_SAG_np_div(out, d_x, d_ptr, d_col, z, zc, 0, V, dim, V, 0, ps, wpb, dist, col_block_rows=blk,
                               accumulate=flags == "acc_relu", relu=flags == "acc_relu",
                               row_scale_out=to_dev(s) if flags == "scale" else None)
        gpu.sync()
        return out.cpu().numpy()

    kw = {}
    if flags == "gin":
        kw = dict(flags=orc.GIN, eps=0.5)
    want, mag = oracle_agg(sh, x, x, dim, **kw)
    if flags == "scale":
        want, mag = want * s[:, None], mag * s[:, None]
    if flags == "acc_relu":
        want, mag = np.maximum(want + base, 0), mag + np.abs(base)
    for ps, wpb, dist in ((16, 4, 1), (4, 2, 3), (32, 8, 16), (0, 0, 0)):
        got = run(block_rows, ps, wpb, dist)
        assert "blocks=%d" % -(-V // block_rows) in gpu.last_agg_kernel()
        assert_close_to_oracle(got, want, mag, FP32_TOL, "column-blocked ps=%d wpb=%d dist=%d" % (ps, wpb, dist))
    plain = run(-1, 16, 4, 1)
    assert "blocks=1" in gpu.last_agg_kernel()
    assert_close_to_oracle(plain, want, mag, FP32_TOL, "plain order")
    # rows not sorted by neighbor id: the request is honoured by falling back to the plain order
    rng = np.random.default_rng(5)
    col_u = col.copy()
    for v in range(0, V, 3):
        rng.shuffle(col_u[ptr[v]:ptr[v + 1]])
    d_col_u = to_dev(col_u)
    out = torch.full((V, dim), 7.5, device="cuda")
    if flags == "plain":
        gpu.mgg_SAG_np_div(out, d_x, d_ptr, d_col_u, z, zc, 0, V, dim, V, 0, 16, 4, 1, col_block_rows=block_rows)
        gpu.sync()
        assert "blocks=1" in gpu.last_agg_kernel()
        assert_close_to_oracle(out.cpu().numpy(), want, mag, FP32_TOL, "unsorted rows")


@pytest.mark.parametrize("dim,core_rows,flags", [(16, 1024, "plain"), (44, 512, "scale"), (41, 2048, "gin"), (8, 1500, "acc_relu"),
                                                 (64, 1024, "plain"), (5, 512, "scale"), (52, 1024, "scale"), (57, 512, "gin")])
def test_dense_core_from_lds(gpu, rmat_graph, dim, core_rows, flags):
    """The dense-core path (core x core block summed from LDS tiles, the rest of the CSR on top): same sums as the
    ordinary path and the oracle with every epilogue, with padded row strides, and together with the column-blocked
    order of what is left.  Widths 52, 57 and 64 are rows of 13, 15 and 16 pieces, which the LDS kernel sums in two
    halves (7 + 6, 8 + 7, 8 + 8)."""
    import torch
    V, ptr, col = rmat_graph
    x = gpu.fill_normal((V, dim), seed=191)
    sh = share_of(ptr, col, V, 1, 0)
    d_ptr, d_col = to_dev(ptr), to_dev(col)
    z, zc = torch.zeros(V + 1, dtype=torch.int32, device="cuda"), torch.zeros(1, dtype=torch.int32, device="cuda")
    ld = dim + 3 if dim == 5 else dim
    d_x = torch.zeros(V, ld, device="cuda")
    d_x[:, :dim] = to_dev(x)
    s = gpu.fill_uniform((V,), 0.5, 2.0, seed=192)
    base = gpu.fill_normal((V, dim), seed=193)

    def run(core, blk, ps, wpb, dist):
        out = torch.full((V, ld), 7.5, device="cuda")
        if flags == "acc_relu":
            out[:, :dim] = to_dev(base)
        if flags == "gin":
            gpu.mgg_GIN_np_div(out, d_x, d_ptr, d_col, z, zc, 0, V, dim, V, 0, ps, wpb, dist, 0.5, col_block_rows=blk, core_rows=core,
                               ld_in=ld, ld_out=ld)
        else:
            gpu.mgg_SAG_np_div(out, d_x, d_ptr, d_col, z, zc, 0, V, dim, V, 0, ps, wpb, dist, col_block_rows=blk, core_rows=core,
                               accumulate=flags == "acc_relu", relu=flags == "acc_relu",
                               row_scale_out=to_dev(s) if flags == "scale" else None, ld_in=ld, ld_out=ld)
        gpu.sync()
        got = out.cpu().numpy()
        assert np.all(got[:, dim:] == 7.5)  # the padding of the output rows is not touched
        return got[:, :dim]

    kw = {}
    if flags == "gin":
        kw = dict(flags=orc.GIN, eps=0.5)
    want, mag = oracle_agg(sh, x, x, dim, **kw)
    if flags == "scale":
        want, mag = want * s[:, None], mag * s[:, None]
    if flags == "acc_relu":
        want, mag = np.maximum(want + base, 0), mag + np.abs(base)
    for blk, ps, wpb, dist in ((-1, 16, 4, 1), (-1, 4, 2, 3), (300, 32, 8, 16), (1000, 16, 4, 2), (0, 0, 0, 0)):  # 1000: six blocks in one batch
        got = run(core_rows, blk, ps, wpb, dist)
        assert "core=%d" % (core_rows // 512 * 512) in gpu.last_agg_kernel()
        assert_close_to_oracle(got, want, mag, FP32_TOL, "dense core, blk=%d ps=%d wpb=%d dist=%d" % (blk, ps, wpb, dist))
    got = run(-1, -1, 16, 4, 1)
    assert "core=" not in gpu.last_agg_kernel()
    assert_close_to_oracle(got, want, mag, FP32_TOL, "without a core")
    # closed form: all ones give the degree exactly, core or not
    ones = torch.ones(V, ld, device="cuda")
    out = torch.zeros(V, ld, device="cuda")
    gpu.mgg_SAG_np_div(out, ones, d_ptr, d_col, z, zc, 0, V, dim, V, 0, 16, 4, 1, core_rows=core_rows, ld_in=ld, ld_out=ld)
    gpu.sync()
    assert np.array_equal(out.cpu().numpy()[:, :dim], np.repeat(np.diff(ptr).astype(np.float32)[:, None], dim, 1))


@pytest.mark.parametrize("dim,core_rows", [(16, 12800), (44, 13824)])
def test_dense_core_with_tile_runs_of_unequal_length(gpu, dim, core_rows):
    """A core of 50 / 54 row groups and as many 256-column tiles, large enough for its workgroups to be cut into runs of
    tiles of unequal length (one tile for the heaviest row groups, many for the lightest): every (row group, tile) cell
    summed exactly once, at both row-width classes of the cut."""
    import torch
    from mgg_osdi23_amd import host
    V = 30000
    ptr, col = host.gen_rmat(15, V, 1_400_000, seed=23)
    x = gpu.fill_normal((V, dim), seed=301)
    sh = share_of(ptr, col, V, 1, 0)
    d_ptr, d_col, d_x = to_dev(ptr), to_dev(col), to_dev(x)
    z, zc = torch.zeros(V + 1, dtype=torch.int32, device="cuda"), torch.zeros(1, dtype=torch.int32, device="cuda")
    want, mag = oracle_agg(sh, x, x, dim)
    for blk in (-1, 0):
        out = torch.full((V, dim), 7.5, device="cuda")
        gpu.mgg_SAG_np_div(out, d_x, d_ptr, d_col, z, zc, 0, V, dim, V, 0, 0, 0, 0, col_block_rows=blk, core_rows=core_rows)
        gpu.sync()
        assert "core=%d" % core_rows in gpu.last_agg_kernel()
        assert_close_to_oracle(out.cpu().numpy(), want, mag, FP32_TOL, "core of %d rows, blk=%d" % (core_rows, blk))
    ones = torch.ones(V, dim, device="cuda")
    out = torch.zeros(V, dim, device="cuda")
    gpu.mgg_SAG_np_div(out, ones, d_ptr, d_col, z, zc, 0, V, dim, V, 0, 0, 0, 0, core_rows=core_rows)
    gpu.sync()
    assert np.array_equal(out.cpu().numpy(), np.repeat(np.diff(ptr).astype(np.float32)[:, None], dim, 1))


def test_dense_core_on_a_share_with_unsorted_rows_and_parallel_edges(gpu, rmat_graph):
    """The local half of a share whose rows start at lb > 0, neighbor lists shuffled and some edges listed twice: the
    core's index lists carry order and multiplicity as they come, so the sums still match the oracle."""
    import torch
    V, ptr, col = rmat_graph
    dim = 24
    sh = share_of(ptr, col, V, 2, 1)
    lb, ub = sh["lb"], sh["ub"]
    R = ub - lb
    rng = np.random.default_rng(3)
    lp, lc = sh["ptr_l"], sh["col_l"]
    new_ptr, new_col = [0], []
    for v in range(R):
        nb = lc[lp[v]:lp[v + 1]].copy()
        if len(nb) and v % 5 == 0:
            nb = np.concatenate([nb, nb[: 1 + len(nb) // 3]])  # parallel edges
        rng.shuffle(nb)
        new_col.append(nb)
        new_ptr.append(new_ptr[-1] + len(nb))
    p2 = np.array(new_ptr, np.int32)
    c2 = np.concatenate(new_col).astype(np.int32)
    x = gpu.fill_normal((V, dim), seed=197)
    xl = np.ascontiguousarray(x[lb:ub])
    sh2 = dict(npp=sh["npp"], lb=lb, ub=ub, ptr_l=p2, col_l=c2, ptr_r=np.zeros(R + 1, np.int32), col_r=np.zeros(0, np.int32))
    want, mag = oracle_agg(sh2, xl, x, dim)
    z, zc = torch.zeros(R + 1, dtype=torch.int32, device="cuda"), torch.zeros(1, dtype=torch.int32, device="cuda")
    out = torch.full((R, dim), 7.5, device="cuda")
    gpu.mgg_SAG_np_div(out, to_dev(xl), to_dev(p2), to_dev(c2), z, zc, lb, ub, dim, sh["npp"], 1, 16, 4, 2, core_rows=1024)
    gpu.sync()
    assert "core=1024" in gpu.last_agg_kernel()
    assert_close_to_oracle(out.cpu().numpy(), want, mag, FP32_TOL, "dense core, lb > 0, shuffled rows, parallel edges")


def test_dense_core_falls_back_and_is_searched(gpu, rmat_graph):
    """A core the graph cannot hold (fewer rows than one unit), bf16 tables and remote edges fall back to the ordinary
    path; the search returns a setting with or without a core and later calls reuse it."""
    import torch
    V, ptr, col = rmat_graph
    dim = 16
    x = gpu.fill_normal((V, dim), seed=195)
    sh = share_of(ptr, col, V, 1, 0)
    want, mag = oracle_agg(sh, x, x, dim)
    z, zc = torch.zeros(V + 1, dtype=torch.int32, device="cuda"), torch.zeros(1, dtype=torch.int32, device="cuda")
    d_ptr, d_col, d_x = to_dev(ptr), to_dev(col), to_dev(x)
    out = torch.full((V, dim), 7.5, device="cuda")
    gpu.mgg_SAG_np_div(out, d_x, d_ptr, d_col, z, zc, 0, V, dim, V, 0, 16, 4, 1, core_rows=300)
    gpu.sync()
    assert "core=" not in gpu.last_agg_kernel()
    assert_close_to_oracle(out.cpu().numpy(), want, mag, FP32_TOL, "core smaller than a unit")
    kn, ms = gpu.tune_np_div(out, d_x, d_ptr, d_col, z, zc, 0, V, dim, V, 16, core_rows=1024)
    gpu.sync()
    assert kn["core_rows"] == 1024 and ms > 0
    assert_close_to_oracle(out.cpu().numpy(), want, mag, FP32_TOL, "after the search")
    out.fill_(7.5)
    gpu.mgg_SAG_np_div(out, d_x, d_ptr, d_col, z, zc, 0, V, dim, V, 0, 0, 0, 0)
    gpu.sync()
    assert "core=1024" in gpu.last_agg_kernel()
    assert_close_to_oracle(out.cpu().numpy(), want, mag, FP32_TOL, "searched setting reused")
    # a share with remote edges: the request is ignored
    sh2 = share_of(ptr, col, V, 2, 0)
    got = torch.full((sh2["ub"] - sh2["lb"], dim), 7.5, device="cuda")
    gpu.mgg_SAG_np_div(got, to_dev(x[sh2["lb"]:sh2["ub"]]), to_dev(sh2["ptr_l"]), to_dev(sh2["col_l"]), to_dev(sh2["ptr_r"]),
                       to_dev(sh2["col_r"]), sh2["lb"], sh2["ub"], dim, sh2["npp"], 0, 16, 4, 1, input_remote=d_x, core_rows=512)
    gpu.sync()
    assert "core=" not in gpu.last_agg_kernel()
    w2, m2 = oracle_agg(sh2, x[sh2["lb"]:sh2["ub"]], x, dim)
    assert_close_to_oracle(got.cpu().numpy(), w2, m2, FP32_TOL, "share with remote edges")


def test_column_blocked_order_with_bf16_tables(gpu, rmat_graph):
    """bf16 feature rows, fp32 partial rows and output: the blocked order must give what the plain order gives."""
    import torch
    V, ptr, col = rmat_graph
    dim = 64
    x = gpu.fill_normal((V, dim), seed=95)
    d_x = to_dev(x).to(torch.bfloat16)
    xr = d_x.float().cpu().numpy()
    sh = share_of(ptr, col, V, 1, 0)
    d_ptr, d_col = to_dev(ptr), to_dev(col)
    z, zc = torch.zeros(V + 1, dtype=torch.int32, device="cuda"), torch.zeros(1, dtype=torch.int32, device="cuda")
    want, mag = oracle_agg(sh, xr, xr, dim, flags=orc.GIN, eps=0.25)
    for blk in (200, -1):
        out = torch.full((V, dim), 7.5, device="cuda")
        gpu.mgg_GIN_np_div(out, d_x, d_ptr, d_col, z, zc, 0, V, dim, V, 0, 16, 4, 2, 0.25, col_block_rows=blk)
        gpu.sync()
        assert ("blocks=30" in gpu.last_agg_kernel()) == (blk > 0)
        assert_close_to_oracle(out.cpu().numpy(), want, mag, FP32_TOL, "bf16 tables, col_block_rows=%d" % blk)


def test_column_blocked_with_empty_rows_and_search(gpu):
    """Rows without neighbors, rows whose neighbors all fall in one block, and the search over both orders."""
    import torch
    V, dim = 5000, 16
    rng = np.random.default_rng(11)
    deg = rng.integers(0, 400, V)
    deg[rng.integers(0, V, 500)] = 0
    ptr = np.zeros(V + 1, np.int32)
    ptr[1:] = np.cumsum(deg)
    col = np.concatenate([np.sort(rng.choice(V if v % 7 else 50, d, replace=d > 50)) for v, d in enumerate(deg)] + [np.zeros(0, np.int64)]).astype(np.int32)
    x = gpu.fill_normal((V, dim), seed=94)
    sh = share_of(ptr, col, V, 1, 0)
    want, mag = oracle_agg(sh, x, x, dim)
    d_ptr, d_col, d_x = to_dev(ptr), to_dev(col), to_dev(x)
    z, zc = torch.zeros(V + 1, dtype=torch.int32, device="cuda"), torch.zeros(1, dtype=torch.int32, device="cuda")
    out = torch.full((V, dim), 7.5, device="cuda")
    gpu.mgg_SAG_np_div(out, d_x, d_ptr, d_col, z, zc, 0, V, dim, V, 0, 16, 4, 2, col_block_rows=512)
    gpu.sync()
    assert "blocks=10" in gpu.last_agg_kernel()
    assert_close_to_oracle(out.cpu().numpy(), want, mag, FP32_TOL, "column-blocked, empty rows")
    out.fill_(7.5)
    kn, ms = gpu.tune_np_div(out, d_x, d_ptr, d_col, z, zc, 0, V, dim, V, 0, col_block_rows=512)
    assert kn["ps"] in (16, 32) and kn["col_block_rows"] == 512 and ms > 0
    assert_close_to_oracle(out.cpu().numpy(), want, mag, FP32_TOL, "result left by the search")
    out.fill_(7.5)
    gpu.mgg_SAG_np_div(out, d_x, d_ptr, d_col, z, zc, 0, V, dim, V, 0, 0, 0, 0)
    gpu.sync()
    assert "blocks=10" in gpu.last_agg_kernel()   # the remembered setting
    assert_close_to_oracle(out.cpu().numpy(), want, mag, FP32_TOL, "remembered setting")


@pytest.mark.parametrize("dim,dtype", [(16, "f32"), (44, "f32"), (128, "bf16")])
def test_compact_remote_table_gives_the_same_sums(gpu, rmat_graph, dim, dtype):
    """Remote rows staged compactly (one row per distinct remote id, most referenced first) with the column array
    rewritten to match: bit-identical output to the table indexed by global id, and within tolerance of the oracle."""
    import torch
    V, ptr, col = rmat_graph
    x = gpu.fill_normal((V, dim), seed=70)
    sh = share_of(ptr, col, V, 4, 2)
    lb, ub = sh["lb"], sh["ub"]
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    d_x = to_dev(x).to(td)
    d_xl = d_x[lb:ub].clone()
    compact, ids = gpu.compact_remote(sh["col_r"])
    d_compact, d_ids_dev = gpu.compact_remote_device(to_dev(sh["col_r"]), len(sh["col_r"]))  # the same on the GPU: bit-identical
    assert np.array_equal(d_compact.cpu().numpy(), compact) and np.array_equal(d_ids_dev.cpu().numpy(), ids)
    d_ids = to_dev(ids)
    staged = torch.full((len(ids), dim), 3.0, device="cuda", dtype=td)
    gpu.gather_rows(staged, d_x, d_ids, len(ids), dim * d_x.element_size())
    gpu.sync()
    assert torch.equal(staged, d_x[d_ids.long()])
    d = [to_dev(sh["ptr_l"]), to_dev(sh["col_l"]), to_dev(sh["ptr_r"])]
    out_a = torch.full((ub - lb, dim), 7.5, device="cuda")
    out_b = torch.full((ub - lb, dim), 7.5, device="cuda")
    gpu.mgg_SAG_np_div(out_a, d_xl, d[0], d[1], d[2], to_dev(sh["col_r"]), lb, ub, dim, sh["npp"], 0, 16, 4, 2, input_remote=d_x)
    gpu.mgg_SAG_np_div(out_b, d_xl, d[0], d[1], d[2], to_dev(compact), lb, ub, dim, sh["npp"], 0, 16, 4, 2, input_remote=staged)
    gpu.sync()
    assert torch.equal(out_a, out_b)
    xr = d_x.float().cpu().numpy()
    want, mag = oracle_agg(sh, xr[lb:ub], xr, dim)
    assert_close_to_oracle(out_b.cpu().numpy(), want, mag, FP32_TOL, "compact remote table")


def test_bad_arguments_return_errors_not_faults(gpu, rmat_graph):
    """Shapes the kernels are not built for are refused on the host, with a message, before any launch."""
    import torch
    V, ptr, col = rmat_graph
    d_ptr, d_col = to_dev(ptr), to_dev(col)
    z = torch.zeros(V + 1, dtype=torch.int32, device="cuda")
    x = torch.zeros(V, 16, device="cuda")
    out = torch.zeros(V, 16, device="cuda")
    call = lambda **kw: gpu.mgg_SAG_np_div(out, x, d_ptr, d_col, z, z, 0, V, kw.get("dim", 16), kw.get("npp", V), 0,
                                           kw.get("ps", 16), kw.get("wpb", 4), kw.get("dist", 1), ld_in=kw.get("ld_in", 0))
    for bad in (dict(dim=0), dict(dim=300), dict(wpb=17), dict(wpb=-1), dict(dist=-2), dict(ps=-1), dict(npp=V - 1), dict(ld_in=8)):
        with pytest.raises(gpu.MggxError):
            call(**bad)
    with pytest.raises(gpu.MggxError):
        gpu.dense_forward(out, x, x, V, 16, 16, ld_x=8)
    with pytest.raises(gpu.MggxError):
        gpu.dense_forward(x, x, out, V, 16, 16)  # in place
    with pytest.raises(gpu.MggxError):
        gpu.softmax_forward(out, x, V, 0)
    call()  # the library is still usable afterwards
    gpu.sync()


def test_plan_cache_eviction_and_release(gpu):
    """More distinct graphs than the plan cache holds, then an explicit release: results stay right."""
    import torch
    dim = 8
    graphs = []
    for i in range(20):
        V = 200 + 10 * i
        ptr, col = gpu.gen_rmat(9, V, 1500, seed=100 + i)
        x = gpu.fill_normal((V, dim), seed=i)
        graphs.append((V, ptr, col, x, to_dev(ptr), to_dev(col), to_dev(x)))
    z = torch.zeros(600, dtype=torch.int32, device="cuda")
    for rnd in range(2):
        for V, ptr, col, x, d_ptr, d_col, d_x in graphs:
            out = torch.empty(V, dim, device="cuda")
            gpu.mgg_SAG_np_div(out, d_x, d_ptr, d_col, z, z, 0, V, dim, V, 0, 4, 2, 1)
            gpu.sync()
            want = orc.sag_np_div(x, x, ptr, col, None, None, 0, V, dim, V)
            assert np.allclose(out.cpu().numpy(), want, rtol=1e-5, atol=1e-5)
        gpu.release_cached()


def test_forget_lets_a_csr_array_be_rewritten(gpu):
    """The plan cache is keyed by address: after forget(), the same device arrays may hold another graph."""
    import torch
    V, dim = 500, 16
    x = gpu.fill_normal((V, dim), seed=9)
    d_x = to_dev(x)
    z = torch.zeros(V + 1, dtype=torch.int32, device="cuda")
    d_ptr = torch.zeros(V + 1, dtype=torch.int32, device="cuda")
    d_col = torch.zeros(40000, dtype=torch.int32, device="cuda")
    for seed in (1, 2):
        ptr, col = gpu.gen_rmat(9, V, 6000, seed=seed)
        assert len(col) <= 40000
        gpu.forget(d_ptr)
        d_ptr.copy_(torch.from_numpy(ptr))
        d_col[:len(col)].copy_(torch.from_numpy(col))
        out = torch.empty(V, dim, device="cuda")
        gpu.mgg_SAG_np_div(out, d_x, d_ptr, d_col, z, z, 0, V, dim, V, 0, 16, 4, 2)
        gpu.sync()
        want = orc.sag_np_div(x, x, ptr, col, None, None, 0, V, dim, V)
        assert np.allclose(out.cpu().numpy(), want, rtol=1e-5, atol=1e-5)


# --------------------------------------------------------------------------- widths, strides, options
@pytest.mark.parametrize("dim", [1, 2, 3, 4, 5, 8, 12, 16, 17, 24, 32, 41, 47, 64, 100, 128, 200, 256])
def test_feature_widths(gpu, rmat_graph, dim):
    V, ptr, col = rmat_graph
    x = gpu.fill_normal((V, dim), seed=100 + dim)
    sh = share_of(ptr, col, V, 2, 0)
    xl = x[sh["lb"]:sh["ub"]]
    got = run_agg(gpu, sh, to_dev(xl), to_dev(x), dim, 16, 4, 2)
    want, mag = oracle_agg(sh, xl, x, dim)
    assert_close_to_oracle(got, want, mag, FP32_TOL, "dim=%d" % dim)


@pytest.mark.parametrize("dim,ld", [(41, 44), (16, 20), (47, 48), (10, 12)])
def test_padded_row_strides(gpu, rmat_graph, dim, ld):
    V, ptr, col = rmat_graph
    xp = gpu.fill_normal((V, ld), seed=9)  # padding columns hold junk on purpose
    sh = share_of(ptr, col, V, 2, 1)
    got = run_agg(gpu, sh, to_dev(xp[sh["lb"]:sh["ub"]]), to_dev(xp), dim, 8, 4, 1, ld_in=ld, ld_out=ld)
    x = np.ascontiguousarray(xp[:, :dim])
    want, mag = oracle_agg(sh, x[sh["lb"]:sh["ub"]], x, dim)
    assert_close_to_oracle(got[:, :dim], want, mag, FP32_TOL, "dim=%d ld=%d" % (dim, ld))
    assert np.all(got[:, dim:] == 7.5), "padding columns of the output must stay untouched"


@pytest.mark.parametrize("dim", [16, 41, 64])
def test_gin_accumulate_relu(gpu, rmat_graph, dim):
    V, ptr, col = rmat_graph
    x = gpu.fill_normal((V, dim), seed=4)
    sh = share_of(ptr, col, V, 3, 1)
    xl = x[sh["lb"]:sh["ub"]]
    R = sh["ub"] - sh["lb"]
    # GIN: (1+eps) x_v + sum
    got = run_agg(gpu, sh, to_dev(xl), to_dev(x), dim, 16, 8, 1, gin=True, eps=0.25)
    want, mag = oracle_agg(sh, xl, x, dim, flags=orc.GIN, eps=0.25)
    assert_close_to_oracle(got, want, mag, FP32_TOL, "GIN")
    # accumulate: out += sum (the reference's SAG behaviour)
    base = gpu.fill_normal((R, dim), seed=5)
    got = run_agg(gpu, sh, to_dev(xl), to_dev(x), dim, 16, 8, 1, accumulate_into=base)
    want, mag = oracle_agg(sh, xl, x, dim, flags=orc.ACCUMULATE, out=base.copy())
    assert_close_to_oracle(got, want, mag + np.abs(base), FP32_TOL, "accumulate")
    # ReLU epilogue
    got = run_agg(gpu, sh, to_dev(xl), to_dev(x), dim, 16, 8, 1, relu=True)
    want, mag = oracle_agg(sh, xl, x, dim)
    assert_close_to_oracle(got, np.maximum(want, 0), mag, FP32_TOL, "relu")


# --------------------------------------------------------------------------- ragged / empty inputs
def test_empty_rows_isolated_nodes_and_hub(gpu):
    # hand-built graph: empty rows at both ends and in the middle, one hub with 5000 neighbors
    V, dim = 300, 16
    rows = [[] for _ in range(V)]
    rng = np.random.default_rng(0)
    rows[5] = list(rng.integers(0, V, 5000))
    rows[6] = [1, 2, 3]
    rows[150] = list(rng.integers(0, V, 33))
    rows[298] = [0]
    ptr = np.zeros(V + 1, np.int32)
    ptr[1:] = np.cumsum([len(r) for r in rows])
    col = np.array([c for r in rows for c in r], np.int32)
    x = gpu.fill_normal((V, dim), seed=8)
    for num_gpus, pe in [(1, 0), (2, 0), (2, 1)]:
        sh = share_of(ptr, col, V, num_gpus, pe)
        xl = x[sh["lb"]:sh["ub"]]
        for ps, wpb, dist in [(16, 1, 1), (16, 4, 1), (4, 2, 3), (65536, 4, 1)]:
            got = run_agg(gpu, sh, to_dev(xl), to_dev(x), dim, ps, wpb, dist)
            want, mag = oracle_agg(sh, xl, x, dim)
            assert_close_to_oracle(got, want, mag, FP32_TOL, "ragged %s" % ((num_gpus, pe, ps, wpb, dist),))
            got = run_agg(gpu, sh, to_dev(xl), to_dev(x), dim, ps, wpb, dist, gin=True, eps=0.0)
            want, mag = oracle_agg(sh, xl, x, dim, flags=orc.GIN)
            assert_close_to_oracle(got, want, mag, FP32_TOL, "ragged GIN")


def test_graph_without_edges_and_zero_rows(gpu):
    import torch
    V, dim = 64, 16
    ptr = np.zeros(V + 1, np.int32)
    col = np.zeros(0, np.int32)
    x = gpu.fill_normal((V, dim), seed=1)
    sh = share_of(ptr, col, V, 1, 0)
    got = run_agg(gpu, sh, to_dev(x), to_dev(x), dim, 16, 4, 1)
    assert np.array_equal(got, np.zeros((V, dim), np.float32))
    # zero rows: a no-op that must not fail
    z = torch.zeros(1, dtype=torch.int32, device="cuda")
    gpu.mgg_SAG_np_div(torch.zeros(1, dim, device="cuda"), to_dev(x), z, z, z, z, 0, 0, dim, 16, 0, 16, 4, 1)
    gpu.sync()


@pytest.mark.parametrize("ps", [1, 2, 3, 5, 6, 7, 8, 15])
def test_small_partitions_are_summed_in_groups_of_at_most_16_neighbors(gpu, rmat_graph, ps):
    """ps < 16: consecutive partitions of a row are consecutive edges, so a slot of the kernel takes floor(16 / ps) of them
    at once -- one descriptor per group, not one per partition.  Same sums; and the plan holds about a sixteenth of a
    descriptor (16 bytes) per edge at every ps, where one descriptor per partition would hold 16 / ps bytes per edge."""
    V, ptr, col = rmat_graph
    dim = 16
    x = gpu.fill_normal((V, dim), seed=2)
    sh = share_of(ptr, col, V, 2, 0)
    xl = x[sh["lb"]:sh["ub"]]
    gpu.release_cached()
    got = run_agg(gpu, sh, to_dev(xl), to_dev(x), dim, ps, 4, 2)
    want, mag = oracle_agg(sh, xl, x, dim)
    assert_close_to_oracle(got, want, mag, FP32_TOL, "ps=%d" % ps)
    st = gpu.cache_stats()
    rows, nnz = sh["ub"] - sh["lb"], len(sh["col_l"]) + len(sh["col_r"])
    unit = ps * (16 // ps)
    units = int(np.sum(-(-np.diff(sh["ptr_l"]) // unit)) + np.sum(-(-np.diff(sh["ptr_r"]) // unit)))
    assert st["plans"] == 1 and st["plan_bytes"] == 16 * units + 4 * (rows + 1) + 4 * rows
    assert 16 * units <= 1.6 * nnz  # this graph: 36 neighbors per row and side on average, the last group of a row part full
    gpu.release_cached()


# --------------------------------------------------------------------------- explicit partition arrays
@pytest.mark.parametrize("ps,wpb,dist", [(16, 4, 1), (3, 2, 2), (32, 8, 1), (1, 4, 2), (2, 1, 1), (5, 4, 4), (7, 8, 1)])
def test_explicit_partition_arrays(gpu, rmat_graph, ps, wpb, dist):
    """SAG_host / SAG_host_fused_interleaved (local half): build_part arrays in, out += partition sums."""
    import torch
    V, ptr, col = rmat_graph
    dim = 16
    sh = share_of(ptr, col, V, 2, 1)
    R = sh["ub"] - sh["lb"]
    x = gpu.fill_normal((V, dim), seed=6)
    xl = np.ascontiguousarray(x[sh["lb"]:sh["ub"]])
    pp, p2n, _ = orc.build_part(sh["ptr_l"], R, ps)
    base = gpu.fill_normal((R, dim), seed=7)
    out = to_dev(base)
    gpu.SAG_host(out, to_dev(xl), to_dev(sh["ptr_l"]), to_dev(sh["col_l"]), to_dev(pp), to_dev(p2n), sh["lb"], R, len(p2n),
                 ps, dim, 32, wpb, dist)
    gpu.sync()
    want = orc.sag_parts(xl, sh["col_l"], pp, p2n, sh["lb"], dim, base.copy())
    only_local = dict(sh, ptr_r=np.zeros(R + 1, np.int32), col_r=np.zeros(0, np.int32))
    _, mag = oracle_agg(only_local, xl, x, dim)
    assert_close_to_oracle(out.cpu().numpy(), want, mag + np.abs(base), FP32_TOL, "explicit parts")


def test_explicit_parts_missing_terminal_entry(gpu):
    """The reference leaves partPtr[numParts] at 0 when the last node has no neighbors; lengths come from the row
    pointers here, so the last partition is still summed."""
    ptr = np.array([0, 3, 3, 8, 8], np.int32)
    col = np.array([0, 1, 3, 0, 1, 2, 3, 2], np.int32)
    pp, p2n, _ = orc.build_part(ptr, 4, 2)
    assert pp[-1] == 0
    x = np.arange(4 * 4, dtype=np.float32).reshape(4, 4) + 1
    import torch
    out = torch.zeros(4, 4, device="cuda")
    gpu.SAG_host(out, to_dev(x), to_dev(ptr), to_dev(col), to_dev(pp), to_dev(p2n), 0, 4, len(p2n), 2, 4, 32, 2, 1)
    gpu.sync()
    want = orc.sag_ref(x, ptr, col)
    assert np.array_equal(out.cpu().numpy(), want)


def test_single_gpu_spmm(gpu, rmat_graph):
    import torch
    V, ptr, col = rmat_graph
    dim = 32
    x = gpu.fill_normal((V, dim), seed=12)
    out = torch.zeros(V, dim, device="cuda")
    gpu.SpMM(out, to_dev(x), to_dev(ptr), to_dev(col), V, dim, 16, 8)
    gpu.sync()
    want = orc.sag_np_div(x, x, ptr, col, None, None, 0, V, dim, V)
    rows = np.arange(V, dtype=np.int32)
    mag = orc.sag_np_div_rows(rows, x, x, ptr, col, None, None, 0, V, dim, V, abs_sum=True)
    assert_close_to_oracle(out.cpu().numpy(), want, mag, FP32_TOL, "spmm")


# --------------------------------------------------------------------------- GPU-side build_part (bit-exact)
@pytest.mark.parametrize("ps", [1, 2, 16, 65536])
def test_build_part_device_bit_exact(gpu, rmat_graph, ps):
    V, ptr, col = rmat_graph
    for indptr in (ptr, np.array([0, 3, 3, 8, 8], np.int32), np.array([0, 0, 0], np.int32), np.array([0, 5], np.int32)):
        n = len(indptr) - 1
        want = orc.build_part(indptr, n, ps)
        got = gpu.build_part_device(to_dev(indptr), n, ps, compat=True)
        for g, w, name in zip(got, want, ("partPtr", "part2Node", "node2Part")):
            assert np.array_equal(g.cpu().numpy(), w), name


@pytest.mark.parametrize("num_gpus,pe", [(1, 0), (3, 0), (3, 1), (3, 2), (8, 5)])
def test_split_csr_device_bit_exact(gpu, rmat_graph, num_gpus, pe):
    V, ptr, col = rmat_graph
    npp, lb, ub = orc.range_partition(V, num_gpus, pe)
    want = orc.split_csr(ptr, col, lb, ub)
    got = gpu.split_CSR_device(to_dev(ptr), to_dev(col), lb, ub)
    for g, w, name in zip(got, want, ("local_ptr", "remote_ptr", "local_col_idx", "remote_col_idx")):
        assert np.array_equal(g.cpu().numpy(), w), name
    # ragged: empty rows, an unsorted row, a 5000-neighbor row
    rng = np.random.default_rng(1)
    deg = np.array([0, 5000, 3, 0, 0, 130, 64, 1, 0], np.int64)
    p = np.zeros(len(deg) + 1, np.int32)
    p[1:] = np.cumsum(deg)
    c = rng.integers(0, len(deg), int(p[-1])).astype(np.int32)
    want = orc.split_csr(p, c, 2, 7)
    got = gpu.split_CSR_device(to_dev(p), to_dev(c), 2, 7)
    for g, w in zip(got, want):
        assert np.array_equal(g.cpu().numpy(), w)


# --------------------------------------------------------------------------- dense update and softmax
@pytest.mark.parametrize("n,d1,d2", [(1000, 602, 16), (1000, 16, 41), (777, 100, 64), (512, 64, 64), (300, 64, 47),
                                     (256, 128, 128), (65, 7, 3), (1, 1, 1), (130, 33, 130), (100, 1500, 64), (70, 65, 16)])
def test_dense_update(gpu, n, d1, d2):
    import torch
    x = gpu.fill_normal((n, d1), seed=20)
    w = gpu.glorot(d1, d2, seed=21)
    out = torch.full((n, d2), 3.0, device="cuda")
    gpu.dense_forward(out, to_dev(x), to_dev(w), n, d1, d2)
    gpu.sync()
    want = orc.dense(x, w, f64=True)
    mag = np.abs(x).astype(np.float64) @ np.abs(w).astype(np.float64)
    assert_close_to_oracle(out.cpu().numpy(), want, mag, FP32_TOL, "dense %dx%dx%d" % (n, d1, d2))
    # the same rows inside a wider table (row pitch d1 + 3, unaligned rows), poisoned padding
    xp = np.full((n, d1 + 3), np.nan, np.float32)
    xp[:, :d1] = x
    out = torch.full((n, d2), 3.0, device="cuda")
    gpu.dense_forward(out, to_dev(xp), to_dev(w), n, d1, d2, ld_x=d1 + 3)
    gpu.sync()
    assert_close_to_oracle(out.cpu().numpy(), want, mag, FP32_TOL, "dense %dx%dx%d, strided X" % (n, d1, d2))


@pytest.mark.parametrize("n,d1,d2,ld_out,relu,scale", [(4096, 602, 16, 16, False, False), (4099, 130, 7, 9, True, True),
                                                         (5000, 767, 16, 16, False, True), (4111, 301, 1, 1, False, False),
                                                         (70001, 250, 13, 16, True, False), (4111, 602, 16, 20, True, True)])
def test_dense_update_in_flat_tiles(gpu, n, d1, d2, ld_out, relu, scale):
    """4096 rows and more of densely packed rows that are no multiple of 32 bytes, at most 16 columns out: whole tiles of 16
    rows go through the kernel that reads them as flat runs of memory (K split over the wavefronts of a workgroup), the
    rows after the last whole tile through the general kernel."""
    import torch
    x = gpu.fill_normal((n, d1), seed=70)
    w = gpu.glorot(d1, d2, seed=71)
    s = gpu.fill_uniform((n,), 0.5, 1.5, seed=72) if scale else None
    out = torch.full((n, ld_out), 9.0, device="cuda")
    gpu.dense_forward(out, to_dev(x), to_dev(w), n, d1, d2, ld_out=ld_out, row_scale=to_dev(s) if scale else None, relu=relu)
    gpu.sync()
    want = orc.dense(x, w, f64=True)
    mag = np.abs(x).astype(np.float64) @ np.abs(w).astype(np.float64)
    if scale:
        want, mag = want * s[:, None], mag * s[:, None]
    if relu:
        want = np.maximum(want, 0)
    got = out.cpu().numpy()
    assert_close_to_oracle(got[:, :d2], want, mag, FP32_TOL, "dense in flat tiles %dx%dx%d" % (n, d1, d2))
    assert np.all(got[:, d2:] == 9.0)
    # closed form: ones times ones is d1, exactly, in every row
    out = torch.zeros(n, d2, device="cuda")
    gpu.dense_forward(out, torch.ones(n, d1, device="cuda"), torch.ones(d1, d2, device="cuda"), n, d1, d2)
    gpu.sync()
    assert np.array_equal(out.cpu().numpy(), np.full((n, d2), float(d1), np.float32))


def test_dense_closed_forms_and_epilogue(gpu):
    import torch
    n, d1, d2 = 200, 602, 16
    out = torch.zeros(n, d2, device="cuda")
    gpu.dense_forward(out, torch.ones(n, d1, device="cuda"), torch.ones(d1, d2, device="cuda"), n, d1, d2)
    gpu.sync()
    assert np.array_equal(out.cpu().numpy(), np.full((n, d2), float(d1), np.float32))  # the reference's all-ones setup
    x = gpu.fill_normal((n, 48), seed=3)
    out = torch.zeros(n, 48, device="cuda")
    gpu.dense_forward(out, to_dev(x), torch.eye(48, device="cuda"), n, 48, 48)
    gpu.sync()
    assert np.array_equal(out.cpu().numpy(), x)
    # row scale + relu epilogue, padded output stride
    s = gpu.fill_uniform((n,), 0.1, 2.0, seed=4)
    w = gpu.glorot(48, 41, seed=5)
    out = torch.full((n, 44), 9.0, device="cuda")
    gpu.dense_forward(out, to_dev(x), to_dev(w), n, 48, 41, ld_out=44, row_scale=to_dev(s), relu=True)
    gpu.sync()
    want = np.maximum(orc.dense(x, w) * s[:, None], 0)
    mag = (np.abs(x).astype(np.float64) @ np.abs(w).astype(np.float64)) * s[:, None]
    got = out.cpu().numpy()
    assert_close_to_oracle(got[:, :41], want, mag, FP32_TOL, "dense epilogue")
    assert np.all(got[:, 41:] == 9.0)


@pytest.mark.parametrize("n,d1,h,d3,relu_mid", [(1000, 64, 64, 64, True), (777, 64, 64, 47, True), (130, 100, 33, 5, False),
                                                 (17, 7, 16, 64, True), (4099, 200, 48, 17, True),
                                                 # 4096 rows and more of 64 -> 64 -> 33..64: the split-operand kernel on the bf16 matrix cores
                                                 (4096, 64, 64, 64, True), (5003, 64, 64, 47, True), (70001, 64, 64, 33, False), (4100, 64, 64, 64, False)])
def test_fused_two_layer_update(gpu, n, d1, h, d3, relu_mid):
    """act(X.Wa).Wb in one pass against the oracle's two dense updates (and against two library calls)."""
    import torch
    x = gpu.fill_normal((n, d1), seed=60)
    wa = gpu.glorot(d1, h, seed=61)
    wb = gpu.glorot(h, d3, seed=62)
    s = gpu.fill_uniform((n,), 0.5, 1.5, seed=63)
    ldo = d3 + 3
    out = torch.full((n, ldo), 9.0, device="cuda")
    gpu.mlp2_forward(out, to_dev(x), to_dev(wa), to_dev(wb), n, d1, h, d3, ld_out=ldo, row_scale=to_dev(s), relu_mid=relu_mid)
    gpu.sync()
    t = orc.dense(x, wa, f64=True)
    mag_t = np.abs(x).astype(np.float64) @ np.abs(wa).astype(np.float64)
    if relu_mid:
        t = np.maximum(t, 0)
    want = (t @ wb.astype(np.float64)) * s[:, None]
    mag = (mag_t @ np.abs(wb).astype(np.float64)) * s[:, None]
    got = out.cpu().numpy()
    assert_close_to_oracle(got[:, :d3], want, mag, 2 * FP32_TOL, "fused two-layer update")
    assert np.all(got[:, d3:] == 9.0)
    # the two-call form of the same thing
    mid = torch.empty(n, h, device="cuda")
    two = torch.empty(n, d3, device="cuda")
    gpu.dense_forward(mid, to_dev(x), to_dev(wa), n, d1, h, relu=relu_mid)
    gpu.dense_forward(two, mid, to_dev(wb), n, h, d3, row_scale=to_dev(s))
    gpu.sync()
    assert_close_to_oracle(two.cpu().numpy(), want, mag, 2 * FP32_TOL, "two calls")
    with pytest.raises(gpu.MggxError):
        gpu.mlp2_forward(out, to_dev(x), to_dev(wa), to_dev(wb), n, d1, 65, d3)


@pytest.mark.parametrize("n,d1,h,d3", [(1000, 64, 64, 47), (5003, 64, 64, 47), (4100, 64, 64, 64), (130, 100, 33, 5), (70001, 64, 64, 33)])
def test_fused_two_layer_update_ends_in_softmax(gpu, n, d1, h, d3):
    """The last update of a forward with the row softmax in the same pass: against the oracle's softmax of its own two dense
    updates, and against the library's separate calls (fused update, then mggx_softmax_rows)."""
    import torch
    x = gpu.fill_normal((n, d1), seed=80)
    wa = gpu.glorot(d1, h, seed=81)
    wb = gpu.glorot(h, d3, seed=82) * 4
    s = gpu.fill_uniform((n,), 0.5, 1.5, seed=83)
    ldo = d3 + 1
    out = torch.full((n, ldo), 9.0, device="cuda")
    gpu.mlp2_forward(out, to_dev(x), to_dev(wa), to_dev(wb), n, d1, h, d3, ld_out=ldo, row_scale=to_dev(s), relu_mid=True, softmax_out=True)
    gpu.sync()
    t = np.maximum(orc.dense(x, wa, f64=True), 0)
    logits = (t @ wb.astype(np.float64)) * s[:, None]
    e = np.exp(logits - logits.max(1, keepdims=True))
    want = e / e.sum(1, keepdims=True)
    got = out.cpu().numpy()
    assert np.allclose(got[:, :d3], want, rtol=2e-5, atol=1e-7), np.abs(got[:, :d3] - want).max()
    assert np.allclose(got[:, :d3].sum(1), 1.0, atol=1e-5)
    assert np.all(got[:, d3:] == 9.0)
    lg = torch.empty(n, d3, device="cuda")
    two = torch.empty(n, d3, device="cuda")
    gpu.mlp2_forward(lg, to_dev(x), to_dev(wa), to_dev(wb), n, d1, h, d3, row_scale=to_dev(s), relu_mid=True)
    gpu.softmax_forward(two, lg, n, d3)
    gpu.sync()
    assert np.allclose(got[:, :d3], two.cpu().numpy(), rtol=1e-5, atol=1e-7)
    # packed rows (ld_out = d3; where d3 is no multiple of 4 and there are 4096 rows or more, tiles leave as contiguous runs)
    packed = torch.full((n + 1, d3), 9.0, device="cuda")
    gpu.mlp2_forward(packed, to_dev(x), to_dev(wa), to_dev(wb), n, d1, h, d3, row_scale=to_dev(s), relu_mid=True, softmax_out=True)
    gpu.sync()
    pk = packed.cpu().numpy()
    assert np.allclose(pk[:n], want, rtol=2e-5, atol=1e-7), np.abs(pk[:n] - want).max()
    assert np.all(pk[n] == 9.0)  # nothing written past the last row
    lgw = np.maximum(logits, 0)
    gpu.mlp2_forward(packed, to_dev(x), to_dev(wa), to_dev(wb), n, d1, h, d3, row_scale=to_dev(s), relu_mid=True, relu_out=True)
    gpu.sync()
    pk = packed.cpu().numpy()
    mag = ((np.abs(x).astype(np.float64) @ np.abs(wa).astype(np.float64)) @ np.abs(wb).astype(np.float64)) * s[:, None]
    assert_close_to_oracle(pk[:n], lgw, mag, 2 * FP32_TOL, "packed rows, ReLU out")
    assert np.all(pk[n] == 9.0)
    with pytest.raises(AssertionError):
        gpu.mlp2_forward(out, to_dev(x), to_dev(wa), to_dev(wb), n, d1, h, d3, relu_out=True, softmax_out=True)


@pytest.mark.parametrize("n,c", [(1000, 41), (333, 47), (64, 1), (10, 200), (5, 64)])
def test_softmax_rows(gpu, n, c):
    import torch
    x = gpu.fill_normal((n, c), seed=30) * 5
    out = torch.zeros(n, c, device="cuda")
    gpu.softmax_forward(out, to_dev(x), n, c)
    gpu.sync()
    want = orc.softmax_rows(x)
    got = out.cpu().numpy()
    assert np.allclose(got, want, rtol=1e-5, atol=1e-7)
    assert np.allclose(got.sum(1), 1.0, atol=1e-5)
    # in place
    t = to_dev(x)
    gpu.softmax_forward(t, t, n, c)
    gpu.sync()
    assert np.allclose(t.cpu().numpy(), want, rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("rows,ld,row_bytes", [(1000, 64, 64), (333, 192, 176), (77, 256, 256), (5, 32, 16)])
def test_gather_yardstick_counts_its_loads(gpu, rows, ld, row_bytes):
    """On a table of ones every lane that holds a piece of a row sums 4 per load; the other lanes issue none."""
    import torch
    table = torch.ones(rows * ld // 4, device="cuda")
    sink = torch.full((262144,), -1.0, device="cuda")
    done = gpu.gather_probe(sink, table, rows, ld, row_bytes, 1_000_000)
    gpu.sync()
    lanes = 4 if row_bytes <= 64 else 16
    per_launch = 1024 * 4 * (64 // lanes) * 8
    assert done >= 1_000_000 and done % per_launch == 0
    s = sink.cpu().numpy().reshape(-1, lanes)
    on = row_bytes // 16
    assert np.all(s[:, :on] == 4.0 * 8 * (done // per_launch)) and np.all(s[:, on:] == 0.0)
    with pytest.raises(gpu.MggxError):
        gpu.gather_probe(sink, table, rows, ld, 24, 1000)


# --------------------------------------------------------------------------- bf16 tables, fp32 accumulation
@pytest.mark.parametrize("dim", [8, 64, 128, 256])
def test_bf16_tables(gpu, rmat_graph, dim):
    import torch
    V, ptr, col = rmat_graph
    x = gpu.fill_normal((V, dim), seed=40)
    xb = to_dev(x).to(torch.bfloat16)
    xf = xb.to(torch.float32).cpu().numpy()  # the exact values the kernel sees
    sh = share_of(ptr, col, V, 2, 0)
    got = run_agg(gpu, sh, xb[sh["lb"]:sh["ub"]].contiguous(), xb, dim, 16, 8, 1)
    want, mag = oracle_agg(sh, xf[sh["lb"]:sh["ub"]], xf, dim)
    assert_close_to_oracle(got, want, mag, FP32_TOL, "bf16 in, fp32 accumulate (vs the same rounded inputs)")
    want_f, mag_f = oracle_agg(sh, x[sh["lb"]:sh["ub"]], x, dim)
    assert_close_to_oracle(got, want_f, mag_f, BF16_TOL, "bf16 in vs unrounded inputs")


# --------------------------------------------------------------------------- dense update on the bf16 matrix cores
@pytest.mark.parametrize("n,d1,d2", [(1000, 128, 128), (333, 64, 47), (257, 100, 64), (64, 602, 16), (17, 7, 3), (500, 256, 200)])
@pytest.mark.parametrize("x_bf16,out_bf16", [(False, False), (True, False), (False, True), (True, True)])
def test_dense_update_bf16(gpu, n, d1, d2, x_bf16, out_bf16):
    import torch
    x = gpu.fill_normal((n, d1), seed=50)
    w = gpu.glorot(d1, d2, seed=51)
    wb = to_dev(w).to(torch.bfloat16)
    xd = to_dev(x)
    xr = xd.to(torch.bfloat16)          # what the kernel's own round-to-nearest-even must reproduce
    x_in = xr if x_bf16 else xd
    out = torch.full((n, d2), 3.0, device="cuda", dtype=torch.bfloat16 if out_bf16 else torch.float32)
    gpu.dense_forward_bf16(out, x_in, wb, n, d1, d2)
    gpu.sync()
    xf = xr.to(torch.float32).cpu().numpy()
    wf = wb.to(torch.float32).cpu().numpy()
    want = orc.dense(xf, wf, f64=True)
    mag = np.abs(xf).astype(np.float64) @ np.abs(wf).astype(np.float64)
    got = out.to(torch.float32).cpu().numpy()
    if out_bf16:
        assert_close_to_oracle(got, want, mag + np.abs(want) * 400, FP32_TOL, "bf16 out: fp32 result rounded to bf16")
    else:
        assert_close_to_oracle(got, want, mag, FP32_TOL, "bf16 MFMA vs the same rounded inputs")
    # against the unrounded inputs: the bf16 tolerance
    want_f = orc.dense(x, w, f64=True)
    mag_f = np.abs(x).astype(np.float64) @ np.abs(w).astype(np.float64)
    assert_close_to_oracle(got, want_f, mag_f, BF16_TOL, "bf16 MFMA vs unrounded inputs")


@pytest.mark.parametrize("n,d1,d2,ld_x,ld_out,relu", [(4096, 128, 128, 0, 0, False), (5003, 128, 128, 0, 0, True), (70001, 128, 64, 132, 72, False),
                                                     (4099, 64, 128, 0, 136, True), (9000, 64, 64, 68, 0, False)])
def test_dense_update_bf16_in_whole_lines(gpu, n, d1, d2, ld_x, ld_out, relu):
    """fp32 rows of 64 or 128 to bf16 rows of 64 or 128, 4096 rows and more: the kernel that reads and writes whole rows through
    LDS, takes its tiles in launch order and W from the image a small kernel prepares.  Ragged row counts (the last
    workgroup and the last tile are partial), padded pitches, row scale and ReLU; two calls in a row with different W (the
    image is rewritten per call); rows past n and the pitch padding stay untouched."""
    import torch
    x = gpu.fill_normal((n, d1), seed=60)
    rs = (np.abs(gpu.fill_normal((n,), seed=61)) + 0.5).astype(np.float32)
    px, po = ld_x or d1, ld_out or d2
    xd = torch.zeros((n, px), device="cuda")
    xd[:, :d1] = to_dev(x)
    xr = xd[:, :d1].to(torch.bfloat16).to(torch.float32).cpu().numpy()
    for seed in (62, 63):
        w = gpu.glorot(d1, d2, seed=seed)
        wb = to_dev(w).to(torch.bfloat16)
        wf = wb.to(torch.float32).cpu().numpy()
        out = torch.full((n + 3, po), 3.0, device="cuda", dtype=torch.bfloat16)
        gpu.dense_forward_bf16(out, xd, wb, n, d1, d2, ld_x=px, ld_out=po, row_scale=to_dev(rs), relu=relu)
        gpu.sync()
        want = orc.dense(xr, wf, f64=True) * rs[:, None].astype(np.float64)
        mag = (np.abs(xr).astype(np.float64) @ np.abs(wf).astype(np.float64)) * rs[:, None]
        if relu:
            want = np.maximum(want, 0.0)
        got = out.to(torch.float32).cpu().numpy()
        assert_close_to_oracle(got[:n, :d2], want, mag + np.abs(want) * 400, FP32_TOL, "whole-line bf16 update, W seed %d" % seed)
        assert np.all(got[n:] == 3.0) and np.all(got[:, d2:] == 3.0)


# --------------------------------------------------------------------------- softmax inside the aggregation
def _softmax_want(sh, xl, x, dim, s):
    """softmax_forward(aggregate(...)) as the reference runs them back to back (src/mgg_np_div_mem.cu:221-225), in double."""
    want, mag = oracle_agg(sh, xl, x, dim, rs_out=s)
    w = want.astype(np.float64)
    e = np.exp(w - w.max(1, keepdims=True))
    return e / e.sum(1, keepdims=True), mag


@pytest.mark.parametrize("dim,ld", [(16, 16), (41, 41), (41, 48), (47, 47), (100, 100), (7, 7)])
@pytest.mark.parametrize("path", ["plain", "blocked", "core", "core+blocked"])
def test_softmax_epilogue_on_every_path(gpu, rmat_graph, dim, ld, path):
    """MGGX_AGG_SOFTMAX: rows finished inside a slot, across the wavefronts of a workgroup, across workgroups (tiny
    workgroups force long carry chains), rows without neighbors, the column-blocked finish and both dense-core finishes
    must all give softmax(row scale x sum) -- against the oracle's aggregation followed by a softmax in double."""
    import torch
    if path.startswith("core") and dim > 64:
        pytest.skip("the dense core takes rows of at most 64 columns")
    V, ptr0, col0 = rmat_graph
    if path == "core+blocked":  # dense enough that what the core leaves still has long rows per column block
        V = 4000
        ptr0, col0 = gpu.gen_rmat(12, V, 1_500_000, seed=15)
    # a few rows without neighbors, so the empty-row branch runs
    deg = np.diff(ptr0)
    keep = np.ones(V, bool)
    keep[[5, 77, V - 1]] = False
    ptr = np.zeros(V + 1, np.int32)
    ptr[1:] = np.cumsum(np.where(keep, deg, 0))
    col = np.concatenate([col0[ptr0[v]:ptr0[v + 1]] for v in range(V) if keep[v]]).astype(np.int32)
    sh = share_of(ptr, col, V, 1, 0)
    x = (gpu.fill_normal((V, dim), seed=300 + dim) * 0.3).astype(np.float32)
    s = (1.0 / np.sqrt(np.maximum(np.diff(ptr), 1))).astype(np.float32)
    want, mag = _softmax_want(sh, x, x, dim, s)
    xp = np.zeros((V, ld), np.float32)
    xp[:, :dim] = x
    d_ptr, d_col, d_x, d_s = to_dev(ptr), to_dev(col), to_dev(xp), to_dev(s)
    z, zc = torch.zeros(V + 1, dtype=torch.int32, device="cuda"), torch.zeros(1, dtype=torch.int32, device="cuda")
    blk = 1500 if "blocked" in path else -1
    core = 1024 if path.startswith("core") else -1
    for ps, wpb, dist in [(16, 4, 2), (4, 1, 1), (16, 8, 16)]:
        out = torch.full((V, ld), 7.5, device="cuda")
        gpu.mgg_SAG_np_div(out, d_x, d_ptr, d_col, z, zc, 0, V, dim, V, 0, ps, wpb, dist, ld_in=ld, ld_out=ld, row_scale_out=d_s, softmax=True,
                           col_block_rows=blk, core_rows=core)
        gpu.sync()
        k = gpu.last_agg_kernel()
        assert ("core=1024" in k) == (core > 0) and (("blocks=1 " in k + " ") == (blk < 0)), k
        if path == "core+blocked":
            assert "merged_finish" in k
        got = out.cpu().numpy()
        # d softmax_i / d logit_j is bounded by 1/4: an error of FP32_TOL * mag in the logits gives at most that in the output
        bound = FP32_TOL * (mag.max(1, keepdims=True) + 1.0)
        assert np.all(np.abs(got[:, :dim] - want) <= bound), (path, dim, ps, wpb, dist, float(np.abs(got[:, :dim] - want).max()))
        assert np.allclose(got[:, :dim].sum(1), 1.0, atol=1e-5)
        if ld > dim:
            assert np.all(got[:, dim:] == 7.5)  # padding columns are not touched
        assert np.allclose(got[5, :dim], 1.0 / dim, atol=1e-7)  # a row without neighbors: uniform
    gpu.forget(d_ptr)
