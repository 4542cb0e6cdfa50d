"""Cached plans against the caller's memory: arrays rewritten in place without mggx_forget, captured graphs that outlive
a growing workspace, first uses inside a capture."""
import numpy as np
import pytest

from oracle import orc
from tests.util import FP32_TOL, assert_close_to_oracle, to_dev

pytestmark = pytest.mark.gpu


def _agg(gpu, out, x, d_ptr, d_col, V, dim, ps=16, wpb=4, dist=2, **kw):
    import torch
    zp = torch.zeros(V + 1, dtype=torch.int32, device="cuda")
    zc = torch.zeros(1, dtype=torch.int32, device="cuda")
    _agg.keep = (zp, zc)
    gpu.mgg_SAG_np_div(out, x, d_ptr, d_col, zp, zc, 0, V, dim, V, 0, ps, wpb, dist, **kw)


def _want(x, ptr, col, V, dim):
    want = orc.sag_np_div(x, x, ptr, col, None, None, 0, V, dim, V)
    mag = orc.sag_np_div_rows(np.arange(V, dtype=np.int32), x, x, ptr, col, None, None, 0, V, dim, V, abs_sum=True)
    return want, mag


@pytest.fixture(params=[1, 2])
def check_level(gpu, request):
    """Both levels of the content check: live edge counts inside the kernels; the fingerprint kernel on top."""
    gpu.set_plan_check(request.param)
    yield request.param
    gpu.set_plan_check(1)


@pytest.mark.parametrize("core_rows", [-1, 1024])
def test_csr_rewritten_in_place_without_forget(gpu, core_rows, check_level):
    """A different graph written into the same device arrays, and no mggx_forget: the cached plan (and dense-core plan)
    no longer fits.  The call must give an error or the right answer, never a sum through the stale plan."""
    import torch
    V, dim = 6000, 16
    ptr_a, col_a = gpu.gen_rmat(13, V, 200_000, seed=1)
    ptr_b, col_b = gpu.gen_rmat(13, V, 120_000, seed=2)
    assert len(col_b) < len(col_a)
    x = gpu.fill_normal((V, dim), seed=3)
    d_x = to_dev(x)
    d_ptr, d_col = to_dev(ptr_a), to_dev(col_a)
    zp = torch.zeros(V + 1, dtype=torch.int32, device="cuda")
    zc = torch.zeros(1, dtype=torch.int32, device="cuda")
    call = lambda out: gpu.mgg_SAG_np_div(out, d_x, d_ptr, d_col, zp, zc, 0, V, dim, V, 0, 16, 4, 2, core_rows=core_rows)
    out = torch.empty(V, dim, device="cuda")
    call(out)
    gpu.sync()
    want, mag = _want(x, ptr_a, col_a, V, dim)
    assert_close_to_oracle(out.cpu().numpy(), want, mag, FP32_TOL, "graph A")
    # graph B into the same arrays, behind the library's back
    d_ptr.copy_(torch.from_numpy(ptr_b))
    d_col[: len(col_b)].copy_(torch.from_numpy(col_b))
    torch.cuda.synchronize()
    want, mag = _want(x, ptr_b, col_b, V, dim)
    out.fill_(-7.0)
    errors = 0
    for attempt in range(3):
        try:
            call(out)
            gpu.sync()
        except gpu.MggxError as e:
            assert "changed" in str(e)
            errors += 1
            # the stale plan's kernels did nothing
            assert bool((out == -7.0).all()), "kernels of a stale plan wrote to the output"
            continue
        break
    else:
        raise AssertionError("no call succeeded after the rewrite")
    assert errors == 1
    assert_close_to_oracle(out.cpu().numpy(), want, mag, FP32_TOL, "graph B after the rewrite")
    gpu.forget(d_ptr)


def test_same_edge_count_other_graph_needs_the_fingerprint(gpu):
    """Level 2 also catches a rewrite that keeps the edge count (here: the rows of the graph rotated by one)."""
    import torch
    V, dim = 3000, 16
    ptr, col = gpu.gen_rmat(12, V, 50_000, seed=11)
    deg = np.diff(ptr)
    deg_b = np.roll(deg, 1)
    ptr_b = np.zeros(V + 1, np.int32)
    ptr_b[1:] = np.cumsum(deg_b)
    assert ptr_b[-1] == ptr[-1] and not np.array_equal(ptr_b, ptr)
    x = gpu.fill_normal((V, dim), seed=3)
    d_x, d_ptr, d_col = to_dev(x), to_dev(ptr), to_dev(col)
    zp, zc = torch.zeros(V + 1, dtype=torch.int32, device="cuda"), torch.zeros(1, dtype=torch.int32, device="cuda")
    out = torch.empty(V, dim, device="cuda")
    call = lambda: gpu.mgg_SAG_np_div(out, d_x, d_ptr, d_col, zp, zc, 0, V, dim, V, 0, 16, 4, 2)
    gpu.set_plan_check(2)
    try:
        call()
        gpu.sync()
        d_ptr.copy_(torch.from_numpy(ptr_b))
        torch.cuda.synchronize()
        out.fill_(-7.0)
        with pytest.raises(gpu.MggxError, match="changed"):
            call()
            gpu.sync()
        assert bool((out == -7.0).all())
        call()
        gpu.sync()
        want, mag = _want(x, ptr_b, col, V, dim)
        assert_close_to_oracle(out.cpu().numpy(), want, mag, FP32_TOL, "rows rotated")
    finally:
        gpu.set_plan_check(1)
        gpu.forget(d_ptr)


def test_explicit_partition_arrays_rewritten_in_place(gpu, check_level):
    import torch
    V, dim, ps = 4000, 16, 8
    ptr_a, col_a = gpu.gen_rmat(12, V, 60_000, seed=4)
    ptr_b, col_b = gpu.gen_rmat(12, V, 30_000, seed=5)
    x = gpu.fill_normal((V, dim), seed=6)
    pa, p2na, _ = orc.build_part(ptr_a, V, ps)
    pb, p2nb, _ = orc.build_part(ptr_b, V, ps)
    assert len(p2nb) < len(p2na) and len(col_b) < len(col_a)
    d_ptr, d_col, d_pp, d_p2n, d_x = to_dev(ptr_a), to_dev(col_a), to_dev(pa), to_dev(p2na), to_dev(x)
    out = torch.zeros(V, dim, device="cuda")
    gpu.SAG_host(out, d_x, d_ptr, d_col, d_pp, d_p2n, 0, V, len(p2na), ps, dim, 32, 4, 1)
    gpu.sync()
    assert np.allclose(out.cpu().numpy(), orc.sag_ref(x, ptr_a, col_a), rtol=1e-4, atol=1e-4)
    # same arrays, same partition count passed, other contents
    d_ptr.copy_(torch.from_numpy(ptr_b))
    d_col[: len(col_b)].copy_(torch.from_numpy(col_b))
    d_pp.zero_()
    d_pp[: len(pb)].copy_(torch.from_numpy(pb))
    d_p2n[: len(p2nb)].copy_(torch.from_numpy(p2nb))
    torch.cuda.synchronize()
    out.fill_(-7.0)
    with pytest.raises(gpu.MggxError, match="changed"):
        gpu.SAG_host(out, d_x, d_ptr, d_col, d_pp, d_p2n, 0, V, len(p2na), ps, dim, 32, 4, 1)
        gpu.sync()
    assert bool((out == -7.0).all())
    gpu.forget(d_ptr)


def test_captured_graph_survives_workspace_growth_and_cache_pressure(gpu):
    """A captured forward keeps pointing at the plan and the scratch block of its capture.  Later eager calls that need a
    larger block, and enough other plans to fill the cache, must not free what the graph uses."""
    import torch
    V, dim = 5000, 16
    ptr, col = gpu.gen_rmat(13, V, 150_000, seed=9)
    x = gpu.fill_normal((V, dim), seed=1)
    d_ptr, d_col, d_x = to_dev(ptr), to_dev(col), to_dev(x)
    zp, zc = torch.zeros(V + 1, dtype=torch.int32, device="cuda"), torch.zeros(1, dtype=torch.int32, device="cuda")
    out = torch.empty(V, dim, device="cuda")
    big_V = 60_000
    bptr, bcol = gpu.gen_rmat(16, big_V, 1_500_000, seed=10)
    d_bptr, d_bcol = to_dev(bptr), to_dev(bcol)
    bzp = torch.zeros(big_V + 1, dtype=torch.int32, device="cuda")
    d_bx, bout = to_dev(gpu.fill_normal((big_V, 64), seed=2)), torch.empty(big_V, 64, device="cuda")
    call = lambda: gpu.mgg_SAG_np_div(out, d_x, d_ptr, d_col, zp, zc, 0, V, dim, V, 0, 16, 4, 2)
    gpu.release_cached()  # start from an empty workspace, so the capture below pins a small one
    side = torch.cuda.Stream()
    try:
        with torch.cuda.stream(side):
            gpu.use_torch_stream()
            call()
            side.synchronize()
            want = out.clone()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                gpu.use_torch_stream()
                call()
                # a first use inside the capture is refused before anything is launched or allocated
                with pytest.raises(gpu.MggxError, match="capture"):
                    gpu.mgg_SAG_np_div(out, d_x, d_ptr, d_col, zp, zc, 0, V, dim, V, 0, 7, 4, 2)
            before = gpu.cache_stats()
            # eager: a much larger call (the workspace must grow) and 20 other plans (the cache holds 16)
            gpu.use_torch_stream()
            gpu.mgg_SAG_np_div(bout, d_bx, d_bptr, d_bcol, bzp, zc, 0, big_V, 64, big_V, 0, 16, 1, 1)
            for ps in range(20, 40):
                gpu.mgg_SAG_np_div(bout, d_bx, d_bptr, d_bcol, bzp, zc, 0, big_V, 64, big_V, 0, ps, 8, 1)
            side.synchronize()
            after = gpu.cache_stats()
            assert after["workspace_bytes"] > before["workspace_bytes"]
            assert after["retired_bytes"] >= before["workspace_bytes"] > 0
            for i in range(2):
                out.fill_(-1.0)
                graph.replay()
                side.synchronize()
                assert torch.equal(out, want), "replay %d after the workspace grew differs" % i
    finally:
        torch.cuda.synchronize()
        gpu.use_torch_stream()
        gpu.release_cached()


@pytest.mark.parametrize("core_rows", [-1, 1024])
def test_captured_graph_survives_forget(gpu, core_rows):
    """mggx_forget on a CSR array whose plans a captured graph still launches: the records leave the lookup tables, but
    their device blocks (descriptors, row offsets, the dense-core lists, the fingerprint word) are retired, not freed -- a
    replay reads the old plan, never freed memory."""
    import torch
    V, dim = 6000, 16
    ptr, col = gpu.gen_rmat(13, V, 200_000, seed=21)
    x = gpu.fill_normal((V, dim), seed=1)
    d_ptr, d_col, d_x = to_dev(ptr), to_dev(col), to_dev(x)
    zp, zc = torch.zeros(V + 1, dtype=torch.int32, device="cuda"), torch.zeros(1, dtype=torch.int32, device="cuda")
    out = torch.empty(V, dim, device="cuda")
    call = lambda: gpu.mgg_SAG_np_div(out, d_x, d_ptr, d_col, zp, zc, 0, V, dim, V, 0, 16, 4, 2, core_rows=core_rows)
    gpu.release_cached()
    gpu.set_plan_check(2)  # the fingerprint kernel is captured too and writes the record's verdict word on every replay
    side = torch.cuda.Stream()
    try:
        with torch.cuda.stream(side):
            gpu.use_torch_stream()
            call()
            side.synchronize()
            want = out.clone()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                gpu.use_torch_stream()
                call()
            gpu.use_torch_stream()
            before = gpu.cache_stats()
            assert before["plans"] >= 1 and before["retired_bytes"] == 0
            gpu.forget(d_ptr)
            after = gpu.cache_stats()
            assert after["plans"] == 0 and after["core_plans"] == 0
            assert after["retired_bytes"] >= before["plan_bytes"] + before["core_plan_bytes"] > 0
            # memory handed out now must not be what the graph reads
            junk = [torch.full((1 << 20,), -1, dtype=torch.int32, device="cuda") for _ in range(8)]
            for i in range(2):
                out.fill_(-1.0)
                graph.replay()
                side.synchronize()
                assert torch.equal(out, want), "replay %d after mggx_forget differs" % i
            del junk
            # an eager call afterwards builds fresh records and gives the same sums
            out.fill_(-1.0)
            call()
            side.synchronize()
            assert torch.equal(out, want)
    finally:
        torch.cuda.synchronize()
        gpu.use_torch_stream()
        gpu.set_plan_check(1)
        gpu.release_cached()
    assert gpu.cache_stats()["retired_bytes"] == 0


def test_plans_go_with_their_graph_record(gpu):
    """The content check lives with the graph record (32 cached).  A dense-core plan must not outlive the record it was
    built under: after 33 other CSR sets have passed through, the first set's arrays are rewritten in place with another
    graph of another size; the next call makes a fresh record from what is there now -- and must not find the old graph's
    dense-core plan (which holds its own copy of the old remaining CSR) by address."""
    import torch
    V, dim = 6000, 16
    ptr_a, col_a = gpu.gen_rmat(13, V, 200_000, seed=31)
    ptr_b, col_b = gpu.gen_rmat(13, V, 120_000, seed=32)
    assert len(col_b) < len(col_a)
    x = gpu.fill_normal((V, dim), seed=3)
    d_x, d_ptr, d_col = to_dev(x), to_dev(ptr_a), to_dev(col_a)
    zp, zc = torch.zeros(V + 1, dtype=torch.int32, device="cuda"), torch.zeros(1, dtype=torch.int32, device="cuda")
    out = torch.empty(V, dim, device="cuda")
    call = lambda: gpu.mgg_SAG_np_div(out, d_x, d_ptr, d_col, zp, zc, 0, V, dim, V, 0, 16, 4, 2, core_rows=1024)
    gpu.release_cached()
    call()
    gpu.sync()
    assert "core=1024" in gpu.last_agg_kernel() and gpu.cache_stats()["core_plans"] == 1
    want, mag = _want(x, ptr_a, col_a, V, dim)
    assert_close_to_oracle(out.cpu().numpy(), want, mag, FP32_TOL, "graph A")
    # 33 other CSR sets (no dense core: core plans are only displaced by other core plans)
    n = 300
    sp, sc = gpu.gen_rmat(9, n, 3000, seed=33)
    others = [(to_dev(sp), to_dev(sc)) for _ in range(33)]
    szp, sx, so = torch.zeros(n + 1, dtype=torch.int32, device="cuda"), to_dev(gpu.fill_normal((n, dim), seed=4)), torch.empty(n, dim, device="cuda")
    for p_, c_ in others:
        gpu.mgg_SAG_np_div(so, sx, p_, c_, szp, zc, 0, n, dim, n, 0, 16, 4, 2, core_rows=-1)
    gpu.sync()
    assert gpu.cache_stats()["core_plans"] == 0, "the dense-core plan outlived its graph record"
    d_ptr.copy_(torch.from_numpy(ptr_b))
    d_col[: len(col_b)].copy_(torch.from_numpy(col_b))
    torch.cuda.synchronize()
    out.fill_(-7.0)
    call()
    gpu.sync()
    want, mag = _want(x, ptr_b, col_b, V, dim)
    assert_close_to_oracle(out.cpu().numpy(), want, mag, FP32_TOL, "graph B in the arrays of graph A, new record")
    for p_, _c in others:
        gpu.forget(p_)
    gpu.forget(d_ptr)


def test_two_records_over_one_row_pointer_array_keep_their_own_plans(gpu):
    """Two CSRs that share the row-pointer array but not the column array are two graph records, each with its own plan:
    alternating between them rebuilds nothing."""
    import torch
    V, dim = 4000, 16
    ptr, col = gpu.gen_rmat(12, V, 60_000, seed=41)
    rng = np.random.default_rng(0)
    col2 = rng.integers(0, V, len(col)).astype(np.int32)
    x = gpu.fill_normal((V, dim), seed=5)
    d_x, d_ptr, d_c1, d_c2 = to_dev(x), to_dev(ptr), to_dev(col), to_dev(col2)
    zp, zc = torch.zeros(V + 1, dtype=torch.int32, device="cuda"), torch.zeros(1, dtype=torch.int32, device="cuda")
    out = torch.empty(V, dim, device="cuda")
    gpu.release_cached()
    for d_c in (d_c1, d_c2):
        gpu.mgg_SAG_np_div(out, d_x, d_ptr, d_c, zp, zc, 0, V, dim, V, 0, 16, 4, 2, core_rows=-1, col_block_rows=-1)
    gpu.sync()
    built = gpu.cache_stats()
    assert built["plans"] == 2
    for d_c, c in ((d_c1, col), (d_c2, col2), (d_c1, col)):
        gpu.mgg_SAG_np_div(out, d_x, d_ptr, d_c, zp, zc, 0, V, dim, V, 0, 16, 4, 2, core_rows=-1, col_block_rows=-1)
        gpu.sync()
        want, mag = _want(x, ptr, c, V, dim)
        assert_close_to_oracle(out.cpu().numpy(), want, mag, FP32_TOL, "shared row pointers")
    now = gpu.cache_stats()
    assert now["plans"] == 2 and now["plan_build_ms"] == built["plan_build_ms"]
    gpu.forget(d_ptr)


# --------------------------------------------------------------------------- dense-core plan built on the GPU
@pytest.mark.parametrize("shape", ["rmat", "ragged", "unsorted_parallel"])
def test_core_plan_built_on_the_gpu_is_the_host_layout(gpu, shape):
    """The plan the aggregation builds on the device (radix sort, counting pass, prefix sums, fill pass) against the host
    builder, whose arrays the CPU tests check against numpy: every array bit for bit."""
    rng = np.random.default_rng(5)
    if shape == "rmat":
        V, lb, core = 9000, 0, 2048
        ptr, col = gpu.gen_rmat(14, V, 400_000, seed=17)
    elif shape == "ragged":  # empty rows, equal degrees (ties by id), a share that starts at lb > 0
        V, lb, core = 3000, 5000, 1024
        deg = rng.integers(0, 40, V)
        deg[rng.random(V) < 0.3] = 0
        deg[:50] = 700
        ptr = np.zeros(V + 1, np.int32)
        ptr[1:] = np.cumsum(deg)
        col = (np.concatenate([np.sort(rng.choice(V, d, replace=False)) for d in deg]) + lb).astype(np.int32)
    else:  # neighbor lists in random order with repeated edges
        V, lb, core = 2500, 0, 512
        deg = rng.integers(1, 300, V)
        ptr = np.zeros(V + 1, np.int32)
        ptr[1:] = np.cumsum(deg)
        col = rng.integers(0, V, int(ptr[-1])).astype(np.int32)
    want = gpu.core_layout(ptr, col, lb, core)
    d_ptr, d_col = to_dev(ptr), to_dev(col)
    got = gpu.core_layout_device(d_ptr, d_col, V, lb, core)
    assert got["core"] == want["core"] and got["core_nnz"] == want["core_nnz"] and got["core_nnz"] > 0
    for k in ("order", "rank", "blk_off", "rem_ptr", "rem_col", "idx"):
        assert np.array_equal(got[k], want[k]), k
    gpu.forget(d_ptr)


def test_core_plan_refuses_ids_outside_the_share(gpu):
    ptr = np.arange(0, 2049 * 4, 4, dtype=np.int32)
    col = np.tile(np.array([0, 1, 2, 5000], np.int32), 2048)  # 5000 is not a row of this share
    d_ptr, d_col = to_dev(ptr), to_dev(col)
    with pytest.raises(gpu.MggxError, match="outside"):
        gpu.core_layout_device(d_ptr, d_col, 2048, 0, 1024)
    gpu.forget(d_ptr)
