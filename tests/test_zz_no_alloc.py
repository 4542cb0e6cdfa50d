"""The aggregation entry point that allocates nothing (mggx_sag_parts_static) against mggx_sag_parts, through the C ABI."""
import numpy as np
import pytest

from oracle import orc
from tests.util import FP32_TOL, assert_close_to_oracle, share_of, to_dev

pytestmark = pytest.mark.gpu


def _case(gpu, V, scale, draws, seed, dim, ps, wpb, dist):
    ptr, col = gpu.gen_rmat(scale, V, draws, seed=seed)
    sh = share_of(ptr, col, V, 2, 1)
    R = sh["ub"] - sh["lb"]
    x = gpu.fill_normal((V, dim), seed=seed + 1)
    xl = np.ascontiguousarray(x[sh["lb"]:sh["ub"]])
    pp, p2n, _ = orc.build_part(sh["ptr_l"], R, ps)
    base = gpu.fill_normal((R, dim), seed=seed + 2)
    args = (to_dev(xl), to_dev(sh["ptr_l"]), to_dev(sh["col_l"]), to_dev(pp), to_dev(p2n), sh["lb"], R, len(p2n), ps, dim, 32, wpb, dist)
    want_dev = to_dev(base)
    gpu.SAG_host(want_dev, *args)
    got_dev = to_dev(base)
    gpu.SAG_host_static(got_dev, *args)
    gpu.sync()
    got, want = got_dev.cpu().numpy(), want_dev.cpu().numpy()
    # same kernels, same order of summation: bit for bit
    assert np.array_equal(got, want), "static entry point differs from mggx_sag_parts (V=%d dim=%d)" % (V, dim)
    # and both against the oracle
    ref = orc.sag_parts(xl, sh["col_l"], pp, p2n, sh["lb"], dim, base.copy())
    only_local = dict(sh, ptr_r=np.zeros(R + 1, np.int32), col_r=np.zeros(0, np.int32))
    rows = np.arange(R, dtype=np.int32)
    mag = orc.sag_np_div_rows(rows, xl, x, only_local["ptr_l"], only_local["col_l"], only_local["ptr_r"], only_local["col_r"],
                              sh["lb"], sh["ub"], dim, sh["npp"], abs_sum=True)
    assert_close_to_oracle(got, ref, mag + np.abs(base), FP32_TOL, "static explicit parts")


def test_static_entry_point_matches_sag_parts_twice(gpu):
    """Two calls in a row through the one static array, the second smaller (what the first left behind must not leak in)."""
    _case(gpu, 40_000, 16, 1_200_000, 3, 16, 16, 4, 2)
    _case(gpu, 3_000, 12, 40_000, 5, 16, 16, 4, 2)
    # other row widths and knobs, again larger then smaller
    _case(gpu, 20_000, 15, 600_000, 7, 41, 8, 8, 1)
    _case(gpu, 500, 9, 3_000, 9, 64, 3, 2, 3)
    # partitions smaller than a slot (several per descriptor, their number left on the device): larger, then smaller
    _case(gpu, 30_000, 15, 800_000, 11, 16, 1, 4, 4)
    _case(gpu, 2_000, 11, 20_000, 13, 41, 5, 4, 1)
    _case(gpu, 700, 10, 5_000, 15, 16, 2, 1, 1)


def test_static_entry_point_runs_under_capture_and_allocates_nothing(gpu):
    """What the entry point exists for: a call launches kernels and nothing else.  It is recorded into a HIP graph on a
    stream in global capture mode -- an allocation, a copy to the host or a synchronisation inside the call would fail the
    capture -- the replays are compared with the eager result, and neither the library's caches nor the device's free
    memory move across an eager call."""
    import torch
    V, dim, ps = 30_000, 16, 16
    ptr, col = gpu.gen_rmat(15, V, 700_000, seed=13)
    x = gpu.fill_normal((V, dim), seed=14)
    pp, p2n, _ = orc.build_part(ptr, V, ps)
    d_x, d_ptr, d_col, d_pp, d_p2n = to_dev(x), to_dev(ptr), to_dev(col), to_dev(pp), to_dev(p2n)
    args = (d_x, d_ptr, d_col, d_pp, d_p2n, 0, V, len(p2n), ps, dim, 32, 4, 2)
    out = torch.zeros(V, dim, device="cuda")
    gpu.SAG_host_static(out, *args)  # code loaded, the array's address looked up
    gpu.sync()
    want = out.clone()
    out.zero_()
    torch.cuda.synchronize()
    stats0, free0 = gpu.cache_stats(), torch.cuda.mem_get_info()[0]  # no torch operation between here and the second reading
    gpu.SAG_host_static(out, *args)
    gpu.sync()
    free1 = torch.cuda.mem_get_info()[0]
    assert free1 == free0, "device memory was allocated or freed across the call"
    assert gpu.cache_stats() == stats0, "the static entry point touched the library's caches"
    assert torch.equal(out, want)
    side = torch.cuda.Stream()
    try:
        with torch.cuda.stream(side):
            gpu.use_torch_stream()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side, capture_error_mode="global"):
                gpu.use_torch_stream()
                gpu.SAG_host_static(out, *args)
            for i in range(3):
                out.zero_()  # the call accumulates into its output
                graph.replay()
                side.synchronize()
                assert torch.equal(out, want), "replay %d differs from the eager call" % i
                gpu.use_torch_stream()
                gpu.SAG_host_static(out, *args)  # eager work between the replays shares the array
                side.synchronize()
    finally:
        torch.cuda.synchronize()
        gpu.use_torch_stream()
    assert gpu.cache_stats() == stats0


def test_static_entry_point_rejects_what_does_not_fit(gpu):
    import torch
    z = torch.zeros(4, dtype=torch.int32, device="cuda")
    f = torch.zeros(16, device="cuda")
    with pytest.raises(gpu.MggxError, match="static scratch"):
        gpu.SAG_host_static(f, f, z, z, z, z, 0, 1 << 20, 1 << 23, 16, 16, 32, 4, 1)  # 128 MiB of descriptors
    # nothing to do: fine
    gpu.SAG_host_static(f, f, z, z, z, z, 0, 0, 0, 16, 16, 32, 4, 1)
    gpu.sync()
