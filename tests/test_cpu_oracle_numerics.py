"""Pins the floating-point half of the CPU oracle without the reference: closed forms, brute force on small
inputs, library routines (numpy matmul, scipy softmax) and invariants a plausible mistake would break (a dropped
remote half, a wrong local index base, a transposed weight, a missing self term)."""
import numpy as np
import pytest
import scipy.sparse as sp
import scipy.special

from mgg_osdi23_amd import host
from oracle import orc


def graph(n=300, draws=4000, seed=3):
    scale = int(np.ceil(np.log2(n)))
    return host.gen_rmat(scale, n, draws, seed=seed)


def share(ptr, col, n, num_gpus, pe):
    npp, lb, ub = orc.range_partition(n, num_gpus, pe)
    lp, rp, lc, rc = orc.split_csr(ptr, col, lb, ub)
    return npp, lb, ub, lp, lc, rp, rc


@pytest.mark.parametrize("num_gpus,pe", [(1, 0), (3, 0), (3, 1), (3, 2)])
@pytest.mark.parametrize("f64", [True, False])
def test_aggregation_is_the_sparse_matrix_product(num_gpus, pe, f64):
    n, dim = 300, 7
    ptr, col = graph(n)
    x = host.fill_normal((num_gpus * -(-n // num_gpus), dim), seed=1)  # padded global table
    npp, lb, ub, lp, lc, rp, rc = share(ptr, col, n, num_gpus, pe)
    A = sp.csr_matrix((np.ones(len(col)), col, ptr), shape=(n, x.shape[0]))
    want = (A[lb:ub] @ x.astype(np.float64))
    got = orc.sag_np_div(x[lb:lb + npp], x, lp, lc, rp, rc, lb, ub, dim, npp, f64=f64, ps=4, wpb=3, dist=2)
    assert np.allclose(got, want, rtol=1e-5, atol=1e-5)
    # a local table that is NOT a slice of the remote one: local rows must come from it, remote rows from the other
    xl = host.fill_normal((npp, dim), seed=2)
    Al = sp.csr_matrix((np.ones(len(lc)), lc - lb, lp), shape=(ub - lb, npp))
    Ar = sp.csr_matrix((np.ones(len(rc)), rc, rp), shape=(ub - lb, x.shape[0]))
    want = Al @ xl.astype(np.float64) + Ar @ x.astype(np.float64)
    got = orc.sag_np_div(xl, x, lp, lc, rp, rc, lb, ub, dim, npp, f64=f64)
    assert np.allclose(got, want, rtol=1e-5, atol=1e-5)


def test_all_ones_and_one_hot_closed_forms():
    n, dim = 200, 4
    ptr, col = graph(n, 3000, seed=5)
    npp, lb, ub, lp, lc, rp, rc = share(ptr, col, n, 2, 1)
    ones = np.ones((2 * npp, dim), np.float32)
    deg = (np.diff(lp) + np.diff(rp)).astype(np.float32)
    for f64 in (True, False):
        got = orc.sag_np_div(ones[:npp], ones, lp, lc, rp, rc, lb, ub, dim, npp, f64=f64)
        assert np.array_equal(got, np.repeat(deg[:, None], dim, 1))
        got = orc.sag_np_div(ones[:npp], ones, lp, lc, rp, rc, lb, ub, dim, npp, f64=f64, flags=orc.GIN, eps=0.5)
        assert np.array_equal(got, np.repeat((deg + 1.5)[:, None], dim, 1))
    eye = np.eye(2 * npp, dtype=np.float32)
    got = orc.sag_np_div(eye[lb:lb + npp], eye, lp, lc, rp, rc, lb, ub, 2 * npp, npp)
    A = sp.csr_matrix((np.ones(len(col), np.float32), col, ptr), shape=(n, 2 * npp)).toarray()
    assert np.array_equal(got, A[lb:ub])


def test_knobs_do_not_change_the_sum():
    n, dim = 400, 16
    ptr, col = graph(n, 9000, seed=6)
    x = host.fill_normal((n, dim), seed=3)
    base = orc.sag_np_div(x, x, ptr, col, None, None, 0, n, dim, n, f64=True)
    mag = orc.sag_np_div_rows(np.arange(n, dtype=np.int32), x, x, ptr, col, None, None, 0, n, dim, n, abs_sum=True)
    for ps, wpb, dist in [(1, 1, 1), (16, 4, 1), (16, 8, 16), (4, 16, 2), (65536, 1, 1)]:
        got = orc.sag_np_div(x, x, ptr, col, None, None, 0, n, dim, n, f64=False, ps=ps, wpb=wpb, dist=dist)
        assert np.all(np.abs(got.astype(np.float64) - base) <= 1e-5 * mag + 1e-30), (ps, wpb, dist)
    # neighbor order inside a row does not matter either (sum is commutative)
    rng = np.random.default_rng(0)
    col2 = col.copy()
    for r in range(n):
        rng.shuffle(col2[ptr[r]:ptr[r + 1]])
    got = orc.sag_np_div(x, x, ptr, col2, None, None, 0, n, dim, n, f64=True)
    assert np.all(np.abs(got.astype(np.float64) - base) <= 1e-6 * mag + 1e-30)


def test_options_accumulate_gin_scales_rows_subset():
    n, dim = 250, 5
    ptr, col = graph(n, 3000, seed=8)
    x = host.fill_normal((n, dim), seed=4)
    A = sp.csr_matrix((np.ones(len(col)), col, ptr), shape=(n, n))
    Ax = A @ x.astype(np.float64)
    prev = host.fill_normal((n, dim), seed=5)
    got = orc.sag_np_div(x, x, ptr, col, None, None, 0, n, dim, n, flags=orc.ACCUMULATE, out=prev.copy())
    assert np.allclose(got, prev + Ax, rtol=1e-5, atol=1e-5)
    got = orc.sag_np_div(x, x, ptr, col, None, None, 0, n, dim, n, flags=orc.GIN, eps=0.25)
    assert np.allclose(got, 1.25 * x + Ax, rtol=1e-5, atol=1e-5)
    s = host.fill_uniform((n,), 0.2, 1.5, seed=6)
    got = orc.sag_np_div(x, x, ptr, col, None, None, 0, n, dim, n, rs_in=s, rs_out=s)
    want = s[:, None] * (A @ (s[:, None] * x.astype(np.float64)))
    assert np.allclose(got, want, rtol=1e-5, atol=1e-5)
    rows = np.array([0, 17, 249, 100], np.int32)
    sub = orc.sag_np_div_rows(rows, x, x, ptr, col, None, None, 0, n, dim, n)
    assert np.allclose(sub, Ax[rows], rtol=1e-5, atol=1e-5)
    mag = orc.sag_np_div_rows(rows, x, x, ptr, col, None, None, 0, n, dim, n, abs_sum=True)
    assert np.allclose(mag, (A @ np.abs(x).astype(np.float64))[rows], rtol=1e-5)


def test_explicit_parts_and_spmm_equal_the_serial_reference_sum():
    n, dim = 300, 6
    ptr, col = graph(n, 5000, seed=9)
    x = host.fill_normal((n, dim), seed=7)
    ref = orc.sag_ref(x, ptr, col)
    for ps in (1, 5, 16):
        pp, p2n, _ = orc.build_part(ptr, n, ps)
        # the terminal entry is present here because every row has its self loop
        got = orc.sag_parts(x, col, pp, p2n, 0, dim, np.zeros((n, dim), np.float32))
        assert np.allclose(got, ref, rtol=1e-5, atol=1e-5)
        got = orc.spmm(x, ptr, col, dim, ps, 4, np.zeros((n, dim), np.float32))
        assert np.allclose(got, ref, rtol=1e-5, atol=1e-5)
    # lowbound: ids are global, the table is the rank's own
    npp, lb, ub, lp, lc, rp, rc = share(ptr, col, n, 2, 1)
    pp, p2n, _ = orc.build_part(lp, ub - lb, 4)
    got = orc.sag_parts(np.ascontiguousarray(x[lb:ub]), lc, pp, p2n, lb, dim, np.zeros((ub - lb, dim), np.float32))
    Al = sp.csr_matrix((np.ones(len(lc)), lc - lb, lp), shape=(ub - lb, ub - lb))
    assert np.allclose(got, Al @ x[lb:ub].astype(np.float64), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("n,d1,d2", [(50, 602, 16), (33, 16, 41), (20, 1, 1), (7, 100, 600)])
def test_dense_is_x_times_w(n, d1, d2):
    x = host.fill_normal((n, d1), seed=1)
    w = host.glorot(d1, d2, seed=2)
    want = x.astype(np.float64) @ w.astype(np.float64)
    assert np.allclose(orc.dense(x, w, f64=True), want, rtol=1e-6, atol=1e-6)
    assert np.allclose(orc.dense(x, w, f64=False), want, rtol=1e-4, atol=1e-4)
    # all-ones inputs (the reference's own initialisation): every entry equals d1
    assert np.array_equal(orc.dense(np.ones((n, d1), np.float32), np.ones((d1, d2), np.float32)), np.full((n, d2), d1, np.float32))
    # a non-symmetric W catches a transposed operand
    if d1 == d2 == 1:
        return
    e = np.zeros((d1, d2), np.float32)
    e[0, d2 - 1] = 1.0
    got = orc.dense(x, e)
    assert np.array_equal(got[:, d2 - 1], x[:, 0]) and np.count_nonzero(got[:, :d2 - 1]) == 0


def test_softmax_rows():
    x = host.fill_normal((40, 41), seed=3) * 10
    got = orc.softmax_rows(x)
    assert np.allclose(got, scipy.special.softmax(x.astype(np.float64), axis=1), rtol=1e-6, atol=1e-9)
    assert np.allclose(got.sum(1), 1.0, atol=1e-6)
    assert np.allclose(orc.softmax_rows(x + 1000.0), got, rtol=1e-4, atol=1e-7)  # shift invariance, no overflow


def test_gcn_forward_wiring_all_ones():
    """All-ones X and W: Y1 = in, H1 = in*deg, Y2 = hidden*H1, H2[v] = hidden*in*sum_{u in N(v)} deg(u) -- integers."""
    n, in_dim, hidden, out_dim = 120, 6, 4, 3
    ptr, col = graph(n, 900, seed=10)
    X = np.ones((n, in_dim), np.float32)
    W1 = np.ones((in_dim, hidden), np.float32)
    W2 = np.ones((hidden, out_dim), np.float32)
    A = sp.csr_matrix((np.ones(len(col)), col, ptr), shape=(n, n))
    deg = np.asarray(A.sum(1)).ravel()
    for f64 in (True, False):
        P, H2, H1 = orc.gcn2_forward(X, W1, W2, ptr, col, None, None, 0, n, n, f64=f64)
        assert np.array_equal(H1, np.repeat((in_dim * deg)[:, None], hidden, 1).astype(np.float32))
        assert np.array_equal(H2, np.repeat((hidden * in_dim * (A @ deg))[:, None], out_dim, 1).astype(np.float32))
        assert np.allclose(P, 1.0 / out_dim)
    # general inputs against scipy/numpy, with the symmetric normalisation
    X = host.fill_normal((n, in_dim), seed=1)
    W1 = host.glorot(in_dim, hidden, seed=2)
    W2 = host.glorot(hidden, out_dim, seed=3)
    s = 1.0 / np.sqrt(deg)
    An = sp.diags(s) @ A @ sp.diags(s)
    H1w = An @ (X.astype(np.float64) @ W1)
    H2w = An @ (H1w @ W2)
    P, H2, H1 = orc.gcn2_forward(X, W1, W2, ptr, col, None, None, 0, n, n, rs=s.astype(np.float32))
    assert np.allclose(H1, H1w, rtol=1e-4, atol=1e-5) and np.allclose(H2, H2w, rtol=1e-4, atol=1e-5)
    assert np.allclose(P, scipy.special.softmax(H2w, axis=1), rtol=1e-4, atol=1e-6)


def test_gin_forward_wiring():
    n, in_dim, hidden, out_dim, L, eps = 90, 5, 4, 3, 5, 0.5
    ptr, col = graph(n, 600, seed=11)
    A = sp.csr_matrix((np.ones(len(col)), col, ptr), shape=(n, n))
    X = host.fill_normal((n, in_dim), seed=1)
    Ws = [host.glorot(in_dim, hidden, seed=2)] + [host.glorot(hidden, hidden, seed=3 + i) for i in range(L - 1)] + \
         [host.glorot(hidden, out_dim, seed=20)]
    Y = X.astype(np.float64) @ Ws[0]
    for l in range(1, L + 1):
        Y = ((1 + eps) * Y + A @ Y) @ Ws[l]
    P, logits = orc.gin_forward(X, Ws, ptr, col, None, None, 0, n, n, eps)
    assert np.allclose(logits, Y, rtol=1e-4, atol=1e-4)
    assert np.allclose(P, scipy.special.softmax(Y, axis=1), rtol=1e-3, atol=1e-6)
