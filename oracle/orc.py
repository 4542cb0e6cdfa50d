"""ctypes access to the CPU oracle (oracle/liborc.so) and, where it was built,
to the reference's own host code (oracle/_ref/libmgg_ref.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
bench.py's cpu_baseline leg -- never by the mgg_osdi23_amd package.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from typing import Optional

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ORC_PATH = os.path.join(HERE, "liborc.so")
REF_PATH = os.path.join(HERE, "_ref", "libmgg_ref.so")

ACCUMULATE = 1
GIN = 2

_orc = None
_ref = None


def build(force: bool = False) -> None:
    """Compiles liborc.so (and _ref when the reference tree is present)."""
    if force or not os.path.exists(ORC_PATH) or os.path.getmtime(ORC_PATH) < os.path.getmtime(os.path.join(HERE, "mgg_oracle.c")):
        subprocess.run(["make", "-C", HERE, "liborc.so"], check=True, stdout=subprocess.DEVNULL)
    if os.path.isdir(os.environ.get("MGG_REFERENCE", "/root/reference")):
        subprocess.run(["make", "-C", HERE, "ref"], check=True, stdout=subprocess.DEVNULL)


def orc() -> C.CDLL:
    global _orc
    if _orc is None:
        if not os.path.exists(ORC_PATH):
            build()
        _orc = C.CDLL(ORC_PATH)
    return _orc


def have_ref() -> bool:
    return os.path.exists(REF_PATH)


def ref() -> C.CDLL:
    global _ref
    if _ref is None:
        _ref = C.CDLL(REF_PATH)
    return _ref


def _i(a: Optional[np.ndarray]):
    if a is None:
        return None
    assert a.dtype == np.int32 and a.flags["C_CONTIGUOUS"], (a.dtype, a.flags)
    return a.ctypes.data_as(C.POINTER(C.c_int))


def _f(a: Optional[np.ndarray]):
    if a is None:
        return None
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def max_threads() -> int:
    return int(orc().orc_max_threads())


# ----------------------------------------------------------------------------- oracle (restatement)
def range_partition(num_nodes, num_gpus, pe):
    npp, lb, ub = C.c_int(), C.c_int(), C.c_int()
    orc().orc_range_partition(num_nodes, num_gpus, pe, C.byref(npp), C.byref(lb), C.byref(ub))
    return npp.value, lb.value, ub.value


def split_csr(ptr, col, lb, ub):
    ptr, col = _i32(ptr), _i32(col)
    nl, nr = C.c_int64(), C.c_int64()
    orc().orc_split_csr(_i(ptr), _i(col), lb, ub, None, None, None, None, C.byref(nl), C.byref(nr))
    lp = np.zeros(ub - lb + 1, np.int32)
    rp = np.zeros(ub - lb + 1, np.int32)
    lc = np.zeros(nl.value, np.int32)
    rc = np.zeros(nr.value, np.int32)
    orc().orc_split_csr(_i(ptr), _i(col), lb, ub, _i(lp), _i(rp), _i(lc), _i(rc), C.byref(nl), C.byref(nr))
    return lp, rp, lc, rc


def build_part(indptr, num_nodes, ps):
    indptr = _i32(indptr)
    n = orc().orc_build_part(_i(indptr), num_nodes, ps, None, None, None)
    pp = np.zeros(n + 1, np.int32)
    p2n = np.zeros(n, np.int32)
    n2p = np.zeros(num_nodes + 2, np.int32)
    orc().orc_build_part(_i(indptr), num_nodes, ps, _i(pp), _i(p2n), _i(n2p))
    return pp, p2n, n2p


def graph_load(beg, csr, weight):
    v, e = C.c_int(), C.c_int()
    rc = orc().orc_graph_load(beg.encode(), csr.encode(), weight.encode(), C.byref(v), C.byref(e), None, None, None)
    if rc:
        raise IOError("orc_graph_load: %d" % rc)
    b = np.zeros(v.value + 1, np.int32)
    c = np.zeros(e.value, np.int32)
    w = np.zeros(e.value, np.int32)
    rc = orc().orc_graph_load(beg.encode(), csr.encode(), weight.encode(), C.byref(v), C.byref(e), _i(b), _i(c), _i(w))
    if rc:
        raise IOError("orc_graph_load: %d" % rc)
    return b, c, w


def mtx_load(path):
    m, l = C.c_int(), C.c_int()
    rc = orc().orc_mtx_load(path.encode(), C.byref(m), C.byref(l), None, None)
    if rc:
        raise IOError("orc_mtx_load: %d" % rc)
    rp = np.zeros(m.value + 1, np.int32)
    ci = np.zeros(l.value, np.int32)
    orc().orc_mtx_load(path.encode(), C.byref(m), C.byref(l), _i(rp), _i(ci))
    return rp, ci


def sag_ref(inp, ptr, col, out=None):
    n = len(ptr) - 1
    dim = inp.shape[1]
    upd = np.zeros((n, dim), np.float32) if out is None else out
    orc().orc_sag_ref(_f(upd), _f(np.ascontiguousarray(inp, np.float32)), _i(_i32(ptr)), _i(_i32(col)), n, dim)
    return upd


def _agg_common(in_local, in_remote, ptr_l, col_l, ptr_r, col_r):
    in_local = np.ascontiguousarray(in_local, np.float32)
    in_remote = in_local if in_remote is None else np.ascontiguousarray(in_remote, np.float32)
    ptr_l, col_l = _i32(ptr_l), _i32(col_l)
    if ptr_r is not None:
        ptr_r, col_r = _i32(ptr_r), _i32(col_r)
    return in_local, in_remote, ptr_l, col_l, ptr_r, col_r


def sag_np_div(in_local, in_remote, ptr_l, col_l, ptr_r, col_r, lb, ub, dim, npp, *, ps=16, wpb=8, dist=1, flags=0,
               eps=0.0, rs_in=None, rs_out=None, f64=True, out=None, ld_in=None, threads=0):
    """Aggregation oracle; f64=True accumulates in double (the tolerance anchor), f64=False follows the
    reference kernel's per-warp fp32 accumulation structure."""
    in_local, in_remote, ptr_l, col_l, ptr_r, col_r = _agg_common(in_local, in_remote, ptr_l, col_l, ptr_r, col_r)
    ld = in_local.shape[1] if ld_in is None else ld_in
    res = np.zeros((ub - lb, dim), np.float32) if out is None else out
    th = threads or max_threads()
    rs_in = None if rs_in is None else np.ascontiguousarray(rs_in, np.float32)
    rs_out = None if rs_out is None else np.ascontiguousarray(rs_out, np.float32)
    if f64:
        orc().orc_sag_np_div_f64(_f(res), _f(in_local), _f(in_remote), _i(ptr_l), _i(col_l), _i(ptr_r), _i(col_r), lb, ub,
                                 dim, C.c_int64(ld), C.c_int64(dim), npp, flags, C.c_float(eps), _f(rs_in), _f(rs_out), th)
    else:
        orc().orc_sag_np_div_f32(_f(res), _f(in_local), _f(in_remote), _i(ptr_l), _i(col_l), _i(ptr_r), _i(col_r), lb, ub,
                                 dim, C.c_int64(ld), C.c_int64(dim), npp, ps, wpb, dist, flags, C.c_float(eps), _f(rs_in),
                                 _f(rs_out), th)
    return res


def sag_np_div_rows(rows, in_local, in_remote, ptr_l, col_l, ptr_r, col_r, lb, ub, dim, npp, *, flags=0, eps=0.0,
                    rs_in=None, rs_out=None, ld_in=None, abs_sum=False, threads=0):
    """Selected rows only (double accumulation) -> [len(rows) x dim]; abs_sum=True gives sum |terms| instead."""
    in_local, in_remote, ptr_l, col_l, ptr_r, col_r = _agg_common(in_local, in_remote, ptr_l, col_l, ptr_r, col_r)
    rows = _i32(rows)
    ld = in_local.shape[1] if ld_in is None else ld_in
    res = np.zeros((len(rows), dim), np.float32)
    th = threads or max_threads()
    rs_in = None if rs_in is None else np.ascontiguousarray(rs_in, np.float32)
    rs_out = None if rs_out is None else np.ascontiguousarray(rs_out, np.float32)
    fn = orc().orc_sag_np_div_abs_sum if abs_sum else orc().orc_sag_np_div_rows_f64
    fn(_f(res), _i(rows), len(rows), _f(in_local), _f(in_remote), _i(ptr_l), _i(col_l), _i(ptr_r), _i(col_r), lb, ub, dim,
       C.c_int64(ld), C.c_int64(dim), npp, flags, C.c_float(eps), _f(rs_in), _f(rs_out), th)
    return res


def sag_parts(inp, col, part_ptr, part2node, lowbound, dim, out):
    orc().orc_sag_parts_f32(_f(out), _f(np.ascontiguousarray(inp, np.float32)), _i(_i32(col)), _i(_i32(part_ptr)),
                            _i(_i32(part2node)), lowbound, len(part2node), dim)
    return out


def spmm(inp, ptr, col, dim, ps, wpb, out):
    orc().orc_spmm_f32(_f(out), _f(np.ascontiguousarray(inp, np.float32)), _i(_i32(ptr)), _i(_i32(col)), len(ptr) - 1, dim,
                       ps, wpb)
    return out


def dense(X, W, *, f64=True, threads=0):
    X = np.ascontiguousarray(X, np.float32)
    W = np.ascontiguousarray(W, np.float32)
    n, d1 = X.shape
    d2 = W.shape[1]
    out = np.zeros((n, d2), np.float32)
    orc().orc_dense_f32(_f(out), _f(X), _f(W), C.c_int64(n), d1, d2, C.c_int64(d1), C.c_int64(d2), int(f64),
                        threads or max_threads())
    return out


def softmax_rows(X, threads=0):
    X = np.ascontiguousarray(X, np.float32)
    n, c = X.shape
    out = np.zeros((n, c), np.float32)
    orc().orc_softmax_rows(_f(out), _f(X), C.c_int64(n), c, C.c_int64(c), C.c_int64(c), threads or max_threads())
    return out


def gcn2_forward(X, W1, W2, ptr_l, col_l, ptr_r, col_r, lb, ub, npp, *, rs=None, f64=True, threads=0):
    """-> (P, H2, H1): softmax output, second and first aggregation outputs."""
    X = np.ascontiguousarray(X, np.float32)
    W1 = np.ascontiguousarray(W1, np.float32)
    W2 = np.ascontiguousarray(W2, np.float32)
    ptr_l, col_l = _i32(ptr_l), _i32(col_l)
    if ptr_r is not None:
        ptr_r, col_r = _i32(ptr_r), _i32(col_r)
    R = ub - lb
    in_dim, hidden = W1.shape
    out_dim = W2.shape[1]
    P = np.zeros((R, out_dim), np.float32)
    H2 = np.zeros((R, out_dim), np.float32)
    H1 = np.zeros((R, hidden), np.float32)
    rs = None if rs is None else np.ascontiguousarray(rs, np.float32)
    orc().orc_gcn2_forward(_f(P), _f(H2), _f(H1), _f(X), _f(W1), _f(W2), _i(ptr_l), _i(col_l), _i(ptr_r), _i(col_r), lb, ub,
                           npp, in_dim, hidden, out_dim, _f(rs), int(f64), threads or max_threads())
    return P, H2, H1


def gin_forward(X, Ws, ptr_l, col_l, ptr_r, col_r, lb, ub, npp, eps, *, f64=True, threads=0):
    """Ws = [W0 (in x hidden), W1..W_{L-1} (hidden x hidden), W_L (hidden x out)] -> (P, logits)."""
    X = np.ascontiguousarray(X, np.float32)
    Ws = [np.ascontiguousarray(w, np.float32) for w in Ws]
    ptr_l, col_l = _i32(ptr_l), _i32(col_l)
    if ptr_r is not None:
        ptr_r, col_r = _i32(ptr_r), _i32(col_r)
    R = ub - lb
    in_dim, hidden = Ws[0].shape
    out_dim = Ws[-1].shape[1]
    n_layers = len(Ws) - 1
    arr = (C.POINTER(C.c_float) * len(Ws))(*[_f(w) for w in Ws])
    P = np.zeros((R, out_dim), np.float32)
    logits = np.zeros((R, out_dim), np.float32)
    orc().orc_gin_forward(_f(P), _f(logits), _f(X), arr, n_layers, _i(ptr_l), _i(col_l), _i(ptr_r), _i(col_r), lb, ub, npp,
                          in_dim, hidden, out_dim, C.c_float(eps), int(f64), threads or max_threads())
    return P, logits


# ----------------------------------------------------------------------------- reference's own host code
def ref_split_csr(ptr, col, lb, ub):
    ptr, col = _i32(ptr), _i32(col)
    n = (C.c_int64 * 4)()
    ref().ref_split_csr(_i(ptr), C.c_int64(len(ptr)), _i(col), C.c_int64(len(col)), lb, ub, None, None, None, None, n)
    outs = [np.zeros(n[i], np.int32) for i in range(4)]
    ref().ref_split_csr(_i(ptr), C.c_int64(len(ptr)), _i(col), C.c_int64(len(col)), lb, ub, _i(outs[0]), _i(outs[1]),
                        _i(outs[2]), _i(outs[3]), n)
    return tuple(outs)


def ref_build_part(indptr, num_nodes, ps):
    indptr = _i32(indptr)
    n = (C.c_int64 * 3)()
    ref().ref_build_part(_i(indptr), C.c_int64(len(indptr)), num_nodes, ps, None, None, None, n)
    outs = [np.zeros(n[i], np.int32) for i in range(3)]
    ref().ref_build_part(_i(indptr), C.c_int64(len(indptr)), num_nodes, ps, _i(outs[0]), _i(outs[1]), _i(outs[2]), n)
    return tuple(outs)


def ref_sag_ref(inp, ptr, col):
    inp = np.ascontiguousarray(inp, np.float32)
    ptr, col = _i32(ptr), _i32(col)
    n = len(ptr) - 1
    upd = np.zeros((n, inp.shape[1]), np.float32)
    ref().ref_sag_ref(_f(upd), _f(inp), _i(ptr), _i(col), n, len(col), inp.shape[1])
    return upd


def ref_graph_load(beg, csr, weight):
    v, e = C.c_int(), C.c_int()
    ref().ref_graph_load(beg.encode(), csr.encode(), weight.encode(), C.byref(v), C.byref(e), None, None, None)
    b = np.zeros(v.value + 1, np.int32)
    c = np.zeros(e.value, np.int32)
    w = np.zeros(e.value, np.int32)
    ref().ref_graph_load(beg.encode(), csr.encode(), weight.encode(), C.byref(v), C.byref(e), _i(b), _i(c), _i(w))
    return b, c, w


def ref_mtx_load(path):
    n = (C.c_int64 * 2)()
    ref().ref_mtx_load(path.encode(), None, None, n)
    rp = np.zeros(n[0], np.int32)
    ci = np.zeros(n[1], np.int32)
    ref().ref_mtx_load(path.encode(), _i(rp), _i(ci), n)
    return rp, ci


def _l(a):
    return a.ctypes.data_as(C.POINTER(C.c_long))


def ref_split_csr_long(ptr, col, lb, ub):
    """split_CSR<long> of the reference -> the four arrays as int64."""
    ptr, col = np.ascontiguousarray(ptr, np.int64), np.ascontiguousarray(col, np.int64)
    n = (C.c_int64 * 4)()
    ref().ref_split_csr_long(_l(ptr), C.c_int64(len(ptr)), _l(col), C.c_int64(len(col)), C.c_long(lb), C.c_long(ub), None, None, None, None, n)
    outs = [np.zeros(n[i], np.int64) for i in range(4)]
    ref().ref_split_csr_long(_l(ptr), C.c_int64(len(ptr)), _l(col), C.c_int64(len(col)), C.c_long(lb), C.c_long(ub), _l(outs[0]), _l(outs[1]),
                             _l(outs[2]), _l(outs[3]), n)
    return tuple(outs)


def ref_build_part_long(indptr, num_nodes, ps):
    indptr = np.ascontiguousarray(indptr, np.int64)
    n = (C.c_int64 * 3)()
    ref().ref_build_part_long(_l(indptr), C.c_int64(len(indptr)), C.c_long(num_nodes), C.c_long(ps), None, None, None, n)
    outs = [np.zeros(n[i], np.int64) for i in range(3)]
    ref().ref_build_part_long(_l(indptr), C.c_int64(len(indptr)), C.c_long(num_nodes), C.c_long(ps), _l(outs[0]), _l(outs[1]), _l(outs[2]), n)
    return tuple(outs)


def ref_mtx_load_other(path, symmetric):
    """assemble_csr_matrix / assemble_simetric_csr_matrix of the reference -> dict(row_ptr, col_ind, val, bandwidth, text):
    getBandwidth of the result and what printMatrix prints for it (with row_ptr[0] = 1, see build_ref.sh)."""
    n = (C.c_int64 * 3)()
    ref().ref_mtx_load_other(int(symmetric), path.encode(), None, None, None, n, None, None, C.c_int64(0))
    rp, ci, val = np.zeros(n[0], np.int32), np.zeros(n[1], np.int32), np.zeros(n[2], np.float64)
    bw = C.c_int()
    text = C.create_string_buffer(1 << 20)
    ref().ref_mtx_load_other(int(symmetric), path.encode(), _i(rp), _i(ci), val.ctypes.data_as(C.POINTER(C.c_double)), n, C.byref(bw),
                             text, C.c_int64(len(text)))
    return {"row_ptr": rp, "col_ind": ci, "val": val, "bandwidth": bw.value, "text": text.value.decode()}
