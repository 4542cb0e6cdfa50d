"""ctypes binding of libmggx.so: the same C ABI the C++ layer in include/mgg/ uses.

Function names follow the reference's host API (split_CSR, build_part,
mgg_SAG_np_div, mgg_GIN_np_div, SAG_host, dense/softmax forward).  Device
memory is passed as torch CUDA tensors (their data_ptr()); torch is used for
nothing else.  There is no CPU fallback: a missing library raises.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional, Tuple

import numpy as np

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libmggx.so")

AGG_ACCUMULATE = 1
AGG_GIN = 2
AGG_RELU = 4
AGG_SOFTMAX = 8
F32 = 0
BF16 = 1


class MggxError(RuntimeError):
    pass


class _AggOpts(C.Structure):
    _fields_ = [("flags", C.c_uint32), ("eps", C.c_float), ("ld_in", C.c_int64), ("ld_out", C.c_int64),
                ("d_row_scale_out", C.c_void_p), ("in_dtype", C.c_int), ("col_block_rows", C.c_int), ("core_rows", C.c_int)]


class _AggKnobs(C.Structure):
    _fields_ = [("ps", C.c_int), ("wpb", C.c_int), ("dist", C.c_int), ("col_block_rows", C.c_int), ("core_rows", C.c_int)]


class _CacheStats(C.Structure):
    _fields_ = [("plans", C.c_int64), ("plan_bytes", C.c_int64), ("core_plans", C.c_int64), ("core_plan_bytes", C.c_int64),
                ("workspace_bytes", C.c_int64), ("core_scratch_bytes", C.c_int64), ("retired_bytes", C.c_int64),
                ("plan_build_ms", C.c_double), ("core_plan_build_ms", C.c_double), ("search_ms", C.c_double)]


class _DenseOpts(C.Structure):
    _fields_ = [("ld_x", C.c_int64), ("ld_out", C.c_int64), ("d_row_scale", C.c_void_p), ("relu", C.c_uint32)]


class _Mlp2Opts(C.Structure):
    _fields_ = [("ld_x", C.c_int64), ("ld_out", C.c_int64), ("d_row_scale", C.c_void_p), ("relu_mid", C.c_uint32),
                ("relu_out", C.c_uint32)]


_lib = None

# every symbol include/mggx.h declares
EXPORTS = [
    "mggx_last_error", "mggx_version", "mggx_init", "mggx_device_name", "mggx_set_stream", "mggx_sync",
    "mggx_malloc", "mggx_malloc_tables", "mggx_free", "mggx_memset", "mggx_memcpy_h2d", "mggx_memcpy_d2h", "mggx_memcpy_d2d",
    "mggx_timer_create", "mggx_timer_start", "mggx_timer_stop", "mggx_timer_elapsed_ms", "mggx_timer_destroy",
    "mggx_release_cached", "mggx_forget", "mggx_set_plan_check", "mggx_cache_stats", "mggx_range_partition", "mggx_split_csr", "mggx_compact_remote", "mggx_build_part", "mggx_core_layout_build", "mggx_core_layout_fetch", "mggx_core_layout_device", "mggx_convert_probe", "mggx_graph_read",
    "mggx_graph_write", "mggx_mtx_read", "mggx_gen_rmat", "mggx_gen_er", "mggx_gen_fetch", "mggx_fill_normal",
    "mggx_fill_uniform", "mggx_build_part_device", "mggx_split_csr_device", "mggx_compact_remote_device", "mggx_edgelist_to_bin", "mggx_sag_np_div", "mggx_sag_np_div_tune", "mggx_sag_parts", "mggx_sag_parts_static", "mggx_mlp2_xw", "mggx_spmm",
    "mggx_dense_xw", "mggx_dense_xw_bf16", "mggx_softmax_rows", "mggx_cast_f32_to_bf16", "mggx_copy_bytes", "mggx_copy_bytes_nt", "mggx_gather_probe", "mggx_lds_probe", "mggx_gather_rows", "mggx_last_agg_kernel", "mggx_set_gather_addressing",
]


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise MggxError("libmggx.so is not built (run `python -m mgg_osdi23_amd.build`); there is no fallback path")
        _lib = C.CDLL(LIB_PATH)
        _lib.mggx_last_error.restype = C.c_char_p
        _lib.mggx_version.restype = C.c_char_p
    return _lib


def _check(rc: int) -> None:
    if rc != 0:
        raise MggxError("mggx error %d: %s" % (rc, lib().mggx_last_error().decode()))


def _iptr(a: Optional[np.ndarray]):
    if a is None:
        return None
    assert a.dtype == np.int32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(C.POINTER(C.c_int))


def _dptr(t) -> C.c_void_p:
    """Device address of a torch CUDA tensor (None -> NULL)."""
    if t is None:
        return C.c_void_p(0)
    assert t.is_cuda and t.is_contiguous(), "device tensors must be contiguous CUDA tensors"
    return C.c_void_p(t.data_ptr())


# --------------------------------------------------------------------------- host-side graph preparation
def range_partition(num_nodes: int, num_gpus: int, pe: int) -> Tuple[int, int, int]:
    npp, lb, ub = C.c_int(), C.c_int(), C.c_int()
    _check(lib().mggx_range_partition(num_nodes, num_gpus, pe, C.byref(npp), C.byref(lb), C.byref(ub)))
    return npp.value, lb.value, ub.value


def split_CSR(ptr: np.ndarray, col: np.ndarray, lb: int, ub: int):
    """-> (local_ptr, remote_ptr, local_col_idx, remote_col_idx), the reference's return order."""
    ptr = np.ascontiguousarray(ptr, dtype=np.int32)
    col = np.ascontiguousarray(col, dtype=np.int32)
    nl, nr = C.c_int64(), C.c_int64()
    _check(lib().mggx_split_csr(_iptr(ptr), _iptr(col), lb, ub, None, None, None, None, C.byref(nl), C.byref(nr)))
    rows = ub - lb
    lp = np.zeros(rows + 1, np.int32)
    rp = np.zeros(rows + 1, np.int32)
    lc = np.zeros(nl.value, np.int32)
    rc = np.zeros(nr.value, np.int32)
    _check(lib().mggx_split_csr(_iptr(ptr), _iptr(col), lb, ub, _iptr(lp), _iptr(rp), _iptr(lc), _iptr(rc),
                                C.byref(nl), C.byref(nr)))
    return lp, rp, lc, rc


def compact_remote(remote_col: np.ndarray):
    """-> (remote_col_compact, fetch_ids): the distinct remote ids in staging order (most referenced first) and the
    column array rewritten to positions in it; stage `table[fetch_ids]` as the remote table."""
    rc = np.ascontiguousarray(remote_col, dtype=np.int32)
    nu = C.c_int64()
    _check(lib().mggx_compact_remote(_iptr(rc), C.c_int64(len(rc)), None, None, C.byref(nu)))
    out = np.zeros(len(rc), np.int32)
    ids = np.zeros(nu.value, np.int32)
    _check(lib().mggx_compact_remote(_iptr(rc), C.c_int64(len(rc)), _iptr(out), _iptr(ids), C.byref(nu)))
    return out, ids


def compact_remote_device(d_remote_col, n_remote: int):
    """compact_remote on the GPU -> (remote_col_compact, fetch_ids) as device tensors."""
    import torch
    nu = C.c_int64()
    _check(lib().mggx_compact_remote_device(_dptr(d_remote_col), C.c_int64(n_remote), None, None, C.byref(nu)))
    out = torch.zeros(max(n_remote, 1), dtype=torch.int32, device=d_remote_col.device)
    ids = torch.zeros(max(nu.value, 1), dtype=torch.int32, device=d_remote_col.device)
    _check(lib().mggx_compact_remote_device(_dptr(d_remote_col), C.c_int64(n_remote), _dptr(out), _dptr(ids), C.byref(nu)))
    return out[:n_remote], ids[: nu.value]


def gather_rows(dst, table, ids, n: int, row_bytes: int) -> None:
    """dst row i = table row ids[i] on the device (staging a compact remote table)."""
    _check(lib().mggx_gather_rows(_dptr(dst), _dptr(table), _dptr(ids), C.c_int64(n), C.c_size_t(row_bytes)))


def build_part(indptr: np.ndarray, num_nodes: int, part_size: int, compat: bool = True):
    """-> (partPtr, part2Node, node2Part), the reference's return order."""
    indptr = np.ascontiguousarray(indptr, dtype=np.int32)
    n = C.c_int()
    _check(lib().mggx_build_part(_iptr(indptr), num_nodes, part_size, int(compat), None, None, None, C.byref(n)))
    pp = np.zeros(n.value + 1, np.int32)
    p2n = np.zeros(n.value, np.int32)
    n2p = np.zeros(num_nodes + 2, np.int32)
    _check(lib().mggx_build_part(_iptr(indptr), num_nodes, part_size, int(compat), _iptr(pp), _iptr(p2n), _iptr(n2p),
                                 C.byref(n)))
    return pp, p2n, n2p


def graph_read(beg_file: str, csr_file: str, weight_file: str):
    v, e = C.c_int(), C.c_int()
    _check(lib().mggx_graph_read(beg_file.encode(), csr_file.encode(), weight_file.encode(), C.byref(v), C.byref(e),
                                 None, None, None))
    beg = np.zeros(v.value + 1, np.int32)
    csr = np.zeros(e.value, np.int32)
    w = np.zeros(e.value, np.int32)
    _check(lib().mggx_graph_read(beg_file.encode(), csr_file.encode(), weight_file.encode(), C.byref(v), C.byref(e),
                                 _iptr(beg), _iptr(csr), _iptr(w)))
    return beg, csr, w


def graph_write(beg_file: str, csr_file: str, weight_file: str, beg_pos: np.ndarray, csr: np.ndarray,
                weight: Optional[np.ndarray] = None) -> None:
    beg_pos = np.ascontiguousarray(beg_pos, dtype=np.int32)
    csr = np.ascontiguousarray(csr, dtype=np.int32)
    if weight is not None:
        weight = np.ascontiguousarray(weight, dtype=np.int32)
    _check(lib().mggx_graph_write(beg_file.encode(), csr_file.encode(), weight_file.encode(), len(beg_pos) - 1,
                                  _iptr(beg_pos), _iptr(csr), _iptr(weight)))


def mtx_read(path: str):
    m, l = C.c_int(), C.c_int()
    _check(lib().mggx_mtx_read(path.encode(), C.byref(m), C.byref(l), None, None))
    rp = np.zeros(m.value + 1, np.int32)
    ci = np.zeros(l.value, np.int32)
    _check(lib().mggx_mtx_read(path.encode(), C.byref(m), C.byref(l), _iptr(rp), _iptr(ci)))
    return rp, ci


def edgelist_to_bin(path: str, out_prefix: str, is_mtx: bool = False):
    """Text edge list (.mtx or 0-based 'src dst') -> <prefix>_beg_pos.bin/_csr.bin/_weight.bin; returns (V, E)."""
    v, e = C.c_int(), C.c_int64()
    _check(lib().mggx_edgelist_to_bin(path.encode(), int(is_mtx), out_prefix.encode(), C.byref(v), C.byref(e)))
    return v.value, e.value


def split_CSR_device(d_ptr, d_col, lb: int, ub: int):
    """split_CSR on the GPU -> (local_ptr, remote_ptr, local_col_idx, remote_col_idx) as device tensors."""
    import torch
    rows = ub - lb
    lp = torch.zeros(rows + 1, dtype=torch.int32, device=d_ptr.device)
    rp = torch.zeros(rows + 1, dtype=torch.int32, device=d_ptr.device)
    nl, nr = C.c_int64(), C.c_int64()
    _check(lib().mggx_split_csr_device(_dptr(d_ptr), _dptr(d_col), lb, ub, _dptr(lp), _dptr(rp), None, None,
                                       C.byref(nl), C.byref(nr)))
    lc = torch.zeros(max(nl.value, 1), dtype=torch.int32, device=d_ptr.device)
    rc = torch.zeros(max(nr.value, 1), dtype=torch.int32, device=d_ptr.device)
    _check(lib().mggx_split_csr_device(_dptr(d_ptr), _dptr(d_col), lb, ub, _dptr(lp), _dptr(rp), _dptr(lc), _dptr(rc),
                                       C.byref(nl), C.byref(nr)))
    sync()
    return lp, rp, lc[: nl.value], rc[: nr.value]


def gen_rmat(scale: int, num_nodes: int, num_draws: int, a=0.57, b=0.19, c=0.19, seed=0, scramble=False,
             row_lo=0, row_hi=None, threads=0):
    if row_hi is None:
        row_hi = num_nodes
    h, nnz = C.c_void_p(), C.c_int64()
    _check(lib().mggx_gen_rmat(scale, num_nodes, C.c_int64(num_draws), C.c_double(a), C.c_double(b), C.c_double(c),
                               C.c_uint64(seed), int(scramble), row_lo, row_hi, threads, C.byref(h), C.byref(nnz)))
    ptr = np.zeros(row_hi - row_lo + 1, np.int32)
    col = np.zeros(nnz.value, np.int32)
    _check(lib().mggx_gen_fetch(h, _iptr(ptr), _iptr(col)))
    return ptr, col


def gen_er(num_nodes: int, avg_degree: float, seed=0):
    h, nnz = C.c_void_p(), C.c_int64()
    _check(lib().mggx_gen_er(num_nodes, C.c_double(avg_degree), C.c_uint64(seed), C.byref(h), C.byref(nnz)))
    ptr = np.zeros(num_nodes + 1, np.int32)
    col = np.zeros(nnz.value, np.int32)
    _check(lib().mggx_gen_fetch(h, _iptr(ptr), _iptr(col)))
    return ptr, col


def fill_normal(shape, seed: int) -> np.ndarray:
    out = np.empty(shape, np.float32)
    _check(lib().mggx_fill_normal(out.ctypes.data_as(C.POINTER(C.c_float)), C.c_int64(out.size), C.c_uint64(seed)))
    return out


def fill_uniform(shape, lo: float, hi: float, seed: int) -> np.ndarray:
    out = np.empty(shape, np.float32)
    _check(lib().mggx_fill_uniform(out.ctypes.data_as(C.POINTER(C.c_float)), C.c_int64(out.size), C.c_float(lo),
                                   C.c_float(hi), C.c_uint64(seed)))
    return out


def glorot(d1: int, d2: int, seed: int) -> np.ndarray:
    lim = float(np.sqrt(6.0 / (d1 + d2)))
    return fill_uniform((d1, d2), -lim, lim, seed)


# --------------------------------------------------------------------------- device side
def init(device: int = 0) -> None:
    _check(lib().mggx_init(device))


def use_torch_stream() -> None:
    """Issue the library's work on torch's current stream (so torch ops and events order with it)."""
    import torch
    _check(lib().mggx_set_stream(C.c_void_p(torch.cuda.current_stream().cuda_stream)))


def sync() -> None:
    _check(lib().mggx_sync())


_pinned = {}  # CSR tensors of cached plans, by address: keeps the addresses from being reused while cached
_captured = set()  # keys of _pinned that were used while a stream capture was recording: a captured graph reads those arrays
_PIN_MAX_SETS, _PIN_MAX_BYTES = 64, 8 << 30


def _pin(*tensors) -> None:
    """Holds a reference to the CSR tensors of a call so that torch's allocator does not hand their addresses to other
    data while the library has plans cached for them; bounded by count and bytes, oldest first, and the library forgets
    a set before it is let go.  Sets used inside a stream capture are never let go here (a replay of the captured graph
    reads them); forget() and release_cached() are the ways to drop those."""
    import torch
    key = tuple(t.data_ptr() if t is not None else 0 for t in tensors)
    if torch.cuda.is_current_stream_capturing():
        _captured.add(key)
    if key in _pinned:
        return
    _pinned[key] = tensors
    size = lambda ts: sum(t.numel() * t.element_size() for t in ts if t is not None)
    while True:
        loose = [k for k in _pinned if k not in _captured and k != key]
        over = len(_pinned) > _PIN_MAX_SETS or sum(size(ts) for ts in _pinned.values()) > _PIN_MAX_BYTES
        if not over or not loose:
            break
        old = _pinned.pop(loose[0])
        for t in old:
            if t is not None:
                _check(lib().mggx_forget(C.c_void_p(t.data_ptr())))


def forget(tensor) -> None:
    """Drops the plans and search results the library keeps for this CSR tensor (call before rewriting it in place)."""
    _check(lib().mggx_forget(C.c_void_p(tensor.data_ptr())))
    for key in [k for k in _pinned if tensor.data_ptr() in k]:
        _pinned.pop(key)
        _captured.discard(key)


def release_cached() -> None:
    _check(lib().mggx_release_cached())
    _pinned.clear()
    _captured.clear()


def set_plan_check(level: int) -> None:
    """Content checks of cached plans against the caller's CSR arrays: 0 = off, 1 = live edge counts inside every kernel
    (default), 2 = also a fingerprint kernel before every call."""
    _check(lib().mggx_set_plan_check(int(level)))


def cache_stats() -> dict:
    """What the library holds (plans, scratch) and what its set-up has cost so far (ms, host clock)."""
    st = _CacheStats()
    _check(lib().mggx_cache_stats(C.byref(st)))
    return {k: getattr(st, k) for k, _ in _CacheStats._fields_}


def device_name() -> str:
    buf = C.create_string_buffer(256)
    _check(lib().mggx_device_name(buf, 256))
    return buf.value.decode()


def set_gather_addressing(mode: int) -> None:
    _check(lib().mggx_set_gather_addressing(mode))


def last_agg_kernel() -> str:
    buf = C.create_string_buffer(256)
    _check(lib().mggx_last_agg_kernel(buf, 256))
    return buf.value.decode()


def build_part_device(d_indptr, num_nodes: int, part_size: int, compat: bool = True):
    import torch
    n = C.c_int()
    _check(lib().mggx_build_part_device(_dptr(d_indptr), num_nodes, part_size, int(compat), None, None, None, C.byref(n)))
    pp = torch.zeros(n.value + 1, dtype=torch.int32, device=d_indptr.device)
    p2n = torch.zeros(max(n.value, 1), dtype=torch.int32, device=d_indptr.device)[: n.value]
    n2p = torch.zeros(num_nodes + 2, dtype=torch.int32, device=d_indptr.device)
    _check(lib().mggx_build_part_device(_dptr(d_indptr), num_nodes, part_size, int(compat), _dptr(pp),
                                        C.c_void_p(p2n.data_ptr()) if n.value else C.c_void_p(pp.data_ptr()),
                                        _dptr(n2p), C.byref(n)))
    return pp, p2n, n2p


def _agg(out, in_local, in_remote, ptr_l, col_l, ptr_r, col_r, lb, ub, dim, npp, ps, wpb, dist, flags, eps,
         ld_in, ld_out, row_scale_out, col_block_rows=0, core_rows=0):
    import torch
    o = _AggOpts()
    o.flags = flags
    o.eps = eps
    o.ld_in = ld_in
    o.ld_out = ld_out
    o.d_row_scale_out = row_scale_out.data_ptr() if row_scale_out is not None else None
    o.in_dtype = BF16 if in_local.dtype == torch.bfloat16 else F32
    o.col_block_rows = col_block_rows
    o.core_rows = core_rows
    _pin(ptr_l, ptr_r, col_l, col_r)
    _check(lib().mggx_sag_np_div(_dptr(out), _dptr(in_local), _dptr(in_remote), _dptr(ptr_l), _dptr(col_l),
                                 _dptr(ptr_r), _dptr(col_r), lb, ub, dim, npp, ps, wpb, dist, C.byref(o)))


def tune_np_div(output, input, row_pointers_l, column_index_l, row_pointers_r, column_index_r, lb, ub, dim, nodePerPE,
                np_size, *, input_remote=None, gin_eps=None, ld_in=0, ld_out=0, row_scale_out=None, relu=False, softmax=False,
                col_block_rows=0, core_rows=0):
    """The search of the reference's bench_MGG_DSE_dist_ps.py / bench_MGG_DSE_dist_wpb.py in one call: times
    partSize (as given, or 16 and 32 when 0) x plain / column-blocked order x without / with a dense core x warpPerBlock x
    interleaved_dist on this input, returns ({"ps", "wpb", "dist", "col_block_rows", "core_rows"}, ms) of the fastest and makes later calls that leave the
    knobs at 0 on the same CSR tensors use it."""
    import torch
    o = _AggOpts()
    o.flags = (AGG_RELU if relu else 0) | (AGG_GIN if gin_eps is not None else 0) | (AGG_SOFTMAX if softmax else 0)
    o.eps = float(gin_eps or 0.0)
    o.ld_in = ld_in
    o.ld_out = ld_out
    o.d_row_scale_out = row_scale_out.data_ptr() if row_scale_out is not None else None
    o.in_dtype = BF16 if input.dtype == torch.bfloat16 else F32
    o.col_block_rows = col_block_rows
    o.core_rows = core_rows
    _pin(row_pointers_l, row_pointers_r, column_index_l, column_index_r)
    k, ms = _AggKnobs(), C.c_float()
    rem = input_remote if input_remote is not None else input
    _check(lib().mggx_sag_np_div_tune(_dptr(output), _dptr(input), _dptr(rem), _dptr(row_pointers_l), _dptr(column_index_l),
                                      _dptr(row_pointers_r), _dptr(column_index_r), lb, ub, dim, nodePerPE, np_size,
                                      C.byref(o), C.byref(k), C.byref(ms)))
    return {"ps": k.ps, "wpb": k.wpb, "dist": k.dist, "col_block_rows": k.col_block_rows, "core_rows": k.core_rows}, ms.value


def mgg_SAG_np_div(output, input, row_pointers_l, column_index_l, row_pointers_r, column_index_r, lb, ub, dim,
                   nodePerPE, peid, np_size, warpPerBlock, interleaved_dist, *, input_remote=None, accumulate=False,
                   ld_in=0, ld_out=0, row_scale_out=None, relu=False, softmax=False, col_block_rows=0, core_rows=0):
    """Argument order of the reference's mgg_SAG_np_div.  `input` is this rank's table; `input_remote` the
    global-id-indexed table the reference reaches with remote GETs (defaults to `input`, the single-GPU case).
    The reference adds into `output`; pass accumulate=True for that, the default overwrites.  softmax=True applies the row
    softmax of the reference's last layer (softmax_forward) inside the same call."""
    flags = (AGG_ACCUMULATE if accumulate else 0) | (AGG_RELU if relu else 0) | (AGG_SOFTMAX if softmax else 0)
    _agg(output, input, input_remote if input_remote is not None else input, row_pointers_l, column_index_l,
         row_pointers_r, column_index_r, lb, ub, dim, nodePerPE, np_size, warpPerBlock, interleaved_dist, flags, 0.0,
         ld_in, ld_out, row_scale_out, col_block_rows, core_rows)


def mgg_GIN_np_div(output, input, row_pointers_l, column_index_l, row_pointers_r, column_index_r, lb, ub, dim,
                   nodePerPE, peid, np_size, warpPerBlock, interleaved_dist, eps, *, input_remote=None, ld_in=0,
                   ld_out=0, col_block_rows=0, core_rows=0):
    _agg(output, input, input_remote if input_remote is not None else input, row_pointers_l, column_index_l,
         row_pointers_r, column_index_r, lb, ub, dim, nodePerPE, np_size, warpPerBlock, interleaved_dist, AGG_GIN,
         float(eps), ld_in, ld_out, None, col_block_rows, core_rows)


def SAG_host(output, input, row_pointers, column_index, part_pointers, part2Node, lowbound, num_nodes, num_parts,
             partSize, dim, dimWorker, warpPerBlock, interleaved_dist=1):
    _pin(row_pointers, part_pointers, part2Node)
    _check(lib().mggx_sag_parts(_dptr(output), _dptr(input), _dptr(row_pointers), _dptr(column_index),
                                _dptr(part_pointers), _dptr(part2Node), lowbound, num_nodes, num_parts, partSize, dim,
                                warpPerBlock, interleaved_dist))


def SAG_host_static(output, input, row_pointers, column_index, part_pointers, part2Node, lowbound, num_nodes, num_parts,
                    partSize, dim, dimWorker, warpPerBlock, interleaved_dist=1):
    """SAG_host through the entry point that allocates nothing (fixed device scratch, nothing cached)."""
    _check(lib().mggx_sag_parts_static(_dptr(output), _dptr(input), _dptr(row_pointers), _dptr(column_index),
                                       _dptr(part_pointers), _dptr(part2Node), lowbound, num_nodes, num_parts, partSize, dim,
                                       warpPerBlock, interleaved_dist))


def SpMM(output, input, row_pointers, column_index, num_nodes, dim, partSize, warpPerBlock):
    _pin(row_pointers, column_index)
    _check(lib().mggx_spmm(_dptr(output), _dptr(input), _dptr(row_pointers), _dptr(column_index), num_nodes, dim,
                           partSize, warpPerBlock))


def dense_forward(out, x, w, n, d1, d2, ld_x=0, ld_out=0, row_scale=None, relu=False):
    o = _DenseOpts()
    o.ld_x = ld_x
    o.ld_out = ld_out
    o.d_row_scale = row_scale.data_ptr() if row_scale is not None else None
    o.relu = int(relu)
    _check(lib().mggx_dense_xw(_dptr(out), _dptr(x), _dptr(w), C.c_int64(n), d1, d2, C.byref(o)))


def mlp2_forward(out, x, wa, wb, n, d1, h, d3, ld_x=0, ld_out=0, row_scale=None, relu_mid=True, relu_out=False,
                 softmax_out=False):
    """Out = act(X . Wa) . Wb in one pass (h, d3 <= 64): two dense_hidden_forward calls without the round trip of the
    intermediate through memory.  softmax_out: the row softmax of the result (softmax_new_forward) in the same pass."""
    o = _Mlp2Opts()
    o.ld_x = ld_x
    o.ld_out = ld_out
    o.d_row_scale = row_scale.data_ptr() if row_scale is not None else None
    o.relu_mid = int(relu_mid)
    assert not (relu_out and softmax_out)
    o.relu_out = 2 if softmax_out else int(relu_out)
    _check(lib().mggx_mlp2_xw(_dptr(out), _dptr(x), _dptr(wa), _dptr(wb), C.c_int64(n), d1, h, d3, C.byref(o)))


def dense_forward_bf16(out, x, w_bf16, n, d1, d2, ld_x=0, ld_out=0, row_scale=None, relu=False):
    """Out = X . W on the bf16 matrix cores; X fp32 or bf16, W bf16, Out fp32 or bf16 (taken from the tensors)."""
    import torch
    o = _DenseOpts()
    o.ld_x = ld_x
    o.ld_out = ld_out
    o.d_row_scale = row_scale.data_ptr() if row_scale is not None else None
    o.relu = int(relu)
    assert w_bf16.dtype == torch.bfloat16
    xd = BF16 if x.dtype == torch.bfloat16 else F32
    od = BF16 if out.dtype == torch.bfloat16 else F32
    _check(lib().mggx_dense_xw_bf16(_dptr(out), _dptr(x), _dptr(w_bf16), C.c_int64(n), d1, d2, xd, od, C.byref(o)))


def cast_f32_to_bf16(dst, src, n) -> None:
    _check(lib().mggx_cast_f32_to_bf16(_dptr(dst), _dptr(src), C.c_int64(n)))


def softmax_forward(out, x, n, c, ld_in=0, ld_out=0):
    _check(lib().mggx_softmax_rows(_dptr(out), _dptr(x), C.c_int64(n), c, C.c_int64(ld_in), C.c_int64(ld_out)))


def copy_bytes(dst, src, nbytes: int) -> None:
    _check(lib().mggx_copy_bytes(_dptr(dst), _dptr(src), C.c_size_t(nbytes)))


def copy_bytes_nt(dst, src, nbytes: int) -> None:
    _check(lib().mggx_copy_bytes_nt(_dptr(dst), _dptr(src), C.c_size_t(nbytes)))


def convert_probe(dst, src, n: int, pieces_per_workgroup: int = 1, persistent_workgroups: int = 0) -> None:
    """fp32 -> bf16 (truncated) streaming conversion of n values: the 2:1 read/write yardstick of the dense update."""
    _check(lib().mggx_convert_probe(_dptr(dst), _dptr(src), C.c_int64(n), pieces_per_workgroup, persistent_workgroups))


def gather_probe(sink, table, rows: int, ld_bytes: int, row_bytes: int, n_gathers: int, seed: int = 1) -> int:
    """Random row gathers from `table` (rows x ld_bytes bytes); `sink` holds 262144 floats.  Returns the number issued."""
    done = C.c_int64(0)
    _check(lib().mggx_gather_probe(_dptr(sink), _dptr(table), C.c_int64(rows), C.c_size_t(ld_bytes), C.c_size_t(row_bytes),
                                   C.c_int64(n_gathers), C.c_uint(seed), C.byref(done)))
    return int(done.value)


def lds_probe(sink, row_bytes: int, n_reads: int, seed: int = 1) -> int:
    """Random row reads from an LDS tile laid out like the dense-core kernel's; returns the number issued."""
    done = C.c_int64(0)
    _check(lib().mggx_lds_probe(_dptr(sink), C.c_size_t(row_bytes), C.c_int64(n_reads), C.c_uint(seed), C.byref(done)))
    return int(done.value)


def core_layout(ptr: np.ndarray, col: np.ndarray, lb: int, core_rows: int, tile_cols: int = 256):
    """The dense-core layout of a local CSR as the library builds it -> dict(core, ntiles, core_nnz, order, rank,
    blk_off, idx, rem_ptr, rem_col)."""
    ptr = np.ascontiguousarray(ptr, dtype=np.int32)
    col = np.ascontiguousarray(col, dtype=np.int32)
    rows = len(ptr) - 1
    h = C.c_void_p()
    sizes = (C.c_int64 * 5)()
    _check(lib().mggx_core_layout_build(_iptr(ptr), _iptr(col), rows, lb, core_rows, tile_cols, C.byref(h), sizes))
    core = int(sizes[0])
    order, rank = np.zeros(core, np.int32), np.zeros(rows, np.int32)
    blk_off, idx = np.zeros(int(sizes[1]), np.uint32), np.zeros(int(sizes[2]), np.uint16)
    rem_ptr, rem_col = np.zeros(rows + 1, np.int32), np.zeros(int(sizes[3]), np.int32)
    _check(lib().mggx_core_layout_fetch(h, _iptr(order), _iptr(rank), blk_off.ctypes.data_as(C.c_void_p),
                                        idx.ctypes.data_as(C.c_void_p), _iptr(rem_ptr), _iptr(rem_col)))
    return dict(core=core, ntiles=core // tile_cols, core_nnz=int(sizes[4]), order=order, rank=rank, blk_off=blk_off, idx=idx,
                rem_ptr=rem_ptr, rem_col=rem_col)


def core_layout_device(d_ptr, d_col, rows: int, lb: int, core_rows: int):
    """The dense-core layout as the aggregation builds it on the GPU (from device tensors) -> the same dict as core_layout."""
    sizes = (C.c_int64 * 5)()
    _pin(d_ptr, d_col)
    _check(lib().mggx_core_layout_device(_dptr(d_ptr), _dptr(d_col), rows, lb, core_rows, sizes, None, None, None, None, None, None))
    core = int(sizes[0])
    order, rank = np.zeros(core, np.int32), np.zeros(rows, np.int32)
    blk_off, idx = np.zeros(int(sizes[1]), np.uint32), np.zeros(int(sizes[2]), np.uint16)
    rem_ptr, rem_col = np.zeros(rows + 1, np.int32), np.zeros(int(sizes[3]), np.int32)
    _check(lib().mggx_core_layout_device(_dptr(d_ptr), _dptr(d_col), rows, lb, core_rows, sizes, _iptr(order), _iptr(rank),
                                         blk_off.ctypes.data_as(C.c_void_p), idx.ctypes.data_as(C.c_void_p), _iptr(rem_ptr), _iptr(rem_col)))
    return dict(core=core, ntiles=core // 256, core_nnz=int(sizes[4]), order=order, rank=rank, blk_off=blk_off, idx=idx,
                rem_ptr=rem_ptr, rem_col=rem_col)
