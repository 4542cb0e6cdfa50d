"""Shared helpers of the test-suite: seeded inputs and the parity comparison."""
from __future__ import annotations

import numpy as np

from oracle import orc

FP32_TOL = 1e-5   # |gpu - oracle| <= FP32_TOL * sum|terms|  (fp32 features)
BF16_TOL = 2e-2   # same bound for bf16 inputs with fp32 accumulation


def share_of(ptr, col, num_nodes, num_gpus, pe):
    """Range partition + local/remote split (oracle side) of rank `pe`."""
    npp, lb, ub = orc.range_partition(num_nodes, num_gpus, pe)
    lp, rp, lc, rc = orc.split_csr(ptr, col, lb, ub)
    return dict(npp=npp, lb=lb, ub=ub, ptr_l=lp, col_l=lc, ptr_r=rp, col_r=rc)


def sym_norm_scale(ptr):
    """D^-1/2 of the row degrees (self loops are already part of the graph)."""
    deg = np.diff(ptr).astype(np.float64)
    return (1.0 / np.sqrt(np.maximum(deg, 1.0))).astype(np.float32)


def assert_close_to_oracle(got, want, abs_sum, tol, what=""):
    """Element-wise |got - want| <= tol * abs_sum + tiny, and a norm-wise check per row."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    bound = tol * np.asarray(abs_sum, np.float64) + 1e-30
    err = np.abs(got - want)
    bad = err > bound
    if bad.any():
        i = np.unravel_index(np.argmax(err / bound), err.shape)
        raise AssertionError("%s: %d elements out of tolerance; worst at %s: got %r want %r bound %r" %
                             (what, int(bad.sum()), i, got[i], want[i], bound[i]))


def to_dev(a, dtype=None):
    import torch
    t = torch.from_numpy(np.ascontiguousarray(a)).cuda()
    if dtype is not None:
        t = t.to(dtype)
    return t
