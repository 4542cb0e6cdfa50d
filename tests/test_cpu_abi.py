"""The C ABI as a boundary: libmggx.so loads, exports exactly what include/mggx.h declares, the C++ host layer
under include/mgg/ compiles as plain C++ (no device header) and links against it, and device entry points fail
loudly -- with an error code and a message, never a silent fallback -- when no GPU is present."""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest

from mgg_osdi23_amd import host

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "mggx.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mggx_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(host.LIB_PATH)
    names = declared_symbols()
    assert len(names) >= 35
    for n in names:
        assert hasattr(lib, n), "libmggx.so does not export %s" % n
    assert sorted(host.EXPORTS) == names, "host.EXPORTS and include/mggx.h disagree"
    out = subprocess.run(["nm", "-D", "--defined-only", host.LIB_PATH], capture_output=True, text=True, check=True).stdout
    exported = {l.split()[-1] for l in out.splitlines() if " T " in l}
    stray = {s for s in exported if not s.startswith("mggx_") and not s.startswith("_")}
    assert not stray, "unexpected public symbols: %s" % sorted(stray)
    assert lib.mggx_version and host.lib().mggx_version().startswith(b"mggx")


def test_header_is_plain_c(tmp_path):
    src = tmp_path / "t.c"
    src.write_text('#include "mggx.h"\nint main(void){ mggx_agg_opts o = {0}; (void)o; return MGGX_OK; }\n')
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"), "-c", str(src), "-o",
                    str(tmp_path / "t.o")], check=True)


def test_cpp_host_layer_compiles_and_links_without_device_headers(tmp_path):
    src = tmp_path / "dropin.cpp"
    src.write_text(r'''
#include <limits>
#include "mgg/graph.h"
#include "mgg/csr_formatter.h"
#include "mgg/neighbor_utils.h"
#include "mgg/layer_new.h"
#include "mgg/gnn_layer.h"
#ifdef __HIP__
#error "the host layer must not need a device compiler"
#endif
int main() {
    std::vector<int> ptr = {0, 3, 3, 8, 9}, col = {0, 1, 3, 0, 1, 2, 3, 2, 1};
    auto s = split_CSR<int>(ptr, col, 0, 2);
    auto p = build_part<int>("t", ptr, 4, 2);
    std::vector<long> lptr(ptr.begin(), ptr.end()), lcol(col.begin(), col.end());
    auto s2 = split_CSR<long>(lptr, lcol, 0L, 2L);
    auto p2 = build_part<long>("t", lptr, 4L, 2L);
    bool ok = s[2].size() == 2 && s[3].size() == 1 && p[0].size() == 7 && p[2].size() == 6;
    for (size_t i = 0; i < 4; ++i) ok = ok && s[i].size() == s2[i].size();
    for (size_t i = 0; i < 3; ++i) { ok = ok && p[i].size() == p2[i].size(); for (size_t j = 0; j < p[i].size(); ++j) ok = ok && p[i][j] == (int)p2[i][j]; }
    // the device-facing wrappers must exist with the reference's signatures
    void (*f1)(float*, const float*, const nidType*, const nidType*, const nidType*, const nidType*, const nidType, const nidType,
               const int, const int, const int, const int, const int, const int) = &mgg_SAG_np_div;
    void (*f2)(float*, const float*, const nidType*, const nidType*, const nidType*, const nidType*, const nidType, const nidType,
               const int, const int, const int, const int, const int, const int, float) = &mgg_GIN_np_div;
    void (*f3)(dense_param_beg*) = &dense_beg_forward;
    void (*f4)(softmax_new_param*) = &softmax_new_forward;
    void (*f5)(sparse_param_hidden*) = &sparse_hidden_forward;
    void (*f6)(float*, const float*, const int*, const int*, const int*, const int*, const int, const int, const int, const int,
               const int, const int, const int) = &SAG_host<int, float, int>;
    return (ok && f1 && f2 && f3 && f4 && f5 && f6) ? 0 : 1;
}
''')
    exe = tmp_path / "dropin"
    subprocess.run(["g++", "-std=c++17", "-Wall", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe), "-L",
                    os.path.dirname(host.LIB_PATH), "-lmggx", "-Wl,-rpath," + os.path.dirname(host.LIB_PATH)], check=True)
    r = subprocess.run([str(exe)], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr


def test_product_sources_do_not_touch_the_oracle():
    """The shipped package and headers must not import, include, link or load anything under oracle/."""
    bad = []
    for base in (os.path.join(ROOT, "mgg_osdi23_amd"), os.path.join(ROOT, "include")):
        for d, _, files in os.walk(base):
            for f in files:
                if f.endswith((".py", ".h", ".hip", ".cpp", ".c")):
                    t = open(os.path.join(d, f), errors="ignore").read()
                    if re.search(r"\boracle\b|liborc|libmgg_ref|orc_[a-z]", t):
                        bad.append(os.path.join(d, f))
    assert not bad, bad


def test_device_calls_fail_loudly_without_a_gpu():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    lib = host.lib()
    assert lib.mggx_init(0) == -2 and b"HIP" in lib.mggx_last_error() or b"device" in lib.mggx_last_error()
    p = ctypes.c_void_p()
    assert lib.mggx_malloc(ctypes.byref(p), 16) != 0
    one = (ctypes.c_int * 2)(0, 0)
    f = (ctypes.c_float * 4)()
    rc = lib.mggx_sag_np_div(f, f, f, one, one, one, one, 0, 1, 4, 1, 16, 4, 1, None)
    assert rc != 0 and len(lib.mggx_last_error()) > 0
    assert lib.mggx_dense_xw(f, f, f, ctypes.c_int64(1), 1, 1, None) != 0
    assert lib.mggx_softmax_rows(f, f, ctypes.c_int64(1), 1, ctypes.c_int64(1), ctypes.c_int64(1)) != 0


def test_missing_library_raises(monkeypatch):
    monkeypatch.setattr(host, "_lib", None)
    monkeypatch.setattr(host, "LIB_PATH", "/nonexistent/libmggx.so")
    with pytest.raises(host.MggxError):
        host.lib()
