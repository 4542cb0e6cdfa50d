"""Builds libmggx.so (gfx950) in-tree.

    python -m mgg_osdi23_amd.build [--force] [--jobs N]

Host code is compiled with g++ (OpenMP, libstdc++ parallel sort), the HIP
translation units with hipcc for gfx950 only; everything is linked into
mgg_osdi23_amd/libmggx.so next to this file.
"""
from __future__ import annotations

import argparse
import concurrent.futures
import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
BUILD = os.path.join(PKG_DIR, "build")
LIB = os.path.join(PKG_DIR, "libmggx.so")

HIP_SOURCES = ["mggx_runtime.hip", "mggx_plan.hip", "mggx_agg.hip", "mggx_dense.hip", "mggx_prep.hip", "mggx_core.hip"]
HOST_SOURCES = ["mggx_host.cpp"]
HEADERS = [os.path.join(CSRC, "mggx_internal.h"), os.path.join(CSRC, "mggx_dev.h"), os.path.join(ROOT, "include", "mggx.h")]

HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-I", os.path.join(ROOT, "include"), "-I", CSRC,
] + os.environ.get("MGGX_HIPCC_EXTRA", "").split()
HOST_FLAGS = ["-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-fopenmp", "-Wall",
              "-I", os.path.join(ROOT, "include"), "-I", CSRC]


def _newer(target: str, deps: list[str]) -> bool:
    if not os.path.exists(target):
        return False
    t = os.path.getmtime(target)
    return all(os.path.getmtime(d) <= t for d in deps)


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    if out.strip():
        print(out)


def build(force: bool = False, jobs: int = 4) -> str:
    os.makedirs(BUILD, exist_ok=True)
    tasks = []
    objs = []
    for src in HIP_SOURCES:
        s = os.path.join(CSRC, src)
        o = os.path.join(BUILD, src + ".o")
        objs.append(o)
        if force or not _newer(o, [s] + HEADERS):
            tasks.append([HIPCC] + HIP_FLAGS + ["-c", s, "-o", o])
    for src in HOST_SOURCES:
        s = os.path.join(CSRC, src)
        o = os.path.join(BUILD, src + ".o")
        objs.append(o)
        if force or not _newer(o, [s] + HEADERS):
            tasks.append(["g++"] + HOST_FLAGS + ["-c", s, "-o", o])
    with concurrent.futures.ThreadPoolExecutor(max_workers=max(1, jobs)) as ex:
        list(ex.map(_run, tasks))
    if force or tasks or not _newer(LIB, objs):
        _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs + ["-fopenmp", "-lgomp"])
    return LIB


def build_examples(force: bool = False) -> list[str]:
    """Compiles the harness programs (plain C++ against include/mgg/*.h and libmggx.so) into mgg_osdi23_amd/bin/."""
    src_dir = os.path.join(PKG_DIR, "harness")
    out_dir = os.path.join(PKG_DIR, "bin")
    os.makedirs(out_dir, exist_ok=True)
    outs = []
    hdrs = [os.path.join(src_dir, "harness_common.h")] + [
        os.path.join(ROOT, "include", "mgg", h) for h in os.listdir(os.path.join(ROOT, "include", "mgg"))]
    for name in sorted(os.listdir(src_dir)):
        if not name.endswith(".cpp"):
            continue
        src = os.path.join(src_dir, name)
        exe = os.path.join(out_dir, name[:-4])
        outs.append(exe)
        if force or not _newer(exe, [src, LIB] + hdrs):
            _run(["g++", "-O2", "-std=c++17", "-Wall", "-I", os.path.join(ROOT, "include"), "-I", src_dir, src, "-o", exe,
                  "-L", PKG_DIR, "-lmggx", "-Wl,-rpath,$ORIGIN/.."])
    return outs


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    ap.add_argument("--jobs", type=int, default=4)
    args = ap.parse_args()
    print(build(args.force, args.jobs))
    sys.exit(0)
