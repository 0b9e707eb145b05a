"""Build libhpt_hip.so (the C-ABI library with the gfx950 kernels) in-tree.

    python -m hpt_amd.build            # build if sources are newer than the library
    python -m hpt_amd.build --force    # rebuild everything

Every translation unit is compiled by hipcc for gfx950 only; the per-op and
per-kind sources are compiled once per op / kind (a -D selects which) so the
objects build in parallel.
"""
from __future__ import annotations

import concurrent.futures as cf
import os
import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent
CSRC = ROOT / "csrc"
INCLUDE = ROOT.parent / "include"
OBJ = ROOT / "lib" / "obj"
LIB = ROOT / "lib" / "libhpt_hip.so"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "-std=c++17", "-O3", "--offload-arch=gfx950", "-fPIC",
    f"-I{INCLUDE}", f"-I{CSRC}",
    # keep the compiler from forming packed-FP32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    # the device code of every object is zstd-compressed inside its fat binary (the runtime
    # unpacks it when the library is loaded): a third of the size, nothing else changes
    "--offload-compress", "--offload-compression-level=16",
]

N_REDUCE_ENTRIES = 16  # 14 reduce ops + argmin + argmax
N_NORM_KINDS = 6  # softmax, log_softmax, layernorm, add+layernorm, causal softmax / log_softmax


def units():
    """(object name, source, extra flags)"""
    # (the longest compilations first: the softmax kinds and their interleaved rows)
    u = []
    for k in range(N_NORM_KINDS):
        u.append((f"norm_op_{k}.o", CSRC / "norm_op.hip", [f"-DHPT_NORM_KIND={k}"]))
        if k < 2:
            u.append((f"norm_interleaved_{k}.o", CSRC / "norm_interleaved.hip", [f"-DHPT_NORM_KIND={k}"]))
    for e in range(N_REDUCE_ENTRIES):
        u.append((f"reduce_op_{e}.o", CSRC / "reduce_op.hip", [f"-DHPT_REDUCE_ENTRY={e}"]))
    u += [("layout.o", CSRC / "layout.cpp", ["-x", "hip"]), ("api.o", CSRC / "api.hip", []),
          ("elementwise.o", CSRC / "elementwise.hip", [])]
    if (CSRC / "transpose_norm.hip").exists():
        u.append(("transpose_norm.o", CSRC / "transpose_norm.hip", []))
    return u


def _newest_header() -> float:
    hs = list(CSRC.glob("*.hpp")) + list(INCLUDE.glob("*.h"))
    return max(h.stat().st_mtime for h in hs)


def _compile(name, src, extra, force, hdr_time):
    obj = OBJ / name
    if not force and obj.exists() and obj.stat().st_mtime > max(src.stat().st_mtime, hdr_time):
        return name, 0, ""
    cmd = [HIPCC, *FLAGS, *extra, "-c", str(src), "-o", str(obj)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    return name, r.returncode, err


def build(force: bool = False, jobs: int | None = None, verbose: bool = True) -> Path:
    OBJ.mkdir(parents=True, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)
    hdr_time = _newest_header()
    us = units()
    failed = False
    with cf.ThreadPoolExecutor(max_workers=jobs) as ex:
        futs = [ex.submit(_compile, n, s, e, force, hdr_time) for n, s, e in us]
        for f in cf.as_completed(futs):
            name, rc, err = f.result()
            if err.strip() and verbose:
                print(f"[{name}]\n{err}", file=sys.stderr)
            if rc != 0:
                failed = True
    if failed:
        raise RuntimeError("hipcc failed; see messages above")
    objs = [str(OBJ / n) for n, _, _ in us]
    newest_obj = max(Path(o).stat().st_mtime for o in objs)
    if force or not LIB.exists() or LIB.stat().st_mtime < newest_obj:
        cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", *objs, "-o", str(LIB)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n" + r.stderr)
    build_host_test(force)
    return LIB


HOST_TEST_SRC = ROOT.parent / "tests" / "cpp" / "host_api_test.cpp"
HOST_TEST_BIN = ROOT / "lib" / "host_api_test"


def build_host_test(force: bool = False) -> Path:
    """The C++ host side (include/hpt_hip.hpp) and its device test program, compiled with the host
    compiler alone: the ABI is plain C, no HIP header is needed above it."""
    deps = [HOST_TEST_SRC, INCLUDE / "hpt_hip.hpp", INCLUDE / "hpt_hip.h", LIB]
    if not force and HOST_TEST_BIN.exists() and HOST_TEST_BIN.stat().st_mtime > max(d.stat().st_mtime for d in deps):
        return HOST_TEST_BIN
    cmd = [os.environ.get("CXX", "g++"), "-std=c++17", "-O1", "-Wall", f"-I{INCLUDE}", str(HOST_TEST_SRC),
           "-o", str(HOST_TEST_BIN), f"-L{LIB.parent}", "-lhpt_hip", "-Wl,-rpath,$ORIGIN",
           "-Wl,-rpath-link,/opt/rocm/lib"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("host test build failed:\n" + r.stderr)
    return HOST_TEST_BIN


if __name__ == "__main__":
    lib = build(force="--force" in sys.argv)
    print(lib)
