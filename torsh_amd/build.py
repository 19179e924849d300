"""Builds libtorsh_hipq.so (the C-ABI library) for gfx950 with hipcc.

Run as ``python -m torsh_amd.build``.  hipcc cross-compiles, so no GPU is
needed to build.  Objects are compiled in parallel and linked in-tree at
``torsh_amd/lib/libtorsh_hipq.so``.
"""
from __future__ import annotations

import concurrent.futures as cf
import os
import shutil
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
OBJ_DIR = os.path.join(PKG, "lib", "obj")
LIB_PATH = os.path.join(PKG, "lib", "libtorsh_hipq.so")

ARCH = "gfx950"

# -ffp-contract=off and the correctly rounded divide keep every f32 operation an
# individually rounded IEEE operation (bit parity with the CPU reference path);
# packed-fp32 instructions are switched off for the device pass.
HIPCC_FLAGS = [
    "-O3",
    "-std=c++17",
    f"--offload-arch={ARCH}",
    "-fPIC",
    "-fvisibility=hidden",
    "-ffp-contract=off",
    "-fno-fast-math",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-command-line-argument",
    "-I", os.path.join(ROOT, "include"),
    "-I", CSRC,
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the HIP toolchain is required to build torsh_hipq")
    return exe


def sources() -> list[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _headers_mtime() -> float:
    paths = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    paths.append(os.path.join(ROOT, "include", "torsh_hipq.h"))
    return max(os.path.getmtime(p) for p in paths)


def _compile(src: str, force: bool) -> str:
    obj = os.path.join(OBJ_DIR, os.path.basename(src) + ".o")
    if not force and os.path.exists(obj):
        if os.path.getmtime(obj) >= max(os.path.getmtime(src), _headers_mtime()):
            return obj
    cmd = [hipcc(), *HIPCC_FLAGS, "-c", src, "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{proc.stdout}\n{proc.stderr}")
    warn = "\n".join(l for l in proc.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if warn:
        sys.stderr.write(warn + "\n")
    return obj


def build(force: bool = True, jobs: int = 8) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = sources()
    with cf.ThreadPoolExecutor(max_workers=max(1, min(jobs, len(srcs)))) as pool:
        objs = list(pool.map(lambda s: _compile(s, force), srcs))
    cmd = [hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stdout}\n{proc.stderr}")
    return LIB_PATH


if __name__ == "__main__":
    incremental = "--incremental" in sys.argv
    print(build(force=not incremental))
