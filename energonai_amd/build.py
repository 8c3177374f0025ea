"""Builds libenergon_hip.so (gfx950) from energonai_amd/csrc/*.hip with hipcc, and
libenergon_linear.so (host code over hipBLASLt) from csrc/linear_blaslt.cpp.

    python -m energonai_amd.build            # compile every source, link the library
    python -m energonai_amd.build --force    # recompile even if objects look fresh

The library is a plain C-ABI shared object (see include/energon_hip.h); it
links against the HIP runtime only, never against torch.  hipcc cross-compiles
for gfx950 without a GPU present.
"""
from __future__ import annotations

import argparse
import hashlib
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
INCLUDE = os.path.join(ROOT, "include")
OBJ_DIR = os.path.join(PKG_DIR, "build")
LIB_PATH = os.path.join(PKG_DIR, "libenergon_hip.so")
# host-only hipBLASLt front end for the projection GEMMs; the only piece that links more than the HIP runtime
LINEAR_SRC = os.path.join(CSRC, "linear_blaslt.cpp")
LINEAR_LIB_PATH = os.path.join(PKG_DIR, "libenergon_linear.so")

ARCH = "gfx950"
# packed fp32 VALU ops are switched off for device code on purpose (they have
# produced silently wrong results on this hardware); the host pass warns that it
# does not know the feature, which is harmless.
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
    f"-I{INCLUDE}", f"-I{CSRC}",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the HIP extension cannot be built")
    return exe


def sources() -> list:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _digest(paths) -> str:
    h = hashlib.sha256()
    for path in sorted(paths, key=os.path.basename):
        h.update(os.path.basename(path).encode() + b"\0")
        with open(path, "rb") as f:
            h.update(f.read())
        h.update(b"\0")
    return h.hexdigest()[:32]


def source_hash() -> str:
    """Digest of every file libenergon_hip.so is compiled from.  The build stores it in the library
    (``en_source_hash``); loading compares the two, so a library older than the sources next to it is
    refused instead of silently tested."""
    return _digest(sources() + [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")] +
                   [os.path.join(INCLUDE, "energon_hip.h")])


def linear_source_hash() -> str:
    return _digest([LINEAR_SRC, os.path.join(INCLUDE, "energon_linear.h")])


def _stale(src: str, obj: str) -> bool:
    if not os.path.exists(obj):
        return True
    t = os.path.getmtime(obj)
    deps = [src, os.path.join(INCLUDE, "energon_hip.h")] + [
        os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    return any(os.path.getmtime(d) > t for d in deps)


def _compile(src: str, force: bool, verbose: bool) -> str:
    obj = os.path.join(OBJ_DIR, os.path.basename(src) + ".o")
    carries_hash = os.path.basename(src) == "abi.hip"     # recompiled every time: the digest changes with any source
    if force or carries_hash or _stale(src, obj):
        cmd = [_hipcc()] + HIPCC_FLAGS + ([f'-DEN_SOURCE_HASH="{source_hash()}"'] if carries_hash else []) + \
              ["-c", src, "-o", obj]
        proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed for {src}:\n{out}")
        if verbose and out.strip():
            print(out)
    return obj


def build(force: bool = True, verbose: bool = False, jobs: int = 4) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = sources()
    with ThreadPoolExecutor(max_workers=max(1, min(jobs, len(srcs)))) as pool:
        objs = list(pool.map(lambda s: _compile(s, force, verbose), srcs))
    tmp = LIB_PATH + ".tmp"
    cmd = [_hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", tmp] + objs
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("link failed:\n" + proc.stdout)
    os.replace(tmp, LIB_PATH)
    build_linear()
    return LIB_PATH


def build_linear() -> str:
    rocm_lib = os.path.join(os.path.dirname(os.path.dirname(os.path.realpath(_hipcc()))), "lib")
    tmp = LINEAR_LIB_PATH + ".tmp"
    cmd = [_hipcc(), "-O2", "-std=c++17", "-fPIC", "-shared", f"-I{INCLUDE}",
           f'-DEN_SOURCE_HASH="{linear_source_hash()}"', LINEAR_SRC, "-o", tmp,
           f"-L{rocm_lib}", "-L/opt/rocm/lib", "-lhipblaslt", "-lamdhip64"]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("building libenergon_linear.so failed:\n" + proc.stdout)
    os.replace(tmp, LINEAR_LIB_PATH)
    return LINEAR_LIB_PATH


def ensure_built() -> None:
    """Builds the two libraries if, and only if, one of them is missing (tests, the smoke run and the
    benchmark load what is there; they compile only when nothing is)."""
    if not (os.path.exists(LIB_PATH) and os.path.exists(LINEAR_LIB_PATH)):
        build(force=False)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--force", action="store_true", help="recompile every source")
    ap.add_argument("-v", "--verbose", action="store_true")
    ap.add_argument("-j", "--jobs", type=int, default=4)
    ns = ap.parse_args(argv)
    path = build(force=ns.force, verbose=ns.verbose, jobs=ns.jobs)
    print(path)
    return 0


if __name__ == "__main__":
    sys.exit(main())
