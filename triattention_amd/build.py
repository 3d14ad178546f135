"""Builds libtriattention_hip.so in-tree with hipcc for gfx950.

Usage:  python -m triattention_amd.build
"""
from __future__ import annotations

import hashlib
import os
import re
import shutil
import subprocess
import sys
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
INCLUDE = PKG.parent / "include"
LIB_NAME = "libtriattention_hip.so"
LIB_PATH = PKG / LIB_NAME
SOURCES = ["tri_capi.hip", "tri_score.hip", "tri_fused.hip", "tri_fused_mfma.hip", "tri_select.hip", "tri_compact.hip", "tri_calib.hip"]

# Packed fp32 instructions are switched off on purpose: hipcc forms them from
# ordinary float code and some forms have given wrong results on this hardware.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(exe).exists():
        raise RuntimeError("hipcc not found; ROCm is required to build the gfx950 kernels")
    return exe


def source_digest() -> str:
    """SHA-256 over everything the library is built from: every file under csrc/ and include/ (name
    and content) and the compiler flags.  build() compiles it into the library."""
    h = hashlib.sha256()
    files = sorted(p for d in (CSRC, INCLUDE) for p in d.iterdir() if p.suffix in (".hip", ".h"))
    for path in files:
        h.update(path.name.encode() + b"\0" + path.read_bytes() + b"\0")
    h.update(" ".join(HIPCC_FLAGS).encode())
    return h.hexdigest()


def built_digest(lib: Path | None = None) -> str | None:
    """The digest compiled into a built library (read from the file's bytes: nothing is loaded), or
    None when the file is missing or carries none."""
    lib = lib or LIB_PATH
    if not lib.exists():
        return None
    m = re.search(rb"TRI_SOURCE_DIGEST=([0-9a-f]{64})", lib.read_bytes())
    return m.group(1).decode() if m else None


def stale() -> str | None:
    """Why the built library does not belong to the sources next to it (None: it does)."""
    if not LIB_PATH.exists():
        return f"{LIB_PATH} is missing"
    have, want = built_digest(), source_digest()
    if have != want:
        return (f"{LIB_PATH} was built from other sources (digest {have and have[:12]} in the library, "
                f"{want[:12]} for csrc/ + include/ + flags now)")
    return None


def build(verbose: bool = True, jobs: int | None = None) -> Path:
    """Compile every .hip source and link the shared library; always recompiles."""
    objdir = PKG / "build"
    objdir.mkdir(exist_ok=True)
    jobs = jobs or min(len(SOURCES), os.cpu_count() or 1, 8)
    procs = []
    objs = []
    digest = source_digest()
    for src in SOURCES:
        obj = objdir / (Path(src).stem + ".o")
        objs.append(str(obj))
        cmd = [hipcc(), *HIPCC_FLAGS, f"-I{INCLUDE}", f"-I{CSRC}", "-c", str(CSRC / src), "-o", str(obj)]
        if src == "tri_capi.hip":
            cmd.insert(-4, f'-DTRI_SOURCE_DIGEST="{digest}"')
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        if len(procs) >= jobs:
            _drain(procs, verbose)
    _drain(procs, verbose)
    link = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", str(LIB_PATH)]
    if verbose:
        print(" ".join(link), flush=True)
    subprocess.run(link, check=True)
    return LIB_PATH


def ensure_built(verbose: bool = False) -> Path:
    """For tests, the smoke run and the benchmark: build the library when there is none **or when
    the one that is there was built from other sources** (the digest of csrc/, include/ and the flags
    is compiled into the library, so this does not depend on file times), and say so; otherwise
    leave what is built alone.  The product itself never calls this: ``_lib.load()`` raises when
    the library is missing."""
    why = stale()
    if why is not None:
        print(f"triattention_amd.build: {why}; building", file=sys.stderr, flush=True)
        build(verbose=verbose)
    return LIB_PATH


def _drain(procs, verbose):
    while procs:
        src, p = procs.pop(0)
        out, _ = p.communicate()
        # hipcc's host pass does not know the packed-fp32 feature name and says so; harmless.
        out = "\n".join(l for l in out.splitlines() if "is not a recognized feature" not in l)
        if out.strip() and verbose:
            print(out, flush=True)
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{out}")


if __name__ == "__main__":
    build()
    print("built", LIB_PATH)
    sys.exit(0)
