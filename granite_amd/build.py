"""Build recipe for libgranite_hip.so (gfx950 only) and the C++ host layer.

`python -m granite_amd.build` compiles everything in-tree; nothing is cached
outside the repository, so the built libraries travel with the source tree.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG = Path(__file__).resolve().parent
ROOT = PKG.parent
CSRC = PKG / "csrc"
HOST = PKG / "host"
LIBDIR = PKG / "lib"
BINDIR = PKG / "bin"

HIP_SOURCES = ["capi.hip", "kv_ops.hip", "rope.hip", "qkv_q4k.hip", "decode.hip", "decode_stream.hip", "prefill.hip", "prefill_dma.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++20",
    "-fPIC",
    "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unknown-warning-option",
    "-Wno-unused-command-line-argument",
    f"-I{ROOT / 'include'}",
    f"-I{CSRC}",
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError("hipcc not found: the gfx950 library cannot be built")


def _run(cmd: list[str]) -> None:
    print("+", " ".join(str(c) for c in cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "'-packed-fp32-ops' is not a recognized feature"
    for stream in (res.stdout, res.stderr):
        for line in stream.splitlines():
            if noise in line:
                continue
            print(line, flush=True)
    if res.returncode != 0:
        raise RuntimeError(f"command failed ({res.returncode}): {' '.join(map(str, cmd))}")


def build_hip_library(jobs: int = 4, extra_flags: list[str] | None = None) -> Path:
    """Compile the HIP sources and link granite_amd/lib/libgranite_hip.so."""
    from concurrent.futures import ThreadPoolExecutor

    hipcc = _hipcc()
    LIBDIR.mkdir(exist_ok=True)
    objdir = LIBDIR / "obj"
    objdir.mkdir(exist_ok=True)
    flags = HIPCC_FLAGS + (extra_flags or [])
    objs = []
    cmds = []
    for src in HIP_SOURCES:
        obj = objdir / (Path(src).stem + ".o")
        objs.append(obj)
        cmds.append([hipcc, *flags, "-c", str(CSRC / src), "-o", str(obj)])
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(_run, cmds))
    out = LIBDIR / "libgranite_hip.so"
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(out), *map(str, objs)])
    # the measurement aid of bench.py's mfma_calibration workload: a library of its own
    _run([hipcc, *flags, "-shared", str(CSRC / "calibration.hip"), "-o", str(LIBDIR / "libgranite_hip_calibration.so")])
    return out


def build_host_layer() -> list[Path]:
    """Compile the C++20 host layer (backend, compute API, operator, KV state)
    and its test programs with g++; they bind libgranite_hip.so through the C ABI."""
    _run(["make", "-C", str(HOST), "-B", "-j4"])
    return sorted(BINDIR.glob("*"))


def build_oracle() -> None:
    """The CPU oracle is test infrastructure; building it is not using it."""
    _run(["make", "-C", str(ROOT / "oracle")])


def build_all() -> None:
    build_hip_library()
    build_oracle()  # the host layer's test programs link it as their checker
    build_host_layer()


if __name__ == "__main__":
    build_all()
    print("build ok", file=sys.stderr)
