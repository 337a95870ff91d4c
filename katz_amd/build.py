"""Build the katz_hip shared library (hand-written HIP for gfx950) in-tree with hipcc.

`python -m katz_amd.build` compiles every `csrc/*.hip` translation unit to an object and links
`katz_amd/libkatz_hip.so`.  The library has a plain C ABI (include/katz_hip.h) and does not link
against torch.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_PATH = PKG_DIR / "libkatz_hip.so"
BUILD_DIR = PKG_DIR / "build"

# -packed-fp32-ops is switched off: the compiler must not form v_pk_*_f32 from float code.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the katz_hip kernels cannot be built")
    return exe


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "not a recognized feature" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(cmd)}\n{out}")
    if out.strip():
        print(out, file=sys.stderr)


def build_library(force: bool = True, jobs: int = 8) -> Path:
    """Compile all kernels for gfx950 and link libkatz_hip.so. Returns the library path."""
    hipcc = _hipcc()
    BUILD_DIR.mkdir(exist_ok=True)
    srcs = sources()
    if not srcs:
        raise RuntimeError(f"no .hip sources under {CSRC}")
    headers = list(CSRC.glob("*.h"))
    newest_dep = max(p.stat().st_mtime for p in srcs + headers)
    if not force and LIB_PATH.exists() and LIB_PATH.stat().st_mtime >= newest_dep:
        return LIB_PATH
    objs = [BUILD_DIR / (s.stem + ".o") for s in srcs]

    def compile_one(pair):
        src, obj = pair
        _run([hipcc, *HIPCC_FLAGS, "-c", str(src), "-o", str(obj)])

    with ThreadPoolExecutor(max_workers=min(jobs, len(srcs))) as ex:
        list(ex.map(compile_one, zip(srcs, objs)))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB_PATH), *map(str, objs)])
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(force=True))
