"""Builds libkascade_hip.so (gfx950) from kascade_amd/csrc with hipcc.

The library is built in-tree (kascade_amd/libkascade_hip.so).  ``build()``
always recompiles; ``ensure_built()`` compiles only when no library exists.
Run ``python -m kascade_amd.build`` to build from a shell.
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
LIB_PATH = PKG_DIR / "libkascade_hip.so"
SOURCES = ["capi.hip", "decode.hip", "topk.hip", "prefill.hip", "paged.hip", "diag.hip"]
ARCH = "gfx950"

# -packed-fp32-ops is switched off for device code: hipcc otherwise forms
# v_pk_*_f32 from ordinary float code.  The host pass does not know the feature
# and prints a harmless warning.
COMMON_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: libkascade_hip.so cannot be built")
    return exe


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines()
                    if "is not a recognized feature for this target" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(map(str, cmd)) + "\n" + out)
    return out


def build(verbose: bool = False, extra_flags=()) -> Path:
    hipcc = _hipcc()
    objdir = PKG_DIR / "build"
    objdir.mkdir(exist_ok=True)
    objs = []

    def compile_one(src):
        obj = objdir / (src + ".o")
        out = _run([hipcc, *COMMON_FLAGS, *extra_flags, "-c", str(CSRC / src), "-o", str(obj)])
        if verbose and out.strip():
            print(out)
        return obj

    with ThreadPoolExecutor(max_workers=min(4, len(SOURCES))) as ex:
        objs = list(ex.map(compile_one, SOURCES))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-Wno-unused-command-line-argument",
          *map(str, objs), "-o", str(tmp)])
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


def ensure_built() -> Path:
    if not LIB_PATH.exists():
        build()
    return LIB_PATH


if __name__ == "__main__":
    path = build(verbose=True, extra_flags=sys.argv[1:])
    print(path)
