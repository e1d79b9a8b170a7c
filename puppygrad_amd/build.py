"""Builds libpuppygrad_hip.so for gfx950 with hipcc (cross-compiles without a GPU)."""
from __future__ import annotations

import os
import subprocess
import sys
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_PATH = PKG_DIR / "libpuppygrad_hip.so"
SOURCES = ["pg_kernels.hip", "pg_decode.hip", "pg_prefill.hip", "pg_ops_dev.hip", "pg_sample.hip",
           "pg_host.cpp", "pg_assets.cpp"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# Packed-FP32 instruction selection is switched off for every device pass.
DEVICE_FLAGS = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def build_library(verbose: bool = True) -> Path:
    """Compile every source to an object, then link the shared library."""
    objs = []
    procs = []
    for src in SOURCES:
        path = CSRC / src
        if not path.exists():
            continue
        obj = CSRC / (path.stem + ".o")
        cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-x", "hip",
               *DEVICE_FLAGS, "-Wno-unused-command-line-argument", "-c", str(path), "-o", str(obj)]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
        objs.append(str(obj))
    for src, p in procs:
        out, _ = p.communicate()
        text = out.decode(errors="replace")
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{text}")
        if verbose and text.strip():
            print(text, flush=True)
    link = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB_PATH), *objs, "-lpthread"]
    if verbose:
        print(" ".join(link), flush=True)
    subprocess.run(link, check=True)
    return LIB_PATH


if __name__ == "__main__":
    build_library()
    print(f"built {LIB_PATH}")
    sys.exit(0)
