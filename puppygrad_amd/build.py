"""Builds libpuppygrad_hip.so for gfx950 with hipcc (cross-compiles without a GPU)."""
from __future__ import annotations

import os
import subprocess
import sys
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_PATH = PKG_DIR / "libpuppygrad_hip.so"
# Development build with the persistent decode kernel's in-kernel timestamps compiled in
# (python -m puppygrad_amd.build --stamps; read by puppygrad_amd.decode_stamps).
STAMPS_LIB_PATH = PKG_DIR / "libpuppygrad_hip_stamps.so"
SOURCES = ["pg_kernels.hip", "pg_decode.hip", "pg_prefill.hip", "pg_ops_dev.hip", "pg_sample.hip",
           "pg_host.cpp", "pg_assets.cpp"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# Packed-FP32 instruction selection is switched off for every device pass.
DEVICE_FLAGS = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def build_library(verbose: bool = True, stamps: bool = False) -> Path:
    """Compile every source to an object, then link the shared library."""
    objs = []
    procs = []
    lib = STAMPS_LIB_PATH if stamps else LIB_PATH
    extra = ["-DPG_DECODE_PROF_BUILD"] if stamps else []
    for src in SOURCES:
        path = CSRC / src
        if not path.exists():
            continue
        obj = CSRC / (path.stem + (".stamps.o" if stamps else ".o"))
        cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-x", "hip",
               *DEVICE_FLAGS, *extra, "-Wno-unused-command-line-argument", "-c", str(path), "-o", str(obj)]
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
    link = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(lib), *objs, "-lpthread"]
    if verbose:
        print(" ".join(link), flush=True)
    subprocess.run(link, check=True)
    return lib


if __name__ == "__main__":
    built = build_library(stamps="--stamps" in sys.argv[1:])
    print(f"built {built}")
    sys.exit(0)
