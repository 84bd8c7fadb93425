"""Build libommx_hip.so in-tree with hipcc for gfx950.

    python -m open_ommx_serve_amd.csrc.build

Each .hip file is compiled to an object and the objects are linked into one shared
library next to the sources.  The store kernel is compiled with floating-point
contraction off: its arithmetic has to round exactly where the reference packer rounds.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libommx_hip.so")
ARCH = "gfx950"
SOURCES = {
    "ommx_store.hip": ["-ffp-contract=off"],
    "ommx_store_generic.hip": ["-ffp-contract=off"],
    "ommx_decode_ref.hip": [],
    "ommx_decode.hip": [],
    "ommx_decode_gqa4.hip": [],
    "ommx_combine.hip": [],
    "ommx_ring.hip": [],
    "ommx_merge.hip": [],
    "ommx_index.hip": [],
    "ommx_capi.hip": [],
}
COMMON = ["-O3", "-fPIC", "-std=c++17", f"--offload-arch={ARCH}",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          "-Wno-unused-command-line-argument"]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libommx_hip.so cannot be built")
    return exe


def _compile(src: str, extra) -> str:
    obj = os.path.join(HERE, src.replace(".hip", ".o"))
    cmd = [_hipcc(), *COMMON, *extra, "-c", os.path.join(HERE, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{r.stdout}\n{r.stderr}")
    noise = [ln for ln in r.stderr.splitlines()
             if ln.strip() and "packed-fp32-ops" not in ln and "not a recognized feature" not in ln]
    if noise:
        print("\n".join(noise), file=sys.stderr)
    return obj


def build(verbose: bool = True) -> str:
    with ThreadPoolExecutor(max_workers=4) as ex:
        objs = list(ex.map(lambda kv: _compile(*kv), SOURCES.items()))
    cmd = [_hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", *objs, "-o", LIB]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"built {LIB} ({os.path.getsize(LIB)} bytes)")
    return LIB


if __name__ == "__main__":
    build()
