"""Builds libmfsdp_hip.so (gfx950) from the HIP sources next to this file.

Usage: ``python matrix-fsdp_amd/csrc/build.py``.  hipcc cross-compiles
without a GPU; the library is written beside the package so that it is found
in-tree.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

CSRC = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(CSRC)
LIB_PATH = os.path.join(PKG, "libmfsdp_hip.so")
SOURCES = ("common.hip", "segment_copy.hip", "segment_copy_device.hip", "muon_elementwise.hip", "muon_gemm.hip", "muon.hip", "adamw.hip")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wall",
    "-Wno-unused-function",
    # keep the compiler from emitting packed fp32 arithmetic (v_pk_fma_f32 and friends).  A device-pass feature: the
    # gfx950 pass honours it (tests/test_build_flags.py compiles a probe both ways), hipcc's host pass does not know it
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the x86 host pass of every hipcc call prints this once per source for the device-only feature above
    noise = "'-packed-fp32-ops' is not a recognized feature for this target"
    out = "\n".join(line for line in proc.stdout.splitlines() if noise not in line)
    if proc.returncode != 0:
        raise RuntimeError(f"{' '.join(cmd)}\nfailed with exit code {proc.returncode}:\n{out}")
    if out.strip():
        print(out, file=sys.stderr)


def build(verbose: bool = True) -> str:
    objdir = os.path.join(CSRC, "build")
    os.makedirs(objdir, exist_ok=True)
    sources = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    objects = [os.path.join(objdir, s.replace(".hip", ".o")) for s in sources]

    def compile_one(pair):
        src, obj = pair
        _run([HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj])
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(sources))) as pool:
        list(pool.map(compile_one, zip(sources, objects)))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objects, "-o", LIB_PATH])
    if verbose:
        print(f"built {LIB_PATH} from {', '.join(sources)}")
    return LIB_PATH


if __name__ == "__main__":
    build()
