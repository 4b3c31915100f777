"""Builds liblvx.so (the gfx950 kernels + C ABI) in-tree with hipcc.

    python lv-xattn_amd/build.py [--force] [--verbose]

hipcc cross-compiles for gfx950 without a GPU.  The library lands next to the
Python host package (lv-xattn_amd/lv_xattn/liblvx.so) so that it travels with
the source tree.
"""
from __future__ import annotations

import argparse
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT_DIR = os.path.join(HERE, "lv_xattn")
BUILD_DIR = os.path.join(HERE, "build")
LIB = os.path.join(OUT_DIR, "liblvx.so")

SOURCES = ["lvx_api.hip", "lvx_fwd.hip", "lvx_bwd.hip", "lvx_rowwise.hip", "lvx_gemm.hip"]

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    # keep the compiler from forming packed-fp32 VALU ops out of scalar float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA results in arch VGPRs (the VALU reads them without copies); the
    # register allocator then parks long-lived MFMA operands in AGPRs instead
    "-mllvm", "-amdgpu-mfma-vgpr-form",
    "-Wno-unused-command-line-argument", "-Wno-inline-asm",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; liblvx.so cannot be built")
    return exe


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in r.stderr.splitlines() if noise not in l)
    if r.returncode != 0:
        raise RuntimeError(f"command failed: {' '.join(cmd)}\n{r.stdout}\n{err}")
    if verbose and err.strip():
        print(err)


# hand-scheduled inner loops: (generator, arguments, include file it writes)
GENERATED = [("gen_fwd_loop.py", ["bf16"], "lvx_fwd_loop_bf16.inc"),
             ("gen_fwd_loop_wide.py", [], "lvx_fwd_loop_wide.inc"),
             ("gen_bwd_loop.py", ["p"], "lvx_bwd_loop_p.inc"),
             ("gen_bwd_loop.py", ["d"], "lvx_bwd_loop_d.inc"),
             ("gen_gemm_loop.py", ["bp"], "lvx_gemm_loop_bp.inc"),
             ("gen_gemm_loop.py", ["bt"], "lvx_gemm_loop_bt.inc")]


def generate() -> None:
    """Runs the loop generators; an include file is rewritten only when its text changes."""
    for gen, args, out in GENERATED:
        r = subprocess.run([sys.executable, os.path.join(CSRC, gen), *args], capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"{gen} failed:\n{r.stdout}\n{r.stderr}")
        path = os.path.join(CSRC, out)
        if not os.path.exists(path) or open(path).read() != r.stdout:
            with open(path, "w") as f:
                f.write(r.stdout)


def build(force: bool = True, verbose: bool = False, extra_flags=()) -> str:
    os.makedirs(BUILD_DIR, exist_ok=True)
    cc = hipcc()
    generate()
    headers = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".hpp", ".inc"))]
    headers.append(os.path.join(HERE, "..", "include", "lvx.h"))
    newest_hdr = max(os.path.getmtime(h) for h in headers)
    objs, jobs = [], []
    for src in SOURCES:
        s = os.path.join(CSRC, src)
        o = os.path.join(BUILD_DIR, src.replace(".hip", ".o"))
        objs.append(o)
        stale = force or not os.path.exists(o) or os.path.getmtime(o) < max(os.path.getmtime(s), newest_hdr)
        if stale:
            jobs.append([cc, *FLAGS, *extra_flags, "-c", s, "-o", o])
    with ThreadPoolExecutor(max_workers=min(8, max(1, len(jobs)))) as ex:
        list(ex.map(lambda c: _run(c, verbose), jobs))
    if jobs or not os.path.exists(LIB):
        _run([cc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", *objs, "-o", LIB], verbose)
    return LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    ap.add_argument("--verbose", action="store_true")
    a = ap.parse_args()
    print(build(force=a.force, verbose=a.verbose))
