"""Builds the gfx950 shared library `libsfm_attn.so` in-tree (next to this file) with hipcc.

Run as `python self-forcing_amd/build.py` or through `__graft_entry__.build()`.  hipcc
cross-compiles gfx950 code objects without a GPU present.
"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libsfm_attn.so")
SOURCES = ["sfm_api.hip", "monarch_mfma.hip", "monarch_fused.hip", "monarch_generic.hip", "dense_attn.hip", "dense_attn_bwd.hip", "qk_prologue.hip", "block_fused.hip", "block_gemm.hip",
           "monarch_bwd_gemm.hip", "monarch_bwd_left.hip", "monarch_bwd_right.hip", "probe.hip", "conv3d_cl.hip"]

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed-fp32 VALU forms are disabled for every device translation unit
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found")
    return exe


def build(verbose=True, jobs=4):
    """Compiles every source (always, even when a library is already there) and links the .so."""
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    cc = hipcc()
    procs = []
    objs = []
    for src in SOURCES:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        objs.append(obj)
        cmd = [cc] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        if len(procs) >= jobs:
            _drain(procs, verbose)
    _drain(procs, verbose)
    cmd = [cc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB + ".tmp"] + objs
    out = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if out.returncode:
        raise RuntimeError("link failed:\n" + out.stdout)
    os.replace(LIB + ".tmp", LIB)
    if verbose:
        print("built", LIB)
    return LIB


def _drain(procs, verbose):
    while procs:
        src, p = procs.pop(0)
        out, _ = p.communicate()
        if p.returncode:
            raise RuntimeError(f"hipcc failed on {src}:\n{out}")
        if verbose and out.strip():
            lines = [l for l in out.splitlines() if "packed-fp32-ops" not in l and l.strip()]
            if lines:
                print("\n".join(lines))


if __name__ == "__main__":
    build()
    sys.exit(0)
