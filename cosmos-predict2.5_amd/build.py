"""Build recipe for the C-ABI HIP library (gfx950 only).

``build_library()`` runs hipcc on ``csrc/*.hip`` and writes ``libcosmos_attn_hip.so`` next to this
file.  The library is built ahead of time, in-tree; nothing is compiled at import or at call time.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_ROOT = os.path.dirname(PKG_DIR)
LIB_NAME = "libcosmos_attn_hip.so"
LIB_PATH = os.path.join(PKG_DIR, LIB_NAME)
SOURCES = [os.path.join(PKG_DIR, "csrc", name) for name in ("attn_fwd_jvp_gfx950.hip", "attn_bwd_gfx950.hip", "norm_rope_gfx950.hip", "block_elementwise_gfx950.hip")]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    # packed fp32 VALU ops are kept off for all device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def find_hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or add /opt/rocm/bin to PATH)")


def _run(cmd, verbose):
    if verbose:
        print("[build]", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "is not a recognized feature for this target" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{out}")
    if verbose and out.strip():
        print(out)


def build_library(verbose: bool = True, extra_flags=()) -> str:
    """Compile every source to an object (in parallel), link them into the shared library."""
    from concurrent.futures import ThreadPoolExecutor

    hipcc = find_hipcc()
    inc = ["-I", os.path.join(REPO_ROOT, "include")]
    objs = [src + ".o.tmp" for src in SOURCES]
    cmds = [[hipcc, *HIPCC_FLAGS, *extra_flags, *inc, "-c", src, "-o", obj] for src, obj in zip(SOURCES, objs)]
    try:
        with ThreadPoolExecutor(max_workers=len(cmds)) as pool:
            list(pool.map(lambda c: _run(c, verbose), cmds))
        _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB_PATH + ".tmp"], verbose)
    finally:
        for obj in objs:
            if os.path.exists(obj):
                os.remove(obj)
    os.replace(LIB_PATH + ".tmp", LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose="-q" not in sys.argv))
