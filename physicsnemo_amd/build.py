"""Build libphysattn.so for gfx950 with hipcc (in-tree, next to the sources).

Every source is compiled to an object file of its own (in parallel), then linked.  `build()` recompiles everything;
`python -m physicsnemo_amd.build --incremental` skips objects that are newer than their source and the headers.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
OBJ_DIR = os.path.join(CSRC, "build")
LIB_PATH = os.path.join(PKG_DIR, "libphysattn.so")
SOURCES = ["pa_api.hip", "pa_general.hip", "pa_mfma.hip", "pa_mlp.hip", "pa_backward.hip", "pa_gemm.hip", "pa_mfma_bwd.hip",
           "pa_mfma_staged.hip", "pa_gale.hip", "pa_flare.hip", "pa_ball_query.hip", "pa_noalloc.hip", "pa_conv.hip", "pa_rows_f32.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed-FP32 VALU forms are kept off for every kernel in this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def _headers_mtime() -> float:
    hdrs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    hdrs.append(os.path.join(os.path.dirname(PKG_DIR), "include", "physattn.h"))
    return max(os.path.getmtime(h) for h in hdrs if os.path.exists(h))


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{out}")
    if verbose and out.strip():
        print(out)


def build(verbose: bool = True, incremental: bool = False, jobs: int | None = None) -> str:
    """Compile every HIP source and link them into one shared library; returns its path.  Raises on failure."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    hdr_time = _headers_mtime()
    todo, objs = [], []
    for s in srcs:
        src, obj = os.path.join(CSRC, s), os.path.join(OBJ_DIR, s + ".o")
        objs.append(obj)
        fresh = (incremental and os.path.exists(obj) and os.path.getmtime(obj) > os.path.getmtime(src)
                 and os.path.getmtime(obj) > hdr_time)
        if not fresh:
            todo.append([hipcc, *HIPCC_FLAGS, "-c", src, "-o", obj])
    jobs = jobs or min(len(todo) or 1, max(1, min(16, os.cpu_count() or 1)))
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(lambda c: _run(c, verbose), todo))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB_PATH + ".tmp"], verbose)
    os.replace(LIB_PATH + ".tmp", LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    build(incremental="--incremental" in sys.argv[1:])
    sys.exit(0)
