"""Builds libpcmi355.so (HIP, gfx950) in-tree.  Run: python lvd-pg_amd/build.py [--incremental]

Every source file becomes an object under build/ (compiled side by side), then one link.  A full
build recompiles everything; --incremental skips objects newer than their source and every header."""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
SOURCES = ["api.hip", "hclt_engine.hip", "hclt_queries.hip", "hclt_kld.hip", "hclt_wide.hip", "chow_liu.hip",
           "pairwise_mi_static.hip", "sparse_engine.hip", "param_rows.hip", "flow_rows.hip", "stream_probe.hip"]
OUT = os.path.join(HERE, "libpcmi355.so")
OBJ_DIR = os.path.join(HERE, "build")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
         # packed-fp32 code generation is switched off for every device function
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stderr=subprocess.PIPE, text=True)
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if err.strip():
        print(err, file=sys.stderr)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed: " + " ".join(cmd[-3:]))


def build_library(verbose=True, incremental=False):
    csrc = os.path.join(HERE, "csrc")
    os.makedirs(OBJ_DIR, exist_ok=True)
    headers = [os.path.join(csrc, f) for f in os.listdir(csrc) if f.endswith((".hpp", ".h"))]
    headers.append(os.path.join(os.path.dirname(HERE), "include", "pcmi355.h"))
    newest_header = max(os.path.getmtime(h) for h in headers)
    jobs, objs = [], []
    for s in SOURCES:
        src = os.path.join(csrc, s)
        obj = os.path.join(OBJ_DIR, s + ".o")
        objs.append(obj)
        fresh = os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(src), newest_header)
        if not (incremental and fresh):
            jobs.append(["hipcc", *FLAGS, "-c", "-o", obj, src])
    with ThreadPoolExecutor(max_workers=8) as pool:
        list(pool.map(lambda c: _run(c, verbose), jobs))
    _run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", OUT, *objs], verbose)
    return OUT


if __name__ == "__main__":
    build_library(incremental="--incremental" in sys.argv[1:])
