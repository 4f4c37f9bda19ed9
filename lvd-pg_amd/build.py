"""Builds libpcmi355.so (HIP, gfx950) in-tree.  Run: python lvd-pg_amd/build.py"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SOURCES = ["api.hip", "hclt_engine.hip", "hclt_queries.hip", "hclt_kld.hip", "hclt_wide.hip", "chow_liu.hip", "pairwise_mi_static.hip", "sparse_engine.hip"]
OUT = os.path.join(HERE, "libpcmi355.so")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
         # packed-fp32 code generation is switched off for every device function
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def build_library(verbose=True):
    srcs = [os.path.join(HERE, "csrc", s) for s in SOURCES if os.path.exists(os.path.join(HERE, "csrc", s))]
    cmd = ["hipcc", *FLAGS, "-o", OUT, *srcs]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stderr=subprocess.PIPE, text=True)
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if err.strip():
        print(err, file=sys.stderr)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed")
    return OUT


if __name__ == "__main__":
    build_library()
