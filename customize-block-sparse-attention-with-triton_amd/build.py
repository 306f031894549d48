"""Builds libbsattn.so (gfx950 HIP kernels + C ABI) in-tree with hipcc.

Usage: python build.py [--force]
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
LIB = os.path.join(HERE, "fa2_custom_mask", "libbsattn.so")
SOURCES = ["api.hip", "mask_index.hip", "attn_fwd.hip", "attn_fwd_pair.hip", "attn_bwd.hip", "reorder.hip"]
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-I" + INCLUDE, "-I" + CSRC,
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",   # no packed fp32 VALU ops
         "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option"]


def build(force=True, verbose=False):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objs = []
    procs = []
    for src in SOURCES:
        s = os.path.join(CSRC, src)
        o = os.path.join(CSRC, src.replace(".hip", ".o"))
        objs.append(o)
        deps = [s] + [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")] + \
               [os.path.join(INCLUDE, "bsattn.h")]
        if not force and os.path.exists(o) and all(os.path.getmtime(o) > os.path.getmtime(d) for d in deps):
            continue
        cmd = [hipcc] + FLAGS + ["-c", s, "-o", o]
        if verbose:
            print(" ".join(cmd))
        procs.append((src, subprocess.Popen(cmd, stderr=subprocess.PIPE, text=True)))
    for src, p in procs:
        _, err = p.communicate()
        err = "\n".join(l for l in err.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            raise RuntimeError("hipcc failed on %s:\n%s" % (src, err))
        if verbose and err.strip():
            print(err)
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv, verbose=True))
