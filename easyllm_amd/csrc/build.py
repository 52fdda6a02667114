"""Builds libezl.so (gfx950 only) in-tree with hipcc.  `python -m easyllm_amd.csrc.build`."""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
LIB_DIR = os.path.join(PKG, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libezl.so")
SOURCES = ["api.cpp", "data_index.cpp", "norm.hip", "elementwise.hip", "cross_entropy.hip", "gemm.hip", "attention.hip", "optimizer.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17",
         # packed-fp32 VALU forms are kept out of generated code on purpose
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument"]


def _compile(src):
    obj = os.path.join(LIB_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC] + FLAGS + ["-x", "hip", "-c", os.path.join(HERE, src), "-o", obj]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    return src, obj, r.returncode, r.stdout


def build(verbose=True):
    os.makedirs(LIB_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        results = list(ex.map(_compile, SOURCES))
    objs = []
    for src, obj, rc, out in results:
        msgs = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l and l.strip())
        if rc != 0:
            raise RuntimeError("hipcc failed on %s:\n%s" % (src, out))
        if verbose and msgs:
            print(msgs)
        objs.append(obj)
    # -z defs: a symbol left undefined (a kernel's host-side launch stub, say) fails the link instead of the first dlopen
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-Wl,-z,defs", "-o", LIB_PATH] + objs
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout)
    for o in objs:
        os.remove(o)
    if verbose:
        print("built", LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    build()
    sys.exit(0)
