"""Builds the reference's own native helper (llm/data/cores/helpers.cpp: build_location_idx, pybind11) from the
sources where they lie under /root/reference into oracle/_ref/, to check the restatements against it.

TEST INFRASTRUCTURE ONLY.  Nothing is copied: g++ compiles the reference file in place; only the resulting extension
module lands in oracle/_ref/ (git-ignored).  Needs the pybind11 headers that ship with this image.
    python -m oracle.build_ref
"""
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
REF_SRC = "/root/reference/llm/data/cores/helpers.cpp"
OUT_DIR = os.path.join(HERE, "_ref")


def build(verbose=True):
    """Returns the path of the built module, or None when the reference tree is not present (e.g. on the GPU box)."""
    if not os.path.exists(REF_SRC):
        return None
    import pybind11
    os.makedirs(OUT_DIR, exist_ok=True)
    out = os.path.join(OUT_DIR, "helpers" + sysconfig.get_config_var("EXT_SUFFIX"))
    cmd = ["g++", "-O2", "-shared", "-fPIC", "-std=c++14", "-I" + pybind11.get_include(), "-I" + sysconfig.get_paths()["include"],
           REF_SRC, "-o", out]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("building the reference helper failed:\n" + r.stdout)
    if verbose:
        print("built", out)
    return out


def load():
    """Imports oracle/_ref/helpers if it has been built; None otherwise."""
    import importlib.util
    path = os.path.join(OUT_DIR, "helpers" + sysconfig.get_config_var("EXT_SUFFIX"))
    if not os.path.exists(path):
        return None
    spec = importlib.util.spec_from_file_location("helpers", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


if __name__ == "__main__":
    sys.exit(0 if build() else 1)
