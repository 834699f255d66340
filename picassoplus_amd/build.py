"""Build libpicasso_mesh.so (hand-written HIP for gfx950) in-tree with hipcc.

Usage: ``python -m picassoplus_amd.build`` -- cross-compiles without a GPU.
"""
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
LIB = os.path.join(CSRC, "libpicasso_mesh.so")
SOURCES = ["mesh_api.cpp", "mesh_csr.hip", "mesh_rows.hip", "mesh_f2v_mfma.hip", "mesh_f2f.hip", "mesh_f2f16x3.hip", "mesh_f2f16h2.hip", "mesh_f2f_narrow.hip", "mesh_dense.hip", "mesh_texture.hip", "mesh_decimate.hip", "pcloud_query.hip", "pcloud_ops.hip"]
ARCH = "gfx950"
# packed-fp32 code generation stays off for every device translation unit
FLAGS = ["--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libpicasso_mesh.so cannot be built")
    return exe


def _compile(src):
    obj = os.path.join(CSRC, "build", os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc()] + FLAGS + ["-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (src, err))
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose=False):
    """Compile every source and link the shared library; returns its path."""
    os.makedirs(os.path.join(CSRC, "build"), exist_ok=True)
    with ThreadPoolExecutor(max_workers=4) as pool:
        objs = list(pool.map(_compile, SOURCES))
    cmd = [_hipcc(), "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", LIB] + objs
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n" + res.stderr)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build(verbose=True)
