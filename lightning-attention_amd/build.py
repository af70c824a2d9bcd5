"""Builds liblightning_attn_hip.so (gfx950) with plain hipcc: no torch headers.

    python lightning-attention_amd/build.py [--jobs N]

The library lands next to the Python package (lightning_attn/_C/) so that the
ctypes loader finds it in-tree.
"""
import argparse
import concurrent.futures as cf
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build", "obj")
OUT_DIR = os.path.join(HERE, "lightning_attn", "_C")
OUT = os.path.join(OUT_DIR, "liblightning_attn_hip.so")
OUT_TORCH = os.path.join(OUT_DIR, "liblightning_attn_torch.so")
SOURCES = ["la_api.hip", "la_sweep.hip", "la_sweep_pipe.hip", "la_sweep_pipe_split.hip", "la_sweep_f32.hip", "srmsnorm.hip", "norm_gate.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unknown-warning-option", "-Wno-unused-command-line-argument",
    "-I", os.path.join(ROOT, "include"), "-I", CSRC,
]


def _hipcc():
    for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if c and (os.path.isabs(c) and os.path.exists(c) or not os.path.isabs(c)):
            return c
    raise RuntimeError("hipcc not found")


def _compile(src):
    obj = os.path.join(OBJ, src.replace(".hip", ".o"))
    cmd = [_hipcc(), *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, r.stdout + r.stderr))
    return obj


def _build_torch_binding():
    """liblightning_attn_torch.so: the operators as C++ autograd functions over the C ABI (csrc/torch_binding.cpp).
    Host code only (no device code, no hipify): g++ against PyTorch's headers, linked to the kernel library."""
    import torch
    from torch.utils import cpp_extension as ce

    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-O2", "-fPIC", "-shared", "-std=c++17", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI), "-Wno-deprecated-declarations"]
    for inc in ce.include_paths() + ["/opt/rocm/include", os.path.join(ROOT, "include")]:
        cmd += ["-isystem" if "torch" in inc or "rocm" in inc else "-I", inc]
    cmd += [os.path.join(CSRC, "torch_binding.cpp"), "-L", tlib, "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch",
            "-L", OUT_DIR, "-llightning_attn_hip", "-Wl,-rpath,$ORIGIN", "-o", OUT_TORCH]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("torch binding failed to build:\n" + r.stdout + r.stderr)
    return OUT_TORCH


def build(jobs=4, verbose=True, torch_binding=True):
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(OUT_DIR, exist_ok=True)
    with cf.ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(_compile, SOURCES))
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", OUT]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout + r.stderr)
    if verbose:
        print("built", OUT)
    if torch_binding:
        _build_torch_binding()
        if verbose:
            print("built", OUT_TORCH)
    return OUT


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--jobs", type=int, default=4)
    ap.add_argument("--no-torch-binding", action="store_true", help="kernel library only")
    a = ap.parse_args()
    build(a.jobs, torch_binding=not a.no_torch_binding)
