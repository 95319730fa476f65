"""Builds the two in-tree shared objects with hipcc, for gfx950 only.

  lib/libminfer_attn.so                      HIP kernels behind the C ABI of include/minfer_attn.h
  minfer/kernels/torch_ext/_C.so             PyTorch stable-ABI op registration calling that C ABI

The reference builds its extension through torch's CUDAExtension (reference: setup.py:65-84);
here hipcc is driven directly so that no source translation step is involved.
"""
import os
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
EXT_DIR = os.path.join(HERE, "minfer", "kernels", "torch_ext")
CORE_SO = os.path.join(LIB_DIR, "libminfer_attn.so")
EXT_SO = os.path.join(EXT_DIR, "_C.so")

HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-I" + os.path.join(ROOT, "include"), "-I" + CSRC]
KERNEL_SOURCES = ["attn_prefill.hip", "attn_decode.hip", "rope.hip", "rmsnorm.hip", "gemm.hip", "quant.hip", "calib.hip", "attn_api.hip"]


def _run(cmd):
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + res.stdout)
        raise RuntimeError("build step failed: " + cmd[0])
    return res.stdout


def build_core(verbose=False):
    os.makedirs(LIB_DIR, exist_ok=True)
    obj_dir = os.path.join(HERE, "build")
    os.makedirs(obj_dir, exist_ok=True)
    objs = [os.path.join(obj_dir, s.replace(".hip", ".o")) for s in KERNEL_SOURCES]
    cmds = [["hipcc", *HIP_FLAGS, "-c", os.path.join(CSRC, s), "-o", o] for s, o in zip(KERNEL_SOURCES, objs)]
    with ThreadPoolExecutor(max_workers=len(cmds)) as ex:
        outs = list(ex.map(_run, cmds))
    if verbose:
        print("".join(outs))
    _run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", CORE_SO, *objs])
    return CORE_SO


def build_torch_ext():
    import torch
    tdir = os.path.dirname(torch.__file__)
    tinc = os.path.join(tdir, "include")
    tlib = os.path.join(tdir, "lib")
    pyinc = sysconfig.get_paths()["include"]
    cmd = ["hipcc", "-O2", "-std=c++17", "-fPIC", "-shared", "-x", "c++",
           "-DUSE_ROCM", "-D__HIP_PLATFORM_AMD__", "-DPy_LIMITED_API=0x030a0000",
           "-DTORCH_TARGET_VERSION=0x020a000000000000",
           "-I" + os.path.join(ROOT, "include"), "-I" + tinc, "-I" + pyinc,
           os.path.join(CSRC, "torch_ops.cpp"), "-o", EXT_SO,
           "-L" + LIB_DIR, "-lminfer_attn", "-Wl,-rpath,$ORIGIN/../../../lib",
           "-L" + tlib, "-ltorch", "-ltorch_cpu", "-lc10", "-Wl,-rpath," + tlib]
    _run(cmd)
    return EXT_SO


def build_all(verbose=False):
    return build_core(verbose), build_torch_ext()


if __name__ == "__main__":
    for so in build_all(verbose=True):
        print("built", os.path.relpath(so, ROOT))
