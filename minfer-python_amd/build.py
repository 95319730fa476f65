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


def asm_hazards(asm_text):
    """Distances the compiler cannot keep because one end is inside an asm statement, looked for in the device code:
    (1) a global->LDS copy (always emitted from asm here) whose scalar address pair was written by a vector instruction
        (readfirstlane / readlane) fewer than five instructions earlier;
    (2) a matrix instruction that reads a register written inside an asm statement fewer than two instructions earlier.
    Returns a list of (function, offending instruction, the write it follows too closely)."""
    import re
    found, func, window, in_asm = [], "?", [], False
    for raw in asm_text.split("\n"):
        line = raw.strip()
        if line.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if line.startswith(";;#ASMEND"):
            in_asm = False
            continue
        if not line or line.startswith((";", "//")):
            continue
        if line.endswith(":") or (":" in line and line.split(":")[0].replace("_", "").replace(".", "").replace("$", "").isalnum() and " " not in line.split(":")[0]):
            label = line.split(":")[0]
            if not label.startswith(".L"):
                func, window = label, []
            continue   # a branch target keeps the window: whatever path leads here, these instructions may have just run
        if line.startswith("."):
            continue
        op = line.split()[0]
        if op == "global_load_lds_dwordx4":
            m = re.search(r"s\[(\d+):(\d+)\]", line)
            if m:
                pair = {int(m.group(1)), int(m.group(2))}
                states = 0   # issue slots between the write and this instruction: s_nop N fills N + 1
                for prev, _ in reversed(window):
                    if states >= 5:
                        break
                    w = re.match(r"v_read(?:first)?lane_b32 s(\d+)", prev)
                    if w and int(w.group(1)) in pair:
                        found.append((func, line, prev))
                    n = re.match(r"s_nop (\d+)", prev)
                    states += int(n.group(1)) + 1 if n else 1
        elif op.startswith("v_mfma"):
            srcs = set()
            for m in re.finditer(r"v\[(\d+):(\d+)\]", line.split(",", 1)[1] if "," in line else ""):
                srcs.update(range(int(m.group(1)), int(m.group(2)) + 1))
            for prev, prev_in_asm in window[-2:]:
                if prev_in_asm and prev.startswith("v_"):
                    d = re.match(r"\S+\s+v(\d+)", prev) or re.match(r"\S+\s+v\[(\d+):(\d+)\]", prev)
                    if d:
                        lo = int(d.group(1))
                        hi = int(d.group(2)) if d.lastindex and d.lastindex >= 2 else lo
                        if srcs.intersection(range(lo, hi + 1)):
                            found.append((func, line, prev))
        window.append((line, in_asm))
        if len(window) > 8:
            window.pop(0)
    return found


def build_core(verbose=False):
    os.makedirs(LIB_DIR, exist_ok=True)
    obj_dir = os.path.join(HERE, "build")
    os.makedirs(obj_dir, exist_ok=True)
    objs = [os.path.join(obj_dir, s.replace(".hip", ".o")) for s in KERNEL_SOURCES]
    asms = [os.path.join(obj_dir, s.replace(".hip", ".s")) for s in KERNEL_SOURCES]
    cmds = [["hipcc", *HIP_FLAGS, "-c", os.path.join(CSRC, s), "-o", o] for s, o in zip(KERNEL_SOURCES, objs)]
    # the same device code as text, for the scan below (the objects' code is the same compilation's)
    cmds += [["hipcc", *HIP_FLAGS, "--cuda-device-only", "-S", os.path.join(CSRC, s), "-o", a] for s, a in zip(KERNEL_SOURCES, asms)]
    with ThreadPoolExecutor(max_workers=os.cpu_count() or 8) as ex:
        outs = list(ex.map(_run, cmds))
    if verbose:
        print("".join(outs))
    for a in asms:
        with open(a) as f:
            bad = asm_hazards(f.read())
        if bad:
            raise RuntimeError("asm statement too close to an instruction that depends on it in %s:\n%s" % (
                os.path.basename(a), "\n".join("  %s: %s  <-  %s" % b for b in bad[:20])))
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
