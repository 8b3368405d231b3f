"""Builds libiree_uk_amd.so (plain-C host layer + HIP kernels) for gfx950.

Run as ``python -m iree_amd.build``. hipcc cross-compiles without a GPU.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "obj")
LIB = os.path.join(HERE, "libiree_uk_amd.so")

HIP_SOURCES = ["mmt4d_mfma_s16.hip", "mmt4d_mfma_s8s4.hip",
               "uk_runtime.hip", "uk_probe.hip", "pack_unpack.hip", "pack_tr.hip",
               "mmt4d_generic.hip", "mmt4d_dot2.hip", "conv_nchwc.hip", "mmt4d_mfma.hip", "mmt4d_dispatch.hip"]
# mmt4d_mfma_inst.hip once per (element type, class of tile row widths): the
# kernel instantiations of one pair per object file, built in parallel.
MFMA_TYPES = {"s8": "kS8", "f16": "kF16", "bf16": "kBF16", "f16f16": "kF16F16",
              "bf16bf16": "kBF16BF16", "f32": "kF32", "f8": "kF8"}
MFMA_ROW_CLASSES = {"f32": (4, 8, 16), "f8": (16,)}
MFMA_INSTANCES = [(t, e, rb) for t, e in MFMA_TYPES.items()
                  for rb in MFMA_ROW_CLASSES.get(t, (2, 4, 8, 16))]
C_SOURCES = ["uk_host.c", "uk_plugin.c"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"

HIP_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-fPIC", "-std=c++17",
    "-fvisibility=hidden", "-ffp-contract=off",
    # hipcc -O3 may form packed-f32 ops from ordinary float code; keep them off.
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    f"-I{os.path.join(ROOT, 'include')}", f"-I{CSRC}",
]
C_FLAGS = ["-std=c11", "-O2", "-fPIC", "-fvisibility=hidden", "-Wall", "-Wextra",
           f"-I{os.path.join(ROOT, 'include')}", f"-I{CSRC}"]


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + r.stdout)
        raise RuntimeError(f"build step failed: {cmd[0]} {cmd[-1]}")
    # -packed-fp32-ops is unknown to the host pass; that warning is harmless.
    out = "\n".join(l for l in r.stdout.splitlines()
                    if "packed-fp32-ops" not in l and l.strip())
    if out:
        sys.stderr.write(out + "\n")


def build(verbose: bool = False) -> str:
    os.makedirs(OBJ, exist_ok=True)
    jobs = []
    objs = []
    for s in HIP_SOURCES:
        o = os.path.join(OBJ, s + ".o")
        objs.append(o)
        jobs.append([HIPCC, *HIP_FLAGS, "-c", os.path.join(CSRC, s), "-o", o])
    for t, e, rb in MFMA_INSTANCES:
        o = os.path.join(OBJ, f"mmt4d_mfma_inst_{t}_rb{rb}.o")
        objs.append(o)
        # the longest compilations first
        jobs.insert(0, [HIPCC, *HIP_FLAGS, f"-DUK_INST_ELEM={e}", f"-DUK_INST_RBC={rb}",
                        f"-DUK_INST_NAME=launch_{t}_rb{rb}", "-c",
                        os.path.join(CSRC, "mmt4d_mfma_inst.hip"), "-o", o])
    for s in C_SOURCES:
        o = os.path.join(OBJ, s + ".o")
        objs.append(o)
        jobs.append(["gcc", *C_FLAGS, "-c", os.path.join(CSRC, s), "-o", o])
    with ThreadPoolExecutor(max_workers=min(8, len(jobs))) as ex:
        list(ex.map(_run, jobs))
    _run([HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", LIB, *objs])
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build(verbose=True)
