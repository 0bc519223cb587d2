"""Builds the C-ABI shared library of gfx950 kernels in-tree with hipcc."""
from __future__ import annotations

import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
SOURCES = ("elementwise.hip", "gemm.hip", "attention.hip", "sampling.hip")
LIBRARY = os.path.join(HERE, "liblfm2_hip.so")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off", "-Wno-unused",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def build(verbose: bool = False) -> str:
    """Compile every HIP source for gfx950 and link liblfm2_hip.so next to this file."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objects = []
    procs = []
    for name in SOURCES:
        obj = os.path.join(HERE, "csrc", name.replace(".hip", ".o"))
        cmd = [hipcc, *[f for f in FLAGS if f != "-shared"], "-c", os.path.join(HERE, "csrc", name), "-o", obj]
        procs.append((name, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objects.append(obj)
    for name, proc in procs:
        out, _ = proc.communicate()
        lines = [ln for ln in out.splitlines() if "packed-fp32-ops" not in ln]
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed on {name}:\n" + "\n".join(lines))
        if verbose and lines:
            print("\n".join(lines))
    link = subprocess.run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objects, "-o", LIBRARY],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if link.returncode != 0:
        raise RuntimeError("link failed:\n" + link.stdout)
    return LIBRARY


if __name__ == "__main__":
    print(build(verbose=True))
