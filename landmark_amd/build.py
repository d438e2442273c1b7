"""Builds liblandmark_hip.so (the C-ABI library) for gfx950 with hipcc.

hipcc cross-compiles without a GPU; the shared object is written next to this file so
that it travels with the source tree.  Flags: no floating-point contraction (the
geometry must round like separate PyTorch ops; kernels ask for fused multiply-adds
explicitly), IEEE division, and no packed-fp32 instructions.
"""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
SO_PATH = os.path.join(HERE, "liblandmark_hip.so")
MICROBENCH_PATH = os.path.join(HERE, "build", "mfma_valu_coissue")
SOURCES = ["lm_api.hip", "lm_sample.hip", "lm_gather.hip", "lm_mlp.hip", "lm_composite.hip", "lm_frame.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-fhip-fp32-correctly-rounded-divide-sqrt", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def build(verbose: bool = True, jobs: int = 8) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    procs = []
    objs = []
    for src in SOURCES:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        objs.append(obj)
        cmd = [hipcc, *FLAGS, *os.environ.get("LM_EXTRA_HIPCC_FLAGS", "").split(), "-c", os.path.join(CSRC, src), "-o", obj]
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            failed = True
            sys.stderr.write(f"[build] {src} FAILED\n{out}\n")
        elif verbose and out.strip():
            sys.stderr.write(f"[build] {src}\n{out}\n")
    if failed:
        raise RuntimeError("hipcc failed")
    link = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", SO_PATH, *objs]
    subprocess.check_call(link)
    # the micro-benchmark the colour network's schedule rests on (a program of its own, not part of the library)
    subprocess.check_call([hipcc, "--offload-arch=gfx950", "-O3", "-w", os.path.join(CSRC, "microbench", "mfma_valu_coissue.hip"),
                           "-o", MICROBENCH_PATH])
    if verbose:
        print(f"[build] wrote {SO_PATH}")
    return SO_PATH


if __name__ == "__main__":
    build()
