"""Build recipe for libptm_hip.so: hipcc, gfx950 only, one shared library with a C ABI."""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libptm_hip.so")
SOURCES = ["glue.hip", "q4k_gemv.hip", "q6k_gemv.hip", "flash_decode.hip", "mixed_gemv.hip", "qgemm.hip", "decode.hip", "dispatch.hip", "other_gemv.hip", "gguf.hip", "prefill.hip", "sampler.hip", "tokenizer.hip", "plain_ops.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    # keep the compiler from forming packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option", "-Wno-unused-command-line-argument",
]
# Per-file additions.  prefill.hip: its matrix-core attention rescales the output accumulators between MFMAs with vector
# arithmetic, which cannot touch accumulation registers; with the accumulators there the compiler copies all 64 of them
# out and back on every tile.  One wave per SIMD leaves room for them in ordinary registers.
FILE_FLAGS = {"prefill.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


def build(verbose: bool = True, jobs: int = 8) -> str:
    objs, procs = [], []
    os.makedirs(os.path.join(CSRC, "build"), exist_ok=True)
    for src in SOURCES:
        obj = os.path.join(CSRC, "build", src.replace(".hip", ".o"))
        objs.append(obj)
        cmd = [HIPCC, *FLAGS, *FILE_FLAGS.get(src, []), "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        if len(procs) >= jobs:
            _drain(procs)
    _drain(procs)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB


def _drain(procs):
    for src, p in procs:
        out, _ = p.communicate()
        lines = [l for l in out.splitlines() if "packed-fp32-ops" not in l and l.strip()]
        if p.returncode != 0:
            print("\n".join(lines), file=sys.stderr)
            raise RuntimeError(f"hipcc failed on {src}")
        if lines:
            print("\n".join(lines))
    procs.clear()


if __name__ == "__main__":
    build()
