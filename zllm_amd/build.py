"""Builds libzllm_hip.so for gfx950 with hipcc (in-tree, next to this file)."""
from __future__ import annotations

import hashlib
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libzllm_hip.so")

SOURCES = ["host.cpp", "matvec.hip", "matvec_quant.hip", "matvec_quant_q8.hip", "matvec_quant_q3.hip", "matvec_quant_q4.hip", "matvec_quant_q5.hip", "matvec_quant_q6.hip", "matvec_mfma_resident.hip", "matvec_q8_mfma_stream.hip", "matvec_bf16_mfma_stream.hip", "matvec_q6k_mfma_stream.hip", "matmul_f32.hip", "matmul_mfma.hip", "matmul_mfma_wide.hip", "matmul_q8_bf16.hip", "matmul_q8_bf16_wide.hip", "matmul_stream.hip", "matmul_int8.hip", "matmul_q8_i8.hip",
           "quantize_q8.hip", "elementwise.hip", "no_alloc.hip"]
HEADERS = ["common.h", "decode.h", "matvec_common.h", "matvec_quant.h", "matmul_q8_tiles.h", os.path.join("..", "..", "include", "zllm_hip.h")]

# -packed-fp32-ops off: some packed-FP32 forms have given wrong results on the
# target machines; ordinary float code must not be turned into them.
HIPCC_FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-ffp-contract=on",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option",
]

# Per-file additions. The int8 multiply reads every matrix-core result at once
# (to scale it): with the results in ordinary VGPRs there is no copy out of the
# accumulator file in between.
EXTRA_FLAGS = {"matmul_int8.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"], "matmul_q8_i8.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


def source_hash() -> str:
    h = hashlib.sha256()
    for name in SOURCES + HEADERS:
        with open(os.path.join(CSRC, name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def build(verbose: bool = False) -> str:
    """Compiles every source and links the shared library; returns its path."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    digest = source_hash()
    objs = []
    procs = []
    for name in SOURCES:
        src = os.path.join(CSRC, name)
        obj = os.path.join(CSRC, os.path.splitext(name)[0] + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, *EXTRA_FLAGS.get(name, []), f'-DZHIP_SOURCE_HASH="{digest}"', "-c", src, "-o", obj]
        if name.endswith(".cpp"):
            cmd[1:1] = ["-x", "hip"]
        procs.append((name, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    failed = False
    for name, p in procs:
        out, _ = p.communicate()
        # hipcc's host pass warns that it does not know the packed-fp32 feature: harmless.
        lines = [l for l in out.splitlines() if "packed-fp32-ops" not in l]
        if p.returncode != 0:
            failed = True
            print(f"--- {name} failed ---\n" + "\n".join(lines), file=sys.stderr)
        elif verbose and lines:
            print(f"--- {name} ---\n" + "\n".join(lines))
    if failed:
        raise RuntimeError("hipcc failed")
    subprocess.run([hipcc, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB, *objs], check=True)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
