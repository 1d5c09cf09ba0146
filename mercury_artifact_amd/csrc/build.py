"""Build libmercury_hip.so for gfx950 with hipcc (in-tree, next to the sources).

Usage:  python -m mercury_artifact_amd.csrc.build        (always recompiles)
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
SOURCES = ["api.hip", "attn_fwd.hip", "attn_fwd_fp8.hip", "attn_bwd.hip", "lse_merge.hip", "quantize.hip"]
LIB = os.path.join(HERE, "libmercury_hip.so")
# -packed-fp32-ops off: keep the compiler from forming v_pk_{add,mul,fma}_f32.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


# attn_bwd.hip keeps 128 accumulator registers per lane for dK^T / dV^T and works on T1 / T2 with the vector
# unit: with MFMA results in arithmetic registers (and only the stationary operands in accumulation
# registers) there are no copies between the two register files in its main loop.
EXTRA_FLAGS = {"attn_bwd.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


def _run(cmd):
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build(verbose: bool = False) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objs = [os.path.join(HERE, s.replace(".hip", ".o")) for s in SOURCES]
    cmds = [[hipcc, *FLAGS, *EXTRA_FLAGS.get(s, []), "-c", os.path.join(HERE, s), "-o", o]
            for s, o in zip(SOURCES, objs)]
    with ThreadPoolExecutor(max_workers=min(4, len(cmds))) as ex:
        for out in ex.map(_run, cmds):
            if verbose and out.strip():
                print(out)
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs])
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
    sys.exit(0)
