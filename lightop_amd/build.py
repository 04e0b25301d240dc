"""Builds the HIP extension (lightop_amd/csrc/*.hip -> liblightop_mi355.so) for gfx950.

Run as ``python -m lightop_amd.build``.  hipcc cross-compiles without a GPU, so the
library is built ahead of time and shipped next to the sources; nothing is compiled
at import.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
LIB_NAME = "liblightop_mi355.so"
LIB_PATH = os.path.join(CSRC, LIB_NAME)

# -ffp-contract=off: the kernels spell out every fused multiply-add they want, so that
# the fp32 epilogues round exactly like the scalar definition of the path.
# packed-fp32-ops is disabled on purpose (no v_pk_*_f32 code generation).
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-fno-fast-math", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def build_library(verbose: bool = False, extra_flags=(), out_path: str = LIB_PATH) -> str:
    """Compile every .hip under csrc/ and link them into one shared library."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objs = []

    def compile_one(src):
        obj = os.path.join(CSRC, src[:-4] + f".{os.getpid()}.{abs(hash(out_path)) % 99991}.o")
        cmd = [hipcc, *HIPCC_FLAGS, *extra_flags, "-c", os.path.join(CSRC, src), "-o", obj]
        res = subprocess.run(cmd, capture_output=True, text=True)
        noise = "is not a recognized feature for this target"
        err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{err}")
        if verbose and err.strip():
            print(err, file=sys.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as ex:
        objs = list(ex.map(compile_one, sources()))
    link = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out_path, *objs]
    res = subprocess.run(link, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    for o in objs:
        os.remove(o)
    return out_path


if __name__ == "__main__":
    print(build_library(verbose=True))
