"""
Build recipe of libkvx.so: hipcc for gfx950 on the HIP sources under csrc/, linked into one shared
library next to this file. Cross-compiles without a GPU. Run as `python -m keys_values_amd.build`.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libkvx.so")
SOURCES = ["kvx_api.hip", "sdpa_prefill.hip", "score_sum.hip", "sdpa_decode.hip", "quantize.hip", "h2o.hip", "norm_rope.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-fast-math",          # the quantiser relies on IEEE division and rounding
    "-ffp-contract=off",       # no implicit fused multiply-add; kernels call fmaf where they want one
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
    "-Wno-inline-asm",         # the DMA helpers name m0 as clobbered, which clang reports once per instantiation
]


def _compile(src: str) -> str:
    os.makedirs(OBJ, exist_ok=True)
    obj = os.path.join(OBJ, src.replace(".hip", ".o"))
    cmd = [HIPCC] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{out}")
    if out.strip():
        print(out, file=sys.stderr)
    return obj


def build(verbose: bool = True) -> str:
    with ThreadPoolExecutor(max_workers=min(7, os.cpu_count() or 1)) as ex:
        objs = list(ex.map(_compile, SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}")
    if verbose:
        print(f"built {LIB}")
    return LIB


if __name__ == "__main__":
    build()
