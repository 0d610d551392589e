"""Build libexact_hip.so (gfx950) in-tree with plain hipcc.

    python -m exact_amd.build            # compile every .hip, link the library

hipcc cross-compiles for gfx950 without a GPU, so this runs on a CPU-only
machine; the resulting exact_amd/libexact_hip.so is what the ctypes loader in
exact_amd/_lib.py opens.
"""
from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "build")
LIB = os.path.join(HERE, "libexact_hip.so")

SOURCES = ["abi.hip", "quant_pack.hip", "quant_unpack.hip", "act_mask.hip", "spmm.hip", "spmm_extra.hip", "rp_gemm.hip", "rp_bf16.hip", "colsum.hip", "linear_dw.hip", "stream_probe.hip"]

# -ffp-contract=off: the quantiser's arithmetic is defined as separately
#   rounded fp32 operations; kernels that want FMA call fmaf / MFMA explicitly.
# -packed-fp32-ops disabled: keep hipcc from forming v_pk_*_f32.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-fhip-fp32-correctly-rounded-divide-sqrt", "-fno-fast-math", "-munsafe-fp-atomics",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: libexact_hip.so cannot be built")
    return exe


def _compile(src: str) -> str:
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{res.stdout}\n{res.stderr}")
    noisy = [l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip()]
    if noisy:
        sys.stderr.write("\n".join(noisy) + "\n")
    return obj


def build(verbose: bool = True) -> str:
    os.makedirs(OBJ, exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(len(SOURCES), os.cpu_count() or 1)) as pool:
        objs = list(pool.map(_compile, SOURCES))
    tmp = LIB + ".tmp"
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    os.replace(tmp, LIB)
    if verbose:
        print(f"built {LIB} ({os.path.getsize(LIB) / 1e6:.1f} MB)")
    return LIB


if __name__ == "__main__":
    build()
