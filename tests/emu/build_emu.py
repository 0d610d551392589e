"""Build the library's .hip sources, unchanged, as host C++ against the SIMT
emulator header in tests/emu/include (TESTS ONLY).

    python tests/emu/build_emu.py            # tests/emu/_build/libexact_emu.so
    python tests/emu/build_emu.py --asan     # tests/emu/_build/emu_check (AddressSanitizer executable)
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
CSRC = os.path.join(ROOT, "exact_amd", "csrc")
OUT = os.path.join(HERE, "_build")
CLANG = "/opt/rocm/lib/llvm/bin/clang++"
SOURCES = ["abi.hip", "quant_pack.hip", "quant_unpack.hip", "act_mask.hip", "spmm.hip", "spmm_extra.hip", "rp_gemm.hip", "rp_bf16.hip", "colsum.hip", "linear_dw.hip", "stream_probe.hip"]
COMMON = ["-x", "c++", "-std=c++17", "-ffp-contract=off", "-fno-fast-math", "-pthread", "-fPIC",
          "-I", os.path.join(HERE, "include"), "-Wno-unused-value", "-Wno-unknown-attributes"]
LIB = os.path.join(OUT, "libexact_emu.so")
CHECK = os.path.join(OUT, "emu_check")


def _run(cmd):
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("emulator build failed:\n" + " ".join(cmd) + "\n" + res.stdout + res.stderr)


def build_lib():
    os.makedirs(OUT, exist_ok=True)
    srcs = [os.path.join(CSRC, s) for s in SOURCES]
    _run([CLANG, *COMMON, "-O2", "-shared", "-o", LIB, *srcs])
    return LIB


def build_asan_check():
    os.makedirs(OUT, exist_ok=True)
    srcs = [os.path.join(CSRC, s) for s in SOURCES]
    oracle_o = os.path.join(OUT, "exact_oracle.o")
    _run(["gcc", "-O2", "-ffp-contract=off", "-c", os.path.join(ROOT, "oracle", "exact_oracle.c"), "-o", oracle_o])
    _run([CLANG, *COMMON, "-O1", "-g", "-fsanitize=address,alignment,bounds,shift", "-fno-sanitize-recover=alignment,bounds,shift",
          "-fno-omit-frame-pointer", "-o", CHECK,
          *srcs, "-x", "c++", os.path.join(HERE, "emu_check.cpp"), "-x", "none", oracle_o, "-lm"])
    return CHECK


if __name__ == "__main__":
    print(build_asan_check() if "--asan" in sys.argv else build_lib())
