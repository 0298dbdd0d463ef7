"""Builds the native libraries in-tree (no GPU needed: hipcc cross-compiles for gfx950).

    python -m fasterllama_amd.build            # everything
    python -m fasterllama_amd.build hip synth  # selected targets

Targets
    hip     fasterllama_amd/lib/libfl_decode_attn.so   HIP kernels + C ABI (include/fl_decode_attn.h)
    cxx     fasterllama_amd/lib/libflopendecoder.so    C++ OpenDecoder mirror over the C ABI
    synth   fasterllama_amd/lib/libfl_synth.so         host-side seeded input generator
    oracle  oracle/libfl_ref.so                        CPU checker (test infrastructure)
    cpptest tests/cpp/open_decoder_check               C++ drop-in test driver
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "fasterllama_amd")
CSRC = os.path.join(PKG, "csrc")
LIB = os.path.join(PKG, "lib")

GFX_ARCH = "gfx950"
# Packed-FP32 VALU forms are kept out of the generated code on purpose (scalar fp32 ops only).
HIP_FLAGS = [
    f"--offload-arch={GFX_ARCH}", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option",
]


def _run(cmd: list[str], cwd: str | None = None) -> None:
    print("+", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, cwd=cwd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(
        ln for ln in res.stdout.splitlines()
        if "is not a recognized feature for this target" not in ln  # host pass vs device-only feature
    )
    if out.strip():
        print(out, flush=True)
    if res.returncode != 0:
        raise RuntimeError(f"command failed ({res.returncode}): {' '.join(cmd)}")


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found")
    return exe


def build_hip() -> str:
    os.makedirs(LIB, exist_ok=True)
    out = os.path.join(LIB, "libfl_decode_attn.so")
    _run([hipcc(), *HIP_FLAGS, "-shared", "-o", out, os.path.join(CSRC, "fl_decode_attn.hip")])
    return out


def build_cxx() -> str:
    os.makedirs(LIB, exist_ok=True)
    out = os.path.join(LIB, "libflopendecoder.so")
    _run([hipcc(), "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall",
          "-I", os.path.join(ROOT, "include"), "-o", out,
          os.path.join(CSRC, "open_decoder.cpp"),
          "-L", LIB, "-lfl_decode_attn", "-Wl,-rpath,$ORIGIN"])
    return out


def build_synth() -> str:
    os.makedirs(LIB, exist_ok=True)
    out = os.path.join(LIB, "libfl_synth.so")
    _run(["gcc", "-O2", "-std=c11", "-fPIC", "-shared", "-fopenmp", "-mf16c", "-Wall",
          "-o", out, os.path.join(CSRC, "fl_synth.c"), "-lm"])
    return out


def build_oracle() -> str:
    _run(["make", "-C", os.path.join(ROOT, "oracle"), "-B"])
    return os.path.join(ROOT, "oracle", "libfl_ref.so")


def build_cpptest() -> str:
    src = os.path.join(ROOT, "tests", "cpp", "open_decoder_check.cpp")
    out = os.path.join(ROOT, "tests", "cpp", "open_decoder_check")
    _run([hipcc(), "-O2", "-std=c++17", "-Wall",
          "-I", os.path.join(ROOT, "include"), "-I", CSRC, "-o", out, src,
          "-L", LIB, "-lflopendecoder", "-lfl_decode_attn",
          "-L", os.path.join(ROOT, "oracle"), "-lfl_ref",
          f"-Wl,-rpath,{LIB}", f"-Wl,-rpath,{os.path.join(ROOT, 'oracle')}",
          "-Wl,-rpath,$ORIGIN/../../fasterllama_amd/lib", "-Wl,-rpath,$ORIGIN/../../oracle"])
    return out


TARGETS = {
    "hip": build_hip,
    "cxx": build_cxx,
    "synth": build_synth,
    "oracle": build_oracle,
    "cpptest": build_cpptest,
}


def build_all(targets: list[str] | None = None) -> None:
    for name in targets or list(TARGETS):
        if name == "cxx" and not os.path.exists(os.path.join(CSRC, "open_decoder.cpp")):
            continue
        if name == "cpptest" and not os.path.exists(os.path.join(ROOT, "tests", "cpp", "open_decoder_check.cpp")):
            continue
        TARGETS[name]()


if __name__ == "__main__":
    build_all(sys.argv[1:] or None)
