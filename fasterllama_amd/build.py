"""Builds the native libraries in-tree (no GPU needed: hipcc cross-compiles for gfx950).

    python -m fasterllama_amd.build            # everything
    python -m fasterllama_amd.build hip synth  # selected targets

Targets
    hip     fasterllama_amd/lib/libfl_decode_attn.so   HIP kernels + C ABI (include/fl_decode_attn.h)
    cxx     fasterllama_amd/lib/libflopendecoder.so    C++ OpenDecoder mirror over the C ABI
    synth   fasterllama_amd/lib/libfl_synth.so         host-side seeded input generator
    calib   fasterllama_amd/lib/libfl_calib.so         measurement-only kernels of bench.py --calib
    oracle  oracle/libfl_ref.so                        CPU checker (test infrastructure)
    cpptest tests/cpp/open_decoder_check               C++ drop-in test driver
    cxxbench fasterllama_amd/lib/open_decoder_bench    times OpenDecoder::forward in the reference driver's layer loop
    sanitize (by name only) oracle + C-ABI host logic built with ASan/UBSan and run on the CPU
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


def sources(name: str) -> list[str]:
    """Files a target is built from (a change in any of them makes the built file stale)."""
    import glob
    hip = [os.path.join(CSRC, "fl_decode_attn.hip")] + sorted(glob.glob(os.path.join(CSRC, "*.hpp"))) + \
        [os.path.join(ROOT, "include", "fl_decode_attn.h")]
    return {
        "hip": hip,
        "cxx": [os.path.join(CSRC, "open_decoder.cpp"), os.path.join(CSRC, "open_decoder.h"),
                os.path.join(ROOT, "include", "fl_decode_attn.h")],
        "synth": [os.path.join(CSRC, "fl_synth.c")],
        "calib": [os.path.join(CSRC, "fl_calib.hip")],
        "oracle": [os.path.join(ROOT, "oracle", "fl_ref_decode_attn.c"), os.path.join(ROOT, "oracle", "Makefile")],
        "cpptest": [os.path.join(ROOT, "tests", "cpp", "open_decoder_check.cpp"), os.path.join(CSRC, "open_decoder.h"),
                    os.path.join(ROOT, "include", "fl_decode_attn.h")],
        "cxxbench": [os.path.join(CSRC, "open_decoder_bench.cpp"), os.path.join(CSRC, "open_decoder.h"),
                     os.path.join(ROOT, "include", "fl_decode_attn.h")],
    }[name]


def outputs(name: str) -> str:
    return {
        "hip": os.path.join(LIB, "libfl_decode_attn.so"),
        "cxx": os.path.join(LIB, "libflopendecoder.so"),
        "synth": os.path.join(LIB, "libfl_synth.so"),
        "calib": os.path.join(LIB, "libfl_calib.so"),
        "oracle": os.path.join(ROOT, "oracle", "libfl_ref.so"),
        "cpptest": os.path.join(ROOT, "tests", "cpp", "open_decoder_check"),
        "cxxbench": os.path.join(LIB, "open_decoder_bench"),
    }[name]


def source_hash(name: str) -> str:
    import hashlib
    h = hashlib.sha256()
    for path in sources(name):
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def _stamp(name: str) -> str:
    return outputs(name) + ".srchash"


def is_stale(name: str) -> bool:
    """True when the built file is absent or was built from other sources than the ones on disk (a
    content hash written next to it at build time: file times do not survive every copy of a tree)."""
    if not os.path.exists(outputs(name)) or not os.path.exists(_stamp(name)):
        return True
    with open(_stamp(name)) as f:
        return f.read().strip() != source_hash(name)


def _built(name: str) -> str:
    with open(_stamp(name), "w") as f:
        f.write(source_hash(name) + "\n")
    return outputs(name)


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
    return _built("hip")


def build_cxx() -> str:
    os.makedirs(LIB, exist_ok=True)
    out = os.path.join(LIB, "libflopendecoder.so")
    _run([hipcc(), "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall",
          "-I", os.path.join(ROOT, "include"), "-o", out,
          os.path.join(CSRC, "open_decoder.cpp"),
          "-L", LIB, "-lfl_decode_attn", "-Wl,-rpath,$ORIGIN"])
    return _built("cxx")


def build_synth() -> str:
    os.makedirs(LIB, exist_ok=True)
    out = os.path.join(LIB, "libfl_synth.so")
    _run(["gcc", "-O2", "-std=c11", "-fPIC", "-shared", "-fopenmp", "-mf16c", "-Wall",
          "-o", out, os.path.join(CSRC, "fl_synth.c"), "-lm"])
    return _built("synth")


def build_calib() -> str:
    """Measurement-only kernels for bench.py --calib (a library of its own, not linked into the product)."""
    os.makedirs(LIB, exist_ok=True)
    out = os.path.join(LIB, "libfl_calib.so")
    _run([hipcc(), *HIP_FLAGS, "-shared", "-o", out, os.path.join(CSRC, "fl_calib.hip")])
    return _built("calib")


def build_oracle() -> str:
    _run(["make", "-C", os.path.join(ROOT, "oracle"), "-B"])
    return _built("oracle")


def build_cpptest() -> str:
    src = os.path.join(ROOT, "tests", "cpp", "open_decoder_check.cpp")
    out = os.path.join(ROOT, "tests", "cpp", "open_decoder_check")
    _run([hipcc(), "-O2", "-std=c++17", "-Wall",
          "-I", os.path.join(ROOT, "include"), "-I", CSRC, "-o", out, src,
          "-L", LIB, "-lflopendecoder", "-lfl_decode_attn",
          "-L", os.path.join(ROOT, "oracle"), "-lfl_ref",
          f"-Wl,-rpath,{LIB}", f"-Wl,-rpath,{os.path.join(ROOT, 'oracle')}",
          "-Wl,-rpath,$ORIGIN/../../fasterllama_amd/lib", "-Wl,-rpath,$ORIGIN/../../oracle"])
    return _built("cpptest")


def build_cxxbench() -> str:
    out = outputs("cxxbench")
    _run([hipcc(), "-O2", "-std=c++17", "-Wall", "-I", os.path.join(ROOT, "include"), "-I", CSRC, "-o", out,
          os.path.join(CSRC, "open_decoder_bench.cpp"), "-L", LIB, "-lflopendecoder", "-lfl_decode_attn",
          f"-Wl,-rpath,{LIB}", "-Wl,-rpath,$ORIGIN"])
    return _built("cxxbench")


def run_sanitizers() -> None:
    """Host code under AddressSanitizer + UndefinedBehaviorSanitizer, built and RUN here (no GPU involved):
    the CPU oracle with its driver (`make -C oracle asan`), and the host pass of the C-ABI library with
    tests/cpp/capi_host_check.cpp (validation, planning and workspace arithmetic; every call is rejected
    before a launch).  Raises when a sanitizer reports or a check fails."""
    _run(["make", "-C", os.path.join(ROOT, "oracle"), "-B", "asan"])
    exe = os.path.join(ROOT, "tests", "cpp", "capi_host_check")
    _run([hipcc(), f"--offload-arch={GFX_ARCH}", "-O1", "-g", "-std=c++17",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unknown-warning-option",
          "-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined",
          "-Xarch_host", "-fno-sanitize-recover=all",
          "-I", os.path.join(ROOT, "include"), "-o", exe,
          os.path.join(CSRC, "fl_decode_attn.hip"), os.path.join(ROOT, "tests", "cpp", "capi_host_check.cpp")])
    _run([exe])


TARGETS = {
    "hip": build_hip,
    "cxx": build_cxx,
    "synth": build_synth,
    "calib": build_calib,
    "oracle": build_oracle,
    "cpptest": build_cpptest,
    "cxxbench": build_cxxbench,
    "sanitize": run_sanitizers,
}
DEFAULT_TARGETS = [t for t in TARGETS if t != "sanitize"]  # the sanitizer run is asked for by name (and by the CPU tests)


def build_all(targets: list[str] | None = None) -> None:
    for name in targets or DEFAULT_TARGETS:
        if name == "cxx" and not os.path.exists(os.path.join(CSRC, "open_decoder.cpp")):
            continue
        if name == "cpptest" and not os.path.exists(os.path.join(ROOT, "tests", "cpp", "open_decoder_check.cpp")):
            continue
        TARGETS[name]()


if __name__ == "__main__":
    build_all(sys.argv[1:] or None)
