"""Runs the C++ drop-in driver (tests/cpp/open_decoder_check.cpp): the OpenDecoder mirror called the
way a FasterLLaMA caller calls it, checked against the CPU oracle inside the driver."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "cpp", "open_decoder_check")


@pytest.mark.gpu
def test_open_decoder_cpp_driver(gpu):
    from fasterllama_amd import build
    if build.is_stale("cxx") or build.is_stale("cpptest"):
        build.build_cxx()
        build.build_cpptest()
    res = subprocess.run([EXE], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=100)
    print(res.stdout)
    assert res.returncode == 0, res.stdout
    assert "ALL CHECKS PASSED" in res.stdout
    assert res.stdout.count("PASS ") == 36 and "FAIL" not in res.stdout


def test_open_decoder_library_exports_the_reference_instantiations():
    """The shared library carries the same explicit instantiations as the reference's
    libflopendecoder (open_decoder.cu:377-383): OpenDecoder<FP32,INT8> and OpenDecoder<FP16,INT8>."""
    so = os.path.join(ROOT, "fasterllama_amd", "lib", "libflopendecoder.so")
    from fasterllama_amd import build
    if build.is_stale("cxx"):
        build.build_cxx()
    out = subprocess.run(["nm", "-DC", so], stdout=subprocess.PIPE, text=True, check=True).stdout
    for op in ("(FasterLLaMA::OperationType)0", "(FasterLLaMA::OperationType)1"):
        base = f"FasterLLaMA::OpenDecoder<{op}, (FasterLLaMA::OperationType)2>::"
        for member in ("OpenDecoder(int, int, int, int, int, int)", "initialize(", "getWorkspaceSize()", "forward(",
                       "~OpenDecoder()"):
            assert base + member in out, base + member
