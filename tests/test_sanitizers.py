"""Host code under AddressSanitizer + UndefinedBehaviorSanitizer (CPU only): the oracle with its driver
(oracle/sanitize_check.c) and the host pass of the C-ABI library (tests/cpp/capi_host_check.cpp)."""
import shutil

import pytest


@pytest.mark.skipif(shutil.which("gcc") is None, reason="needs the host compiler")
def test_oracle_and_capi_host_logic_are_clean_under_asan_and_ubsan(capfd):
    from fasterllama_amd import build
    build.run_sanitizers()  # raises on a sanitizer report or a failed check
    out = capfd.readouterr().out
    assert "oracle sanitizer run" in out and "no report" in out
    assert "C-ABI host logic under sanitizers" in out and " 0 failures" in out
