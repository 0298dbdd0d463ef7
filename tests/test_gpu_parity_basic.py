"""First parity gate: HIP path vs the CPU oracle on identical seeded inputs (through the C ABI)."""
import numpy as np
import pytest

from helpers import Case, assert_cache_bit_exact, assert_out_close

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_config1_tiny(gpu, dtype):
    # B=1, 4 heads, D=64, 127 cached tokens + 1 new (reference-runnable plumbing case)
    c = Case(1, 4, 64, 128, dtype, start_pos=127)
    ref64, kc_ref, vc_ref = c.run_oracle(acc_double=True)
    out, kc, vc, _ = c.run_gpu(gpu)
    assert_cache_bit_exact(kc, kc_ref, "k_cache")
    assert_cache_bit_exact(vc, vc_ref, "v_cache")
    assert_out_close(out, ref64, dtype, "config1", head_dim=64)


@pytest.mark.parametrize("nsplit", [0, 1, 2, 7])
def test_config2_llama7b_b8_ctx1024(gpu, nsplit):
    c = Case(8, 32, 128, 1024, "f16", start_pos=1023)
    ref64, kc_ref, vc_ref = c.run_oracle(acc_double=True)
    out, kc, vc, _ = c.run_gpu(gpu, nsplit=nsplit)
    assert_cache_bit_exact(kc, kc_ref, "k_cache")
    assert_cache_bit_exact(vc, vc_ref, "v_cache")
    assert_out_close(out, ref64, "f16", f"config2 nsplit={nsplit}")
