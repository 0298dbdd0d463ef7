"""fl_decode_attn_forward_noalloc — the entry point that uses the library's own per-GPU scratch array
instead of a caller workspace — against fl_decode_attn_forward on the same inputs, through the C ABI."""
import numpy as np
import pytest

from fasterllama_amd import capi
from helpers import Case, assert_cache_bit_exact, assert_out_close

pytestmark = pytest.mark.gpu


def both(c, gpu, nsplit=0):
    want, kc_w, vc_w, op = c.run_gpu(gpu, nsplit=nsplit, entry="forward")
    got, kc_g, vc_g, _ = c.run_gpu(gpu, nsplit=nsplit, entry="noalloc")
    assert_cache_bit_exact(kc_g, kc_w, "k_cache")
    assert_cache_bit_exact(vc_g, vc_w, "v_cache")
    # same kernels, same arithmetic, same order: bit-identical, which is inside any tolerance
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    ref64 = c.run_oracle(acc_double=True, threads=16)[0]
    ok = ~np.isnan(ref64).any(axis=1)
    assert_out_close(got[ok], ref64[ok], c.dtype, "noalloc vs oracle", head_dim=c.D)
    return op


def test_noalloc_two_calls_in_a_row_the_second_smaller(gpu):
    # split context (partials and arrival counters in the scratch array), then a smaller problem that
    # reuses the same array, then the first again
    big = Case(1, 32, 128, 4096, "f16", start_pos=4095, scale_rows=(17, 1000, 4000))
    op = both(big, gpu)
    assert op.plan(4096).nsplit > 1
    small = Case(1, 8, 128, 4096, "f16", start_pos=700, seed=5)
    both(small, gpu)
    both(big, gpu)


@pytest.mark.parametrize("dtype", ["f16", "f32"])
def test_noalloc_ragged_forced_splits_and_unsplit(gpu, dtype):
    lens = np.array([1, 512, 0, 333, 513, 64])
    both(Case(6, 3, 128, 512, dtype, lens=lens, pad=np.nan), gpu, nsplit=5)
    both(Case(2, 4, 64, 256, dtype, start_pos=100), gpu, nsplit=1)  # no scratch needed at all


def test_noalloc_counters_keep_their_place_across_shapes(gpu):
    """The arrival counters own a fixed part of the scratch array: a call with few (batch, head) pairs that writes
    floats into the array (an INT8-only step keeps its float output there; a split step its partials) must not leave
    non-zero words where a later split step with more pairs keeps its counters."""
    import torch
    from fasterllama_amd.decode_attn import DecodeAttention
    # 1. INT8-only, unsplit, B*H = 32: the float output [32, 128] goes through the scratch array
    c1 = Case(1, 32, 128, 512, "f16", start_pos=300, seed=3)
    t = lambda a: torch.from_numpy(a).to(gpu)
    op1 = DecodeAttention(1, 32, 128, 512, torch.float16, nsplit=1, device=gpu)
    res = {}
    for entry in ("forward", "noalloc"):
        q8 = torch.zeros(1, 32 * 128, dtype=torch.int8, device=gpu)
        sc = torch.zeros(1, dtype=torch.float32, device=gpu)
        io = op1.make_io(t(c1.q), t(c1.k_new), t(c1.v_new), t(c1.k_cache), t(c1.v_cache), t(c1.freq), None,
                         start_pos=300, out_int8=q8, out_scale=sc)
        if entry == "noalloc":
            io.workspace, io.workspace_bytes = None, 0
            capi.check(op1.launch_noalloc(io))
        else:
            capi.check(op1.launch(io))
        torch.cuda.synchronize()
        res[entry] = (q8.cpu().numpy(), sc.cpu().numpy())
    assert np.array_equal(res["forward"][0], res["noalloc"][0]) and np.array_equal(res["forward"][1], res["noalloc"][1])
    assert np.abs(res["noalloc"][0]).max() == 127
    # 2. a tiny split step: its partials sit at the start of the array
    both(Case(1, 2, 32, 512, "f32", start_pos=400, seed=4), gpu, nsplit=4)
    # 3. split steps with more pairs, merged inside the launch: B*H = 128 and 200 counters
    op = both(Case(4, 32, 128, 2048, "f16", start_pos=2047, seed=5), gpu)
    plan = op.plan(2048)
    assert plan.nsplit > 1 and plan.two_pass == 2
    both(Case(5, 40, 64, 1024, "f32", start_pos=1000, seed=6), gpu, nsplit=3)
    both(Case(4, 32, 128, 2048, "f16", start_pos=2047, seed=7), gpu)


def test_noalloc_rejects_what_does_not_fit(gpu):
    import ctypes as C
    import torch
    from fasterllama_amd.decode_attn import DecodeAttention
    # B*H = 4096 pairs x 64 forced splits x (128 + 2) floats = 136 MB of partials > 16 MiB
    B, H, D, L = 128, 32, 128, 4096
    op = DecodeAttention(B, H, D, L, torch.float16, nsplit=64, device=gpu)
    x = torch.zeros(16, dtype=torch.float16, device=gpu)  # never dereferenced: validation fails first
    io = op.make_io(x, x, x, x, x, x.float(), x.float(), start_pos=L - 1)
    io.workspace, io.workspace_bytes = None, 0
    st = op.launch_noalloc(io)
    assert st == capi.FL_ATTN_ERR_SCRATCH_LIMIT and "scratch" in capi.strerror(st)


def test_noalloc_call_can_be_captured_in_a_hip_graph(gpu):
    """Callers under graph capture are who the entry point is for: after one eager call on the device (which looks
    up the scratch array's address) the call only enqueues kernels.  Replays, interleaved with unrelated eager work,
    reproduce the eager result bit for bit, with a split context (partials and arrival counters in the scratch array)."""
    import torch
    from fasterllama_amd.decode_attn import DecodeAttention
    B, H, D, L, P = 2, 16, 128, 4096, 3000
    c = Case(B, H, D, L, "f16", start_pos=P)
    t = lambda a: torch.from_numpy(a).to(gpu)
    op = DecodeAttention(B, H, D, L, torch.float16, nsplit=8, device=gpu)
    q, k, v, kc, vc, f = (t(a) for a in (c.q, c.k_new, c.v_new, c.k_cache, c.v_cache, c.freq))
    out = torch.zeros(B, H * D, device=gpu)
    io = op.make_io(q, k, v, kc, vc, f, out, start_pos=P)
    io.workspace, io.workspace_bytes = None, 0
    assert op.launch_noalloc(io) == 0
    torch.cuda.synchronize()
    eager = out.clone()
    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream(device=gpu)
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            assert op.launch_noalloc(io, stream=torch.cuda.current_stream(gpu)) == 0
    torch.cuda.synchronize()
    for rep in range(3):
        out.fill_(float("nan"))
        _ = (torch.randn(1 << 20, device=gpu) * 2).sum().item()  # unrelated eager work + sync
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {rep}"
    want64 = c.run_oracle(acc_double=True, threads=16)[0]
    assert_out_close(out.cpu().numpy(), want64, "f16", "noalloc graph replay", head_dim=D)
