"""GPU tests of the stages either side of the attention core (int32 prologue, INT8 epilogue,
device RoPE table) and of launch behaviour (streams, HIP graphs, pass selection)."""
import numpy as np
import pytest

from fasterllama_amd import capi, synth
from helpers import Case, assert_cache_bit_exact, assert_out_close
from oracle import ref

pytestmark = pytest.mark.gpu


def _t(gpu):
    import torch
    return lambda a: None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(gpu)


# ----------------------------------------------------------------------------- RoPE table producer

@pytest.mark.parametrize("rows,D", [(4096, 128), (128, 64), (37, 32), (2048, 256)])
def test_device_rope_table_matches_host_table(gpu, rows, D):
    from fasterllama_amd.decode_attn import rope_table
    got = rope_table(rows, D, device=gpu).cpu().numpy()
    want = ref.freq_cis(rows, D)
    # both evaluate in double and round once; a last-place difference in the double can flip the float
    ulp = np.spacing(np.abs(want).astype(np.float32)).astype(np.float64)
    assert (np.abs(got.astype(np.float64) - want) <= ulp).all()
    assert (got == want).mean() > 0.999
    assert np.array_equal(got[0, 0::2], np.ones(D // 2, np.float32)) and (got[0, 1::2] == 0).all()


# ----------------------------------------------------------------------------- int32 prologue

@pytest.mark.parametrize("dtype", ["f32", "f16"])
@pytest.mark.parametrize("nsplit", [0, 3])
def test_int32_prologue(gpu, dtype, nsplit):
    import torch
    from fasterllama_amd.decode_attn import DecodeAttention
    B, H, D, L, P = 4, 8, 128, 256, 201
    rng = np.random.default_rng(12)
    qi, ki, vi = (rng.integers(-20000, 20000, (B, 1, H, D), dtype=np.int32) for _ in range(3))
    s_in = ((rng.random(B) + 0.5) * 2e-3).astype(np.float32)
    wq, wk, wv = ((rng.random(H * D) * 3e-2 + 1e-3).astype(np.float32) for _ in range(3))
    c = Case(B, H, D, L, dtype, start_pos=P)
    kc, vc = c.k_cache.copy(), c.v_cache.copy()
    want = ref.decode_attn(qi, ki, vi, kc, vc, c.freq, start_pos=P, inp_scale=s_in, wq_scale=wq, wk_scale=wk,
                           wv_scale=wv, acc_double=True, threads=8)
    t = _t(gpu)
    op = DecodeAttention(B, H, D, L, torch.float16 if dtype == "f16" else torch.float32, nsplit=nsplit, device=gpu)
    kc_d, vc_d = t(c.k_cache), t(c.v_cache)
    out = op.forward(t(qi), t(ki), t(vi), kc_d, vc_d, t(c.freq), start_pos=P, qkv_inp_scale=t(s_in),
                     q_weight_scale=t(wq), k_weight_scale=t(wk), v_weight_scale=t(wv))
    torch.cuda.synchronize()
    assert_cache_bit_exact(kc_d.cpu().numpy(), kc, "k_cache")
    assert_cache_bit_exact(vc_d.cpu().numpy(), vc, "v_cache")
    assert_out_close(out.cpu().numpy(), want, dtype, "int32 prologue", head_dim=D)


# ----------------------------------------------------------------------------- INT8 epilogue

@pytest.mark.parametrize("B,H,D,nsplit", [(4, 32, 128, 0), (3, 40, 128, 4), (2, 4, 64, 1), (2, 2, 1024, 2)])
def test_int8_epilogue(gpu, B, H, D, nsplit):
    import torch
    from fasterllama_amd.decode_attn import DecodeAttention
    L, P = 300, 257
    c = Case(B, H, D, L, "f16", start_pos=P, seed=B + H)
    t = _t(gpu)
    op = DecodeAttention(B, H, D, L, torch.float16, nsplit=nsplit, device=gpu)
    out = torch.empty(B, H * D, dtype=torch.float32, device=gpu)
    q8 = torch.empty(B, H * D, dtype=torch.int8, device=gpu)
    sc = torch.empty(B, dtype=torch.float32, device=gpu)
    op.forward(t(c.q), t(c.k_new), t(c.v_new), t(c.k_cache), t(c.v_cache), t(c.freq), start_pos=P, out=out,
               out_int8=q8, out_scale=sc)
    torch.cuda.synchronize()
    out_h, q_h, s_h = out.cpu().numpy(), q8.cpu().numpy(), sc.cpu().numpy()
    want64, _, _ = c.run_oracle(acc_double=True)
    assert_out_close(out_h, want64, "f16", "float output beside the int8 one")
    # the epilogue applied to the kernel's own float output must be bit-exact with the CPU quantiser
    q_ref, s_ref = ref.attn_quantize(out_h)
    assert np.array_equal(s_h, s_ref)
    assert np.array_equal(q_h, q_ref)
    # and against the oracle's float path it can differ by one quantisation step at most
    q_or, s_or = ref.attn_quantize(want64.astype(np.float32))
    assert np.abs(q_h.astype(np.int32) - q_or.astype(np.int32)).max() <= 1
    assert np.allclose(s_h, s_or, rtol=1e-5)
    # int8-only call (no float output buffer)
    q8b = torch.empty_like(q8); scb = torch.empty_like(sc)
    op.forward(t(c.q), t(c.k_new), t(c.v_new), t(c.k_cache), t(c.v_cache), t(c.freq), start_pos=P, out=None,
               out_int8=q8b, out_scale=scb)
    torch.cuda.synchronize()
    assert torch.equal(q8b, q8) and torch.equal(scb, sc)


def test_prologue_and_epilogue_together_ragged(gpu):
    import torch
    from fasterllama_amd.decode_attn import DecodeAttention
    B, H, D, L = 5, 8, 128, 128
    lens = np.array([1, 128, 64, 65, 100])
    rng = np.random.default_rng(2)
    qi, ki, vi = (rng.integers(-9000, 9000, (B, 1, H, D), dtype=np.int32) for _ in range(3))
    s_in = ((rng.random(B) + 0.5) * 4e-3).astype(np.float32)
    wq, wk, wv = ((rng.random(H * D) * 3e-2 + 1e-3).astype(np.float32) for _ in range(3))
    c = Case(B, H, D, L, "f16", lens=lens, pad=np.nan)
    kc, vc = c.k_cache.copy(), c.v_cache.copy()
    want = ref.decode_attn(qi, ki, vi, kc, vc, c.freq, start_pos_per_seq=lens - 1, inp_scale=s_in, wq_scale=wq,
                           wk_scale=wk, wv_scale=wv, acc_double=True)
    t = _t(gpu)
    op = DecodeAttention(B, H, D, L, torch.float16, device=gpu)
    out = torch.empty(B, H * D, dtype=torch.float32, device=gpu)
    q8 = torch.empty(B, H * D, dtype=torch.int8, device=gpu)
    sc = torch.empty(B, dtype=torch.float32, device=gpu)
    kc_d, vc_d = t(c.k_cache), t(c.v_cache)
    op.forward(t(qi), t(ki), t(vi), kc_d, vc_d, t(c.freq), out=out, start_pos_per_seq=t((lens - 1).astype(np.int32)),
               max_start_pos=127, qkv_inp_scale=t(s_in), q_weight_scale=t(wq), k_weight_scale=t(wk),
               v_weight_scale=t(wv), out_int8=q8, out_scale=sc)
    torch.cuda.synchronize()
    assert_cache_bit_exact(kc_d.cpu().numpy(), kc, "k_cache")
    assert_out_close(out.cpu().numpy(), want, "f16", "prologue+epilogue")
    q_ref, s_ref = ref.attn_quantize(out.cpu().numpy())
    assert np.array_equal(q8.cpu().numpy(), q_ref) and np.array_equal(sc.cpu().numpy(), s_ref)


# ----------------------------------------------------------------------------- launch behaviour

def test_runs_on_a_side_stream_and_passes_compose(gpu):
    import torch
    from fasterllama_amd.decode_attn import DecodeAttention
    c = Case(2, 8, 128, 1024, "f16", start_pos=900)
    want64, kc_ref, _ = c.run_oracle(acc_double=True)
    t = _t(gpu)
    op = DecodeAttention(2, 8, 128, 1024, torch.float16, nsplit=6, device=gpu)
    kc_d, vc_d = t(c.k_cache), t(c.v_cache)
    out = torch.full((2, 8 * 128), float("nan"), device=gpu)
    io = op.make_io(t(c.q), t(c.k_new), t(c.v_new), kc_d, vc_d, t(c.freq), out, start_pos=900)
    s = torch.cuda.Stream(device=gpu)  # default priority
    torch.cuda.synchronize()
    assert op.launch(io, passes=1, stream=s) == 0   # streaming pass only: partials + cache append
    s.synchronize()
    assert torch.isnan(out).all()
    assert_cache_bit_exact(kc_d.cpu().numpy(), kc_ref, "k_cache after pass 1")
    assert op.launch(io, passes=2, stream=s) == 0   # combine pass
    s.synchronize()
    assert_out_close(out.cpu().numpy(), want64, "f16", "pass 1 then pass 2")


def test_hip_graph_replay_matches_eager(gpu):
    """The call only enqueues kernels (no allocation, no memset, no sync), so it can be captured.
    Replays are interleaved with eager work and each replay is compared with the eager result."""
    import torch
    from fasterllama_amd.decode_attn import DecodeAttention
    B, H, D, L, P = 4, 8, 128, 2048, 1500
    c = Case(B, H, D, L, "f16", start_pos=P)
    want64, _, _ = c.run_oracle(acc_double=True)
    t = _t(gpu)
    for nsplit in (1, 8):
        op = DecodeAttention(B, H, D, L, torch.float16, nsplit=nsplit, device=gpu)
        q, k, v, kc, vc, f = (t(a) for a in (c.q, c.k_new, c.v_new, c.k_cache, c.v_cache, c.freq))
        out = torch.zeros(B, H * D, device=gpu)
        io = op.make_io(q, k, v, kc, vc, f, out, start_pos=P)
        eager = op.forward(q, k, v, kc, vc, f, start_pos=P).clone()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream(device=gpu)
        with torch.cuda.stream(side):
            with torch.cuda.graph(g, stream=side):
                assert op.launch(io, stream=torch.cuda.current_stream(gpu)) == 0
        torch.cuda.synchronize()
        for rep in range(4):
            out.fill_(float("nan"))
            _ = (torch.randn(1 << 20, device=gpu) * 2).sum().item()  # unrelated eager work + sync
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager), f"replay {rep} nsplit={nsplit}"
        assert_out_close(out.cpu().numpy(), want64, "f16", "graph replay")
