"""Prompt-phase (seq_len > 1) attention through the C ABI against the CPU oracle."""
import numpy as np
import pytest

from fasterllama_amd import capi, synth
from helpers import assert_cache_bit_exact, assert_out_close
from oracle import ref

pytestmark = pytest.mark.gpu
NP_DT = {"f32": np.float32, "f16": np.float16}


def causal_mask(L, fill=-1e5):
    return np.where(np.arange(L)[None, :] > np.arange(L)[:, None], fill, 0.0).astype(np.float32)


def make(B, H, D, L, S, dtype, seed=11):
    dt = NP_DT[dtype]
    q = synth.normal((B, S, H, D), dt, synth.TENSOR_Q, seed)
    k = synth.normal((B, S, H, D), dt, synth.TENSOR_K_NEW, seed)
    v = synth.normal((B, S, H, D), dt, synth.TENSOR_V_NEW, seed)
    kc = synth.normal((B, H, L, D), dt, synth.TENSOR_K_CACHE, seed)
    vc = synth.normal((B, H, L, D), dt, synth.TENSOR_V_CACHE, seed)
    return q, k, v, kc, vc, synth.freq_cis_table(L, D)


def close(out, want, dtype, what, run, rows=slice(None)):
    """assert_out_close with the float oracle of the same run_both call (its third result) at hand for FP32 caches."""
    fr = run.float_ref if dtype == "f32" else None
    return assert_out_close(out, want, dtype, what, float_ref=None if fr is None else (lambda: fr()[:, :, rows]))


def run_both(gpu, B, H, D, L, S, P, dtype, mask=None, rope_row=-1, pad_nan=True, seed=11):
    import torch
    from fasterllama_amd.decode_attn import PrefillAttention
    q, k, v, kc, vc, f = make(B, H, D, L, S, dtype, seed)
    if pad_nan:  # rows at and after the first new token are stale: they must never be read before being written
        kc[:, :, P:, :] = np.nan
        vc[:, :, P:, :] = np.nan
    kc_ref, vc_ref = kc.copy(), vc.copy()
    want = ref.prefill_attn(q, k, v, kc_ref, vc_ref, f, start_pos=P, rope_row=rope_row, attn_mask=mask,
                            acc_double=True, threads=16)
    # the same inputs through the oracle's float arithmetic (sequential FP32 sums), evaluated on demand
    float_ref = lambda: ref.prefill_attn(q, k, v, kc.copy(), vc.copy(), f, start_pos=P, rope_row=rope_row,
                                                  attn_mask=mask, acc_double=False, threads=16)
    t = lambda a: None if a is None else torch.from_numpy(a).to(gpu)
    op = PrefillAttention(B, H, D, L, S, torch.float16 if dtype == "f16" else torch.float32, device=gpu)
    kc_d, vc_d = t(kc), t(vc)
    out = op.prefill(t(q), t(k), t(v), kc_d, vc_d, t(f), start_pos=P, rope_row=rope_row, attn_mask=t(mask))
    torch.cuda.synchronize()
    kc_g, vc_g = kc_d.cpu().numpy(), vc_d.cpu().numpy()
    # rows past the prompt were NaN before and must still be: compare bit patterns of everything
    assert_cache_bit_exact(kc_g, kc_ref, "k_cache")
    assert_cache_bit_exact(vc_g, vc_ref, "v_cache")
    op.float_ref = float_ref
    return out.cpu().numpy(), want, op


@pytest.mark.parametrize("dtype", ["f32", "f16"])
@pytest.mark.parametrize("S,P", [(1, 0), (2, 0), (31, 0), (32, 0), (33, 0), (100, 0), (128, 0), (129, 0), (300, 0),
                                 (50, 37), (1, 200), (64, 64)])
def test_prefill_matches_oracle(gpu, dtype, S, P):
    L = 512
    out, want, run = run_both(gpu, 2, 3, 128, L, S, P, dtype, mask=causal_mask(L), seed=S + P)
    close(out, want, dtype, f"S={S} P={P}", run=run)


@pytest.mark.parametrize("dtype", ["f32", "f16"])
@pytest.mark.parametrize("D", [32, 64, 96, 128, 256, 512, 1024])
def test_prefill_head_sizes_and_no_mask(gpu, dtype, D):
    # the reference's set of head sizes (decoder_kernels.cu:474-551, :588), plus 32
    out, want, run = run_both(gpu, 2, 5, D, 256, 77, 10, dtype, mask=None, seed=D)
    close(out, want, dtype, f"D={D} no mask", run=run)


@pytest.mark.parametrize("dtype", ["f32", "f16"])
@pytest.mark.parametrize("D", [256, 512, 1024])
@pytest.mark.parametrize("S,P", [(1, 0), (33, 0), (130, 61), (64, 192)])
def test_prefill_wide_heads_with_masks(gpu, dtype, D, S, P):
    """Head sizes above 128 (the head dimension is split across the waves of a workgroup): ragged query
    blocks, chunked prompts, the -1e5 causal mask (every tile evaluated) and the -FLT_MAX one (tiles dropped)."""
    L = 256
    for fill in (-1e5, -FMAX):
        out, want, run = run_both(gpu, 2, 3, D, L, S, P, dtype, mask=causal_mask(L, fill), seed=D + S + P)
        close(out, want, dtype, f"D={D} S={S} P={P} fill={fill}", run=run)


def test_prefill_wide_heads_dense_mask_scaled_keys_and_decode_handover(gpu):
    """D = 256: a dense random mask with an odd row stride, key rows scaled by 8, then decode steps on the
    caches the prompt phase wrote (bit-identical rows)."""
    import torch
    from fasterllama_amd.decode_attn import DecodeAttention, PrefillAttention
    B, H, D, L, S, ld = 2, 3, 256, 160, 100, 171
    for dtype in ("f16", "f32"):
        tdt = torch.float16 if dtype == "f16" else torch.float32
        q, k, v, kc, vc, f = make(B, H, D, L, S, dtype, 91)
        k[:, 17] *= 8
        k[:, 70] *= 8
        mask = (np.random.default_rng(2).standard_normal((L, ld)) * 3).astype(np.float32)
        kc_ref, vc_ref = kc.copy(), vc.copy()
        want = ref.prefill_attn(q, k, v, kc_ref, vc_ref, f, attn_mask=mask, mask_ld=ld, acc_double=True, threads=16)
        t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(gpu)
        op = PrefillAttention(B, H, D, L, S, tdt, device=gpu)
        kc_d, vc_d = t(kc), t(vc)
        out = op.prefill(t(q), t(k), t(v), kc_d, vc_d, t(f), attn_mask=t(mask), mask_ld=ld)
        torch.cuda.synchronize()
        assert_cache_bit_exact(kc_d.cpu().numpy(), kc_ref, "k_cache")
        assert_out_close(out.cpu().numpy(), want, dtype, f"wide dense mask {dtype}",
                         float_ref=lambda: ref.prefill_attn(q, k, v, kc.copy(), vc.copy(), f, attn_mask=mask, mask_ld=ld, threads=16))
        dec = DecodeAttention(B, H, D, L, tdt, device=gpu)
        for step in range(3):
            qs, ks, vs, _, _, _ = make(B, H, D, L, 1, dtype, 200 + step)
            w = ref.decode_attn(qs, ks, vs, kc_ref, vc_ref, f, start_pos=S + step, acc_double=True)
            g = dec.forward(t(qs), t(ks), t(vs), kc_d, vc_d, t(f), start_pos=S + step)
            assert_out_close(g.cpu().numpy(), w, dtype, f"decode step {step} after a wide prompt", head_dim=D)
        assert_cache_bit_exact(kc_d.cpu().numpy(), kc_ref, "k_cache after decode steps")


def test_prefill_strict_mask_first_row_is_nan(gpu):
    # the samples' strict mask hides every key of query 0 at position 0: 0/0 = NaN, as the reference arithmetic
    L = 64
    fm = np.finfo(np.float32).max
    m = np.where(np.arange(L)[:, None] > np.arange(L)[None, :], 0.0, -fm).astype(np.float32)
    out, want, run = run_both(gpu, 1, 2, 64, L, 40, 0, "f32", mask=m)
    assert np.isnan(want[:, :, 0]).all() and np.isnan(out[:, :, 0]).all()
    close(out[:, :, 1:], want[:, :, 1:], "f32", "strict mask rows 1..", rows=slice(1, None), run=run)


FMAX = float(np.finfo(np.float32).max)


@pytest.mark.parametrize("dtype", ["f32", "f16"])
@pytest.mark.parametrize("S,P", [(300, 0), (257, 77), (128, 384), (40, 0)])
def test_prefill_causal_mask_with_flt_max(gpu, dtype, S, P):
    """The reference driver's mask value (samples/llama_fp16.cu:73-81): fully masked tiles contribute exact zeros
    whether a kernel evaluates or drops them."""
    L = 512
    out, want, run = run_both(gpu, 2, 3, 128, L, S, P, dtype, mask=causal_mask(L, -FMAX), seed=3 * S + P)
    close(out, want, dtype, f"-FLT_MAX causal S={S} P={P}", run=run)


@pytest.mark.parametrize("dtype", ["f32", "f16"])
@pytest.mark.parametrize("D", [32, 64])
def test_prefill_small_heads_with_causal_mask(gpu, dtype, D):
    L = 320
    out, want, run = run_both(gpu, 2, 4, D, L, 200, 100, dtype, mask=causal_mask(L, -FMAX), seed=D + 1)
    close(out, want, dtype, f"D={D} -FLT_MAX causal", run=run)


@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_prefill_sharp_softmax_with_scaled_keys(gpu, dtype):
    """Some key rows scaled by 8 (the stress of the B=1, ctx=4096 benchmark configuration): near one-hot weights, running maxima
    that jump late in the walk over the keys, and scores far above the lazily updated reference maximum."""
    import torch
    from fasterllama_amd.decode_attn import PrefillAttention
    B, H, D, L, S = 1, 4, 128, 512, 400
    q, k, v, kc, vc, f = make(B, H, D, L, S, dtype, 33)
    for r in (5, 130, 131, 399):
        k[:, r] *= 8
    q[:, 200:] *= 3
    mask = causal_mask(L, -FMAX)
    kc_ref, vc_ref = kc.copy(), vc.copy()
    want = ref.prefill_attn(q, k, v, kc_ref, vc_ref, f, attn_mask=mask, acc_double=True, threads=8)
    t = lambda a: torch.from_numpy(a).to(gpu)
    op = PrefillAttention(B, H, D, L, S, torch.float16 if dtype == "f16" else torch.float32, device=gpu)
    out = op.prefill(t(q), t(k), t(v), t(kc), t(vc), t(f), attn_mask=t(mask)).cpu().numpy()
    assert np.isfinite(out).all()
    assert_out_close(out, want, dtype, "scaled keys",
                     float_ref=lambda: ref.prefill_attn(q, k, v, kc.copy(), vc.copy(), f, attn_mask=mask, threads=8))
    if dtype == "f16":
        # the opt-in fast first product rounds the rotated queries to fp16: scores of magnitude ~90 then
        # carry ~2e-2 of error each; the flag promises no more than a loose bound on such data
        fast = PrefillAttention(B, H, D, L, S, torch.float16, device=gpu, fast_qk=True)
        out_fast = fast.prefill(t(q), t(k), t(v), t(kc), t(vc), t(f), attn_mask=t(mask)).cpu().numpy()
        err = np.abs(out_fast - want).max()
        assert err < 5e-2, err


def test_prefill_fast_qk_meets_the_bar_on_ordinary_data(gpu):
    import torch
    from fasterllama_amd.decode_attn import PrefillAttention
    B, H, D, L, S, P = 2, 3, 128, 512, 300, 60
    q, k, v, kc, vc, f = make(B, H, D, L, S, "f16", 5)
    mask = causal_mask(L, -FMAX)
    want = ref.prefill_attn(q, k, v, kc.copy(), vc.copy(), f, start_pos=P, attn_mask=mask, acc_double=True, threads=8)
    t = lambda a: torch.from_numpy(a).to(gpu)
    for msk in (mask, None):
        if msk is None:
            want = ref.prefill_attn(q, k, v, kc.copy(), vc.copy(), f, start_pos=P, acc_double=True, threads=8)
        op = PrefillAttention(B, H, D, L, S, torch.float16, device=gpu, fast_qk=True)
        out = op.prefill(t(q), t(k), t(v), t(kc), t(vc), t(f), start_pos=P, attn_mask=None if msk is None else t(msk))
        assert_out_close(out.cpu().numpy(), want, "f16", "fast first product")


def test_prefill_strict_mask_first_row_is_nan_f16(gpu):
    L = 192
    m = np.where(np.arange(L)[:, None] > np.arange(L)[None, :], 0.0, -FMAX).astype(np.float32)
    out, want, run = run_both(gpu, 1, 2, 128, L, 150, 0, "f16", mask=m)
    assert np.isnan(want[:, :, 0]).all() and np.isnan(out[:, :, 0]).all()
    assert not np.isnan(out[:, :, 1:]).any()
    assert_out_close(out[:, :, 1:], want[:, :, 1:], "f16", "strict mask rows 1.. (f16)")


@pytest.mark.parametrize("fill", [-FMAX, -np.inf, -1e5])
def test_prefill_sliding_window_mask_f16(gpu, fill):
    """A band mask leaves fully masked tiles on both sides of the band: the kernel's tile list has gaps."""
    L, S, P, win = 640, 200, 400, 96
    i, j = np.arange(L)[:, None], np.arange(L)[None, :]
    m = np.where((j > i) | (j < i - win), fill, 0.0).astype(np.float32)
    out, want, run = run_both(gpu, 2, 2, 128, L, S, P, "f16", mask=m, seed=5)
    assert_out_close(out, want, "f16", f"sliding window fill={fill}")


def test_prefill_dense_random_mask_f16(gpu):
    """Every tile mixed: the general path, with a row stride that is not a multiple of four."""
    import torch
    from fasterllama_amd.decode_attn import PrefillAttention
    B, H, D, L, S, P = 1, 3, 64, 200, 150, 30
    ld = L + 3
    rng = np.random.default_rng(7)
    full = (rng.standard_normal((L, ld)) * 2).astype(np.float32)
    full[rng.random((L, ld)) < 0.2] = -FMAX
    full[:, 0] = 0.0  # no fully masked row
    q, k, v, kc, vc, f = make(B, H, D, L, S, "f16", 9)
    kc_ref, vc_ref = kc.copy(), vc.copy()
    want = ref.prefill_attn(q, k, v, kc_ref, vc_ref, f, start_pos=P, attn_mask=np.ascontiguousarray(full[:, :L]),
                            acc_double=True, threads=8)
    t = lambda a: torch.from_numpy(a).to(gpu)
    op = PrefillAttention(B, H, D, L, S, torch.float16, device=gpu)
    out = op.prefill(t(q), t(k), t(v), t(kc), t(vc), t(f), start_pos=P, attn_mask=t(full), mask_ld=ld)
    assert_out_close(out.cpu().numpy(), want, "f16", "dense random mask")


@pytest.mark.parametrize("D", [32, 128])
def test_prefill_context_longer_than_one_tile_list_f16(gpu, D):
    """More key tiles than one pass of the kernel's tile list holds (1024 tiles = 32768 keys).  The
    mask is a single row shared by all queries (row stride 0): a key-padding mask that hides two long runs of keys."""
    import torch
    from fasterllama_amd.decode_attn import PrefillAttention
    B, H, L, S = 1, 1, 33100, 96
    P = L - S
    row = np.zeros(L, np.float32)
    row[64:20000] = -FMAX
    row[20040:32800] = -FMAX
    q, k, v, kc, vc, f = make(B, H, D, L, S, "f16", 21)
    t = lambda a: torch.from_numpy(a).to(gpu)
    op = PrefillAttention(B, H, D, L, S, torch.float16, device=gpu)
    for mask in (row, None):
        want = ref.prefill_attn(q, k, v, kc.copy(), vc.copy(), f, start_pos=P, attn_mask=mask, mask_ld=0,
                                acc_double=True, threads=8)
        out = op.prefill(t(q), t(k), t(v), t(kc), t(vc), t(f), start_pos=P,
                         attn_mask=None if mask is None else t(mask), mask_ld=0)
        assert_out_close(out.cpu().numpy(), want, "f16", f"context of {L} keys, mask={'row' if mask is not None else None}")


def test_prefill_hip_graph_replay_matches_eager(gpu):
    """The prompt-phase call only enqueues kernels (append, mask classes, attention): it can be captured, and
    replays — interleaved with unrelated eager work — reproduce the eager result bit for bit."""
    import torch
    from fasterllama_amd.decode_attn import PrefillAttention
    B, H, D, L, S, P = 2, 4, 128, 384, 200, 100
    for dtype in ("f16", "f32"):
        q, k, v, kc, vc, f = make(B, H, D, L, S, dtype, 17)
        t = lambda a: torch.from_numpy(a).to(gpu)
        op = PrefillAttention(B, H, D, L, S, torch.float16 if dtype == "f16" else torch.float32, device=gpu)
        qd, kd, vd, fd, md = t(q), t(k), t(v), t(f), t(causal_mask(L, -FMAX))
        kc_d, vc_d = t(kc), t(vc)
        eager = op.prefill(qd, kd, vd, kc_d, vc_d, fd, start_pos=P, attn_mask=md).clone()
        out = torch.zeros_like(eager)
        io = op.make_io(qd, kd, vd, kc_d, vc_d, fd, out, start_pos=P, attn_mask=md)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream(device=gpu)
        with torch.cuda.stream(side):
            with torch.cuda.graph(g, stream=side):
                assert op.launch_prefill(io, S, stream=torch.cuda.current_stream(gpu)) == 0
        torch.cuda.synchronize()
        for rep in range(3):
            out.fill_(float("nan"))
            _ = (torch.randn(1 << 20, device=gpu) * 2).sum().item()
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager), f"{dtype} replay {rep}"


def test_prefill_literal_rope_rows(gpu):
    # reference as written: token s of the prompt is rotated by table row s (decoder_kernels.cu:440)
    out, want, run = run_both(gpu, 2, 4, 128, 128, 60, 20, "f32", mask=causal_mask(128), rope_row=0)
    close(out, want, "f32", "rope_row=0", run=run)


def test_prefill_llama7b_shape(gpu):
    # B=4, 32 heads, D=128, prompt of 512 tokens, fp16 caches
    L = 640
    out, want, run = run_both(gpu, 4, 32, 128, L, 512, 0, "f16", mask=causal_mask(L))
    assert_out_close(out, want, "f16", "7B prompt 512")


@pytest.mark.parametrize("B,S,pairs,dtype,fast", [(8, 1024, ((0, 0), (3, 17), (7, 31), (4, 5)), "f16", False),
                                                  (8, 1024, ((0, 0), (3, 17), (7, 31), (4, 5)), "f16", True),
                                                  (1, 4096, ((0, 0), (0, 21)), "f16", False),
                                                  (8, 1024, ((1, 2), (6, 30)), "f32", False)])
def test_prefill_benchmark_shape_full_size(gpu, B, S, pairs, dtype, fast):
    """The prompt-phase benchmark shapes at full size (B=8, S=1024 with fp16 and with FP32 caches, B=1, S=4096; H=32,
    D=128, the reference driver's causal mask, tile classes from the persistent table).  Heads are independent, so the
    oracle runs on a sample of (b,h) pairs cut out of the same inputs; their output rows and cache rows are checked,
    the caches bit for bit."""
    import torch
    from fasterllama_amd.decode_attn import PrefillAttention
    H, D, L = 32, 128, S
    dev = gpu
    tdt = torch.float16 if dtype == "f16" else torch.float32
    g = torch.Generator(device="cpu").manual_seed(77)
    q = torch.randn(B, S, H, D, generator=g).to(tdt)
    k = torch.randn(B, S, H, D, generator=g).to(tdt)
    v = torch.randn(B, S, H, D, generator=g).to(tdt)
    f = synth.freq_cis_table(L, D)
    mask = causal_mask(L, -FMAX)
    op = PrefillAttention(B, H, D, L, S, tdt, device=dev, fast_qk=fast)
    md = torch.from_numpy(mask).to(dev)
    table = op.classify_mask(md)
    kc = torch.full((B, H, L, D), float("nan"), dtype=tdt, device=dev)
    vc = torch.full((B, H, L, D), float("nan"), dtype=tdt, device=dev)
    out = op.prefill(q.to(dev), k.to(dev), v.to(dev), kc, vc, torch.from_numpy(f).to(dev), attn_mask=md, mask_tile_classes=table)
    torch.cuda.synchronize()
    assert not torch.isnan(out).any() and not torch.isnan(kc).any() and not torch.isnan(vc).any()
    for b, h in pairs:
        qs, ks, vs = (x[b:b + 1, :, h:h + 1, :].contiguous().numpy() for x in (q, k, v))
        kr = np.full((1, 1, L, D), np.nan, NP_DT[dtype])
        vr = np.full((1, 1, L, D), np.nan, NP_DT[dtype])
        want = ref.prefill_attn(qs, ks, vs, kr, vr, f, start_pos=0, attn_mask=mask, acc_double=True, threads=16)
        assert_cache_bit_exact(kc[b:b + 1, h:h + 1].cpu().numpy(), kr, f"k_cache ({b},{h})")
        assert_cache_bit_exact(vc[b:b + 1, h:h + 1].cpu().numpy(), vr, f"v_cache ({b},{h})")
        got = out[b:b + 1, h:h + 1].cpu().numpy()
        if fast:  # the single-fp16-query product is judged on ordinary data elsewhere; here it must stay inside the bar
            assert np.abs(got - want).max() <= 2e-3
        else:
            float_ref = None
            if dtype == "f32":
                float_ref = lambda: ref.prefill_attn(qs, ks, vs, kr.copy(), vr.copy(), f, start_pos=0, attn_mask=mask, threads=16)
            assert_out_close(got, want, dtype, f"benchmark shape, pair ({b},{h})", float_ref=float_ref)


def test_prefill_then_decode_steps_agree_with_oracle_sequence(gpu):
    """Prompt of 70 tokens, then 5 decode steps on the same caches: every step against the oracle, caches
    bit-identical at the end (the two paths write the same rows the same way)."""
    import torch
    from fasterllama_amd.decode_attn import PrefillAttention
    B, H, D, L, S = 2, 4, 128, 128, 70
    q, k, v, kc, vc, f = make(B, H, D, L, S, "f16", seed=3)
    mask = causal_mask(L)
    kc_ref, vc_ref = kc.copy(), vc.copy()
    t = lambda a: torch.from_numpy(a).to(gpu)
    op = PrefillAttention(B, H, D, L, S, torch.float16, device=gpu)
    kc_d, vc_d, f_d, m_d = t(kc), t(vc), t(f), t(mask)
    want = ref.prefill_attn(q, k, v, kc_ref, vc_ref, f, attn_mask=mask, acc_double=True, threads=8)
    out = op.prefill(t(q), t(k), t(v), kc_d, vc_d, f_d, attn_mask=m_d)
    assert_out_close(out.cpu().numpy(), want, "f16", "prompt")
    for step in range(5):
        qs = synth.normal((B, 1, H, D), np.float16, synth.TENSOR_Q, seed=100 + step)
        ks = synth.normal((B, 1, H, D), np.float16, synth.TENSOR_K_NEW, seed=100 + step)
        vs = synth.normal((B, 1, H, D), np.float16, synth.TENSOR_V_NEW, seed=100 + step)
        w = ref.decode_attn(qs, ks, vs, kc_ref, vc_ref, f, start_pos=S + step, attn_mask=mask, acc_double=True)
        g = op.forward(t(qs), t(ks), t(vs), kc_d, vc_d, f_d, start_pos=S + step, attn_mask=m_d)
        assert_out_close(g.cpu().numpy(), w, "f16", f"decode step {step}")
    assert_cache_bit_exact(kc_d.cpu().numpy(), kc_ref, "k_cache")
    assert_cache_bit_exact(vc_d.cpu().numpy(), vc_ref, "v_cache")


def test_prefill_equals_token_by_token_decode(gpu):
    """With a causal mask, row s of the prompt-phase output equals the decode step at position s."""
    import torch
    from fasterllama_amd.decode_attn import PrefillAttention
    B, H, D, L, S = 1, 2, 64, 64, 40
    q, k, v, kc, vc, f = make(B, H, D, L, S, "f32", seed=9)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(gpu)
    op = PrefillAttention(B, H, D, L, S, torch.float32, device=gpu)
    f_d, m_d = t(f), t(causal_mask(L))
    kc1, vc1 = t(kc), t(vc)
    full = op.prefill(t(q), t(k), t(v), kc1, vc1, f_d, attn_mask=m_d).cpu().numpy()
    kc2, vc2 = t(kc), t(vc)
    for s in range(S):
        o = op.forward(t(q[:, s:s + 1]), t(k[:, s:s + 1]), t(v[:, s:s + 1]), kc2, vc2, f_d, start_pos=s,
                       attn_mask=m_d).cpu().numpy().reshape(B, H, D)
        assert np.abs(o - full[:, :, s]).max() <= 2e-6, s
    assert torch.equal(kc1[:, :, :S], kc2[:, :, :S]) and torch.equal(vc1[:, :, :S], vc2[:, :, :S])


def test_prefill_int32_prologue_and_int8_epilogue(gpu):
    import torch
    from fasterllama_amd.decode_attn import PrefillAttention
    B, H, D, L, S, P = 2, 8, 128, 160, 100, 0
    rng = np.random.default_rng(8)
    qi, ki, vi = (rng.integers(-20000, 20000, (B, S, H, D), dtype=np.int32) for _ in range(3))
    s_in = ((rng.random((B, S)) + 0.5) * 2e-3).astype(np.float32)
    wq, wk, wv = ((rng.random(H * D) * 3e-2 + 1e-3).astype(np.float32) for _ in range(3))
    _, _, _, kc, vc, f = make(B, H, D, L, S, "f16")
    mask = causal_mask(L)
    kc_ref, vc_ref = kc.copy(), vc.copy()
    want = ref.prefill_attn(qi, ki, vi, kc_ref, vc_ref, f, start_pos=P, attn_mask=mask, acc_double=True, threads=8,
                            inp_scale=s_in, wq_scale=wq, wk_scale=wk, wv_scale=wv)
    t = lambda a: torch.from_numpy(a).to(gpu)
    op = PrefillAttention(B, H, D, L, S, torch.float16, device=gpu)
    out = torch.empty(B, H, S, D, device=gpu)
    q8 = torch.empty(B, S, H * D, dtype=torch.int8, device=gpu)
    sc = torch.empty(B, S, device=gpu)
    kc_d, vc_d = t(kc), t(vc)
    op.prefill(t(qi), t(ki), t(vi), kc_d, vc_d, t(f), start_pos=P, out=out, attn_mask=t(mask), qkv_inp_scale=t(s_in),
               q_weight_scale=t(wq), k_weight_scale=t(wk), v_weight_scale=t(wv), out_int8=q8, out_scale=sc)
    torch.cuda.synchronize()
    assert_cache_bit_exact(kc_d.cpu().numpy(), kc_ref, "k_cache")
    assert_out_close(out.cpu().numpy(), want, "f16", "prologue")
    q_ref, s_ref = ref.attn_quantize_transpose(out.cpu().numpy())
    assert np.array_equal(q8.cpu().numpy(), q_ref) and np.array_equal(sc.cpu().numpy(), s_ref)
    q_or, s_or = ref.attn_quantize_transpose(want)
    assert np.abs(q8.cpu().numpy().astype(np.int32) - q_or.astype(np.int32)).max() <= 1


@pytest.mark.parametrize("dtype,D", [("f16", 128), ("f32", 128), ("f16", 64), ("f16", 256), ("f32", 512)])
def test_prefill_with_a_persistent_mask_class_table(gpu, dtype, D):
    """fl_prefill_mask_classify once per mask instead of a classification launch per call: bit-identical outputs
    for masks with dropped, zero and mixed tiles, at start positions that use the table (multiples of 32) and
    at one that falls back to the per-call classification."""
    import torch
    from fasterllama_amd.decode_attn import PrefillAttention
    B, H, L = 2, 3, 320
    tdt = torch.float16 if dtype == "f16" else torch.float32
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(gpu)
    r, c = np.arange(L)[:, None], np.arange(L)[None, :]
    masks = {
        "causal -FLT_MAX": np.where(c > r, -FMAX, 0.0),
        "causal -1e5": np.where(c > r, -1e5, 0.0),
        "window 70": np.where((c > r) | (c < r - 70), -FMAX, 0.0),
        "dense random": np.random.default_rng(4).standard_normal((L, L)) * 2,
    }
    for name, m in masks.items():
        m = m.astype(np.float32)
        for S, P in ((100, 0), (129, 64), (60, 224), (50, 37)):
            q, k, v, kc, vc, f = make(B, H, D, L, S, dtype, 7 + S)
            want = ref.prefill_attn(q, k, v, kc.copy(), vc.copy(), f, start_pos=P, attn_mask=m, acc_double=True, threads=16)
            op = PrefillAttention(B, H, D, L, S, tdt, device=gpu)
            md = t(m)
            table = op.classify_mask(md)
            outs = []
            for tab in (None, table):
                kc_d, vc_d = t(kc), t(vc)
                outs.append(op.prefill(t(q), t(k), t(v), kc_d, vc_d, t(f), start_pos=P, attn_mask=md,
                                       mask_tile_classes=tab).cpu().numpy())
            assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32)), f"{name} S={S} P={P}"
            assert_out_close(outs[1], want, dtype, f"class table, {name} S={S} P={P}",
                             float_ref=lambda: ref.prefill_attn(q, k, v, kc.copy(), vc.copy(), f, start_pos=P, attn_mask=m, threads=16))
    # the table itself: 0 = every entry <= -1e30, 1 = every entry zero, 3 = the diagonal tile of a causal mask (zero
    # up to the row's own place in the tile, <= -1e30 after it), 2 = anything else
    # layout: byte [key tile][row block], rows padded to a multiple of four row blocks
    tab = op.classify_mask(t(masks["causal -FLT_MAX"].astype(np.float32))).cpu().numpy().reshape(10, 12)[:, :10].T
    assert (np.diag(tab) == 3).all() and (np.tril(tab, -1)[np.tril_indices(10, -1)] == 1).all() \
        and (tab[np.triu_indices(10, 1)] == 0).all()
    tab = op.classify_mask(t(masks["causal -1e5"].astype(np.float32))).cpu().numpy().reshape(10, 12)[:, :10].T
    assert (np.diag(tab) == 2).all() and (tab[np.triu_indices(10, 1)] == 2).all()  # -1e5 is not provably zero weight
    tab = op.classify_mask(t(masks["window 70"].astype(np.float32))).cpu().numpy().reshape(10, 12)[:, :10].T
    assert (np.diag(tab) == 3).all() and (tab[np.arange(4, 10), np.arange(0, 6)] == 0).all()


@pytest.mark.parametrize("dtype", ["f16", "f32"])
def test_prefill_passes_append_then_attention_equals_one_call(gpu, dtype):
    """fl_prefill_attn_forward_passes: pass 1 (RoPE + append, classification) followed by pass 2 (attention) gives the
    bits of the whole call, pass 2 alone leaves the caches untouched, and a repeated pass 2 recomputes the same output."""
    import torch
    from fasterllama_amd.decode_attn import PrefillAttention
    B, H, D, L, S, P = 2, 3, 128, 256, 150, 32
    tdt = torch.float16 if dtype == "f16" else torch.float32
    q, k, v, kc, vc, f = make(B, H, D, L, S, dtype, 5)
    mask = causal_mask(L, -FMAX)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(gpu)
    op = PrefillAttention(B, H, D, L, S, tdt, device=gpu)
    qd, kd, vd, fd, md = t(q), t(k), t(v), t(f), t(mask)
    kc1, vc1 = t(kc), t(vc)
    whole = op.prefill(qd, kd, vd, kc1, vc1, fd, start_pos=P, attn_mask=md)
    kc2, vc2 = t(kc), t(vc)
    out = torch.full((B, H, S, D), float("nan"), dtype=torch.float32, device=gpu)
    io = op.make_io(qd, kd, vd, kc2, vc2, fd, out, start_pos=P, attn_mask=md)
    capi.check(op.launch_prefill(io, S, passes=1))
    torch.cuda.synchronize()
    assert torch.isnan(out).all()  # the append pass writes no output
    assert torch.equal(kc2.view(torch.uint8), kc1.view(torch.uint8)) and torch.equal(vc2.view(torch.uint8), vc1.view(torch.uint8))
    for _ in range(2):
        out.fill_(float("nan"))
        capi.check(op.launch_prefill(io, S, passes=2))
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int32), whole.view(torch.int32))
        assert torch.equal(kc2.view(torch.uint8), kc1.view(torch.uint8))
    assert op.launch_prefill(io, S, passes=0) == capi.FL_ATTN_ERR_ARGUMENT


def test_prefill_argument_errors(gpu):
    import torch
    from fasterllama_amd.decode_attn import PrefillAttention
    with pytest.raises(capi.FlAttnError) as e:
        PrefillAttention(1, 2, 48, 64, 16, torch.float16, device=gpu)
    assert e.value.status == capi.FL_ATTN_ERR_HEAD_DIM
    op = PrefillAttention(1, 2, 64, 64, 16, torch.float16, device=gpu)
    z = torch.zeros(1, 16, 2, 64, dtype=torch.float16, device=gpu)
    kc = torch.zeros(1, 2, 64, 64, dtype=torch.float16, device=gpu)
    f = torch.zeros(64, 64, device=gpu)
    with pytest.raises(capi.FlAttnError) as e:
        op.prefill(z, z, z, kc, kc, f, start_pos=50)  # 50 + 16 > 64
    assert e.value.status == capi.FL_ATTN_ERR_POSITION
    with pytest.raises(capi.FlAttnError) as e:
        op.prefill(z, z, z, kc, kc, f, start_pos=0, start_pos_per_seq=torch.zeros(1, dtype=torch.int32, device=gpu))
    assert e.value.status == capi.FL_ATTN_ERR_ARGUMENT
