"""Seeded sweeps over COMBINATIONS of the options the other GPU tests exercise one or two at a time: head size,
cache type, uniform or per-sequence positions, mask kind and row stride, forced splits, entry point, RoPE row,
softmax scale, int32 accumulators in, INT8 out.  Every case is small, drawn from its seed alone, and checked
against the CPU oracle to the same bars as everywhere else: caches bit-exact, FP32 within 1e-5 relative, fp16
within 2e-3 absolute, INT8 bit-exact with the CPU quantiser on the kernel's own float output."""
import numpy as np
import pytest

from fasterllama_amd import capi, synth
from helpers import NP_DT, assert_cache_bit_exact, assert_out_close
from oracle import ref

pytestmark = pytest.mark.gpu
FMAX = float(np.finfo(np.float32).max)


def draw_mask(rng, rows, ld, kind):
    """[rows, ld] additive mask.  Column 0 stays open so that no row is fully masked (that edge has its own test)."""
    r, c = np.arange(rows)[:, None], np.arange(ld)[None, :]
    if kind == "zeros":
        m = np.zeros((rows, ld))
    elif kind == "causal_fmax":
        m = np.where(c > r, -FMAX, 0.0)
    elif kind == "causal_1e5":
        m = np.where(c > r, -1e5, 0.0)
    elif kind == "window":
        w = int(rng.integers(3, 90))
        m = np.where((c > r) | (c < r - w), -FMAX, 0.0)
    elif kind == "inf_holes":
        m = np.where(rng.random((rows, ld)) < 0.3, -np.inf, 0.0)
    else:  # dense: finite biases with a few closed entries
        m = rng.standard_normal((rows, ld)) * 2
        m = np.where(rng.random((rows, ld)) < 0.2, -FMAX, m)
    m = m.astype(np.float32)
    m[:, 0] = 0.0
    return np.ascontiguousarray(m)


def draw_int32_inputs(rng, shape, B_tokens, HD):
    qi, ki, vi = (rng.integers(-20000, 20000, shape, dtype=np.int32) for _ in range(3))
    s_in = ((rng.random(B_tokens) + 0.5) * 2e-3).astype(np.float32)
    wq, wk, wv = ((rng.random(HD) * 3e-2 + 1e-3).astype(np.float32) for _ in range(3))
    return qi, ki, vi, s_in, wq, wk, wv


@pytest.mark.parametrize("seed", range(200))
def test_decode_step_random_combination(gpu, seed):
    import torch
    from fasterllama_amd.decode_attn import DecodeAttention
    rng = np.random.default_rng(1000 + seed)
    dtype = ("f16", "f32")[int(rng.integers(2))]
    D = int(rng.choice([32, 64, 96, 128, 128, 256]))
    B, H = int(rng.integers(1, 6)), int(rng.integers(1, 7))
    L = int(rng.integers(2, 420)) if rng.integers(4) else int(rng.integers(420, 1800))
    ragged = bool(rng.integers(2))
    nsplit = int(rng.choice([0, 0, 1, 2, 3, 5]))
    entry = ("forward", "ready", "noalloc")[int(rng.integers(3))]
    rope_row = int(rng.choice([-1, -1, 0, 1]))
    scale = float(rng.choice([0.0, 0.0, 0.05, 0.2]))
    mask_kind = str(rng.choice(["none", "zeros", "causal_fmax", "causal_1e5", "window", "inf_holes", "dense"]))
    i32, want_int8 = bool(rng.integers(3) == 0), bool(rng.integers(3) == 0)
    mask_ld = L + int(rng.choice([0, 0, 4, 13]))
    pos = rng.integers(0, L, B).astype(np.int32) if ragged else None
    P = 0 if ragged else int(rng.integers(0, L))
    bound = int(pos.max()) if ragged else -1
    what = (f"seed {seed}: {dtype} B={B} H={H} D={D} L={L} {'ragged ' + str(pos.tolist()) if ragged else 'P=' + str(P)} "
            f"nsplit={nsplit} {entry} rope_row={rope_row} scale={scale} mask={mask_kind}/ld{mask_ld} i32={i32} int8={want_int8}")
    print(what, flush=True)

    dt = NP_DT[dtype]
    kc = synth.normal((B, H, L, D), dt, synth.TENSOR_K_CACHE, seed)
    vc = synth.normal((B, H, L, D), dt, synth.TENSOR_V_CACHE, seed)
    for b in range(B):  # rows from the new token's on are stale: never read before they are written
        kc[b, :, (pos[b] if ragged else P):] = np.nan
        vc[b, :, (pos[b] if ragged else P):] = np.nan
    freq = synth.freq_cis_table(L, D)
    mask = None if mask_kind == "none" else draw_mask(rng, L, mask_ld, mask_kind)
    if i32:
        q, k, v, s_in, wq, wk, wv = draw_int32_inputs(rng, (B, 1, H, D), B, H * D)
        scales = dict(inp_scale=s_in, wq_scale=wq, wk_scale=wk, wv_scale=wv)
    else:
        q = synth.normal((B, 1, H, D), dt, synth.TENSOR_Q, seed)
        k = synth.normal((B, 1, H, D), dt, synth.TENSOR_K_NEW, seed)
        v = synth.normal((B, 1, H, D), dt, synth.TENSOR_V_NEW, seed)
        scales = {}

    def oracle(acc_double):
        kr, vr = kc.copy(), vc.copy()
        out = ref.decode_attn(q, k, v, kr, vr, freq, start_pos=P, rope_row=rope_row, attn_mask=mask, mask_ld=mask_ld,
                              start_pos_per_seq=pos, max_start_pos=bound, scale=scale or None, acc_double=acc_double,
                              threads=8, **scales)
        return out, kr, vr

    want, kc_ref, vc_ref = oracle(True)

    t = lambda a: None if a is None else torch.from_numpy(a).to(gpu)
    op = DecodeAttention(B, H, D, L, torch.float16 if dtype == "f16" else torch.float32, nsplit=nsplit,
                         softmax_scale=scale, device=gpu)
    if entry == "ready":
        op.init_workspace()
    kc_d, vc_d = t(kc), t(vc)
    out = torch.full((B, H * D), 7.0, dtype=torch.float32, device=gpu)
    q8 = torch.zeros(B, H * D, dtype=torch.int8, device=gpu) if want_int8 else None
    sc = torch.zeros(B, dtype=torch.float32, device=gpu) if want_int8 else None
    io = op.make_io(t(q), t(k), t(v), kc_d, vc_d, t(freq), out, start_pos=P, rope_row=rope_row, attn_mask=t(mask),
                    mask_ld=mask_ld, start_pos_per_seq=t(pos), max_start_pos=bound,
                    qkv_inp_scale=t(scales.get("inp_scale")), q_weight_scale=t(scales.get("wq_scale")),
                    k_weight_scale=t(scales.get("wk_scale")), v_weight_scale=t(scales.get("wv_scale")),
                    out_int8=q8, out_scale=sc)
    if entry == "noalloc":
        io.workspace, io.workspace_bytes = None, 0
        capi.check(op.launch_noalloc(io))
    else:
        capi.check(op.launch(io))
    torch.cuda.synchronize()
    assert_cache_bit_exact(kc_d.cpu().numpy(), kc_ref, what + " k_cache")
    assert_cache_bit_exact(vc_d.cpu().numpy(), vc_ref, what + " v_cache")
    got = out.cpu().numpy()
    assert_out_close(got, want, dtype, what, head_dim=D, float_ref=lambda: oracle(False)[0])
    if want_int8:
        q_ref, s_ref = ref.attn_quantize(got)
        assert np.array_equal(q8.cpu().numpy(), q_ref) and np.array_equal(sc.cpu().numpy(), s_ref), what


@pytest.mark.parametrize("seed", range(150))
def test_prompt_phase_random_combination(gpu, seed):
    import torch
    from fasterllama_amd.decode_attn import PrefillAttention
    rng = np.random.default_rng(2000 + seed)
    dtype = ("f16", "f32")[int(rng.integers(2))]
    D = int(rng.choice([32, 64, 96, 128, 128, 256, 512]))
    B, H = int(rng.integers(1, 4)), int(rng.integers(1, 5))
    S = int(rng.choice([1, 2, 31, 32, 33, 64, 100, 129, 200]))
    P = int(rng.choice([0, 0, 32, 64, 96, 5, 77]))
    L = P + S + int(rng.choice([0, 0, 7, 64]))
    rope_row = int(rng.choice([-1, -1, 0]))
    scale = float(rng.choice([0.0, 0.0, 0.05, 0.2]))
    mask_kind = str(rng.choice(["none", "zeros", "causal_fmax", "causal_fmax", "causal_1e5", "window", "inf_holes", "dense"]))
    i32, want_int8 = bool(rng.integers(3) == 0), bool(rng.integers(3) == 0)
    use_table = bool(rng.integers(2)) and mask_kind != "none"
    fast_qk = dtype == "f16" and not i32 and scale == 0.0 and bool(rng.integers(4) == 0)  # ordinary data only
    mask_ld = L + (0 if use_table else int(rng.choice([0, 0, 4, 13])))
    what = (f"seed {seed}: {dtype} B={B} H={H} D={D} L={L} S={S} P={P} rope_row={rope_row} scale={scale} "
            f"mask={mask_kind}/ld{mask_ld} table={use_table} i32={i32} int8={want_int8} fast_qk={fast_qk}")
    print(what, flush=True)

    dt = NP_DT[dtype]
    kc = synth.normal((B, H, L, D), dt, synth.TENSOR_K_CACHE, seed)
    vc = synth.normal((B, H, L, D), dt, synth.TENSOR_V_CACHE, seed)
    kc[:, :, P:] = np.nan
    vc[:, :, P:] = np.nan
    freq = synth.freq_cis_table(L, D)
    mask = None if mask_kind == "none" else draw_mask(rng, L, mask_ld, mask_kind)
    if i32:
        q, k, v, s_in, wq, wk, wv = draw_int32_inputs(rng, (B, S, H, D), B * S, H * D)
        scales = dict(inp_scale=s_in, wq_scale=wq, wk_scale=wk, wv_scale=wv)
    else:
        q = synth.normal((B, S, H, D), dt, synth.TENSOR_Q, seed)
        k = synth.normal((B, S, H, D), dt, synth.TENSOR_K_NEW, seed)
        v = synth.normal((B, S, H, D), dt, synth.TENSOR_V_NEW, seed)
        scales = {}

    def oracle(acc_double):
        kr, vr = kc.copy(), vc.copy()
        out = ref.prefill_attn(q, k, v, kr, vr, freq, start_pos=P, rope_row=rope_row, attn_mask=mask, mask_ld=mask_ld,
                               scale=scale or None, acc_double=acc_double, threads=16, **scales)
        return out, kr, vr

    want, kc_ref, vc_ref = oracle(True)

    t = lambda a: None if a is None else torch.from_numpy(a).to(gpu)
    op = PrefillAttention(B, H, D, L, S, torch.float16 if dtype == "f16" else torch.float32, softmax_scale=scale,
                          device=gpu, fast_qk=fast_qk)
    md = t(mask)
    table = op.classify_mask(md, mask_ld) if use_table else None
    kc_d, vc_d = t(kc), t(vc)
    out = torch.full((B, H, S, D), 7.0, dtype=torch.float32, device=gpu)
    q8 = torch.zeros(B, S, H * D, dtype=torch.int8, device=gpu) if want_int8 else None
    sc = torch.zeros(B, S, dtype=torch.float32, device=gpu) if want_int8 else None
    op.prefill(t(q), t(k), t(v), kc_d, vc_d, t(freq), start_pos=P, out=out, rope_row=rope_row, attn_mask=md,
               mask_ld=mask_ld, mask_tile_classes=table, qkv_inp_scale=t(scales.get("inp_scale")),
               q_weight_scale=t(scales.get("wq_scale")), k_weight_scale=t(scales.get("wk_scale")),
               v_weight_scale=t(scales.get("wv_scale")), out_int8=q8, out_scale=sc)
    torch.cuda.synchronize()
    assert_cache_bit_exact(kc_d.cpu().numpy(), kc_ref, what + " k_cache")
    assert_cache_bit_exact(vc_d.cpu().numpy(), vc_ref, what + " v_cache")
    got = out.cpu().numpy()
    assert_out_close(got, want, dtype, what, float_ref=lambda: oracle(False)[0])
    if want_int8:
        q_ref, s_ref = ref.attn_quantize_transpose(got)
        assert np.array_equal(q8.cpu().numpy(), q_ref) and np.array_equal(sc.cpu().numpy(), s_ref), what
