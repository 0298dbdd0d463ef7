"""Parity of the HIP path (through the C ABI) with the CPU oracle: the five benchmark
configurations at full size, edge shapes, masks, head sizes, ragged batches, split invariance."""
import ctypes as C

import numpy as np
import pytest

from fasterllama_amd import capi, synth
from helpers import Case, assert_cache_bit_exact, assert_out_close
from oracle import ref

pytestmark = pytest.mark.gpu


def check(c, gpu, nsplit=0, what="", entry="forward", op=None):
    ref64, kc_ref, vc_ref = c.run_oracle(acc_double=True, threads=16)
    out, kc, vc, op = c.run_gpu(gpu, nsplit=nsplit, entry=entry, op=op)
    assert_cache_bit_exact(kc, kc_ref, what + " k_cache")
    assert_cache_bit_exact(vc, vc_ref, what + " v_cache")
    bad_pos = (c.positions() < 0) | (c.positions() >= c.L)
    if c.pos is not None:
        bad_pos |= c.positions() > c.bound()
    if bad_pos.any():
        assert np.isnan(out[bad_pos]).all() and np.isnan(ref64[bad_pos]).all()
        out, ref64 = out[~bad_pos], ref64[~bad_pos]
    keep = ~bad_pos
    err = assert_out_close(out, ref64, c.dtype, what, head_dim=c.D,
                           float_ref=lambda: c.run_oracle(acc_double=False, threads=16)[0][keep])
    return out, err, op


# ----------------------------------------------------------------------------- the five configurations

def test_config3_headline_full_size(gpu):
    # B=64, 32 heads, D=128, fp16, 2048 attended rows: every output element against the oracle
    c = Case(64, 32, 128, 2048, "f16", start_pos=2047)
    out, err, op = check(c, gpu, what="config3")
    print(f"config3 max_abs_err={err:.3e} plan nsplit={op.plan(2048).nsplit}")
    # size-independent property at full size: each output row is a convex combination of V rows
    vmax = np.abs(c.v_cache.astype(np.float32)).max(axis=2).reshape(64, -1)
    assert (np.abs(out) <= np.maximum(vmax, np.abs(c.v_new.reshape(64, -1).astype(np.float32))) + 1e-6).all()


@pytest.mark.parametrize("nsplit", [0, 1, 2, 7, 64])
def test_config4_long_context_split_invariance(gpu, nsplit):
    # B=1, 32 heads, ctx 4096, a few K rows scaled by 8 (softmax max-subtraction stress)
    c = Case(1, 32, 128, 4096, "f16", start_pos=4095, scale_rows=(17, 1000, 4000))
    check(c, gpu, nsplit=nsplit, what=f"config4 nsplit={nsplit}")


def test_config5_ragged_13b_nan_padding(gpu):
    # B=32, 40 heads, per-sequence lengths U[1,4096], padded slots NaN: must never be read
    B, L = 32, 4096
    lens = synth.uniform_int(B, 1, L, synth.TENSOR_LENS, 1234)
    lens[0], lens[1] = 1, L  # force both extremes
    c = Case(B, 40, 128, L, "f16", lens=lens, pad=np.nan)
    out, err, _ = check(c, gpu, what="config5")
    assert np.isfinite(out).all()


def test_config2_fp32_cache_variant(gpu):
    # the reference's own cache type (float) at the LLaMA2-7B shape
    c = Case(8, 32, 128, 1024, "f32", start_pos=1023)
    check(c, gpu, what="config2 f32")


# ----------------------------------------------------------------------------- one-launch steps (merge inside the streaming kernel)

@pytest.mark.parametrize("nsplit", [0, 2, 7, 64])
def test_config4_one_launch_equals_two_launches_bitwise(gpu, nsplit):
    # after fl_decode_attn_workspace_init the last workgroup of each (b,h) merges the partials: the same
    # arithmetic in the same order as the combine launch, so the outputs agree bit for bit
    c = Case(1, 32, 128, 4096, "f16", start_pos=4095, scale_rows=(17, 1000, 4000))
    two = c.run_gpu(gpu, nsplit=nsplit)[0]
    one, _, op = check(c, gpu, nsplit=nsplit, what=f"config4 one launch nsplit={nsplit}", entry="ready")
    assert op.plan(4096).nsplit > 1
    assert np.array_equal(one, two)
    # the arrival counters are back at zero: the same workspace serves further steps, also other contexts
    for ctx in (4096, 1000, 65, 4096):
        c2 = Case(1, 32, 128, 4096, "f16", start_pos=ctx - 1, seed=ctx)
        check(c2, gpu, what=f"one launch, reused workspace, ctx={ctx}", entry="ready", op=op)


@pytest.mark.parametrize("dtype", ["f16", "f32"])
def test_one_launch_ragged_masks_and_invalid_positions(gpu, dtype):
    B, L = 7, 1024
    lens = np.array([1, 1024, 0, 333, 1025, 64, 65])  # positions -1 and 1024 are invalid
    m = (np.random.default_rng(3).standard_normal((L, L)) * 2).astype(np.float32)
    c = Case(B, 5, 128, L, dtype, lens=lens, pad=np.nan, mask=m)
    _, _, op = check(c, gpu, nsplit=6, what="one launch ragged", entry="ready")
    check(c, gpu, what="one launch ragged, again", entry="ready", op=op)
    lens2 = np.array([4, 302, 1024, 301, 1001, 2, 300])
    c2 = Case(B, 5, 128, L, dtype, lens=lens2, pad=np.nan, max_start_pos=300)
    check(c2, gpu, what="one launch, bound 300", entry="ready", op=op)


@pytest.mark.parametrize("D", [32, 64, 256, 512, 1024])
def test_one_launch_head_sizes(gpu, D):
    for dtype in ("f16", "f32"):
        c = Case(2, 2, D, 300, dtype, start_pos=277, seed=D)
        check(c, gpu, nsplit=3, what=f"one launch D={D} {dtype}", entry="ready")


# ----------------------------------------------------------------------------- context lengths around tile edges

@pytest.mark.parametrize("dtype", ["f16", "f32"])
@pytest.mark.parametrize("ctx", [1, 2, 3, 15, 16, 17, 63, 64, 65, 66, 127, 128, 129, 191, 257, 1000])
def test_context_lengths(gpu, dtype, ctx):
    c = Case(2, 3, 128, 1024, dtype, start_pos=ctx - 1, seed=ctx)
    check(c, gpu, what=f"ctx={ctx}")


def test_ctx1_is_exactly_v_new(gpu):
    c = Case(3, 5, 64, 8, "f16", start_pos=0)
    out, _, _ = check(c, gpu)
    assert np.array_equal(out, c.v_new.reshape(3, -1).astype(np.float32))


@pytest.mark.parametrize("dtype", ["f16", "f32"])
@pytest.mark.parametrize("D", [32, 64, 96, 128, 256, 512, 1024])
def test_head_sizes(gpu, dtype, D):
    c = Case(2, 2, D, 300, dtype, start_pos=277, seed=D)
    check(c, gpu, what=f"D={D}")
    check(c, gpu, nsplit=3, what=f"D={D} nsplit=3")


@pytest.mark.parametrize("B,H", [(1, 1), (3, 5), (5, 7), (2, 40), (1, 64)])
def test_head_and_batch_counts_need_no_divisibility(gpu, B, H):
    # the reference kernels need head_num % 4 == 0 (grid = head_num / 4); this path does not
    c = Case(B, H, 128, 200, "f16", start_pos=150, seed=B * 100 + H)
    check(c, gpu, what=f"B={B} H={H}")


# ----------------------------------------------------------------------------- cache indexing, bit exact

@pytest.mark.parametrize("dtype", ["f32", "f16"])
@pytest.mark.parametrize("P", [0, 1, 4])
def test_store_cache_integer_pattern(gpu, dtype, P):
    # shape of the reference's testStorecache (samples/test.cu:352-362); integer patterns are exact
    B, L, H, D = 2, 5, 32, 128
    c = Case(B, H, D, L, dtype, start_pos=P, rope_row=0)
    dt = c.k_new.dtype
    pat = (np.arange(B * H * D) % 2048).reshape(B, 1, H, D)
    c.k_new[:] = pat.astype(dt)
    c.v_new[:] = (pat + 1).astype(dt)
    c.k_cache[:] = dt.type(-7)
    c.v_cache[:] = dt.type(-9)
    _, kc, vc, _ = c.run_gpu(gpu)
    for b in range(B):
        for h in range(H):
            assert np.array_equal(kc[b, h, P], c.k_new[b, 0, h]) and np.array_equal(vc[b, h, P], c.v_new[b, 0, h])
    keep = np.ones(L, bool); keep[P] = False
    assert (kc[:, :, keep] == -7).all() and (vc[:, :, keep] == -9).all()


def test_multi_step_decode_keeps_caches_bit_identical(gpu):
    import torch
    from fasterllama_amd.decode_attn import DecodeAttention
    B, H, D, L, P0, steps = 2, 4, 128, 96, 40, 24
    c = Case(B, H, D, L, "f16", start_pos=P0, seed=77)
    kc_h, vc_h = c.k_cache.copy(), c.v_cache.copy()
    kc_d, vc_d = torch.from_numpy(c.k_cache).to(gpu), torch.from_numpy(c.v_cache).to(gpu)
    f_d = torch.from_numpy(c.freq).to(gpu)
    op = DecodeAttention(B, H, D, L, torch.float16, device=gpu)
    for t in range(steps):
        q = synth.normal((B, 1, H, D), np.float16, synth.TENSOR_Q, seed=1000 + t)
        k = synth.normal((B, 1, H, D), np.float16, synth.TENSOR_K_NEW, seed=1000 + t)
        v = synth.normal((B, 1, H, D), np.float16, synth.TENSOR_V_NEW, seed=1000 + t)
        want = ref.decode_attn(q, k, v, kc_h, vc_h, c.freq, start_pos=P0 + t, acc_double=True)
        got = op.forward(*(torch.from_numpy(a).to(gpu) for a in (q, k, v)), kc_d, vc_d, f_d, start_pos=P0 + t)
        assert_out_close(got.cpu().numpy(), want, "f16", f"step {t}")
    assert_cache_bit_exact(kc_d.cpu().numpy(), kc_h, "k_cache after 24 steps")
    assert_cache_bit_exact(vc_d.cpu().numpy(), vc_h, "v_cache after 24 steps")


# ----------------------------------------------------------------------------- masks

def causal_mask(L, fill=-1e5):
    # standard causal convention of the reference's softmax test (samples/test.cu:427-437)
    return np.where(np.arange(L)[None, :] > np.arange(L)[:, None], fill, 0.0).astype(np.float32)


def strict_mask(L):
    # the samples' mask: (row > col) ? 0 : -FLT_MAX  (samples/llama_fp16.cu:73-81)
    fm = np.finfo(np.float32).max
    return np.where(np.arange(L)[:, None] > np.arange(L)[None, :], 0.0, -fm).astype(np.float32)


@pytest.mark.parametrize("dtype", ["f16", "f32"])
@pytest.mark.parametrize("nsplit", [0, 4])
def test_causal_and_strict_masks(gpu, dtype, nsplit):
    L, P = 512, 300
    base = Case(2, 4, 128, L, dtype, start_pos=P)
    out0, _, _ = check(base, gpu, nsplit=nsplit)
    c = Case(2, 4, 128, L, dtype, start_pos=P, mask=causal_mask(L))
    out1, _, _ = check(c, gpu, nsplit=nsplit, what="causal")
    assert np.array_equal(out0, out1)  # a zero mask row changes nothing, bit for bit
    check(Case(2, 4, 128, L, dtype, start_pos=P, mask=strict_mask(L)), gpu, nsplit=nsplit, what="strict")
    # random additive mask with a hidden suffix
    m = (np.random.default_rng(1).standard_normal((L, L)) * 2).astype(np.float32)
    m[P, 200:P] = -1e5
    check(Case(2, 4, 128, L, dtype, start_pos=P, mask=m), gpu, nsplit=nsplit, what="random mask")


def test_fully_masked_row_is_nan_like_the_reference_arithmetic(gpu):
    # strict mask at position 0: max stays at the -1e9 floor, every exp underflows to 0, 0/0 = NaN
    c = Case(1, 4, 64, 16, "f32", start_pos=0, mask=strict_mask(16))
    want, _, _ = c.run_oracle()
    out, _, _, _ = c.run_gpu(gpu)
    assert np.isnan(want).all() and np.isnan(out).all()


def test_minus_infinity_mask_entries(gpu):
    L, P = 128, 100
    m = np.zeros((L, L), np.float32)
    m[P, 10:60] = -np.inf
    check(Case(1, 4, 128, L, "f16", start_pos=P, mask=m), gpu, what="-inf mask")
    check(Case(1, 4, 128, L, "f16", start_pos=P, mask=m), gpu, nsplit=5, what="-inf mask split")


# ----------------------------------------------------------------------------- RoPE row, scale, ragged edge cases

def test_literal_reference_rope_row_zero(gpu):
    # the reference as written rotates decode tokens by table row 0 (decoder_kernels.cu:440)
    c = Case(2, 4, 128, 256, "f32", start_pos=200, rope_row=0)
    _, kc, _, _ = c.run_gpu(gpu)
    assert np.array_equal(kc[:, :, 200], c.k_new.reshape(2, 4, 128))
    check(c, gpu, what="rope_row=0")
    check(Case(2, 4, 128, 256, "f32", start_pos=200, rope_row=77), gpu, what="rope_row=77")


def test_ragged_with_out_of_range_positions(gpu):
    B, L = 6, 64
    lens = np.array([1, 64, 0, 33, 65, 17])  # positions -1 and 64 are invalid: NaN output, no store
    c = Case(B, 3, 128, L, "f16", lens=lens)
    check(c, gpu, what="ragged invalid")
    check(c, gpu, nsplit=4, what="ragged invalid split")


@pytest.mark.parametrize("nsplit", [0, 1, 4])
def test_position_above_the_max_start_pos_hint_is_poisoned_not_truncated(gpu, nsplit):
    # the launch is planned for max_start_pos; a device-side position beyond it must not be served from a
    # truncated context, nor make the merge read partials nobody wrote: NaN output, caches untouched
    lens = np.array([4, 302, 2048, 301, 1001, 2])
    c = Case(6, 3, 128, 2048, "f16", lens=lens, pad=np.nan, max_start_pos=300)
    out, _, op = check(c, gpu, nsplit=nsplit, what=f"bound 300 nsplit={nsplit}")
    assert np.isfinite(out).all() and out.shape[0] == 3  # sequences 0, 3 and 5 are served
    c32 = Case(6, 3, 128, 2048, "f32", lens=lens, pad=np.nan, max_start_pos=300)
    check(c32, gpu, nsplit=nsplit, what=f"bound 300 f32 nsplit={nsplit}")


def test_ragged_lengths_all_tile_remainders(gpu):
    lens = np.arange(1, 131)
    c = Case(130, 2, 64, 130, "f16", lens=lens, pad=np.nan)
    check(c, gpu, what="ragged 1..130")
    check(c, gpu, nsplit=3, what="ragged 1..130 split")


def test_determinism(gpu):
    c = Case(4, 8, 128, 2048, "f16", start_pos=2000)
    a = c.run_gpu(gpu, nsplit=5)[0]
    b = c.run_gpu(gpu, nsplit=5)[0]
    assert np.array_equal(a, b)


def test_custom_softmax_scale(gpu):
    import torch
    from fasterllama_amd.decode_attn import DecodeAttention
    c = Case(1, 4, 128, 128, "f32", start_pos=100)
    kc, vc = c.k_cache.copy(), c.v_cache.copy()
    want = ref.decode_attn(c.q, c.k_new, c.v_new, kc, vc, c.freq, start_pos=100, scale=0.05, acc_double=True)
    op = DecodeAttention(1, 4, 128, 128, torch.float32, softmax_scale=0.05, device=gpu)
    t = lambda a: torch.from_numpy(a).to(gpu)
    got = op.forward(t(c.q), t(c.k_new), t(c.v_new), t(c.k_cache), t(c.v_cache), t(c.freq), start_pos=100)
    assert_out_close(got.cpu().numpy(), want, "f32", "scale=0.05", head_dim=128)


# ----------------------------------------------------------------------------- error behaviour on the device path

def test_forward_reports_errors_instead_of_exiting(gpu):
    import torch
    from fasterllama_amd.decode_attn import DecodeAttention
    op = DecodeAttention(2, 4, 128, 64, torch.float16, device=gpu)
    z = lambda *s: torch.zeros(*s, dtype=torch.float16, device=gpu)
    q, kc = z(2, 1, 4, 128), z(2, 4, 64, 128)
    f = torch.zeros(64, 128, device=gpu)
    with pytest.raises(capi.FlAttnError) as e:
        op.forward(q, q, q, kc, kc, f, start_pos=64)
    assert e.value.status == capi.FL_ATTN_ERR_POSITION
    with pytest.raises(capi.FlAttnError) as e:
        op.forward(q, q, q, kc.view(-1)[1:], kc, f, start_pos=3)
    assert e.value.status == capi.FL_ATTN_ERR_ALIGNMENT
    with pytest.raises(capi.FlAttnError) as e:
        DecodeAttention(2, 4, 48, 64, torch.float16, device=gpu)  # the reference rejects it too (decoder_kernels.cu:564-588)
    assert e.value.status == capi.FL_ATTN_ERR_HEAD_DIM
    out = op.forward(q, q, q, kc, kc, f, start_pos=3)  # still usable afterwards
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()


# ----------------------------------------------------------------------------- extreme plans and offsets

@pytest.mark.parametrize("ctx,nsplit", [(100, 64), (4096, 1024), (777, 13), (65, 65)])
def test_forced_tiny_chunks(gpu, ctx, nsplit):
    # chunks of 1-6 rows: every workgroup runs only the bounds-checked tile
    c = Case(1, 4, 128, 4096, "f16", start_pos=ctx - 1, seed=ctx)
    check(c, gpu, nsplit=nsplit, what=f"ctx={ctx} nsplit={nsplit}")


def test_mask_with_custom_row_stride_and_ragged_positions(gpu):
    import torch
    from fasterllama_amd.decode_attn import DecodeAttention
    B, H, D, L, ld = 4, 3, 128, 96, 128  # mask rows padded to 128 floats
    lens = np.array([96, 5, 40, 77])
    mask = (np.random.default_rng(5).standard_normal((L, ld)) * 3).astype(np.float32)
    c = Case(B, H, D, L, "f16", lens=lens, pad=np.nan)
    kc, vc = c.k_cache.copy(), c.v_cache.copy()
    want = ref.decode_attn(c.q, c.k_new, c.v_new, kc, vc, c.freq, attn_mask=mask, mask_ld=ld,
                           start_pos_per_seq=lens - 1, acc_double=True)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(gpu)
    op = DecodeAttention(B, H, D, L, torch.float16, device=gpu)
    kc_d, vc_d = t(c.k_cache), t(c.v_cache)
    out = op.forward(t(c.q), t(c.k_new), t(c.v_new), kc_d, vc_d, t(c.freq), attn_mask=t(mask), mask_ld=ld,
                     start_pos_per_seq=t((lens - 1).astype(np.int32)), max_start_pos=95)
    torch.cuda.synchronize()
    assert_cache_bit_exact(kc_d.cpu().numpy(), kc, "k_cache")
    assert_out_close(out.cpu().numpy(), want, "f16", "mask_ld=128 ragged")


def test_byte_offsets_beyond_4_gib(gpu):
    """fp32 caches of 4 GiB each (B=64, H=32, L=4096, D=128): byte offsets of the last sequences
    exceed 2^32 and element offsets 2^30.  The oracle checks the first and the last sequence."""
    import torch
    from fasterllama_amd.decode_attn import DecodeAttention
    B, H, D, L, P = 64, 32, 128, 4096, 1500
    q = synth.normal((B, 1, H, D), np.float32, synth.TENSOR_Q)
    k = synth.normal((B, 1, H, D), np.float32, synth.TENSOR_K_NEW)
    v = synth.normal((B, 1, H, D), np.float32, synth.TENSOR_V_NEW)
    freq = synth.freq_cis_table(L, D)
    kc_d = torch.empty(B, H, L, D, dtype=torch.float32, device=gpu)
    vc_d = torch.empty_like(kc_d)
    host = {}
    per_seq = H * L * D
    for b in range(B):  # fill sequence by sequence: only two sequences are kept on the host
        kb = synth.normal((1, H, L, D), np.float32, synth.TENSOR_K_CACHE, index0=b * per_seq)
        vb = synth.normal((1, H, L, D), np.float32, synth.TENSOR_V_CACHE, index0=b * per_seq)
        kc_d[b:b + 1].copy_(torch.from_numpy(kb))
        vc_d[b:b + 1].copy_(torch.from_numpy(vb))
        if b in (0, B - 1):
            host[b] = (kb, vb)
    op = DecodeAttention(B, H, D, L, torch.float32, device=gpu)
    t = lambda a: torch.from_numpy(a).to(gpu)
    out = op.forward(t(q), t(k), t(v), kc_d, vc_d, t(freq), start_pos=P)
    torch.cuda.synchronize()
    out_h = out.cpu().numpy()
    assert np.isfinite(out_h).all()
    for b, (kb, vb) in host.items():
        want = ref.decode_attn(q[b:b + 1], k[b:b + 1], v[b:b + 1], kb, vb, freq, start_pos=P, acc_double=True, threads=16)
        assert_out_close(out_h[b:b + 1], want, "f32", f"sequence {b}", head_dim=D)
        assert_cache_bit_exact(kc_d[b:b + 1].cpu().numpy(), kb, f"k_cache of sequence {b}")
        assert_cache_bit_exact(vc_d[b:b + 1].cpu().numpy(), vb, f"v_cache of sequence {b}")
