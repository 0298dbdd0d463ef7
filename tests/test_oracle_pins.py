"""Pins the CPU oracle (oracle/fl_ref_decode_attn.c) WITHOUT running the reference (CUDA-only, not
buildable here) and without retyping the oracle's own formulas: closed forms, invariants, an
independent complex-number/float64 brute force, torch's scaled_dot_product_attention, and committed
golden vectors.  A dropped term, a wrong sign or pairing in RoPE, a transposed operand, an
off-by-one in the attended rows or a wrong mask row fails at least one test here."""
import math
import os

import numpy as np
import pytest

from fasterllama_amd import synth
from oracle import ref

HERE = os.path.dirname(os.path.abspath(__file__))


# ----------------------------------------------------------------------------- independent brute force

def brute_force(q, k_new, v_new, k_cache, v_cache, pos, rope_pos, base=10000.0, mask_row=None, scale=None,
                store=lambda x: x):
    """float64 decode step for ONE (b,h): complex-multiplication RoPE, dense softmax.  Returns
    (out[D], probs[ctx], rotated k).  Shares no code and no formula layout with the oracle:
    pairs are complex numbers z = x0 + i x1 rotated by exp(i * rope_pos * w).  `store` models the
    rounding of the appended key row to the cache's storage type."""
    D = q.shape[-1]
    w = base ** (-2.0 * np.arange(D // 2) / D)
    rot = np.exp(1j * rope_pos * w)
    qc = (q[0::2].astype(np.float64) + 1j * q[1::2].astype(np.float64)) * rot
    kc = (k_new[0::2].astype(np.float64) + 1j * k_new[1::2].astype(np.float64)) * rot
    k_rot = np.empty(D); k_rot[0::2] = kc.real; k_rot[1::2] = kc.imag
    k_rot = store(k_rot)
    q_rot = np.empty(D); q_rot[0::2] = qc.real; q_rot[1::2] = qc.imag
    K = np.concatenate([k_cache[:pos].astype(np.float64), k_rot[None, :]], 0)
    V = np.concatenate([v_cache[:pos].astype(np.float64), v_new[None, :].astype(np.float64)], 0)
    s = K @ q_rot * (scale if scale is not None else 1.0 / math.sqrt(D))
    if mask_row is not None:
        s = s + mask_row[:pos + 1].astype(np.float64)
    m = max(-1e9, s.max())
    e = np.exp(s - m)
    p = e / e.sum()
    return p @ V, p, k_rot


def make(B, H, D, L, dt=np.float32, seed=7):
    q = synth.normal((B, 1, H, D), dt, synth.TENSOR_Q, seed)
    k = synth.normal((B, 1, H, D), dt, synth.TENSOR_K_NEW, seed)
    v = synth.normal((B, 1, H, D), dt, synth.TENSOR_V_NEW, seed)
    kc = synth.normal((B, H, L, D), dt, synth.TENSOR_K_CACHE, seed)
    vc = synth.normal((B, H, L, D), dt, synth.TENSOR_V_CACHE, seed)
    return q, k, v, kc, vc


# ----------------------------------------------------------------------------- RoPE table (A0)

def test_table_closed_forms():
    D, rows = 64, 300
    t = ref.freq_cis(rows, D).astype(np.float64)
    assert np.array_equal(t[0, 0::2], np.ones(D // 2)) and np.array_equal(t[0, 1::2], np.zeros(D // 2))
    assert np.allclose(t[:, 0::2] ** 2 + t[:, 1::2] ** 2, 1.0, atol=3e-7)
    # frequency 0 is 1 rad per position; the last frequency is base^(-(D-2)/D)
    assert abs(t[5, 0] - math.cos(5.0)) < 1e-7 and abs(t[5, 1] - math.sin(5.0)) < 1e-7
    w_last = 10000.0 ** (-(D - 2) / D)
    assert abs(t[299, D - 2] - math.cos(299 * w_last)) < 1e-7
    # angle addition: row(a+b) = row(a) * row(b) as complex numbers
    z = t[:, 0::2] + 1j * t[:, 1::2]
    assert np.allclose(z[100] * z[150], z[250], atol=5e-7)


def test_table_matches_independent_numpy_and_base_argument():
    for D, base in ((8, 10000.0), (128, 10000.0), (64, 500000.0)):
        a = ref.freq_cis(77, D, base)
        b = synth.freq_cis_table(77, D, base)
        assert np.abs(a.astype(np.float64) - b).max() <= 6e-8  # at most 1 ulp of values <= 1


# ----------------------------------------------------------------------------- closed forms of the step

@pytest.mark.parametrize("dt", [np.float32, np.float16])
def test_ctx1_returns_v_new_exactly(dt):
    B, H, D, L = 2, 3, 32, 4
    q, k, v, kc, vc = make(B, H, D, L, dt)
    f = ref.freq_cis(L, D)
    out = ref.decode_attn(q, k, v, kc, vc, f, start_pos=0)
    assert np.array_equal(out, v.reshape(B, H * D).astype(np.float32))  # p == 1.0 exactly
    assert np.array_equal(vc[:, :, 0, :], v.reshape(B, H, D))
    assert np.array_equal(kc[:, :, 0, :], k.reshape(B, H, D))  # RoPE row 0 is the identity


def test_identical_keys_give_mean_of_values():
    B, H, D, L, P = 1, 2, 16, 9, 8
    q, k, v, kc, vc = make(B, H, D, L)
    kc[:] = k.reshape(B, H, 1, D)
    f = ref.freq_cis(L, D)
    out = ref.decode_attn(q, k, v, kc, vc, f, start_pos=P, rope_row=0)  # row 0: k stored unrotated
    V = vc[:, :, :P + 1, :].astype(np.float64)
    assert np.allclose(out.reshape(B, H, D), V.mean(2), atol=2e-6)


def test_rope_pair_norm_and_row_selection():
    B, H, D, L, P = 1, 2, 64, 40, 33
    q, k, v, kc, vc = make(B, H, D, L)
    f = ref.freq_cis(L, D)
    ref.decode_attn(q, k, v, kc, vc, f, start_pos=P)
    stored = kc[0, :, P, :].astype(np.float64)
    src = k.reshape(H, D).astype(np.float64)
    assert np.allclose(stored[:, 0::2] ** 2 + stored[:, 1::2] ** 2, src[:, 0::2] ** 2 + src[:, 1::2] ** 2, rtol=1e-5)
    assert not np.allclose(stored, src)  # position 33 really rotates
    # rope_row selects the table row independently of the storage row (literal-reference mode = row 0)
    kc2, vc2 = kc.copy(), vc.copy()
    ref.decode_attn(q, k, v, kc2, vc2, f, start_pos=P, rope_row=0)
    assert np.array_equal(kc2[0, :, P, :], k.reshape(H, D))


def test_hand_computed_d4():
    # one head, D=4, position 1, theta = [1, 0.01]: worked by hand with complex arithmetic
    D, L = 4, 2
    q = np.array([1.0, 0.0, 0.0, 2.0], np.float32).reshape(1, 1, 1, D)
    k = np.array([0.5, -1.0, 1.0, 1.0], np.float32).reshape(1, 1, 1, D)
    v = np.array([1.0, 2.0, 3.0, 4.0], np.float32).reshape(1, 1, 1, D)
    kc = np.zeros((1, 1, L, D), np.float32); vc = np.zeros((1, 1, L, D), np.float32)
    kc[0, 0, 0] = [1.0, 1.0, 1.0, 1.0]
    vc[0, 0, 0] = [-1.0, 0.0, 1.0, 0.0]
    f = ref.freq_cis(L, D)
    out = ref.decode_attn(q, k, v, kc, vc, f, start_pos=1)
    c1, s1, c2, s2 = math.cos(1.0), math.sin(1.0), math.cos(0.01), math.sin(0.01)
    # (1+0i)e^{i} = c1 + i s1 ; (0+2i)e^{0.01i} = -2 s2 + 2i c2
    qr = [c1, s1, -2 * s2, 2 * c2]
    # (0.5 - i)e^{i} = (0.5c1 + s1) + i(0.5 s1 - c1) ; (1+i)e^{0.01i} = (c2 - s2) + i(c2 + s2)
    kr = [0.5 * c1 + s1, 0.5 * s1 - c1, c2 - s2, c2 + s2]
    assert np.allclose(kc[0, 0, 1], kr, atol=1e-7)
    s_old = sum(qr) * 0.5          # key row 0 is all ones; scale = 1/sqrt(4)
    s_new = sum(a * b for a, b in zip(qr, kr)) * 0.5
    p_new = 1.0 / (1.0 + math.exp(s_old - s_new))
    want = [(1 - p_new) * a + p_new * b for a, b in zip([-1.0, 0.0, 1.0, 0.0], [1.0, 2.0, 3.0, 4.0])]
    assert np.allclose(out[0], want, atol=1e-6)


def test_relative_position_property_via_multi_step_decode():
    """Decode 12 tokens with the oracle (each step appends R_j k_j), then observe the softmax
    probabilities through one-hot V rows and compare with Re(sum q conj(k) e^{i(m-j)w}): the
    score depends on positions only through m - j."""
    H, D, L = 1, 32, 16
    rng = np.random.default_rng(3)
    f = ref.freq_cis(L, D)
    kc = np.zeros((1, H, L, D), np.float32); vc = np.zeros((1, H, L, D), np.float32)
    ks = rng.standard_normal((12, D)).astype(np.float32)
    qs = rng.standard_normal((12, D)).astype(np.float32)
    w = 10000.0 ** (-2.0 * np.arange(D // 2) / D)
    for m in range(12):
        onehot = np.zeros(D, np.float32); onehot[m] = 1.0
        out = ref.decode_attn(qs[m].reshape(1, 1, H, D), ks[m].reshape(1, 1, H, D), onehot.reshape(1, 1, H, D),
                              kc, vc, f, start_pos=m)
        qz = qs[m, 0::2].astype(np.float64) + 1j * qs[m, 1::2]
        s = np.empty(m + 1)
        for j in range(m + 1):
            kz = ks[j, 0::2].astype(np.float64) + 1j * ks[j, 1::2]
            s[j] = np.real(np.sum(qz * np.conj(kz) * np.exp(1j * (m - j) * w))) / math.sqrt(D)
        p = np.exp(s - s.max()); p /= p.sum()
        assert np.allclose(out[0, :m + 1], p, atol=2e-6), m
        assert np.all(out[0, m + 1:] == 0.0)


# ----------------------------------------------------------------------------- brute force / library cross-checks

@pytest.mark.parametrize("dt,tol", [(np.float32, 2e-6), (np.float16, 5e-6)])
def test_config1_against_float64_brute_force(dt, tol):
    B, H, D, L, P = 1, 4, 64, 128, 127  # the reference-runnable plumbing case
    q, k, v, kc, vc = make(B, H, D, L, dt, seed=1234)
    f = ref.freq_cis(L, D)
    kc0, vc0 = kc.copy(), vc.copy()
    out32 = ref.decode_attn(q, k, v, kc, vc, f, start_pos=P)
    out64 = ref.decode_attn(q, k, v, kc0.copy(), vc0.copy(), f, start_pos=P, acc_double=True)
    store = (lambda x: x.astype(np.float32).astype(np.float16).astype(np.float64)) if dt == np.float16 else \
            (lambda x: x.astype(np.float32).astype(np.float64))
    for h in range(H):
        want, p, k_rot = brute_force(q[0, 0, h], k[0, 0, h], v[0, 0, h], kc0[0, h], vc0[0, h], P, P, store=store)
        assert abs(p.sum() - 1.0) < 1e-12
        assert np.abs(kc[0, h, P].astype(np.float64) - k_rot).max() <= (1e-3 if dt == np.float16 else 3e-7)
        assert np.abs(out64[0, h * D:(h + 1) * D] - want).max() < tol
        assert np.abs(out32[0, h * D:(h + 1) * D] - want).max() < 2e-5


def test_against_torch_sdpa():
    torch = pytest.importorskip("torch")
    B, H, D, L, P = 2, 3, 64, 50, 41
    q, k, v, kc, vc = make(B, H, D, L, seed=99)
    f = ref.freq_cis(L, D)
    out = ref.decode_attn(q, k, v, kc, vc, f, start_pos=P, acc_double=True)
    # after the step the cache holds the rotated key / new value at row P: attend with torch over rows 0..P
    cos, sin = f[P, 0::2], f[P, 1::2]
    qq = q.reshape(B, H, D)
    q_rot = np.empty_like(qq)
    q_rot[..., 0::2] = qq[..., 0::2] * cos - qq[..., 1::2] * sin
    q_rot[..., 1::2] = qq[..., 1::2] * cos + qq[..., 0::2] * sin
    tq = torch.from_numpy(q_rot).double().unsqueeze(2)
    tk = torch.from_numpy(kc[:, :, :P + 1]).double()
    tv = torch.from_numpy(vc[:, :, :P + 1]).double()
    want = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv).squeeze(2).reshape(B, H * D).numpy()
    assert np.abs(out - want).max() < 2e-6


# ----------------------------------------------------------------------------- mask semantics (A5 / A9)

def probs_via_onehot(mask, P, L=24, D=32, seed=5, **kw):
    q, k, v, kc, vc = make(1, 1, D, L, seed=seed)
    vc[:] = 0
    for j in range(L):
        vc[0, 0, j, j] = 1.0
    v[:] = 0
    v[0, 0, 0, P] = 1.0
    f = ref.freq_cis(L, D)
    return ref.decode_attn(q, k, v, kc, vc, f, start_pos=P, attn_mask=mask, **kw)[0]


def test_zero_mask_equals_no_mask_and_row_selection():
    L, P = 24, 17
    a = probs_via_onehot(None, P)
    b = probs_via_onehot(np.zeros((L, L), np.float32), P)
    assert np.array_equal(a, b)
    assert abs(a[:P + 1].sum() - 1.0) < 1e-6 and np.all(a[P + 1:] == 0)
    # the row used is start_pos: put the standard causal mask (0 for j<=row, -1e5 otherwise) and a
    # poison value in every other row
    m = np.full((L, L), 123.0, np.float32)
    m[P, :] = np.where(np.arange(L) <= P, 0.0, -1e5)
    assert np.allclose(probs_via_onehot(m, P), a, atol=1e-7)


def test_suffix_mask_equals_shorter_context():
    L, P = 24, 20
    m = np.zeros((L, L), np.float32)
    m[P, 10:P] = -1e5  # hide rows 10..19, keep the new token
    p = probs_via_onehot(m, P)
    assert np.all(p[10:P] == 0.0) and p[P] > 0
    assert abs(p.sum() - 1.0) < 1e-6


def test_strict_mask_hides_the_new_token_and_full_mask_gives_nan():
    # the sample's mask: mask[r][c] = (r > c) ? 0 : -FLT_MAX  (samples/llama_fp16.cu:73-81)
    L, P = 24, 9
    fm = np.finfo(np.float32).max
    m = np.where(np.arange(L)[:, None] > np.arange(L)[None, :], 0.0, -fm).astype(np.float32)
    p = probs_via_onehot(m, P)
    assert p[P] == 0.0 and abs(p[:P].sum() - 1.0) < 1e-6
    # row 0 of that mask hides everything: max stays at the -1e9 floor, every exp is 0, 0/0 = NaN
    assert np.isnan(probs_via_onehot(m, 0)).all()


def test_scale_argument_and_max_subtraction_stress():
    L, D, P = 24, 32, 23
    q, k, v, kc, vc = make(1, 1, D, L, seed=11)
    kc[0, 0, 5] *= 50.0  # a dominating key: softmax must stay finite
    f = ref.freq_cis(L, D)
    out = ref.decode_attn(q, k, v, kc.copy(), vc.copy(), f, start_pos=P)
    assert np.isfinite(out).all()
    want, p, _ = brute_force(q[0, 0, 0], k[0, 0, 0], v[0, 0, 0], kc[0, 0], vc[0, 0], P, P)
    assert np.allclose(out[0], want, atol=1e-5)
    out2 = ref.decode_attn(q, k, v, kc.copy(), vc.copy(), f, start_pos=P, scale=0.03125)
    want2, _, _ = brute_force(q[0, 0, 0], k[0, 0, 0], v[0, 0, 0], kc[0, 0], vc[0, 0], P, P, scale=0.03125)
    assert np.allclose(out2[0], want2, atol=1e-5)


# ----------------------------------------------------------------------------- cache indexing (A3), bit exact

@pytest.mark.parametrize("P", [0, 1, 4])
def test_cache_append_touches_exactly_row_P(P):
    # shape of the reference's testStorecache (samples/test.cu:352-362), one new token
    B, L, H, D = 2, 5, 32, 128
    idx = (np.arange(B * H * D, dtype=np.float32)).reshape(B, 1, H, D)
    q = np.ones((B, 1, H, D), np.float32)
    kc = np.full((B, H, L, D), -7.0, np.float32); vc = np.full((B, H, L, D), -9.0, np.float32)
    f = ref.freq_cis(L, D)
    ref.decode_attn(q, idx.copy(), (idx + 0.5).copy(), kc, vc, f, start_pos=P, rope_row=0)
    for b in range(B):
        for h in range(H):
            assert np.array_equal(kc[b, h, P], idx[b, 0, h]) and np.array_equal(vc[b, h, P], idx[b, 0, h] + 0.5)
    keep = np.ones(L, bool); keep[P] = False
    assert np.all(kc[:, :, keep, :] == -7.0) and np.all(vc[:, :, keep, :] == -9.0)


def test_ragged_equals_per_sequence_runs_and_ignores_padding():
    B, H, D, L = 5, 2, 32, 40
    q, k, v, kc, vc = make(B, H, D, L, np.float16, seed=21)
    lens = np.array([1, 40, 17, 2, 33])
    for b in range(B):
        kc[b, :, lens[b]:, :] = np.nan
        vc[b, :, lens[b]:, :] = np.nan
    f = ref.freq_cis(L, D)
    kc_r, vc_r = kc.copy(), vc.copy()
    out = ref.decode_attn(q, k, v, kc_r, vc_r, f, start_pos_per_seq=lens - 1)
    assert np.isfinite(out).all()
    for b in range(B):
        kb, vb = kc[b:b + 1].copy(), vc[b:b + 1].copy()
        ob = ref.decode_attn(q[b:b + 1], k[b:b + 1], v[b:b + 1], kb, vb, f, start_pos=int(lens[b] - 1))
        assert np.array_equal(ob[0], out[b])
        assert np.array_equal(kb.view(np.uint16), kc_r[b:b + 1].view(np.uint16))


def test_out_of_range_position_poisons_output_and_stores_nothing():
    B, H, D, L = 2, 1, 32, 8
    q, k, v, kc, vc = make(B, H, D, L)
    kc0 = kc.copy()
    out = ref.decode_attn(q, k, v, kc, vc, ref.freq_cis(L, D), start_pos_per_seq=np.array([3, 8]))
    assert np.isfinite(out[0]).all() and np.isnan(out[1]).all()
    assert np.array_equal(kc[1], kc0[1])


def test_position_above_the_promised_bound_is_treated_like_one_outside_the_cache():
    # a ragged batch comes with a bound for its positions (the HIP library plans its launch for it);
    # a sequence beyond that bound gets NaN output and no cache row, its neighbours are untouched by it
    B, H, D, L = 4, 2, 32, 16
    q, k, v, kc, vc = make(B, H, D, L, seed=5)
    kc0, vc0 = kc.copy(), vc.copy()
    pos = np.array([3, 7, 15, 6])
    f = ref.freq_cis(L, D)
    out = ref.decode_attn(q, k, v, kc, vc, f, start_pos_per_seq=pos, max_start_pos=6)
    assert np.isnan(out[1]).all() and np.isnan(out[2]).all()
    assert np.array_equal(kc[1:3], kc0[1:3]) and np.array_equal(vc[1:3], vc0[1:3])
    for b in (0, 3):  # identical to a run of that sequence alone
        kb, vb = kc0[b:b + 1].copy(), vc0[b:b + 1].copy()
        ob = ref.decode_attn(q[b:b + 1], k[b:b + 1], v[b:b + 1], kb, vb, f, start_pos=int(pos[b]))
        assert np.array_equal(ob[0], out[b]) and np.array_equal(kb[0], kc[b]) and np.array_equal(vb[0], vc[b])
    # no bound given (-1) and a bound equal to the maximum: every sequence is served
    for bound in (-1, 15):
        kc1, vc1 = kc0.copy(), vc0.copy()
        assert np.isfinite(ref.decode_attn(q, k, v, kc1, vc1, f, start_pos_per_seq=pos, max_start_pos=bound)).all()
    # the bound applies to ragged batches only: a uniform start_pos ignores it
    kc1, vc1 = kc0.copy(), vc0.copy()
    assert np.isfinite(ref.decode_attn(q, k, v, kc1, vc1, f, start_pos=9, max_start_pos=2)).all()


# ----------------------------------------------------------------------------- fp16 storage (D6 extension)

def test_half_conversions_match_numpy_for_every_half_and_random_floats():
    lib = ref.load()
    allh = np.arange(65536, dtype=np.uint16)
    want = allh.view(np.float16).astype(np.float32)
    got = np.array([lib.fl_ref_half_to_float(int(h)) for h in allh], np.float32)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.isnan(got[np.isnan(want)]).all()
    rng = np.random.default_rng(0)
    xs = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 20000).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001,
                  2.0 ** -14, 6.1e-5, 5.96e-8, np.inf, -np.inf], np.float32),
        # exact ties between adjacent halves
        (np.arange(1024, 2048, dtype=np.float32) + 0.5) / 1024.0,
    ])
    with np.errstate(over="ignore"):
        want_h = xs.astype(np.float16).view(np.uint16)
    got_h = np.array([lib.fl_ref_float_to_half(float(x)) for x in xs], np.uint16)
    assert np.array_equal(got_h, want_h)


def test_f16_cache_row_is_rne_of_fp32_rope():
    B, H, D, L, P = 1, 2, 64, 30, 29
    q, k, v, kc, vc = make(B, H, D, L, np.float16, seed=8)
    f = ref.freq_cis(L, D)
    ref.decode_attn(q, k, v, kc, vc, f, start_pos=P)
    k32 = k.astype(np.float32)
    k32c, v32c = np.zeros((B, H, L, D), np.float32), np.zeros((B, H, L, D), np.float32)
    ref.decode_attn(q.astype(np.float32), k32, v.astype(np.float32), k32c, v32c, f, start_pos=P)
    assert np.array_equal(kc[:, :, P].view(np.uint16), k32c[:, :, P].astype(np.float16).view(np.uint16))
    assert np.array_equal(vc[:, :, P], v.reshape(B, H, D))


# ----------------------------------------------------------------------------- prologue / epilogue ("next" rows)

def test_i32_prologue_equals_dequantised_float_inputs():
    B, H, D, L, P = 2, 4, 32, 12, 7
    rng = np.random.default_rng(4)
    qi, ki, vi = (rng.integers(-30000, 30000, (B, 1, H, D), dtype=np.int32) for _ in range(3))
    s_in = (rng.random(B).astype(np.float32) + 0.5) * np.float32(1e-3)
    wq, wk, wv = (rng.random(H * D).astype(np.float32) * np.float32(2e-2) for _ in range(3))
    _, _, _, kc, vc = make(B, H, D, L, seed=6)
    f = ref.freq_cis(L, D)
    deq = lambda a, w: (a.astype(np.float32) * s_in[:, None, None, None]) * w.reshape(1, 1, H, D)
    kc1, vc1, kc2, vc2 = kc.copy(), vc.copy(), kc.copy(), vc.copy()
    o1 = ref.decode_attn(qi, ki, vi, kc1, vc1, f, start_pos=P, inp_scale=s_in, wq_scale=wq, wk_scale=wk, wv_scale=wv)
    o2 = ref.decode_attn(deq(qi, wq), deq(ki, wk), deq(vi, wv), kc2, vc2, f, start_pos=P)
    assert np.array_equal(o1, o2) and np.array_equal(kc1, kc2) and np.array_equal(vc1, vc2)


def test_int8_epilogue_against_numpy():
    rng = np.random.default_rng(9)
    x = rng.standard_normal((6, 512)).astype(np.float32)
    x[2] *= 1e-3
    x[3, 7] = 40.0
    qv, sc = ref.attn_quantize(x)
    absmax = np.abs(x).max(1)
    assert np.array_equal(sc, (absmax / np.float32(127.0)).astype(np.float32))
    want = np.clip(np.rint((x * np.float32(127.0)) / absmax[:, None]), -128, 127).astype(np.int8)
    assert np.array_equal(qv, want)
    assert (np.abs(qv).max(1) == 127).all()  # the absmax element maps to +-127
    # ties round to even (cvt.rni): 0.5*absmax/127 -> 0, 1.5 -> 2, 2.5 -> 2
    y = np.array([[127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5]], np.float32)
    qy, _ = ref.attn_quantize(y)
    assert qy[0].tolist() == [127, 0, 2, 2, 0, -2, -2, 126]


# ----------------------------------------------------------------------------- committed golden vectors

def test_golden_fixture():
    """Expected values written by tests/golden/make_golden.py from an independent float64
    implementation (complex RoPE + numpy softmax); inputs come from the seeded generator."""
    g = np.load(os.path.join(HERE, "golden", "decode_attn_golden.npz"))
    for name in ("tiny_f32", "cfg1_f32", "cfg1_f16"):
        B, H, D, L, P, seed = (int(x) for x in g[f"{name}_shape"])
        dt = np.float16 if name.endswith("f16") else np.float32
        q, k, v, kc, vc = make(B, H, D, L, dt, seed=seed)
        assert np.array_equal(q.reshape(-1)[:8].astype(np.float32), g[f"{name}_q_head"])  # generator unchanged
        out = ref.decode_attn(q, k, v, kc, vc, ref.freq_cis(L, D), start_pos=P)
        tol_out = 2e-5
        tol_k = 2e-3 if dt == np.float16 else 4e-7
        assert np.abs(out - g[f"{name}_out"]).max() < tol_out
        assert np.abs(kc[:, :, P].astype(np.float64) - g[f"{name}_k_row"]).max() <= tol_k


# ----------------------------------------------------------------------------- prompt phase (seq_len > 1)

def make_prompt(B, H, D, L, S, dt=np.float32, seed=13):
    q = synth.normal((B, S, H, D), dt, synth.TENSOR_Q, seed)
    k = synth.normal((B, S, H, D), dt, synth.TENSOR_K_NEW, seed)
    v = synth.normal((B, S, H, D), dt, synth.TENSOR_V_NEW, seed)
    kc = synth.normal((B, H, L, D), dt, synth.TENSOR_K_CACHE, seed)
    vc = synth.normal((B, H, L, D), dt, synth.TENSOR_V_CACHE, seed)
    return q, k, v, kc, vc


def causal(L, fill=-1e5):
    return np.where(np.arange(L)[None, :] > np.arange(L)[:, None], fill, 0.0).astype(np.float32)


@pytest.mark.parametrize("dt", [np.float32, np.float16])
def test_prefill_with_one_token_is_the_decode_step_bitwise(dt):
    B, H, D, L, P = 2, 3, 64, 40, 17
    q, k, v, kc, vc = make(B, H, D, L, dt)
    f = ref.freq_cis(L, D)
    m = (np.random.default_rng(0).standard_normal((L, L))).astype(np.float32)
    k1, v1, k2, v2 = kc.copy(), vc.copy(), kc.copy(), vc.copy()
    o1 = ref.decode_attn(q, k, v, k1, v1, f, start_pos=P, attn_mask=m)
    o2 = ref.prefill_attn(q, k, v, k2, v2, f, start_pos=P, attn_mask=m)
    assert np.array_equal(o1.ravel(), o2.ravel())
    assert np.array_equal(k1.view(np.uint8), k2.view(np.uint8)) and np.array_equal(v1.view(np.uint8), v2.view(np.uint8))


def test_prefill_equals_token_by_token_decode_under_a_causal_mask():
    B, H, D, L, S, P = 2, 2, 32, 48, 20, 9
    q, k, v, kc, vc = make_prompt(B, H, D, L, S)
    f = ref.freq_cis(L, D)
    m = causal(L)
    k1, v1 = kc.copy(), vc.copy()
    full = ref.prefill_attn(q, k, v, k1, v1, f, start_pos=P, attn_mask=m, acc_double=True)
    k2, v2 = kc.copy(), vc.copy()
    for s in range(S):
        o = ref.decode_attn(np.ascontiguousarray(q[:, s:s + 1]), np.ascontiguousarray(k[:, s:s + 1]),
                            np.ascontiguousarray(v[:, s:s + 1]), k2, v2, f, start_pos=P + s, attn_mask=m, acc_double=True)
        assert np.abs(o.reshape(B, H, D) - full[:, :, s]).max() < 1e-6
    assert np.array_equal(k1, k2) and np.array_equal(v1, v2)


def test_prefill_against_torch_causal_sdpa_and_transposed_layouts():
    torch = pytest.importorskip("torch")
    B, H, D, L, S = 2, 3, 64, 64, 37
    q, k, v, kc, vc = make_prompt(B, H, D, L, S)
    f = ref.freq_cis(L, D)
    out = ref.prefill_attn(q, k, v, kc, vc, f, start_pos=0, attn_mask=causal(L), acc_double=True)
    assert out.shape == (B, H, S, D)
    # appended rows: [B,S,H,D] inputs land transposed at cache[b,h,s,:]; V unchanged, K rotated by row s
    assert np.array_equal(vc[:, :, :S], v.transpose(0, 2, 1, 3))
    cos, sin = f[:S, 0::2][None, :, None, :], f[:S, 1::2][None, :, None, :]
    def rot(x):
        r = np.empty_like(x)
        r[..., 0::2] = x[..., 0::2] * cos - x[..., 1::2] * sin
        r[..., 1::2] = x[..., 1::2] * cos + x[..., 0::2] * sin
        return r
    assert np.allclose(kc[:, :, :S], rot(k).transpose(0, 2, 1, 3), atol=1e-6)
    tq = torch.from_numpy(rot(q).transpose(0, 2, 1, 3).copy()).double()
    tk = torch.from_numpy(kc[:, :, :S].copy()).double()
    tv = torch.from_numpy(vc[:, :, :S].copy()).double()
    want = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, is_causal=True).numpy()
    assert np.abs(out - want).max() < 3e-6


def test_prefill_chunked_prompt_attends_to_earlier_cache_rows():
    # start_pos > 0: the keys are the cache rows [0, start_pos + S); first P rows come from the cache
    B, H, D, L, S, P = 1, 1, 32, 32, 6, 5
    q, k, v, kc, vc = make_prompt(B, H, D, L, S)
    vc[:] = 0
    for j in range(P):
        vc[0, 0, j, j] = 1.0
    v[:] = 0
    for s in range(S):
        v[0, s, 0, P + s] = 1.0
    out = ref.prefill_attn(q, k, v, kc, vc, ref.freq_cis(L, D), start_pos=P, attn_mask=causal(L))
    for s in range(S):
        p = out[0, 0, s]
        assert abs(p[:P + s + 1].sum() - 1.0) < 1e-6 and (p[:P + s + 1] > 0).all() and (p[P + s + 1:] == 0).all()


def test_quantize_transpose_against_numpy():
    rng = np.random.default_rng(5)
    B, H, S, D = 2, 3, 5, 16
    x = rng.standard_normal((B, H, S, D)).astype(np.float32)
    qv, sc = ref.attn_quantize_transpose(x)
    xt = x.transpose(0, 2, 1, 3).reshape(B, S, H * D)
    absmax = np.abs(xt).max(-1)
    assert np.array_equal(sc, (absmax / np.float32(127.0)).astype(np.float32))
    assert np.array_equal(qv, np.clip(np.rint((xt * np.float32(127.0)) / absmax[..., None]), -128, 127).astype(np.int8))
    # S == 1 is the decode-step quantiser
    q1, s1 = ref.attn_quantize_transpose(x[:, :, :1])
    q0, s0 = ref.attn_quantize(x[:, :, 0].reshape(B, H * D))
    assert np.array_equal(q1.reshape(B, H * D), q0) and np.array_equal(s1.ravel(), s0)
