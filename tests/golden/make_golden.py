"""Writes tests/golden/decode_attn_golden.npz: expected outputs of the decode-attention step for
seeded inputs, computed by an independent float64 implementation (complex-number RoPE, dense numpy
softmax).  Neither the oracle nor the HIP library is involved, and no reference code runs (the
reference is CUDA-only and holds no vectors for this path).

    python tests/golden/make_golden.py
"""
import math
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from fasterllama_amd import synth  # noqa: E402  (seeded input generator only)


def step64(q, k_new, v_new, k_cache, v_cache, P, store, base=10000.0):
    B, H, L, D = k_cache.shape
    w = base ** (-2.0 * np.arange(D // 2) / D)
    rot = np.exp(1j * P * w)
    out = np.empty((B, H * D))
    k_rows = np.empty((B, H, D))
    for b in range(B):
        for h in range(H):
            x = q[b, 0, h].astype(np.float64); y = k_new[b, 0, h].astype(np.float64)
            qz = (x[0::2] + 1j * x[1::2]) * rot
            kz = (y[0::2] + 1j * y[1::2]) * rot
            qr = np.empty(D); qr[0::2] = qz.real; qr[1::2] = qz.imag
            kr = np.empty(D); kr[0::2] = kz.real; kr[1::2] = kz.imag
            kr = store(kr)
            K = np.concatenate([k_cache[b, h, :P].astype(np.float64), kr[None]], 0)
            V = np.concatenate([v_cache[b, h, :P].astype(np.float64), v_new[b, 0, h][None].astype(np.float64)], 0)
            s = K @ qr / math.sqrt(D)
            e = np.exp(s - s.max())
            out[b, h * D:(h + 1) * D] = (e / e.sum()) @ V
            k_rows[b, h] = kr
    return out, k_rows


def main():
    cases = {"tiny_f32": (1, 2, 8, 4, 3, 42, np.float32), "cfg1_f32": (1, 4, 64, 128, 127, 1234, np.float32),
             "cfg1_f16": (1, 4, 64, 128, 127, 1234, np.float16)}
    blob = {}
    for name, (B, H, D, L, P, seed, dt) in cases.items():
        q = synth.normal((B, 1, H, D), dt, synth.TENSOR_Q, seed)
        k = synth.normal((B, 1, H, D), dt, synth.TENSOR_K_NEW, seed)
        v = synth.normal((B, 1, H, D), dt, synth.TENSOR_V_NEW, seed)
        kc = synth.normal((B, H, L, D), dt, synth.TENSOR_K_CACHE, seed)
        vc = synth.normal((B, H, L, D), dt, synth.TENSOR_V_CACHE, seed)
        store = (lambda x: x.astype(np.float32).astype(np.float16).astype(np.float64)) if dt == np.float16 \
            else (lambda x: x.astype(np.float32).astype(np.float64))
        out, k_rows = step64(q, k, v, kc, vc, P, store)
        blob[f"{name}_shape"] = np.array([B, H, D, L, P, seed], np.int64)
        blob[f"{name}_q_head"] = q.reshape(-1)[:8].astype(np.float32)
        blob[f"{name}_out"] = out
        blob[f"{name}_k_row"] = k_rows
    np.savez(os.path.join(HERE, "decode_attn_golden.npz"), **blob)
    print("wrote", os.path.join(HERE, "decode_attn_golden.npz"))


if __name__ == "__main__":
    main()
