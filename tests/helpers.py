"""Shared case builder for the parity tests: seeded inputs -> oracle (CPU) and HIP path (GPU)."""
from __future__ import annotations

import numpy as np

from fasterllama_amd import synth
from oracle import ref

NP_DT = {"f32": np.float32, "f16": np.float16}


class Case:
    """Inputs of one decode step.  K/V caches hold `L` rows per (b,h); rows >= ctx of each sequence
    are filled with `pad` (NaN by default in ragged cases) to prove they are never read."""

    def __init__(self, B, H, D, L, dtype="f16", start_pos=None, lens=None, seed=synth.DEFAULT_SEED,
                 mask=None, rope_row=-1, pad=None, scale_rows=(), rope_base=10000.0, table_rows=None):
        self.B, self.H, self.D, self.L, self.dtype = B, H, D, L, dtype
        dt = NP_DT[dtype]
        self.q = synth.normal((B, 1, H, D), dt, synth.TENSOR_Q, seed)
        self.k_new = synth.normal((B, 1, H, D), dt, synth.TENSOR_K_NEW, seed)
        self.v_new = synth.normal((B, 1, H, D), dt, synth.TENSOR_V_NEW, seed)
        self.k_cache = synth.normal((B, H, L, D), dt, synth.TENSOR_K_CACHE, seed)
        self.v_cache = synth.normal((B, H, L, D), dt, synth.TENSOR_V_CACHE, seed)
        for r in scale_rows:  # a few key rows scaled by 8: stresses the max subtraction
            self.k_cache[:, :, r, :] *= dt(8)
        self.freq = synth.freq_cis_table(table_rows or L, D, rope_base)
        self.rope_row = rope_row
        self.mask = mask
        if lens is not None:
            self.pos = np.asarray(lens, dtype=np.int32) - 1  # new token lands at row len-1
            self.start_pos = 0
        else:
            self.pos = None
            self.start_pos = L - 1 if start_pos is None else start_pos
        if pad is not None:
            for b in range(B):
                p = self.pos[b] if self.pos is not None else self.start_pos
                self.k_cache[b, :, max(p, 0):, :] = pad   # row p itself gets overwritten by the step
                self.v_cache[b, :, max(p, 0):, :] = pad

    def positions(self):
        return self.pos if self.pos is not None else np.full(self.B, self.start_pos, np.int32)

    def run_oracle(self, acc_double=False, threads=8):
        kc, vc = self.k_cache.copy(), self.v_cache.copy()
        out = ref.decode_attn(self.q, self.k_new, self.v_new, kc, vc, self.freq, start_pos=self.start_pos,
                              rope_row=self.rope_row, attn_mask=self.mask, start_pos_per_seq=self.pos,
                              acc_double=acc_double, threads=threads)
        return out, kc, vc

    def run_gpu(self, device, nsplit=0, want_passes=3):
        import torch
        from fasterllama_amd.decode_attn import DecodeAttention
        tdt = torch.float16 if self.dtype == "f16" else torch.float32
        op = DecodeAttention(self.B, self.H, self.D, self.L, tdt, nsplit=nsplit, device=device)
        d = lambda a: None if a is None else torch.from_numpy(a).to(device)
        q, k, v = d(self.q), d(self.k_new), d(self.v_new)
        kc, vc = d(self.k_cache), d(self.v_cache)
        f, m, pos = d(self.freq), d(self.mask), d(self.pos)
        out = op.forward(q, k, v, kc, vc, f, start_pos=self.start_pos, rope_row=self.rope_row,
                         attn_mask=m, start_pos_per_seq=pos,
                         max_start_pos=min(int(self.pos.max()), self.L - 1) if self.pos is not None else -1)
        torch.cuda.synchronize(device)
        return out.cpu().numpy(), kc.cpu().numpy(), vc.cpu().numpy(), op


def bits(a: np.ndarray) -> np.ndarray:
    """Bit pattern view for exact comparisons that also treat NaNs as equal to themselves."""
    return a.view(np.uint16 if a.dtype == np.float16 else np.uint32)


def assert_cache_bit_exact(got, want, what=""):
    g, w = bits(np.ascontiguousarray(got)), bits(np.ascontiguousarray(want))
    bad = np.flatnonzero(g.ravel() != w.ravel())
    assert bad.size == 0, f"{what}: {bad.size} cache words differ, first at flat index {bad[:5]}"


def assert_out_close(got, want64, dtype, what=""):
    """FP32 storage: 1e-5 relative (floored at 1e-5 of the row scale so that outputs that cancel to
    ~0 are not held to an unbounded relative bound).  fp16 storage: 2e-3 absolute."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want64, np.float64)
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    err = np.abs(got - want)
    if dtype == "f32":
        floor = np.abs(want).max() if want.size else 1.0
        tol = 1e-5 * np.maximum(np.abs(want), floor)
    else:
        tol = np.full_like(want, 2e-3)
    worst = (err / tol).max() if err.size else 0.0
    assert worst <= 1.0, f"{what}: max err/tol = {worst:.3f}, max abs err {err.max():.3e}"
    return err.max()
