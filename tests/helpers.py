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
                 mask=None, rope_row=-1, pad=None, scale_rows=(), rope_base=10000.0, table_rows=None,
                 max_start_pos=None):
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
        self.max_start_pos = max_start_pos  # ragged cases: the bound handed to the library (None: the true maximum)
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

    def bound(self):
        if self.pos is None:
            return -1
        return min(int(self.pos.max()), self.L - 1) if self.max_start_pos is None else self.max_start_pos

    def run_oracle(self, acc_double=False, threads=8):
        kc, vc = self.k_cache.copy(), self.v_cache.copy()
        out = ref.decode_attn(self.q, self.k_new, self.v_new, kc, vc, self.freq, start_pos=self.start_pos,
                              rope_row=self.rope_row, attn_mask=self.mask, start_pos_per_seq=self.pos,
                              max_start_pos=self.bound(), acc_double=acc_double, threads=threads)
        return out, kc, vc

    def run_gpu(self, device, nsplit=0, entry="forward", op=None):
        """entry: "forward" (fl_decode_attn_forward, two launches when the context is split), "ready"
        (the same after fl_decode_attn_workspace_init: one launch) or "noalloc"
        (fl_decode_attn_forward_noalloc).  op: reuse an operator (and its workspace) of the same shape."""
        import torch
        from fasterllama_amd import capi
        from fasterllama_amd.decode_attn import DecodeAttention
        tdt = torch.float16 if self.dtype == "f16" else torch.float32
        if op is None:
            op = DecodeAttention(self.B, self.H, self.D, self.L, tdt, nsplit=nsplit, device=device)
            if entry == "ready":
                op.init_workspace()
        d = lambda a: None if a is None else torch.from_numpy(a).to(device)
        q, k, v = d(self.q), d(self.k_new), d(self.v_new)
        kc, vc = d(self.k_cache), d(self.v_cache)
        f, m, pos = d(self.freq), d(self.mask), d(self.pos)
        out = torch.full((self.B, self.H * self.D), 7.0, dtype=torch.float32, device=device)
        io = op.make_io(q, k, v, kc, vc, f, out, start_pos=self.start_pos, rope_row=self.rope_row,
                        attn_mask=m, start_pos_per_seq=pos, max_start_pos=self.bound())
        if entry == "noalloc":
            io.workspace, io.workspace_bytes = None, 0
            capi.check(op.launch_noalloc(io))
        else:
            capi.check(op.launch(io))
        torch.cuda.synchronize(device)
        return out.cpu().numpy(), kc.cpu().numpy(), vc.cpu().numpy(), op


def bits(a: np.ndarray) -> np.ndarray:
    """Bit pattern view for exact comparisons that also treat NaNs as equal to themselves."""
    return a.view(np.uint16 if a.dtype == np.float16 else np.uint32)


def assert_cache_bit_exact(got, want, what=""):
    g, w = bits(np.ascontiguousarray(got)), bits(np.ascontiguousarray(want))
    bad = np.flatnonzero(g.ravel() != w.ravel())
    assert bad.size == 0, f"{what}: {bad.size} cache words differ, first at flat index {bad[:5]}"


F32_REL_TOL = 1e-5      # the bar for FP32 storage: within 1e-5 relative
F32_ROW_FLOOR = 0.1     # ... of max(|ref|, 0.1 * largest |ref| of the same (b, h[, s]) output row)
F16_ABS_TOL = 2e-3      # the bar for fp16 storage: within 2e-3 absolute
F32_VS_FLOAT_REF = 1.0   # see assert_out_close


def _f32_excess(got, want, head_dim):
    """max over elements of |err| / (1e-5 * max(|ref|, 0.1 * rowmax)), plus the figures that are printed."""
    e, w = np.abs(got - want).reshape(-1, head_dim), np.abs(want).reshape(-1, head_dim)
    rowmax = w.max(axis=1, keepdims=True)
    tol = F32_REL_TOL * np.maximum(w, F32_ROW_FLOOR * rowmax)
    big = (w >= F32_ROW_FLOOR * rowmax) & (w > 0)
    rel = (e[big] / w[big]).max() if big.any() else 0.0
    return (e / np.maximum(tol, 1e-300)).max(), rel, (e / np.maximum(rowmax, 1e-300)).max()


def assert_out_close(got, want64, dtype, what="", head_dim=None, float_ref=None):
    """Attention output against the double-precision arbiter.

    FP32 storage: every element within 1e-5 RELATIVE, |err| <= 1e-5 * max(|ref|, 0.1 * rowmax), where
    rowmax is the largest |ref| of the element's own output row (the D values of one (b, h) — or
    (b, h, s) — pair; the floor keeps elements that cancel to ~0 from demanding an unbounded relative
    accuracy).  Equivalently: relative error <= 1e-5 for every element that is at least a tenth of its
    row's maximum, and 1e-6 of the row maximum for the smaller ones.  head_dim gives the row length for
    [B, H*D] outputs; [B,H,S,D] outputs use their last axis.
    The bound sits at about ten float ulps of the row maximum, which plain sequential FP32 summation
    — the reference's own arithmetic, restated by the float oracle — does not always keep (short contexts
    with outputs of a few units).  float_ref, a callable returning the float oracle's output for the same
    inputs, covers that: where the kernel misses the bound AND the float oracle misses it too, the kernel's
    error (in units of the bound) must stay within F32_VS_FLOAT_REF times that of the float oracle, so it is
    never further from the arbiter than the reference arithmetic is on the same inputs.  Where the float
    oracle keeps the bound, so must the kernel.
    fp16 storage: 2e-3 absolute."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want64, np.float64)
    assert got.shape == want.shape, f"{what}: shapes {got.shape} vs {want.shape}"
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    err = np.abs(got - want)
    if not err.size:
        return 0.0
    if dtype == "f32":
        if head_dim is None:
            assert got.ndim == 4, f"{what}: head_dim is needed to find the rows of a {got.ndim}-d output"
            head_dim = got.shape[-1]
        worst, rel, vs_rowmax = _f32_excess(got, want, head_dim)
        print(f"{what}: f32 err/tol {worst:.3f}, max rel err (|ref| >= {F32_ROW_FLOOR} rowmax) {rel:.3e}, "
              f"max |err|/rowmax {vs_rowmax:.3e}, max abs err {err.max():.3e}")
        if worst > 1.0 and float_ref is not None:
            ref_worst, ref_rel, _ = _f32_excess(np.asarray(float_ref(), np.float64), want, head_dim)
            print(f"{what}: sequential-FP32 oracle on the same inputs: err/tol {ref_worst:.3f}, max rel err {ref_rel:.3e}")
            assert ref_worst > 1.0 and worst <= F32_VS_FLOAT_REF * ref_worst, \
                f"{what}: err/tol {worst:.3f} (kernel) vs {ref_worst:.3f} (float oracle)"
            return err.max()
    else:
        worst = (err / F16_ABS_TOL).max()
    assert worst <= 1.0, f"{what}: max err/tol = {worst:.3f}, max abs err {err.max():.3e}"
    return err.max()
