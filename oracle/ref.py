"""ctypes loader of the CPU oracle (oracle/libfl_ref.so).  TEST INFRASTRUCTURE: imported only
by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg of bench.py."""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libfl_ref.so")
_lib = None


def load() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: run `make -C oracle`")
        lib = C.CDLL(LIB_PATH)
        lib.fl_ref_decode_attn.argtypes = [
            C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
            C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int64, C.c_int, C.c_void_p, C.c_int, C.c_float,
            C.c_void_p, C.c_int, C.c_int]
        lib.fl_ref_decode_attn.restype = C.c_int
        lib.fl_ref_decode_attn_i32.argtypes = [
            C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
            C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p,
            C.c_int64, C.c_int, C.c_void_p, C.c_int, C.c_float, C.c_void_p, C.c_int, C.c_int]
        lib.fl_ref_decode_attn_i32.restype = C.c_int
        lib.fl_ref_freq_cis.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_double]
        lib.fl_ref_freq_cis.restype = C.c_int
        lib.fl_ref_attn_quantize.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
        lib.fl_ref_attn_quantize.restype = C.c_int
        lib.fl_ref_prefill_attn.argtypes = [
            C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
            C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int64,
            C.c_int, C.c_float, C.c_void_p, C.c_int, C.c_int]
        lib.fl_ref_prefill_attn.restype = C.c_int
        lib.fl_ref_attn_quantize_transpose.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p,
                                                       C.c_void_p]
        lib.fl_ref_attn_quantize_transpose.restype = C.c_int
        lib.fl_ref_half_to_float.argtypes = [C.c_uint16]
        lib.fl_ref_half_to_float.restype = C.c_float
        lib.fl_ref_float_to_half.argtypes = [C.c_float]
        lib.fl_ref_float_to_half.restype = C.c_uint16
        lib.fl_ref_omp_max_threads.argtypes = []
        lib.fl_ref_omp_max_threads.restype = C.c_int
        _lib = lib
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data


def freq_cis(rows: int, D: int, base: float = 10000.0) -> np.ndarray:
    t = np.empty((rows, D), dtype=np.float32)
    rc = load().fl_ref_freq_cis(t.ctypes.data, rows, D, base)
    if rc != 0:
        raise ValueError(f"fl_ref_freq_cis -> {rc}")
    return t


def decode_attn(q, k_new, v_new, k_cache, v_cache, freq, start_pos=0, rope_row=-1, attn_mask=None,
                mask_ld=None, start_pos_per_seq=None, max_start_pos=-1, scale=None, acc_double=False, threads=1,
                inp_scale=None, wq_scale=None, wk_scale=None, wv_scale=None, dtype=None):
    """Runs the oracle IN PLACE on k_cache / v_cache (numpy, C-contiguous) and returns out [B, H*D].

    q/k_new/v_new: [B,1,H,D] (or [B,H,D]) float32/float16, or int32 with the four scale arrays.
    k_cache/v_cache: [B,H,L,D] float32 or float16.  With start_pos_per_seq, max_start_pos >= 0 is the
    bound promised for its entries: a sequence beyond it gets NaN output and no cache row."""
    B, H, L, D = k_cache.shape
    st = np.dtype(k_cache.dtype)
    code = {np.dtype(np.float32): 0, np.dtype(np.float16): 1}[st]
    for a in (q, k_new, v_new, k_cache, v_cache, freq):
        assert a.flags.c_contiguous
    assert v_cache.dtype == st and v_cache.shape == k_cache.shape
    assert q.size == B * H * D and k_new.size == q.size and v_new.size == q.size
    assert freq.dtype == np.float32 and freq.shape[1] == D
    if scale is None:
        scale = float(np.float32(1.0) / np.sqrt(np.float32(D)))
    if mask_ld is None:
        mask_ld = L
    if attn_mask is not None:
        assert attn_mask.dtype == np.float32 and attn_mask.flags.c_contiguous
    if start_pos_per_seq is not None:
        start_pos_per_seq = np.ascontiguousarray(start_pos_per_seq, dtype=np.int32)
        assert start_pos_per_seq.size == B
    out = np.empty((B, H * D), dtype=np.float32)
    lib = load()
    if inp_scale is not None:
        for a in (q, k_new, v_new):
            assert a.dtype == np.int32
        rc = lib.fl_ref_decode_attn_i32(code, B, H, D, L, _p(q), _p(k_new), _p(v_new), _p(inp_scale),
                                        _p(wq_scale), _p(wk_scale), _p(wv_scale), _p(k_cache), _p(v_cache),
                                        _p(freq), rope_row, _p(attn_mask), mask_ld, start_pos,
                                        _p(start_pos_per_seq), max_start_pos, scale, _p(out), int(acc_double),
                                        threads)
    else:
        for a in (q, k_new, v_new):
            assert a.dtype == st
        rc = lib.fl_ref_decode_attn(code, B, H, D, L, _p(q), _p(k_new), _p(v_new), _p(k_cache), _p(v_cache),
                                    _p(freq), rope_row, _p(attn_mask), mask_ld, start_pos,
                                    _p(start_pos_per_seq), max_start_pos, scale, _p(out), int(acc_double), threads)
    if rc != 0:
        raise ValueError(f"fl_ref_decode_attn -> {rc}")
    return out


def attn_quantize(attn: np.ndarray):
    """[B, H*D] float32 -> (int8 [B, H*D], scale [B])."""
    attn = np.ascontiguousarray(attn, dtype=np.float32)
    B, HD = attn.shape
    q = np.empty((B, HD), dtype=np.int8)
    s = np.empty(B, dtype=np.float32)
    rc = load().fl_ref_attn_quantize(B, HD, attn.ctypes.data, q.ctypes.data, s.ctypes.data)
    if rc != 0:
        raise ValueError(f"fl_ref_attn_quantize -> {rc}")
    return q, s


def prefill_attn(q, k_new, v_new, k_cache, v_cache, freq, start_pos=0, rope_row=-1, attn_mask=None, mask_ld=None,
                 scale=None, acc_double=False, threads=1, inp_scale=None, wq_scale=None, wk_scale=None,
                 wv_scale=None):
    """Prompt phase, IN PLACE on the caches.  q/k_new/v_new: [B,S,H,D]; returns out [B,H,S,D] float32."""
    B, H, L, D = k_cache.shape
    S = q.shape[1]
    assert q.shape == (B, S, H, D) and k_new.shape == q.shape and v_new.shape == q.shape
    st = np.dtype(k_cache.dtype)
    code = {np.dtype(np.float32): 0, np.dtype(np.float16): 1}[st]
    for a in (q, k_new, v_new, k_cache, v_cache, freq):
        assert a.flags.c_contiguous
    if inp_scale is None:
        assert q.dtype == st
    else:
        assert q.dtype == np.int32 and inp_scale.size == B * S
    if scale is None:
        scale = float(np.float32(1.0) / np.sqrt(np.float32(D)))
    if mask_ld is None:
        mask_ld = L
    out = np.empty((B, H, S, D), dtype=np.float32)
    rc = load().fl_ref_prefill_attn(code, B, H, D, L, S, _p(q), _p(k_new), _p(v_new), _p(inp_scale), _p(wq_scale),
                                    _p(wk_scale), _p(wv_scale), _p(k_cache), _p(v_cache), _p(freq), rope_row,
                                    _p(attn_mask), mask_ld, start_pos, scale, _p(out), int(acc_double), threads)
    if rc != 0:
        raise ValueError(f"fl_ref_prefill_attn -> {rc}")
    return out


def attn_quantize_transpose(attn: np.ndarray):
    """[B,H,S,D] float32 -> (int8 [B,S,H*D], scale [B,S])."""
    attn = np.ascontiguousarray(attn, dtype=np.float32)
    B, H, S, D = attn.shape
    q = np.empty((B, S, H * D), dtype=np.int8)
    s = np.empty((B, S), dtype=np.float32)
    rc = load().fl_ref_attn_quantize_transpose(B, H, S, D, attn.ctypes.data, q.ctypes.data, s.ctypes.data)
    if rc != 0:
        raise ValueError(f"fl_ref_attn_quantize_transpose -> {rc}")
    return q, s
