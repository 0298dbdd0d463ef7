"""ctypes binding of include/fl_decode_attn.h.

The shared library is the product; this module only marshals pointers.  It raises at load time
when the HIP library has not been built — there is no CPU fallback.
"""
from __future__ import annotations

import ctypes as C
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "lib", "libfl_decode_attn.so")

FL_ATTN_F32 = 0
FL_ATTN_F16 = 1
FL_ATTN_ROPE_AT_POSITION = -1
FL_ATTN_FLAG_FAST_PROMPT_QK = 1

FL_ATTN_OK = 0
FL_ATTN_ERR_NULL_POINTER = -1
FL_ATTN_ERR_HEAD_DIM = -2
FL_ATTN_ERR_SHAPE = -3
FL_ATTN_ERR_POSITION = -4
FL_ATTN_ERR_WORKSPACE = -5
FL_ATTN_ERR_DTYPE = -6
FL_ATTN_ERR_HIP = -7
FL_ATTN_ERR_ALIGNMENT = -8
FL_ATTN_ERR_ARGUMENT = -9
FL_ATTN_ERR_SCRATCH_LIMIT = -10
FL_ATTN_ERR_STRUCT_SIZE = -11
FL_ATTN_IO_WORKSPACE_READY = 1
FL_ATTN_NOALLOC_SCRATCH_BYTES = 16 << 20

# every symbol include/fl_decode_attn.h declares
EXPORTED_SYMBOLS = (
    "fl_decode_attn_workspace_bytes",
    "fl_decode_attn_plan",
    "fl_decode_attn_forward",
    "fl_decode_attn_forward_passes",
    "fl_decode_attn_forward_noalloc",
    "fl_decode_attn_workspace_init",
    "fl_prefill_attn_workspace_bytes",
    "fl_prefill_attn_forward",
    "fl_prefill_attn_forward_passes",
    "fl_prefill_mask_classes_bytes",
    "fl_prefill_mask_classify",
    "fl_rope_table",
    "fl_kv_cache_bytes",
    "fl_attn_strerror",
    "fl_attn_last_hip_error",
    "fl_attn_version",
)


class AttnDesc(C.Structure):
    """fl_attn_desc; AttnDesc(B, H, D, L, dtype, nsplit, softmax_scale, flags) fills struct_size itself."""
    _fields_ = [
        ("struct_size", C.c_uint32),
        ("batch_size", C.c_int32),
        ("head_num", C.c_int32),
        ("size_per_head", C.c_int32),
        ("total_len", C.c_int32),
        ("dtype", C.c_int32),
        ("nsplit", C.c_int32),
        ("softmax_scale", C.c_float),
        ("flags", C.c_int32),
    ]

    def __init__(self, *args, **kw):
        super().__init__(C.sizeof(AttnDesc), *args, **kw)


class AttnIO(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32),
        ("q", C.c_void_p),
        ("k_new", C.c_void_p),
        ("v_new", C.c_void_p),
        ("k_cache", C.c_void_p),
        ("v_cache", C.c_void_p),
        ("freq_cis", C.c_void_p),
        ("attn_mask", C.c_void_p),
        ("start_pos_per_seq", C.c_void_p),
        ("out", C.c_void_p),
        ("workspace", C.c_void_p),
        ("workspace_bytes", C.c_size_t),
        ("mask_ld", C.c_int64),
        ("start_pos", C.c_int32),
        ("rope_row", C.c_int32),
        ("max_start_pos", C.c_int32),
        ("flags", C.c_int32),
        ("qkv_inp_scale", C.c_void_p),
        ("q_weight_scale", C.c_void_p),
        ("k_weight_scale", C.c_void_p),
        ("v_weight_scale", C.c_void_p),
        ("out_int8", C.c_void_p),
        ("out_scale", C.c_void_p),
        ("mask_tile_classes", C.c_void_p),
    ]

    def __init__(self, **kw):
        super().__init__(**kw)
        self.struct_size = C.sizeof(AttnIO)


class AttnPlan(C.Structure):
    _fields_ = [
        ("nsplit", C.c_int32),
        ("chunk_rows", C.c_int32),
        ("threads", C.c_int32),
        ("two_pass", C.c_int32),
    ]


class FlAttnError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"fl_decode_attn status {status}: {message}")
        self.status = status


_lib = None


def load() -> C.CDLL:
    """Loads libfl_decode_attn.so; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m fasterllama_amd.build hip` "
            "(there is no fallback path)")
    lib = C.CDLL(LIB_PATH)
    lib.fl_decode_attn_workspace_bytes.argtypes = [C.POINTER(AttnDesc), C.POINTER(C.c_size_t)]
    lib.fl_decode_attn_workspace_bytes.restype = C.c_int
    lib.fl_kv_cache_bytes.argtypes = [C.POINTER(AttnDesc), C.POINTER(C.c_size_t)]
    lib.fl_kv_cache_bytes.restype = C.c_int
    lib.fl_decode_attn_plan.argtypes = [C.POINTER(AttnDesc), C.c_int32, C.c_int32, C.POINTER(AttnPlan)]
    lib.fl_decode_attn_plan.restype = C.c_int
    lib.fl_decode_attn_forward.argtypes = [C.POINTER(AttnDesc), C.POINTER(AttnIO), C.c_void_p]
    lib.fl_decode_attn_forward.restype = C.c_int
    lib.fl_decode_attn_forward_passes.argtypes = [C.POINTER(AttnDesc), C.POINTER(AttnIO), C.c_void_p, C.c_int]
    lib.fl_decode_attn_forward_passes.restype = C.c_int
    lib.fl_decode_attn_forward_noalloc.argtypes = [C.POINTER(AttnDesc), C.POINTER(AttnIO), C.c_void_p]
    lib.fl_decode_attn_forward_noalloc.restype = C.c_int
    lib.fl_decode_attn_workspace_init.argtypes = [C.POINTER(AttnDesc), C.c_void_p, C.c_size_t, C.c_void_p]
    lib.fl_decode_attn_workspace_init.restype = C.c_int
    lib.fl_prefill_attn_workspace_bytes.argtypes = [C.POINTER(AttnDesc), C.c_int32, C.POINTER(C.c_size_t)]
    lib.fl_prefill_attn_workspace_bytes.restype = C.c_int
    lib.fl_prefill_attn_forward.argtypes = [C.POINTER(AttnDesc), C.POINTER(AttnIO), C.c_int32, C.c_void_p]
    lib.fl_prefill_attn_forward.restype = C.c_int
    lib.fl_prefill_attn_forward_passes.argtypes = [C.POINTER(AttnDesc), C.POINTER(AttnIO), C.c_int32, C.c_void_p, C.c_int]
    lib.fl_prefill_attn_forward_passes.restype = C.c_int
    lib.fl_prefill_mask_classes_bytes.argtypes = [C.POINTER(AttnDesc), C.POINTER(C.c_size_t)]
    lib.fl_prefill_mask_classes_bytes.restype = C.c_int
    lib.fl_prefill_mask_classify.argtypes = [C.POINTER(AttnDesc), C.c_void_p, C.c_int64, C.c_void_p, C.c_size_t, C.c_void_p]
    lib.fl_prefill_mask_classify.restype = C.c_int
    lib.fl_rope_table.argtypes = [C.c_void_p, C.c_int32, C.c_int32, C.c_float, C.c_void_p]
    lib.fl_rope_table.restype = C.c_int
    lib.fl_attn_strerror.argtypes = [C.c_int]
    lib.fl_attn_strerror.restype = C.c_char_p
    lib.fl_attn_last_hip_error.argtypes = []
    lib.fl_attn_last_hip_error.restype = C.c_int
    lib.fl_attn_version.argtypes = []
    lib.fl_attn_version.restype = C.c_int
    _lib = lib
    return lib


def strerror(status: int) -> str:
    return load().fl_attn_strerror(status).decode()


def check(status: int) -> None:
    if status != FL_ATTN_OK:
        raise FlAttnError(status, strerror(status))
