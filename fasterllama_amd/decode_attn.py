"""Thin host-side wrapper: torch owns device memory and the stream, the C ABI does the work.

Mirrors the call made by OpenDecoder::forward for seq_len == 1
(fasterLlama/cuda/open_decoder.cu:138-239): same operands, same layouts.
"""
from __future__ import annotations

import ctypes as C

import torch

from . import capi


def _ptr(t) -> int | None:
    return None if t is None else t.data_ptr()


class DecodeAttention:
    """One decoder layer's attention step over a caller-owned KV cache.

    batch_size, head_num, size_per_head and total_len (= max_prompt_len + max_gen_len) carry the
    meaning of the OpenDecoder constructor arguments (open_decoder.h:66).  dtype is the storage
    type of q/k/v and of the caches: torch.float32 (the reference's cache type) or torch.float16.
    """

    def __init__(self, batch_size: int, head_num: int, size_per_head: int, total_len: int,
                 dtype: torch.dtype = torch.float16, nsplit: int = 0, softmax_scale: float = 0.0,
                 device: str | torch.device = "cuda:0"):
        self.lib = capi.load()
        if dtype not in (torch.float32, torch.float16):
            raise capi.FlAttnError(capi.FL_ATTN_ERR_DTYPE, "dtype must be float32 or float16")
        self.dtype = dtype
        self.device = torch.device(device)
        self.desc = capi.AttnDesc(batch_size, head_num, size_per_head, total_len,
                                  capi.FL_ATTN_F16 if dtype == torch.float16 else capi.FL_ATTN_F32,
                                  nsplit, softmax_scale, 0)
        n = C.c_size_t(0)
        with torch.cuda.device(self.device):
            capi.check(self.lib.fl_decode_attn_workspace_bytes(C.byref(self.desc), C.byref(n)))
        self.workspace_bytes = n.value
        # torch allocations are 512-byte aligned; the library asks for 256
        self.workspace = torch.empty(max(n.value, 256), dtype=torch.uint8, device=self.device)
        self.workspace_ready = False

    def init_workspace(self, stream: torch.cuda.Stream | None = None) -> None:
        """fl_decode_attn_workspace_init: from here on split steps run as one launch."""
        s = stream if stream is not None else torch.cuda.current_stream(self.device)
        with torch.cuda.device(self.device):
            capi.check(self.lib.fl_decode_attn_workspace_init(C.byref(self.desc), self.workspace.data_ptr(),
                                                              self.workspace.numel(), C.c_void_p(s.cuda_stream)))
        self.workspace_ready = True

    def plan(self, ctx: int, ragged: bool = False) -> capi.AttnPlan:
        plan = capi.AttnPlan()
        with torch.cuda.device(self.device):
            capi.check(self.lib.fl_decode_attn_plan(C.byref(self.desc), ctx, int(ragged), C.byref(plan)))
        return plan

    def make_io(self, q, k_new, v_new, k_cache, v_cache, freq_cis, out, start_pos: int = 0,
                rope_row: int = capi.FL_ATTN_ROPE_AT_POSITION, attn_mask=None, mask_ld: int | None = None,
                start_pos_per_seq=None, max_start_pos: int = -1, qkv_inp_scale=None,
                q_weight_scale=None, k_weight_scale=None, v_weight_scale=None, out_int8=None,
                out_scale=None, mask_tile_classes=None) -> capi.AttnIO:
        io = capi.AttnIO()
        io.q, io.k_new, io.v_new = _ptr(q), _ptr(k_new), _ptr(v_new)
        io.k_cache, io.v_cache = _ptr(k_cache), _ptr(v_cache)
        io.freq_cis = _ptr(freq_cis)
        io.attn_mask = _ptr(attn_mask)
        io.start_pos_per_seq = _ptr(start_pos_per_seq)
        io.out = _ptr(out)
        io.workspace = self.workspace.data_ptr()
        io.workspace_bytes = self.workspace.numel()
        io.mask_ld = self.desc.total_len if mask_ld is None else mask_ld
        io.start_pos = start_pos
        io.rope_row = rope_row
        io.max_start_pos = max_start_pos
        io.flags = capi.FL_ATTN_IO_WORKSPACE_READY if self.workspace_ready else 0
        io.qkv_inp_scale = _ptr(qkv_inp_scale)
        io.q_weight_scale = _ptr(q_weight_scale)
        io.k_weight_scale = _ptr(k_weight_scale)
        io.v_weight_scale = _ptr(v_weight_scale)
        io.out_int8 = _ptr(out_int8)
        io.out_scale = _ptr(out_scale)
        io.mask_tile_classes = _ptr(mask_tile_classes)
        return io

    def launch(self, io: capi.AttnIO, passes: int = 3, stream: torch.cuda.Stream | None = None) -> int:
        """Enqueues the step on `stream` (default: torch's current stream); returns the status."""
        s = stream if stream is not None else torch.cuda.current_stream(self.device)
        with torch.cuda.device(self.device):
            return self.lib.fl_decode_attn_forward_passes(C.byref(self.desc), C.byref(io),
                                                          C.c_void_p(s.cuda_stream), passes)

    def launch_noalloc(self, io: capi.AttnIO, stream: torch.cuda.Stream | None = None) -> int:
        """Same step through fl_decode_attn_forward_noalloc (the library's own scratch array)."""
        s = stream if stream is not None else torch.cuda.current_stream(self.device)
        with torch.cuda.device(self.device):
            return self.lib.fl_decode_attn_forward_noalloc(C.byref(self.desc), C.byref(io), C.c_void_p(s.cuda_stream))

    def forward(self, q, k_new, v_new, k_cache, v_cache, freq_cis, start_pos: int = 0, out=None, **kw):
        """RoPE(q, k_new) -> append k/v at row start_pos -> attention over rows [0, start_pos].

        Returns out [B, H*D] float32 (allocated when not given).  Raises FlAttnError on a
        non-zero status."""
        d = self.desc
        if out is None and kw.get("out_int8") is None:
            out = torch.empty(d.batch_size, d.head_num * d.size_per_head, dtype=torch.float32,
                              device=self.device)
        io = self.make_io(q, k_new, v_new, k_cache, v_cache, freq_cis, out, start_pos=start_pos, **kw)
        capi.check(self.launch(io))
        return out


class PrefillAttention(DecodeAttention):
    """Prompt-phase attention (seq_len new tokens per sequence) over the same caller-owned caches.

    q/k_new/v_new are [B, seq_len, H, D]; the result is [B, H, seq_len, D] float32, the layout of the
    reference's qkv_buf_ (open_decoder.h:61)."""

    def __init__(self, batch_size: int, head_num: int, size_per_head: int, total_len: int, max_seq_len: int,
                 dtype: torch.dtype = torch.float16, softmax_scale: float = 0.0,
                 device: str | torch.device = "cuda:0", fast_qk: bool = False):
        super().__init__(batch_size, head_num, size_per_head, total_len, dtype, 0, softmax_scale, device)
        if fast_qk:  # fp16 caches: queries as one fp16 value in the first product (see FL_ATTN_FLAG_FAST_PROMPT_QK)
            self.desc.flags |= capi.FL_ATTN_FLAG_FAST_PROMPT_QK
        n = C.c_size_t(0)
        capi.check(self.lib.fl_prefill_attn_workspace_bytes(C.byref(self.desc), max_seq_len, C.byref(n)))
        self.max_seq_len = max_seq_len
        self.workspace = torch.empty(max(n.value, self.workspace.numel()), dtype=torch.uint8, device=self.device)

    def classify_mask(self, attn_mask, mask_ld: int | None = None) -> torch.Tensor:
        """fl_prefill_mask_classify: the tile classes of a whole [L, L] mask, to pass as mask_tile_classes."""
        n = C.c_size_t(0)
        capi.check(self.lib.fl_prefill_mask_classes_bytes(C.byref(self.desc), C.byref(n)))
        table = torch.empty(n.value, dtype=torch.uint8, device=self.device)
        s = torch.cuda.current_stream(self.device)
        with torch.cuda.device(self.device):
            capi.check(self.lib.fl_prefill_mask_classify(C.byref(self.desc), attn_mask.data_ptr(),
                                                         self.desc.total_len if mask_ld is None else mask_ld,
                                                         table.data_ptr(), table.numel(), C.c_void_p(s.cuda_stream)))
        return table

    def launch_prefill(self, io: capi.AttnIO, seq_len: int, stream: torch.cuda.Stream | None = None, passes: int = 3) -> int:
        """passes: 1 = RoPE + append only, 2 = attention (+ INT8 epilogue) only, 3 = the whole step."""
        s = stream if stream is not None else torch.cuda.current_stream(self.device)
        with torch.cuda.device(self.device):
            if passes == 3:
                return self.lib.fl_prefill_attn_forward(C.byref(self.desc), C.byref(io), seq_len,
                                                        C.c_void_p(s.cuda_stream))
            return self.lib.fl_prefill_attn_forward_passes(C.byref(self.desc), C.byref(io), seq_len,
                                                           C.c_void_p(s.cuda_stream), passes)

    def prefill(self, q, k_new, v_new, k_cache, v_cache, freq_cis, start_pos: int = 0, out=None, **kw):
        d = self.desc
        seq_len = q.shape[1]
        if seq_len > self.max_seq_len:
            raise capi.FlAttnError(capi.FL_ATTN_ERR_WORKSPACE, "seq_len exceeds the workspace this object was sized for")
        if out is None and kw.get("out_int8") is None:
            out = torch.empty(d.batch_size, d.head_num, seq_len, d.size_per_head, dtype=torch.float32,
                              device=self.device)
        io = self.make_io(q, k_new, v_new, k_cache, v_cache, freq_cis, out, start_pos=start_pos, **kw)
        capi.check(self.launch_prefill(io, seq_len))
        return out


def rope_table(rows: int, size_per_head: int, base: float = 10000.0,
               device: str | torch.device = "cuda:0") -> torch.Tensor:
    """Device RoPE table [rows, D] (replaces launchPrecomputeFreqsCis, decoding_kernels.cu:116-135)."""
    lib = capi.load()
    dev = torch.device(device)
    t = torch.empty(rows, size_per_head, dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        capi.check(lib.fl_rope_table(t.data_ptr(), rows, size_per_head, base,
                                     C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)))
    return t
