"""CPU-side checks of the C-ABI library: it loads, exports every symbol the header declares, and
its host logic (validation, planning, workspace sizing, error strings) behaves.  No kernel is
launched: every forward() call here fails validation before any launch."""
import ctypes as C
import os
import re

import pytest

from fasterllama_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def desc(B=2, H=4, D=128, L=64, dtype=capi.FL_ATTN_F16, nsplit=0, scale=0.0, reserved=0):  # reserved: the flags word
    return capi.AttnDesc(B, H, D, L, dtype, nsplit, scale, reserved)


def fake_io(**over):
    """An io block whose pointers are non-NULL, 16-byte aligned and never dereferenced."""
    io = capi.AttnIO()
    for name in ("q", "k_new", "v_new", "k_cache", "v_cache", "freq_cis", "out"):
        setattr(io, name, 0x1000)
    io.workspace, io.workspace_bytes = 0x10000, 1 << 30
    io.mask_ld, io.start_pos, io.rope_row, io.max_start_pos = 64, 3, -1, -1
    for k, v in over.items():
        setattr(io, k, v)
    return io


def test_header_and_binding_agree_and_library_exports_everything():
    text = open(os.path.join(ROOT, "include", "fl_decode_attn.h")).read()
    declared = set(re.findall(r"^(?:int|const char \*)\s*(fl_[a-z0-9_]+)\s*\(", text, re.M))
    assert declared == set(capi.EXPORTED_SYMBOLS)
    lib = capi.load()
    for sym in declared:
        assert hasattr(lib, sym), sym
    assert lib.fl_attn_version() >= 100


def test_struct_layouts_match_the_header():
    # natural alignment on x86-64: 9 x 4 bytes; struct_size (padded to 8) + 10 pointers + size_t + int64 + 4 x int32 + 7 pointers
    assert C.sizeof(capi.AttnDesc) == 36
    assert C.sizeof(capi.AttnIO) == 8 + 10 * 8 + 8 + 8 + 16 + 7 * 8
    assert desc().struct_size == 36 and fake_io().struct_size == C.sizeof(capi.AttnIO)
    assert C.sizeof(capi.AttnPlan) == 16


def test_strerror_covers_every_status():
    msgs = {capi.strerror(s) for s in range(0, -12, -1)}
    assert len(msgs) == 12 and "unknown status" not in msgs
    assert capi.strerror(-99) == "unknown status"


@pytest.mark.parametrize("kw,want", [
    (dict(D=48), capi.FL_ATTN_ERR_HEAD_DIM),      # reference: throw "invalid size_per_head!" (decoder_kernels.cu:588)
    (dict(D=160), capi.FL_ATTN_ERR_HEAD_DIM),
    (dict(D=2048), capi.FL_ATTN_ERR_HEAD_DIM),
    (dict(D=0), capi.FL_ATTN_ERR_HEAD_DIM),
    (dict(B=0), capi.FL_ATTN_ERR_SHAPE),
    (dict(H=-1), capi.FL_ATTN_ERR_SHAPE),
    (dict(L=0), capi.FL_ATTN_ERR_SHAPE),
    (dict(B=70000), capi.FL_ATTN_ERR_SHAPE),
    (dict(dtype=2), capi.FL_ATTN_ERR_DTYPE),
    (dict(nsplit=-1), capi.FL_ATTN_ERR_ARGUMENT),
    (dict(nsplit=5000), capi.FL_ATTN_ERR_ARGUMENT),
    (dict(scale=-1.0), capi.FL_ATTN_ERR_ARGUMENT),
    (dict(scale=float("nan")), capi.FL_ATTN_ERR_ARGUMENT),
    (dict(reserved=2), capi.FL_ATTN_ERR_ARGUMENT),   # unknown flag bit
    (dict(reserved=-1), capi.FL_ATTN_ERR_ARGUMENT),
])
def test_descriptor_validation(kw, want):
    lib = capi.load()
    n = C.c_size_t(0)
    d = desc(**kw)
    assert lib.fl_decode_attn_workspace_bytes(C.byref(d), C.byref(n)) == want
    assert lib.fl_decode_attn_forward(C.byref(d), C.byref(fake_io()), None) == want


def test_struct_size_is_checked_before_any_member_is_trusted():
    """A caller built against another header: struct_size unset, shorter than the first layout that has it, or
    larger than the library's own struct."""
    lib = capi.load()
    n = C.c_size_t(0)
    for bad in (0, 32, C.sizeof(capi.AttnDesc) + 4):
        d = desc()
        d.struct_size = bad
        assert lib.fl_decode_attn_workspace_bytes(C.byref(d), C.byref(n)) == capi.FL_ATTN_ERR_STRUCT_SIZE
        assert lib.fl_prefill_attn_workspace_bytes(C.byref(d), 8, C.byref(n)) == capi.FL_ATTN_ERR_STRUCT_SIZE
        assert lib.fl_decode_attn_forward(C.byref(d), C.byref(fake_io()), None) == capi.FL_ATTN_ERR_STRUCT_SIZE
    for bad in (0, C.sizeof(capi.AttnIO) - 8, C.sizeof(capi.AttnIO) + 8):
        io = fake_io(start_pos=64)  # would be FL_ATTN_ERR_POSITION with a good struct_size
        io.struct_size = bad
        assert lib.fl_decode_attn_forward(C.byref(desc()), C.byref(io), None) == capi.FL_ATTN_ERR_STRUCT_SIZE
        assert lib.fl_decode_attn_forward_noalloc(C.byref(desc()), C.byref(io), None) == capi.FL_ATTN_ERR_STRUCT_SIZE
        assert lib.fl_prefill_attn_forward(C.byref(desc()), C.byref(io), 8, None) == capi.FL_ATTN_ERR_STRUCT_SIZE
    assert lib.fl_decode_attn_forward(C.byref(desc()), C.byref(fake_io(start_pos=64)), None) == capi.FL_ATTN_ERR_POSITION


def test_cache_slices_stay_below_two_gib():
    """The streaming kernel's buffer descriptors span 2^31 bytes from the base of a (batch, head) slice."""
    lib = capi.load()
    n = C.c_size_t(0)
    ok = desc(B=1, H=1, D=128, L=(1 << 31) // 256 - 65, dtype=capi.FL_ATTN_F16)
    assert lib.fl_decode_attn_workspace_bytes(C.byref(ok), C.byref(n)) == 0
    too_long = desc(B=1, H=1, D=128, L=(1 << 31) // 256 - 64, dtype=capi.FL_ATTN_F16)
    assert lib.fl_decode_attn_workspace_bytes(C.byref(too_long), C.byref(n)) == capi.FL_ATTN_ERR_SHAPE
    assert lib.fl_decode_attn_workspace_bytes(C.byref(desc(B=1, H=1, D=128, L=(1 << 31) // 512, dtype=capi.FL_ATTN_F32)),
                                              C.byref(n)) == capi.FL_ATTN_ERR_SHAPE


def test_null_arguments():
    lib = capi.load()
    n = C.c_size_t(0)
    assert lib.fl_decode_attn_workspace_bytes(None, C.byref(n)) == capi.FL_ATTN_ERR_NULL_POINTER
    assert lib.fl_decode_attn_workspace_bytes(C.byref(desc()), None) == capi.FL_ATTN_ERR_NULL_POINTER
    assert lib.fl_decode_attn_forward(C.byref(desc()), None, None) == capi.FL_ATTN_ERR_NULL_POINTER
    assert lib.fl_decode_attn_plan(C.byref(desc()), 8, 0, None) == capi.FL_ATTN_ERR_NULL_POINTER
    assert lib.fl_rope_table(None, 8, 64, 10000.0, None) == capi.FL_ATTN_ERR_NULL_POINTER
    for name in ("q", "k_new", "v_new", "k_cache", "v_cache", "freq_cis", "out"):
        assert lib.fl_decode_attn_forward(C.byref(desc()), C.byref(fake_io(**{name: None})), None) \
            == capi.FL_ATTN_ERR_NULL_POINTER, name


@pytest.mark.parametrize("over,want", [
    (dict(start_pos=64), capi.FL_ATTN_ERR_POSITION),    # start_pos + 1 rows must fit total_len
    (dict(start_pos=-1), capi.FL_ATTN_ERR_POSITION),
    (dict(rope_row=-2), capi.FL_ATTN_ERR_POSITION),
    (dict(start_pos_per_seq=0x2000, max_start_pos=64), capi.FL_ATTN_ERR_POSITION),
    (dict(q=0x1004), capi.FL_ATTN_ERR_ALIGNMENT),
    (dict(k_cache=0x1008), capi.FL_ATTN_ERR_ALIGNMENT),
    (dict(flags=6), capi.FL_ATTN_ERR_ARGUMENT),                          # unknown io flag bits
    (dict(attn_mask=0x3000, mask_ld=-5), capi.FL_ATTN_ERR_ARGUMENT),
    (dict(attn_mask=0x3000, mask_ld=3), capi.FL_ATTN_ERR_ARGUMENT),     # a mask row shorter than the 4 attended columns
    (dict(attn_mask=0x3000, mask_ld=40, start_pos_per_seq=0x2000, max_start_pos=40), capi.FL_ATTN_ERR_ARGUMENT),
    (dict(q_weight_scale=0x3000), capi.FL_ATTN_ERR_ARGUMENT),          # scales without qkv_inp_scale
    (dict(qkv_inp_scale=0x3000), capi.FL_ATTN_ERR_NULL_POINTER),       # inp scale without weight scales
    (dict(out_int8=0x3000), capi.FL_ATTN_ERR_NULL_POINTER),            # int8 output without its scale
])
def test_io_validation(over, want):
    lib = capi.load()
    assert lib.fl_decode_attn_forward(C.byref(desc()), C.byref(fake_io(**over)), None) == want


def test_workspace_validation_for_split_plans():
    lib = capi.load()
    d = desc(B=1, H=2, D=128, L=4096, nsplit=8)
    n = C.c_size_t(0)
    assert lib.fl_decode_attn_workspace_bytes(C.byref(d), C.byref(n)) == 0
    assert n.value >= 1 * 2 * 8 * (128 + 2) * 4 and n.value % 256 == 0
    io = fake_io(start_pos=4000, workspace=None)
    assert lib.fl_decode_attn_forward(C.byref(d), C.byref(io), None) == capi.FL_ATTN_ERR_WORKSPACE
    io = fake_io(start_pos=4000, workspace_bytes=n.value - 1)
    assert lib.fl_decode_attn_forward(C.byref(d), C.byref(io), None) == capi.FL_ATTN_ERR_WORKSPACE
    io = fake_io(start_pos=4000, workspace=0x10010)
    assert lib.fl_decode_attn_forward(C.byref(d), C.byref(io), None) == capi.FL_ATTN_ERR_WORKSPACE
    assert lib.fl_decode_attn_forward_passes(C.byref(d), C.byref(fake_io()), None, 0) == capi.FL_ATTN_ERR_ARGUMENT
    assert lib.fl_decode_attn_forward_passes(C.byref(d), C.byref(fake_io()), None, 4) == capi.FL_ATTN_ERR_ARGUMENT
    assert lib.fl_prefill_attn_forward_passes(C.byref(d), C.byref(fake_io()), 8, None, 0) == capi.FL_ATTN_ERR_ARGUMENT
    assert lib.fl_prefill_attn_forward_passes(C.byref(d), C.byref(fake_io()), 8, None, 4) == capi.FL_ATTN_ERR_ARGUMENT


def test_prompt_grids_that_exceed_the_launch_limit_are_a_shape_error():
    """B * H * ceil(S / 4) workgroups of the append kernel must fit a one-dimensional grid."""
    lib = capi.load()
    d = desc(B=2047, H=1024, D=32, L=8192, dtype=capi.FL_ATTN_F16)
    assert lib.fl_prefill_attn_forward(C.byref(d), C.byref(fake_io(start_pos=0)), 8192, None) == capi.FL_ATTN_ERR_SHAPE
    assert lib.fl_prefill_attn_forward(C.byref(d), C.byref(fake_io(workspace=None)), 64, None) == capi.FL_ATTN_ERR_WORKSPACE


def test_plans_cover_the_context_and_respect_forced_splits():
    lib = capi.load()
    plan = capi.AttnPlan()
    for (B, H, L, dtype) in ((1, 32, 4096, capi.FL_ATTN_F16), (64, 32, 2048, capi.FL_ATTN_F16),
                             (1, 4, 128, capi.FL_ATTN_F32), (32, 40, 4096, capi.FL_ATTN_F16)):
        d = desc(B=B, H=H, L=L, dtype=dtype, D=128 if H > 4 else 64)
        cap = None
        for ctx in (1, 2, 63, 64, 65, 1000, L):
            if ctx > L:
                continue
            for ragged in (0, 1):
                assert lib.fl_decode_attn_plan(C.byref(d), ctx, ragged, C.byref(plan)) == 0
                assert plan.nsplit >= 1 and plan.chunk_rows >= 1
                assert plan.nsplit * plan.chunk_rows >= ctx > (plan.nsplit - 1) * plan.chunk_rows
                assert (plan.two_pass != 0) == (plan.nsplit > 1) and plan.two_pass in (0, 1, 2)
                cap = max(cap or 0, plan.nsplit)
        # the workspace sized from the shape alone covers the largest plan
        n = C.c_size_t(0)
        assert lib.fl_decode_attn_workspace_bytes(C.byref(d), C.byref(n)) == 0
        assert n.value >= B * H * cap * (d.size_per_head + 2) * 4
    d = desc(B=1, H=2, L=4096, nsplit=7)
    assert lib.fl_decode_attn_plan(C.byref(d), 4096, 0, C.byref(plan)) == 0 and plan.nsplit == 7
    assert lib.fl_decode_attn_plan(C.byref(d), 3, 0, C.byref(plan)) == 0 and plan.nsplit == 3  # never more splits than rows
    assert lib.fl_decode_attn_plan(C.byref(d), 0, 0, C.byref(plan)) == capi.FL_ATTN_ERR_POSITION
    assert lib.fl_decode_attn_plan(C.byref(d), 4097, 0, C.byref(plan)) == capi.FL_ATTN_ERR_POSITION


def test_plan_heuristics_at_the_benchmark_shapes():
    """Without a GPU the library assumes 256 compute units; about one streaming workgroup per
    compute unit saturates HBM, so contexts are split only when B*H is smaller than that."""
    lib = capi.load()
    plan = capi.AttnPlan()
    # headline: B*H = 2048 -> single pass, no partials
    d = desc(B=64, H=32, D=128, L=2048)
    assert lib.fl_decode_attn_plan(C.byref(d), 2048, 0, C.byref(plan)) == 0 and (plan.nsplit, plan.two_pass) == (1, 0)
    # small split launches merge inside the streaming launch (2), large ones by a second launch (1)
    d = desc(B=1, H=32, D=128, L=4096)
    assert lib.fl_decode_attn_plan(C.byref(d), 4096, 0, C.byref(plan)) == 0 and plan.two_pass == 2
    d = desc(B=32, H=40, D=128, L=4096)
    assert lib.fl_decode_attn_plan(C.byref(d), 4096, 1, C.byref(plan)) == 0 and plan.two_pass == 1
    # B=8: 256 (b,h) pairs already fill the device -> no split either
    d = desc(B=8, H=32, D=128, L=1024)
    assert lib.fl_decode_attn_plan(C.byref(d), 1024, 0, C.byref(plan)) == 0 and (plan.nsplit, plan.chunk_rows) == (1, 1024)
    # B=1, ctx 4096: 32 pairs -> 8 splits of 512 rows
    d = desc(B=1, H=32, D=128, L=4096)
    assert lib.fl_decode_attn_plan(C.byref(d), 4096, 0, C.byref(plan)) == 0 and (plan.nsplit, plan.chunk_rows) == (8, 512)
    assert lib.fl_decode_attn_plan(C.byref(d), 200, 0, C.byref(plan)) == 0 and plan.nsplit == 1  # short contexts stay whole
    # ragged 13B batch: ~256 KB of K+V per workgroup -> 512-row chunks
    d = desc(B=32, H=40, D=128, L=4096)
    assert lib.fl_decode_attn_plan(C.byref(d), 4096, 1, C.byref(plan)) == 0 and (plan.nsplit, plan.chunk_rows) == (8, 512)
    assert lib.fl_decode_attn_plan(C.byref(d), 4096, 0, C.byref(plan)) == 0 and plan.nsplit == 1


def test_kv_cache_bytes_uses_64_bit_sizes():
    lib = capi.load()
    n = C.c_size_t(0)
    # B=64, H=32, L=4096, D=128 floats = 4 GiB: overflows the reference's int arithmetic
    assert lib.fl_kv_cache_bytes(C.byref(desc(B=64, H=32, L=4096, D=128, dtype=capi.FL_ATTN_F32)), C.byref(n)) == 0
    assert n.value == 64 * 32 * 4096 * 128 * 4
    assert lib.fl_kv_cache_bytes(C.byref(desc(B=64, H=32, L=2048, D=128)), C.byref(n)) == 0
    assert n.value == 1 << 30


def test_rope_table_argument_validation():
    lib = capi.load()
    assert lib.fl_rope_table(0x1000, 0, 64, 10000.0, None) == capi.FL_ATTN_ERR_SHAPE
    assert lib.fl_rope_table(0x1000, 8, 63, 10000.0, None) == capi.FL_ATTN_ERR_HEAD_DIM
    assert lib.fl_rope_table(0x1000, 8, 64, 0.0, None) == capi.FL_ATTN_ERR_ARGUMENT
    assert lib.fl_rope_table(0x1004, 8, 64, 10000.0, None) == capi.FL_ATTN_ERR_ALIGNMENT


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(capi, "_lib", None)
    monkeypatch.setattr(capi, "LIB_PATH", str(tmp_path / "libfl_decode_attn.so"))
    with pytest.raises(RuntimeError, match="no fallback"):
        capi.load()
