// Host-side logic of the C ABI (validation, planning, workspace sizing) under AddressSanitizer + UBSan.
// Linked with a sanitizer build of fl_decode_attn.hip's host pass; no kernel is ever launched: every
// forward() call here is rejected before a launch, so the program runs on a machine without a GPU.
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

#include "fl_decode_attn.h"

static int checks = 0, failures = 0;
#define EXPECT(cond)                                                      \
    do {                                                                  \
        ++checks;                                                         \
        if (!(cond)) {                                                    \
            ++failures;                                                   \
            std::fprintf(stderr, "FAIL line %d: %s\n", __LINE__, #cond);  \
        }                                                                 \
    } while (0)

static fl_attn_desc desc(int B, int H, int D, int L, int dtype, int nsplit)
{
    fl_attn_desc d;
    std::memset(&d, 0, sizeof d);
    d.struct_size = sizeof d;
    d.batch_size = B; d.head_num = H; d.size_per_head = D; d.total_len = L; d.dtype = dtype; d.nsplit = nsplit;
    return d;
}

static fl_attn_io fake_io()
{
    fl_attn_io io;
    std::memset(&io, 0, sizeof io);
    io.struct_size = sizeof io;
    void *fake = reinterpret_cast<void *>(0x1000);
    io.q = io.k_new = io.v_new = fake;
    io.k_cache = io.v_cache = fake;
    io.freq_cis = static_cast<const float *>(fake);
    io.out = static_cast<float *>(fake);
    io.workspace = reinterpret_cast<void *>(0x10000);
    io.workspace_bytes = size_t(1) << 40;
    io.mask_ld = 64; io.start_pos = 3; io.rope_row = -1; io.max_start_pos = -1;
    return io;
}

int main()
{
    const int Ds[] = {32, 64, 96, 128, 256, 512, 1024};
    const int Ls[] = {1, 2, 63, 64, 65, 1000, 4096, 33100};
    for (int dtype = 0; dtype < 2; ++dtype)
        for (int D : Ds)
            for (int L : Ls)
                for (int B : {1, 3, 64})
                    for (int nsplit : {0, 1, 7, 1024}) {
                        fl_attn_desc d = desc(B, 5, D, L, dtype, nsplit);
                        size_t ws = 0, kv = 0;
                        EXPECT(fl_decode_attn_workspace_bytes(&d, &ws) == FL_ATTN_OK && ws % 256 == 0);
                        EXPECT(fl_kv_cache_bytes(&d, &kv) == FL_ATTN_OK && kv == (size_t)B * 5 * L * D * (dtype ? 2 : 4));
                        for (int ctx : {1, L / 2 + 1, L})
                            for (int ragged = 0; ragged < 2; ++ragged) {
                                fl_attn_plan plan;
                                EXPECT(fl_decode_attn_plan(&d, ctx, ragged, &plan) == FL_ATTN_OK);
                                EXPECT(plan.nsplit >= 1 && plan.chunk_rows >= 1 && (int64_t)plan.nsplit * plan.chunk_rows >= ctx);
                                EXPECT((int64_t)(plan.nsplit - 1) * plan.chunk_rows < ctx);
                                EXPECT(ws >= (size_t)B * 5 * plan.nsplit * (D + 2) * 4);
                            }
                        size_t pws = 0;
                        const int st = fl_prefill_attn_workspace_bytes(&d, L, &pws);
                        EXPECT(st == FL_ATTN_OK || st == FL_ATTN_ERR_HEAD_DIM);
                    }
    // rejected before any launch
    fl_attn_desc d = desc(2, 4, 128, 64, FL_ATTN_F16, 0);
    fl_attn_io io = fake_io();
    io.start_pos = 64;
    EXPECT(fl_decode_attn_forward(&d, &io, nullptr) == FL_ATTN_ERR_POSITION);
    EXPECT(fl_decode_attn_forward_noalloc(&d, &io, nullptr) == FL_ATTN_ERR_POSITION);
    io = fake_io();
    io.q = reinterpret_cast<void *>(0x1004);
    EXPECT(fl_decode_attn_forward(&d, &io, nullptr) == FL_ATTN_ERR_ALIGNMENT);
    io = fake_io();
    io.attn_mask = reinterpret_cast<const float *>(0x3000);
    io.mask_ld = 3;
    EXPECT(fl_decode_attn_forward(&d, &io, nullptr) == FL_ATTN_ERR_ARGUMENT);
    EXPECT(fl_prefill_attn_forward(&d, &io, 8, nullptr) == FL_ATTN_ERR_ARGUMENT);
    io = fake_io();
    io.flags = 6;
    EXPECT(fl_decode_attn_forward(&d, &io, nullptr) == FL_ATTN_ERR_ARGUMENT);
    fl_attn_desc big = desc(128, 32, 128, 4096, FL_ATTN_F16, 64);
    io = fake_io();
    io.start_pos = 4095;
    EXPECT(fl_decode_attn_forward_noalloc(&big, &io, nullptr) == FL_ATTN_ERR_SCRATCH_LIMIT);
    io.workspace_bytes = 16;
    EXPECT(fl_decode_attn_forward(&big, &io, nullptr) == FL_ATTN_ERR_WORKSPACE);
    EXPECT(fl_decode_attn_workspace_init(&big, io.workspace, 16, nullptr) == FL_ATTN_ERR_WORKSPACE);
    fl_attn_desc huge = desc(1, 1, 1024, 2000000, FL_ATTN_F32, 0); // a (b,h) slice beyond 32-bit row offsets
    size_t n = 0;
    EXPECT(fl_decode_attn_workspace_bytes(&huge, &n) == FL_ATTN_ERR_SHAPE);
    // struct_size: unset, too small, or from a newer header -> rejected before any member is trusted
    d = desc(2, 4, 128, 64, FL_ATTN_F16, 0);
    io = fake_io();
    d.struct_size = 0;
    EXPECT(fl_decode_attn_workspace_bytes(&d, &n) == FL_ATTN_ERR_STRUCT_SIZE);
    d.struct_size = sizeof d + 8;
    EXPECT(fl_decode_attn_forward(&d, &io, nullptr) == FL_ATTN_ERR_STRUCT_SIZE);
    d.struct_size = sizeof d;
    io.struct_size = sizeof io - 8;
    EXPECT(fl_decode_attn_forward(&d, &io, nullptr) == FL_ATTN_ERR_STRUCT_SIZE);
    EXPECT(fl_prefill_attn_forward(&d, &io, 8, nullptr) == FL_ATTN_ERR_STRUCT_SIZE);
    io.struct_size = sizeof io + 16;
    EXPECT(fl_decode_attn_forward_noalloc(&d, &io, nullptr) == FL_ATTN_ERR_STRUCT_SIZE);
    for (int s = 0; s >= -12; --s) EXPECT(fl_attn_strerror(s) != nullptr && std::strlen(fl_attn_strerror(s)) > 0);
    std::printf("C-ABI host logic under sanitizers: %d checks, %d failures\n", checks, failures);
    return failures ? 1 : 0;
}
