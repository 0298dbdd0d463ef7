// C ABI of the decode-step attention library (see include/fl_decode_attn.h).
// Host side: argument validation, launch planning and kernel dispatch.  Enqueue-only: no
// allocation, no synchronisation; between calls the library remembers two immutable facts per device
// (its compute unit count and the address of its scratch array) and nothing about the caller.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <type_traits>

#include "../../include/fl_decode_attn.h"
#include "decode_attn_kernels.hpp"
#include "prefill_attn_kernels.hpp"

namespace {

using flattn::Params;

thread_local int g_last_hip_error = 0;

#ifndef FLATTN_WAVES
#define FLATTN_WAVES 4
#endif
#ifndef FLATTN_UNROLL
#define FLATTN_UNROLL 4
#endif
constexpr int kWaves = FLATTN_WAVES; // waves per streaming workgroup
constexpr int kMinChunkRows = 64; // never split a context finer than this
constexpr int kMaxSplits = 1024;

inline bool check_hip(hipError_t e)
{
    if (e != hipSuccess) {
        g_last_hip_error = (int)e;
        return false;
    }
    return true;
}

// Compute units of the current device.  The only thing the library remembers between calls: an
// immutable property of the hardware, cached per device id (256 when no device can be queried).
int device_cus()
{
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = 256;
        cached[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

bool head_dim_ok(int D)
{
    // the reference's set: the multiples of 32 up to 128 (decoder_kernels.cu:564-571, :640, :960) and 256, 512, 1024
    return D == 32 || D == 64 || D == 96 || D == 128 || D == 256 || D == 512 || D == 1024;
}

// The caller's struct, struct_size bytes of it, copied into a zeroed struct of this build: members the caller's
// header did not have yet read as zero / NULL.  MIN is the size of the first layout that carried struct_size.
constexpr size_t kDescMinBytes = offsetof(fl_attn_desc, flags) + sizeof(int32_t);
constexpr size_t kIoMinBytes = offsetof(fl_attn_io, mask_tile_classes) + sizeof(void *);

template <typename S>
int import_struct(const S *in, S *out, size_t min_bytes)
{
    if (!in) return FL_ATTN_ERR_NULL_POINTER;
    uint32_t n;
    std::memcpy(&n, in, sizeof n); // struct_size is the first member of both structs
    if (n < min_bytes || n > sizeof(S)) return FL_ATTN_ERR_STRUCT_SIZE;
    std::memset(static_cast<void *>(out), 0, sizeof(S));
    std::memcpy(static_cast<void *>(out), in, n);
    return FL_ATTN_OK;
}

int validate_desc(const fl_attn_desc *d)
{
    if (d->dtype != FL_ATTN_F32 && d->dtype != FL_ATTN_F16) return FL_ATTN_ERR_DTYPE;
    if (d->batch_size <= 0 || d->head_num <= 0 || d->total_len <= 0) return FL_ATTN_ERR_SHAPE;
    if (d->batch_size > 65535 || d->head_num > 65535) return FL_ATTN_ERR_SHAPE;
    if (!head_dim_ok(d->size_per_head)) return FL_ATTN_ERR_HEAD_DIM;
    if (d->nsplit < 0 || d->nsplit > kMaxSplits || (d->flags & ~FL_ATTN_FLAG_FAST_PROMPT_QK) != 0) return FL_ATTN_ERR_ARGUMENT;
    if (!(d->softmax_scale >= 0.f) || std::isinf(d->softmax_scale)) return FL_ATTN_ERR_ARGUMENT;
    // Row offsets inside one (b,h) slice of a cache are 32-bit byte offsets in the kernels, and the buffer descriptors
    // of the streaming kernel span 2^31 bytes from the slice's base: a slice stays below that, with room for the whole
    // tiles the prompt-phase kernels address past the last row (up to 63 rows, which fail the range check and read as
    // zeros).
    if (((int64_t)d->total_len + 64) * d->size_per_head * (d->dtype == FL_ATTN_F16 ? 2 : 4) >= ((int64_t)1 << 31)) return FL_ATTN_ERR_SHAPE;
    // the streaming grid is one-dimensional: B*H*splits workgroups must fit the 2^31 limit
    if ((int64_t)d->batch_size * d->head_num > (int64_t)INT32_MAX / kMaxSplits) return FL_ATTN_ERR_SHAPE;
    return FL_ATTN_OK;
}

// Rows a streaming workgroup consumes per loop trip; chunk sizes are multiples of it.
int rows_per_tile(const fl_attn_desc *d, int unroll)
{
    const int vec = d->dtype == FL_ATTN_F16 ? 8 : 4;
    const int lpr = flattn::lanes_per_row(d->size_per_head / vec);
    return kWaves * (64 / lpr) * unroll;
}

int unroll_for(const fl_attn_desc *d)
{
    const int vec = d->dtype == FL_ATTN_F16 ? 8 : 4;
    const int ch = d->size_per_head / vec;
    const int cpl = ch <= 64 ? 1 : ch / 64;
    return cpl >= 4 ? 1 : (cpl == 2 ? 2 : FLATTN_UNROLL);
}

// ---- launch planning ---------------------------------------------------------------------------
// A streaming workgroup alone pulls about 23 GB/s (one 64-row tile of 32 KB per ~1.4 us with eight
// 16-byte loads per lane in flight), so about one workgroup per compute unit already saturates HBM
// (measured: 256 workgroups reach 5.9 TB/s, 512 reach 6.9 TB/s).  Splitting the context buys nothing
// beyond that and costs the partial traffic plus a combine launch (~3.5 us), so:
//   uniform batches: nsplit = ceil(CUs / (B*H)), never finer than one tile per split, and contexts
//   of at most four tiles stay whole;
//   ragged batches (per-sequence positions on the device): work per (b,h) varies, so splits are
//   also capped at ~256 KB of K+V per workgroup, which measured best on 13B-shaped ragged batches.
constexpr size_t kRaggedChunkBytes = 256 * 1024;

int row_bytes(const fl_attn_desc *d) { return d->size_per_head * (d->dtype == FL_ATTN_F16 ? 2 : 4); }

int min_chunk_rows(const fl_attn_desc *d)
{
    const int tile = rows_per_tile(d, unroll_for(d));
    return tile > kMinChunkRows ? tile : kMinChunkRows;
}

int uniform_splits(const fl_attn_desc *d, int ctx)
{
    const int64_t bh = (int64_t)d->batch_size * d->head_num;
    const int64_t cus = device_cus();
    int64_t n = (cus + bh - 1) / bh;
    const int64_t most = ((int64_t)ctx + min_chunk_rows(d) - 1) / min_chunk_rows(d);
    if (n > most) n = most;
    // a combine launch costs about as much as streaming three more tiles in one workgroup
    // (measured 5.1 us unsplit vs 7.7 us split at B=1, H=4, ctx=128): short contexts stay whole
    if (ctx <= 4 * min_chunk_rows(d)) n = 1;
    if (n < 1) n = 1;
    if (n > kMaxSplits) n = kMaxSplits;
    return (int)n;
}

int ragged_splits(const fl_attn_desc *d, int max_ctx)
{
    const int64_t by_bytes = ((int64_t)max_ctx * 2 * row_bytes(d) + kRaggedChunkBytes - 1) / (int64_t)kRaggedChunkBytes;
    int64_t n = uniform_splits(d, max_ctx);
    if (by_bytes > n) n = by_bytes;
    const int64_t most = ((int64_t)max_ctx + min_chunk_rows(d) - 1) / min_chunk_rows(d);
    if (n > most) n = most;
    if (n < 1) n = 1;
    if (n > kMaxSplits) n = kMaxSplits;
    return (int)n;
}

// Upper bound of splits for any call with this shape (both estimates grow with the context length
// and the ragged one dominates): sizes the workspace.
int split_cap(const fl_attn_desc *d)
{
    if (d->nsplit > 0) return d->nsplit;
    return ragged_splits(d, d->total_len);
}

// The merge inside the streaming launch pays for small launches, where a second launch is a large part
// of the step (B=1, H=32, ctx 4096: 15.0 us against 15.7); with thousands of workgroups the arrival round
// trip in each of them costs more than the merge launch it saves (B=32, H=40 ragged: 214-219 us against 210).
bool fused_merge_pays(const fl_attn_desc *d, int nsplit)
{
    return kWaves * 64 == flattn::kCombineThreads &&
           (int64_t)nsplit * d->batch_size * d->head_num <= 4 * (int64_t)device_cus();
}

void make_plan(const fl_attn_desc *d, int ctx, bool ragged, fl_attn_plan *plan)
{
    const int tile = rows_per_tile(d, unroll_for(d));
    int n = d->nsplit > 0 ? d->nsplit : (ragged ? ragged_splits(d, ctx) : uniform_splits(d, ctx));
    if (n > ctx) n = ctx > 0 ? ctx : 1;
    int chunk = (ctx + n - 1) / n;
    if (chunk > tile) chunk = (chunk + tile - 1) / tile * tile; // whole tiles per split (may lower nsplit)
    if (chunk < 1) chunk = 1;
    plan->chunk_rows = chunk;
    plan->nsplit = (ctx + chunk - 1) / chunk;
    plan->threads = kWaves * 64;
    plan->two_pass = plan->nsplit <= 1 ? 0 : (fused_merge_pays(d, plan->nsplit) ? 2 : 1);
}

// Every entry point works on its own copy of the caller's descriptor (see import_struct).
int import_desc(const fl_attn_desc **desc, fl_attn_desc *copy)
{
    const int st = import_struct(*desc, copy, kDescMinBytes);
    if (st != FL_ATTN_OK) return st;
    *desc = copy;
    return validate_desc(copy);
}

size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// Row stride of the persistent mask tile class table: the 32-row blocks of one key tile, padded to whole words.
size_t class_table_ld(int total_len) { return align_up(((size_t)total_len + 31) / 32, 4); }

// Kernel launch that reports its own status: hipLaunchKernel returns the error of this launch,
// whereas hipGetLastError would also return (and clear) an error left behind by an earlier,
// unrelated HIP call of the calling thread.
template <typename T> struct same_type { typedef T type; };
template <typename... KArgs>
hipError_t launch(void (*kernel)(KArgs...), dim3 grid, dim3 block, hipStream_t stream, typename same_type<KArgs>::type... args)
{
    void *ptrs[] = {const_cast<void *>(static_cast<const void *>(&args))...};
    return hipLaunchKernel(reinterpret_cast<const void *>(kernel), grid, block, ptrs, 0, stream);
}

// Workspace layout: [arrivals B*H] [float output B*H*D (used when the caller asks for INT8 only)]
//                   [part_o slots*D] [part_m slots] [part_l slots], each 256-byte aligned,
// slots = B*H*cap.  The arrival counters come first so that their place depends on B and H only (not on
// the cache type or a forced split count).  The caller's workspace is laid out for the largest plan
// of the shape (cap = split_cap(desc)); the library's own scratch array for the plan of the call.
struct WorkspaceLayout {
    size_t arrivals, tmp_out, part_o, part_m, part_l, total;
};

WorkspaceLayout workspace_layout(const fl_attn_desc *d, int cap)
{
    const size_t bh = (size_t)d->batch_size * d->head_num;
    const size_t slots = bh * (size_t)cap;
    WorkspaceLayout w;
    w.arrivals = 0;
    w.tmp_out = align_up(bh * sizeof(int32_t), 256);
    w.part_o = w.tmp_out + align_up(bh * d->size_per_head * sizeof(float), 256);
    w.part_m = w.part_o + align_up(slots * d->size_per_head * sizeof(float), 256);
    w.part_l = w.part_m + align_up(slots * sizeof(float), 256);
    w.total = w.part_l + align_up(slots * sizeof(float), 256);
    return w;
}

WorkspaceLayout workspace_layout(const fl_attn_desc *d) { return workspace_layout(d, split_cap(d)); }

size_t workspace_need(const fl_attn_desc *d) { return workspace_layout(d).total; }

// Scratch memory of fl_decode_attn_forward_noalloc: one array per GPU, part of the library's code
// object, so that entry point never allocates.  Static storage starts out zero, which is the state the
// arrival counters need, and every launch that uses them leaves them zero again.  The counters own the
// last kScratchCounterBytes of the array, whatever the shape of the call: the float output and the split
// partials of any call stay below them, so no call can leave a non-zero word where a later call with
// another batch or head count expects a counter.
constexpr size_t kScratchBytes = FL_ATTN_NOALLOC_SCRATCH_BYTES;
constexpr size_t kScratchCounterBytes = 64u << 10; // 16384 (batch, head) pairs; larger steps merge in a second launch
constexpr size_t kScratchDataBytes = kScratchBytes - kScratchCounterBytes;
static __device__ __align__(256) unsigned char g_scratch[kScratchBytes];

// Layout of a step inside the library's own array: data sections packed from byte 0, counters in their fixed tail.
WorkspaceLayout scratch_layout(const fl_attn_desc *d, int cap)
{
    WorkspaceLayout w = workspace_layout(d, cap);
    const size_t shift = w.tmp_out; // the caller-workspace layout starts with its counters
    w.tmp_out -= shift; w.part_o -= shift; w.part_m -= shift; w.part_l -= shift; w.total -= shift;
    w.arrivals = kScratchDataBytes;
    return w;
}

// Device address of g_scratch on the current device (each GPU holds its own copy at its own address);
// looked up once per device.  In host code the array's name is only a handle for this lookup.
hipError_t scratch_address(char **ptr)
{
    static std::atomic<char *> cached[64];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= 64) return hipErrorInvalidDevice;
    char *p = cached[dev].load(std::memory_order_acquire);
    if (!p) {
        void *sym = nullptr;
        e = hipGetSymbolAddress(&sym, HIP_SYMBOL(g_scratch));
        if (e != hipSuccess) return e;
        if (!sym) return hipErrorInvalidSymbol;
        p = static_cast<char *>(sym);
        cached[dev].store(p, std::memory_order_release);
    }
    *ptr = p;
    return hipSuccess;
}

__global__ void fill_zero_kernel(int32_t *dst, int64_t n)
{
    for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) dst[i] = 0;
}

template <int D>
hipError_t launch_combine(const Params &p, int bh, hipStream_t stream)
{
    return launch(flattn::decode_attn_combine_kernel<D>, dim3(bh), dim3(flattn::kCombineThreads), stream, p);
}

hipError_t dispatch_combine(int D, const Params &p, int bh, hipStream_t stream)
{
    switch (D) {
    case 32: return launch_combine<32>(p, bh, stream);
    case 64: return launch_combine<64>(p, bh, stream);
    case 96: return launch_combine<96>(p, bh, stream);
    case 128: return launch_combine<128>(p, bh, stream);
    case 256: return launch_combine<256>(p, bh, stream);
    case 512: return launch_combine<512>(p, bh, stream);
    case 1024: return launch_combine<1024>(p, bh, stream);
    default: return hipErrorInvalidValue;
    }
}

// fp16 storage streams half the bytes per row, so its softmax uses the one-instruction base-2
// exponential; fp32 storage (the reference's cache type) keeps expf.
template <typename T> constexpr bool kFastExp = std::is_same<T, _Float16>::value;

template <typename T, int D>
hipError_t launch_split(const Params &p, dim3 grid, hipStream_t stream)
{
    constexpr int VEC = flattn::Vec16<T>::N;
    constexpr int CH = D / VEC;
    constexpr int CPL = CH <= 64 ? 1 : CH / 64;
    constexpr int UNROLL = CPL >= 4 ? 1 : (CPL == 2 ? 2 : FLATTN_UNROLL);
    if constexpr (kWaves * 64 == flattn::kCombineThreads) {
        if (p.arrivals && p.attn_mask) // one launch: the last workgroup of each (b,h) merges the partials
            return launch(flattn::decode_attn_split_kernel<T, D, kWaves, UNROLL, true, kFastExp<T>, true>, grid,
                          dim3(kWaves * 64), stream, p);
        if (p.arrivals)
            return launch(flattn::decode_attn_split_kernel<T, D, kWaves, UNROLL, false, kFastExp<T>, true>, grid,
                          dim3(kWaves * 64), stream, p);
    }
    if (p.attn_mask)
        return launch(flattn::decode_attn_split_kernel<T, D, kWaves, UNROLL, true, kFastExp<T>>, grid, dim3(kWaves * 64),
                      stream, p);
    return launch(flattn::decode_attn_split_kernel<T, D, kWaves, UNROLL, false, kFastExp<T>>, grid, dim3(kWaves * 64),
                  stream, p);
}

template <typename T>
hipError_t dispatch_split(int D, const Params &p, dim3 grid, hipStream_t stream)
{
    switch (D) {
    case 32: return launch_split<T, 32>(p, grid, stream);
    case 64: return launch_split<T, 64>(p, grid, stream);
    case 96: return launch_split<T, 96>(p, grid, stream);
    case 128: return launch_split<T, 128>(p, grid, stream);
    case 256: return launch_split<T, 256>(p, grid, stream);
    case 512: return launch_split<T, 512>(p, grid, stream);
    case 1024: return launch_split<T, 1024>(p, grid, stream);
    default: return hipErrorInvalidValue;
    }
}

// ---- prompt phase helpers

bool prefill_head_dim_ok(int D) { return head_dim_ok(D); }
constexpr bool prefill_wide(int D) { return D > 128; } // head dimension split across the waves of a workgroup

// Workspace layout of the prompt phase: [float output B*H*S*D (used when the caller asks for INT8
// only)] [mask tile classes: one word per 128-query block and 32-key tile, sized for a context that
// fills the cache], each 256-byte aligned.
struct PrefillWorkspace {
    size_t tmp_out, tile_class, total;
};

PrefillWorkspace prefill_workspace(const fl_attn_desc *d, int S)
{
    const size_t n = align_up((size_t)d->batch_size * d->head_num * (size_t)S * d->size_per_head * sizeof(float), 256);
    const size_t qblocks = ((size_t)S + flattn::kPrefillQueriesPerBlock - 1) / flattn::kPrefillQueriesPerBlock;
    const size_t ktiles = ((size_t)d->total_len + flattn::kPrefillKeysPerStep - 1) / flattn::kPrefillKeysPerStep;
    PrefillWorkspace w;
    w.tmp_out = 0;
    w.tile_class = n;
    w.total = n + align_up(qblocks * ktiles * sizeof(uint32_t), 256);
    return w;
}

template <typename T, int D>
hipError_t launch_prefill(const flattn::PrefillParams &p, hipStream_t stream, int passes)
{
    constexpr int VEC = flattn::Vec16<T>::N;
    constexpr int LPR = flattn::lanes_per_row(D / VEC);
    constexpr int ROWS = 256 / LPR;
    // lane groups of the append kernel: one per token and four heads for fp16 inputs where the head count allows
    // (B=8,S=1024: 49.0 -> 44.2 us; FP32 rows and int32 accumulators, twice the bytes per lane already, gain
    // nothing or lose: 71.2 -> 74.8 us)
    const int hpt = std::is_same<T, _Float16>::value && !p.inp_scale && p.H % 4 == 0 ? 4 : 1;
    const int64_t groups = (int64_t)p.B * p.S * (p.H / hpt);
    if ((groups + ROWS - 1) / ROWS > (int64_t)INT32_MAX) return hipErrorInvalidValue; // one-dimensional grid
    const dim3 agrid((unsigned)((groups + ROWS - 1) / ROWS));
    hipError_t e = hipSuccess;
    const unsigned qblocks = (unsigned)((p.S + flattn::kPrefillQueriesPerBlock - 1) / flattn::kPrefillQueriesPerBlock);
    if (passes & 1) {
        e = hpt == 4 ? launch(flattn::prefill_rope_append_kernel<T, D, 4>, agrid, dim3(256), stream, p)
                     : launch(flattn::prefill_rope_append_kernel<T, D, 1>, agrid, dim3(256), stream, p);
        if (e != hipSuccess) return e;
        if (p.attn_mask && !p.class_table) { // no table of the whole mask at hand: classify the rows of this call
            const int ktiles = (p.start_pos + p.S + flattn::kPrefillKeysPerStep - 1) / flattn::kPrefillKeysPerStep;
            e = launch(flattn::prefill_mask_classify_kernel, dim3((unsigned)ktiles, qblocks), dim3(256), stream, p, ktiles);
            if (e != hipSuccess) return e;
        }
    }
    if (!(passes & 2)) return hipSuccess;
    if constexpr (prefill_wide(D)) {
        const unsigned qb32 = (unsigned)((p.S + flattn::kWideQueriesPerBlock - 1) / flattn::kWideQueriesPerBlock);
        const dim3 wgrid(qb32 * (unsigned)(p.B * p.H)), wblock(flattn::kWideWaves * 64);
        if (p.attn_mask) return launch(flattn::prefill_attn_wide_kernel<T, D, true>, wgrid, wblock, stream, p);
        return launch(flattn::prefill_attn_wide_kernel<T, D, false>, wgrid, wblock, stream, p);
    } else {
        const dim3 grid(qblocks * (unsigned)(p.B * p.H)); // mapped to (query block, head) by prefill_block_to_tile
        if constexpr (std::is_same<T, _Float16>::value) {
            if (p.attn_mask && p.fast_qk) return launch(flattn::prefill_attn_f16_kernel<D, true, false>, grid, dim3(256), stream, p);
            if (p.attn_mask) return launch(flattn::prefill_attn_f16_kernel<D, true, true>, grid, dim3(256), stream, p);
            if (p.fast_qk) return launch(flattn::prefill_attn_f16_kernel<D, false, false>, grid, dim3(256), stream, p);
            return launch(flattn::prefill_attn_f16_kernel<D, false, true>, grid, dim3(256), stream, p);
        } else {
            if (p.attn_mask) return launch(flattn::prefill_attn_kernel<T, D, true>, grid, dim3(256), stream, p);
            return launch(flattn::prefill_attn_kernel<T, D, false>, grid, dim3(256), stream, p);
        }
    }
}

template <typename T>
hipError_t dispatch_prefill(int D, const flattn::PrefillParams &p, hipStream_t stream, int passes)
{
    switch (D) {
    case 32: return launch_prefill<T, 32>(p, stream, passes);
    case 64: return launch_prefill<T, 64>(p, stream, passes);
    case 96: return launch_prefill<T, 96>(p, stream, passes);
    case 128: return launch_prefill<T, 128>(p, stream, passes);
    case 256: return launch_prefill<T, 256>(p, stream, passes);
    case 512: return launch_prefill<T, 512>(p, stream, passes);
    case 1024: return launch_prefill<T, 1024>(p, stream, passes);
    default: return hipErrorInvalidValue;
    }
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

} // namespace

extern "C" {

int fl_attn_version(void) { return 300; }

int fl_attn_last_hip_error(void) { return g_last_hip_error; }

const char *fl_attn_strerror(int status)
{
    switch (status) {
    case FL_ATTN_OK: return "ok";
    case FL_ATTN_ERR_NULL_POINTER: return "a required pointer is NULL";
    case FL_ATTN_ERR_HEAD_DIM:
        return "invalid size_per_head (32, 64, 96, 128, 256, 512 or 1024)";
    case FL_ATTN_ERR_SHAPE: return "invalid batch_size / head_num / total_len";
    case FL_ATTN_ERR_POSITION: return "start_pos or rope_row out of range for total_len";
    case FL_ATTN_ERR_WORKSPACE: return "workspace missing, too small or not 256-byte aligned";
    case FL_ATTN_ERR_DTYPE: return "dtype must be FL_ATTN_F32 or FL_ATTN_F16";
    case FL_ATTN_ERR_HIP: return "a HIP runtime call failed";
    case FL_ATTN_ERR_ALIGNMENT: return "tensor base pointers must be 16-byte aligned";
    case FL_ATTN_ERR_ARGUMENT: return "inconsistent arguments";
    case FL_ATTN_ERR_STRUCT_SIZE:
        return "struct_size of fl_attn_desc / fl_attn_io is not set or comes from a newer header than this library";
    case FL_ATTN_ERR_SCRATCH_LIMIT:
        return "the step needs more scratch than fl_decode_attn_forward_noalloc holds (FL_ATTN_NOALLOC_SCRATCH_BYTES); "
               "use fl_decode_attn_forward with a caller-owned workspace";
    default: return "unknown status";
    }
}

int fl_decode_attn_workspace_bytes(const fl_attn_desc *desc, size_t *bytes)
{
    if (!bytes) return FL_ATTN_ERR_NULL_POINTER;
    fl_attn_desc desc_copy;
    int st = import_desc(&desc, &desc_copy);
    if (st != FL_ATTN_OK) return st;
    *bytes = workspace_need(desc);
    return FL_ATTN_OK;
}

int fl_kv_cache_bytes(const fl_attn_desc *desc, size_t *bytes)
{
    if (!bytes) return FL_ATTN_ERR_NULL_POINTER;
    fl_attn_desc desc_copy;
    int st = import_desc(&desc, &desc_copy);
    if (st != FL_ATTN_OK) return st;
    const size_t e = desc->dtype == FL_ATTN_F16 ? 2 : 4;
    *bytes = (size_t)desc->batch_size * desc->head_num * (size_t)desc->total_len * desc->size_per_head * e;
    return FL_ATTN_OK;
}

int fl_decode_attn_plan(const fl_attn_desc *desc, int32_t ctx, int32_t ragged, fl_attn_plan *plan)
{
    if (!plan) return FL_ATTN_ERR_NULL_POINTER;
    fl_attn_desc desc_copy;
    int st = import_desc(&desc, &desc_copy);
    if (st != FL_ATTN_OK) return st;
    if (ctx < 1 || ctx > desc->total_len) return FL_ATTN_ERR_POSITION;
    make_plan(desc, ctx, ragged != 0, plan);
    return FL_ATTN_OK;
}

} // extern "C"

namespace {

// The decode step behind every entry point.  own_scratch: take the split partials and arrival
// counters from the library's per-GPU scratch array instead of io->workspace (no allocation either way).
int decode_forward(const fl_attn_desc *desc, const fl_attn_io *io_in, void *hip_stream, int passes, bool own_scratch)
{
    fl_attn_desc desc_copy;
    int st = import_desc(&desc, &desc_copy);
    if (st != FL_ATTN_OK) return st;
    fl_attn_io io_copy;
    st = import_struct(io_in, &io_copy, kIoMinBytes);
    if (st != FL_ATTN_OK) return st;
    const fl_attn_io *io = &io_copy;
    if ((passes & ~3) != 0 || passes == 0) return FL_ATTN_ERR_ARGUMENT;
    if (!io->q || !io->k_new || !io->v_new || !io->k_cache || !io->v_cache || !io->freq_cis)
        return FL_ATTN_ERR_NULL_POINTER;
    const bool quant = io->out_int8 != nullptr;
    if (!io->out && !quant) return FL_ATTN_ERR_NULL_POINTER;
    if (quant && !io->out_scale) return FL_ATTN_ERR_NULL_POINTER;
    if (quant && (reinterpret_cast<uintptr_t>(io->out_int8) & 3u) != 0) return FL_ATTN_ERR_ALIGNMENT; // written four at a time
    if ((io->flags & ~FL_ATTN_IO_WORKSPACE_READY) != 0) return FL_ATTN_ERR_ARGUMENT;
    const bool i32 = io->qkv_inp_scale != nullptr;
    if (i32 && (!io->q_weight_scale || !io->k_weight_scale || !io->v_weight_scale)) return FL_ATTN_ERR_NULL_POINTER;
    if (!i32 && (io->q_weight_scale || io->k_weight_scale || io->v_weight_scale)) return FL_ATTN_ERR_ARGUMENT;
    if (!aligned16(io->q) || !aligned16(io->k_new) || !aligned16(io->v_new) || !aligned16(io->k_cache) ||
        !aligned16(io->v_cache) || !aligned16(io->freq_cis) || !aligned16(io->out) ||
        (i32 && (!aligned16(io->q_weight_scale) || !aligned16(io->k_weight_scale) || !aligned16(io->v_weight_scale))))
        return FL_ATTN_ERR_ALIGNMENT;

    const int L = desc->total_len;
    const bool ragged = io->start_pos_per_seq != nullptr;
    int max_pos;
    if (ragged) {
        max_pos = io->max_start_pos < 0 ? L - 1 : io->max_start_pos;
        if (max_pos >= L) return FL_ATTN_ERR_POSITION;
    } else {
        // reference: rows attended = start_pos + seq_len must fit the cache (open_decoder.cu:170-171)
        if (io->start_pos < 0 || io->start_pos >= L) return FL_ATTN_ERR_POSITION;
        max_pos = io->start_pos;
    }
    if (io->rope_row < FL_ATTN_ROPE_AT_POSITION) return FL_ATTN_ERR_POSITION;
    // a mask row must cover every attended column; mask_ld == 0 is the one-row (broadcast) mask
    if (io->attn_mask && (io->mask_ld < 0 || (io->mask_ld != 0 && io->mask_ld < (int64_t)max_pos + 1)))
        return FL_ATTN_ERR_ARGUMENT;

    fl_attn_plan plan;
    make_plan(desc, max_pos + 1, ragged, &plan);
    const int cap = own_scratch ? plan.nsplit : split_cap(desc);
    if (plan.nsplit > cap) return FL_ATTN_ERR_ARGUMENT;

    const bool direct = plan.nsplit == 1; // the streaming kernel normalises and writes the output itself
    const bool need_ws = !direct || (quant && !io->out);
    const WorkspaceLayout wl = own_scratch ? scratch_layout(desc, cap) : workspace_layout(desc, cap);
    char *ws = static_cast<char *>(io->workspace);
    if (own_scratch) {
        ws = nullptr;
        if (need_ws) {
            if (wl.total > kScratchDataBytes) return FL_ATTN_ERR_SCRATCH_LIMIT;
            if (!check_hip(scratch_address(&ws))) return FL_ATTN_ERR_HIP;
        }
    } else if (need_ws) {
        if (!io->workspace || io->workspace_bytes < wl.total) return FL_ATTN_ERR_WORKSPACE;
        if ((reinterpret_cast<uintptr_t>(io->workspace) & 255u) != 0) return FL_ATTN_ERR_WORKSPACE;
    }
    // One launch with the merge inside needs arrival counters that are zero: the library's own scratch
    // always is (between launches), the caller's workspace when it says so.
    const bool counters_fit = (size_t)desc->batch_size * desc->head_num * sizeof(int32_t) <= kScratchCounterBytes;
    const bool fused = plan.two_pass == 2 && passes == 3 &&
                       (own_scratch ? counters_fit : (io->flags & FL_ATTN_IO_WORKSPACE_READY) != 0);

    const int D = desc->size_per_head;
    Params p{};
    p.q = io->q; p.k_new = io->k_new; p.v_new = io->v_new;
    p.k_cache = io->k_cache; p.v_cache = io->v_cache;
    p.freq_cis = io->freq_cis; p.attn_mask = io->attn_mask; p.pos_per_seq = io->start_pos_per_seq;
    p.out = io->out ? io->out : reinterpret_cast<float *>(ws + wl.tmp_out);
    if (!direct) {
        p.part_o = reinterpret_cast<float *>(ws + wl.part_o);
        p.part_m = reinterpret_cast<float *>(ws + wl.part_m);
        p.part_l = reinterpret_cast<float *>(ws + wl.part_l);
        if (fused) p.arrivals = reinterpret_cast<int32_t *>(ws + wl.arrivals);
    }
    p.inp_scale = io->qkv_inp_scale; p.wq_scale = io->q_weight_scale;
    p.wk_scale = io->k_weight_scale; p.wv_scale = io->v_weight_scale;
    p.mask_ld = io->mask_ld;
    p.B = desc->batch_size; p.H = desc->head_num; p.L = L;
    p.start_pos = io->start_pos; p.rope_row = io->rope_row; p.max_pos = max_pos;
    p.chunk = plan.chunk_rows; p.split_cap = cap; p.direct = direct ? 1 : 0;
    p.scale = desc->softmax_scale > 0.f ? desc->softmax_scale : 1.0f / sqrtf((float)D);
    p.log2_domain = desc->dtype == FL_ATTN_F16 ? 1 : 0;

    hipStream_t stream = static_cast<hipStream_t>(hip_stream);
    const int bh = desc->batch_size * desc->head_num;
    if (passes & 1) {
        dim3 grid((unsigned)plan.nsplit * (unsigned)bh);
        hipError_t e = desc->dtype == FL_ATTN_F16 ? dispatch_split<_Float16>(D, p, grid, stream)
                                                  : dispatch_split<float>(D, p, grid, stream);
        if (!check_hip(e)) return FL_ATTN_ERR_HIP;
    }
    if (passes & 2) {
        if (!direct && !fused && !check_hip(dispatch_combine(D, p, bh, stream))) return FL_ATTN_ERR_HIP;
        if (quant) {
            if (!check_hip(launch(flattn::attn_quantize_transpose_kernel, dim3(desc->batch_size), dim3(flattn::kQuantThreads), stream, p.out,
                                  io->out_int8, io->out_scale, desc->head_num, 1, D)))
                return FL_ATTN_ERR_HIP;
        }
    }
    return FL_ATTN_OK;
}

} // namespace

extern "C" {

int fl_decode_attn_forward_passes(const fl_attn_desc *desc, const fl_attn_io *io, void *hip_stream, int passes)
{
    return decode_forward(desc, io, hip_stream, passes, false);
}

int fl_decode_attn_forward(const fl_attn_desc *desc, const fl_attn_io *io, void *hip_stream)
{
    return decode_forward(desc, io, hip_stream, 3, false);
}

int fl_decode_attn_forward_noalloc(const fl_attn_desc *desc, const fl_attn_io *io, void *hip_stream)
{
    return decode_forward(desc, io, hip_stream, 3, true);
}

int fl_decode_attn_workspace_init(const fl_attn_desc *desc, void *workspace, size_t workspace_bytes, void *hip_stream)
{
    fl_attn_desc desc_copy;
    int st = import_desc(&desc, &desc_copy);
    if (st != FL_ATTN_OK) return st;
    const WorkspaceLayout wl = workspace_layout(desc);
    if (!workspace || workspace_bytes < wl.total || (reinterpret_cast<uintptr_t>(workspace) & 255u) != 0)
        return FL_ATTN_ERR_WORKSPACE;
    const int64_t n = (int64_t)desc->batch_size * desc->head_num;
    // a fill kernel, not a memset: memset nodes are the one thing a caller cannot safely capture in a HIP graph
    if (!check_hip(launch(fill_zero_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), static_cast<hipStream_t>(hip_stream),
                          reinterpret_cast<int32_t *>(static_cast<char *>(workspace) + wl.arrivals), n)))
        return FL_ATTN_ERR_HIP;
    return FL_ATTN_OK;
}

// ---- prompt phase --------------------------------------------------------------------------------

int fl_prefill_attn_workspace_bytes(const fl_attn_desc *desc, int32_t seq_len, size_t *bytes)
{
    if (!bytes) return FL_ATTN_ERR_NULL_POINTER;
    fl_attn_desc desc_copy;
    int st = import_desc(&desc, &desc_copy);
    if (st != FL_ATTN_OK) return st;
    if (!prefill_head_dim_ok(desc->size_per_head)) return FL_ATTN_ERR_HEAD_DIM;
    if (seq_len < 1 || seq_len > desc->total_len) return FL_ATTN_ERR_POSITION;
    *bytes = prefill_workspace(desc, seq_len).total;
    return FL_ATTN_OK;
}

int fl_prefill_attn_forward(const fl_attn_desc *desc, const fl_attn_io *io_in, int32_t seq_len, void *hip_stream)
{
    return fl_prefill_attn_forward_passes(desc, io_in, seq_len, hip_stream, 3);
}

int fl_prefill_attn_forward_passes(const fl_attn_desc *desc, const fl_attn_io *io_in, int32_t seq_len, void *hip_stream, int passes)
{
    if (passes < 1 || passes > 3) return FL_ATTN_ERR_ARGUMENT;
    fl_attn_desc desc_copy;
    int st = import_desc(&desc, &desc_copy);
    if (st != FL_ATTN_OK) return st;
    if (!prefill_head_dim_ok(desc->size_per_head)) return FL_ATTN_ERR_HEAD_DIM;
    fl_attn_io io_copy;
    st = import_struct(io_in, &io_copy, kIoMinBytes);
    if (st != FL_ATTN_OK) return st;
    const fl_attn_io *io = &io_copy;
    if (!io->q || !io->k_new || !io->v_new || !io->k_cache || !io->v_cache || !io->freq_cis)
        return FL_ATTN_ERR_NULL_POINTER;
    const bool quant = io->out_int8 != nullptr;
    if (!io->out && !quant) return FL_ATTN_ERR_NULL_POINTER;
    if (quant && !io->out_scale) return FL_ATTN_ERR_NULL_POINTER;
    if (quant && (reinterpret_cast<uintptr_t>(io->out_int8) & 3u) != 0) return FL_ATTN_ERR_ALIGNMENT; // written four at a time
    if (io->flags != 0 || io->start_pos_per_seq) return FL_ATTN_ERR_ARGUMENT; // uniform positions only
    const bool i32 = io->qkv_inp_scale != nullptr;
    if (i32 && (!io->q_weight_scale || !io->k_weight_scale || !io->v_weight_scale)) return FL_ATTN_ERR_NULL_POINTER;
    if (!i32 && (io->q_weight_scale || io->k_weight_scale || io->v_weight_scale)) return FL_ATTN_ERR_ARGUMENT;
    if (!aligned16(io->q) || !aligned16(io->k_new) || !aligned16(io->v_new) || !aligned16(io->k_cache) ||
        !aligned16(io->v_cache) || !aligned16(io->freq_cis) || !aligned16(io->out) ||
        (i32 && (!aligned16(io->q_weight_scale) || !aligned16(io->k_weight_scale) || !aligned16(io->v_weight_scale))))
        return FL_ATTN_ERR_ALIGNMENT;
    const int L = desc->total_len;
    if (seq_len < 1 || io->start_pos < 0 || (int64_t)io->start_pos + seq_len > L) return FL_ATTN_ERR_POSITION;
    if (io->rope_row < FL_ATTN_ROPE_AT_POSITION) return FL_ATTN_ERR_POSITION;
    if (io->attn_mask && (io->mask_ld < 0 || (io->mask_ld != 0 && io->mask_ld < (int64_t)io->start_pos + seq_len)))
        return FL_ATTN_ERR_ARGUMENT;
    // one-dimensional grids: the attention kernels take a workgroup per 32 or 128 queries of a head, the append kernel
    // one per 4 to 64 (token, head) rows
    if ((int64_t)desc->batch_size * desc->head_num * ((seq_len + 3) / 4) > (int64_t)INT32_MAX) return FL_ATTN_ERR_SHAPE;

    const PrefillWorkspace wl = prefill_workspace(desc, seq_len);
    if (!io->workspace || io->workspace_bytes < wl.total) return FL_ATTN_ERR_WORKSPACE;
    if ((reinterpret_cast<uintptr_t>(io->workspace) & 255u) != 0) return FL_ATTN_ERR_WORKSPACE;
    char *ws = static_cast<char *>(io->workspace);

    const int D = desc->size_per_head;
    flattn::PrefillParams p{};
    p.q = io->q; p.k_new = io->k_new; p.v_new = io->v_new;
    p.k_cache = io->k_cache; p.v_cache = io->v_cache;
    p.freq_cis = io->freq_cis; p.attn_mask = io->attn_mask;
    p.tile_class = reinterpret_cast<uint32_t *>(ws + wl.tile_class);
    if (io->mask_tile_classes && io->attn_mask && io->mask_ld >= L && io->start_pos % 32 == 0) {
        if ((reinterpret_cast<uintptr_t>(io->mask_tile_classes) & 3u) != 0) return FL_ATTN_ERR_ALIGNMENT; // read a word at a time
        p.class_table = static_cast<const uint8_t *>(io->mask_tile_classes);
        p.class_ld = (int32_t)class_table_ld(L);
    }
    p.out = io->out ? io->out : reinterpret_cast<float *>(ws + wl.tmp_out);
    p.inp_scale = io->qkv_inp_scale; p.wq_scale = io->q_weight_scale;
    p.wk_scale = io->k_weight_scale; p.wv_scale = io->v_weight_scale;
    p.mask_ld = io->mask_ld;
    p.B = desc->batch_size; p.H = desc->head_num; p.L = L; p.S = seq_len;
    p.start_pos = io->start_pos; p.rope_row = io->rope_row;
    p.scale = desc->softmax_scale > 0.f ? desc->softmax_scale : 1.0f / sqrtf((float)D);
    p.fast_qk = (desc->flags & FL_ATTN_FLAG_FAST_PROMPT_QK) != 0;

    hipStream_t stream = static_cast<hipStream_t>(hip_stream);
    hipError_t e = desc->dtype == FL_ATTN_F16 ? dispatch_prefill<_Float16>(D, p, stream, passes) : dispatch_prefill<float>(D, p, stream, passes);
    if (!check_hip(e)) return FL_ATTN_ERR_HIP;
    if (quant && (passes & 2)) {
        if (!check_hip(launch(flattn::attn_quantize_transpose_kernel, dim3((unsigned)(desc->batch_size * seq_len)), dim3(flattn::kQuantThreads),
                              stream, p.out, io->out_int8, io->out_scale, desc->head_num, seq_len, D)))
            return FL_ATTN_ERR_HIP;
    }
    return FL_ATTN_OK;
}

int fl_prefill_mask_classes_bytes(const fl_attn_desc *desc, size_t *bytes)
{
    if (!bytes) return FL_ATTN_ERR_NULL_POINTER;
    fl_attn_desc desc_copy;
    int st = import_desc(&desc, &desc_copy);
    if (st != FL_ATTN_OK) return st;
    const size_t n = ((size_t)desc->total_len + 31) / 32;
    *bytes = n * class_table_ld(desc->total_len);
    return FL_ATTN_OK;
}

int fl_prefill_mask_classify(const fl_attn_desc *desc, const float *attn_mask, int64_t mask_ld, void *classes,
                             size_t classes_bytes, void *hip_stream)
{
    fl_attn_desc desc_copy;
    int st = import_desc(&desc, &desc_copy);
    if (st != FL_ATTN_OK) return st;
    if (!attn_mask || !classes) return FL_ATTN_ERR_NULL_POINTER;
    const int L = desc->total_len;
    const size_t n = ((size_t)L + 31) / 32;
    if (mask_ld < L) return FL_ATTN_ERR_ARGUMENT;
    if (classes_bytes < n * class_table_ld(L)) return FL_ATTN_ERR_WORKSPACE;
    if ((reinterpret_cast<uintptr_t>(classes) & 3u) != 0) return FL_ATTN_ERR_ALIGNMENT;
    if (n > 65535) return FL_ATTN_ERR_SHAPE;
    if (!check_hip(launch(flattn::mask_class_table_kernel, dim3((unsigned)n, (unsigned)n), dim3(64), static_cast<hipStream_t>(hip_stream),
                          attn_mask, mask_ld, L, L, static_cast<uint8_t *>(classes), (int)class_table_ld(L))))
        return FL_ATTN_ERR_HIP;
    return FL_ATTN_OK;
}

int fl_rope_table(float *freq_cis, int32_t rows, int32_t size_per_head, float base, void *hip_stream)
{
    if (!freq_cis) return FL_ATTN_ERR_NULL_POINTER;
    if (rows <= 0) return FL_ATTN_ERR_SHAPE;
    if (size_per_head <= 0 || (size_per_head & 1)) return FL_ATTN_ERR_HEAD_DIM;
    if (!(base > 0.f)) return FL_ATTN_ERR_ARGUMENT;
    if ((reinterpret_cast<uintptr_t>(freq_cis) & 7u) != 0) return FL_ATTN_ERR_ALIGNMENT;
    const int64_t n = (int64_t)rows * (size_per_head / 2);
    int64_t blocks = (n + 255) / 256;
    if (blocks > 65535) blocks = 65535;
    if (!check_hip(launch(flattn::rope_table_kernel, dim3((unsigned)blocks), dim3(256), static_cast<hipStream_t>(hip_stream),
                          freq_cis, rows, size_per_head, (double)base)))
        return FL_ATTN_ERR_HIP;
    return FL_ATTN_OK;
}

} // extern "C"
