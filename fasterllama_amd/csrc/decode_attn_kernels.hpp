// Decode-step self-attention kernels for gfx950 (MI355X): wave64, 128-bit coalesced K/V loads,
// DPP row reductions, online softmax per lane-group, split along the context axis.
//
// Replaces the kernel sequence of FasterLLaMA's generation branch
// (fasterLlama/cuda/open_decoder.cu:138-239): RoPE (decoder_kernels.cu:425-464), V pass-through
// (:858-884), cache append (:597-632), Q K^T GEMV, block softmax (:800-835) and P V GEMV.
//
// Work decomposition
//   grid = nsplit * B * H workgroups, linear id = split * (B*H) + (b*H + h); one workgroup streams
//   `chunk` consecutive cache rows of one (b, h).  Consecutive ids go round-robin to the 8 XCDs, so
//   with (b,h) fastest every XCD receives the same mix of splits: in a ragged batch the high splits
//   are empty for short sequences, and a split-fastest order would starve the XCDs that own them.
//   A row of D elements is 16-byte chunks; LPR = min(64, D*sizeof(T)/16) lanes own one row, so a
//   wave covers 64/LPR rows per load instruction and every load instruction of a workgroup
//   touches one contiguous span of the cache.  Each lane-group keeps a private online-softmax
//   state (m, l, o[its dims]); the groups of a workgroup are merged through LDS at the end.
//   With nsplit == 1 the merged result is normalised and written to `out`; otherwise the
//   unnormalised (m, l, o[D]) partial goes to the workspace for the combine kernel.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

// Every fused multiply-add in this file is written as fmaf(); the compiler must not form others,
// so that e.g. a zero mask row and a NULL mask give bit-identical outputs.
#pragma clang fp contract(off)

namespace flattn {

struct Params {
    const void *q, *k_new, *v_new;
    void *k_cache, *v_cache;
    const float *freq_cis;
    const float *attn_mask;
    const int32_t *pos_per_seq;
    float *out;
    float *part_o; // [B*H, split_cap, D]
    float *part_m; // [B*H, split_cap]
    float *part_l; // [B*H, split_cap]
    int32_t *arrivals; // [B*H] split workgroups that have published their partial; zero between launches
    const float *inp_scale, *wq_scale, *wk_scale, *wv_scale;
    int64_t mask_ld;
    int32_t B, H, L;
    int32_t start_pos, rope_row;
    int32_t max_pos;   // largest position the launch plan covers: nsplit * chunk > max_pos
    int32_t chunk;     // cache rows per split
    int32_t split_cap; // stride of the partial arrays along the split axis
    int32_t direct;    // 1: single split, write normalised output straight to `out`
    int32_t log2_domain; // 1: partial maxima are in base-2 units (fast-exp streaming kernel)
    float scale;
};

constexpr float kMaxFloor = -1e9f; // reference: float max_val = -1e9f (decoder_kernels.cu:811)

// ---------------------------------------------------------------- lane-group reductions (DPP)

template <int CTRL>
__device__ __forceinline__ float dpp_move(float x)
{
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, true));
}

// Sum over the LPR consecutive lanes that share a cache row; every lane gets the same bits.
template <int LPR>
__device__ __forceinline__ float group_sum(float x)
{
    if constexpr (LPR >= 2) x += dpp_move<0xB1>(x);  // quad_perm [1,0,3,2]
    if constexpr (LPR >= 4) x += dpp_move<0x4E>(x);  // quad_perm [2,3,0,1]
    if constexpr (LPR >= 8) x += dpp_move<0x141>(x); // row_half_mirror
    if constexpr (LPR >= 16) x += dpp_move<0x140>(x); // row_mirror
    if constexpr (LPR >= 32) x += __shfl_xor(x, 16);
    if constexpr (LPR >= 64) x += __shfl_xor(x, 32);
    return x;
}

// Same reduction for N independent values, one butterfly step at a time across all of them, so
// the data-parallel-primitive wait states of one value are filled by the others.
template <int LPR, int N>
__device__ __forceinline__ void group_sum_n(float (&x)[N])
{
#define FLATTN_STEP(COND, EXPR)                     \
    if constexpr (COND) {                           \
        _Pragma("unroll") for (int u = 0; u < N; ++u) x[u] += (EXPR); \
    }
    FLATTN_STEP(LPR >= 2, dpp_move<0xB1>(x[u]))
    FLATTN_STEP(LPR >= 4, dpp_move<0x4E>(x[u]))
    FLATTN_STEP(LPR >= 8, dpp_move<0x141>(x[u]))
    FLATTN_STEP(LPR >= 16, dpp_move<0x140>(x[u]))
    FLATTN_STEP(LPR >= 32, __shfl_xor(x[u], 16))
    FLATTN_STEP(LPR >= 64, __shfl_xor(x[u], 32))
#undef FLATTN_STEP
}

// exp in the softmax.  Natural domain: expf, as the reference (decoder_kernels.cu:824).
// Base-2 domain (FAST): scores are pre-multiplied by log2(e) and one v_exp_f32 evaluates 2^x.
template <bool FAST>
__device__ __forceinline__ float softmax_exp(float x)
{
    if constexpr (FAST) return __builtin_amdgcn_exp2f(x);
    else return expf(x);
}

constexpr float kLog2e = 1.4426950408889634f;

__device__ __forceinline__ float wave_max(float x)
{
    x = fmaxf(x, dpp_move<0xB1>(x));
    x = fmaxf(x, dpp_move<0x4E>(x));
    x = fmaxf(x, dpp_move<0x141>(x));
    x = fmaxf(x, dpp_move<0x140>(x));
    x = fmaxf(x, __shfl_xor(x, 16));
    x = fmaxf(x, __shfl_xor(x, 32));
    return x;
}

// ---------------------------------------------------------------- 16-byte element vectors

template <typename T> struct Vec16;
template <> struct Vec16<float> {
    static constexpr int N = 4;
    typedef float type __attribute__((ext_vector_type(4)));
};
template <> struct Vec16<_Float16> {
    static constexpr int N = 8;
    typedef _Float16 type __attribute__((ext_vector_type(8)));
};

// Raw buffer loads: address = base (in a 128-bit descriptor held in scalar registers) + a scalar byte
// offset + a 32-bit per-lane byte offset (+ an immediate).  The streaming loop needs no 64-bit vector
// address arithmetic and no register pairs for addresses, whatever the compiler's addressing heuristics
// decide elsewhere.  The hardware compares the per-lane offset with the descriptor's size: a lane whose
// offset is kLaneOutOfRange reads nothing and receives zeros.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
constexpr uint32_t kLaneOutOfRange = 0x80000000u;
constexpr int kLoadNonTemporal = 2; // cache-policy bits of the buffer builtins: bit 1 = nt

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_buffer(const void *base)
{
    // stride 0 (raw), 2^31 addressable bytes past `base`, 32-bit data format
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)kLaneOutOfRange, 0x00020000);
}

// RoPE of one interleaved pair; the operation order is part of the contract with the CPU
// checker so that the appended cache row is bit-identical:
//   o0 = fma(x0, c, -(x1*s)),  o1 = fma(x1, c, x0*s)      (decoder_kernels.cu:455-458)
__device__ __forceinline__ void rope_pair(float x0, float x1, float c, float s, float &o0, float &o1)
{
    float t0 = __fmul_rn(x1, s);
    float t1 = __fmul_rn(x0, s);
    o0 = __fmaf_rn(x0, c, -t0);
    o1 = __fmaf_rn(x1, c, t1);
}

// float -> storage type in two separately rounded steps (fp32 result first, then nearest-even to
// the storage type).  The empty asm keeps the compiler from folding the conversion into a
// mixed-precision FMA that would round the exact product-sum straight to half.
template <typename T>
__device__ __forceinline__ T to_storage(float x)
{
    asm volatile("" : "+v"(x));
    return (T)x;
}

// Loads VEC consecutive elements of a [B,1,H,D] operand as float: storage dtype, or int32
// accumulators scaled by inp_scale[b] * w_scale[h*D + d] (decoder_kernels.cu:449-452).
template <typename T, int VEC>
__device__ __forceinline__ void load_token_chunk(const void *base, size_t elem_off, bool is_i32,
                                                 float inp_scale, const float *w_scale_at,
                                                 float (&dst)[VEC])
{
    if (is_i32) {
        const int32_t *p = reinterpret_cast<const int32_t *>(base) + elem_off;
#pragma unroll
        for (int i = 0; i < VEC; i += 4) {
            int4 a = *reinterpret_cast<const int4 *>(p + i);
            float4 w = *reinterpret_cast<const float4 *>(w_scale_at + i);
            dst[i + 0] = __fmul_rn(__fmul_rn((float)a.x, inp_scale), w.x);
            dst[i + 1] = __fmul_rn(__fmul_rn((float)a.y, inp_scale), w.y);
            dst[i + 2] = __fmul_rn(__fmul_rn((float)a.z, inp_scale), w.z);
            dst[i + 3] = __fmul_rn(__fmul_rn((float)a.w, inp_scale), w.w);
        }
    } else {
        typedef typename Vec16<T>::type V;
        V v = *reinterpret_cast<const V *>(reinterpret_cast<const T *>(base) + elem_off);
#pragma unroll
        for (int i = 0; i < VEC; ++i) dst[i] = (float)v[i];
    }
}

// ---------------------------------------------------------------- merge of split partials

__device__ __forceinline__ float wave_sum(float x)
{
    x += dpp_move<0xB1>(x);
    x += dpp_move<0x4E>(x);
    x += dpp_move<0x141>(x);
    x += dpp_move<0x140>(x);
    x += __shfl_xor(x, 16);
    x += __shfl_xor(x, 32);
    return x;
}

constexpr int kCombineThreads = 256;
constexpr int kCombineMaxSplits = 1024;

// LDS of one merge: the split weights, two cross-wave reductions and the per-split-group sums.
template <int D>
struct CombineShared {
    static constexpr int TPG = D / 4 < kCombineThreads ? D / 4 : kCombineThreads; // threads per split-group
    static constexpr int SG = kCombineThreads / TPG;                             // split-groups (whole ones: at D = 96 the
                                                                                 // last 16 threads of the workgroup own none)
    float w[kCombineMaxSplits];
    float red[2][kCombineThreads / 64];
    float4 acc[SG][D / 4];
};

// Loads and stores of split partials.  DEVICE_COHERENT: relaxed atomic accesses at device scope, which
// go past the caches that are private to a compute unit or to one of the eight XCDs (each XCD has its own
// L2), so that a workgroup on one XCD reads what a workgroup on another has written in the same launch
// — without the whole-cache write-back and invalidation that a device-scope fence costs on this chip.
template <bool DEVICE_COHERENT>
__device__ __forceinline__ float load_partial(const float *p)
{
    if constexpr (DEVICE_COHERENT) return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else return *p;
}

template <bool DEVICE_COHERENT>
__device__ __forceinline__ float4 load_partial4(const float4 *p)
{
    if constexpr (DEVICE_COHERENT) {
        const float *f = reinterpret_cast<const float *>(p);
        return make_float4(load_partial<true>(f), load_partial<true>(f + 1), load_partial<true>(f + 2), load_partial<true>(f + 3));
    } else {
        return *p;
    }
}

template <bool DEVICE_COHERENT>
__device__ __forceinline__ void store_partial(float *p, float v)
{
    if constexpr (DEVICE_COHERENT) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else *p = v;
}

// Merges the (m, l, o[D]) partials of the first nsp splits of one (b,h), by the 256 threads of a workgroup:
//   M = max_s m_s;  w_s = exp(m_s - M);  out[d] = sum_s w_s o_s[d] / sum_s w_s l_s.
// The weights are computed once per split (threads over s), then the weighted sum over splits runs
// with D/4 threads per split-group (float4 per thread) and 256/(D/4) split-groups side by side, so
// the partial loads of a group are independent and in flight together.
template <int D, bool DEVICE_COHERENT>
__device__ __forceinline__ void combine_partials(const Params &p, int bh, int nsp, int tid, CombineShared<D> &sh)
{
    constexpr int TPG = CombineShared<D>::TPG, SG = CombineShared<D>::SG;
    constexpr int VPT = D / 4 / TPG; // float4 per thread
    const size_t slot0 = (size_t)bh * p.split_cap;
    const float floor_m = p.log2_domain ? kMaxFloor * kLog2e : kMaxFloor;

    // Every load whose address is known up front is issued before the first barrier — the statistics of
    // the first 256 splits and the first four partial rows of this thread's split-group — so that the
    // merge waits for memory once, not once per phase.  The arithmetic and its order do not depend on it.
    const int sg = tid / TPG, t = tid % TPG;
    const bool in_group = SG * TPG == kCombineThreads || sg < SG; // this thread belongs to a whole split-group
    const float4 *po = reinterpret_cast<const float4 *>(p.part_o + slot0 * D);
    const float m_first = tid < nsp ? load_partial<DEVICE_COHERENT>(p.part_m + slot0 + tid) : floor_m;
    const float l_first = tid < nsp ? load_partial<DEVICE_COHERENT>(p.part_l + slot0 + tid) : 0.f;
    float4 x_first[4][VPT];
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
        for (int v = 0; v < VPT; ++v)
            x_first[k][v] = in_group && sg + k * SG < nsp ? load_partial4<DEVICE_COHERENT>(po + (size_t)(sg + k * SG) * (D / 4) + v * TPG + t)
                                              : make_float4(0.f, 0.f, 0.f, 0.f);

    float mx = floor_m;
    if (tid < nsp) {
        sh.w[tid] = m_first;
        mx = fmaxf(mx, m_first);
    }
    for (int s = tid + kCombineThreads; s < nsp; s += kCombineThreads) {
        const float ms = load_partial<DEVICE_COHERENT>(p.part_m + slot0 + s);
        sh.w[s] = ms;
        mx = fmaxf(mx, ms);
    }
    mx = wave_max(mx);
    if ((tid & 63) == 0) sh.red[0][tid >> 6] = mx;
    __syncthreads();
    float M = sh.red[0][0];
#pragma unroll
    for (int w = 1; w < kCombineThreads / 64; ++w) M = fmaxf(M, sh.red[0][w]);

    float lsum = 0.f;
    for (int s = tid; s < nsp; s += kCombineThreads) {
        const float dm = sh.w[s] - M;
        const float w = p.log2_domain ? __builtin_amdgcn_exp2f(dm) : expf(dm);
        sh.w[s] = w;
        lsum = fmaf(s == tid ? l_first : load_partial<DEVICE_COHERENT>(p.part_l + slot0 + s), w, lsum);
    }
    lsum = wave_sum(lsum);
    if ((tid & 63) == 0) sh.red[1][tid >> 6] = lsum;
    __syncthreads();
    float Lsum = sh.red[1][0];
#pragma unroll
    for (int w = 1; w < kCombineThreads / 64; ++w) Lsum += sh.red[1][w];

    float4 acc[VPT];
#pragma unroll
    for (int v = 0; v < VPT; ++v) acc[v] = make_float4(0.f, 0.f, 0.f, 0.f);
    auto add_row = [&](const float4 (&x)[VPT], float w) {
#pragma unroll
        for (int v = 0; v < VPT; ++v) {
            acc[v].x = fmaf(x[v].x, w, acc[v].x);
            acc[v].y = fmaf(x[v].y, w, acc[v].y);
            acc[v].z = fmaf(x[v].z, w, acc[v].z);
            acc[v].w = fmaf(x[v].w, w, acc[v].w);
        }
    };
#pragma unroll
    for (int k = 0; k < 4; ++k)
        if (in_group && sg + k * SG < nsp) add_row(x_first[k], sh.w[sg + k * SG]);
    int s = in_group ? sg + 4 * SG : nsp;
    for (; s + 3 * SG < nsp; s += 4 * SG) { // four independent partial rows in flight
        float4 x[4][VPT];
#pragma unroll
        for (int k = 0; k < 4; ++k)
#pragma unroll
            for (int v = 0; v < VPT; ++v) x[k][v] = load_partial4<DEVICE_COHERENT>(po + (size_t)(s + k * SG) * (D / 4) + v * TPG + t);
#pragma unroll
        for (int k = 0; k < 4; ++k) add_row(x[k], sh.w[s + k * SG]);
    }
    for (; s < nsp; s += SG) {
        float4 x[VPT];
#pragma unroll
        for (int v = 0; v < VPT; ++v) x[v] = load_partial4<DEVICE_COHERENT>(po + (size_t)s * (D / 4) + v * TPG + t);
        add_row(x, sh.w[s]);
    }
    if (in_group) {
#pragma unroll
        for (int v = 0; v < VPT; ++v) sh.acc[sg][v * TPG + t] = acc[v];
    }
    __syncthreads();
    for (int d4 = tid; d4 < D / 4; d4 += kCombineThreads) {
        float4 r = sh.acc[0][d4];
#pragma unroll
        for (int k = 1; k < SG; ++k) {
            const float4 y = sh.acc[k][d4];
            r.x += y.x; r.y += y.y; r.z += y.z; r.w += y.w;
        }
        r.x = r.x / Lsum; r.y = r.y / Lsum; r.z = r.z / Lsum; r.w = r.w / Lsum;
        reinterpret_cast<float4 *>(p.out + (size_t)bh * D)[d4] = r;
    }
}

// Splits of one (b,h) that stream rows (the others return at once): ceil((P+1)/chunk), which is at most
// ceil((max_pos+1)/chunk) = launched splits <= split_cap <= kCombineMaxSplits.
__device__ __forceinline__ int active_splits(const Params &p, int P)
{
    return min((P + p.chunk) / p.chunk, min(p.split_cap, kCombineMaxSplits));
}

// grid = B*H, block = 256: the merge as a launch of its own (second pass of a two-pass step).
template <int D>
__global__ __launch_bounds__(kCombineThreads) void decode_attn_combine_kernel(const Params p)
{
    __shared__ CombineShared<D> sh;
    const int bh = blockIdx.x, tid = threadIdx.x;
    const int b = bh / p.H;
    const int P = p.pos_per_seq ? p.pos_per_seq[b] : p.start_pos;
    if (P < 0 || P >= p.L || P > p.max_pos) { // uniform per block; no partial of this (b,h) was written
        for (int d = tid; d < D; d += kCombineThreads) p.out[(size_t)bh * D + d] = __builtin_nanf("");
        return;
    }
    combine_partials<D, false>(p, bh, active_splits(p, P), tid, sh);
}

// ---------------------------------------------------------------- streaming (split) kernel

// Lanes that share one cache row of `chunks` 16-byte chunks: the next power of two, at most a wave.
constexpr int lanes_per_row(int chunks)
{
    int n = 1;
    while (n < chunks && n < 64) n *= 2;
    return n;
}

#ifndef FLATTN_MIN_WAVES_PER_EU
#define FLATTN_MIN_WAVES_PER_EU 8
#endif

// Occupancy the register allocator must leave room for: 8 waves per SIMD (<= 64 VGPRs) when one
// lane owns a single 16-byte chunk of the row, fewer for the large head sizes.
template <typename T, int D>
constexpr int min_waves_per_eu()
{
    constexpr int cpl = (D / Vec16<T>::N) <= 64 ? 1 : (D / Vec16<T>::N) / 64;
    if (lanes_per_row(D / Vec16<T>::N) != D / Vec16<T>::N && cpl == 1) return 4; // padded lane groups (96): the extra
                                                                                  // predicate spills at 64 registers
    if (lanes_per_row(D / Vec16<T>::N) < 8) return 4; // 16 rows per wave: the group merge needs the registers
    return cpl == 1 ? FLATTN_MIN_WAVES_PER_EU : (cpl == 2 ? 4 : 2);
}

// FAST selects the base-2 softmax (fp16 storage); the fp32-storage kernels keep expf.
// FUSED (split launches only): the workgroup that publishes the last partial of a (b,h) also merges
// them, so the step is one launch.  Arrivals are counted in p.arrivals[b*H + h], which must be zero
// when the launch starts and is zero again when it ends.
template <typename T, int D, int WAVES, int UNROLL, bool HAS_MASK, bool FAST, bool FUSED = false>
__global__ __launch_bounds__(WAVES * 64)
__attribute__((amdgpu_waves_per_eu(min_waves_per_eu<T, D>(), 8)))
void decode_attn_split_kernel(const Params p)
{
    typedef typename Vec16<T>::type V;
    constexpr int VEC = Vec16<T>::N;
    constexpr int CH = D / VEC;             // 16-byte chunks per row
    constexpr int LPR = lanes_per_row(CH);  // lanes per row: a power of two, for the butterfly reductions
    constexpr int CPL = (CH + LPR - 1) / LPR; // chunks per lane
    constexpr bool PADDED = LPR * CPL != CH; // size_per_head 96: the last lanes of a row's group own no chunk; they load
                                             // out of range (zeros) and add zeros to every sum
    constexpr int GPW = 64 / LPR;           // rows per wave per load instruction
    constexpr int GROUPS = WAVES * GPW;     // rows per workgroup per load instruction
    constexpr int EPL = CPL * VEC;          // elements of a row owned by one lane
    constexpr int ROW_BYTES = D * (int)sizeof(T);
    static_assert(CH * VEC == D && (!PADDED || CPL == 1), "head size must tile into 16-byte chunks");

    __shared__ float s_o[GROUPS][D];
    __shared__ float s_m[GROUPS];
    __shared__ float s_l[GROUPS];
    __shared__ typename std::conditional<FUSED, CombineShared<D>, char>::type s_merge;
    __shared__ int s_last;
    static_assert(!FUSED || WAVES * 64 == kCombineThreads, "the fused merge runs on a 256-thread workgroup");

    const int H = p.H, L = p.L;
    const int BH = p.B * H;
    const int split = blockIdx.x / BH, bh = blockIdx.x % BH;
    const int b = bh / H, h = bh % H;
    const int P = p.pos_per_seq ? p.pos_per_seq[b] : p.start_pos;
    const int tid = threadIdx.x;

    // A position outside the cache, or beyond the bound the launch was planned for (no split would
    // own its row): store nothing, poison the output.
    if (P < 0 || P >= L || P > p.max_pos) {
        if ((p.direct || FUSED) && split == 0)
            for (int d = tid; d < D; d += WAVES * 64) p.out[(size_t)bh * D + d] = __builtin_nanf("");
        return;
    }
    const int ctx = P + 1;
    const int start = split * p.chunk;
    if (start >= ctx) return;
    const int end = min(start + p.chunk, ctx);
    const bool owns_new = (end == ctx);           // exactly one split per (b,h)
    const int cache_end = owns_new ? P : end;     // rows [start, cache_end) come from the cache

    const int lane = tid & 63, wave = tid >> 6;
    const int g = lane / LPR, lig = lane % LPR;
    const int group = wave * GPW + g;

    // Uniform (scalar) base of this (b,h) plus a 32-bit per-lane byte offset: the loads below are
    // "scalar base + vector offset" with no per-row 64-bit vector address arithmetic.
    const char *Kb = reinterpret_cast<const char *>(p.k_cache) + (size_t)bh * L * ROW_BYTES;
    const char *Vb = reinterpret_cast<const char *>(p.v_cache) + (size_t)bh * L * ROW_BYTES;
    const bool has_chunk = !PADDED || lig < CH;
    const uint32_t lane_off = has_chunk ? (uint32_t)(group * ROW_BYTES + lig * 16) : kLaneOutOfRange;
    const float *mrow = HAS_MASK ? p.attn_mask + (size_t)P * p.mask_ld : nullptr;
    // descriptors of this (b,h)'s K rows, V rows and mask row; row offsets go into the scalar offset
    // (the host checks that L * ROW_BYTES fits 32 bits)
    const __amdgpu_buffer_rsrc_t Kbuf = make_buffer(Kb), Vbuf = make_buffer(Vb);
    const __amdgpu_buffer_rsrc_t Mbuf = make_buffer(HAS_MASK ? (const void *)mrow : (const void *)Kb);

    // One tile = UNROLL rows per lane-group.  CHECK guards the ragged last tile.
    V kv[UNROLL][CPL], vv[UNROLL][CPL];
    bool ok[UNROLL];
    constexpr int ROWS_PER_TILE = GROUPS * UNROLL;
    // Mask entries of a tile: lane-group `group` needs those of rows r0 + u*GROUPS + group, u < UNROLL.
    // Each lane fetches ONE of them — that of u = lane % 4 — so a single load instruction and a single
    // register carry the tile's mask, and a quad broadcast (DPP) hands entry u to every lane when the
    // scores are formed.  (One load per (lane, u) kept four more registers live across the K/V loads,
    // which the 64-register budget of the 8-waves-per-SIMD occupancy does not have.)
    static_assert(!HAS_MASK || (LPR >= 4 && UNROLL <= 4), "the mask broadcast works on quads of lanes");
    float mkv = 0.f;
    const uint32_t mask_off = (uint32_t)((((lane & 3) < UNROLL ? (lane & 3) : 0) * GROUPS + group) * 4);

    // Issues every load of the tile that starts at row r0 and fences the scheduler so that all
    // 2*UNROLL*CPL of them stay in flight together.
    auto issue_tile = [&](int r0, auto check_tag) {
        constexpr bool CHECK = decltype(check_tag)::value;
        const uint32_t tile_off = (uint32_t)r0 * (uint32_t)ROW_BYTES; // uniform
        if constexpr (HAS_MASK) { // first, so that it has landed when the K rows have
            uint32_t moff = mask_off;
            if (CHECK && r0 + (int)(moff >> 2) >= cache_end) moff = kLaneOutOfRange; // reads nothing; the score is discarded
            mkv = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(Mbuf, moff, (uint32_t)r0 * 4u, 0));
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            ok[u] = !CHECK || (r0 + u * GROUPS + group) < cache_end;
            const uint32_t off = (CHECK && !ok[u]) ? kLaneOutOfRange : lane_off; // rows past the end: zeros, discarded
#pragma unroll
            for (int c = 0; c < CPL; ++c)
                kv[u][c] = __builtin_bit_cast(V, __builtin_amdgcn_raw_buffer_load_b128(
                                                     Kbuf, off + (uint32_t)(c * LPR * 16),
                                                     tile_off + (uint32_t)(u * GROUPS * ROW_BYTES), kLoadNonTemporal));
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const uint32_t off = (CHECK && !ok[u]) ? kLaneOutOfRange : lane_off;
#pragma unroll
            for (int c = 0; c < CPL; ++c)
                vv[u][c] = __builtin_bit_cast(V, __builtin_amdgcn_raw_buffer_load_b128(
                                                     Vbuf, off + (uint32_t)(c * LPR * 16),
                                                     tile_off + (uint32_t)(u * GROUPS * ROW_BYTES), kLoadNonTemporal));
        }
        __builtin_amdgcn_sched_barrier(0);
    };

    const bool is_i32 = p.inp_scale != nullptr;
    const float inp_scale = is_i32 ? p.inp_scale[b] : 0.f;
    const int rope_row = p.rope_row < 0 ? P : p.rope_row;
    const float *freq = p.freq_cis + (size_t)rope_row * D;

    // RoPE(q) for the dims this lane owns, kept in registers (fp32)
    float qr[EPL];
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
        const int e0 = (c * LPR + lig) * VEC;
        if (PADDED && !has_chunk) {
#pragma unroll
            for (int i = 0; i < VEC; ++i) qr[c * VEC + i] = 0.f;
            continue;
        }
        float x[VEC];
        load_token_chunk<T, VEC>(p.q, (size_t)bh * D + e0, is_i32, inp_scale,
                                 is_i32 ? p.wq_scale + h * D + e0 : nullptr, x);
#pragma unroll
        for (int i = 0; i < VEC; i += 4) {
            float4 f = *reinterpret_cast<const float4 *>(freq + e0 + i);
            rope_pair(x[i], x[i + 1], f.x, f.y, qr[c * VEC + i], qr[c * VEC + i + 1]);
            rope_pair(x[i + 2], x[i + 3], f.z, f.w, qr[c * VEC + i + 2], qr[c * VEC + i + 3]);
        }
    }

    // v = qk*scaler + mask (decoder_kernels.cu:815); the base-2 path folds log2(e) into both terms
    const float scale = FAST ? p.scale * kLog2e : p.scale;
    const float floor_m = FAST ? kMaxFloor * kLog2e : kMaxFloor;

    float m = floor_m, l = 0.f;
    float o[EPL];
#pragma unroll
    for (int e = 0; e < EPL; ++e) o[e] = 0.f;

    // Scores, online-softmax update and weighted V sum for the tile held in kv/vv.
    auto consume_tile = [&](auto check_tag) {
        constexpr bool CHECK = decltype(check_tag)::value;
        float s[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            float acc = 0.f;
#pragma unroll
            for (int c = 0; c < CPL; ++c)
#pragma unroll
                for (int i = 0; i < VEC; ++i) acc = fmaf((float)kv[u][c][i], qr[c * VEC + i], acc);
            s[u] = acc;
        }
        group_sum_n<LPR, UNROLL>(s);
        float tmax = m;
        float mk[UNROLL];
        if constexpr (HAS_MASK) { // entry u of the tile's mask sits in lane u of every quad
            const float mq = FAST ? mkv * kLog2e : mkv;
            mk[0] = dpp_move<0x00>(mq);
            if constexpr (UNROLL > 1) mk[1] = dpp_move<0x55>(mq);
            if constexpr (UNROLL > 2) mk[2] = dpp_move<0xAA>(mq);
            if constexpr (UNROLL > 3) mk[3] = dpp_move<0xFF>(mq);
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            s[u] = HAS_MASK ? fmaf(s[u], scale, mk[u]) : s[u] * scale;
            if (CHECK && !ok[u]) s[u] = -__builtin_inff();
            tmax = fmaxf(tmax, s[u]);
        }
        const float alpha = softmax_exp<FAST>(m - tmax);
        m = tmax;
        l *= alpha;
#pragma unroll
        for (int e = 0; e < EPL; ++e) o[e] *= alpha;
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            if (CHECK && !ok[u]) continue;
            const float pr = softmax_exp<FAST>(s[u] - m);
            l += pr;
#pragma unroll
            for (int c = 0; c < CPL; ++c)
#pragma unroll
                for (int i = 0; i < VEC; ++i)
                    o[c * VEC + i] = fmaf(pr, (float)vv[u][c][i], o[c * VEC + i]);
        }
    };

    // (Issuing the first tile before q is fetched and rotated was tried: it saves one memory latency
    // per workgroup but keeps 32 more registers live across the prologue, and the spills it causes at
    // 64 VGPRs cost more than the latency saved: 310 -> 331 us at B=64, H=32, ctx=2048.)
    int r = start;
    for (; r + ROWS_PER_TILE <= cache_end; r += ROWS_PER_TILE) {
        issue_tile(r, std::false_type{});
        consume_tile(std::false_type{});
    }
    if (r < cache_end) {
        issue_tile(r, std::true_type{});
        consume_tile(std::true_type{});
    }

    // The new token: RoPE(k_new) and v_new are rounded to the storage type, appended at row P
    // (decoder_kernels.cu:605-610) and attended to from registers.  Every group of wave 0
    // evaluates the row (keeps the wave convergent for the DPP reduction); group 0 applies it.
    if (owns_new && wave == 0) {
        T *kdst = reinterpret_cast<T *>(p.k_cache) + ((size_t)bh * L + P) * D;
        T *vdst = reinterpret_cast<T *>(p.v_cache) + ((size_t)bh * L + P) * D;
        float kf[EPL], vf[EPL];
        float acc = 0.f;
#pragma unroll
        for (int c = 0; c < CPL; ++c) {
            const int e0 = (c * LPR + lig) * VEC;
            if (PADDED && !has_chunk) { // no chunk of the row: nothing to load or store, zeros into the sums
#pragma unroll
                for (int i = 0; i < VEC; ++i) kf[c * VEC + i] = vf[c * VEC + i] = 0.f;
                continue;
            }
            float kx[VEC], vx[VEC];
            load_token_chunk<T, VEC>(p.k_new, (size_t)bh * D + e0, is_i32, inp_scale,
                                     is_i32 ? p.wk_scale + h * D + e0 : nullptr, kx);
            load_token_chunk<T, VEC>(p.v_new, (size_t)bh * D + e0, is_i32, inp_scale,
                                     is_i32 ? p.wv_scale + h * D + e0 : nullptr, vx);
            V kt, vt;
#pragma unroll
            for (int i = 0; i < VEC; i += 4) {
                float4 f = *reinterpret_cast<const float4 *>(freq + e0 + i);
                float r0, r1, r2, r3;
                rope_pair(kx[i], kx[i + 1], f.x, f.y, r0, r1);
                rope_pair(kx[i + 2], kx[i + 3], f.z, f.w, r2, r3);
                kt[i] = to_storage<T>(r0); kt[i + 1] = to_storage<T>(r1);
                kt[i + 2] = to_storage<T>(r2); kt[i + 3] = to_storage<T>(r3);
            }
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
                vt[i] = to_storage<T>(vx[i]);
                kf[c * VEC + i] = (float)kt[i];
                vf[c * VEC + i] = (float)vt[i];
                acc = fmaf(kf[c * VEC + i], qr[c * VEC + i], acc);
            }
            if (g == 0) {
                *reinterpret_cast<V *>(kdst + e0) = kt;
                *reinterpret_cast<V *>(vdst + e0) = vt;
            }
        }
        acc = group_sum<LPR>(acc);
        if (g == 0) {
            const float mk = HAS_MASK ? (FAST ? mrow[P] * kLog2e : mrow[P]) : 0.f;
            const float s = fmaf(acc, scale, mk);
            const float m_new = fmaxf(m, s);
            const float alpha = softmax_exp<FAST>(m - m_new);
            const float pr = softmax_exp<FAST>(s - m_new);
            m = m_new;
            l = fmaf(l, alpha, pr);
#pragma unroll
            for (int e = 0; e < EPL; ++e) o[e] = fmaf(o[e], alpha, pr * vf[e]);
        }
    }

    // Merge the lane-groups of the workgroup.
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
        const int e0 = (c * LPR + lig) * VEC;
        if (PADDED && !has_chunk) continue;
#pragma unroll
        for (int i = 0; i < VEC; i += 4)
            *reinterpret_cast<float4 *>(&s_o[group][e0 + i]) =
                make_float4(o[c * VEC + i], o[c * VEC + i + 1], o[c * VEC + i + 2], o[c * VEC + i + 3]);
    }
    if (lig == 0) {
        s_m[group] = m;
        s_l[group] = l;
    }
    __syncthreads();

    for (int d = tid; d < D; d += WAVES * 64) {
        float M = floor_m;
#pragma unroll
        for (int k = 0; k < GROUPS; ++k) M = fmaxf(M, s_m[k]);
        float Lsum = 0.f, O = 0.f;
#pragma unroll
        for (int k = 0; k < GROUPS; ++k) {
            const float w = softmax_exp<FAST>(s_m[k] - M);
            Lsum = fmaf(s_l[k], w, Lsum);
            O = fmaf(s_o[k][d], w, O);
        }
        if (p.direct) {
            p.out[(size_t)bh * D + d] = O / Lsum; // p = e / sum (decoder_kernels.cu:833)
        } else {
            const size_t slot = (size_t)bh * p.split_cap + split;
            store_partial<FUSED>(p.part_o + slot * D + d, O);
            if (d == 0) {
                store_partial<FUSED>(p.part_m + slot, M);
                store_partial<FUSED>(p.part_l + slot, Lsum);
            }
        }
    }

    if constexpr (FUSED) {
        if (!p.direct) {
            // Ordering of publish -> count -> merge, step by step:
            //  1. the partial went out through device-coherent stores (sc1: written through to memory that
            //     every XCD sees);
            //  2. every thread waits until the memory system has acknowledged ITS stores (vmcnt counts
            //     stores on this architecture).  A workgroup barrier alone does not: it orders at workgroup
            //     scope only, and the counter below lives in another channel than the partials;
            //  3. the barrier: every thread of the workgroup has passed step 2, so all of the workgroup's
            //     partial is in memory.  Steps 2 + 3 are the release;
            //  4. one thread counts the workgroup in with a device-scope read-modify-write, executed at
            //     the memory side, and waits for the returned value before it writes s_last;
            //  5. the barrier, after which the last workgroup to arrive knows it is the last: every other
            //     workgroup of this (b,h) incremented before it, hence finished steps 1-3 before;
            //  6. its device-coherent (sc1) loads are issued after step 5 and bypass the caches that could
            //     hold stale lines.  Steps 4-6 are the acquire.
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            const int nsp = active_splits(p, P);
            if (tid == 0) {
#ifndef FLATTN_ARRIVAL_ORDER
#define FLATTN_ARRIVAL_ORDER __ATOMIC_RELAXED
#endif
                const int before = __hip_atomic_fetch_add(p.arrivals + bh, 1, FLATTN_ARRIVAL_ORDER, __HIP_MEMORY_SCOPE_AGENT);
                s_last = before == nsp - 1;
                if (before == nsp - 1) // every split has arrived: nobody touches the counter again in this launch
                    __hip_atomic_store(p.arrivals + bh, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            __syncthreads();
            if (s_last) combine_partials<D, true>(p, bh, nsp, tid, s_merge);
        }
    }
}

// ---------------------------------------------------------------- RoPE table producer

// freq_cis[r, 2i] = cos(r * base^(-2i/D)), freq_cis[r, 2i+1] = sin(same); evaluated in double
// and rounded once (the reference uses __powf/__cosf/__sinf, decoding_kernels.cu:100-114).
__global__ void rope_table_kernel(float *table, int rows, int D, double base)
{
    const int half = D >> 1;
    const int64_t n = (int64_t)rows * half;
    for (int64_t t = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; t < n;
         t += (int64_t)gridDim.x * blockDim.x) {
        const int r = (int)(t / half), i = (int)(t % half);
        const double theta = (double)r * pow(base, -2.0 * (double)i / (double)D);
        double sn, cs;
        sincos(theta, &sn, &cs);
        *reinterpret_cast<float2 *>(table + (size_t)r * D + 2 * i) = make_float2((float)cs, (float)sn);
    }
}

} // namespace flattn
