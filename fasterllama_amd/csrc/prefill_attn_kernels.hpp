// Prompt-phase (seq_len > 1) self-attention for gfx950: the dense branch of the same block of
// FasterLLaMA's OpenDecoder::forward (fasterLlama/cuda/open_decoder.cu:138-191, :207-228):
//   RoPE + transpose + cache append     decoder_kernels.cu:425-464, :597-632, :858-884
//   scores = Q K^T  (cublasGemmStridedBatchedEx, open_decoder.cu:181-190)
//   block softmax with mask row start_pos + q  (decoder_kernels.cu:800-835)
//   out = P V       (cublasGemmStridedBatchedEx, open_decoder.cu:218-227)
// Unlike the decode step this is a dense contraction (S x ctx x D per head), so it runs on the
// matrix cores.  FP32 caches: FP32 MFMA (v_mfma_f32_32x32x2_f32) with FP32 operands, which keeps the
// 1e-5 parity bar of the FP32 path.  fp16 caches: fp16 MFMA (v_mfma_f32_32x32x16_f16) with FP32
// accumulation (prefill_attn_f16_kernel).
//
// Kernels:
//   prefill_rope_append_kernel    elementwise: RoPE(k), v -> cache rows start_pos + s (bit-identical
//                                 to the decode step's rows)
//   prefill_mask_classify_kernel  classes of the 32x32 tiles of the additive mask (skip / zero / mixed)
//   prefill_attn_kernel,          flash-attention style: a workgroup owns 128 queries of one (b,h)
//   prefill_attn_f16_kernel       (32 per wave), rotates them as it loads them, and walks the keys
//                                 32 at a time through LDS.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "decode_attn_kernels.hpp"

namespace flattn {

struct PrefillParams {
    const void *q, *k_new, *v_new; // [B,S,H,D] storage dtype, or int32 accumulators
    void *k_cache, *v_cache;       // [B,H,L,D]
    const float *freq_cis;
    const float *attn_mask;
    uint32_t *tile_class; // workspace [ceil(S/128), ceil((start_pos+S)/32)]: mask tile classes of this call, or
    const uint8_t *class_table; // the caller's table over the whole mask (mask_class_table_kernel), row stride class_ld
    int32_t class_ld;
    float *out;   // [B,H,S,D] fp32
    const float *inp_scale, *wq_scale, *wk_scale, *wv_scale;
    int64_t mask_ld;
    int32_t B, H, L, S;
    int32_t start_pos, rope_row;
    float scale;
    int32_t fast_qk; // fp16 kernel: rotated queries as one fp16 value instead of an fp16 pair
};

// ---------------------------------------------------------------- RoPE + transpose + append

// One lane-group (LPR lanes) per token and HPT consecutive heads; grid covers B*S*H/HPT such groups, 256 threads
// per block.  The heads of a group share the token's cos/sin chunk, and all their loads are issued before the
// first value is used, so a lane has 2*HPT independent 16-byte loads in flight.
template <typename T, int D, int HPT>
__global__ __launch_bounds__(256) void prefill_rope_append_kernel(const PrefillParams p)
{
    typedef typename Vec16<T>::type V;
    constexpr int VEC = Vec16<T>::N;
    constexpr int CH = D / VEC;
    constexpr int LPR = lanes_per_row(CH); // a power of two; at size_per_head 96 the last lanes of a group own no chunk
    constexpr int CPL = (CH + LPR - 1) / LPR;
    constexpr int ROWS = 256 / LPR;

    const int HG = p.H / HPT; // head groups per token (the launcher picks HPT so that it divides H)
    const int64_t groups = (int64_t)p.B * p.S * HG;
    const int64_t g = (int64_t)blockIdx.x * ROWS + threadIdx.x / LPR; // index into [B,S,H/HPT]
    if (g >= groups) return;
    const int lig = threadIdx.x % LPR;
    if (LPR * CPL != CH && lig >= CH) return;
    const int h0 = (int)(g % HG) * HPT;
    const int64_t bs = g / HG;
    const int s = (int)(bs % p.S), b = (int)(bs / p.S);
    const int pos = p.start_pos + s;
    const int rope_row = p.rope_row < 0 ? pos : p.rope_row + s;
    const float *freq = p.freq_cis + (size_t)rope_row * D;
    const bool is_i32 = p.inp_scale != nullptr;
    const float inp_scale = is_i32 ? p.inp_scale[bs] : 0.f;

#pragma unroll
    for (int c = 0; c < CPL; ++c) {
        const int e0 = (c * LPR + lig) * VEC;
        float kx[HPT][VEC], vx[HPT][VEC];
        float4 f[VEC / 4];
#pragma unroll
        for (int i = 0; i < VEC; i += 4) f[i / 4] = *reinterpret_cast<const float4 *>(freq + e0 + i);
        if (is_i32) { // uniform: one straight run of loads per input format
#pragma unroll
            for (int hh = 0; hh < HPT; ++hh) {
                const size_t in_off = (size_t)(bs * p.H + h0 + hh) * D + e0;
                load_token_chunk<T, VEC>(p.k_new, in_off, true, inp_scale, p.wk_scale + (h0 + hh) * D + e0, kx[hh]);
                load_token_chunk<T, VEC>(p.v_new, in_off, true, inp_scale, p.wv_scale + (h0 + hh) * D + e0, vx[hh]);
            }
        } else {
            V kraw[HPT], vraw[HPT];
#pragma unroll
            for (int hh = 0; hh < HPT; ++hh) {
                const size_t in_off = (size_t)(bs * p.H + h0 + hh) * D + e0;
                kraw[hh] = *reinterpret_cast<const V *>(reinterpret_cast<const T *>(p.k_new) + in_off);
                vraw[hh] = *reinterpret_cast<const V *>(reinterpret_cast<const T *>(p.v_new) + in_off);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int hh = 0; hh < HPT; ++hh)
#pragma unroll
                for (int i = 0; i < VEC; ++i) { kx[hh][i] = (float)kraw[hh][i]; vx[hh][i] = (float)vraw[hh][i]; }
        }
#pragma unroll
        for (int hh = 0; hh < HPT; ++hh) {
            const size_t bh = (size_t)b * p.H + h0 + hh;
            V kt, vt;
#pragma unroll
            for (int i = 0; i < VEC; i += 4) {
                float r0, r1, r2, r3;
                rope_pair(kx[hh][i], kx[hh][i + 1], f[i / 4].x, f[i / 4].y, r0, r1);
                rope_pair(kx[hh][i + 2], kx[hh][i + 3], f[i / 4].z, f[i / 4].w, r2, r3);
                kt[i] = to_storage<T>(r0); kt[i + 1] = to_storage<T>(r1);
                kt[i + 2] = to_storage<T>(r2); kt[i + 3] = to_storage<T>(r3);
            }
#pragma unroll
            for (int i = 0; i < VEC; ++i) vt[i] = to_storage<T>(vx[hh][i]);
            *reinterpret_cast<V *>(reinterpret_cast<T *>(p.k_cache) + (bh * p.L + pos) * D + e0) = kt;
            *reinterpret_cast<V *>(reinterpret_cast<T *>(p.v_cache) + (bh * p.L + pos) * D + e0) = vt;
        }
    }
}

// ---------------------------------------------------------------- dense attention on MFMA

// RoPE(q) for the head dims one lane of the FP32-MFMA kernels owns — dims d_first + 8c + (0..3) for c < NC — of one
// prompt token, in FP32: the attention kernels rotate their own queries while they load them
// (decoder_kernels.cu:449-458), so the rotated queries never travel through memory.  `token` indexes [B,S],
// `row` is the table row.  The input format (int32 accumulators or not) is branched on ONCE and all loads of a
// batch are issued before the first value is used: with the branch and the use inside the loop over chunks a
// wave waited out one memory round trip per chunk, sixteen in a row at D = 128.
template <typename T, int NC>
__device__ __forceinline__ void rotated_query_lane(const PrefillParams &p, int D, int64_t token, int h, int d_first, int row,
                                                   float (&out)[NC][4])
{
    const size_t q_off = (size_t)(token * p.H + h) * D + d_first;
    const float *freq = p.freq_cis + (size_t)row * D + d_first;
    auto rotate = [&](const float (&x)[4], const float4 &f, float (&o)[4]) __attribute__((always_inline)) {
        rope_pair(x[0], x[1], f.x, f.y, o[0], o[1]);
        rope_pair(x[2], x[3], f.z, f.w, o[2], o[3]);
    };
    if (p.inp_scale != nullptr) {
        const float sc = p.inp_scale[token];
        const int32_t *qi = reinterpret_cast<const int32_t *>(p.q) + q_off;
        const float *w = p.wq_scale + h * D + d_first;
        constexpr int BATCH = NC > 8 ? 8 : NC;
#pragma unroll
        for (int c0 = 0; c0 < NC; c0 += BATCH) {
            int4 a[BATCH];
            float4 ws[BATCH], f[BATCH];
#pragma unroll
            for (int j = 0; j < BATCH; ++j) {
                a[j] = *reinterpret_cast<const int4 *>(qi + 8 * (c0 + j));
                ws[j] = *reinterpret_cast<const float4 *>(w + 8 * (c0 + j));
                f[j] = *reinterpret_cast<const float4 *>(freq + 8 * (c0 + j));
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < BATCH; ++j) { // decoder_kernels.cu:449-452
                const float x[4] = {__fmul_rn(__fmul_rn((float)a[j].x, sc), ws[j].x), __fmul_rn(__fmul_rn((float)a[j].y, sc), ws[j].y),
                                    __fmul_rn(__fmul_rn((float)a[j].z, sc), ws[j].z), __fmul_rn(__fmul_rn((float)a[j].w, sc), ws[j].w)};
                rotate(x, f[j], out[c0 + j]);
            }
        }
    } else {
        typedef T vec4 __attribute__((ext_vector_type(4)));
        const T *qt = reinterpret_cast<const T *>(p.q) + q_off;
        vec4 a[NC];
        float4 f[NC];
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            a[c] = *reinterpret_cast<const vec4 *>(qt + 8 * c);
            f[c] = *reinterpret_cast<const float4 *>(freq + 8 * c);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const float x[4] = {(float)a[c][0], (float)a[c][1], (float)a[c][2], (float)a[c][3]};
            rotate(x, f[c], out[c]);
        }
    }
}

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kPrefillQueriesPerBlock = 128; // 4 waves x 32 queries
constexpr int kPrefillKeysPerStep = 32;
constexpr uint32_t kTileSkip = 0, kTileZero = 1, kTileMixed = 2, kTileDiag = 3; // mask tile classes, see prefill_mask_classify_kernel

// Classes of key tile t for the four 32-query sub-blocks of 128-query block qb, one per byte: from the words
// this call's classify kernel wrote, or from the caller's persistent table over the whole mask (one byte per
// 32-key tile x 32-row block, rows in blocks of 32 from mask row 0; start_pos is a multiple of 32 then).  The
// table keeps the row blocks of one key tile together (byte t * class_ld + row block, class_ld a multiple of 4),
// so the four bytes are one aligned word whenever start_pos is a multiple of 128.
__device__ __forceinline__ uint32_t tile_class_word(const PrefillParams &p, int qb, int t, int NT)
{
    if (p.class_table) {
        const int rb0 = p.start_pos / 32 + 4 * qb;
        const uint8_t *e = p.class_table + (size_t)t * p.class_ld + rb0;
        uint32_t w = 0;
        if ((rb0 & 3) == 0) {
            w = *reinterpret_cast<const uint32_t *>(e);
        } else {
#pragma unroll
            for (int k = 0; k < 4; ++k)
                if (rb0 + k < p.class_ld) w |= (uint32_t)e[k] << (8 * k);
        }
#pragma unroll
        for (int k = 1; k < 4; ++k) // sub-blocks beyond the prompt (their table bytes may be padding): kTileSkip
            if (qb * kPrefillQueriesPerBlock + 32 * k >= p.S) w &= ~(0xffu << (8 * k));
        return w;
    }
    return p.tile_class[(size_t)qb * NT + t];
}

// Workgroup id -> (query block, head).  Consecutive ids go round-robin to the 8 XCDs, each with its
// own L2, and every query block of a (b,h) reads that head's whole K and V: the blocks of one head
// are therefore given consecutive slots of ONE XCD, so they run at the same time, walk the keys in
// step and share each K/V tile through that L2 (with heads fastest, the heads resident on an XCD at
// once need several times its L2 and most tiles come from memory again).  Longest block first
// under a causal mask.
__device__ __forceinline__ void prefill_block_to_tile(int block, int BH, int QB, bool longest_first, int &qb, int &bh)
{
    if (longest_first) { // query blocks in descending order across all heads
        bh = block % BH;
        qb = QB - 1 - block / BH;
    } else if (BH % 8 == 0) {
        const int x = block & 7, j = block >> 3;
        bh = (j / QB) * 8 + x;
        qb = QB - 1 - j % QB;
    } else {
        bh = block % BH;
        qb = QB - 1 - block / BH;
    }
}

// The tiles of [c0, c1) that some wave of the workgroup (256 threads, 128 queries: block qb) needs, in order, as a
// list in LDS: entry = tile << 8 | the four waves' classes (2 bits each).  Returns their number; ends with a
// barrier.  w_first: this thread's class word of tile c0 + tid where the caller has loaded it already.
__device__ __forceinline__ int build_tile_list(const PrefillParams &p, int qb, int c0, int c1, int NT, bool have_first,
                                               uint32_t w_first, uint32_t *s_list, int *s_wave_cnt)
{
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int count = 0;
    for (int base = c0; base < c1; base += 256) {
        const int t = base + tid;
        uint32_t w = 0;
        if (have_first && base == c0) w = w_first;
        else if (t < c1) w = tile_class_word(p, qb, t, NT);
        const bool active = w != 0u;
        const unsigned long long bal = __ballot(active);
        if (lane == 0) s_wave_cnt[wave] = __popcll(bal);
        __syncthreads();
        int off = count;
        for (int k = 0; k < wave; ++k) off += s_wave_cnt[k];
        if (active) {
            const uint32_t packed = (w & 3u) | ((w >> 8) & 3u) << 2 | ((w >> 16) & 3u) << 4 | ((w >> 24) & 3u) << 6;
            s_list[off + __popcll(bal & ((1ull << lane) - 1ull))] = (uint32_t)t << 8 | packed;
        }
        count += s_wave_cnt[0] + s_wave_cnt[1] + s_wave_cnt[2] + s_wave_cnt[3];
        __syncthreads();
    }
    return count;
}
constexpr int kTileListCap = 1024; // tiles per pass over the context (32768 keys); longer contexts take several passes

typedef int int4v __attribute__((ext_vector_type(4)));

// Raw buffer descriptor over `bytes` bytes at base: loads at or beyond the end return zeros.
__device__ __forceinline__ int4v raw_descriptor(const void *base, uint32_t bytes)
{
    const uint64_t a = reinterpret_cast<uint64_t>(base);
    return int4v{(int)(uint32_t)a, (int)(uint32_t)(a >> 32), (int)bytes, 0x00020000};
}

// Two direct loads global -> LDS (buffer_load_dwordx4 ... lds: lane i's 16 bytes land at lds + 16 i; a lane whose
// offset is out of the descriptor's range writes zeros).  Written as assembly on purpose: the compiler treats a
// direct load as a store to LDS that any later LDS read may alias, and as pending work every workgroup barrier
// must drain — it would put `s_waitcnt vmcnt(0)` before such reads and before each barrier, which waits for the
// tile that was requested a moment ago and serialises the pipeline.  The callers wait (s_waitcnt vmcnt(n)) for
// exactly the tile they are about to read.  M0 carries the LDS address; one wait state separates its write from
// the load that uses it; it is the compiler's register elsewhere and is handed back as it was.
__device__ __forceinline__ void direct_load_pair(uint32_t lds_a, uint32_t off_a, const int4v &desc_a, uint32_t lds_b,
                                                 uint32_t off_b, const int4v &desc_b)
{
    uint32_t m0_saved;
    asm volatile("s_mov_b32 %0, m0\n\t"
                 "s_mov_b32 m0, %1\n\ts_nop 0\n\tbuffer_load_dwordx4 %2, %3, 0 offen lds\n\t"
                 "s_mov_b32 m0, %4\n\ts_nop 0\n\tbuffer_load_dwordx4 %5, %6, 0 offen lds\n\t"
                 "s_mov_b32 m0, %0"
                 : "=&s"(m0_saved)
                 : "s"(lds_a), "v"(off_a), "s"(desc_a), "s"(lds_b), "v"(off_b), "s"(desc_b)
                 : "memory");
}

// MFMA operand layouts used below (v_mfma_f32_32x32x2_f32, D += A(32x2) * B(2x32)):
//   A: lane holds A[row = lane % 32][k = lane / 32];  B: lane holds B[k = lane / 32][col = lane % 32];
//   D: register v of a lane holds D[row = 8*(v/4) + 4*(lane/32) + (v%4)][col = lane % 32].
// Scores are formed transposed, S^T = K Q^T (rows = keys, cols = queries), so a lane ends up with
// 16 probabilities of ONE query — exactly the B operand of the second product O^T = V^T P^T:
// no LDS transpose of P, and the softmax row reductions are in-lane plus one cross-half exchange.
// The contraction index of the first product is enumerated as d = 8c + 4*(lane/32) + r
// (c = chunk, r = 0..3) so that each lane fetches its K operand as one 128-bit LDS read.
template <typename T, int D, bool HAS_MASK>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 8))) // two workgroups per compute unit
void prefill_attn_kernel(const PrefillParams p)
{
    typedef typename Vec16<T>::type V;
    constexpr int VEC = Vec16<T>::N;
    constexpr int BN = kPrefillKeysPerStep;
    constexpr int NC = D / 8;
    constexpr int NDT = D / 32;
    constexpr int CPR = D / VEC; // 16-byte chunks per cache row
    static_assert(D % 32 == 0, "head size must be a multiple of 32"); // NC = D / 8 is even: the score chunks go in pairs
    static_assert(std::is_same<T, float>::value, "the FP32-MFMA kernel works on FP32 caches");

    // D >= 64: the key tiles go from global memory straight into LDS, two buffers deep, so the next tile
    // travels while this one is multiplied (128 MFMAs of 64 cycles per wave and tile: the products cover
    // the memory latency with room to spare, and no register is spent on staging).  A direct load lays the
    // lanes' 16-byte chunks down back to back — one instruction is 1 KB: RPI whole rows — so rows cannot
    // be padded against bank conflicts; they are swizzled instead: K keeps chunk c of row r at c ^ (r & 15)
    // (the 16 lanes of a 128-bit read pass, keys r..r+15 at one d, hit 16 different bank groups), V keeps it at
    // c ^ 8 for the rows with bit 2 set (the two key rows of a 32-bit read, four apart, use different halves
    // of the banks).  Each lane applies the swizzle to the GLOBAL address it loads from.
    constexpr bool DMA = D == 64 || D == 128; // (96: rows of 384 bytes do not tile the 1 KB of a direct load; staged path)
    constexpr int ROWB = D * 4;          // bytes per cache row
    constexpr int RPI = DMA ? 1024 / ROWB : 1; // rows per direct load
    constexpr int NI = DMA ? BN / RPI / 4 : 1; // direct loads per wave, tile and matrix
    constexpr uint32_t TILEB = BN * ROWB; // bytes of one K (or V) tile
    constexpr int LDK = D + 4;           // staged path: padded LDS row (floats), rows start 4 banks apart
    constexpr int SMEM_FLOATS = DMA ? 4 * BN * D : 2 * BN * LDK;
    __shared__ __attribute__((aligned(16))) float smem[SMEM_FLOATS];
    float (*sK)[LDK] = reinterpret_cast<float (*)[LDK]>(smem);            // staged path only
    float (*sV)[LDK] = reinterpret_cast<float (*)[LDK]>(smem + BN * LDK); // staged path only
    __shared__ uint32_t s_list[HAS_MASK && DMA ? kTileListCap : 1];
    __shared__ int s_wave_cnt[4];

    const int BH = p.B * p.H;
    int qb, bh;
    prefill_block_to_tile((int)blockIdx.x, BH, (p.S + kPrefillQueriesPerBlock - 1) / kPrefillQueriesPerBlock, HAS_MASK, qb, bh);
    const int S = p.S, P = p.start_pos, L = p.L;
    const int ctx = P + S;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int qi = lane & 31, hf = lane >> 5;
    const int q_row = qb * kPrefillQueriesPerBlock + wave * 32 + qi;
    const bool q_ok = q_row < S;
    const int NTC = (ctx + BN - 1) / BN;
    const T *Kb = reinterpret_cast<const T *>(p.k_cache) + (size_t)bh * L * D;
    const T *Vb = reinterpret_cast<const T *>(p.v_cache) + (size_t)bh * L * D;

    // direct path: requests of one tile (tile t -> buffer buf); rows at or beyond the context arrive as zeros
    const int4v Kdesc = raw_descriptor(Kb, (uint32_t)ctx * (uint32_t)ROWB), Vdesc = raw_descriptor(Vb, (uint32_t)ctx * (uint32_t)ROWB);
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    typedef __attribute__((address_space(3))) float *lds_float_ptr;
    const uint32_t lds_wave = (uint32_t)(uintptr_t)(lds_float_ptr)smem + (uint32_t)(wave_u * NI) * 1024u;
    uint32_t dk_off0 = 0, dv_off0 = 0;
    if constexpr (DMA) {
        const int r0 = wave * NI * RPI + lane / (64 / RPI), pc = lane % (64 / RPI);
        dk_off0 = (uint32_t)(r0 * ROWB + ((pc ^ (r0 & 15)) << 4));
        dv_off0 = (uint32_t)(r0 * ROWB + (pc << 4)); // bit 2 of the row comes from the load's index below
    }
    auto dma = [&](int t, int buf) __attribute__((always_inline)) {
        const uint32_t slab = (uint32_t)t * TILEB; // part of the lane offset: the range check does not see a scalar offset
#pragma unroll
        for (int j = 0; j < NI; ++j) { // rows r0 + j * RPI: the swizzle terms of j touch bits of their own
            const uint32_t k_off = (dk_off0 ^ (uint32_t)(((j * RPI) & 15) << 4)) + (uint32_t)(j * 1024) + slab;
            const uint32_t v_off = (dv_off0 ^ (uint32_t)((((j * RPI) >> 2) & 1) << 7)) + (uint32_t)(j * 1024) + slab;
            const uint32_t k_lds = lds_wave + (uint32_t)buf * 2u * TILEB + (uint32_t)(j * 1024);
            direct_load_pair(k_lds, k_off, Kdesc, k_lds + TILEB, v_off, Vdesc);
        }
    };
    // The tile list of the first pass and its first tile are requested before the queries.
    const int first_c1 = min(kTileListCap, NTC);
    int n_first = first_c1;
    if constexpr (DMA) {
        if constexpr (HAS_MASK) n_first = build_tile_list(p, qb, 0, first_c1, NTC, false, 0u, s_list, s_wave_cnt);
        if (n_first > 0) dma(HAS_MASK ? (int)(__builtin_amdgcn_readfirstlane(s_list[0]) >> 8) : 0, 0);
    }

    float qreg[NC][4];
    {
        const int64_t token = (int64_t)(bh / p.H) * S + (q_ok ? q_row : 0);
        const int row = (p.rope_row < 0 ? P : p.rope_row) + (q_ok ? q_row : 0);
        rotated_query_lane<T, NC>(p, D, token, bh % p.H, 4 * hf, row, qreg);
#pragma unroll
        for (int c = 0; c < NC; ++c)
            if (!q_ok) qreg[c][0] = qreg[c][1] = qreg[c][2] = qreg[c][3] = 0.f;
    }

    floatx16 ot[NDT];
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
        for (int v = 0; v < 16; ++v) ot[dt][v] = 0.f;
    float m = kMaxFloor, l = 0.f;
    const float *mrow = HAS_MASK ? p.attn_mask + (size_t)(P + (q_ok ? q_row : 0)) * p.mask_ld : nullptr;
    const float scale = p.scale;

    // LDS addresses of the operands on the direct path (bytes from the tile buffer's start): the K operand of chunk
    // c is one XOR away from k_swz; the V operand of output tile dt sits in the half of its 256 bytes that dt ^ hf names.
    const uint32_t k_swz = (uint32_t)(qi * ROWB + ((hf ^ (qi & 15)) << 4));
    const uint32_t v_lane = (uint32_t)(4 * hf * ROWB + qi * 4);

    // One key tile (keys k0..k0+31, class tc for this wave) against the wave's 32 queries; the tile's K rows at
    // kt, V rows at vt (staged path: padded rows; direct path: swizzled rows in buffer `buf`).
    auto multiply_tile = [&](int k0, uint32_t tc, const float (&mk)[16], auto direct_tag, int buf) __attribute__((always_inline)) {
        constexpr bool DIRECT = decltype(direct_tag)::value;
        const char *kt = reinterpret_cast<const char *>(smem) + (DIRECT ? (uint32_t)buf * 2u * TILEB : 0u);
        const char *vt = kt + TILEB;
        // S^T tile: 32 keys x 32 queries, contraction over D.  Two accumulators, even and odd chunks, added at the
        // end: each sums D/2 products, so the partial sums stay smaller and the rounding error of a score is
        // about 0.7 of what one sequential chain over D leaves (the scores' error is a relative error of the weights).
        floatx16 st, st1;
#pragma unroll
        for (int v = 0; v < 16; ++v) st[v] = st1[v] = 0.f;
#pragma unroll
        for (int c = 0; c < NC; c += 2) {
            const float4 ka = DIRECT ? *reinterpret_cast<const float4 *>(kt + (k_swz ^ (uint32_t)(c << 5)))
                                     : *reinterpret_cast<const float4 *>(&sK[qi][8 * c + 4 * hf]);
            const float4 kb = DIRECT ? *reinterpret_cast<const float4 *>(kt + (k_swz ^ (uint32_t)((c + 1) << 5)))
                                     : *reinterpret_cast<const float4 *>(&sK[qi][8 * (c + 1) + 4 * hf]);
            st = __builtin_amdgcn_mfma_f32_32x32x2f32(ka.x, qreg[c][0], st, 0, 0, 0);
            st1 = __builtin_amdgcn_mfma_f32_32x32x2f32(kb.x, qreg[c + 1][0], st1, 0, 0, 0);
            st = __builtin_amdgcn_mfma_f32_32x32x2f32(ka.y, qreg[c][1], st, 0, 0, 0);
            st1 = __builtin_amdgcn_mfma_f32_32x32x2f32(kb.y, qreg[c + 1][1], st1, 0, 0, 0);
            st = __builtin_amdgcn_mfma_f32_32x32x2f32(ka.z, qreg[c][2], st, 0, 0, 0);
            st1 = __builtin_amdgcn_mfma_f32_32x32x2f32(kb.z, qreg[c + 1][2], st1, 0, 0, 0);
            st = __builtin_amdgcn_mfma_f32_32x32x2f32(ka.w, qreg[c][3], st, 0, 0, 0);
            st1 = __builtin_amdgcn_mfma_f32_32x32x2f32(kb.w, qreg[c + 1][3], st1, 0, 0, 0);
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) st[v] += st1[v];
        __builtin_amdgcn_sched_barrier(0);

        // softmax update of this lane's query: v = s*scale + mask, floor -1e9 (decoder_kernels.cu:811-820)
        float sc[16];
        float mx = m;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int key = k0 + 8 * (v / 4) + 4 * hf + (v % 4);
            float x = HAS_MASK ? fmaf(st[v], scale, mk[v]) : st[v] * scale;
            if (key >= ctx) x = -__builtin_inff();
            sc[v] = x;
            mx = fmaxf(mx, x);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32)); // the other half-wave holds the other 16 keys of this query
        const float alpha = expf(m - mx);
        m = mx;
        l *= alpha;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
            for (int v = 0; v < 16; ++v) ot[dt][v] *= alpha;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            sc[v] = expf(sc[v] - m);
            l += sc[v];
        }

        // O^T += V^T P^T: contraction over the 32 keys, two per MFMA (key of step t in half hf:
        // 8*(t/4) + 4*hf + (t%4), the key whose probability this lane holds in sc[t]).  The tile's 32 terms are
        // summed in an accumulator of their own and added to the running output once: the running sums, which
        // carry the large partial results, are rounded once per tile instead of once per key.
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) {
            floatx16 part;
#pragma unroll
            for (int v = 0; v < 16; ++v) part[v] = 0.f;
#pragma unroll
            for (int t = 0; t < 16; ++t) {
                const float va = DIRECT ? *reinterpret_cast<const float *>(vt + v_lane + (uint32_t)((((dt & 1) ^ hf) << 7) + (dt >> 1) * 256 +
                                                                                                   (8 * (t / 4) + (t % 4)) * ROWB))
                                        : sV[8 * (t / 4) + 4 * hf + (t % 4)][32 * dt + qi];
                part = __builtin_amdgcn_mfma_f32_32x32x2f32(va, sc[t], part, 0, 0, 0);
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) ot[dt][v] += part[v];
            __builtin_amdgcn_sched_barrier(0); // one output tile at a time: operands hoisted across tiles cost registers the kernel does not have
        }
        (void)tc;
    };
    // mask values of this lane's query, gathered straight from global memory: the FP32-MFMA kernel
    // is matrix-core bound with every register in use, so the gather hides behind the products
    // (staging the tile in LDS, as the fp16 kernel does, costs occupancy here: 1.53 -> 2.09 ms)
    auto gather_mask = [&](int k0, uint32_t tc, float (&mk)[16]) __attribute__((always_inline)) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int key = k0 + 8 * (v / 4) + 4 * hf + (v % 4);
            mk[v] = (HAS_MASK && tc >= kTileMixed && key < ctx) ? mrow[key] : 0.f; // (a DIAG tile is read like a MIXED one here)
        }
    };

    // Mask tile classes (see prefill_mask_classify_kernel): a tile no wave of the workgroup needs is
    // neither loaded nor multiplied, a wave skips the tiles it alone does not need, and the mask is
    // only read where it is not all zero.  Each of these leaves every bit of the result as it is:
    // the dropped terms are exp(v - max) == 0 and fma(s, scale, 0) == s*scale.
    if constexpr (DMA) {
        auto list_entry = [&](int c0, int i) __attribute__((always_inline)) -> uint32_t { // without a mask every tile is needed and every class is ZERO
            if constexpr (HAS_MASK) return s_list[i];
            else return (uint32_t)(c0 + i) << 8 | 0x55u;
        };
        for (int c0 = 0; c0 < NTC; c0 += kTileListCap) {
            const int c1 = min(c0 + kTileListCap, NTC);
            int n = c1 - c0;
            if (c0 == 0) n = n_first; // built, and its first tile requested, above
            else if constexpr (HAS_MASK) n = build_tile_list(p, qb, c0, c1, NTC, false, 0u, s_list, s_wave_cnt); // ends with a barrier
            else __syncthreads();                                                                              // both buffers are free
            if (n == 0) continue;
            uint32_t e0 = __builtin_amdgcn_readfirstlane(list_entry(c0, 0));
            uint32_t e1 = n > 1 ? __builtin_amdgcn_readfirstlane(list_entry(c0, 1)) : 0u;
            uint32_t e2 = n > 2 ? list_entry(c0, 2) : 0u;
            if (c0 > 0) dma((int)(e0 >> 8), 0);
            auto tile_step = [&](int i, auto buf_tag) __attribute__((always_inline)) {
                constexpr int buf = decltype(buf_tag)::value;
                const int k0 = (int)(e0 >> 8) * BN;
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // this wave's part of the tile has landed
                __syncthreads();                                  // all of it is visible; every wave is done with the other buffer
                uint32_t tc = kTileZero;
                if constexpr (HAS_MASK) tc = __builtin_amdgcn_readfirstlane((e0 >> (2 * wave)) & 3u);
                float mk[16];
                gather_mask(k0, tc, mk);
                if (i + 1 < n) dma((int)(e1 >> 8), buf ^ 1);
                if (tc != kTileSkip) multiply_tile(k0, tc, mk, std::integral_constant<bool, true>{}, buf);
                e0 = e1;
                e1 = __builtin_amdgcn_readfirstlane(e2);
                e2 = i + 3 < n ? list_entry(c0, i + 3) : 0u;
            };
            for (int i = 0; i < n; i += 2) {
                tile_step(i, std::integral_constant<int, 0>{});
                if (i + 1 < n) tile_step(i + 1, std::integral_constant<int, 1>{});
            }
        }
    } else {
        uint32_t word_next = HAS_MASK ? tile_class_word(p, qb, 0, NTC) : 0u;
        for (int k0 = 0; k0 < ctx; k0 += BN) {
            uint32_t tc = kTileZero;
            if constexpr (HAS_MASK) {
                const uint32_t word = __builtin_amdgcn_readfirstlane(word_next);
                if (k0 + BN < ctx) word_next = tile_class_word(p, qb, k0 / BN + 1, NTC); // in flight during this tile
                if (word == 0u) continue;
                tc = (word >> (8 * wave)) & 0xffu;
            }
            __syncthreads(); // every wave is done with the previous tile
            for (int idx = tid; idx < BN * CPR; idx += 256) {
                const int r = idx / CPR, cc = idx % CPR;
                const int key = k0 + r;
                float kf[VEC], vf[VEC];
                if (key < ctx) {
                    const V kx = *reinterpret_cast<const V *>(Kb + (size_t)key * D + cc * VEC);
                    const V vx = *reinterpret_cast<const V *>(Vb + (size_t)key * D + cc * VEC);
#pragma unroll
                    for (int i = 0; i < VEC; ++i) { kf[i] = (float)kx[i]; vf[i] = (float)vx[i]; }
                } else { // past the context: zeros, and the scores are forced to -inf below
#pragma unroll
                    for (int i = 0; i < VEC; ++i) { kf[i] = 0.f; vf[i] = 0.f; }
                }
#pragma unroll
                for (int i = 0; i < VEC; i += 4) {
                    *reinterpret_cast<float4 *>(&sK[r][cc * VEC + i]) = make_float4(kf[i], kf[i + 1], kf[i + 2], kf[i + 3]);
                    *reinterpret_cast<float4 *>(&sV[r][cc * VEC + i]) = make_float4(vf[i], vf[i + 1], vf[i + 2], vf[i + 3]);
                }
            }
            float mk[16];
            gather_mask(k0, tc, mk);
            __syncthreads();
            if (tc == kTileSkip) continue; // wave-uniform; the barriers above are this iteration's only ones
            multiply_tile(k0, tc, mk, std::integral_constant<bool, false>{}, 0);
        }
    }

    l += __shfl_xor(l, 32);
    if (q_ok) {
        float *dst = p.out + ((size_t)bh * S + q_row) * D;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                float4 r;
                r.x = ot[dt][4 * g4 + 0] / l; // p = e / sum (decoder_kernels.cu:833)
                r.y = ot[dt][4 * g4 + 1] / l;
                r.z = ot[dt][4 * g4 + 2] / l;
                r.w = ot[dt][4 * g4 + 3] / l;
                *reinterpret_cast<float4 *>(dst + 32 * dt + 8 * g4 + 4 * hf) = r;
            }
    }
}

// ---------------------------------------------------------------- mask tile classes

// The additive mask is caller data, but the masks that occur in practice are piecewise trivial: a
// causal mask is all zero below the diagonal band and all "minus huge" above it.  A small kernel
// classifies every 32-query x 32-key tile of the mask rows this call uses, once per call (the mask
// is shared by all (b,h)), and the attention kernels then
//   SKIP   never touch a tile whose entries are all <= -1e30: with finite K the scores
//          v = s*scale + mask stay below every running maximum (floor -1e9) and exp(v - max) is
//          exactly 0, so the tile contributes exact zeros to the sum and the output — skipping it
//          is bit-identical to evaluating it (decoder_kernels.cu:811-833 arithmetic);
//   ZERO   drop the mask term where all entries are +-0 (fma(s, scale, 0) == s*scale);
//   MIXED  evaluate the general form;
//   DIAG   the diagonal tile of a causal mask, whole inside the prompt and the context: +-0 where the key's
//          place in the tile is at or before the query's, <= -1e30 after it.  The fp16 kernel builds such a
//          tile's term from lane indices (-inf for the masked entries: exp gives the same exact 0, and the
//          tile's own diagonal keeps every row's maximum finite) and never reads the mask under the usual
//          causal mask; the other kernels read it like a MIXED tile.
// One 32-bit word per (128-query block, key tile): byte w is the class of the block's w-th wave.
constexpr float kMaskedBelow = -1e30f;
constexpr float kLazyMax = 8.0f; // base-2 units
constexpr float kPairLogit = 4.0f; // fp16 prompt kernel: scores (after scaling, natural units) above which the query remainders are multiplied in

// Class of a wave's 32 x 32 tile from its lanes' findings (each lane has looked at 16 entries of one column).
__device__ __forceinline__ uint32_t classify_ballots(bool open, bool nonzero, bool diag)
{
    if (__ballot(open) == 0ull) return kTileSkip;
    if (__ballot(nonzero) == 0ull) return kTileZero;
    return __ballot(!diag) == 0ull ? kTileDiag : kTileMixed;
}

// grid = (key tiles, query blocks), block = 256.
__global__ __launch_bounds__(256) void prefill_mask_classify_kernel(const PrefillParams p, int NT)
{
    __shared__ uint32_t s_cls[4];
    const int t = blockIdx.x, qb = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int ctx = p.start_pos + p.S;
    const int q0 = qb * kPrefillQueriesPerBlock + wave * 32;
    uint32_t cls = kTileSkip; // a wave whose queries are all beyond the prompt has nothing to do
    if (q0 < p.S) {
        // entries beyond the prompt or the context repeat the last valid row / column: neutral for both tests
        const int col = min(t * kPrefillKeysPerStep + (lane & 31), ctx - 1);
        uint32_t nonzero = 0;
        bool open = false;
        bool diag = q0 + 32 <= p.S && (t + 1) * kPrefillKeysPerStep <= ctx; // no repeated row or column
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const int q = min(q0 + 2 * j + (lane >> 5), p.S - 1);
            const float v = p.attn_mask[(size_t)(p.start_pos + q) * p.mask_ld + col];
            nonzero |= __float_as_uint(v) << 1; // the sign is shifted out: -0 counts as zero
            open |= !(v <= kMaskedBelow);       // a NaN entry keeps the tile
            diag &= (lane & 31) <= 2 * j + (lane >> 5) ? (__float_as_uint(v) << 1) == 0u : v <= kMaskedBelow;
        }
        cls = classify_ballots(open, nonzero != 0u, diag);
    }
    if (lane == 0) s_cls[wave] = cls;
    __syncthreads();
    if (tid == 0) p.tile_class[(size_t)qb * NT + t] = s_cls[0] | (s_cls[1] << 8) | (s_cls[2] << 16) | (s_cls[3] << 24);
}

// The same classes for a WHOLE mask [rows, cols] (row stride mask_ld), once per mask instead of once per call:
// one byte per (32-key tile, 32-row block) at table[tile * table_ld + row block]; entries past the last row /
// column repeat the last one.  grid = (ceil(cols/32), ceil(rows/32)), block = 64.
__global__ __launch_bounds__(64) void mask_class_table_kernel(const float *mask, int64_t mask_ld, int rows, int cols,
                                                              uint8_t *table, int table_ld)
{
    const int t = blockIdx.x, rb = blockIdx.y, lane = threadIdx.x;
    const int col = min(t * kPrefillKeysPerStep + (lane & 31), cols - 1);
    uint32_t nonzero = 0;
    bool open = false;
    bool diag = rb * 32 + 32 <= rows && (t + 1) * kPrefillKeysPerStep <= cols; // no repeated row or column
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const int r = min(rb * 32 + 2 * j + (lane >> 5), rows - 1);
        const float v = mask[(size_t)r * mask_ld + col];
        nonzero |= __float_as_uint(v) << 1; // the sign is shifted out: -0 counts as zero
        open |= !(v <= kMaskedBelow);       // a NaN entry keeps the tile
        diag &= (lane & 31) <= 2 * j + (lane >> 5) ? (__float_as_uint(v) << 1) == 0u : v <= kMaskedBelow;
    }
    const uint32_t cls = classify_ballots(open, nonzero != 0u, diag);
    if (lane == 0) table[(size_t)t * table_ld + rb] = (uint8_t)cls;
}

// ---------------------------------------------------------------- fp16 caches: fp16 MFMA

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float2v __attribute__((ext_vector_type(2)));

// max over both 32-lane halves of a wave, in every lane: one v_permlane32_swap (the upper half of
// the first operand trades places with the lower half of the second) and one v_max.
__device__ __forceinline__ float cross_half_max(float x)
{
    const unsigned u = __float_as_uint(x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

// ds_read_b64_tr_b16: within each group of 16 lanes, lanes 4j..4j+3 address 16 consecutive halfs of
// matrix row j (j < 4, four halfs per lane) and lane i receives element i of rows 0, 1, 2, 3.
typedef short short4v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ half4 lds_read_tr16(const _Float16 *lds)
{
    typedef short4v __attribute__((address_space(3))) * lds_ptr;
    return __builtin_bit_cast(half4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)lds));
}

__device__ __forceinline__ float max16(const floatx16 &a)
{
    float r = fmaxf(fmaxf(a[0], a[1]), a[2]); // pairs of fmaxf fold into v_max3_f32
#pragma unroll
    for (int v = 3; v < 15; v += 2) r = fmaxf(fmaxf(r, a[v]), a[v + 1]);
    return fmaxf(r, a[15]);
}

// Same algorithm as prefill_attn_kernel for fp16 caches, on v_mfma_f32_32x32x16_f16: K and V tiles
// stay fp16 in LDS, rotated queries and probabilities are rounded to fp16 as MFMA operands, every
// accumulation is FP32 (scores, softmax statistics, output).  The rounding of q and p costs ~1e-4
// absolute on the output, inside the 2e-3 bar of the fp16 path.  The softmax runs in base 2 like the
// fp16 decode kernels.
//
// The matrix cores need 512 cycles per wave and 32x32 tile at D = 128 (768 with the query pair); the
// softmax between the two products runs on the vector ALU of the same SIMD (4 cycles per instruction,
// 8 for v_exp_f32), and two or three waves per SIMD overlap one wave's softmax with another's MFMAs —
// as far as the clock allows: with the whole chip on the matrix cores it drops to 1.7-1.9 GHz, and a
// vector wave beside a matrix wave hides only about half of its time.  Per score the common tile costs: 1/2 v_max3 (maximum over the raw products; the scale is
// positive, so it commutes with max), 1 v_fma (s*scale - m), 1 v_exp, 1/2 v_cvt_pk_f16_f32 and
// 1/2 v_dot2c_f32_f16 (the row sum, taken over the rounded probabilities that are multiplied in).
// The additive mask and the -inf of keys past the context enter as the initial value of the score
// accumulator; the output accumulators are rescaled lazily (kLazyMax).
//
// Data path: K and V tiles (32 keys) pass through LDS, one barrier per tile.  D = 128: loaded straight
// into swizzled LDS rows (buffer_load ... lds), three buffers, two tiles ahead; D = 32 / 64: row-major
// with padded rows, two buffers, the loads of tile t+2 in flight in registers while tile t is multiplied.
// The first product reads K rows as 128-bit operands (S^T = K Q^T).  The second, O^T = V^T P^T, needs eight
// keys of one d per lane: ds_read_b64_tr_b16 delivers exactly that from the row-major tile (within
// 16 lanes, lanes 4j..4j+3 address 16 consecutive halfs of row j; lane i receives element i of rows
// 0..3), so V is never transposed in memory.  Contraction slots of the second product: a lane-half
// hf holds the keys 16u + 4hf + r (r < 4) and 16u + 8 + 4hf + (r - 4) after the first.
//
// With a mask, tiles are processed according to their class (see above): each workgroup compacts the
// tiles some wave of it needs into a list in LDS, and tiles that every wave skips are not even loaded.

template <int D, bool HAS_MASK, bool QSPLIT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 8)))
void prefill_attn_f16_kernel(const PrefillParams p)
{
    // Operand prefetch.  Where the kernel runs two waves per SIMD anyway, all K operands of a tile are read
    // from LDS before the first product is issued (and, with the single fp16 query, the V operands before the
    // softmax), so LDS latency is paid once per tile and not once per pair of matrix instructions.  The
    // unmasked single-query instance is left alone: it fits 168 registers, runs THREE waves per SIMD and
    // loses more from a fourth dozen of registers than it gains (B=8, S=1024: 0.221 ms against 0.240).  The
    // masked single-query instance is the other way round: squeezed into 168 registers without the prefetch
    // it runs three waves per SIMD and is 5-10 % slower than with the prefetch at two.
    constexpr bool PF_KA = HAS_MASK || QSPLIT;
    constexpr bool PF_VA = HAS_MASK && !QSPLIT;
    constexpr int BN = kPrefillKeysPerStep; // 32
    // D = 128: the key tiles go from global memory STRAIGHT into LDS (buffer_load ... lds, 16 bytes per lane): no
    // staging registers, no ds_write, no wait for a load in the middle of the loop.  Such a load lays the 64 lanes'
    // chunks down back to back (1 KB = four 256-byte rows), so rows cannot be padded against bank conflicts;
    // the tiles are swizzled instead — row r keeps its 16-byte chunk c of K at position c ^ (r & 15), and its
    // 32-byte unit u of V at position u ^ (r & 7) — which each lane applies to the GLOBAL address it loads from.
    constexpr bool DMA = D == 128;
    constexpr int NBUF = DMA ? 3 : 2;       // tile buffers: a direct load is issued two tiles ahead
    constexpr int LDK = DMA ? D : D + 8;    // halfs; padded rows start 4 banks apart (128-bit operand reads)
    constexpr int LDV = DMA ? D : (D == 96 ? D + 48 : D + 32); // halfs; padded rows start 16 banks apart (8 rows x 64 bytes per transposing read; 8 banks at D = 96)
    constexpr int NC = D / 16;
    constexpr int NDT = D / 32;
    constexpr int CPR = D / 8; // 16-byte chunks per cache row
    constexpr int LPT = (BN * CPR + 255) / 256; // chunks per thread per tile, for K and for V
    static_assert(D % 32 == 0, "head size must be a multiple of 32");

    constexpr int LDQ = D + 8;              // halfs; the workgroup's rotated queries pass through the tile buffers once
    constexpr int HALF_D = D >= 128 ? 64 : 32; // output columns per epilogue pass
    constexpr int LDO = HALF_D + 4;         // floats; the output block passes through the tile buffers too
    constexpr int TILE_HALFS = NBUF * BN * (LDK + LDV), Q_HALFS = kPrefillQueriesPerBlock * LDQ,
                  O_HALFS = kPrefillQueriesPerBlock * LDO * 2;
    // Padded layout: K tiles, then V tiles; the queries pass through the same bytes before the first tile is
    // stored.  Swizzled layout: tile buffer b = K (8 KB) then V (8 KB) at b * 16 KB, and the queries pass through
    // the bytes BEHIND buffer 0, so that the first tile can be requested before the queries are.
    constexpr int Q_OFF = DMA ? BN * (LDK + LDV) : 0; // halfs
    constexpr int Q_END = Q_OFF + Q_HALFS;
    constexpr int SMEM_HALFS = TILE_HALFS > Q_END ? (TILE_HALFS > O_HALFS ? TILE_HALFS : O_HALFS)
                                                  : (Q_END > O_HALFS ? Q_END : O_HALFS);
    __shared__ __attribute__((aligned(16))) _Float16 smem[SMEM_HALFS];
    _Float16 *const sQ = smem + Q_OFF;
    _Float16 (*sK)[BN][LDK] = reinterpret_cast<_Float16 (*)[BN][LDK]>(smem);                   // padded layout only
    _Float16 (*sV)[BN][LDV] = reinterpret_cast<_Float16 (*)[BN][LDV]>(smem + NBUF * BN * LDK); // padded layout only
    constexpr uint32_t kTileBytes = (uint32_t)(BN * (LDK + LDV) * 2), kVOff = (uint32_t)(BN * LDK * 2); // swizzled layout
    __shared__ uint32_t s_list[HAS_MASK ? kTileListCap : 1];
    __shared__ int s_wave_cnt[4];

    const int BH = p.B * p.H;
    int qb, bh;
    prefill_block_to_tile((int)blockIdx.x, BH, (p.S + kPrefillQueriesPerBlock - 1) / kPrefillQueriesPerBlock, HAS_MASK, qb, bh);
    const int S = p.S, P = p.start_pos, L = p.L;
    const int ctx = P + S;
    const int NT = (ctx + BN - 1) / BN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int qi = lane & 31, hf = lane >> 5;
    const int q_row = qb * kPrefillQueriesPerBlock + wave * 32 + qi;

    // The tiles some wave of this workgroup needs, as a list in LDS (build_tile_list): built once per pass of
    // kTileListCap tiles, so the loop below never chases a class word through memory.
    auto build_list = [&](int c0, int c1, bool have_first, uint32_t w_first) __attribute__((always_inline)) -> int {
        return build_tile_list(p, qb, c0, c1, NT, have_first, w_first, s_list, s_wave_cnt);
    };
    // entry i of the current chunk; without a mask every tile is needed and every class is ZERO
    auto list_entry = [&](int c0, int i) __attribute__((always_inline)) -> uint32_t {
        if constexpr (HAS_MASK) return s_list[i];
        else return (uint32_t)(c0 + i) << 8 | 0x55u;
    };

    const _Float16 *Kb = reinterpret_cast<const _Float16 *>(p.k_cache) + (size_t)bh * L * D;
    const _Float16 *Vb = reinterpret_cast<const _Float16 *>(p.v_cache) + (size_t)bh * L * D;

    // global -> registers (fetch) and registers -> LDS (commit) of one key tile.  Raw buffer loads whose
    // descriptors end at the context's last row: a row at or beyond the context — it may hold anything —
    // arrives as zeros by the hardware's range check, with no branch, and the addresses are one scalar
    // base plus one 32-bit offset per chunk.
    half8 kstage[LPT], vstage[LPT];
    constexpr bool EXACT = (BN * CPR) % 256 == 0; // every thread owns LPT chunks of each matrix
    const __amdgpu_buffer_rsrc_t Kbuf = __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16 *>(Kb), 0, (int)((uint32_t)ctx * (uint32_t)(D * 2)), 0x00020000);
    const __amdgpu_buffer_rsrc_t Vbuf = __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16 *>(Vb), 0, (int)((uint32_t)ctx * (uint32_t)(D * 2)), 0x00020000);
    uint32_t src_off[LPT], k_dst[LPT], v_dst[LPT]; // byte offsets: in a 32-row slab of the cache, in the LDS tiles
#pragma unroll
    for (int j = 0; j < LPT; ++j) {
        const int idx = tid + j * 256;
        const int r = idx / CPR, cc = idx % CPR;
        src_off[j] = (EXACT || idx < BN * CPR) ? (uint32_t)(r * D * 2 + cc * 16) : kLaneOutOfRange;
        k_dst[j] = (uint32_t)((r * LDK + cc * 8) * 2);
        v_dst[j] = (uint32_t)((NBUF * BN * LDK + r * LDV + cc * 8) * 2);
    }
    auto fetch = [&](int t) __attribute__((always_inline)) {
        const uint32_t slab = (uint32_t)t * (uint32_t)(BN * D * 2); // uniform; part of the checked offset
#pragma unroll
        for (int j = 0; j < LPT; ++j) {
            kstage[j] = __builtin_bit_cast(half8, __builtin_amdgcn_raw_buffer_load_b128(Kbuf, src_off[j] + slab, 0, 0));
            vstage[j] = __builtin_bit_cast(half8, __builtin_amdgcn_raw_buffer_load_b128(Vbuf, src_off[j] + slab, 0, 0));
        }
    };
    auto commit = [&](int buf) __attribute__((always_inline)) {
        char *base = reinterpret_cast<char *>(smem);
#pragma unroll
        for (int j = 0; j < LPT; ++j) {
            if (EXACT || tid + j * 256 < BN * CPR) {
                *reinterpret_cast<half8 *>(base + k_dst[j] + (uint32_t)(buf * BN * LDK * 2)) = kstage[j];
                *reinterpret_cast<half8 *>(base + v_dst[j] + (uint32_t)(buf * BN * LDV * 2)) = vstage[j];
            }
        }
    };

    // Direct path.  One instruction moves 1 KB, four rows: lane -> row lane/16, 16-byte position lane%16.  Wave w
    // issues the blocks 2w and 2w+1 of K and of V.  The range check of the descriptor (rows at or beyond the
    // context arrive as zeros: a lane out of range writes 16 zero bytes into LDS, it does not skip its write)
    // applies to the lane offset only, so the tile's slab is added to it.
    uint32_t dk_off[DMA ? 2 : 1], dv_off[DMA ? 2 : 1];
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    if constexpr (DMA) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int r = 8 * wave + 4 * j + (lane >> 4), pc = lane & 15;
            dk_off[j] = (uint32_t)(r * 256 + ((pc ^ (r & 15)) << 4));
            dv_off[j] = (uint32_t)(r * 256 + ((((pc >> 2) ^ (r & 3)) << 2 | (pc & 3)) << 4));
        }
    }
    // (direct_load_pair: assembly, because the compiler would wait for every direct load in flight before each LDS
    // read that might alias it and before each barrier.)  The loop below waits for exactly the tile it is about to
    // read (s_waitcnt vmcnt(4): the newer tile's four loads may stay in flight) before its barrier.
    const int4v Kdesc = raw_descriptor(Kb, (uint32_t)ctx * (uint32_t)(D * 2)), Vdesc = raw_descriptor(Vb, (uint32_t)ctx * (uint32_t)(D * 2));
    typedef __attribute__((address_space(3))) _Float16 *lds_half_ptr;
    const uint32_t lds_tiles = (uint32_t)(uintptr_t)(lds_half_ptr)smem + (uint32_t)wave_u * 2048u; // this wave's blocks
    auto dma = [&](int t, int buf) __attribute__((always_inline)) {
        const uint32_t slab = (uint32_t)t * (uint32_t)(BN * D * 2);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint32_t k_lds = lds_tiles + (uint32_t)buf * kTileBytes + (uint32_t)(j * 1024);
            direct_load_pair(k_lds, dk_off[DMA ? j : 0] + slab, Kdesc, k_lds + kVOff, dv_off[DMA ? j : 0] + slab, Vdesc);
        }
    };
    // LDS addresses of the operands.  Padded layout: plain rows.  Swizzled layout: K chunk 2c+hf of row qi sits
    // at chunk (2c+hf) ^ (qi & 15) — one XOR with a constant per read — and the 64-byte unit dt of a V row at
    // unit dt ^ (row & 3); the rows a lane reads differ by multiples of 8, which leaves row & 3 alone.
    const uint32_t k_swz = (uint32_t)(qi * 256 + (((2 * 0 + hf) ^ (qi & 15)) << 4));
    auto k_operand = [&](int buf, int c) __attribute__((always_inline)) -> half8 {
        if constexpr (DMA) return *reinterpret_cast<const half8 *>(reinterpret_cast<const char *>(smem) + (uint32_t)buf * kTileBytes + (k_swz ^ (uint32_t)(c << 5)));
        else return *reinterpret_cast<const half8 *>(&sK[buf][qi][16 * c + 8 * hf]);
    };

    // The class words of the first chunk, key tile 0 and the queries are requested together, so that they
    // travel at the same time instead of one memory round trip after the other.  Tile 0 is a guess at the first
    // listed tile (right without a mask and under every causal mask); the list is built after the queries are
    // in, and a workgroup whose list starts elsewhere requests that tile then.
    const int first_c1 = min(kTileListCap, NT);
    if constexpr (DMA) dma(0, 0);
    else fetch(0);
    uint32_t w_first = 0;
    if constexpr (HAS_MASK) {
        if (tid < first_c1) w_first = tile_class_word(p, qb, tid, NT);
    }

    // Rotated queries.  Every wave loads and rotates ITS OWN 32 queries cooperatively (CPR lanes per row, so the
    // [B,S,H,D] rows are read whole; reading them per lane instead — 32 rows a wave, 16 bytes a lane — keeps the
    // texture units busy for longer than ten key tiles take), rounds them once to fp16 as MFMA operands and turns
    // them into the operand layout through its own slice of LDS: no workgroup barrier on the way.
    half8 qreg[NC];
    half8 qlo[QSPLIT ? NC : 1]; // remainders q - fp16(q): the first product runs on the pair, see below
    {
        const int b = bh / p.H, h = bh % p.H;
        const int row0 = p.rope_row < 0 ? P : p.rope_row;
        constexpr int QPL = 32 * CPR / 64;  // 16-byte chunks per lane
        // Rows of a power-of-two number of chunks: a lane keeps its column chunk over all its rows (RPI rows per
        // load instruction).  Otherwise (size_per_head 96: 12 chunks) the wave's 32 * CPR chunks are dealt out
        // in order, lane + 64 j, and row and column change with j.
        constexpr bool FIXED_COL = 64 % CPR == 0;
        constexpr int RPI = FIXED_COL ? 64 / CPR : 1; // query rows per load instruction
        static_assert((32 * CPR) % 64 == 0, "every lane owns the same number of query chunks");
        auto q_rl = [&](int j) __attribute__((always_inline)) -> int { return FIXED_COL ? lane / CPR + j * RPI : (lane + 64 * j) / CPR; };
        auto q_cc = [&](int j) __attribute__((always_inline)) -> int { return FIXED_COL ? lane % CPR : (lane + 64 * j) % CPR; };
        const int q_first = qb * kPrefillQueriesPerBlock + wave * 32;
        _Float16 *const sq = sQ + wave * 32 * LDQ;
        float x[QPL][8];
        // All loads of a batch are issued before the first value is used (rows past the prompt read the
        // prompt's last row and are zeroed afterwards): left to the compiler, or with the loads under a branch,
        // a wave waits for one chunk before it requests the next — up to eight memory round trips in a row.
        auto load_queries = [&](auto i32_tag) __attribute__((always_inline)) {
            constexpr bool I32 = decltype(i32_tag)::value != 0;
            constexpr int BATCH = I32 && QPL > 1 ? QPL / 2 : QPL; // int32 accumulators: twice the registers
            float4 w[FIXED_COL ? 1 : BATCH][2];
            if constexpr (I32 && FIXED_COL) {
                w[0][0] = *reinterpret_cast<const float4 *>(p.wq_scale + h * D + q_cc(0) * 8);
                w[0][1] = *reinterpret_cast<const float4 *>(p.wq_scale + h * D + q_cc(0) * 8 + 4);
            }
#pragma unroll
            for (int j0 = 0; j0 < QPL; j0 += BATCH) {
                half8 rh[I32 ? 1 : BATCH];
                int4 ri[I32 ? BATCH : 1][2];
                float sc[I32 ? BATCH : 1];
                float4 rf[BATCH][2];
#pragma unroll
                for (int jj = 0; jj < BATCH; ++jj) {
                    const int cc = q_cc(j0 + jj);
                    const int q = min(q_first + q_rl(j0 + jj), S - 1);
                    const int64_t token = (int64_t)b * S + q;
                    const size_t off = (size_t)(token * p.H + h) * D + cc * 8;
                    if constexpr (I32) {
                        const int4 *src = reinterpret_cast<const int4 *>(reinterpret_cast<const int32_t *>(p.q) + off);
                        ri[jj][0] = src[0];
                        ri[jj][1] = src[1];
                        sc[jj] = p.inp_scale[token];
                        if constexpr (!FIXED_COL) {
                            w[jj][0] = *reinterpret_cast<const float4 *>(p.wq_scale + h * D + cc * 8);
                            w[jj][1] = *reinterpret_cast<const float4 *>(p.wq_scale + h * D + cc * 8 + 4);
                        }
                    } else {
                        rh[jj] = *reinterpret_cast<const half8 *>(reinterpret_cast<const _Float16 *>(p.q) + off);
                    }
                    const float4 *fr = reinterpret_cast<const float4 *>(p.freq_cis + (size_t)(row0 + q) * D + cc * 8);
                    rf[jj][0] = fr[0];
                    rf[jj][1] = fr[1];
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int jj = 0; jj < BATCH; ++jj) {
                    float v[8];
                    if constexpr (I32) { // decoder_kernels.cu:449-452
                        const float4 *wj = w[FIXED_COL ? 0 : jj];
                        const int a[8] = {ri[jj][0].x, ri[jj][0].y, ri[jj][0].z, ri[jj][0].w, ri[jj][1].x, ri[jj][1].y, ri[jj][1].z, ri[jj][1].w};
                        const float ws[8] = {wj[0].x, wj[0].y, wj[0].z, wj[0].w, wj[1].x, wj[1].y, wj[1].z, wj[1].w};
#pragma unroll
                        for (int i = 0; i < 8; ++i) v[i] = __fmul_rn(__fmul_rn((float)a[i], sc[jj]), ws[i]);
                    } else {
#pragma unroll
                        for (int i = 0; i < 8; ++i) v[i] = (float)rh[jj][i];
                    }
                    float *o = x[j0 + jj];
                    rope_pair(v[0], v[1], rf[jj][0].x, rf[jj][0].y, o[0], o[1]);
                    rope_pair(v[2], v[3], rf[jj][0].z, rf[jj][0].w, o[2], o[3]);
                    rope_pair(v[4], v[5], rf[jj][1].x, rf[jj][1].y, o[4], o[5]);
                    rope_pair(v[6], v[7], rf[jj][1].z, rf[jj][1].w, o[6], o[7]);
                }
            }
        };
        if (p.inp_scale != nullptr) load_queries(std::integral_constant<int, 1>{});
        else load_queries(std::integral_constant<int, 0>{});
        auto wave_sync = [] { // orders this wave's LDS writes and reads; the slice belongs to the wave alone
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        };
        half8 lo_keep[QSPLIT ? QPL : 1];
#pragma unroll
        for (int j = 0; j < QPL; ++j) {
            const bool valid = q_first + q_rl(j) < S;
            half8 hq;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                hq[i] = valid ? (_Float16)x[j][i] : (_Float16)0;
                if constexpr (QSPLIT) lo_keep[j][i] = valid ? (_Float16)(x[j][i] - (float)hq[i]) : (_Float16)0;
            }
            *reinterpret_cast<half8 *>(sq + q_rl(j) * LDQ + q_cc(j) * 8) = hq;
        }
        wave_sync();
#pragma unroll
        for (int c = 0; c < NC; ++c) qreg[c] = *reinterpret_cast<const half8 *>(sq + qi * LDQ + 16 * c + 8 * hf);
        if constexpr (QSPLIT) {
            wave_sync();
#pragma unroll
            for (int j = 0; j < QPL; ++j) *reinterpret_cast<half8 *>(sq + q_rl(j) * LDQ + q_cc(j) * 8) = lo_keep[j];
            wave_sync();
#pragma unroll
            for (int c = 0; c < NC; ++c) qlo[c] = *reinterpret_cast<const half8 *>(sq + qi * LDQ + 16 * c + 8 * hf);
        }
    }
    // The slices lie in the tile buffers (behind the first one, on the direct path): every wave must be done with
    // its own before a tile is stored there.  With a mask the barriers of the list build see to that.
    if constexpr (!HAS_MASK) __syncthreads();
    int n_first = first_c1;
    if constexpr (HAS_MASK) n_first = build_list(0, first_c1, true, w_first);
    if (n_first > 0) {
        const int t_first = (int)(__builtin_amdgcn_readfirstlane(list_entry(0, 0)) >> 8);
        if (t_first != 0) {
            if constexpr (DMA) { // the guessed tile must have landed, in every wave, before its buffer is written again
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __syncthreads();
                dma(t_first, 0);
            } else {
                fetch(t_first);
            }
        }
    }

    floatx16 ot[NDT];
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
        for (int v = 0; v < 16; ++v) ot[dt][v] = 0.f;
    const float scale = p.scale * kLog2e;
    float m = kMaxFloor * kLog2e, l = 0.f;
    // per-lane source of the transposing V reads: row 4hf + (lane%16)/4, halfs 16*((lane/16)%2) + 4*(lane%4)
    const int vrow = 4 * hf + ((lane & 15) >> 2), vcol = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    const uint32_t v_swz = (uint32_t)(vrow * 256 + ((vrow & 3) << 6) + vcol * 2);
    auto v_operand = [&](int buf, int row0, int dt) __attribute__((always_inline)) -> half4 { // row0: 16u or 16u + 8
        if constexpr (DMA) return lds_read_tr16(reinterpret_cast<const _Float16 *>(reinterpret_cast<const char *>(smem) + (uint32_t)buf * kTileBytes + kVOff + (uint32_t)(row0 * 256) + (v_swz ^ (uint32_t)(dt << 6))));
        else return lds_read_tr16(&sV[buf][row0 + vrow][32 * dt + vcol]);
    };
    const bool mask_vec4 = HAS_MASK && (p.mask_ld & 3) == 0 && (reinterpret_cast<uintptr_t>(p.attn_mask) & 15u) == 0;

    // The rotated queries must have landed before the loop: a wait inside it would also wait for
    // the tile prefetches that are meant to stay in flight.
#pragma unroll
    for (int c = 0; c < NC; ++c) asm volatile("" : "+v"(qreg[c]));

    // Software pipeline over the listed tiles: entry e0's tile in LDS buffer `buf`, e1's in
    // registers, the loads of e2's issued before e0's is multiplied; the list is read three entries
    // ahead so that its LDS latency never stalls the loop.
    for (int c0 = 0; c0 < NT; c0 += kTileListCap) {
        const int c1 = min(c0 + kTileListCap, NT);
        int n = c1 - c0;
        if (c0 == 0) n = n_first; // built, and its first tile requested, in the prologue
        else if constexpr (HAS_MASK) n = build_list(c0, c1, false, 0u); // ends with a barrier: the tile buffers are free again
        else __syncthreads();
        if (n == 0) continue;
        uint32_t e0 = __builtin_amdgcn_readfirstlane(list_entry(c0, 0));
        uint32_t e1 = n > 1 ? __builtin_amdgcn_readfirstlane(list_entry(c0, 1)) : 0u;
        uint32_t e2 = n > 2 ? __builtin_amdgcn_readfirstlane(list_entry(c0, 2)) : 0u;
        uint32_t e3 = n > 3 ? list_entry(c0, 3) : 0u;
        if constexpr (DMA) {
            if (c0 > 0) dma((int)(e0 >> 8), 0);
            if (n > 1) dma((int)(e1 >> 8), 1);
        } else {
            if (c0 > 0) fetch((int)(e0 >> 8));
            commit(0);
            if (n > 1) fetch((int)(e1 >> 8));
        }
        // one tile of the pipeline; the LDS buffer index is a compile-time constant (the loop below is
        // unrolled by two), so every LDS address is a register plus an immediate
        auto tile_step = [&](int i, auto buf_tag) __attribute__((always_inline)) {
            constexpr int buf = decltype(buf_tag)::value;
            const int t = (int)(e0 >> 8);
            if constexpr (DMA) { // this wave's part of tile t has landed; tile t+1 (four loads) may still be in flight
                if (i + 1 < n) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
                else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            }
            __syncthreads(); // tile t is visible; every wave is done with the previous tile's buffer

            // The additive term enters as the initial value of the score accumulator, in units of the
            // raw product: (s + mask/scale)*scale.  Zero for most tiles; the mask entries where the tile
            // is mixed; -inf for keys beyond the context.  The mask is read before the prefetch below is
            // issued: loads return in order, so waiting for it then does not wait for the prefetch.
            const int k0 = t * BN;
            uint32_t tc = kTileZero;
            if constexpr (HAS_MASK) tc = __builtin_amdgcn_readfirstlane((e0 >> (2 * wave)) & 3u);
            const bool special = tc != kTileSkip && (k0 + BN > ctx || tc >= kTileMixed);
            floatx16 st;
            if (special) {
#pragma unroll
                for (int v = 0; v < 16; ++v) st[v] = 0.f;
                if constexpr (HAS_MASK) {
                    if (tc == kTileDiag) { // keys after the query's place in the tile are masked: no memory access
#pragma unroll
                        for (int v = 0; v < 16; ++v) st[v] = 8 * (v / 4) + 4 * hf + (v % 4) > qi ? -__builtin_inff() : 0.f;
                    }
                    if (tc == kTileMixed) {
                        // Mask entries of this lane's query, straight into the score layout (four runs of
                        // four keys).  Only tiles that straddle a mask boundary come here — the diagonal
                        // band of a causal mask — so the gather's poor coalescing does not matter; the
                        // entries of keys beyond the context are overwritten below.
                        const float *mrow = p.attn_mask + (size_t)(P + min(q_row, S - 1)) * p.mask_ld;
                        if (mask_vec4 && k0 + BN <= ctx) {
#pragma unroll
                            for (int g4 = 0; g4 < 4; ++g4) {
                                const float4 x = *reinterpret_cast<const float4 *>(mrow + k0 + 8 * g4 + 4 * hf);
                                st[4 * g4 + 0] = x.x; st[4 * g4 + 1] = x.y; st[4 * g4 + 2] = x.z; st[4 * g4 + 3] = x.w;
                            }
                        } else {
#pragma unroll
                            for (int v = 0; v < 16; ++v) st[v] = mrow[min(k0 + 8 * (v / 4) + 4 * hf + (v % 4), ctx - 1)];
                        }
                    }
                }
            }

            if constexpr (DMA) {
                // The compiler does not see the direct loads, so its wait for the mask entries counts them as
                // landed ones: with the request for tile t+2 in flight behind the mask loads it would wait for
                // that tile as well.  The mask entries are therefore waited for first (tile t+1, requested a
                // tile ago, is all that is older).
                if constexpr (HAS_MASK) {
                    if (special) asm volatile("" : "+v"(st));
                }
                if (i + 2 < n) dma((int)(e2 >> 8), (buf + 2) % NBUF); // the buffer of tile t-1
            } else if (i + 1 < n) {
                commit(buf ^ 1);
                if (i + 2 < n) fetch((int)(e2 >> 8));
            }

            if (tc != kTileSkip) {
                half8 kall[PF_KA ? NC : 1];
                if constexpr (PF_KA) {
#pragma unroll
                    for (int c = 0; c < NC; ++c) kall[c] = k_operand(buf, c);
                    __builtin_amdgcn_sched_barrier(0);
                } else {
                    kall[0] = k_operand(buf, 0);
                }
                const half8 ka0 = kall[0];
                if (special) {
                    // (1 / scale is formed here, where it is needed: as a value kept across the loop it cost the
                    // masked pair instance the registers it does not have)
                    float sc = p.scale;
                    asm volatile("" : "+v"(sc));
                    const float inv_scale = 1.0f / sc;
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        st[v] *= inv_scale;
                        if (k0 + 8 * (v / 4) + 4 * hf + (v % 4) >= ctx) st[v] = -__builtin_inff();
                    }
                    st = __builtin_amdgcn_mfma_f32_32x32x16_f16(ka0, qreg[0], st, 0, 0, 0);
                } else {
                    floatx16 zero;
#pragma unroll
                    for (int v = 0; v < 16; ++v) zero[v] = 0.f;
                    st = __builtin_amdgcn_mfma_f32_32x32x16_f16(ka0, qreg[0], zero, 0, 0, 0); // the literal 0 operand
                }
#pragma unroll
                for (int c = 1; c < NC; ++c) {
                    const half8 ka = PF_KA ? kall[PF_KA ? c : 0] : k_operand(buf, c);
                    st = __builtin_amdgcn_mfma_f32_32x32x16_f16(ka, qreg[c], st, 0, 0, 0);
                }
                half4 vlo[PF_VA ? NDT : 1][2], vhi[PF_VA ? NDT : 1][2];
                if constexpr (PF_VA) {
#pragma unroll
                    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                        for (int u = 0; u < 2; ++u) {
                            vlo[dt][u] = v_operand(buf, 16 * u, dt);
                            vhi[dt][u] = v_operand(buf, 16 * u + 8, dt);
                        }
                    __builtin_amdgcn_sched_barrier(0);
                }
                // Without the full prefetch the V operands are read one output tile ahead of the products that
                // use them, and the first set before the softmax: left to itself the compiler reads each pair
                // right before its product, and every product waits out an LDS round trip.
                half4 vst[2][4];
                auto v_stage = [&](int stage, int dt) __attribute__((always_inline)) {
#pragma unroll
                    for (int u = 0; u < 2; ++u) {
                        vst[stage][2 * u] = v_operand(buf, 16 * u, dt);
                        vst[stage][2 * u + 1] = v_operand(buf, 16 * u + 8, dt);
                    }
                };
                if constexpr (!PF_VA) {
                    v_stage(0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                }
                // With QSPLIT the K operands also multiply the queries' remainders q - fp16(q): the pair carries
                // 22 significant bits, so the scores keep FP32-level accuracy at any magnitude (a single fp16
                // query leaves about |s| * 2^-12 of error in a score s).  The remainder product is additive, so it
                // is issued only where it can matter: when the largest score of some query in the wave's tile
                // exceeds kPairLogit in magnitude after scaling (wave-uniform test on the maximum the softmax needs
                // anyway; a NaN, or a query whose keys are all masked, takes the full path).  A score s below its
                // query's maximum M enters the output with weight w = e^(s - M) <= 1 and relative error |s| * 2^-12;
                // with |M| <= kPairLogit that is at most kPairLogit * 2^-12 ~ 1e-3 of a weight at the very worst
                // (for s < -kPairLogit, |s| * e^(s - M) <= |s| * e^(s + kPairLogit) <= kPairLogit) and ~1.5e-4
                // typically, the size of the rounding of the weights to fp16 that every tile carries anyway.
                float mxq = cross_half_max(max16(st)); // raw units
                if constexpr (QSPLIT) {
                    if (__ballot(!(fabsf(mxq * scale) <= kPairLogit * kLog2e)) != 0ull) { // (scale carries log2 e)
#pragma unroll
                        for (int c = 0; c < NC; ++c) st = __builtin_amdgcn_mfma_f32_32x32x16_f16(kall[PF_KA ? c : 0], qlo[c], st, 0, 0, 0);
                        mxq = cross_half_max(max16(st));
                    }
                }

                // Softmax update of this lane's query (decoder_kernels.cu:811-833 in base 2).  The reference
                // maximum m may lag the true running maximum by up to kLazyMax (weights up to 2^kLazyMax,
                // well inside fp16 and exact in the final ratio): with 32 queries per wave some maximum
                // moves in almost every tile, and rescaling 64 accumulators each time would cost as much
                // vector time as the softmax itself.
                const float mx = fmaxf(m, mxq * scale);
                if (__ballot(mx > m + kLazyMax) != 0ull) { // wave-uniform
                    const float alpha = __builtin_amdgcn_exp2f(m - mx);
                    m = mx;
                    l *= alpha;
#pragma unroll
                    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                        for (int v = 0; v < 16; ++v) ot[dt][v] *= alpha;
                }
                const float nm = -m;
                half8 pr[2];
#pragma unroll
                for (int v = 0; v < 16; v += 2) {
                    float2v e;
                    e[0] = __builtin_amdgcn_exp2f(fmaf(st[v], scale, nm));
                    e[1] = __builtin_amdgcn_exp2f(fmaf(st[v + 1], scale, nm));
                    const half2v h = __builtin_convertvector(e, half2v);
                    pr[v / 8][v % 8] = h[0];
                    pr[v / 8][v % 8 + 1] = h[1];
                    l = __builtin_amdgcn_fdot2(h, half2v{(_Float16)1, (_Float16)1}, l, false); // the weights actually multiplied in
                }

                // O^T += V^T P^T, 16 keys per MFMA
#pragma unroll
                for (int dt = 0; dt < NDT; ++dt) {
                    if constexpr (!PF_VA) {
                        if (dt + 1 < NDT) v_stage((dt + 1) & 1, dt + 1);
                        __builtin_amdgcn_sched_barrier(0);
                    }
#pragma unroll
                    for (int u = 0; u < 2; ++u) {
                        const half4 lo = PF_VA ? vlo[PF_VA ? dt : 0][u] : vst[dt & 1][2 * u];
                        const half4 hi = PF_VA ? vhi[PF_VA ? dt : 0][u] : vst[dt & 1][2 * u + 1];
                        half8 va;
                        va[0] = lo[0]; va[1] = lo[1]; va[2] = lo[2]; va[3] = lo[3];
                        va[4] = hi[0]; va[5] = hi[1]; va[6] = hi[2]; va[7] = hi[3];
                        ot[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(va, pr[u], ot[dt], 0, 0, 0);
                    }
                    if constexpr (!PF_VA) __builtin_amdgcn_sched_barrier(0);
                }
            }

            e0 = e1;
            e1 = e2;
            e2 = __builtin_amdgcn_readfirstlane(e3);
            e3 = i + 4 < n ? list_entry(c0, i + 4) : 0u;
        };
        if constexpr (DMA) {
            for (int i = 0; i < n; i += 3) {
                tile_step(i, std::integral_constant<int, 0>{});
                if (i + 1 < n) tile_step(i + 1, std::integral_constant<int, 1>{});
                if (i + 2 < n) tile_step(i + 2, std::integral_constant<int, 2>{});
            }
        } else {
            for (int i = 0; i < n; i += 2) {
                tile_step(i, std::integral_constant<int, 0>{});
                if (i + 1 < n) tile_step(i + 1, std::integral_constant<int, 1>{});
            }
        }
    }

    // Epilogue: p = e / sum (decoder_kernels.cu:833) as one reciprocal and 64 products per lane (the
    // quotient differs from a true division by an ulp, far inside the fp16 path's tolerance; a fully
    // masked row still gives 0 * inf = NaN).  The lane's values are 16-byte pieces of 32 different
    // output rows; each wave turns its 32 x D block through its own slice of the tile buffers so that
    // the global stores are whole 256-byte row segments.
    l += __shfl_xor(l, 32);
    const float rl = 1.0f / l;
    if constexpr (DMA) asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // (a workgroup with an empty list never waited for its guessed tile)
    __syncthreads(); // every wave is done with the last K/V tile
    {
        // The lane's place is derived again from the thread index here: values computed before the loop and used
        // only after it would have to stay in registers across it (the masked pair instance has none to spare).
        int tid_e = threadIdx.x;
        asm volatile("" : "+v"(tid_e));
        const int lane_e = tid_e & 63, wave_e = tid_e >> 6, qi_e = tid_e & 31, hf_e = (tid_e >> 5) & 1;
        float *so = reinterpret_cast<float *>(smem) + wave_e * 32 * LDO;
        const int q0 = qb * kPrefillQueriesPerBlock + wave_e * 32;
        float *dst0 = p.out + ((size_t)bh * S + q0) * D;
        constexpr int LPRW = HALF_D / 4;               // lanes per row when reading back
        constexpr int RPI = 64 / LPRW;                 // rows per store instruction
#pragma unroll
        for (int pass = 0; pass < D / HALF_D; ++pass) {
#pragma unroll
            for (int dd = 0; dd < HALF_D / 32; ++dd) {
                const int dt = pass * (HALF_D / 32) + dd;
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4)
                    *reinterpret_cast<float4 *>(so + qi_e * LDO + 32 * dd + 8 * g4 + 4 * hf_e) =
                        make_float4(ot[dt][4 * g4 + 0] * rl, ot[dt][4 * g4 + 1] * rl, ot[dt][4 * g4 + 2] * rl,
                                    ot[dt][4 * g4 + 3] * rl);
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int r0 = 0; r0 < 32; r0 += RPI) {
                const int r = r0 + lane_e / LPRW, c4 = lane_e % LPRW;
                const float4 v = *reinterpret_cast<const float4 *>(so + r * LDO + 4 * c4);
                if (q0 + r < S) *reinterpret_cast<float4 *>(dst0 + (size_t)r * D + pass * HALF_D + 4 * c4) = v;
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier(); // the slice is rewritten by the next pass
        }
    }
}

// ---------------------------------------------------------------- head sizes 256 / 512 / 1024

// The reference serves size_per_head 256, 512 and 1024 as well (decoder_kernels.cu:474-551, :588).  With
// such rows the per-wave state of the kernels above (rotated queries and output accumulators of 32 queries)
// no longer fits the register file, so here the HEAD DIMENSION is split across the waves of a workgroup:
// a workgroup of 8 waves owns 32 queries of one (b,h); wave w owns the DW = D/8 dims [w*DW, (w+1)*DW).
//   scores   every wave forms the partial S^T = K[:, its dims] Q^T[its dims, :] of the 32-key tile; the
//            eight partials meet in LDS and every wave adds them up in the same order, so all waves hold
//            the same scores and run the same softmax (decoder_kernels.cu:811-833, expf, true division);
//   output   O^T[its dims, :] += V^T[its dims, :] P^T, in registers until the end.
// FP32 MFMA (v_mfma_f32_32x32x2_f32) for both cache types — fp16 rows are widened on load, their products
// are exact — which keeps the 1e-5 bar of the FP32 path and needs no transposing reads: K and V operands
// come straight from global memory (K: 16 bytes of one row per lane, V: 32 consecutive elements of one
// row per half-wave), nothing is staged.  Mask tile classes as above.  Slower than the kernels for the
// common head sizes by design: correctness first for shapes no LLaMA model uses.
constexpr int kWideWaves = 8;
constexpr int kWideQueriesPerBlock = 32;

template <typename T, int D, bool HAS_MASK>
__global__ __launch_bounds__(kWideWaves * 64) void prefill_attn_wide_kernel(const PrefillParams p)
{
    constexpr int BN = kPrefillKeysPerStep;
    constexpr int DW = D / kWideWaves; // dims per wave: 32, 64 or 128
    constexpr int NC = DW / 8, NDT = DW / 32;
    static_assert(DW % 32 == 0, "each wave owns whole 32-column output tiles");

    __shared__ float s_part[2][kWideWaves][16][64]; // partial score tiles of two consecutive key tiles

    const int S = p.S, P = p.start_pos, L = p.L;
    const int ctx = P + S;
    const int QB = (S + kWideQueriesPerBlock - 1) / kWideQueriesPerBlock;
    const int BH = p.B * p.H;
    const int bh = (int)blockIdx.x % BH;
    const int qb = QB - 1 - (int)blockIdx.x / BH; // long query blocks first under a causal mask
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int qi = lane & 31, hf = lane >> 5;
    const int q_row = qb * kWideQueriesPerBlock + qi;
    const bool q_ok = q_row < S;
    const int d_wave = wave * DW;

    float qreg[NC][4];
    {
        const int64_t token = (int64_t)(bh / p.H) * S + (q_ok ? q_row : 0);
        const int row = (p.rope_row < 0 ? P : p.rope_row) + (q_ok ? q_row : 0);
        rotated_query_lane<T, NC>(p, D, token, bh % p.H, d_wave + 4 * hf, row, qreg);
#pragma unroll
        for (int c = 0; c < NC; ++c)
            if (!q_ok) qreg[c][0] = qreg[c][1] = qreg[c][2] = qreg[c][3] = 0.f;
    }

    floatx16 ot[NDT];
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
        for (int v = 0; v < 16; ++v) ot[dt][v] = 0.f;
    float m = kMaxFloor, l = 0.f;
    const float *mrow = HAS_MASK ? p.attn_mask + (size_t)(P + (q_ok ? q_row : 0)) * p.mask_ld : nullptr;
    const T *Kb = reinterpret_cast<const T *>(p.k_cache) + (size_t)bh * L * D;
    const T *Vb = reinterpret_cast<const T *>(p.v_cache) + (size_t)bh * L * D;
    const float scale = p.scale;
    const int NT = (ctx + BN - 1) / BN;
    // class of this 32-query block per key tile: byte (qb % 4) of the word of its 128-query block

    int buf = 0;
    for (int t = 0; t < NT; ++t) {
        uint32_t tc = kTileZero;
        if constexpr (HAS_MASK) {
            tc = (__builtin_amdgcn_readfirstlane(tile_class_word(p, qb / 4, t, NT)) >> (8 * (qb & 3))) & 0xffu;
            if (tc == kTileSkip) continue; // uniform over the workgroup: every wave skips the same tiles
        }
        const int k0 = t * BN;

        // partial S^T over this wave's dims: keys k0 + qi (rows), queries (columns)
        floatx16 st;
#pragma unroll
        for (int v = 0; v < 16; ++v) st[v] = 0.f;
        {
            const int key = k0 + qi;
            const T *krow = Kb + (size_t)(key < ctx ? key : 0) * D + d_wave + 4 * hf;
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                float ka[4];
                if constexpr (std::is_same<T, float>::value) {
                    const float4 x = *reinterpret_cast<const float4 *>(krow + 8 * c);
                    ka[0] = x.x; ka[1] = x.y; ka[2] = x.z; ka[3] = x.w;
                } else {
                    const half4 x = *reinterpret_cast<const half4 *>(krow + 8 * c);
                    ka[0] = (float)x[0]; ka[1] = (float)x[1]; ka[2] = (float)x[2]; ka[3] = (float)x[3];
                }
                if (key >= ctx) ka[0] = ka[1] = ka[2] = ka[3] = 0.f; // rows past the context may hold anything
#pragma unroll
                for (int r = 0; r < 4; ++r) st = __builtin_amdgcn_mfma_f32_32x32x2f32(ka[r], qreg[c][r], st, 0, 0, 0);
            }
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) s_part[buf][wave][v][lane] = st[v];
        __syncthreads(); // the buffer written two tiles ago was read before the previous tile's barrier
        float sc[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            float x = s_part[buf][0][v][lane];
#pragma unroll
            for (int w = 1; w < kWideWaves; ++w) x += s_part[buf][w][v][lane];
            sc[v] = x;
        }
        // v = qk * scale + mask (decoder_kernels.cu:815); fma(s, scale, 0) == s * scale, so tiles whose mask
        // entries are all zero take the short way
        if (HAS_MASK && tc >= kTileMixed) { // (a DIAG tile is read like a MIXED one here)
#pragma unroll
            for (int v = 0; v < 16; ++v) sc[v] = fmaf(sc[v], scale, mrow[min(k0 + 8 * (v / 4) + 4 * hf + (v % 4), ctx - 1)]);
        } else {
#pragma unroll
            for (int v = 0; v < 16; ++v) sc[v] *= scale;
        }
        float mx = m;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            if (k0 + 8 * (v / 4) + 4 * hf + (v % 4) >= ctx) sc[v] = -__builtin_inff();
            mx = fmaxf(mx, sc[v]);
        }
        buf ^= 1;
        mx = fmaxf(mx, __shfl_xor(mx, 32)); // the other half-wave holds the other 16 keys of this query
        const float alpha = expf(m - mx);
        m = mx;
        l *= alpha;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
            for (int v = 0; v < 16; ++v) ot[dt][v] *= alpha;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            sc[v] = expf(sc[v] - m);
            l += sc[v];
        }

        // O^T[this wave's dims] += V^T P^T: two keys per MFMA; step s of half hf is key 8*(s/4) + 4*hf + s%4,
        // the key whose probability this lane holds in sc[s]
#pragma unroll
        for (int s4 = 0; s4 < 16; ++s4) {
            const int key = k0 + 8 * (s4 / 4) + 4 * hf + (s4 % 4);
            const T *vrow = Vb + (size_t)(key < ctx ? key : 0) * D + d_wave + qi;
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt) {
                float va = (float)vrow[32 * dt];
                if (key >= ctx) va = 0.f;
                ot[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(va, sc[s4], ot[dt], 0, 0, 0);
            }
        }
    }

    l += __shfl_xor(l, 32);
    if (q_ok) {
        float *dst = p.out + ((size_t)bh * S + q_row) * D + d_wave;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                float4 r;
                r.x = ot[dt][4 * g4 + 0] / l; // p = e / sum (decoder_kernels.cu:833)
                r.y = ot[dt][4 * g4 + 1] / l;
                r.z = ot[dt][4 * g4 + 2] / l;
                r.w = ot[dt][4 * g4 + 3] / l;
                *reinterpret_cast<float4 *>(dst + 32 * dt + 8 * g4 + 4 * hf) = r;
            }
    }
}

// ---------------------------------------------------------------- INT8 epilogue with transpose

// grid = B*S, block = kQuantThreads.  attn [B,H,S,D] float -> out_q [B,S,H*D] int8, out_scale [B,S]
// (launchAttnQuantizedTransposeKernel, decoder_kernels.cu:1179-1255); S == 1 is the decode case.
// One small workgroup per token, so that a compute unit has eight tokens in flight: the kernel is one memory
// round trip, a reduction and a store per token, and its bandwidth is what is in flight (1024-thread workgroups,
// two per compute unit, reached 3.1 TB/s).
constexpr int kQuantThreads = 256;
__global__ __launch_bounds__(kQuantThreads) void attn_quantize_transpose_kernel(const float *__restrict__ attn,
                                                                                int8_t *__restrict__ out_q,
                                                                                float *__restrict__ out_scale, int H, int S, int D)
{
    constexpr int T = kQuantThreads;
    __shared__ float s_red[T / 64];
    const int bs = blockIdx.x, tid = threadIdx.x;
    const int b = bs / S, s = bs % S;
    const int HD = H * D;
    const float *x = attn + ((size_t)b * H * S + s) * D; // + h * S * D + d
    // A token of up to 8192 values is read ONCE, four consecutive values per lane and trip, and stays in
    // registers between the absmax reduction and the rounding; longer tokens are read twice.
    constexpr int KEEP = 8; // float4 per thread held in registers
    const bool keep = HD <= T * 4 * KEEP && (D & 3) == 0;
    float4 held[KEEP];
    float absmax = kMaxFloor;
    if (keep) {
        // every load is issued before the first value is used: chunks past the token's end re-read its last one
        // (under a branch the compiler waits for each load before it requests the next)
#pragma unroll
        for (int k = 0; k < KEEP; ++k) {
            const int e = min((tid + k * T) * 4, HD - 4);
            held[k] = *reinterpret_cast<const float4 *>(x + (size_t)(e / D) * S * D + e % D);
        }
#pragma unroll
        for (int k = 0; k < KEEP; ++k) {
            if ((tid + k * T) * 4 < HD)
                absmax = fmaxf(fmaxf(absmax, fmaxf(fabsf(held[k].x), fabsf(held[k].y))), fmaxf(fabsf(held[k].z), fabsf(held[k].w)));
        }
    } else {
        for (int e = tid; e < HD; e += T) absmax = fmaxf(absmax, fabsf(x[(size_t)(e / D) * S * D + e % D]));
    }
    absmax = wave_max(absmax);
    if ((tid & 63) == 0) s_red[tid >> 6] = absmax;
    __syncthreads();
    absmax = s_red[0];
#pragma unroll
    for (int w = 1; w < T / 64; ++w) absmax = fmaxf(absmax, s_red[w]);
    if (tid == 0) out_scale[bs] = absmax / 127.0f;
    auto quant = [&](float value) __attribute__((always_inline)) -> int {
        const float v = rintf(__fmul_rn(value, 127.0f) / absmax);
        return (v != v) ? 0 : (int)fminf(fmaxf(v, -128.f), 127.f); // NaN -> 0, saturate
    };
    if (keep) {
#pragma unroll
        for (int k = 0; k < KEEP; ++k) {
            const int e = (tid + k * T) * 4;
            if (e < HD) {
                const uint32_t packed = (uint32_t)(quant(held[k].x) & 0xff) | (uint32_t)(quant(held[k].y) & 0xff) << 8 |
                                        (uint32_t)(quant(held[k].z) & 0xff) << 16 | (uint32_t)(quant(held[k].w) & 0xff) << 24;
                *reinterpret_cast<uint32_t *>(out_q + (size_t)bs * HD + e) = packed;
            }
        }
    } else {
        for (int e = tid; e < HD; e += T)
            out_q[(size_t)bs * HD + e] = (int8_t)quant(x[(size_t)(e / D) * S * D + e % D]);
    }
}

} // namespace flattn
