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
// Two kernels:
//   prefill_rope_append_kernel  elementwise: RoPE(q) -> workspace [B,H,S,D], RoPE(k), v ->
//                               cache rows start_pos + s (bit-identical to the decode step's rows)
//   prefill_attn_kernel         flash-attention style: a workgroup owns 128 queries of one (b,h)
//                               (32 per wave) and walks the keys 32 at a time through LDS.
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
    void *q_rot;  // workspace [B,H,S,D]: fp32 for FP32 caches, fp16 (the MFMA operand type) for fp16 caches
    float *out;   // [B,H,S,D] fp32
    const float *inp_scale, *wq_scale, *wk_scale, *wv_scale;
    int64_t mask_ld;
    int32_t B, H, L, S;
    int32_t start_pos, rope_row;
    float scale;
};

// ---------------------------------------------------------------- RoPE + transpose + append

// One lane-group (LPR lanes) per token-head row; grid covers B*S*H rows, 256 threads per block.
template <typename T, int D>
__global__ __launch_bounds__(256) void prefill_rope_append_kernel(const PrefillParams p)
{
    typedef typename Vec16<T>::type V;
    constexpr int VEC = Vec16<T>::N;
    constexpr int CH = D / VEC;
    constexpr int LPR = CH < 64 ? CH : 64;
    constexpr int CPL = CH / LPR;
    constexpr int ROWS = 256 / LPR;

    const int64_t rows = (int64_t)p.B * p.S * p.H;
    const int64_t row = (int64_t)blockIdx.x * ROWS + threadIdx.x / LPR; // index into [B,S,H]
    if (row >= rows) return;
    const int lig = threadIdx.x % LPR;
    const int h = (int)(row % p.H);
    const int64_t bs = row / p.H;
    const int s = (int)(bs % p.S), b = (int)(bs / p.S);
    const int pos = p.start_pos + s;
    const int rope_row = p.rope_row < 0 ? pos : p.rope_row + s;
    const float *freq = p.freq_cis + (size_t)rope_row * D;
    const bool is_i32 = p.inp_scale != nullptr;
    const float inp_scale = is_i32 ? p.inp_scale[bs] : 0.f;
    const size_t in_off = (size_t)row * D;
    const size_t bh = (size_t)b * p.H + h;
    T *qdst = reinterpret_cast<T *>(p.q_rot) + (bh * p.S + s) * D;
    T *kdst = reinterpret_cast<T *>(p.k_cache) + (bh * p.L + pos) * D;
    T *vdst = reinterpret_cast<T *>(p.v_cache) + (bh * p.L + pos) * D;

#pragma unroll
    for (int c = 0; c < CPL; ++c) {
        const int e0 = (c * LPR + lig) * VEC;
        float qx[VEC], kx[VEC], vx[VEC];
        load_token_chunk<T, VEC>(p.q, in_off + e0, is_i32, inp_scale, is_i32 ? p.wq_scale + h * D + e0 : nullptr, qx);
        load_token_chunk<T, VEC>(p.k_new, in_off + e0, is_i32, inp_scale, is_i32 ? p.wk_scale + h * D + e0 : nullptr, kx);
        load_token_chunk<T, VEC>(p.v_new, in_off + e0, is_i32, inp_scale, is_i32 ? p.wv_scale + h * D + e0 : nullptr, vx);
        V kt, vt, qt;
#pragma unroll
        for (int i = 0; i < VEC; i += 4) {
            const float4 f = *reinterpret_cast<const float4 *>(freq + e0 + i);
            float4 qo;
            rope_pair(qx[i], qx[i + 1], f.x, f.y, qo.x, qo.y);
            rope_pair(qx[i + 2], qx[i + 3], f.z, f.w, qo.z, qo.w);
            qt[i] = (T)qo.x; qt[i + 1] = (T)qo.y; qt[i + 2] = (T)qo.z; qt[i + 3] = (T)qo.w;
            float r0, r1, r2, r3;
            rope_pair(kx[i], kx[i + 1], f.x, f.y, r0, r1);
            rope_pair(kx[i + 2], kx[i + 3], f.z, f.w, r2, r3);
            kt[i] = to_storage<T>(r0); kt[i + 1] = to_storage<T>(r1);
            kt[i + 2] = to_storage<T>(r2); kt[i + 3] = to_storage<T>(r3);
        }
#pragma unroll
        for (int i = 0; i < VEC; ++i) vt[i] = to_storage<T>(vx[i]);
        *reinterpret_cast<V *>(qdst + e0) = qt;
        *reinterpret_cast<V *>(kdst + e0) = kt;
        *reinterpret_cast<V *>(vdst + e0) = vt;
    }
}

// ---------------------------------------------------------------- dense attention on MFMA

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kPrefillQueriesPerBlock = 128; // 4 waves x 32 queries
constexpr int kPrefillKeysPerStep = 32;
constexpr int kMaskTileLd = kPrefillKeysPerStep + 4; // padded: 128-bit reads of 8 consecutive rows hit 32 banks

// Stages the additive-mask tile of a workgroup (128 queries x 32 keys, rows start_pos + q of the
// caller's [*, mask_ld] matrix) in LDS with coalesced loads: 256 cache-line reads per tile, where
// per-lane gathers (each lane a different mask row) cost 4096 and made the texture path the bottleneck
// of the fp16 kernel.  Entries outside the prompt or the context are 0 (their scores are forced to
// -inf or never used).  `mul` pre-scales the mask for the base-2 softmax.
__device__ __forceinline__ void stage_mask_tile(const PrefillParams &p, float (*sM)[kMaskTileLd], int qb, int k0, int ctx,
                                                int tid, float mul)
{
    // thread -> (row r0 + 8j, column c): 32 consecutive lanes read one 128-byte row segment
    const int c = tid & 31, r0 = tid >> 5;
    const int q0 = qb * kPrefillQueriesPerBlock + r0;
    const bool key_ok = k0 + c < ctx;
    const float *src = p.attn_mask + (size_t)(p.start_pos + q0) * p.mask_ld + k0 + c;
    const size_t step = (size_t)8 * p.mask_ld;
    float x[kPrefillQueriesPerBlock / 8];
#pragma unroll
    for (int j = 0; j < kPrefillQueriesPerBlock / 8; ++j) { // all 16 loads in flight together
        x[j] = 0.f;
        if (key_ok && q0 + 8 * j < p.S) x[j] = src[j * step];
    }
#pragma unroll
    for (int j = 0; j < kPrefillQueriesPerBlock / 8; ++j) sM[r0 + 8 * j][c] = x[j] * mul;
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
__global__ __launch_bounds__(256) void prefill_attn_kernel(const PrefillParams p)
{
    typedef typename Vec16<T>::type V;
    constexpr int VEC = Vec16<T>::N;
    constexpr int BN = kPrefillKeysPerStep;
    constexpr int LDK = D + 4; // padded LDS row (floats): rows start 4 banks apart
    constexpr int NC = D / 8;
    constexpr int NDT = D / 32;
    constexpr int CPR = D / VEC; // 16-byte chunks per cache row
    static_assert(D % 32 == 0, "head size must be a multiple of 32");

    __shared__ float sK[BN][LDK];
    __shared__ float sV[BN][LDK];

    const int BH = p.B * p.H;
    const int qb = blockIdx.x / BH, bh = blockIdx.x % BH;
    const int S = p.S, P = p.start_pos, L = p.L;
    const int ctx = P + S;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int qi = lane & 31, hf = lane >> 5;
    const int q_row = qb * kPrefillQueriesPerBlock + wave * 32 + qi;
    const bool q_ok = q_row < S;

    float qreg[NC][4];
    {
        static_assert(std::is_same<T, float>::value, "the FP32-MFMA kernel reads FP32 rotated queries");
        const float *qsrc = reinterpret_cast<const float *>(p.q_rot) + ((size_t)bh * S + (q_ok ? q_row : 0)) * D + 4 * hf;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            float4 t = q_ok ? *reinterpret_cast<const float4 *>(qsrc + 8 * c) : make_float4(0.f, 0.f, 0.f, 0.f);
            qreg[c][0] = t.x; qreg[c][1] = t.y; qreg[c][2] = t.z; qreg[c][3] = t.w;
        }
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

    for (int k0 = 0; k0 < ctx; k0 += BN) {
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
        // mask values of this lane's query, gathered straight from global memory: the FP32-MFMA kernel
        // is matrix-core bound with every register in use, so the gather hides behind the products
        // (staging the tile in LDS, as the fp16 kernel does, costs occupancy here: 1.53 -> 2.09 ms)
        float mk[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int key = k0 + 8 * (v / 4) + 4 * hf + (v % 4);
            mk[v] = (HAS_MASK && key < ctx) ? mrow[key] : 0.f;
        }
        __syncthreads();

        // S^T tile: 32 keys x 32 queries, contraction over D
        floatx16 st;
#pragma unroll
        for (int v = 0; v < 16; ++v) st[v] = 0.f;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const float4 ka = *reinterpret_cast<const float4 *>(&sK[qi][8 * c + 4 * hf]);
            st = __builtin_amdgcn_mfma_f32_32x32x2f32(ka.x, qreg[c][0], st, 0, 0, 0);
            st = __builtin_amdgcn_mfma_f32_32x32x2f32(ka.y, qreg[c][1], st, 0, 0, 0);
            st = __builtin_amdgcn_mfma_f32_32x32x2f32(ka.z, qreg[c][2], st, 0, 0, 0);
            st = __builtin_amdgcn_mfma_f32_32x32x2f32(ka.w, qreg[c][3], st, 0, 0, 0);
        }

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
        // 8*(t/4) + 4*hf + (t%4), the key whose probability this lane holds in sc[t])
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
            for (int t = 0; t < 16; ++t) {
                const float va = sV[8 * (t / 4) + 4 * hf + (t % 4)][32 * dt + qi];
                ot[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(va, sc[t], ot[dt], 0, 0, 0);
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

// ---------------------------------------------------------------- fp16 caches: fp16 MFMA

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));

// Same algorithm as prefill_attn_kernel for fp16 caches, on v_mfma_f32_32x32x16_f16: K and V tiles
// stay fp16 in LDS (V transposed, so a lane fetches the eight keys of one MFMA as two 64-bit reads),
// rotated queries and probabilities are rounded to fp16 as MFMA operands, every accumulation is
// FP32 (scores, softmax statistics, output).  The rounding of q and p costs ~1e-4 absolute on the
// output, inside the 2e-3 bar of the fp16 path.  The softmax runs in base 2 like the fp16 decode
// kernels.  Contraction slots: a lane-half hf supplies eight consecutive slots of each MFMA; for the
// first product they are d = 16c + 8hf + r, for the second the keys this lane holds after the first:
// 16u + 4hf + r (r < 4) and 16u + 8 + 4hf + (r - 4).
// Two waves per SIMD with the next tile prefetched into registers (244 VGPRs) beat three waves per
// SIMD without prefetch (168 VGPRs): 0.48 -> 0.47 ms at B=8, S=1024 and 0.82 -> 0.66 ms at B=1, S=4096.
#ifndef FLATTN_PREFILL_F16_WAVES
#define FLATTN_PREFILL_F16_WAVES 2
#endif
template <int D, bool HAS_MASK>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(FLATTN_PREFILL_F16_WAVES, 8)))
void prefill_attn_f16_kernel(const PrefillParams p)
{
    constexpr int BN = kPrefillKeysPerStep; // 32
    constexpr int LDK = D + 8;              // halfs; rows start 4 banks apart
    constexpr int LDV = BN + 4;             // halfs; 18-dword rows: 16 lanes x 64-bit reads hit 32 distinct banks
    constexpr int NC = D / 16;
    constexpr int NDT = D / 32;
    constexpr int CPR = D / 8; // 16-byte chunks per cache row
    static_assert(D % 32 == 0, "head size must be a multiple of 32");

    __shared__ __attribute__((aligned(16))) _Float16 sK[BN][LDK];
    __shared__ __attribute__((aligned(16))) _Float16 sVt[D][LDV];
    __shared__ float sM[HAS_MASK ? kPrefillQueriesPerBlock : 1][kMaskTileLd];

    const int BH = p.B * p.H;
    const int qb = blockIdx.x / BH, bh = blockIdx.x % BH;
    const int S = p.S, P = p.start_pos, L = p.L;
    const int ctx = P + S;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int qi = lane & 31, hf = lane >> 5;
    const int q_row = qb * kPrefillQueriesPerBlock + wave * 32 + qi;
    const bool q_ok = q_row < S;

    half8 qreg[NC];
    {
        const _Float16 *qsrc = reinterpret_cast<const _Float16 *>(p.q_rot) + ((size_t)bh * S + (q_ok ? q_row : 0)) * D + 8 * hf;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
#pragma unroll
            for (int i = 0; i < 8; ++i) qreg[c][i] = (_Float16)0;
            if (q_ok) qreg[c] = *reinterpret_cast<const half8 *>(qsrc + 16 * c);
        }
    }

    floatx16 ot[NDT];
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
        for (int v = 0; v < 16; ++v) ot[dt][v] = 0.f;
    const float scale = p.scale * kLog2e;
    float m = kMaxFloor * kLog2e, l = 0.f;
    const _Float16 *Kb = reinterpret_cast<const _Float16 *>(p.k_cache) + (size_t)bh * L * D;
    const _Float16 *Vb = reinterpret_cast<const _Float16 *>(p.v_cache) + (size_t)bh * L * D;

    // Tile staging in two halves so that the global loads of tile i+1 fly while tile i is multiplied:
    // fetch (global -> registers: K and V chunks and the mask tile), commit (registers -> LDS).
    constexpr int LPT = (BN * CPR + 255) / 256; // 16-byte chunks per thread per tile, for K and for V
    constexpr int MPT = kPrefillQueriesPerBlock / 8; // mask values per thread per tile
    half8 kstage[LPT], vstage[LPT];
    float mstage[HAS_MASK ? MPT : 1];
    const int mc = tid & 31, mr0 = tid >> 5; // mask tile: 32 consecutive lanes read one 128-byte row segment
    const int mq0 = qb * kPrefillQueriesPerBlock + mr0;
    const float *msrc = HAS_MASK ? p.attn_mask + (size_t)(P + mq0) * p.mask_ld + mc : nullptr;
    const size_t mstep = (size_t)8 * p.mask_ld;

    auto fetch = [&](int k0) {
#pragma unroll
        for (int j = 0; j < LPT; ++j) {
            const int idx = tid + j * 256;
            { // K: chunk index fastest (coalesced rows)
                const int r = idx / CPR, cc = idx % CPR;
#pragma unroll
                for (int i = 0; i < 8; ++i) kstage[j][i] = (_Float16)0;
                if (idx < BN * CPR && k0 + r < ctx)
                    kstage[j] = *reinterpret_cast<const half8 *>(Kb + (size_t)(k0 + r) * D + cc * 8);
            }
            { // V: key index fastest (it is stored transposed)
                const int r = idx % BN, cc = idx / BN;
#pragma unroll
                for (int i = 0; i < 8; ++i) vstage[j][i] = (_Float16)0;
                if (idx < BN * CPR && k0 + r < ctx)
                    vstage[j] = *reinterpret_cast<const half8 *>(Vb + (size_t)(k0 + r) * D + cc * 8);
            }
        }
        if constexpr (HAS_MASK) {
            const bool key_ok = k0 + mc < ctx;
#pragma unroll
            for (int j = 0; j < MPT; ++j) {
                mstage[j] = 0.f;
                if (key_ok && mq0 + 8 * j < S) mstage[j] = msrc[k0 + j * mstep];
            }
        }
    };
    auto commit = [&]() {
#pragma unroll
        for (int j = 0; j < LPT; ++j) {
            const int idx = tid + j * 256;
            if (idx < BN * CPR) {
                *reinterpret_cast<half8 *>(&sK[idx / CPR][(idx % CPR) * 8]) = kstage[j];
                const int r = idx % BN, cc = idx / BN;
#pragma unroll
                for (int i = 0; i < 8; ++i) sVt[cc * 8 + i][r] = vstage[j][i]; // consecutive lanes, consecutive halfs
            }
        }
        if constexpr (HAS_MASK) {
#pragma unroll
            for (int j = 0; j < MPT; ++j) sM[mr0 + 8 * j][mc] = mstage[j] * kLog2e; // pre-scaled for the base-2 softmax
        }
    };

    fetch(0);
    for (int k0 = 0; k0 < ctx; k0 += BN) {
        __syncthreads(); // every wave is done with the previous tile
        commit();
        __syncthreads();
        if (k0 + BN < ctx) fetch(k0 + BN); // in flight during the products below
        float mk[16];
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
            float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
            if constexpr (HAS_MASK) t = *reinterpret_cast<const float4 *>(&sM[wave * 32 + qi][8 * g4 + 4 * hf]);
            mk[4 * g4 + 0] = t.x; mk[4 * g4 + 1] = t.y; mk[4 * g4 + 2] = t.z; mk[4 * g4 + 3] = t.w;
        }

        floatx16 st;
#pragma unroll
        for (int v = 0; v < 16; ++v) st[v] = 0.f;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const half8 ka = *reinterpret_cast<const half8 *>(&sK[qi][16 * c + 8 * hf]);
            st = __builtin_amdgcn_mfma_f32_32x32x16_f16(ka, qreg[c], st, 0, 0, 0);
        }

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
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        if (__ballot(mx != m) != 0ull) { // wave-uniform: once the maxima have settled alpha is exactly 1
            const float alpha = __builtin_amdgcn_exp2f(m - mx);
            m = mx;
            l *= alpha;
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                for (int v = 0; v < 16; ++v) ot[dt][v] *= alpha;
        }
        half8 pr[2];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const _Float16 e = (_Float16)__builtin_amdgcn_exp2f(sc[v] - m);
            pr[v / 8][v % 8] = e;
            l += (float)e; // normalise by the weights actually multiplied in
        }

        // O^T += V^T P^T, 16 keys per MFMA
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const half4 lo = *reinterpret_cast<const half4 *>(&sVt[32 * dt + qi][16 * u + 4 * hf]);
                const half4 hi = *reinterpret_cast<const half4 *>(&sVt[32 * dt + qi][16 * u + 8 + 4 * hf]);
                half8 va;
                va[0] = lo[0]; va[1] = lo[1]; va[2] = lo[2]; va[3] = lo[3];
                va[4] = hi[0]; va[5] = hi[1]; va[6] = hi[2]; va[7] = hi[3];
                ot[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(va, pr[u], ot[dt], 0, 0, 0);
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
                r.x = ot[dt][4 * g4 + 0] / l;
                r.y = ot[dt][4 * g4 + 1] / l;
                r.z = ot[dt][4 * g4 + 2] / l;
                r.w = ot[dt][4 * g4 + 3] / l;
                *reinterpret_cast<float4 *>(dst + 32 * dt + 8 * g4 + 4 * hf) = r;
            }
    }
}

// ---------------------------------------------------------------- INT8 epilogue with transpose

// grid = B*S, block = 1024.  attn [B,H,S,D] float -> out_q [B,S,H*D] int8, out_scale [B,S]
// (launchAttnQuantizedTransposeKernel, decoder_kernels.cu:1179-1255); S == 1 is the decode case.
__global__ __launch_bounds__(1024) void attn_quantize_transpose_kernel(const float *__restrict__ attn,
                                                                       int8_t *__restrict__ out_q,
                                                                       float *__restrict__ out_scale, int H, int S, int D)
{
    __shared__ float s_red[16];
    const int bs = blockIdx.x, tid = threadIdx.x;
    const int b = bs / S, s = bs % S;
    const int HD = H * D;
    const float *x = attn + ((size_t)b * H * S + s) * D; // + h * S * D + d
    float absmax = kMaxFloor;
    for (int e = tid; e < HD; e += 1024) absmax = fmaxf(absmax, fabsf(x[(size_t)(e / D) * S * D + e % D]));
    absmax = wave_max(absmax);
    if ((tid & 63) == 0) s_red[tid >> 6] = absmax;
    __syncthreads();
    absmax = s_red[0];
#pragma unroll
    for (int w = 1; w < 16; ++w) absmax = fmaxf(absmax, s_red[w]);
    if (tid == 0) out_scale[bs] = absmax / 127.0f;
    for (int e = tid; e < HD; e += 1024) {
        const float v = rintf(__fmul_rn(x[(size_t)(e / D) * S * D + e % D], 127.0f) / absmax);
        const int qv = (v != v) ? 0 : (int)fminf(fmaxf(v, -128.f), 127.f); // NaN -> 0, saturate
        out_q[(size_t)bs * HD + e] = (int8_t)qv;
    }
}

} // namespace flattn
