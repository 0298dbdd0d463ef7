/*
 * TEST INFRASTRUCTURE — NOT PRODUCT CODE.
 *
 * Scalar CPU restatement of the decode-step (seq_len == 1) self-attention math of
 * FasterLLaMA's OpenDecoder::forward.  It exists only as the checker for the HIP path
 * (tests, the smoke check) and as the timed CPU baseline of the benchmark.  Nothing in the
 * shipped library links, loads or calls it.
 *
 * Reference lines followed (paths relative to the reference checkout):
 *   RoPE table ............ fasterLlama/cuda/decoding_kernels.cu:100-114
 *   RoPE pairing / sign .... fasterLlama/cuda/decoder_kernels.cu:455-458 (table row: :440)
 *   K/V append offsets ..... fasterLlama/cuda/decoder_kernels.cu:605-610
 *   scores s = K q ......... fasterLlama/cuda/open_decoder.cu:181-190 (prefill witness of the
 *                            intended math) and :194-201 (decode GEMV, rows = start_pos+seq_len)
 *   softmax ................ fasterLlama/cuda/decoder_kernels.cu:806-833, scale from
 *                            fasterLlama/cuda/open_decoder.cu:207-208, mask row start_pos
 *   o = p V ................ fasterLlama/cuda/open_decoder.cu:231-238
 *   output layout .......... fasterLlama/open_decoder.h:61  ([B, H, 1, D] == [B, H*D])
 *   int32 dequant prologue . fasterLlama/cuda/decoder_kernels.cu:449-452, :875-878
 *   int8 quant epilogue .... fasterLlama/cuda/decoder_kernels.cu:1179-1212,
 *                            fasterLlama/cuda/cuda_kernels.cuh:34-41
 *
 * Parity pins (see tests/test_oracle_*.py): closed forms (ctx == 1, identical keys, RoPE row 0,
 * pair-norm and relative-position invariants, hand-computed D == 4 case), an independent
 * numpy/float64 brute force, torch scaled_dot_product_attention on CPU, and committed golden
 * fixtures.  The reference holds no golden vectors for this path and its CUDA sources cannot be
 * built in this image, so no function here is checked against a run of the reference itself.
 *
 * Arithmetic conventions that the HIP kernels share so that the appended cache rows are
 * bit-identical: RoPE is evaluated as  o0 = fma(x0, c, -(x1*s)),  o1 = fma(x1, c, x0*s)
 * (the contraction a CUDA compiler applies to the reference expression), and fp16 storage
 * rounds to nearest-even.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define FL_REF_F32 0
#define FL_REF_F16 1

/* ------------------------------------------------------------------ fp16 <-> fp32, software */

static float half_bits_to_float(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do {
                man <<= 1;
                ++e;
            } while ((man & 0x400u) == 0);
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* round-to-nearest-even, IEEE overflow to inf, gradual underflow */
static uint16_t float_to_half_bits(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) { /* inf / nan */
        if (ax > 0x7f800000u)
            return (uint16_t)(sign | 0x7e00u | ((ax >> 13) & 0x3ffu));
        return (uint16_t)(sign | 0x7c00u);
    }
    if (ax >= 0x477ff000u) /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7c00u);
    if (ax < 0x33000001u) /* <= 2^-25 rounds to zero (tie at 2^-25 goes to even = 0) */
        return sign;
    int32_t e = (int32_t)(ax >> 23) - 127;
    uint32_t man = (ax & 0x7fffffu) | 0x800000u;
    int shift;
    uint32_t base;
    if (e < -14) { /* subnormal half */
        shift = 13 + (-14 - e);
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
        man &= 0x7fffffu;
    }
    uint32_t q = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u)))
        ++q;
    return (uint16_t)(sign | (base + q)); /* mantissa carry walks into the exponent correctly */
}

float fl_ref_half_to_float(uint16_t h) { return half_bits_to_float(h); }
uint16_t fl_ref_float_to_half(float f) { return float_to_half_bits(f); }

static inline float load_elem(const void *p, size_t i, int dtype)
{
    return dtype == FL_REF_F16 ? half_bits_to_float(((const uint16_t *)p)[i]) : ((const float *)p)[i];
}

static inline void store_elem(void *p, size_t i, int dtype, float v)
{
    if (dtype == FL_REF_F16)
        ((uint16_t *)p)[i] = float_to_half_bits(v);
    else
        ((float *)p)[i] = v;
}

/* ------------------------------------------------------------------ RoPE table (row producer) */

/* freq_cis[pos, 2i] = cos(pos * 10000^(-2i/D)), freq_cis[pos, 2i+1] = sin(same)
 * (decoding_kernels.cu:100-114).  The reference evaluates it with fast device intrinsics; the
 * table is an *input* of the attention path, so it is produced here in double and rounded once. */
int fl_ref_freq_cis(float *table, int rows, int D, double base)
{
    if (!table || rows < 0 || D <= 0 || (D & 1))
        return -1;
    for (int pos = 0; pos < rows; ++pos) {
        for (int i = 0; i < D / 2; ++i) {
            double theta = (double)pos * pow(base, -2.0 * (double)i / (double)D);
            table[(size_t)pos * D + 2 * i] = (float)cos(theta);
            table[(size_t)pos * D + 2 * i + 1] = (float)sin(theta);
        }
    }
    return 0;
}

/* ------------------------------------------------------------------ the decode step */

/* rope of one interleaved pair, shared convention with the device code */
static inline void rope_pair(float x0, float x1, float c, float s, float *o0, float *o1)
{
    *o0 = fmaf(x0, c, -(x1 * s));
    *o1 = fmaf(x1, c, x0 * s);
}

/* int32 GEMM accumulator -> float (decoder_kernels.cu:449-452, :875-878):
 *   x = (float)acc * inp_scale[b] * weight_scale[h*D + d], evaluated left to right */
static inline float dequant(int32_t acc, float inp_scale, float w_scale)
{
    return (float)acc * inp_scale * w_scale;
}

typedef struct {
    int dtype, B, H, D, L;
    const void *q, *k_new, *v_new; /* [B,1,H,D] storage dtype, or int32 when q_scale != NULL */
    void *k_cache, *v_cache;       /* [B,H,L,D] storage dtype */
    const float *freq_cis;         /* [rows, D] */
    int rope_row;                  /* >=0: that row for every sequence; <0: row start_pos[b] */
    const float *attn_mask;        /* NULL or base of [*, mask_ld]; row start_pos[b] is added */
    int64_t mask_ld;
    int start_pos;
    const int32_t *start_pos_per_seq; /* NULL or [B] */
    int max_start_pos;                /* with start_pos_per_seq: bound the caller promised, <0 = L-1 */
    float scale;
    float *out; /* [B, H*D] */
    int acc_double;
    /* optional int32 prologue */
    const float *inp_scale;              /* [B] or NULL */
    const float *wq_scale, *wk_scale, *wv_scale; /* [H*D] */
} ref_args;

static void one_head(const ref_args *a, int b, int h, float *scratch)
{
    const int D = a->D, H = a->H, L = a->L, dt = a->dtype;
    const int P = a->start_pos_per_seq ? a->start_pos_per_seq[b] : a->start_pos;
    float *o_row = a->out + ((size_t)b * H + h) * D;
    const int bound = (a->start_pos_per_seq && a->max_start_pos >= 0) ? a->max_start_pos : L - 1;
    /* position outside the cache, or beyond the bound the caller promised for a ragged batch
     * (the HIP library plans its launch for that bound): nothing stored, output poisoned */
    if (P < 0 || P >= L || P > bound) {
        for (int d = 0; d < D; ++d)
            o_row[d] = NAN;
        return;
    }
    const int ctx = P + 1;
    const int row = a->rope_row < 0 ? P : a->rope_row;
    const float *f = a->freq_cis + (size_t)row * D;
    const size_t in_off = ((size_t)b * H + h) * D;
    const size_t cache_row0 = ((size_t)b * H + h) * (size_t)L * D; /* decoder_kernels.cu:606 */
    const size_t new_off = cache_row0 + (size_t)P * D;

    float *qr = scratch;          /* D */
    float *sc = scratch + D;      /* ctx scores / probabilities */

    /* RoPE(q), RoPE(k_new) -> cache row P, v_new -> cache row P */
    for (int i = 0; i < D; i += 2) {
        float q0, q1, k0, k1, v0, v1;
        if (a->inp_scale) {
            const int32_t *qi = (const int32_t *)a->q, *ki = (const int32_t *)a->k_new,
                          *vi = (const int32_t *)a->v_new;
            float s = a->inp_scale[b];
            q0 = dequant(qi[in_off + i], s, a->wq_scale[h * D + i]);
            q1 = dequant(qi[in_off + i + 1], s, a->wq_scale[h * D + i + 1]);
            k0 = dequant(ki[in_off + i], s, a->wk_scale[h * D + i]);
            k1 = dequant(ki[in_off + i + 1], s, a->wk_scale[h * D + i + 1]);
            v0 = dequant(vi[in_off + i], s, a->wv_scale[h * D + i]);
            v1 = dequant(vi[in_off + i + 1], s, a->wv_scale[h * D + i + 1]);
        } else {
            q0 = load_elem(a->q, in_off + i, dt);
            q1 = load_elem(a->q, in_off + i + 1, dt);
            k0 = load_elem(a->k_new, in_off + i, dt);
            k1 = load_elem(a->k_new, in_off + i + 1, dt);
            v0 = load_elem(a->v_new, in_off + i, dt);
            v1 = load_elem(a->v_new, in_off + i + 1, dt);
        }
        float c = f[i], s = f[i + 1], r0, r1;
        rope_pair(q0, q1, c, s, &qr[i], &qr[i + 1]);
        rope_pair(k0, k1, c, s, &r0, &r1);
        store_elem(a->k_cache, new_off + i, dt, r0);
        store_elem(a->k_cache, new_off + i + 1, dt, r1);
        store_elem(a->v_cache, new_off + i, dt, v0);
        store_elem(a->v_cache, new_off + i + 1, dt, v1);
    }

    const float *mrow = a->attn_mask ? a->attn_mask + (size_t)P * (size_t)a->mask_ld : NULL;

    if (!a->acc_double) {
        /* s_j = sum_d K[j,d] q[d];  v_j = s_j*scale + mask_j;  m = max(-1e9, max_j v_j) */
        float m = -1e9f;
        for (int j = 0; j < ctx; ++j) {
            float acc = 0.0f;
            const size_t r = cache_row0 + (size_t)j * D;
            for (int d = 0; d < D; ++d)
                acc += load_elem(a->k_cache, r + d, dt) * qr[d];
            float v = acc * a->scale + (mrow ? mrow[j] : 0.0f);
            sc[j] = v;
            m = fmaxf(m, v);
        }
        float sum = 0.0f;
        for (int j = 0; j < ctx; ++j) {
            float e = expf(sc[j] - m);
            sc[j] = e;
            sum += e;
        }
        for (int j = 0; j < ctx; ++j)
            sc[j] = sc[j] / sum;
        for (int d = 0; d < D; ++d)
            o_row[d] = 0.0f;
        for (int j = 0; j < ctx; ++j) {
            const size_t r = cache_row0 + (size_t)j * D;
            const float p = sc[j];
            for (int d = 0; d < D; ++d)
                o_row[d] += p * load_elem(a->v_cache, r + d, dt);
        }
    } else {
        /* same stored operands, every accumulation and exp in double: the arbiter */
        double *scd = (double *)(scratch + D + ((ctx + 1) & ~1));
        double m = -1e9;
        for (int j = 0; j < ctx; ++j) {
            double acc = 0.0;
            const size_t r = cache_row0 + (size_t)j * D;
            for (int d = 0; d < D; ++d)
                acc += (double)load_elem(a->k_cache, r + d, dt) * (double)qr[d];
            double v = acc * (double)a->scale + (mrow ? (double)mrow[j] : 0.0);
            scd[j] = v;
            if (v > m)
                m = v;
        }
        double sum = 0.0;
        for (int j = 0; j < ctx; ++j) {
            scd[j] = exp(scd[j] - m);
            sum += scd[j];
        }
        for (int d = 0; d < D; ++d) {
            double acc = 0.0;
            for (int j = 0; j < ctx; ++j)
                acc += scd[j] * (double)load_elem(a->v_cache, cache_row0 + (size_t)j * D + d, dt);
            o_row[d] = (float)(acc / sum);
        }
    }
}

static int run(const ref_args *a, int threads)
{
    if (!a->q || !a->k_new || !a->v_new || !a->k_cache || !a->v_cache || !a->freq_cis || !a->out)
        return -1;
    if (a->B <= 0 || a->H <= 0 || a->D <= 0 || (a->D & 1) || a->L <= 0)
        return -3;
    if (a->dtype != FL_REF_F32 && a->dtype != FL_REF_F16)
        return -6;
    if (!a->start_pos_per_seq && (a->start_pos < 0 || a->start_pos >= a->L))
        return -4;
    const int BH = a->B * a->H;
    const size_t per = (size_t)a->D + (size_t)a->L + 2 + 2 * ((size_t)a->L + 2);
    if (threads < 1)
        threads = 1;
#ifdef _OPENMP
    int fail = 0;
#pragma omp parallel num_threads(threads)
    {
        float *scratch = (float *)malloc(per * sizeof(float));
        if (!scratch) {
#pragma omp atomic write
            fail = 1;
        }
#pragma omp for schedule(dynamic, 1)
        for (int bh = 0; bh < BH; ++bh)
            if (scratch)
                one_head(a, bh / a->H, bh % a->H, scratch);
        free(scratch);
    }
    return fail ? -7 : 0;
#else
    (void)threads;
    float *scratch = (float *)malloc(per * sizeof(float));
    if (!scratch)
        return -7;
    for (int bh = 0; bh < BH; ++bh)
        one_head(a, bh / a->H, bh % a->H, scratch);
    free(scratch);
    return 0;
#endif
}

/*
 * One decode step for every (batch, head): RoPE(q, k_new) -> append k/v at row start_pos ->
 * scores over rows [0, start_pos] -> masked softmax -> weighted sum of V rows.
 * With start_pos_per_seq, max_start_pos >= 0 is the bound the caller promises for its entries; a
 * sequence beyond it is handled like one outside the cache.
 * dtype selects the storage type of q/k_new/v_new and of both caches (0 = float, 1 = IEEE half);
 * all arithmetic is float (acc_double == 0) or double (acc_double == 1).
 * Returns 0, or a negative code mirroring the C-ABI of the HIP library.
 */
int fl_ref_decode_attn(int dtype, int B, int H, int D, int L, const void *q, const void *k_new,
                       const void *v_new, void *k_cache, void *v_cache, const float *freq_cis,
                       int rope_row, const float *attn_mask, int64_t mask_ld, int start_pos,
                       const int32_t *start_pos_per_seq, int max_start_pos, float scale, float *out,
                       int acc_double, int threads)
{
    ref_args a;
    memset(&a, 0, sizeof a);
    a.dtype = dtype; a.B = B; a.H = H; a.D = D; a.L = L;
    a.q = q; a.k_new = k_new; a.v_new = v_new; a.k_cache = k_cache; a.v_cache = v_cache;
    a.freq_cis = freq_cis; a.rope_row = rope_row; a.attn_mask = attn_mask; a.mask_ld = mask_ld;
    a.start_pos = start_pos; a.start_pos_per_seq = start_pos_per_seq; a.max_start_pos = max_start_pos;
    a.scale = scale; a.out = out;
    a.acc_double = acc_double;
    return run(&a, threads);
}

/* Same step fed by the int32 accumulators of the INT8 Q/K/V projections plus their scales
 * (decoder_kernels.cu:449-452, :875-878): x = (float)acc * inp_scale[b] * w_scale[h*D+d]. */
int fl_ref_decode_attn_i32(int dtype, int B, int H, int D, int L, const int32_t *q_acc,
                           const int32_t *k_acc, const int32_t *v_acc, const float *inp_scale,
                           const float *wq_scale, const float *wk_scale, const float *wv_scale,
                           void *k_cache, void *v_cache, const float *freq_cis, int rope_row,
                           const float *attn_mask, int64_t mask_ld, int start_pos,
                           const int32_t *start_pos_per_seq, int max_start_pos, float scale, float *out,
                           int acc_double, int threads)
{
    if (!inp_scale || !wq_scale || !wk_scale || !wv_scale)
        return -1;
    ref_args a;
    memset(&a, 0, sizeof a);
    a.dtype = dtype; a.B = B; a.H = H; a.D = D; a.L = L;
    a.q = q_acc; a.k_new = k_acc; a.v_new = v_acc; a.k_cache = k_cache; a.v_cache = v_cache;
    a.freq_cis = freq_cis; a.rope_row = rope_row; a.attn_mask = attn_mask; a.mask_ld = mask_ld;
    a.start_pos = start_pos; a.start_pos_per_seq = start_pos_per_seq; a.max_start_pos = max_start_pos;
    a.scale = scale; a.out = out;
    a.acc_double = acc_double;
    a.inp_scale = inp_scale; a.wq_scale = wq_scale; a.wk_scale = wk_scale; a.wv_scale = wv_scale;
    return run(&a, threads);
}

/* ------------------------------------------------------------------ the prompt phase (seq_len > 1)
 *
 * Restates the seq_len > 1 branch of the same block (open_decoder.cu:138-191, :207-228):
 *   RoPE of every new token with table row (position of the token) (decoder_kernels.cu:440, :455-458),
 *   transpose [B,S,H,D] -> [B,H,S,D] (:461), append at cache rows start_pos + s (:605-610),
 *   scores = Q K^T (open_decoder.cu:181-190), softmax row q with mask row start_pos + q
 *   (decoder_kernels.cu:806-833 with mask_offset = seq_q_id * max_seq_len on top of the
 *   start_pos * total_len_ offset of open_decoder.cu:207), out = P V (open_decoder.cu:218-227),
 *   output layout [B,H,S,D] (open_decoder.h:61).
 * The reference multiplies by the NEW keys only (key_out_buf_), which equals the cache rows
 * [0, S) because its driver always calls the prompt phase with start_pos == 0
 * (decoding_sampling.cu:197-258).  This restatement attends over cache rows [0, start_pos + S),
 * which is the same thing for start_pos == 0 and extends it to a chunked prompt otherwise.
 * With S == 1 it performs exactly the operations of fl_ref_decode_attn, in the same order.
 */
static void prefill_one_head(const ref_args *a, int S, int b, int h, float *scratch)
{
    const int D = a->D, H = a->H, L = a->L, dt = a->dtype, P = a->start_pos;
    const int ctx = P + S;
    const size_t cache_row0 = ((size_t)b * H + h) * (size_t)L * D;
    float *qr = scratch;                 /* S * D rotated queries */
    float *sc = scratch + (size_t)S * D; /* ctx scores */

    for (int s = 0; s < S; ++s) {
        const int row = a->rope_row < 0 ? P + s : a->rope_row + s;
        const float *f = a->freq_cis + (size_t)row * D;
        const size_t in_off = (((size_t)b * S + s) * H + h) * D; /* [B,S,H,D] */
        const size_t new_off = cache_row0 + (size_t)(P + s) * D;
        for (int i = 0; i < D; i += 2) {
            float q0, q1, k0, k1, v0, v1;
            if (a->inp_scale) {
                const int32_t *qi = (const int32_t *)a->q, *ki = (const int32_t *)a->k_new,
                              *vi = (const int32_t *)a->v_new;
                float sc_in = a->inp_scale[(size_t)b * S + s]; /* [B,S] */
                q0 = dequant(qi[in_off + i], sc_in, a->wq_scale[h * D + i]);
                q1 = dequant(qi[in_off + i + 1], sc_in, a->wq_scale[h * D + i + 1]);
                k0 = dequant(ki[in_off + i], sc_in, a->wk_scale[h * D + i]);
                k1 = dequant(ki[in_off + i + 1], sc_in, a->wk_scale[h * D + i + 1]);
                v0 = dequant(vi[in_off + i], sc_in, a->wv_scale[h * D + i]);
                v1 = dequant(vi[in_off + i + 1], sc_in, a->wv_scale[h * D + i + 1]);
            } else {
                q0 = load_elem(a->q, in_off + i, dt);
                q1 = load_elem(a->q, in_off + i + 1, dt);
                k0 = load_elem(a->k_new, in_off + i, dt);
                k1 = load_elem(a->k_new, in_off + i + 1, dt);
                v0 = load_elem(a->v_new, in_off + i, dt);
                v1 = load_elem(a->v_new, in_off + i + 1, dt);
            }
            float c = f[i], sn = f[i + 1], r0, r1;
            rope_pair(q0, q1, c, sn, &qr[(size_t)s * D + i], &qr[(size_t)s * D + i + 1]);
            rope_pair(k0, k1, c, sn, &r0, &r1);
            store_elem(a->k_cache, new_off + i, dt, r0);
            store_elem(a->k_cache, new_off + i + 1, dt, r1);
            store_elem(a->v_cache, new_off + i, dt, v0);
            store_elem(a->v_cache, new_off + i + 1, dt, v1);
        }
    }

    for (int s = 0; s < S; ++s) {
        const float *q = qr + (size_t)s * D;
        float *o_row = a->out + ((((size_t)b * H + h) * S) + s) * D; /* [B,H,S,D] */
        const float *mrow = a->attn_mask ? a->attn_mask + (size_t)(P + s) * (size_t)a->mask_ld : NULL;
        if (!a->acc_double) {
            float m = -1e9f;
            for (int j = 0; j < ctx; ++j) {
                float acc = 0.0f;
                const size_t r = cache_row0 + (size_t)j * D;
                for (int d = 0; d < D; ++d)
                    acc += load_elem(a->k_cache, r + d, dt) * q[d];
                float v = acc * a->scale + (mrow ? mrow[j] : 0.0f);
                sc[j] = v;
                m = fmaxf(m, v);
            }
            float sum = 0.0f;
            for (int j = 0; j < ctx; ++j) {
                float e = expf(sc[j] - m);
                sc[j] = e;
                sum += e;
            }
            for (int j = 0; j < ctx; ++j)
                sc[j] = sc[j] / sum;
            for (int d = 0; d < D; ++d)
                o_row[d] = 0.0f;
            for (int j = 0; j < ctx; ++j) {
                const size_t r = cache_row0 + (size_t)j * D;
                const float p = sc[j];
                for (int d = 0; d < D; ++d)
                    o_row[d] += p * load_elem(a->v_cache, r + d, dt);
            }
        } else {
            double *scd = (double *)(scratch + (size_t)S * D + ((ctx + 1) & ~1));
            double m = -1e9;
            for (int j = 0; j < ctx; ++j) {
                double acc = 0.0;
                const size_t r = cache_row0 + (size_t)j * D;
                for (int d = 0; d < D; ++d)
                    acc += (double)load_elem(a->k_cache, r + d, dt) * (double)q[d];
                double v = acc * (double)a->scale + (mrow ? (double)mrow[j] : 0.0);
                scd[j] = v;
                if (v > m)
                    m = v;
            }
            double sum = 0.0;
            for (int j = 0; j < ctx; ++j) {
                scd[j] = exp(scd[j] - m);
                sum += scd[j];
            }
            for (int d = 0; d < D; ++d) {
                double acc = 0.0;
                for (int j = 0; j < ctx; ++j)
                    acc += scd[j] * (double)load_elem(a->v_cache, cache_row0 + (size_t)j * D + d, dt);
                o_row[d] = (float)(acc / sum);
            }
        }
    }
}

/*
 * Prompt-phase attention for S new tokens per sequence at positions start_pos .. start_pos+S-1.
 * q/k_new/v_new: [B,S,H,D] in the storage dtype (or int32 accumulators when inp_scale != NULL, with
 * inp_scale [B,S]); out: [B,H,S,D] float.  rope_row < 0: table row = token position; otherwise
 * row = rope_row + s.
 */
int fl_ref_prefill_attn(int dtype, int B, int H, int D, int L, int S, const void *q, const void *k_new,
                        const void *v_new, const float *inp_scale, const float *wq_scale,
                        const float *wk_scale, const float *wv_scale, void *k_cache, void *v_cache,
                        const float *freq_cis, int rope_row, const float *attn_mask, int64_t mask_ld,
                        int start_pos, float scale, float *out, int acc_double, int threads)
{
    if (!q || !k_new || !v_new || !k_cache || !v_cache || !freq_cis || !out)
        return -1;
    if (B <= 0 || H <= 0 || D <= 0 || (D & 1) || L <= 0 || S <= 0)
        return -3;
    if (dtype != FL_REF_F32 && dtype != FL_REF_F16)
        return -6;
    if (start_pos < 0 || start_pos + S > L)
        return -4;
    if (inp_scale && (!wq_scale || !wk_scale || !wv_scale))
        return -1;
    ref_args a;
    memset(&a, 0, sizeof a);
    a.dtype = dtype; a.B = B; a.H = H; a.D = D; a.L = L;
    a.q = q; a.k_new = k_new; a.v_new = v_new; a.k_cache = k_cache; a.v_cache = v_cache;
    a.freq_cis = freq_cis; a.rope_row = rope_row; a.attn_mask = attn_mask; a.mask_ld = mask_ld;
    a.start_pos = start_pos; a.scale = scale; a.out = out; a.acc_double = acc_double;
    a.inp_scale = inp_scale; a.wq_scale = wq_scale; a.wk_scale = wk_scale; a.wv_scale = wv_scale;
    const int BH = B * H;
    const size_t per = (size_t)S * D + (size_t)L + 2 + 2 * ((size_t)L + 2);
    if (threads < 1)
        threads = 1;
    int fail = 0;
#ifdef _OPENMP
#pragma omp parallel num_threads(threads)
#endif
    {
        float *scratch = (float *)malloc(per * sizeof(float));
        if (!scratch) {
#ifdef _OPENMP
#pragma omp atomic write
#endif
            fail = 1;
        }
#ifdef _OPENMP
#pragma omp for schedule(dynamic, 1)
#endif
        for (int bh = 0; bh < BH; ++bh)
            if (scratch)
                prefill_one_head(&a, S, bh / H, bh % H, scratch);
        free(scratch);
    }
    return fail ? -7 : 0;
}

/*
 * Per-token absmax INT8 quantisation with the [B,H,S,D] -> [B,S,H*D] transpose of
 * launchAttnQuantizedTransposeKernel (decoder_kernels.cu:1179-1255): one scale per (b, s) over the
 * H*D values of that token.  attn: [B,H,S,D] float; out_q: [B,S,H*D] int8; out_scale: [B,S].
 */
int fl_ref_attn_quantize_transpose(int B, int H, int S, int D, const float *attn, int8_t *out_q,
                                   float *out_scale)
{
    if (!attn || !out_q || !out_scale)
        return -1;
    for (int b = 0; b < B; ++b)
        for (int s = 0; s < S; ++s) {
            float absmax = -1e9f;
            for (int h = 0; h < H; ++h)
                for (int d = 0; d < D; ++d)
                    absmax = fmaxf(absmax, fabsf(attn[(((size_t)b * H + h) * S + s) * D + d]));
            out_scale[(size_t)b * S + s] = absmax / 127.0f;
            for (int h = 0; h < H; ++h)
                for (int d = 0; d < D; ++d) {
                    float v = attn[(((size_t)b * H + h) * S + s) * D + d] * 127.0f / absmax;
                    float r = nearbyintf(v);
                    int8_t o;
                    if (v != v)
                        o = 0;
                    else if (r > 127.0f)
                        o = 127;
                    else if (r < -128.0f)
                        o = -128;
                    else
                        o = (int8_t)r;
                    out_q[((size_t)b * S + s) * H * D + (size_t)h * D + d] = o;
                }
        }
    return 0;
}

/*
 * Per-row absmax INT8 quantisation of the attention output
 * (decoder_kernels.cu:1179-1212 for seq_len == 1):
 *   absmax = max(-1e9, max_{h,d} |x[b,h,d]|);  scale[b] = absmax / 127;
 *   q = sat_s8(rint(x * 127 / absmax))         (cvt.rni.sat.s8.f32, cuda_kernels.cuh:34-41)
 * attn: [B, H*D] float, out_q: [B, H*D] int8, out_scale: [B].
 */
int fl_ref_attn_quantize(int B, int HD, const float *attn, int8_t *out_q, float *out_scale)
{
    if (!attn || !out_q || !out_scale)
        return -1;
    for (int b = 0; b < B; ++b) {
        const float *x = attn + (size_t)b * HD;
        float absmax = -1e9f;
        for (int i = 0; i < HD; ++i)
            absmax = fmaxf(absmax, fabsf(x[i]));
        out_scale[b] = absmax / 127.0f;
        for (int i = 0; i < HD; ++i) {
            float v = x[i] * 127.0f / absmax;
            float r = nearbyintf(v); /* default rounding mode: nearest-even, as cvt.rni */
            int8_t o;
            if (v != v)
                o = 0; /* cvt.*.sat of NaN yields 0 */
            else if (r > 127.0f)
                o = 127;
            else if (r < -128.0f)
                o = -128;
            else
                o = (int8_t)r;
            out_q[(size_t)b * HD + i] = o;
        }
    }
    return 0;
}

int fl_ref_omp_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
