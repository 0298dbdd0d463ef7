/*
 * TEST INFRASTRUCTURE.  Drives every entry point of the CPU oracle (fl_ref_decode_attn.c) on small seeded
 * shapes under AddressSanitizer + UndefinedBehaviorSanitizer (`make -C oracle asan` builds and runs it):
 * ragged batches with positions at, inside and outside every bound, the promised-bound branch, both
 * storage types, masks with a custom row stride, the int32 prologue, the prompt phase and both quantisers.
 * A sanitizer report aborts the run; the values themselves are checked by tests/test_oracle_pins.py.
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

int fl_ref_decode_attn(int dtype, int B, int H, int D, int L, const void *q, const void *k_new, const void *v_new,
                       void *k_cache, void *v_cache, const float *freq_cis, int rope_row, const float *attn_mask,
                       int64_t mask_ld, int start_pos, const int32_t *start_pos_per_seq, int max_start_pos, float scale,
                       float *out, int acc_double, int threads);
int fl_ref_decode_attn_i32(int dtype, int B, int H, int D, int L, const int32_t *q_acc, const int32_t *k_acc,
                           const int32_t *v_acc, const float *inp_scale, const float *wq_scale, const float *wk_scale,
                           const float *wv_scale, void *k_cache, void *v_cache, const float *freq_cis, int rope_row,
                           const float *attn_mask, int64_t mask_ld, int start_pos, const int32_t *start_pos_per_seq,
                           int max_start_pos, float scale, float *out, int acc_double, int threads);
int fl_ref_prefill_attn(int dtype, int B, int H, int D, int L, int S, const void *q, const void *k_new, const void *v_new,
                        const float *inp_scale, const float *wq_scale, const float *wk_scale, const float *wv_scale,
                        void *k_cache, void *v_cache, const float *freq_cis, int rope_row, const float *attn_mask,
                        int64_t mask_ld, int start_pos, float scale, float *out, int acc_double, int threads);
int fl_ref_attn_quantize(int B, int HD, const float *attn, int8_t *out_q, float *out_scale);
int fl_ref_attn_quantize_transpose(int B, int H, int S, int D, const float *attn, int8_t *out_q, float *out_scale);
int fl_ref_freq_cis(float *table, int rows, int D, double base);
uint16_t fl_ref_float_to_half(float f);
float fl_ref_half_to_float(uint16_t h);

static uint32_t rng_state = 12345u;
static float rnd(void)
{
    rng_state = rng_state * 1664525u + 1013904223u;
    return (float)((rng_state >> 8) & 0xffff) / 32768.0f - 1.0f;
}

/* exactly-sized heap blocks: an access one element outside any of them is a sanitizer report */
static void *filled(size_t n, int dtype)
{
    if (dtype == 1) {
        uint16_t *p = malloc(n * sizeof *p);
        for (size_t i = 0; i < n; ++i) p[i] = fl_ref_float_to_half(rnd());
        return p;
    }
    float *p = malloc(n * sizeof *p);
    for (size_t i = 0; i < n; ++i) p[i] = rnd();
    return p;
}

static int checks = 0;
#define EXPECT(cond)                                                         \
    do {                                                                     \
        ++checks;                                                            \
        if (!(cond)) {                                                       \
            fprintf(stderr, "FAIL line %d: %s\n", __LINE__, #cond);          \
            return 1;                                                        \
        }                                                                    \
    } while (0)

int main(void)
{
    for (int dtype = 0; dtype < 2; ++dtype) {
        for (int acc = 0; acc < 2; ++acc) {
            const int B = 5, H = 3, D = 32, L = 19, ld = 23;
            void *q = filled((size_t)B * H * D, dtype), *k = filled((size_t)B * H * D, dtype), *v = filled((size_t)B * H * D, dtype);
            void *kc = filled((size_t)B * H * L * D, dtype), *vc = filled((size_t)B * H * L * D, dtype);
            float *freq = malloc((size_t)L * D * sizeof *freq), *mask = filled((size_t)L * ld, 0);
            float *out = malloc((size_t)B * H * D * sizeof *out);
            EXPECT(fl_ref_freq_cis(freq, L, D, 10000.0) == 0);
            /* uniform positions at both ends of the cache, with and without a mask, literal RoPE row */
            EXPECT(fl_ref_decode_attn(dtype, B, H, D, L, q, k, v, kc, vc, freq, -1, NULL, 0, 0, NULL, -1, 0.17f, out, acc, 2) == 0);
            EXPECT(fl_ref_decode_attn(dtype, B, H, D, L, q, k, v, kc, vc, freq, 0, mask, ld, L - 1, NULL, -1, 0.17f, out, acc, 2) == 0);
            EXPECT(fl_ref_decode_attn(dtype, B, H, D, L, q, k, v, kc, vc, freq, -1, mask, ld, L, NULL, -1, 0.17f, out, acc, 1) == -4);
            /* ragged: first row, last row, below zero, past the end, above the promised bound */
            const int32_t pos[5] = {0, L - 1, -1, L, 7};
            EXPECT(fl_ref_decode_attn(dtype, B, H, D, L, q, k, v, kc, vc, freq, -1, mask, ld, 0, pos, -1, 0.17f, out, acc, 3) == 0);
            EXPECT(isnan(out[2 * H * D]) && isnan(out[3 * H * D]) && !isnan(out[4 * H * D]) && !isnan(out[1 * H * D]));
            EXPECT(fl_ref_decode_attn(dtype, B, H, D, L, q, k, v, kc, vc, freq, -1, mask, ld, 0, pos, 6, 0.17f, out, acc, 3) == 0);
            EXPECT(!isnan(out[0]) && isnan(out[1 * H * D]) && isnan(out[4 * H * D]));
            /* int32 prologue */
            int32_t *qi = malloc((size_t)B * H * D * sizeof *qi), *ki = malloc((size_t)B * H * D * sizeof *ki), *vi = malloc((size_t)B * H * D * sizeof *vi);
            for (int i = 0; i < B * H * D; ++i) { qi[i] = (int32_t)(rnd() * 20000); ki[i] = (int32_t)(rnd() * 20000); vi[i] = (int32_t)(rnd() * 20000); }
            float *s_in = filled(B, 0), *wq = filled((size_t)H * D, 0), *wk = filled((size_t)H * D, 0), *wv = filled((size_t)H * D, 0);
            EXPECT(fl_ref_decode_attn_i32(dtype, B, H, D, L, qi, ki, vi, s_in, wq, wk, wv, kc, vc, freq, -1, mask, ld, 0, pos, -1, 0.17f, out, acc, 2) == 0);
            /* quantiser on the [B, H*D] output (NaN rows included: they quantise to 0) */
            int8_t *o8 = malloc((size_t)B * H * D);
            float *os = malloc(B * sizeof *os);
            EXPECT(fl_ref_attn_quantize(B, H * D, out, o8, os) == 0);
            /* prompt phase: chunk that ends exactly at the cache's last row */
            const int S = 6, P = L - S;
            void *pq = filled((size_t)B * S * H * D, dtype), *pk = filled((size_t)B * S * H * D, dtype), *pv = filled((size_t)B * S * H * D, dtype);
            float *pout = malloc((size_t)B * H * S * D * sizeof *pout);
            EXPECT(fl_ref_prefill_attn(dtype, B, H, D, L, S, pq, pk, pv, NULL, NULL, NULL, NULL, kc, vc, freq, -1, mask, ld, P, 0.17f, pout, acc, 2) == 0);
            EXPECT(fl_ref_prefill_attn(dtype, B, H, D, L, S, pq, pk, pv, NULL, NULL, NULL, NULL, kc, vc, freq, -1, mask, ld, P + 1, 0.17f, pout, acc, 2) == -4);
            int32_t *pqi = malloc((size_t)B * S * H * D * sizeof *pqi);
            for (int i = 0; i < B * S * H * D; ++i) pqi[i] = (int32_t)(rnd() * 20000);
            float *ps = filled((size_t)B * S, 0);
            EXPECT(fl_ref_prefill_attn(dtype, B, H, D, L, S, pqi, pqi, pqi, ps, wq, wk, wv, kc, vc, freq, 0, NULL, 0, 0, 0.17f, pout, acc, 1) == 0);
            int8_t *p8 = malloc((size_t)B * S * H * D);
            float *pscale = malloc((size_t)B * S * sizeof *pscale);
            EXPECT(fl_ref_attn_quantize_transpose(B, H, S, D, pout, p8, pscale) == 0);
            free(q); free(k); free(v); free(kc); free(vc); free(freq); free(mask); free(out); free(qi); free(ki); free(vi);
            free(s_in); free(wq); free(wk); free(wv); free(o8); free(os); free(pq); free(pk); free(pv); free(pout); free(pqi);
            free(ps); free(p8); free(pscale);
        }
    }
    /* half conversions over every bit pattern and over the float edge cases */
    for (uint32_t h = 0; h < 65536u; ++h) {
        const float f = fl_ref_half_to_float((uint16_t)h);
        if (f == f) EXPECT(fl_ref_float_to_half(f) == (uint16_t)h);
    }
    const float edge[] = {0.0f, -0.0f, 65504.0f, 65520.0f, 1e30f, -1e30f, 5.96e-8f, 2.98e-8f, 1e-30f, INFINITY, -INFINITY, NAN};
    for (size_t i = 0; i < sizeof edge / sizeof edge[0]; ++i) (void)fl_ref_float_to_half(edge[i]);
    printf("oracle sanitizer run: %d checks, no report\n", checks);
    return 0;
}
