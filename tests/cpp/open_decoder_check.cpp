// Drop-in check of the C++ OpenDecoder mirror on a real GPU: the calls a FasterLLaMA caller makes
// (constructor, getWorkspaceSize, initialize, forward) plus decodeAttention, compared with the CPU
// oracle (linked from oracle/libfl_ref.so — checker only).  Prints one line per check and exits
// non-zero on the first failure.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <algorithm>
#include <stdexcept>
#include <vector>

#include "open_decoder.h"

extern "C" {
int fl_ref_decode_attn(int dtype, int B, int H, int D, int L, const void *q, const void *k_new, const void *v_new,
                       void *k_cache, void *v_cache, const float *freq_cis, int rope_row, const float *attn_mask,
                       int64_t mask_ld, int start_pos, const int32_t *start_pos_per_seq, int max_start_pos, float scale,
                       float *out, int acc_double, int threads);
int fl_ref_decode_attn_i32(int dtype, int B, int H, int D, int L, const int32_t *q_acc, const int32_t *k_acc,
                           const int32_t *v_acc, const float *inp_scale, const float *wq_scale, const float *wk_scale,
                           const float *wv_scale, void *k_cache, void *v_cache, const float *freq_cis, int rope_row,
                           const float *attn_mask, int64_t mask_ld, int start_pos, const int32_t *start_pos_per_seq,
                           int max_start_pos, float scale, float *out, int acc_double, int threads);
int fl_ref_attn_quantize(int B, int HD, const float *attn, int8_t *out_q, float *out_scale);
int fl_ref_prefill_attn(int dtype, int B, int H, int D, int L, int S, const void *q, const void *k_new, const void *v_new,
                        const float *inp_scale, const float *wq_scale, const float *wk_scale, const float *wv_scale,
                        void *k_cache, void *v_cache, const float *freq_cis, int rope_row, const float *attn_mask,
                        int64_t mask_ld, int start_pos, float scale, float *out, int acc_double, int threads);
int fl_ref_attn_quantize_transpose(int B, int H, int S, int D, const float *attn, int8_t *out_q, float *out_scale);
int fl_ref_freq_cis(float *table, int rows, int D, double base);
uint16_t fl_ref_float_to_half(float f);
}

using namespace FasterLLaMA;

#define HIP_OK(x)                                                                                  \
    do {                                                                                           \
        hipError_t e_ = (x);                                                                       \
        if (e_ != hipSuccess) {                                                                    \
            std::printf("FAIL hip error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); \
            std::exit(2);                                                                          \
        }                                                                                          \
    } while (0)

static uint64_t g_state = 0x1234567ull;
static float frand() // uniform in [-1, 1)
{
    g_state = g_state * 6364136223846793005ull + 1442695040888963407ull;
    return (float)((g_state >> 40) & 0xFFFFFF) / 8388608.0f - 1.0f;
}

template <typename T> struct DevBuf {
    T *p = nullptr;
    size_t n = 0;
    explicit DevBuf(size_t n_) : n(n_) { HIP_OK(hipMalloc(&p, n * sizeof(T))); }
    ~DevBuf() { (void)hipFree(p); }
    void up(const void *h) { HIP_OK(hipMemcpy(p, h, n * sizeof(T), hipMemcpyHostToDevice)); }
    void down(void *h) const { HIP_OK(hipMemcpy(h, p, n * sizeof(T), hipMemcpyDeviceToHost)); }
};

static int g_fail = 0;
static void report(const char *name, bool ok, double detail = 0.0)
{
    std::printf("%s %s (%.3e)\n", ok ? "PASS" : "FAIL", name, detail);
    std::fflush(stdout);
    if (!ok) g_fail = 1;
}

struct HookCtx {
    const int32_t *q, *k, *v;
    const float *scale;
    int8_t *seen_int8;
    float *seen_scale;
    size_t hidden;
    int calls_pre = 0, calls_post = 0;
};

template <typename T>
static void qkvHook(void *user, const T *, int32_t *qb, int32_t *kb, int32_t *vb, float *sb, int B, int S, hipStream_t s)
{
    HookCtx *c = static_cast<HookCtx *>(user);
    B *= S; // tokens
    const size_t bytes = (size_t)B * c->hidden * sizeof(int32_t);
    HIP_OK(hipMemcpyAsync(qb, c->q, bytes, hipMemcpyDeviceToDevice, s));
    HIP_OK(hipMemcpyAsync(kb, c->k, bytes, hipMemcpyDeviceToDevice, s));
    HIP_OK(hipMemcpyAsync(vb, c->v, bytes, hipMemcpyDeviceToDevice, s));
    HIP_OK(hipMemcpyAsync(sb, c->scale, (size_t)B * sizeof(float), hipMemcpyDeviceToDevice, s));
    c->calls_pre++;
}

template <typename T>
static void postHook(void *user, const int8_t *a8, const float *as, const T *, T *, int B, int S, hipStream_t s)
{
    HookCtx *c = static_cast<HookCtx *>(user);
    B *= S; // tokens
    HIP_OK(hipMemcpyAsync(c->seen_int8, a8, (size_t)B * c->hidden, hipMemcpyDeviceToDevice, s));
    HIP_OK(hipMemcpyAsync(c->seen_scale, as, (size_t)B * sizeof(float), hipMemcpyDeviceToDevice, s));
    c->calls_post++;
}

template <typename CacheT> static CacheT toCache(float x);
template <> float toCache<float>(float x) { return x; }
template <> __half toCache<__half>(float x)
{
    uint16_t b = fl_ref_float_to_half(x);
    __half h;
    std::memcpy(&h, &b, 2);
    return h;
}

template <OperationType Op, typename CacheT> static void runAll(const char *tag)
{
    typedef typename DecoderTransformerTraits<Op>::DataType DataT;
    const int B = 3, H = 8, D = 128, prompt = 40, gen = 24, L = prompt + gen, P = 50, HD = H * D;
    const int code = std::is_same<CacheT, float>::value ? 0 : 1;
    char name[128];

    std::vector<float> freq((size_t)L * D), mask((size_t)L * L);
    fl_ref_freq_cis(freq.data(), L, D, 10000.0);
    for (int r = 0; r < L; ++r)
        for (int c = 0; c < L; ++c) mask[(size_t)r * L + c] = c > r ? -1e5f : 0.0f; // causal (samples/test.cu:427-437)

    std::vector<CacheT> q((size_t)B * HD), k(q.size()), v(q.size()), kc((size_t)B * H * L * D), vc(kc.size());
    for (auto &x : q) x = toCache<CacheT>(frand());
    for (auto &x : k) x = toCache<CacheT>(frand());
    for (auto &x : v) x = toCache<CacheT>(frand());
    for (auto &x : kc) x = toCache<CacheT>(frand());
    for (auto &x : vc) x = toCache<CacheT>(frand());

    DevBuf<float> d_freq(freq.size()), d_mask(mask.size()), d_out((size_t)B * HD);
    DevBuf<CacheT> d_q(q.size()), d_k(k.size()), d_v(v.size()), d_kc(kc.size()), d_vc(vc.size());
    d_freq.up(freq.data()); d_mask.up(mask.data());
    d_q.up(q.data()); d_k.up(k.data()); d_v.up(v.data()); d_kc.up(kc.data()); d_vc.up(vc.data());

    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));

    OpenDecoder<Op, OperationType::INT8> dec(B, prompt, gen, H, D, 4 * HD);
    const int ws_bytes = dec.getWorkspaceSize();
    DevBuf<char> d_ws((size_t)ws_bytes);
    DecoderInitParam<DataT, int8_t> param;
    param.attn_mask = d_mask.p;
    param.stream = stream;

    std::vector<float> wq(HD), wk(HD), wv(HD), s_in(B);
    for (auto &x : wq) x = 0.01f + 0.01f * (frand() + 1.0f);
    for (auto &x : wk) x = 0.01f + 0.01f * (frand() + 1.0f);
    for (auto &x : wv) x = 0.01f + 0.01f * (frand() + 1.0f);
    for (auto &x : s_in) x = 0.002f + 0.001f * (frand() + 1.0f);
    DevBuf<float> d_wq(HD), d_wk(HD), d_wv(HD), d_sin(B);
    d_wq.up(wq.data()); d_wk.up(wk.data()); d_wv.up(wv.data()); d_sin.up(s_in.data());
    param.attention.query_weight.weight_scale = d_wq.p;
    param.attention.key_weight.weight_scale = d_wk.p;
    param.attention.value_weight.weight_scale = d_wv.p;
    dec.initialize(param, d_ws.p);

    // ---- 1. decodeAttention on float/half operands vs the oracle
    {
        std::vector<CacheT> kc_ref(kc), vc_ref(vc), kc_got(kc.size()), vc_got(vc.size());
        std::vector<float> want((size_t)B * HD), got(want.size());
        fl_ref_decode_attn(code, B, H, D, L, q.data(), k.data(), v.data(), kc_ref.data(), vc_ref.data(), freq.data(), -1,
                           mask.data(), L, P, nullptr, -1, 1.0f / std::sqrt((float)D), want.data(), 1, 1);
        dec.decodeAttention(d_q.p, d_k.p, d_v.p, d_freq.p, d_kc.p, d_vc.p, d_out.p, P);
        HIP_OK(hipStreamSynchronize(stream));
        d_out.down(got.data()); d_kc.down(kc_got.data()); d_vc.down(vc_got.data());
        double worst = 0, scale = 0;
        for (float w : want) scale = std::fmax(scale, std::fabs(w));
        for (size_t i = 0; i < want.size(); ++i) {
            double tol = code ? 2e-3 : 1e-5 * std::fmax(std::fabs(want[i]), scale);
            worst = std::fmax(worst, std::fabs((double)got[i] - want[i]) / tol);
        }
        std::snprintf(name, sizeof name, "%s decodeAttention output", tag);
        report(name, worst <= 1.0, worst);
        std::snprintf(name, sizeof name, "%s decodeAttention caches bit-exact", tag);
        report(name, !std::memcmp(kc_got.data(), kc_ref.data(), kc.size() * sizeof(CacheT)) &&
                         !std::memcmp(vc_got.data(), vc_ref.data(), vc.size() * sizeof(CacheT)));
    }

    // ---- 2. forward() with external stages: int32 accumulators in, INT8 + scale out
    std::vector<int32_t> qi((size_t)B * HD), ki(qi.size()), vi(qi.size());
    for (auto &x : qi) x = (int32_t)(frand() * 20000.f);
    for (auto &x : ki) x = (int32_t)(frand() * 20000.f);
    for (auto &x : vi) x = (int32_t)(frand() * 20000.f);
    DevBuf<int32_t> d_qi(qi.size()), d_ki(ki.size()), d_vi(vi.size());
    d_qi.up(qi.data()); d_ki.up(ki.data()); d_vi.up(vi.data());
    DevBuf<int8_t> d_seen8((size_t)B * HD);
    DevBuf<float> d_seens(B);
    HookCtx ctx{d_qi.p, d_ki.p, d_vi.p, d_sin.p, d_seen8.p, d_seens.p, (size_t)HD};
    DecoderExternalStages<DataT> stages_keep;
    {
        d_kc.up(kc.data()); d_vc.up(vc.data());
        stages_keep.user = &ctx;
        stages_keep.qkv_projection = qkvHook<DataT>;
        stages_keep.post_attention = postHook<DataT>;
        dec.setExternalStages(stages_keep);
        DevBuf<DataT> d_from((size_t)B * HD), d_dec_out((size_t)B * HD);
        dec.forward(d_from.p, d_freq.p, d_kc.p, d_vc.p, d_dec_out.p, P, 1);
        HIP_OK(hipStreamSynchronize(stream));

        std::vector<CacheT> kc_ref(kc), vc_ref(vc), kc_got(kc.size());
        std::vector<float> want((size_t)B * HD), want_s(B), got_s(B);
        std::vector<int8_t> want8((size_t)B * HD), got8(want8.size());
        fl_ref_decode_attn_i32(code, B, H, D, L, qi.data(), ki.data(), vi.data(), s_in.data(), wq.data(), wk.data(), wv.data(),
                               kc_ref.data(), vc_ref.data(), freq.data(), -1, mask.data(), L, P, nullptr, -1,
                               1.0f / std::sqrt((float)D), want.data(), 1, 1);
        fl_ref_attn_quantize(B, HD, want.data(), want8.data(), want_s.data());
        d_seen8.down(got8.data()); d_seens.down(got_s.data()); d_kc.down(kc_got.data());
        int worst8 = 0;
        for (size_t i = 0; i < want8.size(); ++i) worst8 = std::max(worst8, std::abs((int)got8[i] - (int)want8[i]));
        double worst_s = 0;
        for (int b = 0; b < B; ++b) worst_s = std::fmax(worst_s, std::fabs(got_s[b] - want_s[b]) / want_s[b]);
        std::snprintf(name, sizeof name, "%s forward int8 within one step", tag);
        report(name, worst8 <= 1 && ctx.calls_pre == 1 && ctx.calls_post == 1, worst8);
        std::snprintf(name, sizeof name, "%s forward output scale", tag);
        report(name, worst_s <= 1e-5, worst_s);
        std::snprintf(name, sizeof name, "%s forward k_cache bit-exact", tag);
        report(name, !std::memcmp(kc_got.data(), kc_ref.data(), kc.size() * sizeof(CacheT)));
    }

    // ---- 3. literal RoPE row: the appended key equals the unrotated key (row 0 = identity)
    {
        d_kc.up(kc.data()); d_vc.up(vc.data());
        dec.setLiteralRopeRow(true);
        dec.decodeAttention(d_q.p, d_k.p, d_v.p, d_freq.p, d_kc.p, d_vc.p, d_out.p, P);
        HIP_OK(hipStreamSynchronize(stream));
        dec.setLiteralRopeRow(false);
        std::vector<CacheT> kc_got(kc.size());
        d_kc.down(kc_got.data());
        bool same = true;
        for (int b = 0; b < B && same; ++b)
            for (int h = 0; h < H && same; ++h)
                same = !std::memcmp(&kc_got[(((size_t)b * H + h) * L + P) * D], &k[((size_t)b * H + h) * D], D * sizeof(CacheT));
        std::snprintf(name, sizeof name, "%s literal RoPE row stores k unrotated", tag);
        report(name, same);
    }

    // ---- 3b. prompt phase through forward(): seq_len = 24 tokens at start_pos 0 (the reference's prefill call)
    {
        const int S = 24;
        std::vector<int32_t> pq((size_t)B * S * HD), pk(pq.size()), pv(pq.size());
        for (auto &x : pq) x = (int32_t)(frand() * 20000.f);
        for (auto &x : pk) x = (int32_t)(frand() * 20000.f);
        for (auto &x : pv) x = (int32_t)(frand() * 20000.f);
        std::vector<float> ps((size_t)B * S);
        for (auto &x : ps) x = 0.002f + 0.001f * (frand() + 1.0f);
        DevBuf<int32_t> d_pq(pq.size()), d_pk(pk.size()), d_pv(pv.size());
        DevBuf<float> d_ps(ps.size()), d_seens2((size_t)B * S);
        DevBuf<int8_t> d_seen82((size_t)B * S * HD);
        d_pq.up(pq.data()); d_pk.up(pk.data()); d_pv.up(pv.data()); d_ps.up(ps.data());
        d_kc.up(kc.data()); d_vc.up(vc.data());
        HookCtx pctx{d_pq.p, d_pk.p, d_pv.p, d_ps.p, d_seen82.p, d_seens2.p, (size_t)HD};
        DecoderExternalStages<DataT> st2;
        st2.user = &pctx;
        st2.qkv_projection = qkvHook<DataT>;
        st2.post_attention = postHook<DataT>;
        dec.setExternalStages(st2);
        DevBuf<DataT> d_from((size_t)B * S * HD), d_dec_out((size_t)B * S * HD);
        dec.classifyMask(); // the mask is in place: its tiles are classified once, not in every prompt-phase call
        dec.forward(d_from.p, d_freq.p, d_kc.p, d_vc.p, d_dec_out.p, 0, S);
        HIP_OK(hipStreamSynchronize(stream));

        std::vector<CacheT> kc_ref(kc), vc_ref(vc), kc_got(kc.size());
        std::vector<float> want((size_t)B * H * S * D), want_s((size_t)B * S), got_s(want_s.size());
        std::vector<int8_t> want8((size_t)B * S * HD), got8(want8.size());
        fl_ref_prefill_attn(code, B, H, D, L, S, pq.data(), pk.data(), pv.data(), ps.data(), wq.data(), wk.data(), wv.data(),
                            kc_ref.data(), vc_ref.data(), freq.data(), -1, mask.data(), L, 0, 1.0f / std::sqrt((float)D),
                            want.data(), 1, 4);
        fl_ref_attn_quantize_transpose(B, H, S, D, want.data(), want8.data(), want_s.data());
        d_seen82.down(got8.data()); d_seens2.down(got_s.data()); d_kc.down(kc_got.data());
        int worst8 = 0;
        for (size_t i = 0; i < want8.size(); ++i) worst8 = std::max(worst8, std::abs((int)got8[i] - (int)want8[i]));
        double worst_s = 0;
        for (size_t i = 0; i < want_s.size(); ++i) worst_s = std::fmax(worst_s, std::fabs(got_s[i] - want_s[i]) / want_s[i]);
        std::snprintf(name, sizeof name, "%s prompt forward int8 within one step", tag);
        report(name, worst8 <= 1 && pctx.calls_pre == 1 && pctx.calls_post == 1, worst8);
        std::snprintf(name, sizeof name, "%s prompt forward output scale", tag);
        report(name, worst_s <= (code ? 1e-3 : 1e-5), worst_s); // half caches: fp16 matrix-core operands
        std::snprintf(name, sizeof name, "%s prompt forward k_cache bit-exact", tag);
        report(name, !std::memcmp(kc_got.data(), kc_ref.data(), kc.size() * sizeof(CacheT)));
        dec.setExternalStages(stages_keep);
    }

    // ---- 4. error behaviour: std::runtime_error, never exit()
    {
        DevBuf<DataT> d_from((size_t)B * HD), d_dec_out((size_t)B * HD);
        int caught = 0;
        try { dec.forward(d_from.p, d_freq.p, d_kc.p, d_vc.p, d_dec_out.p, 0, prompt + 1); } catch (std::runtime_error &) { caught++; }
        try { dec.forward(d_from.p, d_freq.p, d_kc.p, d_vc.p, d_dec_out.p, L, 1); } catch (std::runtime_error &) { caught++; }
        try { dec.decodeAttention(d_q.p, d_k.p, d_v.p, (const float *)nullptr, d_kc.p, d_vc.p, d_out.p, P); } catch (std::runtime_error &) { caught++; }
        try {
            OpenDecoder<Op, OperationType::INT8> bad(B, prompt, gen, H, 48, 4 * HD); // reference: throw "invalid size_per_head!"
            (void)bad.getWorkspaceSize();
        } catch (std::runtime_error &) { caught++; }
        try {
            OpenDecoder<Op, OperationType::INT8> fresh(B, prompt, gen, H, D, 4 * HD); // no stages installed
            fresh.initialize(param, d_ws.p);
            fresh.forward(d_from.p, d_freq.p, d_kc.p, d_vc.p, d_dec_out.p, P, 1);
        } catch (std::runtime_error &) { caught++; }
        std::snprintf(name, sizeof name, "%s errors surface as std::runtime_error", tag);
        report(name, caught == 5, caught);
    }
    HIP_OK(hipStreamDestroy(stream));
}

// The reference driver's loop (decoding_sampling.cu:232-258): ONE decoder object and ONE workspace serve every layer;
// initialize(param[layer], buf) is called before every forward() of every step; each layer owns its slice of the K/V
// cache arena (decoding_sampling.cu:256-257).  One prompt call and `gen_steps` decode steps per layer, with a context
// split so that the decode steps use the arrival counters in the shared workspace; every quantised output and the
// final caches of every layer are compared with the oracle run in the same order.
template <OperationType Op, typename CacheT> static void runLayerLoop(const char *tag)
{
    typedef typename DecoderTransformerTraits<Op>::DataType DataT;
    const int B = 2, H = 4, D = 128, prompt = 24, gen = 8, L = prompt + gen, HD = H * D, layers = 3, gen_steps = 3;
    const int code = std::is_same<CacheT, float>::value ? 0 : 1;
    char name[160];

    std::vector<float> freq((size_t)L * D), mask((size_t)L * L);
    fl_ref_freq_cis(freq.data(), L, D, 10000.0);
    for (int r = 0; r < L; ++r)
        for (int c = 0; c < L; ++c) mask[(size_t)r * L + c] = c > r ? -3.4028234664e38f : 0.0f; // samples/llama_fp16.cu:73-81, causal
    DevBuf<float> d_freq(freq.size()), d_mask(mask.size());
    d_freq.up(freq.data()); d_mask.up(mask.data());

    const size_t layer_elems = (size_t)B * H * L * D;
    std::vector<CacheT> kc(layers * layer_elems), vc(kc.size());
    for (auto &x : kc) x = toCache<CacheT>(frand());
    for (auto &x : vc) x = toCache<CacheT>(frand());
    DevBuf<CacheT> d_kc(kc.size()), d_vc(vc.size());
    d_kc.up(kc.data()); d_vc.up(vc.data());

    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));
    OpenDecoder<Op, OperationType::INT8> dec(B, prompt, gen, H, D, 4 * HD);
    dec.setContextSplits(2);
    DevBuf<char> d_ws(dec.getWorkspaceSizeBytes());

    // per-layer parameters: the scales differ per layer, the mask is the one shared array
    std::vector<std::vector<float>> wq(layers), wk(layers), wv(layers);
    std::vector<DevBuf<float> *> d_w;
    std::vector<DecoderInitParam<DataT, int8_t>> param(layers);
    for (int l = 0; l < layers; ++l) {
        for (auto *w : {&wq[l], &wk[l], &wv[l]}) {
            w->resize(HD);
            for (auto &x : *w) x = 0.01f + 0.01f * (frand() + 1.0f);
            d_w.push_back(new DevBuf<float>(HD));
            d_w.back()->up(w->data());
        }
        param[l].attn_mask = d_mask.p;
        param[l].stream = stream;
        param[l].attention.query_weight.weight_scale = d_w[3 * l]->p;
        param[l].attention.key_weight.weight_scale = d_w[3 * l + 1]->p;
        param[l].attention.value_weight.weight_scale = d_w[3 * l + 2]->p;
    }

    // inputs of every (step, layer): int32 accumulators and activation scales; step 0 is the prompt (24 tokens)
    const int steps = 1 + gen_steps;
    auto tokens_of = [&](int step) { return step == 0 ? prompt : 1; };
    std::vector<std::vector<int32_t>> qi(steps * layers), ki(steps * layers), vi(steps * layers);
    std::vector<std::vector<float>> sc(steps * layers);
    std::vector<DevBuf<int32_t> *> d_i;
    std::vector<DevBuf<float> *> d_s;
    std::vector<DevBuf<int8_t> *> d_seen8;
    std::vector<DevBuf<float> *> d_seens;
    for (int i = 0; i < steps * layers; ++i) {
        const size_t n = (size_t)B * tokens_of(i / layers) * HD;
        for (auto *a : {&qi[i], &ki[i], &vi[i]}) {
            a->resize(n);
            for (auto &x : *a) x = (int32_t)(frand() * 20000.f);
            d_i.push_back(new DevBuf<int32_t>(n));
            d_i.back()->up(a->data());
        }
        sc[i].resize((size_t)B * tokens_of(i / layers));
        for (auto &x : sc[i]) x = 0.002f + 0.001f * (frand() + 1.0f);
        d_s.push_back(new DevBuf<float>(sc[i].size()));
        d_s.back()->up(sc[i].data());
        d_seen8.push_back(new DevBuf<int8_t>(n));
        d_seens.push_back(new DevBuf<float>(sc[i].size()));
    }

    DevBuf<DataT> d_from((size_t)B * prompt * HD), d_dec_out((size_t)B * prompt * HD);
    HookCtx ctx{};
    ctx.hidden = (size_t)HD;
    DecoderExternalStages<DataT> st;
    st.user = &ctx;
    st.qkv_projection = qkvHook<DataT>;
    st.post_attention = postHook<DataT>;
    dec.setExternalStages(st);

    bool classified = false;
    for (int step = 0; step < steps; ++step) {
        const int start_pos = step == 0 ? 0 : prompt + step - 1, S = tokens_of(step);
        for (int l = 0; l < layers; ++l) { // decoding_sampling.cu:242-258
            const int i = step * layers + l;
            dec.initialize(param[l], d_ws.p);
            if (!classified) { // once: the mask is the same array for every layer and call
                dec.classifyMask();
                classified = true;
            }
            ctx.q = d_i[3 * i]->p; ctx.k = d_i[3 * i + 1]->p; ctx.v = d_i[3 * i + 2]->p;
            ctx.scale = d_s[i]->p; ctx.seen_int8 = d_seen8[i]->p; ctx.seen_scale = d_seens[i]->p;
            dec.forward(d_from.p, d_freq.p, d_kc.p + l * layer_elems, d_vc.p + l * layer_elems, d_dec_out.p, start_pos, S);
        }
    }
    HIP_OK(hipStreamSynchronize(stream));

    // the oracle, same order
    int worst8 = 0;
    double worst_s = 0;
    for (int step = 0; step < steps; ++step) {
        const int start_pos = step == 0 ? 0 : prompt + step - 1, S = tokens_of(step);
        for (int l = 0; l < layers; ++l) {
            const int i = step * layers + l;
            CacheT *kl = kc.data() + l * layer_elems, *vl = vc.data() + l * layer_elems;
            std::vector<float> want((size_t)B * H * S * D), want_s((size_t)B * S), got_s(want_s.size());
            std::vector<int8_t> want8((size_t)B * S * HD), got8(want8.size());
            if (S == 1) {
                fl_ref_decode_attn_i32(code, B, H, D, L, qi[i].data(), ki[i].data(), vi[i].data(), sc[i].data(), wq[l].data(),
                                       wk[l].data(), wv[l].data(), kl, vl, freq.data(), -1, mask.data(), L, start_pos, nullptr, -1,
                                       1.0f / std::sqrt((float)D), want.data(), 1, 1);
                fl_ref_attn_quantize(B, HD, want.data(), want8.data(), want_s.data());
            } else {
                fl_ref_prefill_attn(code, B, H, D, L, S, qi[i].data(), ki[i].data(), vi[i].data(), sc[i].data(), wq[l].data(),
                                    wk[l].data(), wv[l].data(), kl, vl, freq.data(), -1, mask.data(), L, start_pos,
                                    1.0f / std::sqrt((float)D), want.data(), 1, 4);
                fl_ref_attn_quantize_transpose(B, H, S, D, want.data(), want8.data(), want_s.data());
            }
            d_seen8[i]->down(got8.data());
            d_seens[i]->down(got_s.data());
            for (size_t j = 0; j < want8.size(); ++j) worst8 = std::max(worst8, std::abs((int)got8[j] - (int)want8[j]));
            for (size_t j = 0; j < want_s.size(); ++j) worst_s = std::fmax(worst_s, std::fabs(got_s[j] - want_s[j]) / want_s[j]);
        }
    }
    std::vector<CacheT> kc_got(kc.size()), vc_got(vc.size());
    d_kc.down(kc_got.data()); d_vc.down(vc_got.data());
    std::snprintf(name, sizeof name, "%s layer loop (initialize before every forward): int8 within one step", tag);
    report(name, worst8 <= 1 && ctx.calls_pre == steps * layers && ctx.calls_post == steps * layers, worst8);
    std::snprintf(name, sizeof name, "%s layer loop: output scales", tag);
    report(name, worst_s <= (code ? 1e-3 : 1e-5), worst_s);
    std::snprintf(name, sizeof name, "%s layer loop: caches of every layer bit-exact", tag);
    report(name, !std::memcmp(kc_got.data(), kc.data(), kc.size() * sizeof(CacheT)) &&
                     !std::memcmp(vc_got.data(), vc.data(), vc.size() * sizeof(CacheT)));
    for (auto *p : d_w) delete p;
    for (auto *p : d_i) delete p;
    for (auto *p : d_s) delete p;
    for (auto *p : d_seen8) delete p;
    for (auto *p : d_seens) delete p;
    HIP_OK(hipStreamDestroy(stream));
}

int main()
{
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n < 1) {
        std::printf("FAIL no GPU\n");
        return 3;
    }
    runAll<OperationType::FP32, float>("OpenDecoder<FP32,INT8>/float-cache");
    runAll<OperationType::FP16, float>("OpenDecoder<FP16,INT8>/float-cache");
    runAll<OperationType::FP16, __half>("OpenDecoder<FP16,INT8>/half-cache");
    runLayerLoop<OperationType::FP32, float>("OpenDecoder<FP32,INT8>/float-cache");
    runLayerLoop<OperationType::FP16, __half>("OpenDecoder<FP16,INT8>/half-cache");
    std::printf(g_fail ? "SOME CHECKS FAILED\n" : "ALL CHECKS PASSED\n");
    return g_fail;
}
