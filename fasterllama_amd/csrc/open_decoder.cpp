// OpenDecoder over the C ABI of libfl_decode_attn (see open_decoder.h in this directory).
#include "open_decoder.h"

#include <climits>
#include <stdexcept>
#include <string>
#include <type_traits>

#include "fl_decode_attn.h"

namespace FasterLLaMA
{
    namespace
    {
        size_t roundUp(size_t x, size_t a) { return (x + a - 1) / a * a; }

        void throwOnStatus(int status, const char *where)
        {
            if (status != FL_ATTN_OK)
                throw std::runtime_error(std::string("[FL][ERROR] ") + where + ": " + fl_attn_strerror(status));
        }

        template <typename CacheT>
        fl_attn_desc makeDesc(int B, int H, int D, int L, int nsplit)
        {
            fl_attn_desc d{};
            d.struct_size = sizeof d;
            d.batch_size = B;
            d.head_num = H;
            d.size_per_head = D;
            d.total_len = L;
            d.dtype = std::is_same<CacheT, float>::value ? FL_ATTN_F32 : FL_ATTN_F16;
            d.nsplit = nsplit;
            return d;
        }
    } // namespace

    template <OperationType OpType_, OperationType QuantizationType>
    OpenDecoder<OpType_, QuantizationType>::OpenDecoder(int batch_size, int max_prompt_len, int max_gen_len, int head_num,
                                                        int size_per_head, int ffn_hidden_units)
        : batch_size_(batch_size), max_prompt_len_(max_prompt_len), max_gen_len_(max_gen_len),
          total_len_(max_prompt_len + max_gen_len), head_num_(head_num), size_per_head_(size_per_head),
          hidden_units_(head_num * size_per_head), ffn_hidden_units_(ffn_hidden_units)
    {
    }

    // Scratch of the decode step: the larger need of the two cache types.
    template <OperationType OpType_, OperationType QuantizationType>
    size_t OpenDecoder<OpType_, QuantizationType>::decodeWorkspaceBytes() const
    {
        size_t need = 0, x = 0;
        fl_attn_desc d32 = makeDesc<float>(batch_size_, head_num_, size_per_head_, total_len_, nsplit_);
        fl_attn_desc d16 = makeDesc<__half>(batch_size_, head_num_, size_per_head_, total_len_, nsplit_);
        throwOnStatus(fl_decode_attn_workspace_bytes(&d32, &x), "getWorkspaceSize");
        need = x;
        throwOnStatus(fl_decode_attn_workspace_bytes(&d16, &x), "getWorkspaceSize");
        return x > need ? x : need;
    }

    // Scratch of the prompt phase (the same for both cache types); 0 when max_prompt_len is 1.
    template <OperationType OpType_, OperationType QuantizationType>
    size_t OpenDecoder<OpType_, QuantizationType>::promptWorkspaceBytes() const
    {
        if (max_prompt_len_ <= 1) return 0;
        size_t x = 0;
        fl_attn_desc d32 = makeDesc<float>(batch_size_, head_num_, size_per_head_, total_len_, nsplit_);
        const int st = fl_prefill_attn_workspace_bytes(&d32, max_prompt_len_, &x);
        if (st == FL_ATTN_ERR_HEAD_DIM) return 0; // a head size the prompt phase does not serve: forward() reports it
        throwOnStatus(st, "getWorkspaceSize");
        return x;
    }

    // Workspace = the buffers of the attention segment for up to batch_size * max_prompt_len tokens, each
    // 256-byte aligned: int8 attention output | activation scales | three int32 accumulator buffers |
    // output scales | scratch of the decode step | scratch of the prompt phase.  The two scratch areas
    // are kept apart: the decode area carries arrival counters that must stay zero between steps.
    template <OperationType OpType_, OperationType QuantizationType>
    size_t OpenDecoder<OpType_, QuantizationType>::getWorkspaceSizeBytes() const
    {
        const size_t tokens = (size_t)batch_size_ * (size_t)(max_prompt_len_ > 1 ? max_prompt_len_ : 1);
        size_t n = 0;
        n += roundUp(tokens * hidden_units_ * sizeof(int8_t), 256);
        n += roundUp(tokens * sizeof(float), 256);
        n += 3 * roundUp(tokens * hidden_units_ * sizeof(int32_t), 256);
        n += roundUp(tokens * sizeof(float), 256);
        size_t classes = 0;
        fl_attn_desc d = makeDesc<float>(batch_size_, head_num_, size_per_head_, total_len_, nsplit_);
        throwOnStatus(fl_prefill_mask_classes_bytes(&d, &classes), "getWorkspaceSize");
        return n + roundUp(decodeWorkspaceBytes(), 256) + roundUp(promptWorkspaceBytes(), 256) + roundUp(classes, 256) +
               256; // slack to align a caller's base pointer
    }

    template <OperationType OpType_, OperationType QuantizationType>
    int OpenDecoder<OpType_, QuantizationType>::getWorkspaceSize()
    {
        const size_t n = getWorkspaceSizeBytes();
        if (n > (size_t)INT_MAX)
            throw std::runtime_error("[FL][ERROR] getWorkspaceSize: size exceeds int, use getWorkspaceSizeBytes()");
        return (int)n;
    }

    // The reference's initialize() is pointer carving and nothing else (open_decoder.cu:25-51), and its driver
    // calls it before every layer of every step with the same buf (decoding_sampling.cu:232-258).  Same here:
    // a call with the workspace that is already prepared only copies `param`.  The one-time work — sizing the
    // scratch areas and a small kernel that zeroes the arrival counters of the decode scratch — happens on the
    // first call, and again only when `buf` changes.  The tile classes of the mask stay valid as long as
    // param.attn_mask is the pointer they were computed from (contents that change behind the same pointer are
    // the caller's classifyMask() call).
    template <OperationType OpType_, OperationType QuantizationType>
    void OpenDecoder<OpType_, QuantizationType>::initialize(DecoderInitParam<DataType_, weight_DataType_> param, char *buf)
    {
        if (!buf)
            throw std::runtime_error("[FL][ERROR] initialize: workspace is null");
        param_ = param;
        if (mask_classified_ && param_.attn_mask != classified_mask_)
            mask_classified_ = false;
        if (buf == prepared_buf_)
            return;
        const size_t tokens = (size_t)batch_size_ * (size_t)(max_prompt_len_ > 1 ? max_prompt_len_ : 1);
        char *p = reinterpret_cast<char *>(roundUp(reinterpret_cast<uintptr_t>(buf), 256));
        from_tensor_int8_buf_ = reinterpret_cast<int8_t *>(p);
        p += roundUp(tokens * hidden_units_ * sizeof(int8_t), 256);
        from_tensor_scale_buf_ = reinterpret_cast<float *>(p);
        p += roundUp(tokens * sizeof(float), 256);
        const size_t acc = roundUp(tokens * hidden_units_ * sizeof(int32_t), 256);
        query_buf_ = reinterpret_cast<int32_t *>(p);
        key_buf_ = reinterpret_cast<int32_t *>(p + acc);
        value_buf_ = reinterpret_cast<int32_t *>(p + 2 * acc);
        p += 3 * acc;
        qkv_buf_ = reinterpret_cast<float *>(p);
        p += roundUp(tokens * sizeof(float), 256);
        attn_workspace_ = p;
        attn_workspace_bytes_ = decodeWorkspaceBytes();
        p += roundUp(attn_workspace_bytes_, 256);
        prompt_workspace_ = p;
        prompt_workspace_bytes_ = promptWorkspaceBytes();
        p += roundUp(prompt_workspace_bytes_, 256);
        mask_classes_ = p;
        mask_classified_ = false; // another table address: nothing has been written there
        // arrival counters of the decode scratch start at zero (a small kernel on the caller's stream); from
        // here on a decode step whose context is split is a single launch
        fl_attn_desc d = makeDesc<float>(batch_size_, head_num_, size_per_head_, total_len_, nsplit_);
        throwOnStatus(fl_decode_attn_workspace_init(&d, attn_workspace_, attn_workspace_bytes_, param_.stream), "initialize");
        throwOnStatus(fl_prefill_mask_classes_bytes(&d, &mask_classes_bytes_), "initialize");
        prepared_buf_ = buf;
    }

    template <OperationType OpType_, OperationType QuantizationType>
    void OpenDecoder<OpType_, QuantizationType>::classifyMask()
    {
        if (!mask_classes_)
            throw std::runtime_error("[FL][ERROR] classifyMask: initialize() has not been called");
        mask_classified_ = false;
        if (!param_.attn_mask) return;
        fl_attn_desc d = makeDesc<float>(batch_size_, head_num_, size_per_head_, total_len_, nsplit_);
        throwOnStatus(fl_prefill_mask_classify(&d, param_.attn_mask, total_len_, mask_classes_, mask_classes_bytes_, param_.stream),
                      "classifyMask");
        mask_classified_ = true;
        classified_mask_ = param_.attn_mask;
    }

    template <OperationType OpType_, OperationType QuantizationType>
    template <typename CacheT>
    void OpenDecoder<OpType_, QuantizationType>::attentionSegment(const float *freq_cis, CacheT *key_cache, CacheT *value_cache,
                                                                  int start_pos, int seq_len, const void *q, const void *k,
                                                                  const void *v, bool int32_inputs, float *out_float,
                                                                  int8_t *out_int8, float *out_scale)
    {
        if (!attn_workspace_)
            throw std::runtime_error("[FL][ERROR] forward: initialize() has not been called");
        fl_attn_desc desc = makeDesc<CacheT>(batch_size_, head_num_, size_per_head_, total_len_, nsplit_);
        fl_attn_io io{};
        io.struct_size = sizeof io;
        io.q = q;
        io.k_new = k;
        io.v_new = v;
        io.k_cache = key_cache;
        io.v_cache = value_cache;
        io.freq_cis = freq_cis;
        io.attn_mask = param_.attn_mask; // row start_pos, stride total_len_ (open_decoder.cu:207)
        io.mask_ld = total_len_;
        io.out = out_float;
        io.workspace = seq_len == 1 ? attn_workspace_ : prompt_workspace_;
        io.workspace_bytes = seq_len == 1 ? attn_workspace_bytes_ : prompt_workspace_bytes_;
        io.flags = seq_len == 1 ? FL_ATTN_IO_WORKSPACE_READY : 0;
        io.mask_tile_classes = mask_classified_ ? mask_classes_ : nullptr;
        io.start_pos = start_pos;
        io.rope_row = literal_rope_row_ ? 0 : FL_ATTN_ROPE_AT_POSITION;
        io.max_start_pos = -1;
        if (int32_inputs)
        {
            io.qkv_inp_scale = from_tensor_scale_buf_;
            io.q_weight_scale = param_.attention.query_weight.weight_scale;
            io.k_weight_scale = param_.attention.key_weight.weight_scale;
            io.v_weight_scale = param_.attention.value_weight.weight_scale;
        }
        io.out_int8 = out_int8;
        io.out_scale = out_scale;
        if (seq_len == 1)
            throwOnStatus(fl_decode_attn_forward(&desc, &io, param_.stream), "decode attention");
        else
            throwOnStatus(fl_prefill_attn_forward(&desc, &io, seq_len, param_.stream), "prompt attention");
    }

    template <OperationType OpType_, OperationType QuantizationType>
    template <typename CacheT>
    void OpenDecoder<OpType_, QuantizationType>::forwardImpl(const DataType_ *from_tensor, const float *freq_cis, CacheT *key_cache,
                                                             CacheT *value_cache, DataType_ *decoder_output, int start_pos,
                                                             int seq_len)
    {
        if (seq_len < 1 || seq_len > (max_prompt_len_ > 1 ? max_prompt_len_ : 1))
            throw std::runtime_error("[FL][ERROR] forward: seq_len must be between 1 and max_prompt_len");
        if (!stages_.qkv_projection || !stages_.post_attention)
            throw std::runtime_error("[FL][ERROR] forward: the Q/K/V projection and post-attention stages are external; "
                                     "install them with setExternalStages(), or call decodeAttention()");
        // RMSNorm + quantise + INT8 Q/K/V GEMMs (open_decoder.cu:92-136) -> int32 accumulators
        stages_.qkv_projection(stages_.user, from_tensor, query_buf_, key_buf_, value_buf_, from_tensor_scale_buf_, batch_size_,
                               seq_len, param_.stream);
        // dequantise + RoPE + cache append + attention + per-token INT8 quantisation (open_decoder.cu:138-246).
        // The reference reuses from_tensor_scale_buf_ for the output scale; here the quantised output gets
        // its own slot so the activation scale stays readable.
        float *attn_scale = qkv_buf_;
        attentionSegment<CacheT>(freq_cis, key_cache, value_cache, start_pos, seq_len, query_buf_, key_buf_, value_buf_, true,
                                 nullptr, from_tensor_int8_buf_, attn_scale);
        // output projection, residual, FFN (open_decoder.cu:256-346)
        stages_.post_attention(stages_.user, from_tensor_int8_buf_, attn_scale, from_tensor, decoder_output, batch_size_,
                               seq_len, param_.stream);
    }

    template <OperationType OpType_, OperationType QuantizationType>
    void OpenDecoder<OpType_, QuantizationType>::forward(const DataType_ *from_tensor, const float *freq_cis, float *key_cache_,
                                                         float *value_cache_, DataType_ *decoder_output, const int start_pos,
                                                         const int seq_len)
    {
        forwardImpl<float>(from_tensor, freq_cis, key_cache_, value_cache_, decoder_output, start_pos, seq_len);
    }

    template <OperationType OpType_, OperationType QuantizationType>
    void OpenDecoder<OpType_, QuantizationType>::forward(const DataType_ *from_tensor, const float *freq_cis, __half *key_cache_,
                                                         __half *value_cache_, DataType_ *decoder_output, const int start_pos,
                                                         const int seq_len)
    {
        forwardImpl<__half>(from_tensor, freq_cis, key_cache_, value_cache_, decoder_output, start_pos, seq_len);
    }

    template <OperationType OpType_, OperationType QuantizationType>
    void OpenDecoder<OpType_, QuantizationType>::decodeAttention(const float *q, const float *k, const float *v, const float *freq_cis,
                                                                 float *key_cache_, float *value_cache_, float *attn_out,
                                                                 int start_pos)
    {
        attentionSegment<float>(freq_cis, key_cache_, value_cache_, start_pos, 1, q, k, v, false, attn_out, nullptr, nullptr);
    }

    template <OperationType OpType_, OperationType QuantizationType>
    void OpenDecoder<OpType_, QuantizationType>::decodeAttention(const __half *q, const __half *k, const __half *v,
                                                                 const float *freq_cis, __half *key_cache_, __half *value_cache_,
                                                                 float *attn_out, int start_pos)
    {
        attentionSegment<__half>(freq_cis, key_cache_, value_cache_, start_pos, 1, q, k, v, false, attn_out, nullptr, nullptr);
    }

    template <OperationType OpType_, OperationType QuantizationType>
    OpenDecoder<OpType_, QuantizationType>::~OpenDecoder()
    {
        // non-owning: the caller's arena holds every buffer (open_decoder.cu:360-375)
    }

    // same instantiations as the reference library (open_decoder.cu:377-383)
    template class OpenDecoder<OperationType::FP32, OperationType::INT8>;
    template class OpenDecoder<OperationType::FP16, OperationType::INT8>;
    template class DecoderInitParam<float, int8_t>;
    template class DecoderInitParam<__half, int8_t>;

} // namespace FasterLLaMA
