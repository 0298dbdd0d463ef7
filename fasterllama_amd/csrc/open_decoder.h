// Host-side C++ mirror of FasterLLaMA's decoder-layer API for the MI355X build.
//
// Keeps the public names, template parameters, argument order and ownership rules of
//   fasterLlama/open_decoder.h:8-23   DecoderInitParam
//   fasterLlama/open_decoder.h:26-79  OpenDecoder {ctor, initialize, getWorkspaceSize, forward}
//   fasterLlama/cuda/common.h:9-47    OperationType and the weight structs
// so a caller written against the reference compiles against this header.  Only the attention
// segment of forward() (open_decoder.cu:138-246) is implemented here — by one call into the C ABI of
// libfl_decode_attn: the decode step (seq_len == 1) and the prompt phase (seq_len > 1).  The stages
// before it (RMSNorm + INT8 Q/K/V projections, open_decoder.cu:92-136) and after it (output
// projection and FFN, open_decoder.cu:256-346) are dense INT8 GEMM work outside this library;
// forward() reaches them through the two callbacks of DecoderExternalStages.
//
// Differences a caller sees, all forced by the platform or by defects of the reference:
//   - DecoderInitParam::stream is a hipStream_t; cublas_handle is an opaque pointer that the
//     attention segment never touches (the GEMV pair is fused into the HIP kernels);
//   - the workspace size is also available as 64 bits (the reference's int overflows at
//     LLaMA2-7B shapes, open_decoder.cu:54-67); getWorkspaceSize() throws instead of wrapping;
//   - forward() has an overload taking half-precision caches (the reference stores FP32 only);
//   - RoPE uses table row start_pos; setLiteralRopeRow(true) restores the reference's literal
//     behaviour of reading row 0 for decode tokens (decoder_kernels.cu:440).
//   - failures surface as std::runtime_error (the type forward() rethrows, open_decoder.cu:354-357)
//     instead of printf + exit(1) (utils.h:50-80).
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <cstdint>

namespace FasterLLaMA
{

    enum class OperationType
    {
        FP32,
        FP16,
        INT8
    };

    template <typename T>
    struct ResNormWeight
    {
        T *gamma = nullptr;
        float eps = 1e-5f;
    };

    template <typename T, typename WeightType>
    struct DenseWeight
    {
        WeightType *kernel = nullptr;
        T *bias = nullptr;
        float *weight_scale = nullptr; // per output channel, absmax / 127
    };

    template <typename T, typename WeightType>
    struct AttentionWeight
    {
        DenseWeight<T, WeightType> query_weight;
        DenseWeight<T, WeightType> key_weight;
        DenseWeight<T, WeightType> value_weight;
        DenseWeight<T, WeightType> attention_output_weight;
    };

    template <typename T, typename WeightType>
    struct FFNWeight
    {
        DenseWeight<T, WeightType> w1_weight;
        DenseWeight<T, WeightType> w2_weight;
        DenseWeight<T, WeightType> w3_weight;
    };

    // Element type per OperationType (the BLAS enums of the reference's traits have no use here).
    template <OperationType Op> struct DecoderTransformerTraits;
    template <> struct DecoderTransformerTraits<OperationType::FP32> { typedef float DataType; };
    template <> struct DecoderTransformerTraits<OperationType::FP16> { typedef __half DataType; };
    template <> struct DecoderTransformerTraits<OperationType::INT8> { typedef int8_t DataType; };

    template <typename T, typename WeightType>
    class DecoderInitParam
    {
    public:
        ResNormWeight<T> attn_resnorm;
        AttentionWeight<T, WeightType> attention;

        float *attn_mask = nullptr; // [total_len, total_len] additive, or nullptr

        ResNormWeight<T> ffn_resnorm;
        FFNWeight<T, WeightType> ffn;

        void *cublas_handle = nullptr; // kept for source compatibility; unused
        hipStream_t stream = nullptr;
    };

    // The parts of a decoder layer that surround the attention segment.  Both run on `stream`.
    template <typename T>
    struct DecoderExternalStages
    {
        void *user = nullptr;
        // from_tensor [B*seq_len, hidden] -> int32 accumulators of the INT8 Q/K/V projections, each
        // [B*seq_len, head_num * size_per_head], and the per-token activation scale [B*seq_len].
        void (*qkv_projection)(void *user, const T *from_tensor, int32_t *query_buf, int32_t *key_buf,
                               int32_t *value_buf, float *from_tensor_scale_buf, int batch_size, int seq_len,
                               hipStream_t stream) = nullptr;
        // attention output, INT8 [B*seq_len, hidden] with its per-token scale [B*seq_len] -> decoder_output
        void (*post_attention)(void *user, const int8_t *attn_int8, const float *attn_scale,
                               const T *from_tensor, T *decoder_output, int batch_size, int seq_len,
                               hipStream_t stream) = nullptr;
    };

    template <OperationType OpType_, OperationType QuantizationType>
    class OpenDecoder
    {
    private:
        typedef DecoderTransformerTraits<OpType_> Traits_;
        typedef DecoderTransformerTraits<QuantizationType> weight_Traits_;
        typedef typename Traits_::DataType DataType_;
        typedef typename weight_Traits_::DataType weight_DataType_;

        DecoderInitParam<DataType_, weight_DataType_> param_;
        DecoderExternalStages<DataType_> stages_;

        int batch_size_;
        int max_prompt_len_;
        int max_gen_len_;
        int total_len_;
        int head_num_;
        int size_per_head_;
        int hidden_units_;
        int ffn_hidden_units_;
        bool literal_rope_row_ = false;
        int nsplit_ = 0;

        // carved from the caller's workspace by initialize(); names follow open_decoder.h:53-64
        // (tokens = batch_size * max_prompt_len)
        int8_t *from_tensor_int8_buf_ = nullptr;  // [tokens, hidden] attention output, quantised
        float *from_tensor_scale_buf_ = nullptr;  // [tokens]
        int32_t *query_buf_ = nullptr;            // [tokens, hidden]
        int32_t *key_buf_ = nullptr;              // [tokens, hidden]
        int32_t *value_buf_ = nullptr;            // [tokens, hidden]
        float *qkv_buf_ = nullptr;                // [tokens] output scales of the quantised attention output
        char *attn_workspace_ = nullptr;          // scratch of the decode-step kernels (split partials, arrival counters)
        size_t attn_workspace_bytes_ = 0;
        char *prompt_workspace_ = nullptr;        // scratch of the prompt-phase kernels
        size_t prompt_workspace_bytes_ = 0;
        char *mask_classes_ = nullptr;            // tile classes of param_.attn_mask, see classifyMask()
        size_t mask_classes_bytes_ = 0;
        bool mask_classified_ = false;
        const float *classified_mask_ = nullptr;  // the attn_mask pointer the table was computed from
        const char *prepared_buf_ = nullptr;      // the workspace whose arrival counters initialize() has zeroed

        size_t decodeWorkspaceBytes() const;
        size_t promptWorkspaceBytes() const;

        template <typename CacheT>
        void attentionSegment(const float *freq_cis, CacheT *key_cache, CacheT *value_cache, int start_pos, int seq_len,
                              const void *q, const void *k, const void *v, bool int32_inputs, float *out_float,
                              int8_t *out_int8, float *out_scale);
        template <typename CacheT>
        void forwardImpl(const DataType_ *from_tensor, const float *freq_cis, CacheT *key_cache, CacheT *value_cache,
                         DataType_ *decoder_output, int start_pos, int seq_len);

    public:
        OpenDecoder(int batch_size, int max_prompt_len, int max_gen_len, int head_num, int size_per_head,
                    int ffn_hidden_units);

        void initialize(DecoderInitParam<DataType_, weight_DataType_> param, char *buf);

        int getWorkspaceSize();
        size_t getWorkspaceSizeBytes() const;

        /**
         * key_cache_, value_cache_: [batch_size, head_num, total_len_, size_per_head]
         * freq_cis: [rows >= start_pos + seq_len, size_per_head]
         * seq_len == 1: decode step; 1 < seq_len <= max_prompt_len: prompt phase.
         */
        void forward(const DataType_ *from_tensor, const float *freq_cis, float *key_cache_, float *value_cache_,
                     DataType_ *decoder_output, const int start_pos, const int seq_len);
        void forward(const DataType_ *from_tensor, const float *freq_cis, __half *key_cache_, __half *value_cache_,
                     DataType_ *decoder_output, const int start_pos, const int seq_len);

        // ---- additions -------------------------------------------------------------------------
        void setExternalStages(const DecoderExternalStages<DataType_> &stages) { stages_ = stages; }
        void setLiteralRopeRow(bool literal) { literal_rope_row_ = literal; }
        void setContextSplits(int nsplit) // 0 = chosen by the library; the scratch areas are sized anew by the next initialize()
        {
            if (nsplit != nsplit_) prepared_buf_ = nullptr;
            nsplit_ = nsplit;
        }
        // Classifies the tiles of param_.attn_mask once (on param_.stream), so that prompt-phase calls do not
        // classify the rows they use on every call.  Call it after the mask has been filled, and again when its
        // contents change; without it every prompt-phase call classifies for itself.
        void classifyMask();

        // The attention segment alone on explicit operands: q/k/v are the float (or half, matching the
        // cache type) outputs of the projections, [B, 1, head_num, size_per_head]; attn_out is
        // [B, head_num * size_per_head] float.  Uses param_.attn_mask and param_.stream.
        void decodeAttention(const float *q, const float *k, const float *v, const float *freq_cis, float *key_cache_,
                             float *value_cache_, float *attn_out, int start_pos);
        void decodeAttention(const __half *q, const __half *k, const __half *v, const float *freq_cis,
                             __half *key_cache_, __half *value_cache_, float *attn_out, int start_pos);

        ~OpenDecoder();
    };

} // namespace FasterLLaMA
