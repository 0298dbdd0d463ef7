/*
 * fl_decode_attn.h — C ABI of the MI355X (gfx950) decode-step self-attention library.
 *
 * One call replaces the seq_len == 1 attention segment of FasterLLaMA's
 * OpenDecoder::forward (fasterLlama/cuda/open_decoder.cu:138-239):
 *
 *   launchQKRoteEmbeddingTranspose      open_decoder.cu:142-146   decoder_kernels.cu:425-464
 *   launchDequantizedVTransposeKernel   open_decoder.cu:157-158   decoder_kernels.cu:858-884
 *   launchStoreKVcacheKernel            open_decoder.cu:170-171   decoder_kernels.cu:597-662
 *   cublasSgemvStridedBatched (Q K^T)   open_decoder.cu:194-201
 *   launchBlockSoftmaxKernel            open_decoder.cu:207-208   decoder_kernels.cu:800-848
 *   cublasSgemvStridedBatched (P V)     open_decoder.cu:231-238
 *
 * and, optionally, the two stages on either side of it:
 *   int32 -> float dequantisation of Q/K/V   decoder_kernels.cu:449-452, :875-878
 *   launchAttnQuantizedTransposeKernel       open_decoder.cu:245-246  decoder_kernels.cu:1179-1300
 *
 * Conventions
 *   - every pointer is a DEVICE pointer owned by the caller; the library allocates nothing and
 *     keeps no state between calls (reference: OpenDecoder stores raw non-owning pointers,
 *     open_decoder.cu:31-45, :360-375);
 *   - work is only enqueued on the given hipStream_t (passed as void*); no host synchronisation;
 *   - functions return FL_ATTN_OK or a negative fl_attn_status; they never exit() or throw
 *     (the reference prints and exits, utils.h:50-80, or throws a const char*,
 *     decoder_kernels.cu:588);
 *   - sizes are 64-bit where the reference's int would overflow (open_decoder.cu:54-67).
 *
 * Layouts (bit-exact with the reference)
 *   q, k_new, v_new : [B, 1, H, D]  == [B, H, 1, D] for one token  (decoder_kernels.cu:461)
 *   k_cache, v_cache: [B, H, L, D], row of token t of (b,h) at ((b*H + h)*L + t)*D
 *                     (decoder_kernels.cu:606-607)
 *   freq_cis        : [rows, D] float, row r = cos/sin interleaved (decoding_kernels.cu:100-114)
 *   attn_mask       : [L, mask_ld] float, additive; the row used is start_pos
 *                     (open_decoder.cu:207: attn_mask + start_pos * total_len_)
 *   out             : [B, H*D] float  (open_decoder.h:61)
 */
#ifndef FL_DECODE_ATTN_H
#define FL_DECODE_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum fl_attn_status {
    FL_ATTN_OK = 0,
    FL_ATTN_ERR_NULL_POINTER = -1,  /* a required pointer is NULL */
    FL_ATTN_ERR_HEAD_DIM = -2,      /* size_per_head not in {32,64,96,128,256,512,1024}
                                       (reference: throw "invalid size_per_head!") */
    FL_ATTN_ERR_SHAPE = -3,         /* non-positive B/H/L, or sizes beyond the grid limits */
    FL_ATTN_ERR_POSITION = -4,      /* start_pos (+1) does not fit in total_len, bad rope_row */
    FL_ATTN_ERR_WORKSPACE = -5,     /* workspace missing, too small or misaligned */
    FL_ATTN_ERR_DTYPE = -6,         /* dtype is neither FL_ATTN_F32 nor FL_ATTN_F16 */
    FL_ATTN_ERR_HIP = -7,           /* a HIP runtime call failed (see fl_attn_last_hip_error) */
    FL_ATTN_ERR_ALIGNMENT = -8,     /* a tensor base is not 16-byte aligned */
    FL_ATTN_ERR_ARGUMENT = -9,      /* inconsistent optional arguments */
    FL_ATTN_ERR_SCRATCH_LIMIT = -10, /* fl_decode_attn_forward_noalloc: the step needs more scratch than
                                        FL_ATTN_NOALLOC_SCRATCH_BYTES */
    FL_ATTN_ERR_STRUCT_SIZE = -11    /* struct_size of fl_attn_desc / fl_attn_io is not one this library knows:
                                        not set, or the caller was built against a newer header */
} fl_attn_status;

enum { FL_ATTN_F32 = 0, FL_ATTN_F16 = 1 };

/* fl_attn_desc.flags.
 * FL_ATTN_FLAG_FAST_PROMPT_QK (prompt phase with FL_ATTN_F16 caches only): the rotated queries enter the
 * matrix cores rounded once to fp16 instead of as an fp16 pair (value + remainder).  The first product
 * costs half the MFMAs; each score s then carries an error of about |s| * 2^-12, harmless for scores
 * of a few units and visible (1e-2 on the output) when keys are scaled so that |s| reaches 30-90. */
#define FL_ATTN_FLAG_FAST_PROMPT_QK 1

/* fl_attn_io.flags.
 * FL_ATTN_IO_WORKSPACE_READY: the workspace was prepared by fl_decode_attn_workspace_init() and nothing
 * but this library has written to it since.  A small step whose context is split (fl_attn_plan.two_pass
 * == 2) then runs as ONE launch: the workgroup that finishes the last partial of a (batch, head) pair
 * merges them (otherwise a second, small launch does). */
#define FL_ATTN_IO_WORKSPACE_READY 1

/* Bytes of device scratch fl_decode_attn_forward_noalloc holds per GPU. */
#define FL_ATTN_NOALLOC_SCRATCH_BYTES (16u << 20)

/* rope_row value meaning "rotate by the table row of each sequence's own position" */
#define FL_ATTN_ROPE_AT_POSITION (-1)

/* Both structs start with their own size as the caller's header defines it, so that they can grow at the
 * end: the library reads struct_size bytes and takes every member beyond them as zero / NULL ("not given").
 * A size below that of the first layout with this member, or above the library's own, is rejected with
 * FL_ATTN_ERR_STRUCT_SIZE instead of being read past its end.
 *   fl_attn_desc d = {sizeof d};  d.batch_size = ...;        fl_attn_io io = {sizeof io};  io.q = ...; */

/* Problem shape; mirrors the OpenDecoder constructor arguments (open_decoder.h:66). */
typedef struct fl_attn_desc {
    uint32_t struct_size;  /* sizeof(fl_attn_desc) */
    int32_t batch_size;    /* B */
    int32_t head_num;      /* H */
    int32_t size_per_head; /* D */
    int32_t total_len;     /* L = max_prompt_len + max_gen_len: rows per (b,h) in each cache */
    int32_t dtype;         /* storage type of q/k_new/v_new and of both caches */
    int32_t nsplit;        /* context splits per (b,h); 0 = chosen by the library */
    float softmax_scale;   /* 0 = 1/sqrt(D) (open_decoder.cu:208) */
    int32_t flags;         /* 0, or a combination of the FL_ATTN_FLAG_ values below */
} fl_attn_desc;

/* Per-call operands; mirrors the arguments of OpenDecoder::forward (open_decoder.h:76-77). */
typedef struct fl_attn_io {
    uint32_t struct_size; /* sizeof(fl_attn_io) */
    const void *q;      /* [B,1,H,D] dtype; int32 accumulators when qkv_inp_scale != NULL */
    const void *k_new;  /* same */
    const void *v_new;  /* same */
    void *k_cache;      /* [B,H,L,D] dtype; row start_pos is written, rows < start_pos are read */
    void *v_cache;      /* same */
    const float *freq_cis;            /* RoPE table */
    const float *attn_mask;           /* NULL = no mask (decoder_kernels.cu:814) */
    const int32_t *start_pos_per_seq; /* NULL, or [B] positions (ragged batches; an extension) */
    float *out;                       /* [B, H*D]; may be NULL when out_int8 is given */
    void *workspace;                  /* fl_decode_attn_workspace_bytes() bytes, 256-aligned */
    size_t workspace_bytes;
    int64_t mask_ld;       /* row stride of attn_mask in floats (the reference uses L); at least the number
                              of attended columns, or 0: one row shared by every position */
    int32_t start_pos;     /* tokens already cached; the new token lands in row start_pos */
    int32_t rope_row;      /* table row for RoPE, or FL_ATTN_ROPE_AT_POSITION */
    int32_t max_start_pos; /* with start_pos_per_seq: upper bound of its entries, <0 = L-1.  The launch is
                              planned for this bound; a sequence whose device-side position exceeds it
                              is treated like one outside the cache: NaN output, nothing stored */
    int32_t flags;         /* 0, or FL_ATTN_IO_ values */
    /* optional prologue: q/k_new/v_new are int32 [B,1,H,D]; x = acc*inp_scale[b]*w_scale[h*D+d] */
    const float *qkv_inp_scale;  /* [B] or NULL */
    const float *q_weight_scale; /* [H*D] */
    const float *k_weight_scale; /* [H*D] */
    const float *v_weight_scale; /* [H*D] */
    /* optional epilogue: per-row absmax INT8 quantisation of out */
    int8_t *out_int8; /* [B, H*D] or NULL; 4-byte aligned */
    float *out_scale; /* [B] (absmax/127), required with out_int8 */
    /* optional, prompt phase: tile classes of the whole attn_mask from fl_prefill_mask_classify(), so that
     * the mask is classified once per mask and not once per call (ignored by the decode step) */
    const void *mask_tile_classes;
} fl_attn_io;

/* Launch plan the library would use for a context of ctx rows (ctx = start_pos + 1). */
typedef struct fl_attn_plan {
    int32_t nsplit;       /* context splits per (b,h) */
    int32_t chunk_rows;   /* cache rows per split */
    int32_t threads;      /* threads per workgroup of the streaming kernel */
    int32_t two_pass;     /* 0: the context is not split.  1: split, a combine launch follows the streaming
                             launch.  2: split and small enough that the merge runs inside the streaming
                             launch when the workspace is ready (FL_ATTN_IO_WORKSPACE_READY) or the
                             library's own scratch is used; a combine launch otherwise */
} fl_attn_plan;

/* Bytes of scratch fl_decode_attn_forward needs for this shape (split partials; covers every
 * start_pos < L).  Replaces the attention share of OpenDecoder::getWorkspaceSize
 * (open_decoder.cu:54-67: query_out_buf_, key_out_buf_, value_out_fp_buf_, qk_buf_). */
int fl_decode_attn_workspace_bytes(const fl_attn_desc *desc, size_t *bytes);

/* The plan for a given context length (for logging and for the benchmark's byte accounting).
 * ragged != 0: the plan used when start_pos_per_seq is given and ctx = max_start_pos + 1. */
int fl_decode_attn_plan(const fl_attn_desc *desc, int32_t ctx, int32_t ragged, fl_attn_plan *plan);

/* One decode step of attention for all (batch, head) pairs. */
int fl_decode_attn_forward(const fl_attn_desc *desc, const fl_attn_io *io, void *hip_stream);

/* Same, restricted to some passes: bit 0 = streaming pass (RoPE, append, partial attention),
 * bit 1 = combine pass (merge of split partials, optional INT8 epilogue).  Lets a profiler or
 * benchmark time the bandwidth-bound kernel alone; fl_decode_attn_forward == passes 3. */
int fl_decode_attn_forward_passes(const fl_attn_desc *desc, const fl_attn_io *io, void *hip_stream,
                                  int passes);

/* Prepares a workspace for steps that carry FL_ATTN_IO_WORKSPACE_READY: zeroes its arrival counters (a small
 * kernel on the given stream; capturable).  Once per workspace, e.g. where OpenDecoder::initialize carves
 * its buffers (open_decoder.cu:31-45); every later step leaves the counters zero again.  A step that was
 * torn down half way (device reset) needs a new call. */
int fl_decode_attn_workspace_init(const fl_attn_desc *desc, void *workspace, size_t workspace_bytes,
                                  void *hip_stream);

/* fl_decode_attn_forward for callers that cannot allocate or hand over device memory at the point of the
 * call (code under HIP-graph capture, tight serving loops, harnesses that forbid hipMalloc): the split
 * partials and arrival counters live in an array of FL_ATTN_NOALLOC_SCRATCH_BYTES that is part of the
 * library's code object (one copy per GPU, held until the process ends) instead of io->workspace, which is
 * ignored together with io->workspace_bytes and FL_ATTN_IO_WORKSPACE_READY.  No counterpart in the
 * reference, whose forward() works in the buffer carved at initialize().  Same operands, results and status
 * codes as fl_decode_attn_forward, plus FL_ATTN_ERR_SCRATCH_LIMIT when the plan of the step needs more than
 * the array holds (B * H * splits * (D + 2) * 4 bytes and B * H counters; nothing when the context is not
 * split and a float output is given).  Every call on a GPU shares that
 * GPU's array: calls that may run at the same time on one GPU (two streams, two threads) race; calls in
 * stream order do not.  The first call on each GPU also looks up the array's device address
 * (hipGetSymbolAddress): make that call outside stream capture. */
int fl_decode_attn_forward_noalloc(const fl_attn_desc *desc, const fl_attn_io *io, void *hip_stream);

/* ---- prompt phase (seq_len > 1): the dense branch of the same block -------------------------------
 * Replaces, for seq_len new tokens per sequence at positions start_pos .. start_pos+seq_len-1
 * (open_decoder.cu:138-191, :207-228, :245-246):
 *   launchQKRoteEmbeddingTranspose / launchDequantizedVTransposeKernel / launchStoreKVcacheKernel,
 *   cublasGemmStridedBatchedEx (Q K^T, :181-190), launchBlockSoftmaxKernel (:207-208),
 *   cublasGemmStridedBatchedEx (P V, :218-227), launchAttnQuantizedTransposeKernel (:245-246).
 * fl_attn_io is read as follows: q/k_new/v_new are [B, seq_len, H, D] (cache dtype, or int32
 * accumulators with qkv_inp_scale [B, seq_len]); out is [B, H, seq_len, D] float (open_decoder.h:61);
 * out_int8 is [B, seq_len, H*D] with out_scale [B, seq_len]; query s uses mask row start_pos + s and
 * RoPE table row start_pos + s (rope_row == FL_ATTN_ROPE_AT_POSITION) or rope_row + s;
 * start_pos_per_seq must be NULL.  Keys are the cache rows [0, start_pos + seq_len) after the append.
 * 32 x 32 tiles of the mask whose entries are all <= -1e30 (the -FLT_MAX of samples/llama_fp16.cu:73-81)
 * are not multiplied: with finite K and V their weights are exactly 0, so no bit of the output changes.
 * Every size_per_head of the decode step is served; 256, 512 and 1024 by a kernel that splits the head
 * dimension across the waves of a workgroup (FP32 matrix instructions for both cache types).  Workspace:
 * fl_prefill_attn_workspace_bytes(). */
int fl_prefill_attn_workspace_bytes(const fl_attn_desc *desc, int32_t seq_len, size_t *bytes);
int fl_prefill_attn_forward(const fl_attn_desc *desc, const fl_attn_io *io, int32_t seq_len,
                            void *hip_stream);

/* Same, restricted to some passes: bit 0 = RoPE + cache append of the new rows (and the per-call classification of
 * the mask rows, where no class table is given), bit 1 = the attention kernel (and the optional INT8 epilogue) over
 * the cache rows as they are.  Lets a profiler or benchmark time the matrix-core kernel alone: pass 2 after a pass
 * 1 (or after a whole call) with the same operands recomputes the same output.  fl_prefill_attn_forward == passes 3.
 * (Reference: the two halves are launchQKRoteEmbeddingTranspose / launchStoreKVcacheKernel, open_decoder.cu:142-177,
 * and the GEMM - softmax - GEMM sequence, :179-228.) */
int fl_prefill_attn_forward_passes(const fl_attn_desc *desc, const fl_attn_io *io, int32_t seq_len,
                                   void *hip_stream, int passes);

/* The mask of the reference is one [L, L] array that every layer and every call reuses
 * (samples/llama_fp16.cu:139-150), so its 32 x 32 tiles can be classified (all <= -1e30 / all zero / the
 * diagonal tile of a causal mask / anything else) once: fl_prefill_mask_classify writes one byte per tile (fl_prefill_mask_classes_bytes bytes: key tile t, row
 * block r at t * ld + r, n = ceil(L/32), ld = n rounded up to a multiple of 4; the table must be 4-byte aligned),
 * for a mask with total_len rows and columns and row stride mask_ld >= total_len.  A prompt-phase call whose
 * io.mask_tile_classes points at that table, with the same attn_mask and mask_ld and a start_pos that is a
 * multiple of 32, skips its own classification launch; any other call classifies the rows it uses as before.
 * The table is valid until the mask's contents change. */
int fl_prefill_mask_classes_bytes(const fl_attn_desc *desc, size_t *bytes);
int fl_prefill_mask_classify(const fl_attn_desc *desc, const float *attn_mask, int64_t mask_ld, void *classes,
                             size_t classes_bytes, void *hip_stream);

/* RoPE table producer on the device: rows x D floats, row r = [cos(r*w_0), sin(r*w_0), ...],
 * w_i = base^(-2i/D).  Replaces launchPrecomputeFreqsCis (decoding_kernels.cu:85-135,
 * called at decoding_sampling.cu:190) with correctly rounded sincos instead of fast intrinsics. */
int fl_rope_table(float *freq_cis, int32_t rows, int32_t size_per_head, float base,
                  void *hip_stream);

/* Bytes of one layer's K (or V) cache, [B,H,L,D] in dtype: the per-layer stride a caller uses
 * to carve its arena (decoding_sampling.cu:118-119, :180, :256-257). */
int fl_kv_cache_bytes(const fl_attn_desc *desc, size_t *bytes);

const char *fl_attn_strerror(int status);

/* hipError_t of the most recent failing HIP call made by this library on this thread. */
int fl_attn_last_hip_error(void);

/* Library/ABI version: major*10000 + minor*100 + patch. */
int fl_attn_version(void);

#ifdef __cplusplus
}
#endif
#endif /* FL_DECODE_ATTN_H */
