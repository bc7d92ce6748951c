/*
 * hipattn - thin C ABI over the MI355X (gfx950) attention kernels.
 *
 * This is the boundary the C++ plugin operators (SdpaOp, PagedAttentionOp), the tests
 * and the benchmark call.  Plain C: pointers, sizes and POD descriptors; no C++ or
 * framework types.  Every pointer named "device" must be device memory of the current
 * HIP device; all calls are asynchronous on the given stream unless stated; no
 * attention call allocates device memory behind the caller's back: scratch memory comes
 * in through the workspace arguments (the counterpart of the reference's
 * WorkbufferRequest, modules/nvidia_plugin/src/cuda_operation_base.hpp:114-117).  Functions return a
 * status code and never throw; hipattn_last_error_string() describes the last failure
 * on the calling thread.
 *
 * Reference citations are relative to modules/nvidia_plugin/ of openvino_contrib.
 */
#ifndef HIPATTN_H_
#define HIPATTN_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HIPATTN_VERSION_MAJOR 0
#define HIPATTN_VERSION_MINOR 4

typedef enum hipattn_status {
    HIPATTN_OK = 0,
    HIPATTN_INVALID_ARGUMENT = 1,   /* null pointer, negative size, inconsistent descriptor */
    HIPATTN_UNSUPPORTED = 2,        /* valid request this build has no kernel for */
    HIPATTN_WORKSPACE_TOO_SMALL = 3,
    HIPATTN_HIP_ERROR = 4,          /* a HIP runtime call failed; see hipattn_last_error_string */
    HIPATTN_NO_DEVICE = 5
} hipattn_status;

typedef enum hipattn_dtype {
    HIPATTN_F32 = 0,
    HIPATTN_F16 = 1,
    HIPATTN_BF16 = 2,
    HIPATTN_U8 = 3 /* KV cache only: rows of [scale f32][zero-point f32][head_dim bytes] */
} hipattn_dtype;

typedef struct hipattn_stream_t* hipattn_stream; /* a hipStream_t; NULL is the default stream */
typedef struct hipattn_event_t* hipattn_event;   /* a hipEvent_t */

typedef struct hipattn_device_info {
    char name[128];
    char arch[32];            /* "gfx950" on MI355X */
    int compute_units;
    int wavefront_size;
    int lds_bytes_per_workgroup;
    int clock_mhz;
    size_t global_mem_bytes;
} hipattn_device_info;

/* ---- device layer: replaces CUDA::Device / Stream / Allocation / Event wrappers
 *      (src/cuda/runtime.hpp:62-324, src/cuda/event.hpp:11-29) -------------------------- */

const char* hipattn_last_error_string(void);
const char* hipattn_status_string(hipattn_status status);
int hipattn_version(void); /* major * 1000 + minor */

hipattn_status hipattn_device_count(int* count);
hipattn_status hipattn_set_device(int device);
hipattn_status hipattn_get_device_info(int device, hipattn_device_info* info);

hipattn_status hipattn_stream_create(hipattn_stream* stream); /* default priority, non-blocking */
hipattn_status hipattn_stream_destroy(hipattn_stream stream);
hipattn_status hipattn_stream_synchronize(hipattn_stream stream);

/* runtime.hpp:188-229, 235, 273-281 (DefaultAllocation, Allocation, Stream::malloc) */
hipattn_status hipattn_malloc(void** device_ptr, size_t bytes);
hipattn_status hipattn_free(void* device_ptr);
hipattn_status hipattn_malloc_async(void** device_ptr, size_t bytes, hipattn_stream stream);
hipattn_status hipattn_free_async(void* device_ptr, hipattn_stream stream);
/* pinned host memory for staging (allocated, never registered) */
hipattn_status hipattn_host_malloc(void** host_ptr, size_t bytes);
hipattn_status hipattn_host_free(void* host_ptr);

/* runtime.hpp:236-252, 267-285 (Stream::upload / download / transfer / memset) */
hipattn_status hipattn_memcpy_h2d_async(void* device_dst, const void* host_src, size_t bytes, hipattn_stream stream);
hipattn_status hipattn_memcpy_d2h_async(void* host_dst, const void* device_src, size_t bytes, hipattn_stream stream);
hipattn_status hipattn_memcpy_d2d_async(void* device_dst, const void* device_src, size_t bytes, hipattn_stream stream);
/* byte fill done by a kernel (safe to record into a captured graph) */
hipattn_status hipattn_fill_async(void* device_dst, int byte_value, size_t bytes, hipattn_stream stream);

/* out = a + b over `count` elements of equal shape: the element-wise sum the reference runs as
 * AddCudaOp (src/ops/add.cpp:17-43, src/kernels/details/elementwise_binary.cuh:24-46), here for the
 * stateful models around the attention operators.  dtype: HIPATTN_F32 / F16 / BF16 (added in fp32,
 * rounded once) or HIPATTN_I32. */
#define HIPATTN_I32 100
hipattn_status hipattn_add_async(void* device_out, const void* device_a, const void* device_b, int64_t count,
                                 int dtype, hipattn_stream stream);

hipattn_status hipattn_event_create(hipattn_event* event);
hipattn_status hipattn_event_destroy(hipattn_event event);
hipattn_status hipattn_event_record(hipattn_event event, hipattn_stream stream);
hipattn_status hipattn_event_synchronize(hipattn_event event);
hipattn_status hipattn_event_elapsed_ms(hipattn_event start, hipattn_event stop, float* ms);

/* Stream capture into an executable graph: replaces CUDA::GraphCapture / CUDA::GraphExec
 * (src/cuda/graph.hpp), which the reference's CudaGraphTopologyRunner is built on
 * (src/cuda_graph_topology_runner.cpp).  Every hipattn_* and hipops_* operator call is capturable
 * (kernel launches and event fork / join only); allocation and host copies are not.
 * hipattn_stream_end_capture instantiates the recorded graph and hands back the executable. */
typedef struct hipattn_graph_t* hipattn_graph; /* a hipGraphExec_t */
hipattn_status hipattn_stream_begin_capture(hipattn_stream stream);
hipattn_status hipattn_stream_end_capture(hipattn_stream stream, hipattn_graph* graph);
hipattn_status hipattn_graph_launch(hipattn_graph graph, hipattn_stream stream);
hipattn_status hipattn_graph_destroy(hipattn_graph graph);

/* ---- v13::ScaledDotProductAttention -------------------------------------------------
 * Replaces the decomposed chain the reference executes after
 * ScaledDotProductAttentionDecomposition (src/transformer/cuda_graph_transformer.cpp:151-156):
 * MatMulOp (src/ops/matmul.cpp:185-227), scale Multiply (src/ops/multiply.cpp:43), the
 * causal mask Range/GreaterEqual/Select/Add (src/ops/select.cpp:50-91, src/ops/add.cpp:17-43),
 * SoftmaxOp (src/ops/softmax.cpp:178-193) and the second MatMulOp, with one fused kernel.
 *
 * q [batch, num_heads_q, len_q, head_dim], k and v [batch, num_heads_kv, len_kv, head_dim],
 * out like q; all contiguous and of `dtype`.  Query head h reads kv head
 * h / (num_heads_q / num_heads_kv).  causal != 0: query row i sees keys j <= i
 * (lower-triangular, top-left aligned).  scale <= 0 selects 1/sqrt(head_dim).
 * Softmax and accumulation are fp32 whatever `dtype` is. */
typedef struct hipattn_sdpa_desc {
    hipattn_dtype dtype;
    int batch;
    int num_heads_q;
    int num_heads_kv;
    int len_q;
    int len_kv;
    int head_dim;
    int causal;
    float scale;
} hipattn_sdpa_desc;

hipattn_status hipattn_sdpa_workspace_size(const hipattn_sdpa_desc* desc, size_t* bytes);
hipattn_status hipattn_sdpa(const hipattn_sdpa_desc* desc, const void* q, const void* k, const void* v, void* out,
                            void* workspace, size_t workspace_bytes, hipattn_stream stream);

/* The same operator with its optional attention_mask input, which the reference executes as the
 * Add / Select nodes of the decomposition (src/ops/add.cpp:17-43, src/ops/select.cpp:50-91).
 * The mask is addressed as [batch, num_heads_q, len_q, len_kv] through strides in elements; a
 * stride of 0 broadcasts that dimension.  dtype F32 / F16 / BF16: the value is added to the
 * scaled score; dtype U8: boolean, nonzero = the key takes part, zero = probability zero.  As the
 * operator specifies, the mask is ignored when desc->causal is set.  A query row whose keys are
 * all masked out yields zeros.  mask_desc and mask are both NULL or both set.
 * At head_dim 128 (and at the multiples of 8 below it) a mask of the operands' 16-bit type, or a boolean one, whose keys lie side by
 * side (stride[3] == 1) rides along in the tuned matrix-core kernel when the mask pointer and the
 * other strides are multiples of 16 bytes (8 elements; 16 for boolean); every other mask beside
 * 16-bit operands with a head_dim that is a multiple of 8 up to 256 takes the plain matrix-core
 * kernel; fp32 operands and larger heads take the shape-generic kernel. */
typedef struct hipattn_mask_desc {
    hipattn_dtype dtype;
    int64_t stride[4];
} hipattn_mask_desc;

hipattn_status hipattn_sdpa_masked(const hipattn_sdpa_desc* desc, const void* q, const void* k, const void* v,
                                   const hipattn_mask_desc* mask_desc, const void* mask, void* out, void* workspace,
                                   size_t workspace_bytes, hipattn_stream stream);

/* ---- PagedAttentionExtension --------------------------------------------------------
 * No counterpart in the reference (its only KV-cache mechanism is the contiguous
 * variable state, src/cuda_variable_state.hpp:135-160, src/ops/read_value.cpp:31-72,
 * src/ops/assign.cpp:29-56, and its nearest scatter is src/kernels/scatter_nd_update.cu:19-34).
 * Argument order follows the OpenVINO operator's inputs.
 *
 *   q                     [num_tokens, num_heads_q * head_dim]              q_dtype
 *   k_new, v_new          [num_tokens, num_heads_kv * head_dim]             kv_dtype
 *   key_cache,value_cache [num_blocks, num_heads_kv, block_size, row]       cache_dtype
 *                         row = head_dim elements, or for HIPATTN_U8
 *                         [scale f32][zero-point f32][head_dim bytes] per token and head
 *   past_lens             [num_seqs] i32      tokens already cached per sequence
 *   subsequence_begins    [num_seqs + 1] i32  token offsets of each sequence in this batch
 *   block_indices         [...] i32           physical block ids, sequence after sequence
 *   block_indices_begins  [num_seqs + 1] i32  offsets into block_indices
 *   out                   [num_tokens, num_heads_q * head_dim]              out_dtype
 *
 * Step 1 (unless HIPATTN_PA_SKIP_CACHE_WRITE): token i of sequence s is written at
 * logical position p = past_lens[s] + i, physical block
 * block_indices[block_indices_begins[s] + p / block_size], row p % block_size; u8 caches
 * are quantised on the fly.  Blocks outside the table or outside [0, num_blocks) are skipped.
 * Step 2: that token attends cache positions j, max(0, p - sliding_window + 1) <= j <= p
 * (all of 0..p when sliding_window <= 0).
 * All index arrays live in device memory and are only read there; the split of the work is
 * planned on the device.  max_context_len (>= max_s(past_lens[s] + q_len[s])) is advisory.
 * A sequence may contribute any number of tokens to a batch, none included.  A batch with
 * num_tokens == num_seqs is planned per token (the host cannot see the lengths, and a decode
 * step should not pay for a prefill launch that finds nothing to do): every token is a decode
 * row with its own context length, whichever sequence it belongs to, so the result is right
 * for any split of the tokens over the sequences; HIPATTN_PA_ANY_LENGTHS only changes how fast
 * such a batch runs when it does hold long multi-token sequences.
 * Kernels: 16-bit and u8 caches with a head_dim that is a multiple of 8 up to 256,
 * a block_size that is a power of two from 16 up and at most 16 query heads per kv head -- or more that split into equal groups of 8 to 16, each kv head's rows then being read once per group (multi-query models: 32, 48, 64 ... heads on one kv head) -- take the tuned matrix-core kernels (stream-K decode for single-token rows, chunked prefill over the
 * block table for multi-token sequences; fastest at head_dim 256, 128 and 64; head sizes between 64 and 128 run the head-128 kernels on rows of fewer columns); other
 * 16-bit and u8 caches with 16-bit queries, a head_dim that is a multiple of 8 up to 256 and a
 * block_size that is a power of two take a plain matrix-core kernel (query tiles over the block
 * table); anything else (fp32, larger heads) takes the shape-generic fp32 kernels.
 * A single-token row with nothing to attend (an empty block table) gets an output row of zeros.
 * A table entry outside [0, num_blocks) names no block: the positions it stands for take no part
 * (probability zero in every kernel; a new token that falls there is not stored), and a row left with
 * nothing to attend is zeros.  No kernel reads outside the cache for such an entry.
 * A mixed batch (single-token and multi-token sequences) with decode_waves == 0 runs its two
 * parts side by side: the call forks from `stream` onto a side stream that the library keeps for
 * that stream (created by the first such call on it, default priority, destroyed by
 * hipattn_stream_destroy; the library keeps at most 32, further streams share one) and joins before
 * it returns, so `stream` order is all the caller has to know, also under stream capture (make the
 * first such call on a stream outside a capture: creating a stream is not a capturable operation).  The
 * option "mixed_overlap" = 0 (hipattn_set_option) switches that off. */
enum {
    HIPATTN_PA_SKIP_CACHE_WRITE = 1, /* attention only; k_new / v_new may be NULL */
    HIPATTN_PA_FORCE_GENERIC = 2,    /* use the shape-generic kernels (testing aid) */
    HIPATTN_PA_ANY_LENGTHS = 8       /* performance hint for a batch with num_tokens == num_seqs that
                                        holds multi-token sequences beside empty ones: send those to
                                        the chunked-prefill kernel instead of treating each of their
                                        tokens as a decode row */
};

typedef struct hipattn_pa_desc {
    hipattn_dtype q_dtype;     /* F16, BF16 or F32 */
    hipattn_dtype kv_dtype;    /* type of k_new / v_new: F16, BF16 or F32 */
    hipattn_dtype cache_dtype; /* F16, BF16, F32 or U8 */
    hipattn_dtype out_dtype;   /* F16, BF16 or F32 */
    int num_heads_q;
    int num_heads_kv;
    int head_dim;
    int block_size;
    int num_blocks;
    int num_tokens;
    int num_seqs;
    int max_context_len;
    int sliding_window;
    float scale;       /* <= 0 selects 1/sqrt(head_dim) */
    int flags;         /* HIPATTN_PA_* */
    int decode_waves;  /* wavefronts the decode contexts are spread over; 0 = as many as the device keeps resident */
    /* The operator's alibi_slopes input: NULL, or num_heads_q floats in device memory.  slope[h] * (j - p) is
     * added to the scaled score of cache position j for a token at position p (ALiBi's linear distance bias;
     * sign and origin restated from the operator's documentation, not checked against OpenVINO).  The decode
     * kernels and the shape-generic kernels take it as one multiply-add per score; multi-token sequences then
     * go to the plain query-tile kernel rather than the tuned chunk kernel, one kernel after the other. */
    const float* alibi_slopes;
    /* The operator's `sinks` input: NULL, or a device pointer to num_heads_q floats, a logit per query head that
     * takes part in the softmax of every row of that head without a value row of its own ("attention sink"):
     * out = sum_j exp(s_j) v_j / (sum_j exp(s_j) + exp(sink)).  A row with nothing to attend stays zeros.  The
     * decode kernels, the query-tile kernel (which takes the multi-token sequences of such a call) and the
     * shape-generic kernels add the term where they normalise; the scores entry point refuses the call. */
    const float* sinks;
} hipattn_pa_desc;

hipattn_status hipattn_paged_attention_workspace_size(const hipattn_pa_desc* desc, size_t* bytes);
hipattn_status hipattn_paged_attention(const hipattn_pa_desc* desc, const void* q, const void* k_new,
                                       const void* v_new, void* key_cache, void* value_cache,
                                       const int32_t* past_lens, const int32_t* subsequence_begins,
                                       const int32_t* block_indices, const int32_t* block_indices_begins, void* out,
                                       void* workspace, size_t workspace_bytes, hipattn_stream stream);

/* The operator's second output, "scores": for every cache position of every sequence the
 * attention probability it received in this step, summed over the query heads and over the last
 * score_aggregation_window[s] query tokens of its sequence (all of the sequence's new tokens when
 * the pointer is NULL) - the figure a cache-eviction policy ranks tokens by.  No counterpart in the
 * reference.  scores is f32; sequence s owns the past_lens[s] + new_tokens(s) entries that follow
 * those of the sequences before it, so the caller sizes it with sum(past_lens) + num_tokens and
 * passes that as scores_capacity (nothing is written beyond it).  Call it after
 * hipattn_paged_attention of the same step, on the same stream: the cache must already hold the
 * new tokens' keys.  Positions outside a query's sliding window and keys in blocks outside the cache
 * count as probability zero, as in the attention itself.  The call needs a workspace of one float
 * per (token, query head).  The size query asks for more where that pays: for head sizes 64 and 128
 * with 16-bit queries (blocks of 16 tokens or more, query heads per kv head as for the tuned attention kernels) it adds room
 * for the scaled scores themselves, num_tokens x num_heads_q x max_context_len floats as long as that
 * stays below 256 MiB, and the call then reads the key rows once, on the matrix cores, instead of
 * twice (a decode batch of 64 sequences of 512..8,192 keys: 0.17 against 0.82 ms); with the smaller
 * workspace it runs as before.  Which tokens and heads OpenVINO aggregates over is restated from its
 * documentation, not checked against it. */
hipattn_status hipattn_paged_attention_scores_workspace_size(const hipattn_pa_desc* desc, size_t* bytes);
hipattn_status hipattn_paged_attention_scores(const hipattn_pa_desc* desc, const void* q, const void* key_cache,
                                              const int32_t* past_lens, const int32_t* subsequence_begins,
                                              const int32_t* block_indices, const int32_t* block_indices_begins,
                                              const int32_t* score_aggregation_window, float* scores,
                                              int64_t scores_capacity, void* workspace, size_t workspace_bytes,
                                              hipattn_stream stream);

/* The same operator for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the
 * reference (its operators get scratch from the memory manager's per-request blob,
 * src/cuda_operation_base.hpp:114-117).  No workspace argument: scratch is a static device array
 * of HIPATTN_NOALLOC_SCRATCH_BYTES that the library holds on every GPU it runs on, and the call
 * makes no hipMalloc / hipFree, creates no stream or event and calls no allocating routine.  A
 * batch whose plan needs more (hipattn_paged_attention_workspace_size tells) is refused with
 * HIPATTN_WORKSPACE_TOO_SMALL.  Mixed batches run their kernels one after the other on `stream`
 * (no side stream).  All calls on one GPU share the array: calls that overlap in time on one GPU,
 * on whatever streams, race; one after the other is fine. */
#define HIPATTN_NOALLOC_SCRATCH_BYTES (16u << 20)
hipattn_status hipattn_paged_attention_noalloc(const hipattn_pa_desc* desc, const void* q, const void* k_new,
                                               const void* v_new, void* key_cache, void* value_cache,
                                               const int32_t* past_lens, const int32_t* subsequence_begins,
                                               const int32_t* block_indices, const int32_t* block_indices_begins,
                                               void* out, hipattn_stream stream);

/* The operator's cache rotation (inputs rotated_block_indices, rotation_deltas, rotation_trig_lut; no
 * counterpart in the reference): the key rows of the listed cache blocks, all kv heads, are turned by the
 * rotary-embedding angle of a table row -- x'[i] = x[i] cos[i] - x[i + D/2] sin[i], x'[i + D/2] = x[i] sin[i]
 * + x[i + D/2] cos[i] for i < D/2 -- which is what moving a token by `delta` positions does to a key stored
 * with its rotary embedding applied.  rotation_deltas is [num_rotated_blocks, deltas_per_block] with
 * deltas_per_block 1 (one table row for the whole block) or block_size (one per token); rotation_trig_lut is
 * [lut_rows, head_dim] of lut_dtype (f32, f16 or bf16), a row holding head_dim / 2 cosines, then as many
 * sines.  A block id outside [0, num_blocks) and a delta outside [0, lut_rows) leave their rows as they are.
 * Computed in fp32 and stored in the cache's type (a u8 row is quantised again).  A caller runs it before
 * hipattn_paged_attention of the step, on the same stream; the value cache is not touched.  Of desc, the
 * cache type, num_heads_kv, head_dim (even), block_size and num_blocks are used.  Table layout, pairing and
 * order are restated from the operator's documentation, not checked against OpenVINO. */
hipattn_status hipattn_rotate_key_cache(const hipattn_pa_desc* desc, void* key_cache,
                                        const int32_t* rotated_block_indices, int num_rotated_blocks,
                                        const int32_t* rotation_deltas, int deltas_per_block,
                                        const void* rotation_trig_lut, int lut_dtype, int lut_rows,
                                        hipattn_stream stream);

/* Step 1 alone: the device-side KV-cache block writer. */
hipattn_status hipattn_kv_cache_write(const hipattn_pa_desc* desc, const void* k_new, const void* v_new,
                                      void* key_cache, void* value_cache, const int32_t* past_lens,
                                      const int32_t* subsequence_begins, const int32_t* block_indices,
                                      const int32_t* block_indices_begins, hipattn_stream stream);

/* Bytes of one cache row (per token and kv head) for a cache type. */
size_t hipattn_cache_row_bytes(hipattn_dtype cache_dtype, int head_dim);

/* Measurement aid (no reference counterpart; the reference's per-op profiler wraps whole
 * Execute calls with events, src/cuda_profiler.hpp:141-146).  While a pair of events is set
 * on the calling thread, hipattn_sdpa / hipattn_paged_attention record `before` immediately
 * ahead of and `after` immediately behind the launch of their dominant kernel (the flash
 * kernel, or the split-context decode kernel when the batch has decode sequences), on the
 * call's stream.  Pass NULLs to switch it off. */
hipattn_status hipattn_profile_dominant_kernel(hipattn_event before, hipattn_event after);

/* Process-wide schedule options (no reference counterpart; the reference's knobs are OpenVINO
 * properties, src/cuda_config.cpp:20-79).  value < 0 restores the default.  Names:
 *   "mixed_overlap"               1 (default): the decode part of a mixed batch runs beside the
 *                                 chunks' kernel; 0: one kernel after the other
 *   "mixed_decode_share_percent"  scales the compute units the plan gives the decode part (100)
 *   "decode_switch_cost"          block-times charged per (sequence, kv head) start when the decode
 *                                 work is cut into equal pieces (5)
 *   "decode_dyn_pieces_per_wave"  on-demand pieces per wavefront for the last quarter of the
 *                                 decode work (0 = none)
 *   "decode_fused_merge"          where pieces of several wavefronts make up one (sequence, kv head): 1 (default):
 *                                 the u8 decode kernels combine them themselves (no merge launch); 0: a merge
 *                                 launch behind every decode kernel (what 16-bit caches always get)
 *   "sdpa_padded_rows"            1 (default): dense SDPA at head sizes below 128 (multiples of 8) runs the
 *                                 tuned head-128 kernel on rows of fewer columns; 0: the plain kernels
 * HIPATTN_<NAME IN CAPITALS> in the environment gives an option its initial value; the
 * environment is read once per process. */
hipattn_status hipattn_set_option(const char* name, int value);

/* Name of the kernel path the last attention call on this thread dispatched to
 * ("flash_mfma", "generic", "decode_mfma+merge", ...).  Diagnostic only. */
const char* hipattn_last_kernel_path(void);

#ifdef __cplusplus
}
#endif
#endif /* HIPATTN_H_ */
