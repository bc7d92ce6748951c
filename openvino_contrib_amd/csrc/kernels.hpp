// Parameter blocks and host-side launchers of the attention kernels (internal to the
// library; the public boundary is include/hipattn.h).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "hipattn.h"

namespace hipattn {

struct KvWriteParams {
    const void* k_new;
    const void* v_new;
    uint8_t* key_cache;
    uint8_t* value_cache;
    const int32_t* past_lens;
    const int32_t* subsequence_begins;
    const int32_t* block_indices;
    const int32_t* block_indices_begins;
    int kv_dtype;
    int cache_dtype;
    int num_tokens;
    int num_seqs;
    int num_heads_kv;
    int head_dim;
    int block_size;
    int num_blocks;
    // kv heads one wavefront writes (set by kv_write_wavefronts): 1 for small batches, all of a
    // token's heads for large ones, where looking up the token's slot per head would dominate
    int heads_per_wave;
    // head size 128, 16-bit new rows, 16-byte aligned pointers (set by kv_write_wavefronts): a
    // wavefront writes four kv heads of a token with 16-byte loads
    int vector_rows;
};

// The operator's cache rotation: the key rows of the listed blocks turned by the angles of their table rows.
struct KeyRotationParams {
    uint8_t* key_cache;
    const int32_t* rotated_block_indices;  // [num_rotated]
    const int32_t* rotation_deltas;        // [num_rotated, deltas_per_block]
    const void* trig_lut;                  // [lut_rows, head_dim]: head_dim / 2 cosines, then as many sines
    int lut_dtype;
    int lut_rows;
    int num_rotated;
    int deltas_per_block;                  // 1 or block_size
    int cache_dtype;
    int num_heads_kv;
    int head_dim;
    int block_size;
    int num_blocks;
};
hipError_t launch_rotate_key_cache(const KeyRotationParams& p, hipStream_t stream);

// Wavefronts the writer needs for p (and p.heads_per_wave, which it sets).
inline int64_t kv_write_wavefronts(KvWriteParams& p) {
    const auto aligned16 = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
    const bool bits16 = p.kv_dtype == HIPATTN_F16 || p.kv_dtype == HIPATTN_BF16;
    const bool cache_ok = p.cache_dtype == HIPATTN_F16 || p.cache_dtype == HIPATTN_BF16 || p.cache_dtype == HIPATTN_U8;
    p.vector_rows = (p.head_dim == 128 && bits16 && cache_ok && aligned16(p.k_new) && aligned16(p.v_new) &&
                     aligned16(p.key_cache) && aligned16(p.value_cache)) ? 1 : 0;
    if (p.vector_rows) {
        p.heads_per_wave = 4;
        return (int64_t)p.num_tokens * ((p.num_heads_kv + 3) / 4);
    }
    const int64_t pairs = (int64_t)p.num_tokens * p.num_heads_kv;
    p.heads_per_wave = pairs > 16384 ? p.num_heads_kv : 1;
    return (int64_t)p.num_tokens * ((p.num_heads_kv + p.heads_per_wave - 1) / p.heads_per_wave);
}

struct SdpaParams {
    const void* q;
    const void* k;
    const void* v;
    void* out;
    int dtype;
    int batch;
    int num_heads_q;
    int num_heads_kv;
    int len_q;
    int len_kv;
    int head_dim;
    int causal;
    float scale;  // already resolved (> 0)
    // optional attention mask (nullptr: none; ignored when causal), broadcast over [batch, head, query, key]
    // by strides in elements; F32 / F16 / BF16 are added to the scaled scores, U8 is boolean (nonzero = attend)
    const void* mask;
    int mask_dtype;
    int64_t mask_stride[4];
};

struct PagedParams {
    const void* q;
    const uint8_t* key_cache;
    const uint8_t* value_cache;
    const int32_t* past_lens;
    const int32_t* subsequence_begins;
    const int32_t* block_indices;
    const int32_t* block_indices_begins;
    void* out;
    int q_dtype;
    int cache_dtype;
    int out_dtype;
    int num_heads_q;
    int num_heads_kv;
    int head_dim;
    int block_size;
    int num_blocks;
    int num_tokens;
    int num_seqs;
    int max_context_len;
    int sliding_window;
    float scale;  // already resolved (> 0)
    // More than 16 query heads per kv head (multi-query models): the stream-K kernels serve 16 heads per
    // (sequence, kv head) segment, so each kv head is entered kv_share times, as num_heads_kv * kv_share heads
    // of num_heads_q / that many query heads each, consecutive ones sharing the K/V rows of kv head h / kv_share
    // (split_kv_heads; 1 otherwise).  Only the K/V addresses divide by it; the chunk kernels get the heads undivided.
    int kv_share;
    const float* sinks;         // nullptr, or [num_heads_q]: a logit per query head in the denominator of every row's softmax (no value row)
    const float* alibi_slopes;  // nullptr, or [num_heads_q]: slope * (key position - query position) joins the scaled score
    // decode: the batch's block-heads are cut into num_waves equal pieces (one per wavefront);
    // pieces that do not cover a whole (sequence, kv head) segment leave partials in the workspace
    int num_waves;        // wavefronts (= single-wavefront workgroups) of the decode kernel
    int switch_cost;      // block-times a wavefront is charged for starting on a new segment
    int dyn_pieces;       // pieces of the last quarter of the work line, handed out on demand
    int dyn_groups;       // wavefront groups, each with its own ticket counter and every dyn_groups-th piece
    int32_t* dyn_counter; // [64] ticket counters (zeroed by the plan)
    // mixed batches: the decode kernel keeps only some compute units (eight wavefronts each) and the
    // chunks' flash kernel runs beside it on the others; the plan decides how many from the work
    // of the two parts and leaves the wavefront count in plan_waves[0] (num_waves is then the most
    // it may choose).  overlap_share scales the decode part's share (1 = as modelled).
    int overlap;          // 0: decode, merge and prefill kernels run one after the other
    float overlap_share;
    int32_t* plan_waves;  // [1]
    int32_t* blk_prefix;  // [num_rows + 1] exclusive prefix of work-line units of the decode rows
    void* seq_info;       // [num_rows] 32-byte records: what each decode row attends (written by the plan)
    float* part_out;      // [num_waves + dyn_pieces + num_rows*num_heads_kv, G, head_dim] unnormalised outputs
    float* part_ml;       // [same, G, 2] running max (log2 domain) and sum
    // fused_merge: the piece that holds the end of a segment combines the segment's partials inside the
    // decode kernel (no merge launch); part_flag[slot] == merge_tag says that slot's partial is complete
    int fused_merge;
    uint64_t* part_flag;  // [same]
    unsigned long long merge_tag;  // differs from call to call (and from whatever a fresh workspace holds)
    // chunked prefill: query-tile schedule built on the device
    int32_t* tile_prefix; // [num_seqs + 1] exclusive prefix of query tiles per sequence
    int max_q_tiles;      // grid upper bound
    int num_rows;         // records of the decode plan: the sequences, or (max_q_tiles == 0) the tokens
    int any_lengths;      // a batch with num_tokens == num_seqs sends its multi-token sequences to the
                          // chunked-prefill kernel too (HIPATTN_PA_ANY_LENGTHS); without it such a batch is
                          // planned per token and every token is a decode row
    int no_side_stream;   // mixed batches run one kernel after the other on the caller's stream
    int tiles_only;       // (flash_small.hip) tile_prefix counts single-token sequences too: there are no decode rows
};

// Optional event pair recorded around the dominant kernel of a call (measurement aid).
struct KernelProbe {
    hipEvent_t before = nullptr;
    hipEvent_t after = nullptr;
};

hipError_t launch_kv_cache_write(const KvWriteParams& p, hipStream_t stream);

// shape-generic fp32 VALU kernels: any head_dim <= 512, any block size, every dtype
hipError_t launch_sdpa_generic(const SdpaParams& p, hipStream_t stream);
hipError_t launch_paged_generic(const PagedParams& p, hipStream_t stream);

// MFMA flash kernels (head_dim 64 or 128, f16 / bf16)
bool sdpa_flash_supported(const SdpaParams& p);
bool sdpa_flash_mask_supported(const SdpaParams& p);  // p.mask can ride along in the flash kernel
hipError_t launch_sdpa_flash(const SdpaParams& p, hipStream_t stream, const KernelProbe& probe);
// head sizes up to 256 that are multiples of 8 on the matrix cores (flash_small.hip)
bool sdpa_flash_small_supported(const SdpaParams& p);
hipError_t launch_sdpa_flash_small(const SdpaParams& p, hipStream_t stream, const KernelProbe& probe);
// paged attention of such shapes, 16-bit caches: every sequence of the batch as query tiles over the
// block table (workspace: paged_tiles_workspace_bytes; the new tokens must be in the cache already)
bool paged_tiles_supported(const PagedParams& p);
size_t paged_tiles_workspace_bytes(const PagedParams& p);
hipError_t launch_paged_tiles(const PagedParams& p, void* workspace, hipStream_t stream, const KernelProbe& probe);

// paged attention fast paths: plan + stream-K decode + merge, and chunked prefill
bool paged_fast_supported(const PagedParams& p);
// p with its kv heads entered several times when that brings a call with more than 16 query heads per kv head
// within the stream-K kernels' reach (paged_fast_supported of the result), else p as it is.
PagedParams split_kv_heads(const PagedParams& p);
size_t paged_fast_workspace_bytes(const PagedParams& p);
void paged_fast_plan(PagedParams& p, void* workspace);  // fills chunking fields and workspace pointers
void release_side_stream(hipStream_t owner);  // drops the side stream mixed batches on `owner` used, if any
// write == nullptr skips the KV-cache write of the new tokens
hipError_t launch_paged_fast(const PagedParams& p, const KvWriteParams* write, hipStream_t stream,
                             const KernelProbe& probe);
hipError_t launch_paged_prefill(const PagedParams& p, hipStream_t stream);  // flash over the block table (needs the plan)
hipError_t launch_paged_prefill_small(const PagedParams& p, hipStream_t stream);  // the same at head size 64 (flash_small.hip)

hipError_t launch_fill_bytes(void* dst, int value, size_t bytes, hipStream_t stream);
// out = a + b over n elements; dtype is a HIPATTN_F32 / F16 / BF16 value, or -1 for int32
hipError_t launch_add(const void* a, const void* b, void* out, int64_t n, int dtype, hipStream_t stream);

// second output of PagedAttentionExtension: aggregated attention probabilities per key position
struct ScoresParams {
    const void* q;
    const uint8_t* key_cache;
    const int32_t* past_lens;
    const int32_t* subsequence_begins;
    const int32_t* block_indices;
    const int32_t* block_indices_begins;
    const int32_t* score_window;  // [num_seqs] or null: every new token of a sequence is aggregated
    float* scores;
    int64_t scores_capacity;      // floats
    float* lse;                   // [num_tokens, num_heads_q] log2-domain log-sum-exp (workspace)
    float2* part;                 // matrix-core form: [num_tokens, num_heads_q, chunks] (max, sum) per wavefront
    float* raw;                   // matrix-core form: [num_tokens, num_heads_q, raw_stride] scaled scores; null: fp32 kernels
    int raw_stride;
    int q_dtype;
    int cache_dtype;
    int num_heads_q;
    int num_heads_kv;
    int head_dim;
    int block_size;
    int num_blocks;
    int num_tokens;
    int num_seqs;
    int max_context_len;          // bound on past + new tokens of any sequence (sizes the grid)
    int sliding_window;
    float scale;                  // already resolved (> 0)
};
hipError_t launch_paged_scores(const ScoresParams& p, hipStream_t stream);
// Workspace of the scores kernels: the log-sum-exps alone (the return value when the shape stays with the fp32
// kernels or the raw scores would exceed 256 MiB), or those, the wavefronts' partial sums and the raw scores of
// the matrix-core form, in that order (lse_bytes / part_bytes: the aligned sizes of the first two areas).
size_t paged_scores_workspace(int q_dtype, int cache_dtype, int head_dim, int block_size, int heads_q, int heads_kv, int num_tokens,
                              int64_t max_context_len, size_t* lse_bytes, size_t* part_bytes);

// Schedule option by name (see paged_decode.hip); value < 0 restores the default.  false: no such option.
bool set_option(const char* name, int value);
bool sdpa_padded_rows_enabled();  // the option sdpa_padded_rows
// Address and size of the current device's copy of the static scratch array (resolved once per device).
hipError_t paged_static_scratch(void** ptr, size_t* bytes);

}  // namespace hipattn
