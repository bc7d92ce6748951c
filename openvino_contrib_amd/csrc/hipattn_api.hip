// C ABI of libhipattn (include/hipattn.h): argument validation, kernel dispatch and a thin
// layer over the HIP runtime.  Nothing here throws; failures come back as status codes with
// a per-thread message.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "hipattn.h"
#include "kernels.hpp"

#define HIPATTN_EXPORT extern "C" __attribute__((visibility("default")))

namespace {

thread_local char g_error[512] = "";
thread_local const char* g_kernel_path = "none";
thread_local hipattn::KernelProbe g_probe;

hipattn_status fail(hipattn_status st, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return st;
}

hipattn_status hip_fail(hipError_t e, const char* what) {
    return fail(HIPATTN_HIP_ERROR, "%s: %s (%s)", what, hipGetErrorString(e), hipGetErrorName(e));
}

#define HIP_TRY(expr)                                   \
    do {                                                \
        hipError_t e_ = (expr);                         \
        if (e_ != hipSuccess) return hip_fail(e_, #expr); \
    } while (0)

inline hipStream_t as_stream(hipattn_stream s) { return reinterpret_cast<hipStream_t>(s); }
inline hipEvent_t as_event(hipattn_event e) { return reinterpret_cast<hipEvent_t>(e); }

bool is_float_dtype(int d) { return d == HIPATTN_F32 || d == HIPATTN_F16 || d == HIPATTN_BF16; }

float resolve_scale(float scale, int head_dim) { return scale > 0.0f ? scale : 1.0f / std::sqrt((float)head_dim); }

hipattn_status validate_sdpa(const hipattn_sdpa_desc* d) {
    if (!d) return fail(HIPATTN_INVALID_ARGUMENT, "sdpa: null descriptor");
    if (!is_float_dtype(d->dtype)) return fail(HIPATTN_INVALID_ARGUMENT, "sdpa: dtype %d is not f32/f16/bf16", d->dtype);
    if (d->batch < 0 || d->len_q < 0 || d->len_kv < 0)
        return fail(HIPATTN_INVALID_ARGUMENT, "sdpa: negative extent (batch %d, len_q %d, len_kv %d)", d->batch,
                    d->len_q, d->len_kv);
    if (d->num_heads_q <= 0 || d->num_heads_kv <= 0 || d->num_heads_q % d->num_heads_kv)
        return fail(HIPATTN_INVALID_ARGUMENT, "sdpa: num_heads_q %d must be a positive multiple of num_heads_kv %d",
                    d->num_heads_q, d->num_heads_kv);
    if (d->head_dim <= 0) return fail(HIPATTN_INVALID_ARGUMENT, "sdpa: head_dim %d", d->head_dim);
    if (d->head_dim > 512) return fail(HIPATTN_UNSUPPORTED, "sdpa: head_dim %d > 512", d->head_dim);
    return HIPATTN_OK;
}

hipattn_status validate_pa(const hipattn_pa_desc* d, bool need_q) {
    if (!d) return fail(HIPATTN_INVALID_ARGUMENT, "paged_attention: null descriptor");
    if (need_q && (!is_float_dtype(d->q_dtype) || !is_float_dtype(d->out_dtype)))
        return fail(HIPATTN_INVALID_ARGUMENT, "paged_attention: q/out dtype must be f32/f16/bf16");
    if (!is_float_dtype(d->cache_dtype) && d->cache_dtype != HIPATTN_U8)
        return fail(HIPATTN_INVALID_ARGUMENT, "paged_attention: cache dtype %d", d->cache_dtype);
    if (!(d->flags & HIPATTN_PA_SKIP_CACHE_WRITE) && !is_float_dtype(d->kv_dtype))
        return fail(HIPATTN_INVALID_ARGUMENT, "paged_attention: kv dtype %d", d->kv_dtype);
    if (d->num_heads_q <= 0 || d->num_heads_kv <= 0 || d->num_heads_q % d->num_heads_kv)
        return fail(HIPATTN_INVALID_ARGUMENT,
                    "paged_attention: num_heads_q %d must be a positive multiple of num_heads_kv %d", d->num_heads_q,
                    d->num_heads_kv);
    if (d->head_dim <= 0 || d->block_size <= 0)
        return fail(HIPATTN_INVALID_ARGUMENT, "paged_attention: head_dim %d, block_size %d", d->head_dim,
                    d->block_size);
    if (d->head_dim > 512) return fail(HIPATTN_UNSUPPORTED, "paged_attention: head_dim %d > 512", d->head_dim);
    if (d->num_blocks < 0 || d->num_tokens < 0 || d->num_seqs < 0 || d->max_context_len < 0)
        return fail(HIPATTN_INVALID_ARGUMENT, "paged_attention: negative extent");
    if (d->num_blocks == 0 && d->num_tokens > 0 && d->num_seqs > 0)
        return fail(HIPATTN_INVALID_ARGUMENT, "paged_attention: %d tokens but a cache of no blocks", d->num_tokens);
    if (d->decode_waves < 0 || d->decode_waves > 65536)
        return fail(HIPATTN_INVALID_ARGUMENT, "paged_attention: decode_waves %d outside [0, 65536]", d->decode_waves);
    if (d->cache_dtype == HIPATTN_U8 && d->head_dim % 8)
        return fail(HIPATTN_UNSUPPORTED, "paged_attention: u8 cache needs head_dim %% 8 == 0 (row alignment)");
    return HIPATTN_OK;
}

hipattn::KvWriteParams make_write_params(const hipattn_pa_desc* d, const void* k_new, const void* v_new,
                                         void* key_cache, void* value_cache, const int32_t* past_lens,
                                         const int32_t* subsequence_begins, const int32_t* block_indices,
                                         const int32_t* block_indices_begins) {
    hipattn::KvWriteParams w{};
    w.k_new = k_new;
    w.v_new = v_new;
    w.key_cache = (uint8_t*)key_cache;
    w.value_cache = (uint8_t*)value_cache;
    w.past_lens = past_lens;
    w.subsequence_begins = subsequence_begins;
    w.block_indices = block_indices;
    w.block_indices_begins = block_indices_begins;
    w.kv_dtype = d->kv_dtype;
    w.cache_dtype = d->cache_dtype;
    w.num_tokens = d->num_tokens;
    w.num_seqs = d->num_seqs;
    w.num_heads_kv = d->num_heads_kv;
    w.head_dim = d->head_dim;
    w.block_size = d->block_size;
    w.num_blocks = d->num_blocks;
    return w;
}

hipattn::PagedParams make_paged_params(const hipattn_pa_desc* d) {
    hipattn::PagedParams p{};
    p.q_dtype = d->q_dtype;
    p.cache_dtype = d->cache_dtype;
    p.out_dtype = d->out_dtype;
    p.num_heads_q = d->num_heads_q;
    p.num_heads_kv = d->num_heads_kv;
    p.head_dim = d->head_dim;
    p.block_size = d->block_size;
    p.num_blocks = d->num_blocks;
    p.num_tokens = d->num_tokens;
    p.num_seqs = d->num_seqs;
    p.max_context_len = d->max_context_len;
    p.sliding_window = d->sliding_window;
    p.scale = resolve_scale(d->scale, d->head_dim);
    p.num_waves = d->decode_waves > 0 ? d->decode_waves : 0;
    p.any_lengths = (d->flags & HIPATTN_PA_ANY_LENGTHS) ? 1 : 0;
    p.alibi_slopes = d->alibi_slopes;
    p.sinks = d->sinks;
    p.kv_share = 1;
    // (more than 16 query heads per kv head: see split_kv_heads; the forced shape-generic path keeps the heads as they are)
    if (!(d->flags & HIPATTN_PA_FORCE_GENERIC)) p = hipattn::split_kv_heads(p);
    return p;
}

}  // namespace

// ------------------------------------------------------------------------------- misc
HIPATTN_EXPORT const char* hipattn_last_error_string(void) { return g_error; }

HIPATTN_EXPORT const char* hipattn_status_string(hipattn_status status) {
    switch (status) {
        case HIPATTN_OK: return "ok";
        case HIPATTN_INVALID_ARGUMENT: return "invalid argument";
        case HIPATTN_UNSUPPORTED: return "unsupported";
        case HIPATTN_WORKSPACE_TOO_SMALL: return "workspace too small";
        case HIPATTN_HIP_ERROR: return "HIP runtime error";
        case HIPATTN_NO_DEVICE: return "no HIP device";
    }
    return "unknown status";
}

HIPATTN_EXPORT int hipattn_version(void) { return HIPATTN_VERSION_MAJOR * 1000 + HIPATTN_VERSION_MINOR; }

HIPATTN_EXPORT const char* hipattn_last_kernel_path(void) { return g_kernel_path; }

HIPATTN_EXPORT hipattn_status hipattn_profile_dominant_kernel(hipattn_event before, hipattn_event after) {
    if ((before == nullptr) != (after == nullptr))
        return fail(HIPATTN_INVALID_ARGUMENT, "profile_dominant_kernel: pass two events or two NULLs");
    g_probe.before = reinterpret_cast<hipEvent_t>(before);
    g_probe.after = reinterpret_cast<hipEvent_t>(after);
    return HIPATTN_OK;
}

HIPATTN_EXPORT hipattn_status hipattn_set_option(const char* name, int value) {
    if (!name) return fail(HIPATTN_INVALID_ARGUMENT, "set_option: null name");
    if (!hipattn::set_option(name, value)) return fail(HIPATTN_INVALID_ARGUMENT, "set_option: no option named '%s'", name);
    return HIPATTN_OK;
}

HIPATTN_EXPORT size_t hipattn_cache_row_bytes(hipattn_dtype cache_dtype, int head_dim) {
    switch (cache_dtype) {
        case HIPATTN_F32: return 4 * (size_t)head_dim;
        case HIPATTN_F16:
        case HIPATTN_BF16: return 2 * (size_t)head_dim;
        case HIPATTN_U8: return (size_t)head_dim + 8;
    }
    return 0;
}

// ----------------------------------------------------------------------- device layer
HIPATTN_EXPORT hipattn_status hipattn_device_count(int* count) {
    if (!count) return fail(HIPATTN_INVALID_ARGUMENT, "device_count: null output");
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) {
        *count = 0;
        (void)hipGetLastError();
        return fail(HIPATTN_NO_DEVICE, "hipGetDeviceCount: %s", hipGetErrorString(e));
    }
    *count = n;
    return n > 0 ? HIPATTN_OK : fail(HIPATTN_NO_DEVICE, "no HIP device visible");
}

HIPATTN_EXPORT hipattn_status hipattn_set_device(int device) {
    HIP_TRY(hipSetDevice(device));
    return HIPATTN_OK;
}

HIPATTN_EXPORT hipattn_status hipattn_get_device_info(int device, hipattn_device_info* info) {
    if (!info) return fail(HIPATTN_INVALID_ARGUMENT, "get_device_info: null output");
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, device));
    memset(info, 0, sizeof(*info));
    snprintf(info->name, sizeof(info->name), "%s", prop.name);
    // gcnArchName is "gfx950:sramecc+:xnack-"; keep the processor name only
    snprintf(info->arch, sizeof(info->arch), "%s", prop.gcnArchName);
    if (char* colon = strchr(info->arch, ':')) *colon = 0;
    info->compute_units = prop.multiProcessorCount;
    info->wavefront_size = prop.warpSize;
    info->lds_bytes_per_workgroup = (int)prop.sharedMemPerBlock;
    info->clock_mhz = prop.clockRate / 1000;
    info->global_mem_bytes = prop.totalGlobalMem;
    return HIPATTN_OK;
}

HIPATTN_EXPORT hipattn_status hipattn_stream_create(hipattn_stream* stream) {
    if (!stream) return fail(HIPATTN_INVALID_ARGUMENT, "stream_create: null output");
    hipStream_t s;
    HIP_TRY(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    *stream = reinterpret_cast<hipattn_stream>(s);
    return HIPATTN_OK;
}
HIPATTN_EXPORT hipattn_status hipattn_stream_destroy(hipattn_stream stream) {
    hipattn::release_side_stream(as_stream(stream));
    HIP_TRY(hipStreamDestroy(as_stream(stream)));
    return HIPATTN_OK;
}
HIPATTN_EXPORT hipattn_status hipattn_stream_synchronize(hipattn_stream stream) {
    HIP_TRY(hipStreamSynchronize(as_stream(stream)));
    return HIPATTN_OK;
}

HIPATTN_EXPORT hipattn_status hipattn_malloc(void** device_ptr, size_t bytes) {
    if (!device_ptr) return fail(HIPATTN_INVALID_ARGUMENT, "malloc: null output");
    *device_ptr = nullptr;
    if (bytes == 0) return HIPATTN_OK;
    HIP_TRY(hipMalloc(device_ptr, bytes));
    return HIPATTN_OK;
}
HIPATTN_EXPORT hipattn_status hipattn_free(void* device_ptr) {
    if (!device_ptr) return HIPATTN_OK;
    HIP_TRY(hipFree(device_ptr));
    return HIPATTN_OK;
}
HIPATTN_EXPORT hipattn_status hipattn_malloc_async(void** device_ptr, size_t bytes, hipattn_stream stream) {
    if (!device_ptr) return fail(HIPATTN_INVALID_ARGUMENT, "malloc_async: null output");
    *device_ptr = nullptr;
    if (bytes == 0) return HIPATTN_OK;
    HIP_TRY(hipMallocAsync(device_ptr, bytes, as_stream(stream)));
    return HIPATTN_OK;
}
HIPATTN_EXPORT hipattn_status hipattn_free_async(void* device_ptr, hipattn_stream stream) {
    if (!device_ptr) return HIPATTN_OK;
    HIP_TRY(hipFreeAsync(device_ptr, as_stream(stream)));
    return HIPATTN_OK;
}
HIPATTN_EXPORT hipattn_status hipattn_host_malloc(void** host_ptr, size_t bytes) {
    if (!host_ptr) return fail(HIPATTN_INVALID_ARGUMENT, "host_malloc: null output");
    *host_ptr = nullptr;
    if (bytes == 0) return HIPATTN_OK;
    HIP_TRY(hipHostMalloc(host_ptr, bytes, hipHostMallocDefault));
    return HIPATTN_OK;
}
HIPATTN_EXPORT hipattn_status hipattn_host_free(void* host_ptr) {
    if (!host_ptr) return HIPATTN_OK;
    HIP_TRY(hipHostFree(host_ptr));
    return HIPATTN_OK;
}

HIPATTN_EXPORT hipattn_status hipattn_memcpy_h2d_async(void* device_dst, const void* host_src, size_t bytes,
                                                       hipattn_stream stream) {
    if (bytes == 0) return HIPATTN_OK;
    if (!device_dst || !host_src) return fail(HIPATTN_INVALID_ARGUMENT, "memcpy_h2d: null pointer");
    HIP_TRY(hipMemcpyAsync(device_dst, host_src, bytes, hipMemcpyHostToDevice, as_stream(stream)));
    return HIPATTN_OK;
}
HIPATTN_EXPORT hipattn_status hipattn_memcpy_d2h_async(void* host_dst, const void* device_src, size_t bytes,
                                                       hipattn_stream stream) {
    if (bytes == 0) return HIPATTN_OK;
    if (!host_dst || !device_src) return fail(HIPATTN_INVALID_ARGUMENT, "memcpy_d2h: null pointer");
    HIP_TRY(hipMemcpyAsync(host_dst, device_src, bytes, hipMemcpyDeviceToHost, as_stream(stream)));
    return HIPATTN_OK;
}
HIPATTN_EXPORT hipattn_status hipattn_memcpy_d2d_async(void* device_dst, const void* device_src, size_t bytes,
                                                       hipattn_stream stream) {
    if (bytes == 0) return HIPATTN_OK;
    if (!device_dst || !device_src) return fail(HIPATTN_INVALID_ARGUMENT, "memcpy_d2d: null pointer");
    HIP_TRY(hipMemcpyAsync(device_dst, device_src, bytes, hipMemcpyDeviceToDevice, as_stream(stream)));
    return HIPATTN_OK;
}
HIPATTN_EXPORT hipattn_status hipattn_fill_async(void* device_dst, int byte_value, size_t bytes,
                                                 hipattn_stream stream) {
    if (bytes == 0) return HIPATTN_OK;
    if (!device_dst) return fail(HIPATTN_INVALID_ARGUMENT, "fill: null pointer");
    HIP_TRY(hipattn::launch_fill_bytes(device_dst, byte_value, bytes, as_stream(stream)));
    return HIPATTN_OK;
}

HIPATTN_EXPORT hipattn_status hipattn_add_async(void* device_out, const void* device_a, const void* device_b,
                                                int64_t count, int dtype, hipattn_stream stream) {
    if (count < 0) return fail(HIPATTN_INVALID_ARGUMENT, "add: negative count");
    if (count == 0) return HIPATTN_OK;
    if (!device_out || !device_a || !device_b) return fail(HIPATTN_INVALID_ARGUMENT, "add: null pointer");
    if (dtype != HIPATTN_I32 && !is_float_dtype(dtype)) return fail(HIPATTN_INVALID_ARGUMENT, "add: dtype %d", dtype);
    HIP_TRY(hipattn::launch_add(device_a, device_b, device_out, count, dtype == HIPATTN_I32 ? -1 : dtype, as_stream(stream)));
    return HIPATTN_OK;
}

HIPATTN_EXPORT hipattn_status hipattn_event_create(hipattn_event* event) {
    if (!event) return fail(HIPATTN_INVALID_ARGUMENT, "event_create: null output");
    hipEvent_t e;
    HIP_TRY(hipEventCreate(&e));
    *event = reinterpret_cast<hipattn_event>(e);
    return HIPATTN_OK;
}
HIPATTN_EXPORT hipattn_status hipattn_event_destroy(hipattn_event event) {
    HIP_TRY(hipEventDestroy(as_event(event)));
    return HIPATTN_OK;
}
HIPATTN_EXPORT hipattn_status hipattn_event_record(hipattn_event event, hipattn_stream stream) {
    HIP_TRY(hipEventRecord(as_event(event), as_stream(stream)));
    return HIPATTN_OK;
}
HIPATTN_EXPORT hipattn_status hipattn_event_synchronize(hipattn_event event) {
    HIP_TRY(hipEventSynchronize(as_event(event)));
    return HIPATTN_OK;
}
HIPATTN_EXPORT hipattn_status hipattn_event_elapsed_ms(hipattn_event start, hipattn_event stop, float* ms) {
    if (!ms) return fail(HIPATTN_INVALID_ARGUMENT, "event_elapsed_ms: null output");
    HIP_TRY(hipEventElapsedTime(ms, as_event(start), as_event(stop)));
    return HIPATTN_OK;
}

// ------------------------------------------------------------------------------- graphs
HIPATTN_EXPORT hipattn_status hipattn_stream_begin_capture(hipattn_stream stream) {
    if (!stream) return fail(HIPATTN_INVALID_ARGUMENT, "stream_begin_capture: the default stream cannot be captured");
    // relaxed: other threads of the process may go on using the device (allocating, copying) meanwhile
    HIP_TRY(hipStreamBeginCapture(as_stream(stream), hipStreamCaptureModeRelaxed));
    return HIPATTN_OK;
}
HIPATTN_EXPORT hipattn_status hipattn_stream_end_capture(hipattn_stream stream, hipattn_graph* graph) {
    if (!graph) return fail(HIPATTN_INVALID_ARGUMENT, "stream_end_capture: null output");
    *graph = nullptr;
    hipGraph_t recorded = nullptr;
    HIP_TRY(hipStreamEndCapture(as_stream(stream), &recorded));
    if (!recorded) return fail(HIPATTN_HIP_ERROR, "stream_end_capture: the capture was invalidated");
    hipGraphExec_t exec = nullptr;
    const hipError_t e = hipGraphInstantiate(&exec, recorded, nullptr, nullptr, 0);
    (void)hipGraphDestroy(recorded);
    if (e != hipSuccess) return fail(HIPATTN_HIP_ERROR, "hipGraphInstantiate: %s", hipGetErrorString(e));
    *graph = (hipattn_graph)exec;
    return HIPATTN_OK;
}
HIPATTN_EXPORT hipattn_status hipattn_graph_launch(hipattn_graph graph, hipattn_stream stream) {
    if (!graph) return fail(HIPATTN_INVALID_ARGUMENT, "graph_launch: null graph");
    HIP_TRY(hipGraphLaunch((hipGraphExec_t)graph, as_stream(stream)));
    return HIPATTN_OK;
}
HIPATTN_EXPORT hipattn_status hipattn_graph_destroy(hipattn_graph graph) {
    if (graph) HIP_TRY(hipGraphExecDestroy((hipGraphExec_t)graph));
    return HIPATTN_OK;
}

// ------------------------------------------------------------------------------- SDPA
HIPATTN_EXPORT hipattn_status hipattn_sdpa_workspace_size(const hipattn_sdpa_desc* desc, size_t* bytes) {
    if (!bytes) return fail(HIPATTN_INVALID_ARGUMENT, "sdpa_workspace_size: null output");
    *bytes = 0;
    return validate_sdpa(desc);
}

HIPATTN_EXPORT hipattn_status hipattn_sdpa_masked(const hipattn_sdpa_desc* desc, const void* q, const void* k,
                                                  const void* v, const hipattn_mask_desc* mask_desc, const void* mask,
                                                  void* out, void* workspace, size_t workspace_bytes,
                                                  hipattn_stream stream) {
    (void)workspace;
    (void)workspace_bytes;
    if (hipattn_status st = validate_sdpa(desc)) return st;
    if ((mask == nullptr) != (mask_desc == nullptr))
        return fail(HIPATTN_INVALID_ARGUMENT, "sdpa: a mask needs a mask descriptor and the other way round");
    if (mask_desc) {
        if (!is_float_dtype(mask_desc->dtype) && mask_desc->dtype != HIPATTN_U8)
            return fail(HIPATTN_INVALID_ARGUMENT, "sdpa: mask dtype %d (f32, f16, bf16, or u8 for boolean)", mask_desc->dtype);
        for (int i = 0; i < 4; i++)
            if (mask_desc->stride[i] < 0) return fail(HIPATTN_INVALID_ARGUMENT, "sdpa: negative mask stride");
    }
    const int64_t out_elems = (int64_t)desc->batch * desc->num_heads_q * desc->len_q * desc->head_dim;
    if (out_elems == 0) return HIPATTN_OK;
    if (!q || !out) return fail(HIPATTN_INVALID_ARGUMENT, "sdpa: null q/out");
    if (desc->len_kv > 0 && (!k || !v)) return fail(HIPATTN_INVALID_ARGUMENT, "sdpa: null k/v");
    hipattn::SdpaParams p{};
    p.q = q;
    p.k = k;
    p.v = v;
    p.out = out;
    p.dtype = desc->dtype;
    p.batch = desc->batch;
    p.num_heads_q = desc->num_heads_q;
    p.num_heads_kv = desc->num_heads_kv;
    p.len_q = desc->len_q;
    p.len_kv = desc->len_kv;
    p.head_dim = desc->head_dim;
    p.causal = desc->causal != 0;
    p.scale = resolve_scale(desc->scale, desc->head_dim);
    if (mask && !p.causal) {  // the operator ignores attention_mask when causal is set
        p.mask = mask;
        p.mask_dtype = mask_desc->dtype;
        for (int i = 0; i < 4; i++) p.mask_stride[i] = mask_desc->stride[i];
    }
    if (hipattn::sdpa_flash_supported(p) && (!p.mask || hipattn::sdpa_flash_mask_supported(p))) {
        g_kernel_path = p.mask ? "sdpa_flash_mfma_masked" : "sdpa_flash_mfma";
        HIP_TRY(hipattn::launch_sdpa_flash(p, as_stream(stream), g_probe));
    } else if (hipattn::sdpa_flash_small_supported(p)) {
        g_kernel_path = p.head_dim == 64 ? "sdpa_flash_mfma_d64" : "sdpa_flash_mfma_small";
        HIP_TRY(hipattn::launch_sdpa_flash_small(p, as_stream(stream), g_probe));
    } else {
        g_kernel_path = "sdpa_generic";
        HIP_TRY(hipattn::launch_sdpa_generic(p, as_stream(stream)));
    }
    return HIPATTN_OK;
}

HIPATTN_EXPORT hipattn_status hipattn_sdpa(const hipattn_sdpa_desc* desc, const void* q, const void* k, const void* v,
                                           void* out, void* workspace, size_t workspace_bytes,
                                           hipattn_stream stream) {
    return hipattn_sdpa_masked(desc, q, k, v, nullptr, nullptr, out, workspace, workspace_bytes, stream);
}

// ------------------------------------------------------------------- paged attention
HIPATTN_EXPORT hipattn_status hipattn_kv_cache_write(const hipattn_pa_desc* desc, const void* k_new, const void* v_new,
                                                     void* key_cache, void* value_cache, const int32_t* past_lens,
                                                     const int32_t* subsequence_begins, const int32_t* block_indices,
                                                     const int32_t* block_indices_begins, hipattn_stream stream) {
    if (hipattn_status st = validate_pa(desc, false)) return st;
    if (!is_float_dtype(desc->kv_dtype)) return fail(HIPATTN_INVALID_ARGUMENT, "kv_cache_write: kv dtype %d", desc->kv_dtype);
    if (desc->num_tokens == 0 || desc->num_seqs == 0) return HIPATTN_OK;
    if (!k_new || !v_new || !key_cache || !value_cache || !past_lens || !subsequence_begins || !block_indices ||
        !block_indices_begins)
        return fail(HIPATTN_INVALID_ARGUMENT, "kv_cache_write: null pointer");
    hipattn::KvWriteParams w = make_write_params(desc, k_new, v_new, key_cache, value_cache, past_lens,
                                                 subsequence_begins, block_indices, block_indices_begins);
    HIP_TRY(hipattn::launch_kv_cache_write(w, as_stream(stream)));
    return HIPATTN_OK;
}

HIPATTN_EXPORT hipattn_status hipattn_rotate_key_cache(const hipattn_pa_desc* desc, void* key_cache,
                                                       const int32_t* rotated_block_indices, int num_rotated_blocks,
                                                       const int32_t* rotation_deltas, int deltas_per_block,
                                                       const void* rotation_trig_lut, int lut_dtype, int lut_rows,
                                                       hipattn_stream stream) {
    if (hipattn_status st = validate_pa(desc, false)) return st;
    if (num_rotated_blocks < 0 || lut_rows < 0) return fail(HIPATTN_INVALID_ARGUMENT, "rotate_key_cache: negative count");
    if (num_rotated_blocks == 0) return HIPATTN_OK;
    if (!key_cache || !rotated_block_indices || !rotation_deltas || !rotation_trig_lut)
        return fail(HIPATTN_INVALID_ARGUMENT, "rotate_key_cache: null pointer");
    if (deltas_per_block != 1 && deltas_per_block != desc->block_size)
        return fail(HIPATTN_INVALID_ARGUMENT, "rotate_key_cache: %d deltas per block (1 or block_size = %d)", deltas_per_block, desc->block_size);
    if (!is_float_dtype(lut_dtype)) return fail(HIPATTN_INVALID_ARGUMENT, "rotate_key_cache: table dtype %d", lut_dtype);
    if (desc->head_dim % 2 != 0) return fail(HIPATTN_UNSUPPORTED, "rotate_key_cache: odd head size %d", desc->head_dim);
    hipattn::KeyRotationParams p{};
    p.key_cache = (uint8_t*)key_cache;
    p.rotated_block_indices = rotated_block_indices;
    p.rotation_deltas = rotation_deltas;
    p.trig_lut = rotation_trig_lut;
    p.lut_dtype = lut_dtype;
    p.lut_rows = lut_rows;
    p.num_rotated = num_rotated_blocks;
    p.deltas_per_block = deltas_per_block;
    p.cache_dtype = desc->cache_dtype;
    p.num_heads_kv = desc->num_heads_kv;
    p.head_dim = desc->head_dim;
    p.block_size = desc->block_size;
    p.num_blocks = desc->num_blocks;
    HIP_TRY(hipattn::launch_rotate_key_cache(p, as_stream(stream)));
    return HIPATTN_OK;
}

HIPATTN_EXPORT hipattn_status hipattn_paged_attention_workspace_size(const hipattn_pa_desc* desc, size_t* bytes) {
    if (!bytes) return fail(HIPATTN_INVALID_ARGUMENT, "paged_attention_workspace_size: null output");
    *bytes = 0;
    if (hipattn_status st = validate_pa(desc, true)) return st;
    hipattn::PagedParams p = make_paged_params(desc);
    if (desc->flags & HIPATTN_PA_FORCE_GENERIC) return HIPATTN_OK;
    if (hipattn::paged_fast_supported(p))
        *bytes = hipattn::paged_fast_workspace_bytes(p);
    else if (hipattn::paged_tiles_supported(p))  // (pointers are not known here: a call with unaligned ones needs none)
        *bytes = hipattn::paged_tiles_workspace_bytes(p);
    return HIPATTN_OK;
}

namespace {
// Body of both paged-attention entry points.  static_scratch: the workspace is the library's
// static device array and nothing may be allocated or created on the way.
hipattn_status paged_attention_impl(const hipattn_pa_desc* desc, const void* q, const void* k_new, const void* v_new,
                                    void* key_cache, void* value_cache, const int32_t* past_lens,
                                    const int32_t* subsequence_begins, const int32_t* block_indices,
                                    const int32_t* block_indices_begins, void* out, void* workspace,
                                    size_t workspace_bytes, hipattn_stream stream, bool static_scratch) {
    if (hipattn_status st = validate_pa(desc, true)) return st;
    if (desc->num_tokens == 0 || desc->num_seqs == 0) return HIPATTN_OK;
    if (!q || !out || !key_cache || !value_cache || !past_lens || !subsequence_begins || !block_indices ||
        !block_indices_begins)
        return fail(HIPATTN_INVALID_ARGUMENT, "paged_attention: null pointer");
    const bool do_write = !(desc->flags & HIPATTN_PA_SKIP_CACHE_WRITE);
    if (do_write && (!k_new || !v_new)) return fail(HIPATTN_INVALID_ARGUMENT, "paged_attention: null k_new/v_new");
    hipattn::KvWriteParams w = make_write_params(desc, k_new, v_new, key_cache, value_cache, past_lens,
                                                 subsequence_begins, block_indices, block_indices_begins);
    hipattn::PagedParams p = make_paged_params(desc);
    p.q = q;
    p.key_cache = (const uint8_t*)key_cache;
    p.value_cache = (const uint8_t*)value_cache;
    p.past_lens = past_lens;
    p.subsequence_begins = subsequence_begins;
    p.block_indices = block_indices;
    p.block_indices_begins = block_indices_begins;
    p.out = out;
    p.no_side_stream = static_scratch ? 1 : 0;  // (creating the side stream of a mixed batch allocates)
    // the caller's workspace, or the static scratch, checked against what the chosen path needs
    const auto take_workspace = [&](size_t need) -> hipattn_status {
        if (static_scratch) {
            if (need > (size_t)HIPATTN_NOALLOC_SCRATCH_BYTES)
                return fail(HIPATTN_WORKSPACE_TOO_SMALL,
                            "paged_attention_noalloc: this batch needs %zu bytes of scratch, the static scratch holds %zu; "
                            "use hipattn_paged_attention with a workspace", need, (size_t)HIPATTN_NOALLOC_SCRATCH_BYTES);
            HIP_TRY(hipattn::paged_static_scratch(&workspace, &workspace_bytes));
        }
        if (need > 0 && (!workspace || workspace_bytes < need))
            return fail(HIPATTN_WORKSPACE_TOO_SMALL, "paged_attention: workspace %zu bytes, need %zu", workspace_bytes,
                        need);
        if ((uintptr_t)workspace % 16)
            return fail(HIPATTN_INVALID_ARGUMENT, "paged_attention: workspace must be 16-byte aligned");
        return HIPATTN_OK;
    };
    const bool forced_generic = (desc->flags & HIPATTN_PA_FORCE_GENERIC) != 0;
    if (!forced_generic && hipattn::paged_fast_supported(p)) {
        if (hipattn_status st = take_workspace(hipattn::paged_fast_workspace_bytes(p))) return st;
        hipattn::paged_fast_plan(p, workspace);
        g_kernel_path = "paged_mfma";
        HIP_TRY(hipattn::launch_paged_fast(p, do_write ? &w : nullptr, as_stream(stream), g_probe));
    } else if (!forced_generic && hipattn::paged_tiles_supported(p)) {
        if (hipattn_status st = take_workspace(hipattn::paged_tiles_workspace_bytes(p))) return st;
        g_kernel_path = "paged_mfma_tiles";
        if (do_write) HIP_TRY(hipattn::launch_kv_cache_write(w, as_stream(stream)));
        HIP_TRY(hipattn::launch_paged_tiles(p, workspace, as_stream(stream), g_probe));
    } else {
        g_kernel_path = "paged_generic";
        if (do_write) HIP_TRY(hipattn::launch_kv_cache_write(w, as_stream(stream)));
        HIP_TRY(hipattn::launch_paged_generic(p, as_stream(stream)));
    }
    return HIPATTN_OK;
}
}  // namespace

HIPATTN_EXPORT hipattn_status hipattn_paged_attention(const hipattn_pa_desc* desc, const void* q, const void* k_new,
                                                      const void* v_new, void* key_cache, void* value_cache,
                                                      const int32_t* past_lens, const int32_t* subsequence_begins,
                                                      const int32_t* block_indices,
                                                      const int32_t* block_indices_begins, void* out, void* workspace,
                                                      size_t workspace_bytes, hipattn_stream stream) {
    return paged_attention_impl(desc, q, k_new, v_new, key_cache, value_cache, past_lens, subsequence_begins,
                                block_indices, block_indices_begins, out, workspace, workspace_bytes, stream, false);
}

HIPATTN_EXPORT hipattn_status hipattn_paged_attention_noalloc(const hipattn_pa_desc* desc, const void* q,
                                                              const void* k_new, const void* v_new, void* key_cache,
                                                              void* value_cache, const int32_t* past_lens,
                                                              const int32_t* subsequence_begins,
                                                              const int32_t* block_indices,
                                                              const int32_t* block_indices_begins, void* out,
                                                              hipattn_stream stream) {
    return paged_attention_impl(desc, q, k_new, v_new, key_cache, value_cache, past_lens, subsequence_begins,
                                block_indices, block_indices_begins, out, nullptr, 0, stream, true);
}

HIPATTN_EXPORT hipattn_status hipattn_paged_attention_scores_workspace_size(const hipattn_pa_desc* desc, size_t* bytes) {
    if (!bytes) return fail(HIPATTN_INVALID_ARGUMENT, "paged_attention_scores_workspace_size: null output");
    *bytes = 0;
    if (hipattn_status st = validate_pa(desc, true)) return st;
    // (the bound the call itself will use, short of the output's capacity, which can only lower it)
    int64_t bound = (int64_t)desc->num_blocks * desc->block_size;
    if (desc->max_context_len > 0) bound = std::min<int64_t>(bound, desc->max_context_len);
    *bytes = hipattn::paged_scores_workspace(desc->q_dtype, desc->cache_dtype, desc->head_dim, desc->block_size, desc->num_heads_q,
                                             desc->num_heads_kv, desc->num_tokens, bound, nullptr, nullptr);
    return HIPATTN_OK;
}

HIPATTN_EXPORT hipattn_status hipattn_paged_attention_scores(const hipattn_pa_desc* desc, const void* q, const void* key_cache,
                                                             const int32_t* past_lens, const int32_t* subsequence_begins,
                                                             const int32_t* block_indices,
                                                             const int32_t* block_indices_begins,
                                                             const int32_t* score_aggregation_window, float* scores,
                                                             int64_t scores_capacity, void* workspace,
                                                             size_t workspace_bytes, hipattn_stream stream) {
    if (hipattn_status st = validate_pa(desc, true)) return st;
    if (scores_capacity < 0) return fail(HIPATTN_INVALID_ARGUMENT, "paged_attention_scores: negative capacity");
    if (desc->num_tokens == 0 || desc->num_seqs == 0 || scores_capacity == 0) return HIPATTN_OK;
    if (!q || !key_cache || !past_lens || !subsequence_begins || !block_indices || !block_indices_begins || !scores)
        return fail(HIPATTN_INVALID_ARGUMENT, "paged_attention_scores: null pointer");
    if (desc->num_seqs > 65535) return fail(HIPATTN_UNSUPPORTED, "paged_attention_scores: %d sequences (at most 65535)", desc->num_seqs);
    if (desc->alibi_slopes) return fail(HIPATTN_UNSUPPORTED, "paged_attention_scores: no distance bias (alibi_slopes) in the scores kernels");
    if (desc->sinks) return fail(HIPATTN_UNSUPPORTED, "paged_attention_scores: no attention sinks in the scores kernels");
    const size_t need = (size_t)desc->num_tokens * desc->num_heads_q * sizeof(float);
    if (!workspace || workspace_bytes < need)
        return fail(HIPATTN_WORKSPACE_TOO_SMALL, "paged_attention_scores: workspace of %zu bytes, %zu needed", workspace_bytes, need);
    if ((uintptr_t)workspace % 4) return fail(HIPATTN_INVALID_ARGUMENT, "paged_attention_scores: workspace must be 4-byte aligned");
    hipattn::ScoresParams p{};
    p.q = q;
    p.key_cache = (const uint8_t*)key_cache;
    p.past_lens = past_lens;
    p.subsequence_begins = subsequence_begins;
    p.block_indices = block_indices;
    p.block_indices_begins = block_indices_begins;
    p.score_window = score_aggregation_window;
    p.scores = scores;
    p.scores_capacity = scores_capacity;
    p.lse = (float*)workspace;
    p.q_dtype = desc->q_dtype;
    p.cache_dtype = desc->cache_dtype;
    p.num_heads_q = desc->num_heads_q;
    p.num_heads_kv = desc->num_heads_kv;
    p.head_dim = desc->head_dim;
    p.block_size = desc->block_size;
    p.num_blocks = desc->num_blocks;
    p.num_tokens = desc->num_tokens;
    p.num_seqs = desc->num_seqs;
    // no sequence is longer than its share of the cache, nor than the output
    int64_t bound = (int64_t)desc->num_blocks * desc->block_size;
    if (desc->max_context_len > 0) bound = std::min<int64_t>(bound, desc->max_context_len);
    bound = std::min<int64_t>(bound, scores_capacity);
    p.max_context_len = (int)std::min<int64_t>(bound, 0x7fffffff);
    p.sliding_window = desc->sliding_window;
    p.scale = desc->scale > 0.f ? desc->scale : 1.0f / sqrtf((float)desc->head_dim);
    // the matrix-core form when the workspace holds its raw scores (a caller that sized the workspace for the
    // log-sum-exps alone gets the fp32 kernels)
    size_t lse_bytes = 0, part_bytes = 0;
    const size_t full = hipattn::paged_scores_workspace(p.q_dtype, p.cache_dtype, p.head_dim, p.block_size, p.num_heads_q, p.num_heads_kv,
                                                        p.num_tokens, p.max_context_len, &lse_bytes, &part_bytes);
    if (part_bytes != 0 && workspace_bytes >= full && (((uintptr_t)workspace | (uintptr_t)key_cache | (uintptr_t)q) & 15) == 0) {
        p.part = (float2*)((uint8_t*)workspace + lse_bytes);
        p.raw = (float*)((uint8_t*)workspace + lse_bytes + part_bytes);
        p.raw_stride = (int)((full - lse_bytes - part_bytes) / sizeof(float) / ((size_t)p.num_tokens * p.num_heads_q));
    }
    g_kernel_path = p.raw ? "scores_mfma" : "scores_fp32";
    HIP_TRY(hipattn::launch_paged_scores(p, as_stream(stream)));
    return HIPATTN_OK;
}

