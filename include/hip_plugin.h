/*
 * C facade over the plugin layer (libhip_plugin.so): Plugin / CompiledModel / InferRequest of the
 * "HIP" device for single-operator models.  It exists so that tests, written in Python, can
 * drive the C++ classes the way the reference's own tests drive theirs
 * (modules/nvidia_plugin/tests/unit/dynamic_shape.cpp:165-172 constructs Plugin directly,
 * compiles a model, creates an infer request, sets tensors, infers and compares).  The classes
 * behind it derive from OpenVINO's ov::IPlugin / ov::ICompiledModel / ov::ISyncInferRequest /
 * ov::IAsyncInferRequest; the Plugin object comes from the exported create_plugin_engine()
 * (src/cuda_create_plugin.cpp:11-12), which is all an ov::Core needs.
 *
 * All functions return 0 on success and a non-zero code on failure (1 ov::Exception, 2 other
 * exception, 3 ov::NotImplemented, 4 ov::Cancelled, 5 ov::Busy); hip_plugin_last_error() then
 * holds the exception text.  dtype arguments are hipattn_dtype values, HIP_PLUGIN_I32 for index
 * tensors, HIP_PLUGIN_BOOL for boolean masks, HIP_PLUGIN_I64 / HIP_PLUGIN_I8 for what Convert may produce.
 */
#ifndef HIP_PLUGIN_H_
#define HIP_PLUGIN_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HIP_PLUGIN_I32 100
#define HIP_PLUGIN_BOOL 101
#define HIP_PLUGIN_I64 102
#define HIP_PLUGIN_I8 103

typedef struct hip_plugin_s hip_plugin_t;
typedef struct hip_model_s hip_model_t;
typedef struct hip_compiled_model_s hip_compiled_model_t;
typedef struct hip_infer_request_s hip_infer_request_t;

const char* hip_plugin_last_error(void);

/* Plugin (src/cuda_plugin.hpp:18-55) */
int hip_plugin_create(hip_plugin_t** plugin); /* through create_plugin_engine() */
void hip_plugin_destroy(hip_plugin_t* plugin);
int hip_plugin_device_name(hip_plugin_t* plugin, char* value, size_t value_size);
int hip_plugin_set_property(hip_plugin_t* plugin, const char* key, const char* value);
int hip_plugin_get_property(hip_plugin_t* plugin, const char* key, char* value, size_t value_size);
/* properties: "KEY=VALUE;KEY=VALUE" or NULL */
int hip_plugin_compile_model(hip_plugin_t* plugin, hip_model_t* model, const char* properties,
                             hip_compiled_model_t** compiled);
/* a stream written by hip_compiled_model_export: [u64 size][model][u64 size][weights]
 * (src/cuda_plugin.cpp:99-138) */
int hip_plugin_import_model(hip_plugin_t* plugin, const void* blob, size_t blob_bytes, const char* properties,
                            hip_compiled_model_t** compiled);
/* writes the friendly names of the supported nodes, separated by ',' */
int hip_plugin_query_model(hip_plugin_t* plugin, hip_model_t* model, char* names, size_t names_size);
/* comma-separated operator type names in the registry (src/cuda_operation_registry.hpp:133-137) */
int hip_plugin_registered_operations(char* names, size_t names_size);

/* Single-operator models, as the reference's functional test builds them
 * (tests/functional/shared_tests_instances/single_layer_tests/scaled_dot_product_attention.cpp:48-62).
 * Shapes may hold -1 for dynamic dimensions.
 * SDPA: mask_dtype < 0: no attention_mask input (mask_rank / mask_shape ignored); scale_mode 0: no
 * scale input, 1: a scalar f32 Parameter named "scale", 2: a Constant holding scale_value.  Inputs
 * appear in the operator's order: query, key, value [, attention_mask [, scale]]. */
int hip_model_create_sdpa(int dtype, int rank, const int64_t* q_shape, const int64_t* kv_shape, int causal,
                          int mask_dtype, int mask_rank, const int64_t* mask_shape, int scale_mode, float scale_value,
                          hip_model_t** model);
/* PagedAttentionExtension with its 13 inputs as Parameters named query, key, value, key_cache,
 * value_cache, past_lens, subsequence_begins, block_indices, block_indices_begins, scale,
 * sliding_window, alibi_slopes, max_context_len.  alibi_len > 0 declares alibi slopes (unsupported).
 * num_extra_inputs more Parameters follow in the operator's order (score_aggregation_window,
 * rotated_block_indices, rotation_deltas, rotation_trig_lut, xattention_threshold,
 * xattention_block_size, xattention_stride, sinks), each of static shape [extra_len].
 * with_scores_result != 0 adds a Result on output 1 (scores). */
int hip_model_create_paged_attention(int q_dtype, int kv_dtype, int cache_dtype, int num_heads_q, int num_heads_kv,
                                     int head_dim, int block_size, int alibi_len, int num_extra_inputs, int extra_len,
                                     int with_scores_result, hip_model_t** model);
/* x -> ReadValue(init_value = x, "v0") -> Add(read, x) -> Assign("v0"), Result(add): the stateful
 * model of tests/functional/shared_tests_instances/single_layer_tests/read_value_assign.cpp:52-64 */
int hip_model_create_accumulator(int dtype, int rank, const int64_t* shape, hip_model_t** model);
/* a model from the stand-in text form (the first part of what export_model writes): one node per
 * line, "<index> <type> <name> inputs=<producer>:<port>,... {key=value;...}", in topological order */
int hip_model_create_from_text(const char* text, hip_model_t** model);
/* a model holding one node of a type no plugin operator handles */
int hip_model_create_unsupported(hip_model_t** model);
void hip_model_destroy(hip_model_t* model);

/* CompiledModel (src/cuda_compiled_model.hpp:42-57) */
void hip_compiled_model_destroy(hip_compiled_model_t* compiled);
int hip_compiled_model_num_inputs(hip_compiled_model_t* compiled);
int hip_compiled_model_num_outputs(hip_compiled_model_t* compiled);
int hip_compiled_model_input_name(hip_compiled_model_t* compiled, int index, char* name, size_t name_size);
int hip_compiled_model_get_property(hip_compiled_model_t* compiled, const char* key, char* value, size_t value_size);
/* export_model (src/cuda_compiled_model.cpp:373-395); blob may be NULL to ask for the size only */
int hip_compiled_model_export(hip_compiled_model_t* compiled, void* blob, size_t blob_capacity, size_t* blob_bytes);
int hip_compiled_model_create_infer_request(hip_compiled_model_t* compiled, hip_infer_request_t** request);

/* InferRequest (src/cuda_infer_request.hpp:42-55, src/cuda_async_infer_request.cpp:26-61).  Host
 * tensors are wrapped, not copied: the memory must stay valid until the request is done.  Device
 * tensors (on_device != 0) are remote tensors of the plugin's context over the caller's device
 * pointer and are used in place: this is how the KV caches stay resident and are updated by the
 * operator, and how an output can be left on the device. */
void hip_infer_request_destroy(hip_infer_request_t* request); /* waits for a pending start_async */
int hip_infer_request_set_input(hip_infer_request_t* request, int index, void* data, int on_device, int dtype,
                                int rank, const int64_t* shape);
/* set_tensors: `count` host tensors of `shape` (first extent 1), one batch entry each, for one input */
int hip_infer_request_set_input_batch(hip_infer_request_t* request, int index, void* const* data, int count, int dtype,
                                      int rank, const int64_t* shape);
int hip_infer_request_set_output(hip_infer_request_t* request, int index, void* data, int on_device, int dtype,
                                 int rank, const int64_t* shape);
int hip_infer_request_infer(hip_infer_request_t* request);
int hip_infer_request_start_async(hip_infer_request_t* request);
int hip_infer_request_wait(hip_infer_request_t* request);   /* 4 when the request was cancelled */
int hip_infer_request_cancel(hip_infer_request_t* request);
/* shape gets up to 8 extents; *bytes the byte size of the output */
int hip_infer_request_output_info(hip_infer_request_t* request, int index, int* dtype, int* rank, int64_t* shape,
                                  size_t* bytes);
int hip_infer_request_copy_output(hip_infer_request_t* request, int index, void* dst, size_t dst_bytes);
/* get_runtime_model: "node_name|layerType|execOrder|execTimeMcs|runtimePrecision|primitiveType" per line, in
 * execution order; execTimeMcs is the average over the infers profiled so far, or "not_executed" */
int hip_compiled_model_runtime_info(hip_compiled_model_t* compiled, char* text, size_t text_size);
/* "node_name|node_type|microseconds" per line */
int hip_infer_request_profiling(hip_infer_request_t* request, char* text, size_t text_size);
/* The last infer's intermediate tensors (operator outputs that are neither views, nor constants, nor bound to
 * the caller's device memory): bytes of the one blob they were packed into by lifetime (the reference's mutable
 * blob, src/memory_manager/model/cuda_memory_model_builder.cpp:11-25), and what they take one beside the other. */
int hip_infer_request_intermediate_memory(hip_infer_request_t* request, size_t* blob_bytes, size_t* apart_bytes);
/* The packing itself, for tests: box i is bytes[i] alive from step start[i] to step end[i]; offsets[i] out,
 * returns the blob size (offsets and sizes in multiples of 256). */
size_t hip_memory_solver_pack(int count, const size_t* bytes, const int* start, const int* end, size_t* offsets);
/* variable states (query_state; src/cuda_variable_state.hpp:62-105) */
int hip_infer_request_num_states(hip_infer_request_t* request);
int hip_infer_request_state_name(hip_infer_request_t* request, int index, char* name, size_t name_size);
int hip_infer_request_state_reset(hip_infer_request_t* request, int index);
int hip_infer_request_state_info(hip_infer_request_t* request, int index, int* dtype, int* rank, int64_t* shape,
                                 size_t* bytes);
int hip_infer_request_state_get(hip_infer_request_t* request, int index, void* dst, size_t dst_bytes);
int hip_infer_request_state_set(hip_infer_request_t* request, int index, void* data, int dtype, int rank,
                                const int64_t* shape);

#ifdef __cplusplus
}
#endif
#endif /* HIP_PLUGIN_H_ */
