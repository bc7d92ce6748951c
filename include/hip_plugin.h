/*
 * C facade over the plugin layer (libhip_plugin.so): Plugin / CompiledModel / InferRequest of the
 * "HIP" device for single-operator attention models.  It exists so that tests, written in
 * Python, can drive the C++ classes the way the reference's own tests drive theirs
 * (modules/nvidia_plugin/tests/unit/dynamic_shape.cpp:165-172 constructs Plugin directly,
 * compiles a model, creates an infer request, sets tensors, infers and compares).  Under a real
 * ov::Core these entry points are replaced by OpenVINO's plugin ABI
 * (src/cuda_create_plugin.cpp:11-12): create_plugin_engine() returning the Plugin object.
 *
 * All functions return 0 on success and a non-zero code on failure;
 * hip_plugin_last_error() then holds the exception text ("file:line(function): message").
 * dtype arguments are hipattn_dtype values, or HIP_PLUGIN_I32 for index tensors.
 */
#ifndef HIP_PLUGIN_H_
#define HIP_PLUGIN_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HIP_PLUGIN_I32 100

typedef struct hip_plugin_s hip_plugin_t;
typedef struct hip_model_s hip_model_t;
typedef struct hip_compiled_model_s hip_compiled_model_t;
typedef struct hip_infer_request_s hip_infer_request_t;

const char* hip_plugin_last_error(void);

/* Plugin (src/cuda_plugin.hpp:18-55) */
int hip_plugin_create(hip_plugin_t** plugin);
void hip_plugin_destroy(hip_plugin_t* plugin);
int hip_plugin_set_property(hip_plugin_t* plugin, const char* key, const char* value);
int hip_plugin_get_property(hip_plugin_t* plugin, const char* key, char* value, size_t value_size);
/* properties: "KEY=VALUE;KEY=VALUE" or NULL */
int hip_plugin_compile_model(hip_plugin_t* plugin, hip_model_t* model, const char* properties,
                             hip_compiled_model_t** compiled);
/* writes the friendly names of the supported nodes, separated by ',' */
int hip_plugin_query_model(hip_plugin_t* plugin, hip_model_t* model, char* names, size_t names_size);
/* comma-separated operator type names in the registry (src/cuda_operation_registry.hpp:133-137) */
int hip_plugin_registered_operations(char* names, size_t names_size);

/* Single-operator models, as the reference's functional test builds them
 * (tests/functional/shared_tests_instances/single_layer_tests/scaled_dot_product_attention.cpp:48-62).
 * Shapes may hold -1 for dynamic dimensions. */
int hip_model_create_sdpa(int dtype, int rank, const int64_t* q_shape, const int64_t* kv_shape, int causal,
                          int with_scale_input, hip_model_t** model);
/* PagedAttentionExtension with its 13 inputs as Parameters named query, key, value, key_cache,
 * value_cache, past_lens, subsequence_begins, block_indices, block_indices_begins, scale,
 * sliding_window, alibi_slopes, max_context_len.  alibi_len > 0 declares alibi slopes (unsupported). */
int hip_model_create_paged_attention(int q_dtype, int kv_dtype, int cache_dtype, int num_heads_q, int num_heads_kv,
                                     int head_dim, int block_size, int alibi_len, hip_model_t** model);
/* a model holding one node of a type no plugin operator handles */
int hip_model_create_unsupported(hip_model_t** model);
void hip_model_destroy(hip_model_t* model);

/* CompiledModel (src/cuda_compiled_model.hpp:42-57) */
void hip_compiled_model_destroy(hip_compiled_model_t* compiled);
int hip_compiled_model_num_inputs(hip_compiled_model_t* compiled);
int hip_compiled_model_input_name(hip_compiled_model_t* compiled, int index, char* name, size_t name_size);
int hip_compiled_model_get_property(hip_compiled_model_t* compiled, const char* key, char* value, size_t value_size);
int hip_compiled_model_create_infer_request(hip_compiled_model_t* compiled, hip_infer_request_t** request);

/* InferRequest (src/cuda_infer_request.hpp:42-55).  Host tensors are wrapped, not copied: the
 * memory must stay valid until infer() returns.  Device tensors (device != 0) are used in place:
 * this is how the KV caches stay resident and are updated by the operator. */
void hip_infer_request_destroy(hip_infer_request_t* request);
int hip_infer_request_set_input(hip_infer_request_t* request, int index, void* data, int on_device, int dtype,
                                int rank, const int64_t* shape);
int hip_infer_request_infer(hip_infer_request_t* request);
int hip_infer_request_start_async(hip_infer_request_t* request);
int hip_infer_request_wait(hip_infer_request_t* request);
/* shape gets up to 8 extents; *bytes the byte size of the output */
int hip_infer_request_output_info(hip_infer_request_t* request, int index, int* dtype, int* rank, int64_t* shape,
                                  size_t* bytes);
int hip_infer_request_copy_output(hip_infer_request_t* request, int index, void* dst, size_t dst_bytes);
/* "node_name|node_type|microseconds" per line */
int hip_infer_request_profiling(hip_infer_request_t* request, char* text, size_t text_size);

#ifdef __cplusplus
}
#endif
#endif /* HIP_PLUGIN_H_ */
