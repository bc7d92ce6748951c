// C facade of the plugin layer (include/hip_plugin.h): exceptions stop here and become codes.
#include "hip_plugin.h"

#include <cstdio>
#include <cstring>
#include <sstream>

#include "plugin.hpp"

using namespace hip_plugin;

struct hip_plugin_s {
    std::shared_ptr<Plugin> impl;
};
struct hip_model_s {
    std::shared_ptr<Model> impl;
};
struct hip_compiled_model_s {
    std::shared_ptr<CompiledModel> impl;
};
struct hip_infer_request_s {
    std::shared_ptr<InferRequest> impl;
};

namespace {
thread_local std::string g_error;

template <typename F>
int guarded(F&& f) {
    try {
        f();
        return 0;
    } catch (const NotImplemented& e) {
        g_error = e.what();
        return 3;
    } catch (const Exception& e) {
        g_error = e.what();
        return 1;
    } catch (const std::exception& e) {
        g_error = e.what();
        return 2;
    }
}

void copy_out(const std::string& s, char* dst, size_t n) {
    if (!dst || n == 0) return;
    if (s.size() + 1 > n) HIP_PLUGIN_THROW("output buffer of " + std::to_string(n) + " bytes is too small");
    std::memcpy(dst, s.c_str(), s.size() + 1);
}

std::string any_str(const Any& a) {
    if (auto p = std::get_if<std::string>(&a)) return *p;
    if (auto p = std::get_if<int64_t>(&a)) return std::to_string(*p);
    if (auto p = std::get_if<bool>(&a)) return *p ? "YES" : "NO";
    return std::to_string(std::get<double>(a));
}

ElementType to_element(int dtype) {
    switch (dtype) {
        case HIPATTN_F32: return ElementType::f32;
        case HIPATTN_F16: return ElementType::f16;
        case HIPATTN_BF16: return ElementType::bf16;
        case HIPATTN_U8: return ElementType::u8;
        case HIP_PLUGIN_I32: return ElementType::i32;
    }
    HIP_PLUGIN_THROW("unknown dtype code " + std::to_string(dtype));
}
int from_element(ElementType t) {
    switch (t) {
        case ElementType::f32: return HIPATTN_F32;
        case ElementType::f16: return HIPATTN_F16;
        case ElementType::bf16: return HIPATTN_BF16;
        case ElementType::u8: return HIPATTN_U8;
        default: return HIP_PLUGIN_I32;
    }
}

AnyMap parse_properties(const char* text) {
    AnyMap m;
    if (!text) return m;
    std::stringstream ss(text);
    std::string item;
    while (std::getline(ss, item, ';')) {
        if (item.empty()) continue;
        const size_t eq = item.find('=');
        if (eq == std::string::npos) HIP_PLUGIN_THROW("malformed property '" + item + "' (KEY=VALUE expected)");
        m[item.substr(0, eq)] = item.substr(eq + 1);
    }
    return m;
}
}  // namespace

extern "C" {

#define API __attribute__((visibility("default")))

API const char* hip_plugin_last_error(void) { return g_error.c_str(); }

API int hip_plugin_create(hip_plugin_t** plugin) {
    return guarded([&] { *plugin = new hip_plugin_s{std::make_shared<Plugin>()}; });
}
API void hip_plugin_destroy(hip_plugin_t* plugin) { delete plugin; }

API int hip_plugin_set_property(hip_plugin_t* plugin, const char* key, const char* value) {
    return guarded([&] { plugin->impl->set_property({{key, std::string(value)}}); });
}
API int hip_plugin_get_property(hip_plugin_t* plugin, const char* key, char* value, size_t value_size) {
    return guarded([&] { copy_out(any_str(plugin->impl->get_property(key)), value, value_size); });
}
API int hip_plugin_compile_model(hip_plugin_t* plugin, hip_model_t* model, const char* properties,
                                 hip_compiled_model_t** compiled) {
    return guarded([&] {
        auto cm = plugin->impl->compile_model(model->impl, parse_properties(properties));
        *compiled = new hip_compiled_model_s{cm};
    });
}
API int hip_plugin_query_model(hip_plugin_t* plugin, hip_model_t* model, char* names, size_t names_size) {
    return guarded([&] {
        std::string all;
        for (auto& kv : plugin->impl->query_model(model->impl)) all += (all.empty() ? "" : ",") + kv.first;
        copy_out(all, names, names_size);
    });
}
API int hip_plugin_registered_operations(char* names, size_t names_size) {
    return guarded([&] {
        std::string all;
        for (auto& n : OperationRegistry::getInstance().registeredTypes()) all += (all.empty() ? "" : ",") + n;
        copy_out(all, names, names_size);
    });
}

API int hip_model_create_sdpa(int dtype, int rank, const int64_t* q_shape, const int64_t* kv_shape, int causal,
                              int with_scale_input, hip_model_t** model) {
    return guarded([&] {
        const ElementType t = to_element(dtype);
        ModelBuilder b("SDPA");
        PartialShape qs(q_shape, q_shape + rank), ks(kv_shape, kv_shape + rank);
        Output q = b.parameter("query", t, qs), k = b.parameter("key", t, ks), v = b.parameter("value", t, ks);
        Output o = b.scaled_dot_product_attention("sdpa", q, k, v, causal != 0);
        if (with_scale_input) {  // a fourth/fifth input as the operator allows: this plugin rejects it
            Output m = b.parameter("attention_mask", t, {1});
            Output s = b.parameter("scale", t, {1});
            o.node->inputs.push_back(m);
            o.node->inputs.push_back(s);
        }
        b.result("out", o);
        *model = new hip_model_s{b.build()};
    });
}

API int hip_model_create_paged_attention(int q_dtype, int kv_dtype, int cache_dtype, int num_heads_q,
                                         int num_heads_kv, int head_dim, int block_size, int alibi_len,
                                         hip_model_t** model) {
    return guarded([&] {
        const ElementType qt = to_element(q_dtype), kt = to_element(kv_dtype), ct = to_element(cache_dtype);
        const int64_t row = head_dim + (ct == ElementType::u8 ? 8 : 0);
        ModelBuilder b("PagedAttention");
        std::vector<Output> in;
        in.push_back(b.parameter("query", qt, {-1, (int64_t)num_heads_q * head_dim}));
        in.push_back(b.parameter("key", kt, {-1, (int64_t)num_heads_kv * head_dim}));
        in.push_back(b.parameter("value", kt, {-1, (int64_t)num_heads_kv * head_dim}));
        in.push_back(b.parameter("key_cache", ct, {-1, num_heads_kv, block_size, row}));
        in.push_back(b.parameter("value_cache", ct, {-1, num_heads_kv, block_size, row}));
        in.push_back(b.parameter("past_lens", ElementType::i32, {-1}));
        in.push_back(b.parameter("subsequence_begins", ElementType::i32, {-1}));
        in.push_back(b.parameter("block_indices", ElementType::i32, {-1}));
        in.push_back(b.parameter("block_indices_begins", ElementType::i32, {-1}));
        in.push_back(b.parameter("scale", ElementType::f32, {-1}));
        in.push_back(b.parameter("sliding_window", ElementType::i32, {-1}));
        in.push_back(b.parameter("alibi_slopes", ElementType::f32, {alibi_len}));
        in.push_back(b.parameter("max_context_len", ElementType::i32, {-1}));
        b.result("out", b.paged_attention("paged_attention", in));
        *model = new hip_model_s{b.build()};
    });
}

API int hip_model_create_unsupported(hip_model_t** model) {
    return guarded([&] {
        ModelBuilder b("Unsupported");
        Output x = b.parameter("x", ElementType::f32, {4});
        b.result("out", b.unknown_op("SuperOperation", "super", {x}));
        *model = new hip_model_s{b.build()};
    });
}
API void hip_model_destroy(hip_model_t* model) { delete model; }

API void hip_compiled_model_destroy(hip_compiled_model_t* compiled) { delete compiled; }
API int hip_compiled_model_num_inputs(hip_compiled_model_t* compiled) { return (int)compiled->impl->inputs().size(); }
API int hip_compiled_model_input_name(hip_compiled_model_t* compiled, int index, char* name, size_t name_size) {
    return guarded([&] { copy_out(compiled->impl->inputs().at(index)->friendly_name, name, name_size); });
}
API int hip_compiled_model_get_property(hip_compiled_model_t* compiled, const char* key, char* value,
                                        size_t value_size) {
    return guarded([&] { copy_out(any_str(compiled->impl->get_property(key)), value, value_size); });
}
API int hip_compiled_model_create_infer_request(hip_compiled_model_t* compiled, hip_infer_request_t** request) {
    return guarded([&] { *request = new hip_infer_request_s{compiled->impl->create_infer_request()}; });
}

API void hip_infer_request_destroy(hip_infer_request_t* request) { delete request; }
API int hip_infer_request_set_input(hip_infer_request_t* request, int index, void* data, int on_device, int dtype,
                                    int rank, const int64_t* shape) {
    return guarded([&] {
        Tensor t;
        t.type = to_element(dtype);
        t.shape.assign(shape, shape + rank);
        t.data = data;
        t.remote = on_device != 0;
        request->impl->set_input_tensor((size_t)index, t);
    });
}
API int hip_infer_request_infer(hip_infer_request_t* request) {
    return guarded([&] { request->impl->infer(); });
}
API int hip_infer_request_start_async(hip_infer_request_t* request) {
    return guarded([&] { request->impl->start_async(); });
}
API int hip_infer_request_wait(hip_infer_request_t* request) {
    return guarded([&] { request->impl->wait(); });
}
API int hip_infer_request_output_info(hip_infer_request_t* request, int index, int* dtype, int* rank, int64_t* shape,
                                      size_t* bytes) {
    return guarded([&] {
        const Tensor t = request->impl->get_output_tensor((size_t)index);
        HIP_PLUGIN_ASSERT(t.shape.size() <= 8, "rank above 8");
        *dtype = from_element(t.type);
        *rank = (int)t.shape.size();
        for (size_t i = 0; i < t.shape.size(); i++) shape[i] = t.shape[i];
        *bytes = t.byte_size();
    });
}
API int hip_infer_request_copy_output(hip_infer_request_t* request, int index, void* dst, size_t dst_bytes) {
    return guarded([&] {
        const Tensor t = request->impl->get_output_tensor((size_t)index);
        HIP_PLUGIN_ASSERT(dst_bytes >= t.byte_size(), "destination too small");
        std::memcpy(dst, t.data, t.byte_size());
    });
}
API int hip_infer_request_profiling(hip_infer_request_t* request, char* text, size_t text_size) {
    return guarded([&] {
        std::string all;
        char line[256];
        for (auto& p : request->impl->get_profiling_info()) {
            snprintf(line, sizeof(line), "%s|%s|%.3f\n", p.node_name.c_str(), p.node_type.c_str(), p.real_time_us);
            all += line;
        }
        copy_out(all, text, text_size);
    });
}

}  // extern "C"
