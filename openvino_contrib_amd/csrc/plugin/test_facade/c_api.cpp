// C facade of the plugin layer (include/hip_plugin.h): builds single-operator ov::Model objects,
// drives Plugin / CompiledModel / InferRequest through OpenVINO's own interfaces (the object comes
// out of create_plugin_engine, as ov::Core would get it), and turns exceptions into codes.  Test
// scaffolding: under a real ov::Core none of this is needed.
#include "hip_plugin.h"

#include <cstdio>
#include <cstring>
#include <sstream>

#include "hip_memory_solver.hpp"
#include "hip_operation.hpp"
#include "hip_plugin.hpp"
#include "openvino/runtime/exec_model_info.hpp"
#include "openvino/op/add.hpp"
#include "openvino/op/assign.hpp"
#include "openvino/op/constant.hpp"
#include "openvino/op/paged_attention.hpp"
#include "openvino/op/parameter.hpp"
#include "openvino/op/read_value.hpp"
#include "openvino/op/result.hpp"
#include "openvino/op/scaled_dot_product_attention.hpp"

extern "C" void create_plugin_engine(std::shared_ptr<ov::IPlugin>& plugin);

using ov::hip_gpu::OperationRegistry;

struct hip_plugin_s {
    std::shared_ptr<ov::IPlugin> impl;
};
struct hip_model_s {
    std::shared_ptr<ov::Model> impl;
};
struct hip_compiled_model_s {
    std::shared_ptr<ov::ICompiledModel> impl;
    std::shared_ptr<ov::IPlugin> plugin;
};
struct hip_infer_request_s {
    std::shared_ptr<ov::IAsyncInferRequest> impl;
    std::shared_ptr<ov::IPlugin> plugin;
};

namespace {
thread_local std::string g_error;

template <typename F>
int guarded(F&& f) {
    try {
        f();
        return 0;
    } catch (const ov::NotImplemented& e) {
        g_error = e.what();
        return 3;
    } catch (const ov::Cancelled& e) {
        g_error = e.what();
        return 4;
    } catch (const ov::Busy& e) {
        g_error = e.what();
        return 5;
    } catch (const ov::Exception& e) {
        g_error = e.what();
        return 1;
    } catch (const std::exception& e) {
        g_error = e.what();
        return 2;
    }
}

void copy_out(const std::string& s, char* dst, size_t n) {
    if (!dst || n == 0) return;
    if (s.size() + 1 > n) OPENVINO_THROW("output buffer of ", n, " bytes is too small");
    std::memcpy(dst, s.c_str(), s.size() + 1);
}

std::string any_str(const ov::Any& a) {
    if (a.is<std::vector<std::string>>()) {
        std::string r;
        for (auto& s : a.as<std::vector<std::string>>()) r += (r.empty() ? "" : " ") + s;
        return r;
    }
    if (a.is<std::vector<ov::PropertyName>>()) {
        std::string r;
        for (auto& s : a.as<std::vector<ov::PropertyName>>()) r += (r.empty() ? "" : " ") + s;
        return r;
    }
    if (a.is<std::tuple<unsigned, unsigned, unsigned>>()) {
        auto t = a.as<std::tuple<unsigned, unsigned, unsigned>>();
        return std::to_string(std::get<0>(t)) + " " + std::to_string(std::get<1>(t)) + " " + std::to_string(std::get<2>(t));
    }
    return a.as<std::string>();
}

ov::element::Type to_element(int dtype) {
    switch (dtype) {
        case HIPATTN_F32: return ov::element::f32;
        case HIPATTN_F16: return ov::element::f16;
        case HIPATTN_BF16: return ov::element::bf16;
        case HIPATTN_U8: return ov::element::u8;
        case HIP_PLUGIN_I32: return ov::element::i32;
        case HIP_PLUGIN_BOOL: return ov::element::boolean;
        case HIP_PLUGIN_I64: return ov::element::i64;
        case HIP_PLUGIN_I8: return ov::element::i8;
    }
    OPENVINO_THROW("unknown dtype code ", dtype);
}
int from_element(const ov::element::Type& t) {
    if (t == ov::element::f32) return HIPATTN_F32;
    if (t == ov::element::f16) return HIPATTN_F16;
    if (t == ov::element::bf16) return HIPATTN_BF16;
    if (t == ov::element::u8) return HIPATTN_U8;
    if (t == ov::element::boolean) return HIP_PLUGIN_BOOL;
    if (t == ov::element::i64) return HIP_PLUGIN_I64;
    if (t == ov::element::i8) return HIP_PLUGIN_I8;
    return HIP_PLUGIN_I32;
}

ov::PartialShape to_partial_shape(int rank, const int64_t* dims) {
    std::vector<ov::Dimension> d;
    for (int i = 0; i < rank; i++) d.push_back(dims[i] < 0 ? ov::Dimension::dynamic() : ov::Dimension(dims[i]));
    return ov::PartialShape(d);
}

ov::AnyMap parse_properties(const char* text) {
    ov::AnyMap m;
    if (!text) return m;
    std::stringstream ss(text);
    std::string item;
    while (std::getline(ss, item, ';')) {
        if (item.empty()) continue;
        const size_t eq = item.find('=');
        if (eq == std::string::npos) OPENVINO_THROW("malformed property '", item, "' (KEY=VALUE expected)");
        m[item.substr(0, eq)] = item.substr(eq + 1);
    }
    return m;
}

std::shared_ptr<ov::op::v0::Parameter> parameter(const std::string& name, const ov::element::Type& type,
                                                 const ov::PartialShape& shape) {
    auto p = std::make_shared<ov::op::v0::Parameter>(type, shape);
    p->set_friendly_name(name);
    p->output(0).set_names({name});
    return p;
}
std::shared_ptr<ov::op::v0::Result> result(const std::string& name, const ov::Output<ov::Node>& value) {
    auto r = std::make_shared<ov::op::v0::Result>(value);
    r->set_friendly_name(name);
    return r;
}
}  // namespace

extern "C" {

#define API __attribute__((visibility("default")))

API const char* hip_plugin_last_error(void) { return g_error.c_str(); }

API int hip_plugin_create(hip_plugin_t** plugin) {
    return guarded([&] {
        std::shared_ptr<ov::IPlugin> p;
        create_plugin_engine(p);
        *plugin = new hip_plugin_s{p};
    });
}
API void hip_plugin_destroy(hip_plugin_t* plugin) { delete plugin; }

API int hip_plugin_device_name(hip_plugin_t* plugin, char* value, size_t value_size) {
    return guarded([&] { copy_out(plugin->impl->get_device_name(), value, value_size); });
}
API int hip_plugin_set_property(hip_plugin_t* plugin, const char* key, const char* value) {
    return guarded([&] { plugin->impl->set_property({{key, std::string(value)}}); });
}
API int hip_plugin_get_property(hip_plugin_t* plugin, const char* key, char* value, size_t value_size) {
    return guarded([&] { copy_out(any_str(plugin->impl->get_property(key, {})), value, value_size); });
}
API int hip_plugin_compile_model(hip_plugin_t* plugin, hip_model_t* model, const char* properties,
                                 hip_compiled_model_t** compiled) {
    return guarded([&] {
        auto cm = plugin->impl->compile_model(model->impl, parse_properties(properties));
        *compiled = new hip_compiled_model_s{cm, plugin->impl};
    });
}
API int hip_plugin_import_model(hip_plugin_t* plugin, const void* blob, size_t blob_bytes, const char* properties,
                                hip_compiled_model_t** compiled) {
    return guarded([&] {
        std::istringstream stream(std::string((const char*)blob, blob_bytes));
        auto cm = plugin->impl->import_model(stream, parse_properties(properties));
        *compiled = new hip_compiled_model_s{cm, plugin->impl};
    });
}
API int hip_plugin_query_model(hip_plugin_t* plugin, hip_model_t* model, char* names, size_t names_size) {
    return guarded([&] {
        std::string all;
        for (auto& kv : plugin->impl->query_model(model->impl, {})) all += (all.empty() ? "" : ",") + kv.first;
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
                              int mask_dtype, int mask_rank, const int64_t* mask_shape, int scale_mode,
                              float scale_value, hip_model_t** model) {
    return guarded([&] {
        const ov::element::Type t = to_element(dtype);
        auto q = parameter("query", t, to_partial_shape(rank, q_shape));
        auto k = parameter("key", t, to_partial_shape(rank, kv_shape));
        auto v = parameter("value", t, to_partial_shape(rank, kv_shape));
        ov::ParameterVector params{q, k, v};
        ov::OutputVector in{q, k, v};
        if (mask_dtype >= 0 || scale_mode != 0) {
            // a scale input needs a mask input in front of it: an empty one when there is no mask
            const int64_t none[1] = {0};
            auto m = mask_dtype >= 0 ? parameter("attention_mask", to_element(mask_dtype), to_partial_shape(mask_rank, mask_shape))
                                     : parameter("attention_mask", t, to_partial_shape(1, none));
            params.push_back(m);
            in.push_back(m);
        }
        if (scale_mode == 1) {
            auto s = parameter("scale", ov::element::f32, ov::PartialShape{});
            params.push_back(s);
            in.push_back(s);
        } else if (scale_mode == 2) {
            auto s = std::make_shared<ov::op::v0::Constant>(ov::element::f32, ov::Shape{}, &scale_value);
            s->set_friendly_name("scale");
            in.push_back(s);
        }
        auto sdpa = std::make_shared<ov::op::v13::ScaledDotProductAttention>(in, causal != 0);
        sdpa->set_friendly_name("sdpa");
        *model = new hip_model_s{std::make_shared<ov::Model>(ov::ResultVector{result("out", sdpa)}, params, "SDPA")};
    });
}

API int hip_model_create_paged_attention(int q_dtype, int kv_dtype, int cache_dtype, int num_heads_q,
                                         int num_heads_kv, int head_dim, int block_size, int alibi_len,
                                         int num_extra_inputs, int extra_len, int with_scores_result,
                                         hip_model_t** model) {
    return guarded([&] {
        const ov::element::Type qt = to_element(q_dtype), kt = to_element(kv_dtype), ct = to_element(cache_dtype);
        const int64_t row = head_dim + (ct == ov::element::u8 ? 8 : 0);
        const auto dyn = ov::Dimension::dynamic();
        ov::ParameterVector params;
        auto add = [&](const std::string& name, const ov::element::Type& t, const ov::PartialShape& s) {
            params.push_back(parameter(name, t, s));
        };
        add("query", qt, {dyn, (int64_t)num_heads_q * head_dim});
        add("key", kt, {dyn, (int64_t)num_heads_kv * head_dim});
        add("value", kt, {dyn, (int64_t)num_heads_kv * head_dim});
        add("key_cache", ct, {dyn, num_heads_kv, block_size, row});
        add("value_cache", ct, {dyn, num_heads_kv, block_size, row});
        add("past_lens", ov::element::i32, {dyn});
        add("subsequence_begins", ov::element::i32, {dyn});
        add("block_indices", ov::element::i32, {dyn});
        add("block_indices_begins", ov::element::i32, {dyn});
        add("scale", ov::element::f32, {dyn});
        add("sliding_window", ov::element::i32, {dyn});
        add("alibi_slopes", ov::element::f32, {alibi_len});
        add("max_context_len", ov::element::i32, {dyn});
        static const char* extra_names[] = {"score_aggregation_window", "rotated_block_indices", "rotation_deltas",
                                            "rotation_trig_lut",        "xattention_threshold",  "xattention_block_size",
                                            "xattention_stride",        "sinks",                 "one_too_many"};
        for (int i = 0; i < num_extra_inputs; i++)
            add(extra_names[std::min(i, 8)], (i == 3 || i == 4 || i == 7) ? ov::element::f32 : ov::element::i32, {extra_len});
        ov::OutputVector in;
        for (auto& p : params) in.emplace_back(p);
        auto pa = std::make_shared<ov::op::PagedAttentionExtension>(in);
        pa->set_friendly_name("paged_attention");
        ov::ResultVector results{result("out", pa->output(0))};
        if (with_scores_result) {
            pa->set_out_type(1, ov::element::f32);
            results.push_back(result("scores", pa->output(1)));
        }
        *model = new hip_model_s{std::make_shared<ov::Model>(results, params, "PagedAttention")};
    });
}

// ReadValue(init_value = x, "v0") -> Add(read, x) -> Assign("v0") and Result: the model of the
// reference's stateful test (tests/functional/shared_tests_instances/single_layer_tests/
// read_value_assign.cpp:52-64).
API int hip_model_create_accumulator(int dtype, int rank, const int64_t* shape, hip_model_t** model) {
    return guarded([&] {
        const ov::element::Type t = to_element(dtype);
        const ov::PartialShape ps = to_partial_shape(rank, shape);
        auto x = parameter("x", t, ps);
        auto variable = std::make_shared<ov::op::util::Variable>(ov::op::util::VariableInfo{ps, t, "v0"});
        auto read = std::make_shared<ov::op::v6::ReadValue>(x, variable);
        read->set_friendly_name("read_value");
        auto sum = std::make_shared<ov::op::v1::Add>(read, x);
        sum->set_friendly_name("add");
        auto assign = std::make_shared<ov::op::v6::Assign>(sum, variable);
        assign->set_friendly_name("assign");
        *model = new hip_model_s{std::make_shared<ov::Model>(ov::ResultVector{result("out", sum)}, ov::SinkVector{assign},
                                                             ov::ParameterVector{x}, "Accumulator")};
    });
}

// A model in the stand-in text form (what export_model writes): lets a test describe any graph of
// the operators the stand-in knows.
API int hip_model_create_from_text(const char* text, hip_model_t** model) {
    return guarded([&] { *model = new hip_model_s{ov::standin::Core().read_model(std::string(text), ov::Tensor())}; });
}

namespace {
class SuperOperation : public ov::Node {
public:
    OPENVINO_OP("SuperOperation", "test")
    explicit SuperOperation(const ov::Output<ov::Node>& x) : ov::Node(ov::OutputVector{x}) {
        set_output_type(0, x.get_element_type(), x.get_partial_shape());
    }
};
}  // namespace
API int hip_model_create_unsupported(hip_model_t** model) {
    return guarded([&] {
        auto x = parameter("x", ov::element::f32, ov::PartialShape{4});
        auto op = std::make_shared<SuperOperation>(x);
        op->set_friendly_name("super");
        *model = new hip_model_s{
            std::make_shared<ov::Model>(ov::ResultVector{result("out", op)}, ov::ParameterVector{x}, "Unsupported")};
    });
}
API void hip_model_destroy(hip_model_t* model) { delete model; }

API void hip_compiled_model_destroy(hip_compiled_model_t* compiled) { delete compiled; }
API int hip_compiled_model_num_inputs(hip_compiled_model_t* compiled) { return (int)compiled->impl->inputs().size(); }
API int hip_compiled_model_num_outputs(hip_compiled_model_t* compiled) { return (int)compiled->impl->outputs().size(); }
API int hip_compiled_model_input_name(hip_compiled_model_t* compiled, int index, char* name, size_t name_size) {
    return guarded([&] { copy_out(compiled->impl->inputs().at(index).get_node()->get_friendly_name(), name, name_size); });
}
API int hip_compiled_model_get_property(hip_compiled_model_t* compiled, const char* key, char* value,
                                        size_t value_size) {
    return guarded([&] { copy_out(any_str(compiled->impl->get_property(key)), value, value_size); });
}
API int hip_compiled_model_export(hip_compiled_model_t* compiled, void* blob, size_t blob_capacity, size_t* blob_bytes) {
    return guarded([&] {
        std::ostringstream stream;
        compiled->impl->export_model(stream);
        const std::string s = stream.str();
        *blob_bytes = s.size();
        if (blob) {
            if (s.size() > blob_capacity) OPENVINO_THROW("export buffer of ", blob_capacity, " bytes is too small");
            std::memcpy(blob, s.data(), s.size());
        }
    });
}
API int hip_compiled_model_create_infer_request(hip_compiled_model_t* compiled, hip_infer_request_t** request) {
    return guarded([&] { *request = new hip_infer_request_s{compiled->impl->create_infer_request(), compiled->plugin}; });
}

API void hip_infer_request_destroy(hip_infer_request_t* request) { delete request; }

namespace {
ov::SoPtr<ov::ITensor> wrap(hip_infer_request_t* request, void* data, int on_device, int dtype, int rank,
                            const int64_t* shape) {
    ov::Shape s(shape, shape + rank);
    if (!on_device) return ov::SoPtr<ov::ITensor>{ov::make_tensor(to_element(dtype), s, data), nullptr};
    auto context = request->plugin->get_default_context({});
    return context->create_tensor(to_element(dtype), s, {{"DEV_PTR", (int64_t)(uintptr_t)data}});
}
}  // namespace

API int hip_infer_request_set_input(hip_infer_request_t* request, int index, void* data, int on_device, int dtype,
                                    int rank, const int64_t* shape) {
    return guarded([&] {
        const auto& ports = request->impl->get_inputs();
        if (index < 0 || (size_t)index >= ports.size()) OPENVINO_THROW("input index ", index, " is out of range");
        request->impl->set_tensor(ports[index], wrap(request, data, on_device, dtype, rank, shape));
    });
}
API int hip_infer_request_set_input_batch(hip_infer_request_t* request, int index, void* const* data, int count, int dtype,
                                          int rank, const int64_t* shape) {
    return guarded([&] {
        const auto& ports = request->impl->get_inputs();
        if (index < 0 || (size_t)index >= ports.size()) OPENVINO_THROW("input index ", index, " is out of range");
        std::vector<ov::SoPtr<ov::ITensor>> tensors;
        for (int i = 0; i < count; i++) tensors.push_back(wrap(request, data[i], 0, dtype, rank, shape));
        request->impl->set_tensors(ports[index], tensors);
    });
}
API int hip_infer_request_set_output(hip_infer_request_t* request, int index, void* data, int on_device, int dtype,
                                     int rank, const int64_t* shape) {
    return guarded([&] {
        const auto& ports = request->impl->get_outputs();
        if (index < 0 || (size_t)index >= ports.size()) OPENVINO_THROW("output index ", index, " is out of range");
        request->impl->set_tensor(ports[index], wrap(request, data, on_device, dtype, rank, shape));
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
API int hip_infer_request_cancel(hip_infer_request_t* request) {
    return guarded([&] { request->impl->cancel(); });
}
API int hip_infer_request_output_info(hip_infer_request_t* request, int index, int* dtype, int* rank, int64_t* shape,
                                      size_t* bytes) {
    return guarded([&] {
        auto t = request->impl->get_tensor(request->impl->get_outputs().at(index));
        const ov::Shape& s = t->get_shape();
        if (s.size() > 8) OPENVINO_THROW("rank above 8");
        *dtype = from_element(t->get_element_type());
        *rank = (int)s.size();
        for (size_t i = 0; i < s.size(); i++) shape[i] = (int64_t)s[i];
        *bytes = t->get_byte_size();
    });
}
API int hip_infer_request_copy_output(hip_infer_request_t* request, int index, void* dst, size_t dst_bytes) {
    return guarded([&] {
        auto t = request->impl->get_tensor(request->impl->get_outputs().at(index));
        if (dst_bytes < t->get_byte_size()) OPENVINO_THROW("destination too small");
        if (t->get_byte_size()) std::memcpy(dst, t->data(), t->get_byte_size());
    });
}
API int hip_compiled_model_runtime_info(hip_compiled_model_t* compiled, char* text, size_t text_size) {
    return guarded([&] {
        std::string all;
        const auto model = compiled->impl->get_runtime_model();
        for (const auto& op : model->get_ordered_ops()) {
            const auto& info = op->get_rt_info();
            const auto field = [&](const char* key) { return info.count(key) ? info.at(key).as<std::string>() : std::string("?"); };
            all += op->get_friendly_name() + "|" + field(ov::exec_model_info::LAYER_TYPE) + "|" + field(ov::exec_model_info::EXECUTION_ORDER) +
                   "|" + field(ov::exec_model_info::PERF_COUNTER) + "|" + field(ov::exec_model_info::RUNTIME_PRECISION) + "|" +
                   field(ov::exec_model_info::IMPL_TYPE) + "\n";
        }
        copy_out(all, text, text_size);
    });
}
API int hip_infer_request_intermediate_memory(hip_infer_request_t* request, size_t* blob_bytes, size_t* apart_bytes) {
    return guarded([&] {
        auto async = std::dynamic_pointer_cast<ov::hip_gpu::AsyncInferRequest>(request->impl);
        if (!async) OPENVINO_THROW("not a request of this plugin");
        const auto m = async->sync_request()->intermediate_memory();
        *blob_bytes = m.first;
        *apart_bytes = m.second;
    });
}
API size_t hip_memory_solver_pack(int count, const size_t* bytes, const int* start, const int* end, size_t* offsets) {
    std::vector<ov::hip_gpu::MemoryBox> boxes;
    for (int i = 0; i < count; i++) boxes.push_back({bytes[i], start[i], end[i]});
    std::vector<size_t> at;
    const size_t total = ov::hip_gpu::solve_memory(boxes, at);
    for (int i = 0; i < count; i++) offsets[i] = at[i];
    return total;
}
API int hip_infer_request_profiling(hip_infer_request_t* request, char* text, size_t text_size) {
    return guarded([&] {
        std::string all;
        char line[256];
        for (auto& p : request->impl->get_profiling_info()) {
            snprintf(line, sizeof(line), "%s|%s|%.3f\n", p.node_name.c_str(), p.node_type.c_str(), (double)p.real_time.count());
            all += line;
        }
        copy_out(all, text, text_size);
    });
}

API int hip_infer_request_num_states(hip_infer_request_t* request) { return (int)request->impl->query_state().size(); }
API int hip_infer_request_state_name(hip_infer_request_t* request, int index, char* name, size_t name_size) {
    return guarded([&] { copy_out(request->impl->query_state().at(index)->get_name(), name, name_size); });
}
API int hip_infer_request_state_reset(hip_infer_request_t* request, int index) {
    return guarded([&] { request->impl->query_state().at(index)->reset(); });
}
API int hip_infer_request_state_info(hip_infer_request_t* request, int index, int* dtype, int* rank, int64_t* shape,
                                     size_t* bytes) {
    return guarded([&] {
        auto t = request->impl->query_state().at(index)->get_state();
        const ov::Shape& s = t->get_shape();
        *dtype = from_element(t->get_element_type());
        *rank = (int)s.size();
        for (size_t i = 0; i < s.size(); i++) shape[i] = (int64_t)s[i];
        *bytes = t->get_byte_size();
    });
}
API int hip_infer_request_state_get(hip_infer_request_t* request, int index, void* dst, size_t dst_bytes) {
    return guarded([&] {
        auto t = request->impl->query_state().at(index)->get_state();
        if (dst_bytes < t->get_byte_size()) OPENVINO_THROW("destination too small");
        if (t->get_byte_size()) std::memcpy(dst, t->data(), t->get_byte_size());
    });
}
API int hip_infer_request_state_set(hip_infer_request_t* request, int index, void* data, int dtype, int rank,
                                    const int64_t* shape) {
    return guarded([&] {
        ov::Shape s(shape, shape + rank);
        request->impl->query_state().at(index)->set_state(ov::SoPtr<ov::ITensor>{ov::make_tensor(to_element(dtype), s, data), nullptr});
    });
}

}  // extern "C"
