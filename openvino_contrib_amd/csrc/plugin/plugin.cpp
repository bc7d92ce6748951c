// Plugin / CompiledModel / InferRequest implementation (see plugin.hpp).
//
// Call stacks follow the reference: Plugin::compile_model -> CompiledModel ctor builds the
// execution sequence through the operator registry
// (modules/nvidia_plugin/src/cuda_plugin.cpp:62-78, src/ops/subgraph.cpp:70-139);
// InferRequest::infer = preprocess (bind / upload inputs) -> start_pipeline (resolve pointers,
// Execute each operator, src/cuda_simple_execution_delegator.hpp:48-63) -> wait_pipeline (stream
// sync) -> postprocess (src/cuda_infer_request.cpp:107-254).  Unlike the reference there is no
// graph transformation stage that decomposes attention: the fused operators are registered.
#include "plugin.hpp"

#include <algorithm>
#include <sstream>

namespace hip_plugin {

// ------------------------------------------------------------------------- Configuration
namespace {
int64_t any_to_int(const Any& v, const std::string& key) {
    if (auto p = std::get_if<int64_t>(&v)) return *p;
    if (auto p = std::get_if<std::string>(&v)) {
        try {
            size_t pos = 0;
            long long x = std::stoll(*p, &pos);
            if (pos == p->size()) return x;
        } catch (...) {
        }
    }
    HIP_PLUGIN_THROW("property " + key + ": integer expected");
}
bool any_to_bool(const Any& v, const std::string& key) {
    if (auto p = std::get_if<bool>(&v)) return *p;
    if (auto p = std::get_if<std::string>(&v)) {
        if (*p == "YES" || *p == "true" || *p == "1") return true;
        if (*p == "NO" || *p == "false" || *p == "0") return false;
    }
    HIP_PLUGIN_THROW("property " + key + ": YES/NO expected");
}
std::string any_to_string(const Any& v, const std::string& key) {
    if (auto p = std::get_if<std::string>(&v)) return *p;
    HIP_PLUGIN_THROW("property " + key + ": string expected");
}
}  // namespace

const std::vector<std::string>& Configuration::rw_properties() {
    static const std::vector<std::string> names = {props::device_id, props::inference_precision,
                                                   props::enable_profiling, props::num_streams,
                                                   props::performance_mode};
    return names;
}

Configuration Configuration::from(const AnyMap& properties, const Configuration& base, bool throw_on_unsupported) {
    Configuration c = base;
    for (const auto& [key, value] : properties) {
        if (key == props::device_id) {
            c.device_id = (int)any_to_int(value, key);
            if (c.device_id < 0) HIP_PLUGIN_THROW("property DEVICE_ID: " + std::to_string(c.device_id));
        } else if (key == props::inference_precision) {
            const std::string p = any_to_string(value, key);
            if (p != "f32" && p != "f16" && p != "bf16" && p != "dynamic")
                HIP_PLUGIN_THROW("property INFERENCE_PRECISION_HINT: '" + p + "' (f32, f16, bf16 or dynamic expected)");
            c.inference_precision = p;
        } else if (key == props::enable_profiling) {
            c.enable_profiling = any_to_bool(value, key);
        } else if (key == props::num_streams) {
            c.num_streams = (int)any_to_int(value, key);
            if (c.num_streams < 1) HIP_PLUGIN_THROW("property NUM_STREAMS must be positive");
        } else if (key == props::performance_mode) {
            const std::string p = any_to_string(value, key);
            if (p != "LATENCY" && p != "THROUGHPUT") HIP_PLUGIN_THROW("property PERFORMANCE_HINT: '" + p + "'");
            c.performance_mode = p;
        } else if (throw_on_unsupported) {
            HIP_PLUGIN_THROW("property '" + key + "' is not supported by the HIP plugin");
        }
    }
    return c;
}

Any Configuration::get(const std::string& name) const {
    if (name == props::device_id) return std::to_string(device_id);
    if (name == props::inference_precision) return inference_precision;
    if (name == props::enable_profiling) return enable_profiling;
    if (name == props::num_streams) return (int64_t)num_streams;
    if (name == props::performance_mode) return performance_mode;
    HIP_PLUGIN_THROW("property '" + name + "' is not supported by the HIP plugin");
}

// -------------------------------------------------------------------------------- Plugin
Plugin::Plugin() {
    int n = 0;
    if (hipattn_device_count(&n) != HIPATTN_OK) n = 0;  // a plugin object may exist without a device
    device_count_ = n;
}

void Plugin::set_property(const AnyMap& properties) {
    std::lock_guard<std::mutex> lock(mutex_);
    config_ = Configuration::from(properties, config_);
}

Configuration Plugin::get_full_config(const AnyMap& properties, bool throw_on_unsupported) const {
    std::lock_guard<std::mutex> lock(mutex_);
    Configuration c = Configuration::from(properties, config_, throw_on_unsupported);
    if (device_count_ > 0 && c.device_id >= device_count_)
        HIP_PLUGIN_THROW("device id " + std::to_string(c.device_id) + " is out of range: " +
                         std::to_string(device_count_) + " HIP device(s) visible");
    return c;
}

Any Plugin::get_property(const std::string& name, const AnyMap& arguments) const {
    if (name == props::supported_properties) {
        std::string all;
        for (auto& n : Configuration::rw_properties()) all += n + " ";
        for (const char* n : {props::supported_properties, props::available_devices, props::full_device_name,
                              props::device_architecture, props::optimal_number_of_infer_requests,
                              props::range_for_async_infer_requests})
            all += std::string(n) + " ";
        all.pop_back();
        return all;
    }
    if (name == props::available_devices) {
        std::string ids;
        for (int i = 0; i < device_count_; i++) ids += (i ? " " : "") + std::to_string(i);
        return ids;
    }
    if (name == props::full_device_name || name == props::device_architecture) {
        const Configuration c = get_full_config(arguments, false);
        hipattn_device_info info;
        HIP_PLUGIN_CHECK(hipattn_get_device_info(c.device_id, &info));
        if (name == props::device_architecture) return std::string("HIP: ") + info.arch;
        return std::string(info.name[0] ? info.name : info.arch);
    }
    if (name == props::optimal_number_of_infer_requests) return (int64_t)1;
    if (name == props::range_for_async_infer_requests) return std::string("1 1 1");
    std::lock_guard<std::mutex> lock(mutex_);
    return config_.get(name);
}

bool Plugin::is_operation_supported(const std::shared_ptr<Node>& node, const Configuration& config) const {
    try {
        CreationContext ctx{config.device_id, false};
        std::vector<TensorID> in(node->inputs.size(), 0), out(node->output_types.size(), 0);
        OperationRegistry::getInstance().createOperation(ctx, node, std::move(in), std::move(out));
        return true;
    } catch (...) {
        return false;
    }
}

std::map<std::string, std::string> Plugin::query_model(const std::shared_ptr<const Model>& model,
                                                       const AnyMap& properties) const {
    const Configuration c = get_full_config(properties, false);
    std::map<std::string, std::string> supported;
    for (const auto& node : model->ordered_ops)
        if (is_operation_supported(node, c)) supported[node->friendly_name] = device_name_;
    return supported;
}

std::shared_ptr<CompiledModel> Plugin::compile_model(const std::shared_ptr<const Model>& model,
                                                     const AnyMap& properties) const {
    const Configuration c = get_full_config(properties);
    if (device_count_ == 0) HIP_PLUGIN_THROW("no HIP device is visible: cannot compile for device HIP");
    return std::make_shared<CompiledModel>(model, c, shared_from_this());
}

// -------------------------------------------------------------------------- CompiledModel
CompiledModel::CompiledModel(const std::shared_ptr<const Model>& model, const Configuration& config,
                             const std::shared_ptr<const Plugin>& plugin)
    : model_(model), config_(config), plugin_(plugin) {
    HIP_PLUGIN_CHECK(hipattn_set_device(config_.device_id));
    CreationContext ctx{config_.device_id, false};
    // tensor ids: one per (node, output port); Result and pass-through nodes get their own id too
    for (const auto& node : model_->ordered_ops) {
        std::vector<TensorID> ids;
        for (size_t i = 0; i < node->output_types.size(); i++) ids.push_back(num_tensors_++);
        output_ids_[node.get()] = ids;
    }
    for (const auto& node : model_->ordered_ops) {
        OperationBase::IndexCollection in, out = output_ids_.at(node.get());
        for (const auto& src : node->inputs) {
            auto it = output_ids_.find(src.node.get());
            HIP_PLUGIN_ASSERT(it != output_ids_.end(), "node '" + node->friendly_name + "' consumes a node outside the model");
            in.push_back(it->second.at(src.index));
        }
        // throws for unknown types and unsupported attribute combinations: compile_model fails as a whole
        auto op = OperationRegistry::getInstance().createOperation(ctx, node, std::move(in), std::move(out));
        exec_sequence_.push_back({node, op});
    }
}

std::shared_ptr<InferRequest> CompiledModel::create_infer_request() const {
    return std::make_shared<InferRequest>(shared_from_this());
}

Any CompiledModel::get_property(const std::string& name) const {
    if (name == props::model_name) return model_->name;
    if (name == props::execution_devices) return std::string("HIP.") + std::to_string(config_.device_id);
    if (name == props::optimal_number_of_infer_requests) return (int64_t)config_.num_streams;
    return config_.get(name);
}

std::vector<std::pair<std::string, std::string>> CompiledModel::get_runtime_model() const {
    std::vector<std::pair<std::string, std::string>> ops;
    for (const auto& step : exec_sequence_) ops.emplace_back(step.op->GetName(), step.op->GetTypeName());
    return ops;
}

// --------------------------------------------------------------------------- InferRequest
InferRequest::InferRequest(const std::shared_ptr<const CompiledModel>& compiled)
    : compiled_(compiled), tensor_buffers_(compiled->num_tensors_), workbuffers_(compiled->exec_sequence_.size()) {}

void InferRequest::set_tensor(const std::string& port_name, const Tensor& tensor) {
    for (const auto& p : compiled_->inputs()) {
        if (p->friendly_name != port_name) continue;
        if (tensor.type != p->output_types[0])
            HIP_PLUGIN_THROW("input '" + port_name + "': element type " + element_name(tensor.type) + ", model expects " +
                             element_name(p->output_types[0]));
        const PartialShape& ps = p->output_shapes[0];
        bool ok = ps.size() == tensor.shape.size();
        for (size_t i = 0; ok && i < ps.size(); i++) ok = ps[i] < 0 || ps[i] == tensor.shape[i];
        if (!ok) HIP_PLUGIN_THROW("input '" + port_name + "': shape does not match the model's partial shape");
        if (shape_size(tensor.shape) > 0 && tensor.data == nullptr) HIP_PLUGIN_THROW("input '" + port_name + "': null data");
        std::lock_guard<std::mutex> lock(mutex_);
        bound_inputs_[port_name] = tensor;
        return;
    }
    HIP_PLUGIN_THROW("the model has no input named '" + port_name + "'");
}

void InferRequest::set_input_tensor(size_t index, const Tensor& tensor) {
    if (index >= compiled_->inputs().size()) HIP_PLUGIN_THROW("input index " + std::to_string(index) + " is out of range");
    set_tensor(compiled_->inputs()[index]->friendly_name, tensor);
}

Tensor InferRequest::get_tensor(const std::string& port_name) const {
    auto it = outputs_.find(port_name);
    if (it != outputs_.end()) return it->second;
    auto in = bound_inputs_.find(port_name);
    if (in != bound_inputs_.end()) return in->second;
    HIP_PLUGIN_THROW("no tensor named '" + port_name + "' (outputs exist after infer())");
}

Tensor InferRequest::get_output_tensor(size_t index) const {
    if (index >= compiled_->outputs().size()) HIP_PLUGIN_THROW("output index " + std::to_string(index) + " is out of range");
    return get_tensor(compiled_->outputs()[index]->friendly_name);
}

void InferRequest::infer() {
    std::lock_guard<std::mutex> lock(mutex_);
    HIP_PLUGIN_CHECK(hipattn_set_device(compiled_->config_.device_id));
    const bool profiling = compiled_->config_.enable_profiling;
    InferenceRequestContext context{stream_, profiling};
    std::vector<TensorView> views(compiled_->num_tensors_);
    std::vector<std::unique_ptr<Event>> ev_begin, ev_end;
    std::vector<size_t> ev_step;
    profiling_.clear();

    for (size_t si = 0; si < compiled_->exec_sequence_.size(); si++) {
        const auto& step = compiled_->exec_sequence_[si];
        const Node& node = *step.node;
        const auto& out_ids = step.op->GetOutputIds();
        if (node.type_name == "Parameter") {
            // ---- preprocess: bind or upload (the reference uploads every input on every infer,
            // src/ops/parameter.cpp:24-33; device-resident tensors are passed through untouched)
            auto it = bound_inputs_.find(node.friendly_name);
            if (it == bound_inputs_.end()) HIP_PLUGIN_THROW("input '" + node.friendly_name + "' has not been set");
            const Tensor& t = it->second;
            TensorView v;
            v.type = t.type;
            v.shape = t.shape;
            if (t.remote) {
                v.device = t.data;
            } else {
                v.host = t.data;
                v.device = tensor_buffers_[out_ids[0]].reserve(std::max<size_t>(t.byte_size(), 16));
                if (t.byte_size()) stream_.upload(v.device, t.data, t.byte_size());
            }
            views[out_ids[0]] = v;
            continue;
        }
        std::vector<TensorView> in;
        std::vector<Shape> in_shapes;
        for (TensorID id : step.op->GetInputIds()) {
            in.push_back(views[id]);
            in_shapes.push_back(views[id].shape);
        }
        const std::vector<Shape> out_shapes = step.op->InferOutputShapes(in_shapes);
        std::vector<TensorView> out;
        for (size_t o = 0; o < out_ids.size(); o++) {
            TensorView v;
            v.type = node.output_types[o];
            v.shape = out_shapes.at(o);
            const int alias = step.op->InplaceInputOf(o);
            if (alias >= 0) {
                v.device = in.at(alias).device;
                v.host = in.at(alias).host;
            } else {
                v.device = tensor_buffers_[out_ids[o]].reserve(std::max<size_t>(v.byte_size(), 16));
            }
            out.push_back(v);
            views[out_ids[o]] = v;
        }
        const WorkbufferRequest req = step.op->GetWorkBufferRequest(in);
        Workbuffers wb;
        size_t total = 0;
        for (size_t b : req.mutable_sizes) total += (b + 255) / 256 * 256;
        if (total) {
            char* base = (char*)workbuffers_[si].reserve(total);
            for (size_t b : req.mutable_sizes) {
                wb.mutable_buffers.push_back(base);
                wb.mutable_sizes.push_back(b);
                base += (b + 255) / 256 * 256;
            }
        }
        if (profiling) {
            ev_begin.emplace_back(new Event());
            ev_end.emplace_back(new Event());
            ev_step.push_back(si);
            ev_begin.back()->record(stream_);
        }
        step.op->Execute(context, in, out, wb);
        if (profiling) ev_end.back()->record(stream_);
    }

    // ---- postprocess: download results into host tensors owned by the request
    for (const auto& r : compiled_->outputs()) {
        const TensorView& v = views[compiled_->output_ids_.at(r.get())[0]];
        Tensor& t = outputs_[r->friendly_name];
        t.type = v.type;
        t.shape = v.shape;
        t.remote = false;
        if (!t.storage) t.storage = std::make_shared<std::vector<uint8_t>>();
        t.storage->resize(std::max<size_t>(v.byte_size(), 1));
        t.data = t.storage->data();
        if (v.byte_size()) stream_.download(t.data, v.device, v.byte_size());
    }
    stream_.synchronize();  // wait_pipeline
    for (size_t i = 0; i < ev_step.size(); i++) {
        const auto& step = compiled_->exec_sequence_[ev_step[i]];
        profiling_.push_back({step.op->GetName(), step.op->GetTypeName(), "HIP",
                              1e3 * ev_begin[i]->elapsed_ms_until(*ev_end[i])});
    }
}

void InferRequest::start_async() {
    wait();
    pending_ = std::async(std::launch::async, [this] { infer(); });
}

void InferRequest::wait() {
    if (pending_.valid()) pending_.get();  // rethrows what infer() threw
}

std::vector<ProfilingInfo> InferRequest::get_profiling_info() const {
    if (!compiled_->config_.enable_profiling)
        HIP_PLUGIN_THROW("profiling was not enabled for this compiled model (set PERF_COUNT to YES)");
    return profiling_;
}

}  // namespace hip_plugin
