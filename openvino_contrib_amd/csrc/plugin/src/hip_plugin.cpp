// Plugin / CompiledModel / InferRequest / AsyncInferRequest implementation (see hip_plugin.hpp).
//
// Call stacks follow the reference: Plugin::compile_model -> CompiledModel ctor builds the
// execution sequence through the operator registry
// (modules/nvidia_plugin/src/cuda_plugin.cpp:62-78, src/ops/subgraph.cpp:70-139);
// InferRequest::infer = infer_preprocess (bind / upload inputs) -> start_pipeline (resolve pointers,
// Execute each operator, src/cuda_simple_execution_delegator.hpp:48-63) -> wait_pipeline (stream
// sync) -> infer_postprocess (src/cuda_infer_request.cpp:107-254), the middle two on a worker
// thread of the device's pool, which owns the stream.
#include "hip_plugin.hpp"
#include "hip_memory_solver.hpp"

#include <algorithm>
#include <sstream>

#include "openvino/op/assign.hpp"
#include "openvino/op/constant.hpp"
#include "openvino/op/parameter.hpp"
#include "openvino/op/read_value.hpp"
#include "openvino/op/result.hpp"
#include "openvino/pass/serialize.hpp"
#include "openvino/runtime/exec_model_info.hpp"
#include "openvino/runtime/icore.hpp"
#include "openvino/runtime/internal_properties.hpp"

namespace ov {
namespace hip_gpu {

// ------------------------------------------------------------------------- Configuration
// the counterpart of NVIDIA_USE_CUDA_GRAPH (include/nvidia/properties.hpp:30)
static const char* const kUseGraphProperty = "HIP_USE_GRAPH";
static const char* const kGraphMinOperatorsProperty = "HIP_GRAPH_MIN_OPERATORS";

const std::vector<std::string>& Configuration::rw_properties() {
    static const std::vector<std::string> names = {ov::device::id.name(), ov::hint::inference_precision.name(),
                                                   ov::enable_profiling.name(), ov::num_streams.name(),
                                                   ov::hint::performance_mode.name(), kUseGraphProperty,
                                                   kGraphMinOperatorsProperty};
    return names;
}

Configuration Configuration::from(const ov::AnyMap& properties, const Configuration& base, bool throw_on_unsupported) {
    Configuration c = base;
    for (const auto& [key, value] : properties) {
        if (key == ov::device::id.name()) {
            c.device_id = value.as<int>();
            if (c.device_id < 0) HIP_PLUGIN_THROW("property DEVICE_ID: " + std::to_string(c.device_id));
        } else if (key == ov::hint::inference_precision.name()) {
            ov::element::Type t;
            if (value.is<ov::element::Type>()) {
                t = value.as<ov::element::Type>();
            } else {
                const std::string p = value.as<std::string>();
                if (p == "f32")
                    t = ov::element::f32;
                else if (p == "f16")
                    t = ov::element::f16;
                else if (p == "bf16")
                    t = ov::element::bf16;
                else if (p == "dynamic")
                    t = ov::element::dynamic;
                else
                    HIP_PLUGIN_THROW("property INFERENCE_PRECISION_HINT: '" + p + "' (f32, f16, bf16 or dynamic expected)");
            }
            if (t != ov::element::f32 && t != ov::element::f16 && t != ov::element::bf16 && t != ov::element::dynamic)
                HIP_PLUGIN_THROW("property INFERENCE_PRECISION_HINT: " + t.get_type_name() +
                                 " (f32, f16, bf16 or dynamic expected)");
            c.inference_precision = t;
        } else if (key == ov::enable_profiling.name()) {
            c.enable_profiling = value.as<bool>();
        } else if (key == kUseGraphProperty) {
            c.use_graph = value.as<bool>();
        } else if (key == kGraphMinOperatorsProperty) {
            c.graph_min_operators = value.as<int>();
            if (c.graph_min_operators < 1) HIP_PLUGIN_THROW(std::string("property ") + kGraphMinOperatorsProperty + ": at least 1 expected");
        } else if (key == ov::num_streams.name()) {
            c.num_streams = value.as<int>();
            if (c.num_streams < 1) HIP_PLUGIN_THROW("property NUM_STREAMS must be positive");
        } else if (key == ov::hint::performance_mode.name()) {
            const std::string p = value.as<std::string>();
            if (p != "LATENCY" && p != "THROUGHPUT") HIP_PLUGIN_THROW("property PERFORMANCE_HINT: '" + p + "'");
            c.performance_mode = p;
        } else if (throw_on_unsupported) {
            HIP_PLUGIN_THROW("property '" + key + "' is not supported by the HIP plugin");
        }
    }
    return c;
}

ov::Any Configuration::get(const std::string& name) const {
    if (name == ov::device::id.name()) return std::to_string(device_id);
    if (name == ov::hint::inference_precision.name()) return inference_precision.get_type_name();
    if (name == ov::enable_profiling.name()) return enable_profiling;
    if (name == kUseGraphProperty) return use_graph;
    if (name == kGraphMinOperatorsProperty) return (int64_t)graph_min_operators;
    if (name == ov::num_streams.name()) return (int64_t)num_streams;
    if (name == ov::hint::performance_mode.name()) return performance_mode;
    HIP_PLUGIN_THROW("property '" + name + "' is not supported by the HIP plugin");
}

// ------------------------------------------------------------------- remote tensors / context
RemoteTensor::RemoteTensor(const ov::element::Type& type, const ov::Shape& shape, void* wrapped,
                           const std::string& device_name)
    : type_(type), shape_(shape), wrapped_(wrapped), device_name_(device_name) {
    if (!wrapped_) owned_.reserve(std::max<size_t>(get_byte_size(), 16));
    properties_["DEV_PTR"] = (int64_t)(uintptr_t)device_ptr();
}

void RemoteTensor::set_shape(ov::Shape shape) {
    const size_t bytes = ov::shape_size(shape) * type_.size();
    if (wrapped_) {
        HIP_PLUGIN_ASSERT(bytes <= get_byte_size(), "a tensor over caller-owned device memory cannot grow");
    } else if (bytes > owned_.capacity()) {
        HIP_PLUGIN_THROW("a device tensor cannot grow beyond its allocation (" + std::to_string(owned_.capacity()) +
                         " bytes); create a new one");
    }
    shape_ = std::move(shape);
}

RemoteContext::RemoteContext(const std::string& device_name, int device_id)
    : device_name_(device_name + "." + std::to_string(device_id)), device_id_(device_id) {
    properties_[ov::device::id.name()] = std::to_string(device_id);
}

ov::SoPtr<ov::IRemoteTensor> RemoteContext::create_tensor(const ov::element::Type& type, const ov::Shape& shape,
                                                          const ov::AnyMap& params) {
    HIP_PLUGIN_CHECK(hipattn_set_device(device_id_));
    void* wrapped = nullptr;
    auto it = params.find("DEV_PTR");
    if (it != params.end()) wrapped = (void*)(uintptr_t)it->second.as<int64_t>();
    return ov::SoPtr<ov::IRemoteTensor>{std::make_shared<RemoteTensor>(type, shape, wrapped, device_name_), nullptr};
}

// --------------------------------------------------------------------------- VariableState
VariableState::VariableState(const ov::op::util::VariableInfo& info)
    : ov::IVariableState(info.variable_id), data_shape_(info.data_shape), type_(info.data_type) {
    // dynamic extents start at 0 (an empty KV state of the right rank); reset() returns to this shape
    for (size_t i = 0; i < data_shape_.size(); i++)
        initial_shape_.push_back(data_shape_[i].is_static() ? (size_t)data_shape_[i].get_length() : 0);
    current_shape_ = initial_shape_;
    if (const size_t bytes = logical_bytes()) {
        Stream stream;
        stream.fill(buffer_.reserve(bytes), 0, bytes);
        stream.synchronize();
    }
    m_state = ov::SoPtr<ov::ITensor>{ov::make_tensor(type_, current_shape_), nullptr};
}

void VariableState::set_state(const ov::SoPtr<ov::ITensor>& state) {
    std::lock_guard<std::mutex> lock(mutex_);
    OPENVINO_ASSERT(data_shape_.compatible(ov::PartialShape(state->get_shape())), "Wrong tensor shape: ",
                    state->get_shape(), " is not compatible with expected: ", data_shape_, " in variable: ", get_name());
    OPENVINO_ASSERT(type_.compatible(state->get_element_type()), "Wrong tensor type: ", state->get_element_type(),
                    " expected: ", type_, " in variable: ", get_name());
    current_shape_ = state->get_shape();
    if (const size_t bytes = logical_bytes()) {
        Stream stream;
        stream.upload(buffer_.reserve(bytes), state->data(), bytes);
        stream.synchronize();
    }
    is_reset_ = false;
}

ov::SoPtr<ov::ITensor> VariableState::get_state() const {
    std::lock_guard<std::mutex> lock(mutex_);
    auto tensor = ov::make_tensor(type_, current_shape_);
    if (const size_t bytes = logical_bytes()) {
        Stream stream;
        stream.download(tensor->data(), buffer_.get(), bytes);
        stream.synchronize();
    }
    return ov::SoPtr<ov::ITensor>{tensor, nullptr};
}

void VariableState::reset() {
    std::lock_guard<std::mutex> lock(mutex_);
    current_shape_ = initial_shape_;
    if (buffer_.capacity()) {
        Stream stream;
        stream.fill(buffer_.get(), 0, buffer_.capacity());
        stream.synchronize();
    }
    is_reset_ = true;
}

bool VariableState::is_reset_state() const {
    std::lock_guard<std::mutex> lock(mutex_);
    return is_reset_;
}
ov::Shape VariableState::shape() const {
    std::lock_guard<std::mutex> lock(mutex_);
    return current_shape_;
}
size_t VariableState::byte_size() const {
    std::lock_guard<std::mutex> lock(mutex_);
    return logical_bytes();
}

void VariableState::update_device_state(const Stream& stream, const void* src, const ov::Shape& new_shape) {
    std::lock_guard<std::mutex> lock(mutex_);
    const size_t bytes = type_.size() * ov::shape_size(new_shape);
    if (bytes > buffer_.capacity()) {
        stream.synchronize();  // a reader of the old buffer may still be in flight on this stream
        buffer_.reserve(bytes);
    }
    current_shape_ = new_shape;
    if (bytes) stream.transfer(buffer_.get(), src, bytes);
    is_reset_ = false;
}

void VariableState::read_device_state(const Stream& stream, void* dst, size_t dst_bytes) const {
    std::lock_guard<std::mutex> lock(mutex_);
    const size_t bytes = std::min(dst_bytes, logical_bytes());
    if (bytes && buffer_.get()) stream.transfer(dst, buffer_.get(), bytes);
}

// ------------------------------------------------------------------------------ ThreadPool
namespace {
thread_local ThreadContext* t_thread_context = nullptr;
}

ThreadPool::ThreadPool(int device_id, unsigned num_threads) : device_id_(device_id) {
    for (unsigned i = 0; i < std::max(1u, num_threads); i++) threads_.emplace_back([this] { worker(); });
}

ThreadPool::~ThreadPool() {
    {
        std::lock_guard<std::mutex> lock(mutex_);
        stopping_ = true;
    }
    wake_.notify_all();
    for (auto& t : threads_) t.join();
}

void ThreadPool::worker() {
    // the thread's device and stream live as long as the thread; a pool on a machine without a device
    // only ever fails the tasks that ask for the stream
    std::unique_ptr<ThreadContext> context;
    if (hipattn_set_device(device_id_) == HIPATTN_OK) {
        try {
            context = std::make_unique<ThreadContext>();
        } catch (const std::exception&) {
        }
    }
    t_thread_context = context.get();
    for (;;) {
        ov::threading::Task task;
        {
            std::unique_lock<std::mutex> lock(mutex_);
            wake_.wait(lock, [this] { return stopping_ || !queue_.empty(); });
            if (queue_.empty()) return;  // stopping and drained
            task = std::move(queue_.front());
            queue_.pop_front();
        }
        task();
    }
}

void ThreadPool::run(ov::threading::Task task) {
    {
        std::lock_guard<std::mutex> lock(mutex_);
        queue_.push_back(std::move(task));
    }
    wake_.notify_one();
}

const ThreadContext& ThreadPool::get_thread_context() {
    if (!t_thread_context) HIP_PLUGIN_THROW("this thread has no HIP stream (not a worker of the device's pool, or no device)");
    return *t_thread_context;
}

// -------------------------------------------------------------------------------- Plugin
Plugin::Plugin() {
    set_device_name("HIP");
    int n = 0;
    if (hipattn_device_count(&n) != HIPATTN_OK) n = 0;  // a plugin object may exist without a device
    device_count_ = n;
}

Plugin::~Plugin() = default;

void Plugin::set_property(const ov::AnyMap& properties) {
    std::lock_guard<std::mutex> lock(mutex_);
    config_ = Configuration::from(properties, config_);
}

Configuration Plugin::get_full_config(const ov::AnyMap& properties, bool throw_on_unsupported) const {
    std::lock_guard<std::mutex> lock(mutex_);
    Configuration c = Configuration::from(properties, config_, throw_on_unsupported);
    if (device_count_ > 0 && c.device_id >= device_count_)
        HIP_PLUGIN_THROW("device id " + std::to_string(c.device_id) + " is out of range: " +
                         std::to_string(device_count_) + " HIP device(s) visible");
    return c;
}

std::shared_ptr<ov::threading::ITaskExecutor> Plugin::get_stream_executor(const Configuration& config) const {
    std::lock_guard<std::mutex> lock(mutex_);
    auto& pool = device_thread_pool_[{config.device_id, config.num_streams}];
    if (!pool) pool = std::make_shared<ThreadPool>(config.device_id, (unsigned)config.num_streams);
    return pool;
}

ov::Any Plugin::get_property(const std::string& name, const ov::AnyMap& arguments) const {
    if (name == ov::supported_properties.name()) {
        std::vector<ov::PropertyName> all;
        for (auto& n : Configuration::rw_properties()) all.emplace_back(n, ov::PropertyMutability::RW);
        for (const char* n : {ov::supported_properties.name(), ov::available_devices.name(), ov::device::full_name.name(),
                              ov::device::architecture.name(), ov::device::capabilities.name(),
                              ov::optimal_number_of_infer_requests.name(), ov::range_for_async_infer_requests.name()})
            all.emplace_back(n, ov::PropertyMutability::RO);
        return all;
    }
    if (name == ov::internal::supported_properties.name())
        return std::vector<ov::PropertyName>{{ov::internal::caching_properties.name(), ov::PropertyMutability::RO}};
    if (name == ov::internal::caching_properties.name())
        return std::vector<ov::PropertyName>{{ov::device::architecture.name(), ov::PropertyMutability::RO},
                                             {ov::hint::inference_precision.name(), ov::PropertyMutability::RW}};
    if (name == ov::available_devices.name()) {
        std::vector<std::string> ids;
        for (int i = 0; i < device_count_; i++) ids.push_back(std::to_string(i));
        return ids;
    }
    if (name == ov::device::capabilities.name())
        return std::vector<std::string>{ov::device::capability::FP32, ov::device::capability::FP16,
                                        ov::device::capability::BF16, ov::device::capability::EXPORT_IMPORT};
    if (name == ov::device::full_name.name() || name == ov::device::architecture.name()) {
        const Configuration c = get_full_config(arguments, false);
        hipattn_device_info info;
        HIP_PLUGIN_CHECK(hipattn_get_device_info(c.device_id, &info));
        if (name == ov::device::architecture.name()) return std::string("HIP: ") + info.arch;
        return std::string(info.name[0] ? info.name : info.arch);
    }
    if (name == ov::optimal_number_of_infer_requests.name()) return (int64_t)1;
    if (name == ov::range_for_async_infer_requests.name()) return std::make_tuple(1u, 1u, 1u);
    std::lock_guard<std::mutex> lock(mutex_);
    return config_.get(name);
}

bool Plugin::is_operation_supported(const std::shared_ptr<ov::Node>& node, const Configuration& config) const {
    try {
        CreationContext ctx{config.device_id, false};
        std::vector<TensorID> in(node->get_input_size(), 0), out(node->get_output_size(), 0);
        OperationRegistry::getInstance().createOperation(ctx, node, std::move(in), std::move(out));
        return true;
    } catch (...) {
        return false;
    }
}

ov::SupportedOpsMap Plugin::query_model(const std::shared_ptr<const ov::Model>& model,
                                        const ov::AnyMap& properties) const {
    const Configuration c = get_full_config(properties, false);
    // no transformation stage: the attention operators are executed as they stand
    auto supported = ov::get_supported_nodes(
        model, [](std::shared_ptr<ov::Model>&) {},
        [&](const std::shared_ptr<ov::Node>& op) { return is_operation_supported(op, c); });
    ov::SupportedOpsMap res;
    for (auto&& name : supported) res.emplace(name, get_device_name() + "." + std::to_string(c.device_id));
    return res;
}

std::shared_ptr<ov::ICompiledModel> Plugin::compile_model(const std::shared_ptr<const ov::Model>& model,
                                                          const ov::AnyMap& properties) const {
    return compile_model(model, properties, {});
}

std::shared_ptr<ov::ICompiledModel> Plugin::compile_model(const std::shared_ptr<const ov::Model>& model,
                                                          const ov::AnyMap& properties,
                                                          const ov::SoPtr<ov::IRemoteContext>&) const {
    const Configuration c = get_full_config(properties);
    if (device_count_ == 0) HIP_PLUGIN_THROW("no HIP device is visible: cannot compile for device HIP");
    return std::make_shared<CompiledModel>(model, c, get_stream_executor(c), shared_from_this(), false);
}

// The stream CompiledModel::export_model writes: [u64 size][model text][u64 size][weights], the
// reference's cache format (src/cuda_compiled_model.cpp:373-395, src/cuda_plugin.cpp:99-138).
std::shared_ptr<ov::ICompiledModel> Plugin::import_model(std::istream& model_stream, const ov::AnyMap& properties) const {
    return import_model(model_stream, {}, properties);
}

std::shared_ptr<ov::ICompiledModel> Plugin::import_model(std::istream& model_stream,
                                                         const ov::SoPtr<ov::IRemoteContext>&,
                                                         const ov::AnyMap& properties) const {
    auto read_size = [&]() {
        std::uint64_t n = 0;
        model_stream.read(reinterpret_cast<char*>(&n), sizeof(n));
        if (!model_stream || n > (std::uint64_t(1) << 40)) HIP_PLUGIN_THROW("import_model: truncated or foreign stream");
        return n;
    };
    std::string xml(read_size(), '\0');
    model_stream.read(xml.data(), (std::streamsize)xml.size());
    ov::Tensor weights;
    if (const std::uint64_t n = read_size()) {
        weights = ov::Tensor(ov::element::u8, ov::Shape{(size_t)n});
        model_stream.read(weights.data<char>(), (std::streamsize)n);
    }
    if (!model_stream) HIP_PLUGIN_THROW("import_model: truncated stream");
    auto model = get_core()->read_model(xml, weights);

    auto props = properties;
    bool loaded_from_cache = false;
    auto it = props.find(ov::loaded_from_cache.name());
    if (it != props.end()) {
        loaded_from_cache = it->second.as<bool>();
        props.erase(it);
    }
    const Configuration c = get_full_config(props);
    if (device_count_ == 0) HIP_PLUGIN_THROW("no HIP device is visible: cannot compile for device HIP");
    return std::make_shared<CompiledModel>(model, c, get_stream_executor(c), shared_from_this(), loaded_from_cache);
}

namespace {
// a tensor of bytes as a stream
class TensorBuf : public std::streambuf {
public:
    explicit TensorBuf(const ov::Tensor& t) {
        char* p = t.data<char>();
        setg(p, p, p + t.get_byte_size());
    }
};
}  // namespace

std::shared_ptr<ov::ICompiledModel> Plugin::import_model(const ov::Tensor& model_stream, const ov::AnyMap& properties) const {
    return import_model(model_stream, {}, properties);
}

std::shared_ptr<ov::ICompiledModel> Plugin::import_model(const ov::Tensor& model_stream,
                                                         const ov::SoPtr<ov::IRemoteContext>& context,
                                                         const ov::AnyMap& properties) const {
    TensorBuf buf(model_stream);
    std::istream stream(&buf);
    return import_model(stream, context, properties);
}

// Unlike the reference (OPENVINO_NOT_IMPLEMENTED, src/cuda_plugin.cpp:161-169) the plugin has a
// remote context: it is how a KV cache stays on the device between infer calls.
ov::SoPtr<ov::IRemoteContext> Plugin::create_context(const ov::AnyMap& remote_properties) const {
    const Configuration c = get_full_config(remote_properties, false);
    return ov::SoPtr<ov::IRemoteContext>{std::make_shared<RemoteContext>(get_device_name(), c.device_id), nullptr};
}

ov::SoPtr<ov::IRemoteContext> Plugin::get_default_context(const ov::AnyMap& remote_properties) const {
    return create_context(remote_properties);
}

// -------------------------------------------------------------------------- CompiledModel
CompiledModel::CompiledModel(const std::shared_ptr<const ov::Model>& model, const Configuration& config,
                             const std::shared_ptr<ov::threading::ITaskExecutor>& wait_executor,
                             const std::shared_ptr<const ov::IPlugin>& plugin, bool loaded_from_cache)
    : ov::ICompiledModel(model, plugin),
      model_(model->clone()),
      exec_model_(model),
      config_(config),
      wait_executor_(wait_executor),
      loaded_from_cache_(loaded_from_cache) {
    HIP_PLUGIN_CHECK(hipattn_set_device(config_.device_id));
    CreationContext ctx{config_.device_id, false};
    const auto ordered = exec_model_->get_ordered_ops();
    // tensor ids: one per (node, output port); Result and pass-through nodes get their own id too
    for (const auto& node : ordered) {
        std::vector<TensorID> ids;
        for (size_t i = 0; i < node->get_output_size(); i++) ids.push_back(num_tensors_++);
        output_ids_[node.get()] = ids;
    }
    for (const auto& node : ordered) {
        OperationBase::IndexCollection in, out = output_ids_.at(node.get());
        for (size_t i = 0; i < node->get_input_size(); i++) {
            const auto src = node->input_value(i);
            auto it = output_ids_.find(src.get_node());
            HIP_PLUGIN_ASSERT(it != output_ids_.end(),
                              "node '" + node->get_friendly_name() + "' consumes a node outside the model");
            in.push_back(it->second.at(src.get_index()));
        }
        // throws for unknown types and unsupported attribute combinations: compile_model fails as a whole
        auto op = OperationRegistry::getInstance().createOperation(ctx, node, std::move(in), std::move(out));
        exec_sequence_.push_back({node, op});
    }
    // outputs nothing consumes (neither an operator nor a Result) need not be produced
    std::set<std::pair<const ov::Node*, size_t>> consumed;
    for (const auto& node : ordered)
        for (size_t i = 0; i < node->get_input_size(); i++) {
            const auto src = node->input_value(i);
            consumed.insert({src.get_node(), src.get_index()});
        }
    for (const auto& step : exec_sequence_)
        for (size_t o = 0; o < step.node->get_output_size(); o++)
            if (!consumed.count({step.node.get(), o})) step.op->MarkOutputUnused(o);
    // tensors every consumer reads on the host only (launch parameters, shape patterns) stay off the device
    std::map<TensorID, bool> host_only;
    for (const auto& step : exec_sequence_) {
        const auto& in_ids = step.op->GetInputIds();
        for (size_t i = 0; i < in_ids.size(); i++) {
            const bool here = step.op->InputIsHostOnly(i);
            auto it = host_only.find(in_ids[i]);
            if (it == host_only.end())
                host_only[in_ids[i]] = here;
            else
                it->second = it->second && here;
        }
    }
    for (const auto& kv : host_only)
        if (kv.second) host_only_tensors_.insert(kv.first);
    // tensors whose host-side value no consumer's launches depend on (OperationBase::InputValueShapesLaunch)
    std::map<TensorID, bool> advisory;
    for (const auto& step : exec_sequence_) {
        const auto& in_ids = step.op->GetInputIds();
        for (size_t i = 0; i < in_ids.size(); i++) {
            const bool here = !step.op->InputValueShapesLaunch(i);
            auto it = advisory.find(in_ids[i]);
            if (it == advisory.end())
                advisory[in_ids[i]] = here;
            else
                it->second = it->second && here;
        }
    }
    for (const auto& kv : advisory)
        if (kv.second) advisory_value_tensors_.insert(kv.first);
}

std::shared_ptr<ov::ISyncInferRequest> CompiledModel::create_sync_infer_request() const {
    return std::make_shared<InferRequest>(std::static_pointer_cast<const CompiledModel>(shared_from_this()), wait_executor_);
}

std::shared_ptr<ov::IAsyncInferRequest> CompiledModel::create_infer_request() const {
    auto sync = std::static_pointer_cast<InferRequest>(create_sync_infer_request());
    return std::make_shared<AsyncInferRequest>(sync, get_task_executor(), wait_executor_, get_callback_executor());
}

void CompiledModel::set_property(const ov::AnyMap&) { OPENVINO_NOT_IMPLEMENTED; }

ov::Any CompiledModel::get_property(const std::string& name) const {
    if (name == ov::model_name.name()) return model_->get_friendly_name();
    if (name == ov::execution_devices.name())
        return std::vector<std::string>{get_plugin()->get_device_name() + "." + std::to_string(config_.device_id)};
    if (name == ov::optimal_number_of_infer_requests.name()) return (int64_t)config_.num_streams;
    if (name == ov::loaded_from_cache.name()) return loaded_from_cache_;
    // graphs recorded / launched by this model's requests so far (the reference reports the count it
    // builds at compile time as NVIDIA_NUMBER_OF_CUDA_GRAPHS, include/nvidia/properties.hpp:35)
    if (name == "HIP_NUMBER_OF_GRAPHS") return (int64_t)graphs_captured_.load();
    if (name == "HIP_GRAPH_LAUNCHES") return (int64_t)graph_launches_.load();
    if (name == ov::supported_properties.name()) {
        std::vector<ov::PropertyName> all;
        for (auto& n : Configuration::rw_properties()) all.emplace_back(n, ov::PropertyMutability::RO);
        for (const char* n : {ov::supported_properties.name(), ov::model_name.name(), ov::execution_devices.name(),
                              ov::optimal_number_of_infer_requests.name(), ov::loaded_from_cache.name(), "HIP_NUMBER_OF_GRAPHS",
                              "HIP_GRAPH_LAUNCHES"})
            all.emplace_back(n, ov::PropertyMutability::RO);
        return all;
    }
    return config_.get(name);
}

void CompiledModel::record_execution_time(const std::string& node_name, uint64_t microseconds) const {
    std::lock_guard<std::mutex> lock(perf_mutex_);
    auto& entry = perf_[node_name];
    entry.first += microseconds;
    entry.second += 1;
}

std::shared_ptr<const ov::Model> CompiledModel::get_runtime_model() const {
    auto model = model_->clone();
    size_t exec_order = 0;
    std::lock_guard<std::mutex> lock(perf_mutex_);
    for (const auto& op : model->get_ordered_ops()) {
        auto& info = op->get_rt_info();
        info[ov::exec_model_info::LAYER_TYPE] = std::string(op->get_type_info().name);
        info[ov::exec_model_info::EXECUTION_ORDER] = std::to_string(exec_order++);
        info[ov::exec_model_info::IMPL_TYPE] = std::string("HIP");
        const auto it = perf_.find(op->get_friendly_name());
        const bool timed = config_.enable_profiling && it != perf_.end() && it->second.second > 0 && it->second.first > 0;
        info[ov::exec_model_info::PERF_COUNTER] = timed ? std::to_string(it->second.first / it->second.second) : std::string("not_executed");
        info[ov::exec_model_info::ORIGINAL_NAMES] = op->get_friendly_name();
        std::string precisions;
        for (size_t i = 0; i < op->get_output_size(); i++) precisions += (i ? "," : "") + op->get_output_element_type(i).get_type_name();
        info[ov::exec_model_info::OUTPUT_PRECISIONS] = precisions;
        info[ov::exec_model_info::RUNTIME_PRECISION] =
            op->get_output_size() ? op->get_output_element_type(0).get_type_name() : std::string("undefined");
    }
    return model;
}

void CompiledModel::export_model(std::ostream& model_stream) const {
    std::stringstream xml_file, bin_file;
    ov::pass::Serialize serializer(xml_file, bin_file);
    serializer.run_on_model(model_);
    const std::string model = xml_file.str(), weights = bin_file.str();
    std::uint64_t n = model.size();
    model_stream.write(reinterpret_cast<const char*>(&n), sizeof(n));
    model_stream.write(model.data(), (std::streamsize)n);
    n = weights.size();
    model_stream.write(reinterpret_cast<const char*>(&n), sizeof(n));
    model_stream.write(weights.data(), (std::streamsize)n);
}

// --------------------------------------------------------------------------- InferRequest
InferRequest::InferRequest(const std::shared_ptr<const CompiledModel>& compiled,
                           const std::shared_ptr<ov::threading::ITaskExecutor>& wait_executor)
    : ov::ISyncInferRequest(compiled),
      compiled_(compiled),
      wait_executor_(wait_executor),
      views_(compiled->num_tensors()),
      tensor_buffers_(compiled->num_tensors()) {
    HIP_PLUGIN_CHECK(hipattn_set_device(compiled_->config().device_id));
    // host tensors for ports of known shape; dynamic outputs are shaped by infer_postprocess
    auto host_tensor = [](const ov::Output<const ov::Node>& port) {
        return [port](ov::SoPtr<ov::ITensor>& tensor) {
            const auto& ps = port.get_partial_shape();
            ov::Shape shape;
            for (const auto& d : ps) shape.push_back(d.is_static() ? (size_t)d.get_length() : 0);
            tensor = ov::SoPtr<ov::ITensor>{ov::make_tensor(port.get_element_type(), shape), nullptr};
        };
    };
    for (const auto& port : get_inputs())
        if (port.get_partial_shape().is_static()) allocate_tensor(port, host_tensor(port));
    for (const auto& port : get_outputs()) allocate_tensor(port, host_tensor(port));
    for (const auto& variable : compiled_->get_runtime_model()->get_variables())
        variables_.add(variable->get_info().variable_id, std::make_shared<VariableState>(variable->get_info()));
    // ReadValue / Assign change host-side state while they enqueue: such a model runs operator by
    // operator (the reference keeps stateful and dynamic models off its graph runner too,
    // src/cuda_compiled_model.cpp:53-62)
    int operators = 0;
    for (const auto& step : compiled_->exec_sequence()) {
        const std::string& type = step.op->GetTypeName();
        operators += (type != "Parameter" && type != "Result" && type != "Constant");
    }
    graph_allowed_ = compiled_->config().use_graph && !compiled_->config().enable_profiling && variables_.all().empty() &&
                     operators >= compiled_->config().graph_min_operators;
}

std::vector<ov::SoPtr<ov::IVariableState>> InferRequest::query_state() const {
    std::vector<ov::SoPtr<ov::IVariableState>> states;
    for (const auto& [id, state] : variables_.all()) states.emplace_back(state, nullptr);
    return states;
}

void InferRequest::infer() {
    // the whole request on a worker of the device's pool, which owns the stream
    // (src/cuda_infer_request.cpp:232-254)
    infer_preprocess();
    auto pool = std::dynamic_pointer_cast<ThreadPool>(wait_executor_);
    wait_executor_->run_and_wait({[this, pool] {
        const ThreadContext& tc = pool->get_thread_context();
        start_pipeline(tc);
        wait_pipeline(tc);
    }});
    infer_postprocess();
}

void InferRequest::set_tensors_impl(const ov::Output<const ov::Node> port, const std::vector<ov::SoPtr<ov::ITensor>>& tensors) {
    for (const auto& input : get_inputs()) {
        if (!(input == port)) continue;
        OPENVINO_ASSERT(!tensors.empty(), "set_tensors: no tensors for input '", port.get_node()->get_friendly_name(), "'");
        const ov::Shape& first = tensors[0]->get_shape();
        for (const auto& t : tensors) {
            OPENVINO_ASSERT(t, "set_tensors: a tensor is not initialized");
            OPENVINO_ASSERT(std::dynamic_pointer_cast<RemoteTensor>(t._ptr) == nullptr,
                            "set_tensors: device tensors cannot be put together into a batch; pass one tensor");
            OPENVINO_ASSERT(port.get_element_type().compatible(t->get_element_type()), "set_tensors: element type ",
                            t->get_element_type(), " does not match the input's ", port.get_element_type());
            OPENVINO_ASSERT(!first.empty() && first[0] == 1 && t->get_shape() == first,
                            "set_tensors: every tensor must hold one batch entry of the same shape, got ", t->get_shape());
        }
        ov::Shape whole = first;
        whole[0] = tensors.size();
        OPENVINO_ASSERT(port.get_partial_shape().compatible(ov::PartialShape(whole)), "set_tensors: ", tensors.size(),
                        " tensors of shape ", first, " do not fit the input's ", port.get_partial_shape());
        batched_tensors_[{port.get_node(), port.get_index()}] = tensors;
        return;
    }
    OPENVINO_THROW("Cannot find input tensors for port ", port.get_node()->get_friendly_name());
}

// (a single tensor set later replaces a batch set before)
void InferRequest::set_tensor(const ov::Output<const ov::Node>& port, const ov::SoPtr<ov::ITensor>& tensor) {
    ov::ISyncInferRequest::set_tensor(port, tensor);
    batched_tensors_.erase({port.get_node(), port.get_index()});
}

// The batches set with set_tensors become one host tensor each, entry after entry along the first axis
// (what ISyncInferRequest::convert_batched_tensors does for the reference, src/cuda_infer_request.cpp:111).
void InferRequest::bind_batched_tensors() {
    for (const auto& input : get_inputs()) {
        const auto it = batched_tensors_.find({input.get_node(), input.get_index()});
        if (it == batched_tensors_.end()) continue;
        const auto& parts = it->second;
        ov::Shape whole = parts[0]->get_shape();
        whole[0] = parts.size();
        auto joined = ov::make_tensor(parts[0]->get_element_type(), whole);
        const size_t bytes = parts[0]->get_byte_size();
        for (size_t i = 0; i < parts.size(); i++) std::memcpy((uint8_t*)joined->data() + i * bytes, parts[i]->data(), bytes);
        ov::ISyncInferRequest::set_tensor(input, ov::SoPtr<ov::ITensor>{joined, nullptr});
    }
}

void InferRequest::infer_preprocess() {
    bind_batched_tensors();
    check_tensors();
    cancellation_.reset();
}

void InferRequest::cancel() { cancellation_.cancel(); }

void InferRequest::start_pipeline(const ThreadContext& thread_context) {
    const Stream& stream = thread_context.stream;
    HIP_PLUGIN_CHECK(hipattn_set_device(compiled_->config().device_id));
    const bool profiling = compiled_->config().enable_profiling;
    const InferenceRequestContext context{stream, profiling, &variables_, &cancellation_};
    ev_begin_.clear();
    ev_end_.clear();
    ev_step_.clear();
    profiling_.clear();
    const auto& results = compiled_->results();

    // Shapes, memory and scratch of every operator first (nothing is enqueued but uploads), then the
    // operators themselves: one after the other, or as one graph when this infer is a repeat of the
    // last one in everything the operators were handed.
    prepare_steps(thread_context, context);
    const bool graph_mode = graph_allowed_ && !profiling;
    if (graph_mode) signature_ = make_signature();
    if (graph_mode && graph_ && signature_ == last_signature_) {
        if (cancellation_.is_cancelled()) throw ov::Cancelled("Infer Request was canceled");
        graph_.launch(stream);
        graph_launches_++;
        compiled_->count_graph_launch();
    } else if (graph_mode && signature_ == last_signature_) {
        // the second infer in a row with this signature: everything it needs is allocated, record it
        Graph::begin_capture(stream);
        bool recorded = false;
        try {
            execute_steps(context, false);
            recorded = graph_.end_capture(stream);
        } catch (...) {
            graph_.end_capture(stream);  // leave capture mode before the error travels on
            graph_.reset();
            throw;
        }
        if (recorded) {
            graphs_captured_++;
            compiled_->count_graph_captured();
            graph_.launch(stream);
            graph_launches_++;
            compiled_->count_graph_launch();
        } else {
            graph_allowed_ = false;  // this model does not record: run it operator by operator from now on
            execute_steps(context, false);
        }
    } else {
        graph_.reset();
        execute_steps(context, profiling);
    }
    if (graph_mode) last_signature_ = signature_;
    // an input an operator updated in place that the caller bound as host memory: the update goes
    // back there (slow -- a KV cache belongs in a device tensor -- but never silently lost)
    const auto& sequence = compiled_->exec_sequence();
    for (size_t si = 0; si < sequence.size(); si++)
        for (size_t idx : sequence[si].op->UpdatedInputs()) {
            const auto& in = prepared_[si].in;
            if (idx < in.size() && in[idx].host && in[idx].byte_size())
                stream.download(const_cast<void*>(in[idx].host), in[idx].device, in[idx].byte_size());
        }

    // results into the host tensors of the output ports (device-bound outputs were written in place,
    // or are copied device to device when they alias something else)
    for (size_t i = 0; i < results.size(); i++) {
        const auto src = results[i]->input_value(0);
        const TensorView& v = views_[compiled_->output_ids(src.get_node()).at(src.get_index())];
        auto t = get_tensor(get_outputs().at(i));
        if (auto remote = std::dynamic_pointer_cast<RemoteTensor>(t._ptr)) {
            if (remote->get_shape() != v.shape) remote->set_shape(v.shape);
            if (remote->device_ptr() != v.device && v.byte_size()) stream.transfer(remote->device_ptr(), v.device, v.byte_size());
            continue;
        }
        if (t->get_shape() != v.shape) t->set_shape(v.shape);
        if (v.byte_size()) stream.download(t->data(), v.device, v.byte_size());
    }
}

void InferRequest::prepare_steps(const ThreadContext& thread_context, const InferenceRequestContext& context) {
    const Stream& stream = thread_context.stream;
    // The request's tensors are kept per port of the compiled model; port i belongs to parameter i /
    // result i of the model the execution sequence was built from.
    const auto& parameters = compiled_->parameters();
    const auto& results = compiled_->results();
    std::map<const ov::Node*, ov::SoPtr<ov::ITensor>> input_tensors;
    for (size_t i = 0; i < parameters.size(); i++) input_tensors[parameters[i].get()] = get_tensor(get_inputs().at(i));
    // output ports bound to device tensors receive the operator's result in place
    std::map<TensorID, void*> remote_outputs;
    for (size_t i = 0; i < results.size(); i++) {
        auto t = get_tensor(get_outputs().at(i));
        if (auto remote = std::dynamic_pointer_cast<RemoteTensor>(t._ptr)) {
            const auto src = results[i]->input_value(0);
            remote_outputs[compiled_->output_ids(src.get_node()).at(src.get_index())] = remote->device_ptr();
        }
    }
    const auto& sequence = compiled_->exec_sequence();
    prepared_.assign(sequence.size(), PreparedStep{});
    // Intermediate tensors -- operator outputs that are neither views of an input, nor bound to a caller's
    // device tensor, nor constants -- live in one blob, at offsets worked out from their lifetimes once every
    // shape of this infer is known (hip_memory_solver.hpp; the reference's mutable blob,
    // src/memory_manager/model/cuda_memory_model_builder.cpp:11-25).  First pass: shapes, and the memory
    // that is known without the blob; second pass: the blob's addresses, then the scratch requests (an
    // operator may size its scratch by which of its inputs are there).
    struct Packed {
        TensorID id;
        size_t bytes;
        int step;
    };
    std::vector<Packed> packed;
    std::vector<TensorID> owner(views_.size());  // the tensor whose memory a tensor is (itself, unless it is a view)
    for (size_t id = 0; id < owner.size(); id++) owner[id] = (TensorID)id;
    const int kToTheEnd = (int)sequence.size();
    std::vector<int> last_use(views_.size(), -1);
    for (size_t si = 0; si < sequence.size(); si++) {
        const auto& step = sequence[si];
        const ov::Node& node = *step.node;
        const auto& out_ids = step.op->GetOutputIds();
        PreparedStep& ps = prepared_[si];
        if (ov::as_type<const ov::op::v0::Parameter>(&node)) {
            // bind or upload (the reference uploads every input on every infer,
            // src/ops/parameter.cpp:24-33; device-resident tensors are passed through untouched)
            auto t = input_tensors.at(&node);
            TensorView v;
            v.type = t->get_element_type();
            v.shape = t->get_shape();
            if (auto remote = std::dynamic_pointer_cast<RemoteTensor>(t._ptr)) {
                v.device = remote->device_ptr();
            } else {
                v.host = t->data();
                if (!compiled_->is_host_only(out_ids[0])) {
                    v.device = tensor_buffers_[out_ids[0]].reserve(std::max<size_t>(v.byte_size(), 16));
                    if (v.byte_size()) stream.upload(v.device, v.host, v.byte_size());
                }
            }
            views_[out_ids[0]] = v;
            ps.out.push_back(v);
            continue;
        }
        for (TensorID id : step.op->GetInputIds()) {
            ps.in.push_back(views_[id]);
            last_use[owner[id]] = std::max(last_use[owner[id]], (int)si);
        }
        const std::vector<ov::Shape> out_shapes = step.op->InferOutputShapes(ps.in, context);
        for (size_t o = 0; o < out_ids.size(); o++) {
            TensorView v;
            v.type = node.get_output_element_type(o);
            v.shape = out_shapes.at(o);
            const int alias = step.op->InplaceInputOf(o);
            auto bound = remote_outputs.find(out_ids[o]);
            if (alias >= 0) {
                v.device = ps.in.at(alias).device;  // (of a tensor in the blob: filled in by the second pass)
                v.host = ps.in.at(alias).host;
                owner[out_ids[o]] = owner[step.op->GetInputIds().at(alias)];
                if (bound != remote_outputs.end() && v.byte_size()) ps.copies.push_back({bound->second, nullptr, v.byte_size(), o});
            } else if (bound != remote_outputs.end()) {
                v.device = bound->second;
            } else if (step.op->HostData(o) && compiled_->is_host_only(out_ids[o])) {
                v.host = step.op->HostData(o);  // a Constant only ever read on the host
            } else if (const void* host = step.op->HostData(o)) {  // a Constant: uploaded once per request
                v.device = tensor_buffers_[out_ids[o]].reserve(std::max<size_t>(v.byte_size(), 16));
                v.host = host;
                if (v.byte_size() && constants_on_device_.insert(out_ids[o]).second) stream.upload(v.device, host, v.byte_size());
            } else {
                packed.push_back({out_ids[o], std::max<size_t>(v.byte_size(), 16), (int)si});
            }
            ps.out.push_back(v);
            views_[out_ids[o]] = v;
        }
    }
    // what the caller reads after the last step stays to the end
    for (size_t i = 0; i < results.size(); i++) {
        const auto src = results[i]->input_value(0);
        last_use[owner[compiled_->output_ids(src.get_node()).at(src.get_index())]] = kToTheEnd;
    }
    std::vector<MemoryBox> boxes;
    size_t apart = 0;
    for (const Packed& t : packed) {
        boxes.push_back({t.bytes, t.step, std::max(last_use[t.id], t.step)});
        apart += (t.bytes + 255) / 256 * 256;
    }
    // (a decode loop asks for the same boxes infer after infer: the solution is kept)
    const auto same_box = [](const MemoryBox& a, const MemoryBox& b) { return a.bytes == b.bytes && a.start == b.start && a.end == b.end; };
    if (!(boxes.size() == solved_boxes_.size() && std::equal(boxes.begin(), boxes.end(), solved_boxes_.begin(), same_box))) {
        packed_bytes_ = solve_memory(boxes, solved_offsets_);
        solved_boxes_ = boxes;
    }
    char* const blob = packed_bytes_ ? (char*)thread_context.blob.reserve(packed_bytes_) : nullptr;
    for (size_t i = 0; i < packed.size(); i++) views_[packed[i].id].device = blob + solved_offsets_[i];
    unpacked_bytes_ = apart;

    // second pass: every view with its final address; scratch -- one arena for all steps (they run one after
    // the other on the request's stream), sized for the largest request before any pointer into it is handed out
    std::vector<WorkbufferRequest> requests(sequence.size());
    for (size_t si = 0; si < sequence.size(); si++) {
        const auto& step = sequence[si];
        if (ov::as_type<const ov::op::v0::Parameter>(step.node.get())) continue;
        PreparedStep& ps = prepared_[si];
        const auto& in_ids = step.op->GetInputIds();
        const auto& out_ids = step.op->GetOutputIds();
        for (size_t i = 0; i < ps.in.size(); i++) ps.in[i].device = views_[in_ids[i]].device;
        for (size_t o = 0; o < ps.out.size(); o++) {
            const int alias = step.op->InplaceInputOf(o);
            if (alias >= 0) views_[out_ids[o]].device = ps.in.at(alias).device;
            ps.out[o].device = views_[out_ids[o]].device;
        }
        for (auto& c : ps.copies) c.from = ps.out.at(c.output).device;
        ps.copies.erase(std::remove_if(ps.copies.begin(), ps.copies.end(), [](const PreparedStep::CopyOut& c) { return c.to == c.from; }),
                        ps.copies.end());
        requests[si] = step.op->GetWorkBufferRequest(ps.in);
    }
    size_t arena = 0;
    for (const auto& req : requests) {
        size_t total = 0;
        for (size_t b : req.mutable_sizes) total += (b + 255) / 256 * 256;
        arena = std::max(arena, total);
    }
    char* const arena_base = arena ? (char*)thread_context.workbuffer.reserve(arena) : nullptr;
    for (size_t si = 0; si < sequence.size(); si++) {
        char* base = arena_base;
        for (size_t b : requests[si].mutable_sizes) {
            prepared_[si].workbuffers.mutable_buffers.push_back(base);
            prepared_[si].workbuffers.mutable_sizes.push_back(b);
            base += (b + 255) / 256 * 256;
        }
    }
}

void InferRequest::execute_steps(const InferenceRequestContext& context, bool profiling) {
    const auto& sequence = compiled_->exec_sequence();
    for (size_t si = 0; si < sequence.size(); si++) {
        const auto& step = sequence[si];
        if (ov::as_type<const ov::op::v0::Parameter>(step.node.get())) continue;
        if (cancellation_.is_cancelled()) throw ov::Cancelled("Infer Request was canceled");
        if (profiling) {
            ev_begin_.emplace_back(new Event());
            ev_end_.emplace_back(new Event());
            ev_step_.push_back(si);
            ev_begin_.back()->record(context.stream);
        }
        step.op->Execute(context, prepared_[si].in, prepared_[si].out, prepared_[si].workbuffers);
        for (const auto& c : prepared_[si].copies) context.stream.transfer(c.to, c.from, c.bytes);
        if (profiling) ev_end_.back()->record(context.stream);
    }
}

// Everything the operators of this infer were handed, as numbers: two infers with equal signatures
// enqueue the same launches on the same memory.  Host-side values an operator may read while it
// launches (scalars such as a scale, a window or a context bound) are part of it when they are
// small; the shapes cover what larger host tensors decide (the extent of the scores output).
std::vector<uint64_t> InferRequest::make_signature() const {
    std::vector<uint64_t> sig;
    auto add_view = [&](const TensorView& v, bool value_matters = true) {
        sig.push_back((uint64_t)(uintptr_t)v.device);
        sig.push_back(v.shape.size());
        for (size_t d : v.shape) sig.push_back(d);
        const size_t bytes = v.byte_size();
        if (v.host != nullptr && bytes > 0 && bytes <= 64 && value_matters) {
            uint64_t words[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            std::memcpy(words, v.host, bytes);
            sig.insert(sig.end(), words, words + (bytes + 7) / 8);
        } else {
            sig.push_back(v.host != nullptr);
        }
    };
    const auto& sequence = compiled_->exec_sequence();
    for (size_t si = 0; si < prepared_.size(); si++) {
        const auto& ps = prepared_[si];
        // (small host-side values are part of the signature unless every consumer says the value is advisory)
        const auto& in_ids = sequence[si].op->GetInputIds();
        const auto& out_ids = compiled_->output_ids(sequence[si].node.get());
        for (size_t i = 0; i < ps.in.size(); i++) add_view(ps.in[i], i >= in_ids.size() || !compiled_->has_advisory_value(in_ids[i]));
        for (size_t o = 0; o < ps.out.size(); o++) add_view(ps.out[o], o >= out_ids.size() || !compiled_->has_advisory_value(out_ids[o]));
        for (size_t i = 0; i < ps.workbuffers.mutable_buffers.size(); i++) {
            sig.push_back((uint64_t)(uintptr_t)ps.workbuffers.mutable_buffers[i]);
            sig.push_back(ps.workbuffers.mutable_sizes[i]);
        }
        for (const auto& c : ps.copies) sig.push_back((uint64_t)(uintptr_t)c.to);
    }
    return sig;
}

void InferRequest::wait_pipeline(const ThreadContext& thread_context) { thread_context.stream.synchronize(); }

void InferRequest::infer_postprocess() {
    const auto& sequence = compiled_->exec_sequence();
    for (size_t i = 0; i < ev_step_.size(); i++) {
        const auto& step = sequence[ev_step_[i]];
        ov::ProfilingInfo info;
        info.status = ov::ProfilingInfo::Status::EXECUTED;
        info.real_time = std::chrono::microseconds((long long)(1e3 * ev_begin_[i]->elapsed_ms_until(*ev_end_[i])));
        info.cpu_time = info.real_time;
        info.node_name = step.op->GetName();
        info.node_type = step.op->GetTypeName();
        info.exec_type = "HIP";
        profiling_.push_back(info);
        compiled_->record_execution_time(info.node_name, (uint64_t)info.real_time.count());
    }
}

std::vector<ov::ProfilingInfo> InferRequest::get_profiling_info() const {
    if (!compiled_->config().enable_profiling)
        HIP_PLUGIN_THROW("profiling was not enabled for this compiled model (set PERF_COUNT to YES)");
    return profiling_;
}

// ---------------------------------------------------------------------- AsyncInferRequest
AsyncInferRequest::AsyncInferRequest(const std::shared_ptr<InferRequest>& request,
                                     const std::shared_ptr<ov::threading::ITaskExecutor>& task_executor,
                                     const std::shared_ptr<ov::threading::ITaskExecutor>& wait_executor,
                                     const std::shared_ptr<ov::threading::ITaskExecutor>& callback_executor)
    : ov::IAsyncInferRequest(request, task_executor, callback_executor), request_(request) {
    // three stages over two executors, as src/cuda_async_infer_request.cpp:26-46: host work on the
    // task executor, everything that touches the stream on a worker of the device's pool
    auto pool = std::dynamic_pointer_cast<ThreadPool>(wait_executor);
    m_pipeline = {{task_executor, [this] { request_->infer_preprocess(); }},
                  {wait_executor,
                   [this, pool] {
                       const ThreadContext& tc = pool->get_thread_context();
                       request_->start_pipeline(tc);
                       request_->wait_pipeline(tc);
                   }},
                  {task_executor, [this] { request_->infer_postprocess(); }}};
}

AsyncInferRequest::~AsyncInferRequest() { ov::IAsyncInferRequest::stop_and_wait(); }

void AsyncInferRequest::cancel() {
    ov::IAsyncInferRequest::cancel();
    request_->cancel();
}

void AsyncInferRequest::infer_thread_unsafe() { start_async_thread_unsafe(); }

}  // namespace hip_gpu
}  // namespace ov
