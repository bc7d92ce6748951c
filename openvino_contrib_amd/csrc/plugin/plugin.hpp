// Plugin / CompiledModel / InferRequest of the "HIP" device, shaped after the reference's
// Plugin : ov::IPlugin (modules/nvidia_plugin/src/cuda_plugin.hpp:18-83),
// CompiledModel : ov::ICompiledModel (src/cuda_compiled_model.hpp:30-83) and
// CudaInferRequest : ov::ISyncInferRequest (src/cuda_infer_request.hpp:34-55), written against the
// stand-in graph types of graph.hpp because OpenVINO's developer headers are not available to
// this build.  Method names, argument meaning and error behaviour follow the OpenVINO interfaces
// so that the classes can be re-based onto them.
#pragma once

#include <future>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <variant>
#include <vector>

#include "graph.hpp"
#include "hip_device.hpp"
#include "operation.hpp"

namespace hip_plugin {

using Any = std::variant<std::string, int64_t, bool, double>;
using AnyMap = std::map<std::string, Any>;

// Property names (OpenVINO's spellings)
namespace props {
constexpr const char* device_id = "DEVICE_ID";
constexpr const char* inference_precision = "INFERENCE_PRECISION_HINT";
constexpr const char* enable_profiling = "PERF_COUNT";
constexpr const char* num_streams = "NUM_STREAMS";
constexpr const char* performance_mode = "PERFORMANCE_HINT";
constexpr const char* supported_properties = "SUPPORTED_PROPERTIES";
constexpr const char* available_devices = "AVAILABLE_DEVICES";
constexpr const char* full_device_name = "FULL_DEVICE_NAME";
constexpr const char* device_architecture = "DEVICE_ARCHITECTURE";
constexpr const char* optimal_number_of_infer_requests = "OPTIMAL_NUMBER_OF_INFER_REQUESTS";
constexpr const char* range_for_async_infer_requests = "RANGE_FOR_ASYNC_INFER_REQUESTS";
constexpr const char* model_name = "NETWORK_NAME";
constexpr const char* execution_devices = "EXECUTION_DEVICES";
}  // namespace props

// Value object rebuilt from an AnyMap over a base, as src/cuda_config.cpp:147-189 does.
struct Configuration {
    int device_id = 0;
    std::string inference_precision = "dynamic";  // keep the model's precision; f32 / f16 / bf16 are accepted
    bool enable_profiling = false;
    int num_streams = 1;
    std::string performance_mode = "LATENCY";

    static Configuration from(const AnyMap& properties, const Configuration& base, bool throw_on_unsupported = true);
    Any get(const std::string& name) const;
    static const std::vector<std::string>& rw_properties();
};

// Host tensor (ov::Tensor over user memory or own storage) or device-resident tensor
// (what an ov::RemoteTensor of this device would be: the KV caches live here and are updated in place).
struct Tensor {
    ElementType type = ElementType::dynamic;
    Shape shape;
    void* data = nullptr;   // host pointer, or device pointer when `remote`
    bool remote = false;
    std::shared_ptr<std::vector<uint8_t>> storage;  // set when the tensor owns host memory
    size_t byte_size() const { return (size_t)shape_size(shape) * element_size(type); }
};

struct ProfilingInfo {
    std::string node_name, node_type, exec_type;
    double real_time_us = 0.0;
};

class Plugin;
class InferRequest;

class CompiledModel : public std::enable_shared_from_this<CompiledModel> {
public:
    CompiledModel(const std::shared_ptr<const Model>& model, const Configuration& config,
                  const std::shared_ptr<const Plugin>& plugin);

    std::shared_ptr<InferRequest> create_infer_request() const;
    std::shared_ptr<InferRequest> create_sync_infer_request() const { return create_infer_request(); }
    const std::vector<std::shared_ptr<Node>>& inputs() const { return model_->parameters; }
    const std::vector<std::shared_ptr<Node>>& outputs() const { return model_->results; }
    Any get_property(const std::string& name) const;
    void set_property(const AnyMap&) { throw NotImplemented("CompiledModel::set_property"); }
    void export_model(std::ostream&) const { throw NotImplemented("CompiledModel::export_model"); }
    // (node name, type) of every executed operator, in execution order
    std::vector<std::pair<std::string, std::string>> get_runtime_model() const;

private:
    friend class InferRequest;
    struct ExecStep {
        std::shared_ptr<Node> node;
        OperationBase::Ptr op;
    };
    std::shared_ptr<const Model> model_;
    Configuration config_;
    std::shared_ptr<const Plugin> plugin_;
    std::vector<ExecStep> exec_sequence_;
    std::map<const Node*, std::vector<TensorID>> output_ids_;  // per node: one TensorID per output port
    size_t num_tensors_ = 0;
};

class InferRequest {
public:
    explicit InferRequest(const std::shared_ptr<const CompiledModel>& compiled);

    void set_tensor(const std::string& port_name, const Tensor& tensor);
    void set_input_tensor(size_t index, const Tensor& tensor);
    Tensor get_tensor(const std::string& port_name) const;
    Tensor get_output_tensor(size_t index) const;
    void infer();                 // preprocess -> start_pipeline -> wait_pipeline -> postprocess
    void start_async();
    void wait();
    std::vector<ProfilingInfo> get_profiling_info() const;
    std::vector<std::string> query_state() const { return {}; }  // no variables: the KV cache is an input

private:
    std::shared_ptr<const CompiledModel> compiled_;
    Stream stream_;
    std::map<std::string, Tensor> bound_inputs_;
    std::map<std::string, Tensor> outputs_;
    std::vector<Allocation> tensor_buffers_;      // per TensorID, grow-only
    std::vector<Allocation> workbuffers_;         // per exec step
    std::vector<ProfilingInfo> profiling_;
    std::future<void> pending_;
    std::mutex mutex_;
};

class Plugin : public std::enable_shared_from_this<Plugin> {
public:
    Plugin();
    const std::string& get_device_name() const { return device_name_; }

    void set_property(const AnyMap& properties);
    Any get_property(const std::string& name, const AnyMap& arguments = {}) const;
    std::shared_ptr<CompiledModel> compile_model(const std::shared_ptr<const Model>& model,
                                                 const AnyMap& properties = {}) const;
    // node friendly name -> device name for every node the plugin can execute
    std::map<std::string, std::string> query_model(const std::shared_ptr<const Model>& model,
                                                   const AnyMap& properties = {}) const;
    std::shared_ptr<CompiledModel> import_model(std::istream&, const AnyMap&) const {
        throw NotImplemented("Plugin::import_model");
    }
    void create_context(const AnyMap&) const { throw NotImplemented("Plugin::create_context"); }
    void get_default_context(const AnyMap&) const { throw NotImplemented("Plugin::get_default_context"); }

    bool is_operation_supported(const std::shared_ptr<Node>& node, const Configuration& config) const;

private:
    Configuration get_full_config(const AnyMap& properties, bool throw_on_unsupported = true) const;
    std::string device_name_ = "HIP";
    int device_count_ = 0;
    Configuration config_;
    mutable std::mutex mutex_;
};

}  // namespace hip_plugin
