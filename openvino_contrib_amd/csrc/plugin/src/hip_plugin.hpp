// Plugin / CompiledModel / InferRequest / AsyncInferRequest of the "HIP" device.
//
// Shaped after the reference's Plugin : ov::IPlugin (modules/nvidia_plugin/src/cuda_plugin.hpp:18-83),
// CompiledModel : ov::ICompiledModel (src/cuda_compiled_model.hpp:30-83), CudaInferRequest :
// ov::ISyncInferRequest (src/cuda_infer_request.hpp:34-55), CudaAsyncInferRequest :
// ov::IAsyncInferRequest (src/cuda_async_infer_request.hpp:14-29), CudaThreadPool
// (src/cuda_thread_pool.hpp) and CudaVariableState (src/cuda_variable_state.hpp:31-183), with the
// same base classes and virtual signatures.  The sources name only OpenVINO's own headers: they
// compile against the developer package where it is installed and against the stand-in tree
// (plugin/standin/) elsewhere.  What differs from the reference by design: no graph transformation
// stage that decomposes attention, shape-polymorphic operators instead of per-shape clones, and a
// remote context, because a paged KV cache has to stay on the device between infer calls.
#pragma once

#include <condition_variable>
#include <deque>
#include <map>
#include <memory>
#include <mutex>
#include <atomic>
#include <set>
#include <string>
#include <thread>
#include <vector>

#include "hip_device.hpp"
#include "hip_memory_solver.hpp"
#include "hip_operation.hpp"
#include "openvino/core/any.hpp"
#include "openvino/core/model.hpp"
#include "openvino/op/util/variable.hpp"
#include "openvino/runtime/iasync_infer_request.hpp"
#include "openvino/runtime/icompiled_model.hpp"
#include "openvino/runtime/iplugin.hpp"
#include "openvino/runtime/iremote_context.hpp"
#include "openvino/runtime/iremote_tensor.hpp"
#include "openvino/runtime/isync_infer_request.hpp"
#include "openvino/runtime/ivariable_state.hpp"
#include "openvino/runtime/make_tensor.hpp"
#include "openvino/runtime/profiling_info.hpp"
#include "openvino/runtime/properties.hpp"
#include "openvino/runtime/threading/itask_executor.hpp"

namespace ov {
namespace hip_gpu {

// Value object rebuilt from an AnyMap over a base, as src/cuda_config.cpp:147-189 does.
struct Configuration {
    int device_id = 0;
    ov::element::Type inference_precision = ov::element::dynamic;  // dynamic: keep the model's precision
    bool enable_profiling = false;
    int num_streams = 1;
    std::string performance_mode = "LATENCY";
    // Replay the operator sequence of an infer request from a captured graph when nothing about it
    // has changed (the reference's NVIDIA_USE_CUDA_GRAPH, nvidia/properties.hpp:30).
    bool use_graph = true;
    // ... for models of at least this many operators (Parameter, Result and Constant not counted).
    // Measured on MI355X / ROCm 7.2 with 64-token RMS + MatMul layers: launching a graph costs more
    // than two kernel launches and less than eight (2 kernels 35 us against 26 us one by one, 8 kernels
    // 65 against 73, 32 kernels 173 against 225), so a lone attention operator stays off the graph.
    int graph_min_operators = 6;

    static Configuration from(const ov::AnyMap& properties, const Configuration& base, bool throw_on_unsupported = true);
    ov::Any get(const std::string& name) const;
    static const std::vector<std::string>& rw_properties();
};

// A tensor that lives in device memory: the KV caches, and anything else the caller keeps on the
// device between infer calls.  Either owns its allocation or wraps a device pointer the caller
// owns (property "DEV_PTR").
class RemoteTensor : public ov::IRemoteTensor {
public:
    RemoteTensor(const ov::element::Type& type, const ov::Shape& shape, void* wrapped, const std::string& device_name);
    void set_shape(ov::Shape shape) override;
    const ov::element::Type& get_element_type() const override { return type_; }
    const ov::Shape& get_shape() const override { return shape_; }
    const ov::AnyMap& get_properties() const override { return properties_; }
    const std::string& get_device_name() const override { return device_name_; }
    void* device_ptr() const { return wrapped_ ? wrapped_ : owned_.get(); }

private:
    ov::element::Type type_;
    ov::Shape shape_;
    void* wrapped_ = nullptr;
    Allocation owned_;
    ov::AnyMap properties_;
    std::string device_name_;
};

class RemoteContext : public ov::IRemoteContext {
public:
    RemoteContext(const std::string& device_name, int device_id);
    const std::string& get_device_name() const override { return device_name_; }
    const ov::AnyMap& get_property() const override { return properties_; }
    ov::SoPtr<ov::IRemoteTensor> create_tensor(const ov::element::Type& type, const ov::Shape& shape,
                                               const ov::AnyMap& params = {}) override;

private:
    std::string device_name_;
    int device_id_;
    ov::AnyMap properties_;
};

// Device-resident variable (ReadValue / Assign): grow-only capacity, logical shape, reset flag.
class VariableState : public ov::IVariableState {
public:
    explicit VariableState(const ov::op::util::VariableInfo& info);
    void set_state(const ov::SoPtr<ov::ITensor>& state) override;
    ov::SoPtr<ov::ITensor> get_state() const override;
    void reset() override;

    // fast path of the operators: device to device on the request's stream
    bool is_reset_state() const;
    ov::Shape shape() const;
    size_t byte_size() const;
    void update_device_state(const Stream& stream, const void* src, const ov::Shape& new_shape);
    void read_device_state(const Stream& stream, void* dst, size_t dst_bytes) const;

private:
    size_t logical_bytes() const { return type_.size() * ov::shape_size(current_shape_); }
    mutable std::mutex mutex_;
    ov::PartialShape data_shape_;
    ov::element::Type type_;
    ov::Shape initial_shape_, current_shape_;
    Allocation buffer_;
    bool is_reset_ = true;
};

// Worker threads of one device; each owns a stream.  Tasks handed to run() execute on one of them
// (src/cuda_thread_pool.cpp:11-72); the stream of the executing thread is get_thread_context().
// A worker also owns the memory of whatever request it is running: the blob that holds an infer's intermediate
// tensors and the scratch arena of its operators.  A compiled model with NUM_STREAMS = n thus holds n blobs however
// many requests exist, and a request that finds every worker busy waits in the pool's queue -- what the reference
// gets from a pool of n blobs that a request blocks on (src/memory_manager/cuda_memory_pool.cpp:34-42).  Both only
// grow; they are touched by the thread that owns the context alone (mutable: handed out as const ThreadContext&).
struct ThreadContext {
    Stream stream;
    mutable Allocation blob;        // every operator output of the running infer that nothing else owns, packed by lifetime
    mutable Allocation workbuffer;  // scratch arena shared by the steps of the running infer
};
class ThreadPool : public ov::threading::ITaskExecutor {
public:
    ThreadPool(int device_id, unsigned num_threads);
    ~ThreadPool() override;
    void run(ov::threading::Task task) override;
    const ThreadContext& get_thread_context();

private:
    void worker();
    int device_id_;
    std::mutex mutex_;
    std::condition_variable wake_;
    std::deque<ov::threading::Task> queue_;
    bool stopping_ = false;
    std::vector<std::thread> threads_;
};

class Plugin;
class InferRequest;

class CompiledModel : public ov::ICompiledModel {
public:
    CompiledModel(const std::shared_ptr<const ov::Model>& model, const Configuration& config,
                  const std::shared_ptr<ov::threading::ITaskExecutor>& wait_executor,
                  const std::shared_ptr<const ov::IPlugin>& plugin, bool loaded_from_cache);

    // the model with execution information in every node's rt_info (src/cuda_compiled_model.cpp:336-371)
    std::shared_ptr<const ov::Model> get_runtime_model() const override;
    // what an infer request measured for one operator (profiling on): feeds the runtime model's execTimeMcs
    void record_execution_time(const std::string& node_name, uint64_t microseconds) const;
    void export_model(std::ostream& model) const override;
    std::shared_ptr<ov::IAsyncInferRequest> create_infer_request() const override;
    void set_property(const ov::AnyMap& properties) override;
    ov::Any get_property(const std::string& name) const override;

    struct ExecStep {
        std::shared_ptr<ov::Node> node;
        OperationBase::Ptr op;
    };
    const std::vector<ExecStep>& exec_sequence() const { return exec_sequence_; }
    size_t num_tensors() const { return num_tensors_; }
    const std::vector<TensorID>& output_ids(const ov::Node* node) const { return output_ids_.at(node); }
    // no consumer of this tensor reads it on the device (OperationBase::InputIsHostOnly)
    bool is_host_only(TensorID id) const { return host_only_tensors_.count(id) != 0; }
    // every consumer takes this tensor's host-side value as advisory (OperationBase::InputValueShapesLaunch)
    bool has_advisory_value(TensorID id) const { return advisory_value_tensors_.count(id) != 0; }
    const Configuration& config() const { return config_; }
    const ov::ParameterVector& parameters() const { return exec_model_->get_parameters(); }
    const ov::ResultVector& results() const { return exec_model_->get_results(); }
    void count_graph_captured() const { graphs_captured_++; }
    void count_graph_launch() const { graph_launches_++; }

protected:
    std::shared_ptr<ov::ISyncInferRequest> create_sync_infer_request() const override;

private:
    std::shared_ptr<ov::Model> model_;             // what get_runtime_model / export_model hand out
    std::shared_ptr<const ov::Model> exec_model_;  // the nodes the execution sequence refers to
    Configuration config_;
    std::shared_ptr<ov::threading::ITaskExecutor> wait_executor_;
    bool loaded_from_cache_;
    std::vector<ExecStep> exec_sequence_;
    std::map<const ov::Node*, std::vector<TensorID>> output_ids_;  // per node: one TensorID per output port
    std::set<TensorID> host_only_tensors_;
    std::set<TensorID> advisory_value_tensors_;
    size_t num_tensors_ = 0;
    mutable std::atomic<size_t> graphs_captured_{0}, graph_launches_{0};
    mutable std::mutex perf_mutex_;
    mutable std::map<std::string, std::pair<uint64_t, uint64_t>> perf_;  // node name -> (microseconds in all, runs)
};

class InferRequest : public ov::ISyncInferRequest {
public:
    InferRequest(const std::shared_ptr<const CompiledModel>& compiled,
                 const std::shared_ptr<ov::threading::ITaskExecutor>& wait_executor);

    void infer() override;
    std::vector<ov::SoPtr<ov::IVariableState>> query_state() const override;
    std::vector<ov::ProfilingInfo> get_profiling_info() const override;
    // several tensors, one batch entry each, for one input (src/cuda_infer_request.cpp:263-272): kept per
    // port and put together along the batch axis when the request runs (infer_preprocess)
    void set_tensors_impl(const ov::Output<const ov::Node> port, const std::vector<ov::SoPtr<ov::ITensor>>& tensors) override;
    void set_tensor(const ov::Output<const ov::Node>& port, const ov::SoPtr<ov::ITensor>& tensor) override;

    // stages of the asynchronous pipeline (src/cuda_infer_request.cpp:107-254)
    void infer_preprocess();
    void start_pipeline(const ThreadContext& thread_context);
    void wait_pipeline(const ThreadContext& thread_context);
    void infer_postprocess();
    void cancel();
    // bytes of the blob that holds the last infer's intermediate tensors, and what they would take one beside the other
    std::pair<size_t, size_t> intermediate_memory() const { return {packed_bytes_, unpacked_bytes_}; }

private:
    std::shared_ptr<const CompiledModel> compiled_;
    std::shared_ptr<ov::threading::ITaskExecutor> wait_executor_;
    std::map<std::pair<const ov::Node*, size_t>, std::vector<ov::SoPtr<ov::ITensor>>> batched_tensors_;
    void bind_batched_tensors();
    std::vector<TensorView> views_;               // per TensorID, rebuilt by every infer
    std::vector<Allocation> tensor_buffers_;      // per TensorID, grow-only: uploaded inputs and constants
    // every other operator output of one infer lies in the blob of the worker that runs it (ThreadContext), packed by lifetime
    size_t packed_bytes_ = 0, unpacked_bytes_ = 0;  // what the last infer took of that blob; what its tensors take side by side
    std::vector<MemoryBox> solved_boxes_;         // the boxes the offsets below were worked out for
    std::vector<size_t> solved_offsets_;
    std::set<TensorID> constants_on_device_;      // Constant outputs already uploaded
    std::vector<std::unique_ptr<Event>> ev_begin_, ev_end_;
    std::vector<size_t> ev_step_;
    std::vector<ov::ProfilingInfo> profiling_;
    VariableContext variables_;
    CancellationToken cancellation_;

    // What the operator sequence of one infer consists of once shapes are known and memory is bound.
    struct PreparedStep {
        std::vector<TensorView> in, out;
        Workbuffers workbuffers;
        // an output that is its input's memory (a view, a pass-through) although its port is bound to a
        // device tensor of the caller's: copied there behind the operator
        struct CopyOut {
            void* to;
            const void* from;
            size_t bytes;
            size_t output;  // the output it copies
        };
        std::vector<CopyOut> copies;
    };
    std::vector<PreparedStep> prepared_;
    // Graph replay (the reference's CudaGraphTopologyRunner, src/cuda_graph_topology_runner.cpp, for a
    // model whose shapes may change from infer to infer): the signature of an infer is every pointer,
    // shape, scratch address and small host-side value its operators were handed.  The second infer
    // in a row with one signature is recorded into a graph, later ones replay it; a new signature
    // starts over.
    std::vector<uint64_t> signature_, last_signature_;
    Graph graph_;
    size_t graph_launches_ = 0, graphs_captured_ = 0;
    bool graph_allowed_ = false;
    std::vector<uint64_t> make_signature() const;
    void prepare_steps(const ThreadContext& thread_context, const InferenceRequestContext& context);
    void execute_steps(const InferenceRequestContext& context, bool profiling);

public:
    size_t graph_launches() const { return graph_launches_; }
    size_t graphs_captured() const { return graphs_captured_; }
};

class AsyncInferRequest : public ov::IAsyncInferRequest {
public:
    AsyncInferRequest(const std::shared_ptr<InferRequest>& request,
                      const std::shared_ptr<ov::threading::ITaskExecutor>& task_executor,
                      const std::shared_ptr<ov::threading::ITaskExecutor>& wait_executor,
                      const std::shared_ptr<ov::threading::ITaskExecutor>& callback_executor);
    ~AsyncInferRequest() override;
    void cancel() override;
    void infer_thread_unsafe() override;
    const std::shared_ptr<InferRequest>& sync_request() const { return request_; }

private:
    std::shared_ptr<InferRequest> request_;
};

class Plugin : public ov::IPlugin {
public:
    Plugin();
    ~Plugin() override;

    void set_property(const ov::AnyMap& properties) override;
    ov::Any get_property(const std::string& name, const ov::AnyMap& arguments) const override;
    std::shared_ptr<ov::ICompiledModel> compile_model(const std::shared_ptr<const ov::Model>& model,
                                                      const ov::AnyMap& properties) const override;
    std::shared_ptr<ov::ICompiledModel> compile_model(const std::shared_ptr<const ov::Model>& model,
                                                      const ov::AnyMap& properties,
                                                      const ov::SoPtr<ov::IRemoteContext>& context) const override;
    std::shared_ptr<ov::ICompiledModel> import_model(std::istream& model_stream,
                                                     const ov::AnyMap& properties) const override;
    std::shared_ptr<ov::ICompiledModel> import_model(std::istream& model_stream,
                                                     const ov::SoPtr<ov::IRemoteContext>& context,
                                                     const ov::AnyMap& properties) const override;
    std::shared_ptr<ov::ICompiledModel> import_model(const ov::Tensor& model_stream,
                                                     const ov::AnyMap& properties) const override;
    std::shared_ptr<ov::ICompiledModel> import_model(const ov::Tensor& model_stream,
                                                     const ov::SoPtr<ov::IRemoteContext>& context,
                                                     const ov::AnyMap& properties) const override;
    ov::SupportedOpsMap query_model(const std::shared_ptr<const ov::Model>& model,
                                    const ov::AnyMap& properties) const override;
    ov::SoPtr<ov::IRemoteContext> create_context(const ov::AnyMap& remote_properties) const override;
    ov::SoPtr<ov::IRemoteContext> get_default_context(const ov::AnyMap& remote_properties) const override;

    bool is_operation_supported(const std::shared_ptr<ov::Node>& node, const Configuration& config) const;

private:
    std::shared_ptr<ov::threading::ITaskExecutor> get_stream_executor(const Configuration& config) const;
    Configuration get_full_config(const ov::AnyMap& properties, bool throw_on_unsupported = true) const;
    int device_count_ = 0;
    Configuration config_;
    mutable std::mutex mutex_;
    // one pool of stream-owning workers per (device, NUM_STREAMS): compiled models that ask for different
    // numbers of streams get pools of their own size
    mutable std::map<std::pair<int, int>, std::shared_ptr<ThreadPool>> device_thread_pool_;
};

}  // namespace hip_gpu
}  // namespace ov
