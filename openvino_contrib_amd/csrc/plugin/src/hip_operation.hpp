// Per-operator contract and registry of the "HIP" plugin.
//
// Mirrors the reference's contract -- IOperationExec / OperationBase
// (modules/nvidia_plugin/src/cuda_operation_base.hpp:33-149), OperationRegistry and
// OPERATION_REGISTER (src/cuda_operation_registry.hpp:48-109, 133-143) -- with one deliberate
// difference: operators are shape-polymorphic.  The reference resolves dynamic shapes by cloning
// a statically shaped operator per distinct input shape (src/cuda_dynamic_operation.cpp:128-230,
// LRU of 300); attention inputs change shape on every step (tokens in the batch, block tables),
// so here Execute() receives the runtime shapes with the pointers and the operator object stays
// immutable and shared by all concurrent requests.
#pragma once

#include <atomic>
#include <functional>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "hip_device.hpp"
#include "openvino/core/node.hpp"
#include "openvino/core/shape.hpp"
#include "openvino/core/type/element_type.hpp"

namespace ov {
namespace hip_gpu {

using TensorID = size_t;
class VariableState;

struct CreationContext {
    int device_id = 0;
    bool op_benchmark = false;
};

// One operand at run time: device pointer, element type, concrete shape.  `host` is a host copy of
// the same bytes when the request has one (small index / scalar inputs set from host memory, and
// Constant nodes).
struct TensorView {
    void* device = nullptr;
    const void* host = nullptr;
    ov::element::Type type;
    ov::Shape shape;
    size_t byte_size() const { return ov::shape_size(shape) * type.size(); }
};

struct WorkbufferRequest {
    std::vector<size_t> immutable_sizes;  // filled once at compile time (unused by the attention ops)
    std::vector<size_t> mutable_sizes;    // per-request scratch
};

struct Workbuffers {
    std::vector<void*> mutable_buffers;
    std::vector<size_t> mutable_sizes;
};

// Set by InferRequest::cancel(); the executor looks at it between operators
// (src/cancellation_token.hpp in the reference).
class CancellationToken {
public:
    void cancel() { cancelled_.store(true); }
    void reset() { cancelled_.store(false); }
    bool is_cancelled() const { return cancelled_.load(); }

private:
    std::atomic<bool> cancelled_{false};
};

// Variable states of one infer request, by variable id (src/cuda_variable_state.hpp:186-238).
class VariableContext {
public:
    void add(const std::string& id, const std::shared_ptr<VariableState>& state) { states_[id] = state; }
    std::shared_ptr<VariableState> get(const std::string& id) const {
        auto it = states_.find(id);
        if (it == states_.end()) HIP_PLUGIN_THROW("no variable state with id '" + id + "'");
        return it->second;
    }
    const std::map<std::string, std::shared_ptr<VariableState>>& all() const { return states_; }

private:
    std::map<std::string, std::shared_ptr<VariableState>> states_;
};

struct InferenceRequestContext {
    const Stream& stream;
    bool profiling = false;
    const VariableContext* variables = nullptr;
    const CancellationToken* cancellation = nullptr;
};

class OperationBase {
public:
    using Ptr = std::shared_ptr<OperationBase>;
    using IndexCollection = std::vector<TensorID>;
    using Inputs = const std::vector<TensorView>&;
    using Outputs = const std::vector<TensorView>&;

    OperationBase(const CreationContext&, const ov::Node& node, IndexCollection&& input_ids, IndexCollection&& output_ids)
        : node_name_(node.get_friendly_name()),
          type_name_(node.get_type_info().name),
          input_ids_(std::move(input_ids)),
          output_ids_(std::move(output_ids)) {}
    virtual ~OperationBase() = default;

    // Concrete output shapes for concrete input shapes (what validate_and_infer_types gives a clone
    // in the reference, src/cuda_dynamic_operation.cpp:419-468).
    virtual std::vector<ov::Shape> InferOutputShapes(const std::vector<TensorView>& inputs,
                                                     const InferenceRequestContext& context) const = 0;
    // Scratch the operator needs for these shapes; the request provides it in Execute().
    virtual WorkbufferRequest GetWorkBufferRequest(const std::vector<TensorView>& /*inputs*/) const { return {}; }
    // Enqueue the operator on context.stream.  const: one instance serves every request.  Must only
    // enqueue (kernel launches, device-to-device copies): a request may record the call into a graph
    // and replay it.  Host bytes of an input (TensorView::host) may steer the launch only when the
    // input holds at most 64 bytes -- those are part of the signature a replay is keyed by; whatever a
    // larger host input decides has to show in InferOutputShapes.
    virtual void Execute(const InferenceRequestContext& context, Inputs inputs, Outputs outputs,
                         const Workbuffers& workbuffers) const = 0;
    // Outputs that alias an input buffer and are updated in place (input index per output, -1 = none).
    virtual int InplaceInputOf(size_t /*output*/) const { return -1; }
    // Inputs the operator updates in place on the device (the KV caches of PagedAttentionExtension).
    // When such an input was bound as a host tensor the request copies it back after the operator,
    // so the caller's memory holds the update; device-resident tensors need nothing.
    virtual std::vector<size_t> UpdatedInputs() const { return {}; }
    // True for an input the operator only ever reads through TensorView::host (a scale, a window, a
    // shape pattern, an order): a tensor all of whose consumers say so is not uploaded, and its
    // TensorView::device is null.
    virtual bool InputIsHostOnly(size_t /*input*/) const { return false; }
    // False for a host-side input whose VALUE changes nothing the operator launches (a bound that is only
    // advisory): the request leaves such a value out of the signature by which it recognises a repeat of
    // the previous infer, so that a value that moves with every step does not keep it from replaying the
    // recorded graph.
    virtual bool InputValueShapesLaunch(size_t /*input*/) const { return true; }
    // Told once, while the model is compiled, that nothing consumes this output: an operator may then
    // skip producing it (the scores of PagedAttentionExtension).
    virtual void MarkOutputUnused(size_t /*output*/) {}
    // Host bytes the operator itself provides for an output (Constant); nullptr otherwise.
    virtual const void* HostData(size_t /*output*/) const { return nullptr; }

    const std::string& GetName() const { return node_name_; }
    const std::string& GetTypeName() const { return type_name_; }
    const IndexCollection& GetInputIds() const { return input_ids_; }
    const IndexCollection& GetOutputIds() const { return output_ids_; }

protected:
    std::string node_name_;
    std::string type_name_;
    const IndexCollection input_ids_;
    const IndexCollection output_ids_;
};

class OperationRegistry final {
public:
    using IndexCollection = OperationBase::IndexCollection;
    using OperationBuilder = std::function<OperationBase::Ptr(const CreationContext&, const std::shared_ptr<ov::Node>&,
                                                              IndexCollection&&, IndexCollection&&)>;
    template <typename TOperation>
    class Register {
    public:
        explicit Register(const std::string& type_name) {
            getInstance().registerOp(type_name, [](const CreationContext& context, const std::shared_ptr<ov::Node>& node,
                                                   IndexCollection&& in, IndexCollection&& out) -> OperationBase::Ptr {
                return std::make_shared<TOperation>(context, *node, std::move(in), std::move(out));
            });
        }
    };

    static OperationRegistry& getInstance() {
        static OperationRegistry registry;
        return registry;
    }
    bool hasOperation(const std::shared_ptr<ov::Node>& node) const {
        return builders_.count(node->get_type_info().name) != 0;
    }
    // Throws when the type is unknown or the operator's constructor rejects the node: that is how
    // query_model learns what is supported (src/cuda_plugin.cpp:171-188).
    OperationBase::Ptr createOperation(const CreationContext& context, const std::shared_ptr<ov::Node>& node,
                                       IndexCollection&& in, IndexCollection&& out) const {
        auto it = builders_.find(node->get_type_info().name);
        if (it == builders_.end())
            HIP_PLUGIN_THROW(std::string("operation '") + node->get_type_info().name + "' (node '" +
                             node->get_friendly_name() + "') is not supported by the HIP plugin");
        return it->second(context, node, std::move(in), std::move(out));
    }
    std::vector<std::string> registeredTypes() const {
        std::vector<std::string> names;
        for (auto& kv : builders_) names.push_back(kv.first);
        return names;
    }

private:
    void registerOp(const std::string& type_name, OperationBuilder&& builder) {
        if (!builders_.emplace(type_name, std::move(builder)).second)
            throw std::runtime_error("HIP plugin: two operator classes claim the node type '" + type_name + "'");
    }
    std::map<std::string, OperationBuilder> builders_;
};

}  // namespace hip_gpu
}  // namespace ov

// Registers `type` (derived from OperationBase, constructible from
// (const CreationContext&, const ov::Node&, IndexCollection&&, IndexCollection&&)) for nodes whose
// type name is `name`.
#define HIP_OPERATION_REGISTER(type, name)                                                                       \
    extern "C" {                                                                                                 \
    [[maybe_unused]] const ::ov::hip_gpu::OperationRegistry::Register<type> hip_plugin_op_register_##name{#name}; \
    }
