// Minimal graph model the plugin-side classes are written against.
//
// The real boundary is OpenVINO's (ov::Model / ov::Node / ov::Tensor); its headers are not
// available to this build, so the handful of facts the attention path needs from a node --
// type name, friendly name, per-port element type and partial shape, a few attributes -- are
// carried by these plain structs.  The names follow OpenVINO's so that the operator classes read
// like the ones in modules/nvidia_plugin/src/ops/ and port mechanically once `ov::Node` is there.
#pragma once

#include <cstdint>
#include <map>
#include <memory>
#include <string>
#include <variant>
#include <vector>

#include "hipattn.h"

namespace hip_plugin {

enum class ElementType { f32, f16, bf16, u8, i32, dynamic };

inline size_t element_size(ElementType t) {
    switch (t) {
        case ElementType::f32:
        case ElementType::i32: return 4;
        case ElementType::f16:
        case ElementType::bf16: return 2;
        case ElementType::u8: return 1;
        default: return 0;
    }
}

inline const char* element_name(ElementType t) {
    switch (t) {
        case ElementType::f32: return "f32";
        case ElementType::f16: return "f16";
        case ElementType::bf16: return "bf16";
        case ElementType::u8: return "u8";
        case ElementType::i32: return "i32";
        default: return "dynamic";
    }
}

// f32 / f16 / bf16 / u8 map onto the C ABI's dtype enum
inline bool to_hipattn_dtype(ElementType t, hipattn_dtype& out) {
    switch (t) {
        case ElementType::f32: out = HIPATTN_F32; return true;
        case ElementType::f16: out = HIPATTN_F16; return true;
        case ElementType::bf16: out = HIPATTN_BF16; return true;
        case ElementType::u8: out = HIPATTN_U8; return true;
        default: return false;
    }
}

using Shape = std::vector<int64_t>;         // static
using PartialShape = std::vector<int64_t>;  // -1 marks a dynamic dimension

inline bool is_dynamic(const PartialShape& s) {
    for (auto d : s)
        if (d < 0) return true;
    return false;
}
inline int64_t shape_size(const Shape& s) {
    int64_t n = 1;
    for (auto d : s) n *= d;
    return n;
}

struct Node;
struct Output {  // a producer port
    std::shared_ptr<Node> node;
    size_t index = 0;
};

using Attribute = std::variant<int64_t, double, bool, std::string>;

struct Node {
    std::string type_name;      // "Parameter", "Result", "ScaledDotProductAttention", "PagedAttentionExtension", ...
    std::string friendly_name;
    std::vector<Output> inputs;
    std::vector<ElementType> output_types;
    std::vector<PartialShape> output_shapes;
    std::map<std::string, Attribute> attrs;

    ElementType get_input_element_type(size_t i) const { return inputs.at(i).node->output_types.at(inputs[i].index); }
    const PartialShape& get_input_partial_shape(size_t i) const {
        return inputs.at(i).node->output_shapes.at(inputs[i].index);
    }
    bool get_bool(const std::string& key, bool dflt) const {
        auto it = attrs.find(key);
        return it == attrs.end() ? dflt : std::get<bool>(it->second);
    }
};

struct Model {
    std::string name;
    std::vector<std::shared_ptr<Node>> ordered_ops;  // topological order
    std::vector<std::shared_ptr<Node>> parameters;
    std::vector<std::shared_ptr<Node>> results;
};

// ---- builders (what ov::op::v0::Parameter, v13::ScaledDotProductAttention, ... would be) ----
class ModelBuilder {
public:
    explicit ModelBuilder(std::string name) { model_->name = std::move(name); }

    Output parameter(const std::string& name, ElementType type, PartialShape shape) {
        auto n = add("Parameter", name, {}, {type}, {std::move(shape)});
        model_->parameters.push_back(n);
        return {n, 0};
    }
    // v13::ScaledDotProductAttention(query, key, value, causal); the output has the query's type and shape
    Output scaled_dot_product_attention(const std::string& name, Output q, Output k, Output v, bool causal) {
        auto n = add("ScaledDotProductAttention", name, {q, k, v}, {q.node->output_types[q.index]},
                     {q.node->output_shapes[q.index]});
        n->attrs["causal"] = causal;
        return {n, 0};
    }
    // PagedAttentionExtension: inputs in the operator's order (query, key, value, key_cache, value_cache,
    // past_lens, subsequence_begins, block_indices, block_indices_begins, scale, sliding_window,
    // alibi_slopes, max_context_len); out0 has the query's type and shape
    Output paged_attention(const std::string& name, const std::vector<Output>& in) {
        const Output& q = in.at(0);
        auto n = add("PagedAttentionExtension", name, in, {q.node->output_types[q.index]},
                     {q.node->output_shapes[q.index]});
        return {n, 0};
    }
    Output unknown_op(const std::string& type, const std::string& name, const std::vector<Output>& in) {
        const Output& a = in.at(0);
        auto n = add(type, name, in, {a.node->output_types[a.index]}, {a.node->output_shapes[a.index]});
        return {n, 0};
    }
    void result(const std::string& name, Output value) {
        auto n = add("Result", name, {value}, {value.node->output_types[value.index]},
                     {value.node->output_shapes[value.index]});
        model_->results.push_back(n);
    }
    std::shared_ptr<Model> build() { return model_; }

private:
    std::shared_ptr<Node> add(const std::string& type, const std::string& name, std::vector<Output> in,
                              std::vector<ElementType> types, std::vector<PartialShape> shapes) {
        auto n = std::make_shared<Node>();
        n->type_name = type;
        n->friendly_name = name;
        n->inputs = std::move(in);
        n->output_types = std::move(types);
        n->output_shapes = std::move(shapes);
        model_->ordered_ops.push_back(n);
        return n;
    }
    std::shared_ptr<Model> model_ = std::make_shared<Model>();
};

}  // namespace hip_plugin
