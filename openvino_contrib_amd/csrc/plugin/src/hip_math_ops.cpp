// Element-wise arithmetic with numpy broadcasting and Softmax: with MatMul and Transpose, the
// operators attention consists of when a model carries it decomposed (what the reference executes
// after ScaledDotProductAttentionDecomposition, modules/nvidia_plugin/src/transformer/
// cuda_graph_transformer.cpp:151-156).  BinaryOp follows ElementwiseBinaryOp
// (src/ops/elementwise_binary.hpp:16-76; AddOp src/ops/add.cpp:17-43, MultiplyOp
// src/ops/multiply.cpp:43, SubtractOp, DivideOp), SoftmaxOp follows src/ops/softmax.cpp:163-196.
#include <algorithm>

#include "hip_operation.hpp"
#include "hipops.h"
#include "openvino/op/add.hpp"
#include "openvino/op/divide.hpp"
#include "openvino/op/multiply.hpp"
#include "openvino/op/softmax.hpp"
#include "openvino/op/subtract.hpp"

namespace ov {
namespace hip_gpu {

namespace {

inline void throw_if_math_error(hipattn_status st, const char* file, int line, const char* func) {
    if (st != HIPATTN_OK)
        throw_ov_exception(std::string(hipattn_status_string(st)) + ": " + hipops_last_error_string(), file, line, func);
}
#define HIP_MATH_CHECK(expr) ::ov::hip_gpu::throw_if_math_error((expr), __FILE__, __LINE__, __func__)

std::string dims_text(const ov::Shape& s) {
    std::string r = "[";
    for (size_t i = 0; i < s.size(); i++) r += (i ? "," : "") + std::to_string(s[i]);
    return r + "]";
}

bool float_code(const ov::element::Type& t, int& out) {
    if (t == ov::element::f32) return out = HIPATTN_F32, true;
    if (t == ov::element::f16) return out = HIPATTN_F16, true;
    if (t == ov::element::bf16) return out = HIPATTN_BF16, true;
    return false;
}

// numpy's rule: shapes aligned at their last axes, an extent of 1 stretches
ov::Shape broadcast(const ov::Shape& a, const ov::Shape& b, const std::string& who) {
    const size_t rank = std::max(a.size(), b.size());
    ov::Shape out(rank);
    for (size_t k = 0; k < rank; k++) {
        const size_t da = k + a.size() >= rank ? a[k + a.size() - rank] : 1;
        const size_t db = k + b.size() >= rank ? b[k + b.size() - rank] : 1;
        HIP_PLUGIN_ASSERT(da == db || da == 1 || db == 1, who + dims_text(a) + " and " + dims_text(b) + " do not broadcast");
        out[k] = da == 1 ? db : da;
    }
    return out;
}

class BinaryOp : public OperationBase {
public:
    BinaryOp(const CreationContext& ctx, const ov::Node& node, IndexCollection&& in, IndexCollection&& out)
        : OperationBase(ctx, node, std::move(in), std::move(out)) {
        const std::string type = node.get_type_info().name;
        who_ = type + " '" + node.get_friendly_name() + "': ";
        if (type == "Add")
            operation_ = HIPOPS_ADD;
        else if (type == "Subtract")
            operation_ = HIPOPS_SUBTRACT;
        else if (type == "Multiply")
            operation_ = HIPOPS_MULTIPLY;
        else if (type == "Divide")
            operation_ = HIPOPS_DIVIDE;
        else
            HIP_PLUGIN_THROW(who_ + "not an element-wise arithmetic node");
        if (node.get_input_size() != 2 || node.get_output_size() != 1) HIP_PLUGIN_THROW(who_ + "two inputs and one output expected");
        type_ = node.get_output_element_type(0);
        // as the reference: all three of one type (elementwise_binary.hpp:31-36)
        if (node.get_input_element_type(0) != type_ || node.get_input_element_type(1) != type_) HIP_PLUGIN_THROW(who_ + "mixed precisions");
        if (!float_code(type_, dtype_) && !(type_ == ov::element::i32 && operation_ == HIPOPS_ADD))
            HIP_PLUGIN_THROW(who_ + "precision " + type_.get_type_name() + " (f32, f16 or bf16 expected; i32 for an Add of equal shapes)");
        if (node.get_input_partial_shape(0).size() > HIPOPS_BINARY_MAX_RANK || node.get_input_partial_shape(1).size() > HIPOPS_BINARY_MAX_RANK)
            HIP_PLUGIN_THROW(who_ + "rank beyond " + std::to_string(HIPOPS_BINARY_MAX_RANK));
    }
    std::vector<ov::Shape> InferOutputShapes(const std::vector<TensorView>& in, const InferenceRequestContext&) const override {
        ov::Shape out = broadcast(in.at(0).shape, in.at(1).shape, who_);
        if (type_ == ov::element::i32) HIP_PLUGIN_ASSERT(in[0].shape == in[1].shape, who_ + "i32 operands must have one shape");
        return {out};
    }
    void Execute(const InferenceRequestContext& context, Inputs in, Outputs out, const Workbuffers&) const override {
        const ov::Shape& to = out[0].shape;
        if (type_ == ov::element::i32) {
            HIP_PLUGIN_CHECK(hipattn_add_async(out[0].device, in[0].device, in[1].device, (int64_t)ov::shape_size(to), HIPATTN_I32,
                                               context.stream.get()));
            return;
        }
        const size_t rank = to.size();
        std::vector<int64_t> od(rank), ad(rank, 1), bd(rank, 1);
        for (size_t k = 0; k < rank; k++) od[k] = (int64_t)to[k];
        for (size_t k = 0; k < in[0].shape.size(); k++) ad[rank - in[0].shape.size() + k] = (int64_t)in[0].shape[k];
        for (size_t k = 0; k < in[1].shape.size(); k++) bd[rank - in[1].shape.size() + k] = (int64_t)in[1].shape[k];
        HIP_MATH_CHECK(hipops_binary(operation_, in[0].device, in[1].device, out[0].device, (int)rank, od.data(), ad.data(), bd.data(), dtype_,
                                     context.stream.get()));
    }

private:
    std::string who_;
    ov::element::Type type_;
    int operation_ = HIPOPS_ADD, dtype_ = 0;
};

class SoftmaxOp : public OperationBase {
public:
    SoftmaxOp(const CreationContext& ctx, const ov::Node& node, IndexCollection&& in, IndexCollection&& out)
        : OperationBase(ctx, node, std::move(in), std::move(out)) {
        const std::string who = "Softmax '" + node.get_friendly_name() + "': ";
        if (node.get_input_size() != 1 || node.get_output_size() != 1) HIP_PLUGIN_THROW(who + "one input and one output expected");
        if (!float_code(node.get_input_element_type(0), dtype_) || node.get_output_element_type(0) != node.get_input_element_type(0))
            HIP_PLUGIN_THROW(who + "f32, f16 or bf16 expected, the output of the input's type");
        const int64_t rank = (int64_t)node.get_input_partial_shape(0).size();
        if (auto v8 = ov::as_type<const ov::op::v8::Softmax>(&node))
            axis_ = v8->get_axis();
        else if (auto v1 = ov::as_type<const ov::op::v1::Softmax>(&node))
            axis_ = (int64_t)v1->get_axis();
        else
            HIP_PLUGIN_THROW(who + "not a Softmax node");
        if (axis_ < 0) axis_ += rank;
        if (rank < 1 || axis_ < 0 || axis_ >= rank) HIP_PLUGIN_THROW(who + "axis out of range for rank " + std::to_string(rank));
    }
    std::vector<ov::Shape> InferOutputShapes(const std::vector<TensorView>& in, const InferenceRequestContext&) const override {
        return {in.at(0).shape};
    }
    void Execute(const InferenceRequestContext& context, Inputs in, Outputs out, const Workbuffers&) const override {
        const ov::Shape& s = in[0].shape;
        int64_t outer = 1, inner = 1;
        for (int64_t k = 0; k < axis_; k++) outer *= (int64_t)s[k];
        for (size_t k = (size_t)axis_ + 1; k < s.size(); k++) inner *= (int64_t)s[k];
        HIP_MATH_CHECK(hipops_softmax(in[0].device, out[0].device, outer, (int64_t)s[axis_], inner, dtype_, context.stream.get()));
    }

private:
    int64_t axis_ = -1;
    int dtype_ = 0;
};

}  // namespace

}  // namespace hip_gpu
}  // namespace ov

using ov::hip_gpu::BinaryOp;
using ov::hip_gpu::SoftmaxOp;
HIP_OPERATION_REGISTER(BinaryOp, Add)
HIP_OPERATION_REGISTER(BinaryOp, Subtract)
HIP_OPERATION_REGISTER(BinaryOp, Multiply)
HIP_OPERATION_REGISTER(BinaryOp, Divide)
HIP_OPERATION_REGISTER(SoftmaxOp, Softmax)
