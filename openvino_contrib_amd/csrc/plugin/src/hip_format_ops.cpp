// Operators that change how a tensor is seen or stored between the others of a decoder layer:
// Reshape, Squeeze and Unsqueeze (views: the output is the input's memory under another shape, as the
// reference's NopOp, modules/nvidia_plugin/src/ops/nop_op.hpp:29-44 and nop_op.cpp:12-16), Transpose
// (src/ops/transpose.cpp:54-135; the order comes from a Constant or from a host tensor at run time,
// :272-300) and Convert (src/ops/convert.cpp:19-58).  The last two call libhipops (include/hipops.h).
#include <algorithm>
#include <cstring>

#include "hip_operation.hpp"
#include "hipops.h"
#include "openvino/op/constant.hpp"
#include "openvino/op/convert.hpp"
#include "openvino/op/reshape.hpp"
#include "openvino/op/squeeze.hpp"
#include "openvino/op/transpose.hpp"
#include "openvino/op/unsqueeze.hpp"

namespace ov {
namespace hip_gpu {

namespace {

inline void throw_if_format_error(hipattn_status st, const char* file, int line, const char* func) {
    if (st != HIPATTN_OK)
        throw_ov_exception(std::string(hipattn_status_string(st)) + ": " + hipops_last_error_string(), file, line, func);
}
#define HIP_FORMAT_CHECK(expr) ::ov::hip_gpu::throw_if_format_error((expr), __FILE__, __LINE__, __func__)

std::string dims_str(const ov::Shape& s) {
    std::string r = "[";
    for (size_t i = 0; i < s.size(); i++) r += (i ? "," : "") + std::to_string(s[i]);
    return r + "]";
}

bool integer_index_type(const ov::element::Type& t) { return t == ov::element::i32 || t == ov::element::i64; }

// The values of a small integer input (a shape pattern, axes, an order) from its host bytes: a
// Constant always has them, a Parameter when the request bound a host tensor.
std::vector<int64_t> host_integers(const TensorView& view, const std::string& who, const char* what) {
    const size_t n = ov::shape_size(view.shape);
    if (n == 0) return {};
    HIP_PLUGIN_ASSERT(view.host != nullptr, who + what + " must be a Constant or a tensor bound from host memory");
    std::vector<int64_t> values(n);
    if (view.type == ov::element::i64) {
        std::memcpy(values.data(), view.host, n * 8);
    } else {
        HIP_PLUGIN_ASSERT(view.type == ov::element::i32, who + what + " of type " + view.type.get_type_name());
        const int32_t* v = static_cast<const int32_t*>(view.host);
        std::copy(v, v + n, values.begin());
    }
    return values;
}

// A view: nothing runs, the output is the input's buffer.
class ViewOp : public OperationBase {
public:
    using OperationBase::OperationBase;
    void Execute(const InferenceRequestContext&, Inputs, Outputs, const Workbuffers&) const override {}
    int InplaceInputOf(size_t) const override { return 0; }
    bool InputIsHostOnly(size_t input) const override { return input == 1; }  // the pattern or the axes
};

class ReshapeOp : public ViewOp {
public:
    ReshapeOp(const CreationContext& ctx, const ov::Node& node, IndexCollection&& in, IndexCollection&& out)
        : ViewOp(ctx, node, std::move(in), std::move(out)), who_("Reshape '" + node.get_friendly_name() + "': ") {
        auto reshape = ov::as_type<const ov::op::v1::Reshape>(&node);
        HIP_PLUGIN_ASSERT(reshape != nullptr, "not a Reshape node");
        if (node.get_input_size() != 2 || !integer_index_type(node.get_input_element_type(1))) HIP_PLUGIN_THROW(who_ + "data and an i32 / i64 pattern expected");
        special_zero_ = reshape->get_special_zero();
    }
    std::vector<ov::Shape> InferOutputShapes(const std::vector<TensorView>& in, const InferenceRequestContext&) const override {
        const ov::Shape& from = in.at(0).shape;
        const std::vector<int64_t> want = host_integers(in.at(1), who_, "the pattern");
        ov::Shape to(want.size());
        size_t known = 1;
        int open = -1;
        for (size_t i = 0; i < want.size(); i++) {
            if (want[i] == 0 && special_zero_) {
                HIP_PLUGIN_ASSERT(i < from.size(), who_ + "a 0 at position " + std::to_string(i) + " has no input axis to copy");
                to[i] = from[i];
            } else if (want[i] == -1) {
                HIP_PLUGIN_ASSERT(open < 0, who_ + "more than one -1 in the pattern");
                open = (int)i;
                continue;
            } else {
                HIP_PLUGIN_ASSERT(want[i] >= 0, who_ + "negative extent in the pattern");
                to[i] = (size_t)want[i];
            }
            known *= to[i];
        }
        const size_t total = ov::shape_size(from);
        if (open >= 0) {
            HIP_PLUGIN_ASSERT(known > 0 ? total % known == 0 : total == 0, who_ + dims_str(from) + " does not divide into the pattern");
            to[open] = known > 0 ? total / known : 0;
            known *= to[open];
        }
        HIP_PLUGIN_ASSERT(known == total, who_ + dims_str(from) + " and " + dims_str(to) + " hold different numbers of elements");
        return {to};
    }

private:
    std::string who_;
    bool special_zero_ = false;
};

class SqueezeOp : public ViewOp {
public:
    SqueezeOp(const CreationContext& ctx, const ov::Node& node, IndexCollection&& in, IndexCollection&& out)
        : ViewOp(ctx, node, std::move(in), std::move(out)), who_("Squeeze '" + node.get_friendly_name() + "': ") {
        if (node.get_input_size() != 1 && node.get_input_size() != 2) HIP_PLUGIN_THROW(who_ + "data [, axes] expected");
        if (node.get_input_size() == 2 && !integer_index_type(node.get_input_element_type(1))) HIP_PLUGIN_THROW(who_ + "i32 / i64 axes expected");
    }
    std::vector<ov::Shape> InferOutputShapes(const std::vector<TensorView>& in, const InferenceRequestContext&) const override {
        const ov::Shape& from = in.at(0).shape;
        ov::Shape to;
        if (in.size() == 1) {
            for (size_t d : from)
                if (d != 1) to.push_back(d);
            return {to};
        }
        std::vector<bool> drop(from.size(), false);
        for (int64_t a : host_integers(in[1], who_, "the axes")) {
            if (a < 0) a += (int64_t)from.size();
            HIP_PLUGIN_ASSERT(a >= 0 && a < (int64_t)from.size(), who_ + "axis out of range for " + dims_str(from));
            drop[(size_t)a] = true;
        }
        for (size_t k = 0; k < from.size(); k++)
            if (!(drop[k] && from[k] == 1)) to.push_back(from[k]);  // an axis that is not 1 stays, as in opset 1
        return {to};
    }

private:
    std::string who_;
};

class UnsqueezeOp : public ViewOp {
public:
    UnsqueezeOp(const CreationContext& ctx, const ov::Node& node, IndexCollection&& in, IndexCollection&& out)
        : ViewOp(ctx, node, std::move(in), std::move(out)), who_("Unsqueeze '" + node.get_friendly_name() + "': ") {
        if (node.get_input_size() != 2 || !integer_index_type(node.get_input_element_type(1))) HIP_PLUGIN_THROW(who_ + "data and i32 / i64 axes expected");
    }
    std::vector<ov::Shape> InferOutputShapes(const std::vector<TensorView>& in, const InferenceRequestContext&) const override {
        const ov::Shape& from = in.at(0).shape;
        const std::vector<int64_t> axes = host_integers(in.at(1), who_, "the axes");
        const int64_t rank = (int64_t)(from.size() + axes.size());
        std::vector<bool> fresh((size_t)rank, false);
        for (int64_t a : axes) {
            if (a < 0) a += rank;
            HIP_PLUGIN_ASSERT(a >= 0 && a < rank && !fresh[(size_t)a], who_ + "axis out of range or repeated");
            fresh[(size_t)a] = true;
        }
        ov::Shape to;
        for (size_t k = 0, next = 0; k < (size_t)rank; k++) to.push_back(fresh[k] ? 1 : from[next++]);
        return {to};
    }

private:
    std::string who_;
};

class TransposeOp : public OperationBase {
public:
    TransposeOp(const CreationContext& ctx, const ov::Node& node, IndexCollection&& in, IndexCollection&& out)
        : OperationBase(ctx, node, std::move(in), std::move(out)), who_("Transpose '" + node.get_friendly_name() + "': ") {
        if (node.get_input_size() != 2 || !integer_index_type(node.get_input_element_type(1))) HIP_PLUGIN_THROW(who_ + "data and an i32 / i64 order expected");
        element_bytes_ = node.get_input_element_type(0).size();
        if (element_bytes_ != 1 && element_bytes_ != 2 && element_bytes_ != 4 && element_bytes_ != 8)
            HIP_PLUGIN_THROW(who_ + "data of type " + node.get_input_element_type(0).get_type_name());
        if (node.get_input_partial_shape(0).size() > HIPOPS_TRANSPOSE_MAX_RANK)
            HIP_PLUGIN_THROW(who_ + "rank " + std::to_string(node.get_input_partial_shape(0).size()) + " (at most " +
                             std::to_string(HIPOPS_TRANSPOSE_MAX_RANK) + ")");
    }
    bool InputIsHostOnly(size_t input) const override { return input == 1; }  // the order
    std::vector<ov::Shape> InferOutputShapes(const std::vector<TensorView>& in, const InferenceRequestContext&) const override {
        const ov::Shape& from = in.at(0).shape;
        const std::vector<int32_t> order = order_of(in);
        ov::Shape to(from.size());
        for (size_t k = 0; k < from.size(); k++) to[k] = from[(size_t)order[k]];
        return {to};
    }
    void Execute(const InferenceRequestContext& context, Inputs in, Outputs out, const Workbuffers&) const override {
        const ov::Shape& from = in[0].shape;
        const std::vector<int32_t> order = order_of(in);
        std::vector<int64_t> dims(from.begin(), from.end());
        HIP_FORMAT_CHECK(hipops_transpose(in[0].device, out[0].device, (int)from.size(), dims.data(), order.data(), (int)element_bytes_,
                                          context.stream.get()));
    }

private:
    // an empty order reverses the axes (OpenVINO's rule)
    std::vector<int32_t> order_of(const std::vector<TensorView>& in) const {
        const size_t rank = in.at(0).shape.size();
        const std::vector<int64_t> given = host_integers(in.at(1), who_, "the order");
        std::vector<int32_t> order(rank);
        if (given.empty()) {
            for (size_t k = 0; k < rank; k++) order[k] = (int32_t)(rank - 1 - k);
            return order;
        }
        HIP_PLUGIN_ASSERT(given.size() == rank, who_ + "the order names " + std::to_string(given.size()) + " axes of " + dims_str(in[0].shape));
        std::vector<bool> seen(rank, false);
        for (size_t k = 0; k < rank; k++) {
            HIP_PLUGIN_ASSERT(given[k] >= 0 && given[k] < (int64_t)rank && !seen[(size_t)given[k]], who_ + "the order is not a permutation of the axes");
            seen[(size_t)given[k]] = true;
            order[k] = (int32_t)given[k];
        }
        return order;
    }
    std::string who_;
    size_t element_bytes_ = 0;
};

bool convert_dtype(const ov::element::Type& t, int& out) {
    if (t == ov::element::f32) return out = HIPATTN_F32, true;
    if (t == ov::element::f16) return out = HIPATTN_F16, true;
    if (t == ov::element::bf16) return out = HIPATTN_BF16, true;
    if (t == ov::element::i32) return out = HIPATTN_I32, true;
    if (t == ov::element::i64) return out = HIPOPS_I64, true;
    if (t == ov::element::u8) return out = HIPOPS_U8, true;
    if (t == ov::element::i8) return out = HIPOPS_I8, true;
    if (t == ov::element::boolean) return out = HIPOPS_BOOL, true;
    return false;
}

class ConvertOp : public OperationBase {
public:
    ConvertOp(const CreationContext& ctx, const ov::Node& node, IndexCollection&& in, IndexCollection&& out)
        : OperationBase(ctx, node, std::move(in), std::move(out)) {
        const std::string who = "Convert '" + node.get_friendly_name() + "': ";
        if (node.get_input_size() != 1 || node.get_output_size() != 1) HIP_PLUGIN_THROW(who + "one input and one output expected");
        if (!convert_dtype(node.get_input_element_type(0), from_) || !convert_dtype(node.get_output_element_type(0), to_))
            HIP_PLUGIN_THROW(who + node.get_input_element_type(0).get_type_name() + " to " + node.get_output_element_type(0).get_type_name() +
                             " (f32, f16, bf16, i32, i64, u8, i8, boolean expected)");
    }
    std::vector<ov::Shape> InferOutputShapes(const std::vector<TensorView>& in, const InferenceRequestContext&) const override {
        return {in.at(0).shape};
    }
    void Execute(const InferenceRequestContext& context, Inputs in, Outputs out, const Workbuffers&) const override {
        HIP_FORMAT_CHECK(hipops_convert(in[0].device, out[0].device, (int64_t)ov::shape_size(in[0].shape), from_, to_, context.stream.get()));
    }

private:
    int from_ = 0, to_ = 0;
};

}  // namespace

}  // namespace hip_gpu
}  // namespace ov

using ov::hip_gpu::ConvertOp;
using ov::hip_gpu::ReshapeOp;
using ov::hip_gpu::SqueezeOp;
using ov::hip_gpu::TransposeOp;
using ov::hip_gpu::UnsqueezeOp;
HIP_OPERATION_REGISTER(ReshapeOp, Reshape)
HIP_OPERATION_REGISTER(SqueezeOp, Squeeze)
HIP_OPERATION_REGISTER(UnsqueezeOp, Unsqueeze)
HIP_OPERATION_REGISTER(TransposeOp, Transpose)
HIP_OPERATION_REGISTER(ConvertOp, Convert)
