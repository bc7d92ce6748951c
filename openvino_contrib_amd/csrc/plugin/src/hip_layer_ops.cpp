// Operators either side of attention in a decoder layer: RMS normalisation, rotary position
// embedding, MatMul, Gather, Concat, and the gated MLP's Swish / GLU; each a thin adapter
// from node + runtime shapes to the C ABI of libhipops (include/hipops.h).
//
// MatMulOp, GatherOp and ConcatOp follow the reference's operators of the same names
// (modules/nvidia_plugin/src/ops/matmul.cpp:22-76 and 185-227, src/ops/gather.cpp:27-127,
// src/ops/concat.cpp:20-102), SwishOp likewise (src/ops/swish.cpp:41-59).  GluOp, RmsOp and RopeOp serve OpenVINO's fused internal operators GLU,
// RMS and RoPE, which the reference would receive unfused (VariadicSplit / Swish / Multiply,
// Power / ReduceMean / Sqrt / Multiply, and Slice / Multiply / Concat / Add).  As everywhere in this plugin a constructor that throws is how
// an unsupported node is reported (src/cuda_plugin.cpp:171-188).
#include <cstring>

#include "hip_operation.hpp"
#include "hipops.h"
#include "openvino/op/concat.hpp"
#include "openvino/op/constant.hpp"
#include "openvino/op/gather.hpp"
#include "openvino/op/matmul.hpp"
#include "openvino/op/swish.hpp"
#include "ov_ops/glu.hpp"
#include "ov_ops/rms.hpp"
#include "ov_ops/rotary_positional_embeddings.hpp"

namespace ov {
namespace hip_gpu {

namespace {

inline void throw_if_ops_error(hipattn_status st, const char* file, int line, const char* func) {
    if (st != HIPATTN_OK)
        throw_ov_exception(std::string(hipattn_status_string(st)) + ": " + hipops_last_error_string(), file, line, func);
}
#define HIP_OPS_CHECK(expr) ::ov::hip_gpu::throw_if_ops_error((expr), __FILE__, __LINE__, __func__)

std::string shape_str(const ov::Shape& s) {
    std::string r = "[";
    for (size_t i = 0; i < s.size(); i++) r += (i ? "," : "") + std::to_string(s[i]);
    return r + "]";
}

bool float_dtype(const ov::element::Type& t, int& out) {
    if (t == ov::element::f32) return out = HIPATTN_F32, true;
    if (t == ov::element::f16) return out = HIPATTN_F16, true;
    if (t == ov::element::bf16) return out = HIPATTN_BF16, true;
    return false;
}

size_t product(const ov::Shape& s, size_t from, size_t to) {
    size_t n = 1;
    for (size_t i = from; i < to; i++) n *= s[i];
    return n;
}

// ------------------------------------------------------------------------------ RMS
class RmsOp : public OperationBase {
public:
    RmsOp(const CreationContext& ctx, const ov::Node& node, IndexCollection&& in, IndexCollection&& out)
        : OperationBase(ctx, node, std::move(in), std::move(out)) {
        const std::string who = "RMS '" + node.get_friendly_name() + "': ";
        auto rms = ov::as_type<const ov::op::internal::RMS>(&node);
        HIP_PLUGIN_ASSERT(rms != nullptr, "not an RMS node");
        if (node.get_input_size() != 2) HIP_PLUGIN_THROW(who + "data and gamma expected");
        if (!float_dtype(node.get_input_element_type(0), x_dtype_) || !float_dtype(node.get_input_element_type(1), gamma_dtype_) ||
            !float_dtype(node.get_output_element_type(0), out_dtype_))
            HIP_PLUGIN_THROW(who + "f32, f16 or bf16 expected");
        if (node.get_input_partial_shape(0).size() < 1) HIP_PLUGIN_THROW(who + "scalar data");
        eps_ = (float)rms->get_epsilon();
    }
    std::vector<ov::Shape> InferOutputShapes(const std::vector<TensorView>& in, const InferenceRequestContext&) const override {
        return {in.at(0).shape};
    }
    void Execute(const InferenceRequestContext& context, Inputs in, Outputs out, const Workbuffers&) const override {
        const ov::Shape& x = in[0].shape;
        const size_t hidden = x.back();
        HIP_PLUGIN_ASSERT(ov::shape_size(in[1].shape) == hidden,
                          "gamma " + shape_str(in[1].shape) + " must hold one value per element of the last axis of " + shape_str(x));
        HIP_OPS_CHECK(hipops_rms_norm(in[0].device, in[1].device, out[0].device, (int64_t)(hidden ? ov::shape_size(x) / hidden : 0),
                                      (int64_t)hidden, eps_, x_dtype_, gamma_dtype_, out_dtype_, context.stream.get()));
    }

private:
    int x_dtype_ = 0, gamma_dtype_ = 0, out_dtype_ = 0;
    float eps_ = 0.f;
};

// ------------------------------------------------------------------------------ RoPE
// Layouts taken: x as [batch, heads, length, size] (input_trans0213 false) or [batch, length, heads,
// size] (true); x as [batch, length, packed] or [tokens, packed] with head_cnt x head_size heads
// starting at slice_start of the last axis.  The result is [batch, heads, length, size], or
// [batch, length, heads, size] with output_trans0213; a rank-2 input gives [tokens, heads * size].
// cos / sin: any shape whose last axis is rotary_ndims (rotate-half) or rotary_ndims / 2 (adjacent
// pairs) wide; the row is the token's index in its sequence, its index in the batch when the table
// has batch x length rows, or the value of the position input.
class RopeOp : public OperationBase {
public:
    RopeOp(const CreationContext& ctx, const ov::Node& node, IndexCollection&& in, IndexCollection&& out)
        : OperationBase(ctx, node, std::move(in), std::move(out)) {
        const std::string who = "RoPE '" + node.get_friendly_name() + "': ";
        auto rope = ov::as_type<const ov::op::internal::RoPE>(&node);
        HIP_PLUGIN_ASSERT(rope != nullptr, "not a RoPE node");
        cfg_ = rope->get_config();
        if (cfg_.is_chatglm || cfg_.is_qwen || cfg_.support_2d_rope || cfg_.use_rope_cache)
            HIP_PLUGIN_THROW(who + "the chatglm / qwen / 2d / cached-table variants are not supported");
        num_inputs_ = node.get_input_size();
        if (num_inputs_ < 3 || num_inputs_ > 4) HIP_PLUGIN_THROW(who + std::to_string(num_inputs_) + " inputs (x, cos, sin [, positions] expected)");
        if (cfg_.gather_position_arg_id != 0 && (cfg_.gather_position_arg_id != 3 || num_inputs_ != 4))
            HIP_PLUGIN_THROW(who + "the position input must be input 3");
        has_positions_ = cfg_.gather_position_arg_id == 3;
        if (has_positions_ && node.get_input_element_type(3) != ov::element::i32) HIP_PLUGIN_THROW(who + "positions must be i32");
        if (!float_dtype(node.get_input_element_type(0), dtype_) || !float_dtype(node.get_input_element_type(1), table_dtype_) ||
            node.get_input_element_type(2) != node.get_input_element_type(1))
            HIP_PLUGIN_THROW(who + "f32, f16 or bf16 expected, cos and sin of one type");
        rank_ = node.get_input_partial_shape(0).size();
        if (rank_ < 2 || rank_ > 4) HIP_PLUGIN_THROW(who + "x of rank " + std::to_string(rank_));
        if (rank_ < 4 && (cfg_.head_cnt == 0 || cfg_.head_size == 0)) HIP_PLUGIN_THROW(who + "a packed x needs head_cnt and head_size");
        if (rank_ == 4 && (cfg_.slice_start || cfg_.slice_stop)) HIP_PLUGIN_THROW(who + "a slice of a rank-4 x");
        if (cfg_.slice_stop && cfg_.slice_stop - cfg_.slice_start != cfg_.head_cnt * cfg_.head_size)
            HIP_PLUGIN_THROW(who + "the slice does not hold head_cnt x head_size elements");
    }

    struct Geometry {
        size_t batch, length, heads, size;
        int64_t x_batch_stride, x_token_stride, x_head_stride, x_offset;
        int64_t o_batch_stride, o_token_stride, o_head_stride;
        ov::Shape out_shape;
    };

    Geometry geometry(const ov::Shape& x) const {
        Geometry g{};
        if (rank_ == 4) {
            g.batch = x[0];
            g.heads = cfg_.input_trans0213 ? x[2] : x[1];
            g.length = cfg_.input_trans0213 ? x[1] : x[2];
            g.size = x[3];
            g.x_batch_stride = (int64_t)(g.heads * g.length * g.size);
            g.x_token_stride = cfg_.input_trans0213 ? (int64_t)(g.heads * g.size) : (int64_t)g.size;
            g.x_head_stride = cfg_.input_trans0213 ? (int64_t)g.size : (int64_t)(g.length * g.size);
        } else {
            g.batch = rank_ == 3 ? x[0] : 1;
            g.length = rank_ == 3 ? x[1] : x[0];
            g.heads = cfg_.head_cnt;
            g.size = cfg_.head_size;
            const size_t packed = x.back();
            HIP_PLUGIN_ASSERT(cfg_.slice_start + g.heads * g.size <= packed, "the heads do not fit the last axis of " + shape_str(x));
            g.x_batch_stride = (int64_t)(g.length * packed);
            g.x_token_stride = (int64_t)packed;
            g.x_head_stride = (int64_t)g.size;
            g.x_offset = (int64_t)cfg_.slice_start;
        }
        const bool out_token_major = rank_ == 2 || cfg_.output_trans0213;
        g.o_batch_stride = (int64_t)(g.heads * g.length * g.size);
        g.o_token_stride = out_token_major ? (int64_t)(g.heads * g.size) : (int64_t)g.size;
        g.o_head_stride = out_token_major ? (int64_t)g.size : (int64_t)(g.length * g.size);
        if (rank_ == 2)
            g.out_shape = ov::Shape{g.length, g.heads * g.size};
        else if (out_token_major)
            g.out_shape = ov::Shape{g.batch, g.length, g.heads, g.size};
        else
            g.out_shape = ov::Shape{g.batch, g.heads, g.length, g.size};
        return g;
    }

    std::vector<ov::Shape> InferOutputShapes(const std::vector<TensorView>& in, const InferenceRequestContext&) const override {
        return {geometry(in.at(0).shape).out_shape};
    }

    void Execute(const InferenceRequestContext& context, Inputs in, Outputs out, const Workbuffers&) const override {
        const Geometry g = geometry(in[0].shape);
        if (g.batch * g.length * g.heads * g.size == 0) return;
        const size_t rotary = cfg_.rotary_ndims ? cfg_.rotary_ndims : g.size;
        const size_t width = cfg_.is_interleaved ? rotary / 2 : rotary;
        const ov::Shape& cs = in[1].shape;
        HIP_PLUGIN_ASSERT(!cs.empty() && cs.back() == width && in[2].shape == cs,
                          "cos / sin " + shape_str(cs) + " must be " + std::to_string(width) + " wide");
        const size_t rows = ov::shape_size(cs) / width;
        size_t table_batch_stride = 0;  // rows
        if (!has_positions_) {
            HIP_PLUGIN_ASSERT(rows == g.length || rows == g.batch * g.length,
                              "cos / sin hold " + std::to_string(rows) + " rows for " + std::to_string(g.batch) + " x " +
                                  std::to_string(g.length) + " tokens and there is no position input");
            if (rows == g.batch * g.length && g.batch > 1) table_batch_stride = g.length;
        } else {
            const size_t n = ov::shape_size(in[3].shape);
            HIP_PLUGIN_ASSERT(n == g.length || n == g.batch * g.length, "positions " + shape_str(in[3].shape));
        }
        const size_t pos_batch_stride = has_positions_ && ov::shape_size(in[3].shape) == g.batch * g.length && g.batch > 1 ? g.length : 0;
        const size_t esz = in[0].type.size(), tsz = in[1].type.size();
        for (size_t b = 0; b < g.batch; b++) {
            hipops_rope_desc d{};
            d.dtype = dtype_, d.table_dtype = table_dtype_;
            d.num_tokens = (int64_t)g.length, d.num_heads = (int)g.heads, d.head_size = (int)g.size;
            d.rotary_ndims = (int)rotary, d.interleaved = cfg_.is_interleaved;
            d.x_token_stride = g.x_token_stride, d.x_head_stride = g.x_head_stride;
            d.out_token_stride = g.o_token_stride, d.out_head_stride = g.o_head_stride;
            d.table_rows = (int64_t)(table_batch_stride ? g.length : rows), d.table_row_stride = (int64_t)width;
            const char* x = (const char*)in[0].device + ((int64_t)b * g.x_batch_stride + g.x_offset) * (int64_t)esz;
            const char* cos = (const char*)in[1].device + b * table_batch_stride * width * tsz;
            const char* sin = (const char*)in[2].device + b * table_batch_stride * width * tsz;
            const int32_t* pos = has_positions_ ? (const int32_t*)in[3].device + b * pos_batch_stride : nullptr;
            char* o = (char*)out[0].device + (int64_t)b * g.o_batch_stride * (int64_t)esz;
            HIP_OPS_CHECK(hipops_rope(&d, x, cos, sin, pos, o, context.stream.get()));
        }
    }

private:
    ov::op::internal::RoPE::Config cfg_;
    size_t num_inputs_ = 3, rank_ = 4;
    bool has_positions_ = false;
    int dtype_ = 0, table_dtype_ = 0;
};

// ------------------------------------------------------------------------------ MatMul
class MatMulOp : public OperationBase {
public:
    MatMulOp(const CreationContext& ctx, const ov::Node& node, IndexCollection&& in, IndexCollection&& out)
        : OperationBase(ctx, node, std::move(in), std::move(out)) {
        const std::string who = "MatMul '" + node.get_friendly_name() + "': ";
        auto mm = ov::as_type<const ov::op::v0::MatMul>(&node);
        HIP_PLUGIN_ASSERT(mm != nullptr, "not a MatMul node");
        if (node.get_input_size() != 2) HIP_PLUGIN_THROW(who + "two inputs expected");
        if (node.get_input_element_type(0) != node.get_input_element_type(1)) HIP_PLUGIN_THROW(who + "mixed input precisions");
        if (!float_dtype(node.get_input_element_type(0), ab_dtype_) || !float_dtype(node.get_output_element_type(0), c_dtype_))
            HIP_PLUGIN_THROW(who + "f32, f16 or bf16 expected");
        if (c_dtype_ != ab_dtype_ && c_dtype_ != HIPATTN_F32) HIP_PLUGIN_THROW(who + "the result must be of the operands' type or f32");
        if (node.get_input_partial_shape(0).size() < 2 || node.get_input_partial_shape(1).size() < 2)
            HIP_PLUGIN_THROW(who + "operands of rank 2 or more expected");
        transpose_a_ = mm->get_transpose_a();
        transpose_b_ = mm->get_transpose_b();
    }

    hipops_matmul_desc describe(const std::vector<TensorView>& in, ov::Shape* out_shape) const {
        const ov::Shape &a = in.at(0).shape, &b = in.at(1).shape;
        const size_t ra = a.size(), rb = b.size();
        hipops_matmul_desc d{};
        d.ab_dtype = ab_dtype_, d.c_dtype = c_dtype_;
        d.transpose_a = transpose_a_, d.transpose_b = transpose_b_;
        d.m = (int64_t)(transpose_a_ ? a[ra - 1] : a[ra - 2]);
        d.k = (int64_t)(transpose_a_ ? a[ra - 2] : a[ra - 1]);
        d.n = (int64_t)(transpose_b_ ? b[rb - 2] : b[rb - 1]);
        HIP_PLUGIN_ASSERT((int64_t)(transpose_b_ ? b[rb - 1] : b[rb - 2]) == d.k,
                          "inner extents of " + shape_str(a) + " and " + shape_str(b) + " differ");
        // batches as the reference takes them (matmul.cpp:38-57): the product of the leading axes, an
        // operand without them is shared by every batch entry
        const size_t batch_a = product(a, 0, ra - 2), batch_b = product(b, 0, rb - 2);
        HIP_PLUGIN_ASSERT(batch_a == batch_b || batch_a == 1 || batch_b == 1,
                          "batches of " + shape_str(a) + " and " + shape_str(b) + " neither match nor broadcast as a whole");
        d.batch = (int64_t)std::max(batch_a, batch_b);
        d.batch_stride_a = batch_a > 1 ? d.m * d.k : 0;
        d.batch_stride_b = batch_b > 1 ? d.k * d.n : 0;
        if (out_shape) {
            const ov::Shape& lead = batch_a >= batch_b ? a : b;
            out_shape->assign(lead.begin(), lead.end() - 2);
            out_shape->push_back((size_t)d.m);
            out_shape->push_back((size_t)d.n);
        }
        return d;
    }

    std::vector<ov::Shape> InferOutputShapes(const std::vector<TensorView>& in, const InferenceRequestContext&) const override {
        ov::Shape out;
        describe(in, &out);
        return {out};
    }
    WorkbufferRequest GetWorkBufferRequest(const std::vector<TensorView>& in) const override {
        const hipops_matmul_desc d = describe(in, nullptr);
        WorkbufferRequest r;
        if (d.m * d.n * d.batch == 0) return r;
        size_t bytes = 0;
        HIP_OPS_CHECK(hipops_matmul_workspace_size(&d, &bytes));
        if (bytes) r.mutable_sizes.push_back(bytes);
        return r;
    }
    void Execute(const InferenceRequestContext& context, Inputs in, Outputs out, const Workbuffers& wb) const override {
        const hipops_matmul_desc d = describe(in, nullptr);
        if (d.m * d.n * d.batch == 0) return;  // no tokens in this step
        void* ws = wb.mutable_buffers.empty() ? nullptr : wb.mutable_buffers[0];
        const size_t ws_bytes = wb.mutable_sizes.empty() ? 0 : wb.mutable_sizes[0];
        HIP_OPS_CHECK(hipops_matmul(&d, in[0].device, in[1].device, out[0].device, ws, ws_bytes, context.stream.get()));
    }

private:
    int ab_dtype_ = 0, c_dtype_ = 0;
    bool transpose_a_ = false, transpose_b_ = false;
};

// ------------------------------------------------------------------------------ Gather
class GatherOp : public OperationBase {
public:
    GatherOp(const CreationContext& ctx, const ov::Node& node, IndexCollection&& in, IndexCollection&& out)
        : OperationBase(ctx, node, std::move(in), std::move(out)) {
        const std::string who = "Gather '" + node.get_friendly_name() + "': ";
        auto gather = dynamic_cast<const ov::op::util::GatherBase*>(&node);
        HIP_PLUGIN_ASSERT(gather != nullptr, "not a Gather node");
        if (node.get_input_size() != 3 || node.get_output_size() != 1) HIP_PLUGIN_THROW(who + "data, indices and axis expected");
        const auto& it = node.get_input_element_type(1);
        if (it != ov::element::i32 && it != ov::element::i64) HIP_PLUGIN_THROW(who + "indices of type " + it.get_type_name());
        index_dtype_ = it == ov::element::i64 ? HIPOPS_I64 : HIPATTN_I32;
        element_bytes_ = node.get_input_element_type(0).size();
        if (element_bytes_ == 0) HIP_PLUGIN_THROW(who + "data of type " + node.get_input_element_type(0).get_type_name());
        axis_ = gather->get_axis();
        batch_dims_ = gather->get_batch_dims();
        const int64_t data_rank = (int64_t)node.get_input_partial_shape(0).size();
        const int64_t index_rank = (int64_t)node.get_input_partial_shape(1).size();
        if (batch_dims_ < 0) batch_dims_ += index_rank;
        if (axis_ < 0 || axis_ >= data_rank || batch_dims_ < 0 || batch_dims_ > axis_ || batch_dims_ > index_rank)
            HIP_PLUGIN_THROW(who + "axis " + std::to_string(axis_) + " / batch_dims " + std::to_string(batch_dims_));
    }
    bool InputIsHostOnly(size_t input) const override { return input == 2; }  // the axis was read from its Constant
    std::vector<ov::Shape> InferOutputShapes(const std::vector<TensorView>& in, const InferenceRequestContext&) const override {
        const ov::Shape &d = in.at(0).shape, &i = in.at(1).shape;
        for (int64_t b = 0; b < batch_dims_; b++)
            HIP_PLUGIN_ASSERT(d[b] == i[b], "batch axes of data " + shape_str(d) + " and indices " + shape_str(i) + " differ");
        ov::Shape out(d.begin(), d.begin() + axis_);
        out.insert(out.end(), i.begin() + batch_dims_, i.end());
        out.insert(out.end(), d.begin() + axis_ + 1, d.end());
        return {out};
    }
    void Execute(const InferenceRequestContext& context, Inputs in, Outputs out, const Workbuffers&) const override {
        const ov::Shape &d = in[0].shape, &i = in[1].shape;
        HIP_OPS_CHECK(hipops_gather(in[0].device, in[1].device, out[0].device, (int64_t)product(d, 0, batch_dims_),
                                    (int64_t)product(d, batch_dims_, axis_), (int64_t)d[axis_],
                                    (int64_t)(product(d, axis_ + 1, d.size()) * element_bytes_),
                                    (int64_t)product(i, batch_dims_, i.size()), index_dtype_, context.stream.get()));
    }

private:
    int index_dtype_ = HIPATTN_I32;
    size_t element_bytes_ = 0;
    int64_t axis_ = 0, batch_dims_ = 0;
};

// ------------------------------------------------------------------------------ Concat
class ConcatOp : public OperationBase {
public:
    ConcatOp(const CreationContext& ctx, const ov::Node& node, IndexCollection&& in, IndexCollection&& out)
        : OperationBase(ctx, node, std::move(in), std::move(out)) {
        const std::string who = "Concat '" + node.get_friendly_name() + "': ";
        auto concat = ov::as_type<const ov::op::v0::Concat>(&node);
        HIP_PLUGIN_ASSERT(concat != nullptr, "not a Concat node");
        if (node.get_input_size() == 0 || node.get_output_size() != 1) HIP_PLUGIN_THROW(who + "at least one input expected");
        const auto& type = node.get_input_element_type(0);
        for (size_t i = 1; i < node.get_input_size(); i++)
            if (node.get_input_element_type(i) != type) HIP_PLUGIN_THROW(who + "mixed input precisions");
        element_bytes_ = type.size();
        if (element_bytes_ == 0) HIP_PLUGIN_THROW(who + "inputs of type " + type.get_type_name());
        axis_ = concat->get_axis();
        const int64_t rank = (int64_t)node.get_input_partial_shape(0).size();
        if (axis_ < 0) axis_ += rank;
        if (axis_ < 0 || axis_ >= rank) HIP_PLUGIN_THROW(who + "axis out of range");
    }
    std::vector<ov::Shape> InferOutputShapes(const std::vector<TensorView>& in, const InferenceRequestContext&) const override {
        ov::Shape out = in.at(0).shape;
        size_t total = 0;
        for (const auto& t : in) {
            HIP_PLUGIN_ASSERT(t.shape.size() == out.size(), "ranks differ");
            for (size_t a = 0; a < out.size(); a++)
                HIP_PLUGIN_ASSERT((int64_t)a == axis_ || t.shape[a] == out[a], "input " + shape_str(t.shape) + " does not line up with " + shape_str(out));
            total += t.shape[axis_];
        }
        out[axis_] = total;
        return {out};
    }
    void Execute(const InferenceRequestContext& context, Inputs in, Outputs out, const Workbuffers&) const override {
        const ov::Shape& first = in[0].shape;
        const size_t tail = product(first, axis_ + 1, first.size()) * element_bytes_;
        std::vector<const void*> ptrs;
        std::vector<int64_t> widths;
        for (const auto& t : in) {
            ptrs.push_back(t.device);
            widths.push_back((int64_t)(t.shape[axis_] * tail));
        }
        HIP_OPS_CHECK(hipops_concat(ptrs.data(), widths.data(), (int)ptrs.size(), (int64_t)product(first, 0, axis_), out[0].device,
                                    context.stream.get()));
    }

private:
    size_t element_bytes_ = 0;
    int64_t axis_ = 0;
};

// ------------------------------------------------------------------------------ Swish, GLU
class SwishOp : public OperationBase {
public:
    SwishOp(const CreationContext& ctx, const ov::Node& node, IndexCollection&& in, IndexCollection&& out)
        : OperationBase(ctx, node, std::move(in), std::move(out)) {
        const std::string who = "Swish '" + node.get_friendly_name() + "': ";
        if (node.get_input_size() != 1 && node.get_input_size() != 2) HIP_PLUGIN_THROW(who + "x [, beta] expected");
        if (!float_dtype(node.get_input_element_type(0), dtype_) || node.get_output_element_type(0) != node.get_input_element_type(0))
            HIP_PLUGIN_THROW(who + "f32, f16 or bf16 expected, output like input");
        if (node.get_input_size() == 2) {
            // beta comes from a Constant, as the reference requires (swish.cpp:19-38)
            auto c = ov::as_type_ptr<const ov::op::v0::Constant>(node.get_input_node_shared_ptr(1));
            if (!c || c->get_output_element_type(0) != ov::element::f32 || c->get_byte_size() != 4)
                HIP_PLUGIN_THROW(who + "beta must be an f32 Constant of one value");
            std::memcpy(&beta_, c->get_data_ptr(), 4);
        }
    }
    bool InputIsHostOnly(size_t input) const override { return input == 1; }  // beta was read from its Constant
    std::vector<ov::Shape> InferOutputShapes(const std::vector<TensorView>& in, const InferenceRequestContext&) const override {
        return {in.at(0).shape};
    }
    void Execute(const InferenceRequestContext& context, Inputs in, Outputs out, const Workbuffers&) const override {
        HIP_OPS_CHECK(hipops_swish(in[0].device, out[0].device, (int64_t)ov::shape_size(in[0].shape), beta_, dtype_, context.stream.get()));
    }

private:
    int dtype_ = 0;
    float beta_ = 1.0f;
};

// act(one half of the last axis) * the other half
class GluOp : public OperationBase {
public:
    GluOp(const CreationContext& ctx, const ov::Node& node, IndexCollection&& in, IndexCollection&& out)
        : OperationBase(ctx, node, std::move(in), std::move(out)) {
        const std::string who = "GLU '" + node.get_friendly_name() + "': ";
        auto glu = ov::as_type<const ov::op::internal::GLU>(&node);
        HIP_PLUGIN_ASSERT(glu != nullptr, "not a GLU node");
        if (!float_dtype(node.get_input_element_type(0), dtype_) || node.get_output_element_type(0) != node.get_input_element_type(0))
            HIP_PLUGIN_THROW(who + "f32, f16 or bf16 expected, output like input");
        const int64_t rank = (int64_t)node.get_input_partial_shape(0).size();
        int64_t axis = glu->get_axis();
        if (axis < 0) axis += rank;
        if (rank < 1 || axis != rank - 1) HIP_PLUGIN_THROW(who + "the split must be along the last axis");
        width_ = glu->get_split_lengths();
        if (width_ <= 0) HIP_PLUGIN_THROW(who + "split_lengths " + std::to_string(width_));
        switch (glu->get_glu_type()) {
            case ov::op::internal::GLU::GluType::Swish: activation_ = HIPOPS_GLU_SWISH; break;
            case ov::op::internal::GLU::GluType::Gelu: activation_ = HIPOPS_GLU_GELU; break;
            case ov::op::internal::GLU::GluType::Gelu_Tanh: activation_ = HIPOPS_GLU_GELU_TANH; break;
            default: HIP_PLUGIN_THROW(who + "unknown activation");
        }
        if (glu->get_split_to_glu_idx() > 1) HIP_PLUGIN_THROW(who + "split_to_glu_idx must be 0 or 1");
        gate_first_ = glu->get_split_to_glu_idx() == 0;
    }
    std::vector<ov::Shape> InferOutputShapes(const std::vector<TensorView>& in, const InferenceRequestContext&) const override {
        ov::Shape out = in.at(0).shape;
        HIP_PLUGIN_ASSERT(!out.empty() && out.back() == (size_t)(2 * width_),
                          "GLU of " + shape_str(out) + " with halves of " + std::to_string(width_));
        out.back() = (size_t)width_;
        return {out};
    }
    void Execute(const InferenceRequestContext& context, Inputs in, Outputs out, const Workbuffers&) const override {
        const int64_t rows = (int64_t)(ov::shape_size(in[0].shape) / (size_t)(2 * width_));
        HIP_OPS_CHECK(hipops_glu(in[0].device, out[0].device, rows, width_, activation_, gate_first_, dtype_, context.stream.get()));
    }

private:
    int dtype_ = 0, activation_ = 0;
    int64_t width_ = 0;
    bool gate_first_ = true;
};

}  // namespace

}  // namespace hip_gpu
}  // namespace ov

using ov::hip_gpu::ConcatOp;
using ov::hip_gpu::GatherOp;
using ov::hip_gpu::GluOp;
using ov::hip_gpu::SwishOp;
using ov::hip_gpu::MatMulOp;
using ov::hip_gpu::RmsOp;
using ov::hip_gpu::RopeOp;
HIP_OPERATION_REGISTER(RmsOp, RMS)
HIP_OPERATION_REGISTER(RopeOp, RoPE)
HIP_OPERATION_REGISTER(MatMulOp, MatMul)
HIP_OPERATION_REGISTER(GatherOp, Gather)
HIP_OPERATION_REGISTER(ConcatOp, Concat)
HIP_OPERATION_REGISTER(SwishOp, Swish)
HIP_OPERATION_REGISTER(GluOp, GLU)
