// Operators of the "HIP" plugin: Parameter / Result / Constant, the two attention operators, and
// the stateful pair ReadValue / Assign;
// each a thin adapter from node + runtime shapes to calls of the C ABI.
//
// SdpaOp stands where the reference lets ScaledDotProductAttentionDecomposition run
// (modules/nvidia_plugin/src/transformer/cuda_graph_transformer.cpp:151-156) and then executes
// MatMulOp / SoftmaxOp / Select / Add / Multiply (src/ops/matmul.cpp:22-75, 185-227,
// src/ops/softmax.cpp:75-147, src/ops/select.cpp:50-91, src/ops/add.cpp:17-43,
// src/ops/multiply.cpp:43); PagedAttentionOp has no counterpart there; ReadValueOp / AssignOp follow
// src/ops/read_value.cpp:31-72 and src/ops/assign.cpp:29-56.  As in the reference, a constructor
// that throws is how an unsupported node is reported (src/cuda_plugin.cpp:171-188).
#include <algorithm>
#include <cmath>
#include <cstring>

#include "hip_operation.hpp"
#include "hip_plugin.hpp"
#include "openvino/op/assign.hpp"
#include "openvino/op/constant.hpp"
#include "openvino/op/paged_attention.hpp"
#include "openvino/op/read_value.hpp"
#include "openvino/op/scaled_dot_product_attention.hpp"
#include "openvino/op/util/variable_extension.hpp"

namespace ov {
namespace hip_gpu {

namespace {

std::string shape_str(const ov::Shape& s) {
    std::string r = "[";
    for (size_t i = 0; i < s.size(); i++) r += (i ? "," : "") + std::to_string(s[i]);
    return r + "]";
}

bool to_hipattn_dtype(const ov::element::Type& t, hipattn_dtype& out) {
    if (t == ov::element::f32) return out = HIPATTN_F32, true;
    if (t == ov::element::f16) return out = HIPATTN_F16, true;
    if (t == ov::element::bf16) return out = HIPATTN_BF16, true;
    if (t == ov::element::u8) return out = HIPATTN_U8, true;
    return false;
}

bool is_float(const ov::element::Type& t) { return t == ov::element::f32 || t == ov::element::f16 || t == ov::element::bf16; }

// a partial shape that can only ever hold zero elements
bool statically_empty(const ov::PartialShape& ps) {
    for (const auto& d : ps)
        if (d.is_static() && d.get_length() == 0) return true;
    return false;
}
// a partial shape that certainly holds at least one element
bool statically_non_empty(const ov::PartialShape& ps) {
    for (const auto& d : ps)
        if (d.is_dynamic() || d.get_length() == 0) return false;
    return true;
}

// Parameter and Result move no data on the device: the infer request binds or uploads inputs
// before the sequence runs and downloads outputs after it (the reference does those copies inside
// ParameterOp / ResultOp, src/ops/parameter.cpp:24-33, src/ops/result.cpp:28-43).
class PassThroughOp : public OperationBase {
public:
    using OperationBase::OperationBase;
    std::vector<ov::Shape> InferOutputShapes(const std::vector<TensorView>& in, const InferenceRequestContext&) const override {
        return in.empty() ? std::vector<ov::Shape>{} : std::vector<ov::Shape>{in[0].shape};
    }
    void Execute(const InferenceRequestContext&, Inputs, Outputs, const Workbuffers&) const override {}
    int InplaceInputOf(size_t) const override { return input_ids_.empty() ? -1 : 0; }
};

// A constant keeps its bytes on the host; the request uploads them and hands operators both views.
class ConstantOp : public OperationBase {
public:
    ConstantOp(const CreationContext& ctx, const ov::Node& node, IndexCollection&& in, IndexCollection&& out)
        : OperationBase(ctx, node, std::move(in), std::move(out)) {
        auto c = ov::as_type<const ov::op::v0::Constant>(&node);
        HIP_PLUGIN_ASSERT(c != nullptr, "not a Constant node");
        shape_ = node.get_output_partial_shape(0).to_shape();
        bytes_.resize(ov::shape_size(shape_) * node.get_output_element_type(0).size());
        if (!bytes_.empty()) std::memcpy(bytes_.data(), c->get_data_ptr(), bytes_.size());
    }
    std::vector<ov::Shape> InferOutputShapes(const std::vector<TensorView>&, const InferenceRequestContext&) const override {
        return {shape_};
    }
    void Execute(const InferenceRequestContext&, Inputs, Outputs, const Workbuffers&) const override {}
    const void* HostData(size_t) const override { return bytes_.data(); }

private:
    ov::Shape shape_;
    std::vector<uint8_t> bytes_;
};

// v13::ScaledDotProductAttention(query, key, value [, attention_mask [, scale]]), attribute causal
class SdpaOp : public OperationBase {
public:
    SdpaOp(const CreationContext& ctx, const ov::Node& node, IndexCollection&& in, IndexCollection&& out)
        : OperationBase(ctx, node, std::move(in), std::move(out)) {
        const std::string who = "ScaledDotProductAttention '" + node.get_friendly_name() + "': ";
        auto sdpa = ov::as_type<const ov::op::v13::ScaledDotProductAttention>(&node);
        HIP_PLUGIN_ASSERT(sdpa != nullptr, "not a ScaledDotProductAttention node");
        num_inputs_ = node.get_input_size();
        if (num_inputs_ < 3 || num_inputs_ > 5) HIP_PLUGIN_THROW(who + std::to_string(num_inputs_) + " inputs (3 to 5 expected)");
        type_ = node.get_input_element_type(0);
        for (size_t i = 0; i < 3; i++) {
            if (node.get_input_element_type(i) != type_) HIP_PLUGIN_THROW(who + "mixed input precisions");
            const size_t rank = node.get_input_partial_shape(i).size();
            if (rank != 3 && rank != 4) HIP_PLUGIN_THROW(who + "rank " + std::to_string(rank) + " inputs (3 or 4 expected)");
        }
        hipattn_dtype dt;
        if (!to_hipattn_dtype(type_, dt) || dt == HIPATTN_U8)
            HIP_PLUGIN_THROW(who + "precision " + type_.get_type_name() + " (f32, f16 or bf16 expected)");
        causal_ = sdpa->get_causal();
        if (num_inputs_ >= 4) {
            mask_type_ = node.get_input_element_type(3);
            if (!is_float(mask_type_) && mask_type_ != ov::element::boolean && mask_type_ != ov::element::u8)
                HIP_PLUGIN_THROW(who + "attention_mask precision " + mask_type_.get_type_name() +
                                 " (boolean, f32, f16 or bf16 expected)");
            if (node.get_input_partial_shape(3).size() > node.get_input_partial_shape(0).size())
                HIP_PLUGIN_THROW(who + "attention_mask has a higher rank than query");
        }
        if (num_inputs_ == 5) {
            const auto& st = node.get_input_element_type(4);
            if (!is_float(st)) HIP_PLUGIN_THROW(who + "scale precision " + st.get_type_name());
            const auto& ss = node.get_input_partial_shape(4);
            if (ss.is_static() && ov::shape_size(ss.to_shape()) != 1) HIP_PLUGIN_THROW(who + "scale must hold one value");
            scale_type_ = st;
        }
    }

    bool InputIsHostOnly(size_t input) const override { return input == 4; }  // the scale: a launch parameter
    std::vector<ov::Shape> InferOutputShapes(const std::vector<TensorView>& in, const InferenceRequestContext&) const override {
        return {in.at(0).shape};
    }

    void Execute(const InferenceRequestContext& context, Inputs inputs, Outputs outputs,
                 const Workbuffers&) const override {
        hipattn_sdpa_desc d = describe(inputs);
        hipattn_mask_desc md{};
        const void* mask = nullptr;
        // an empty mask tensor stands for "no mask" (a scale input needs a placeholder in front of it)
        if (num_inputs_ >= 4 && ov::shape_size(inputs[3].shape) > 0) {
            md = describe_mask(inputs, d);
            mask = inputs[3].device;
        }
        HIP_PLUGIN_CHECK(hipattn_sdpa_masked(&d, inputs[0].device, inputs[1].device, inputs[2].device,
                                             mask ? &md : nullptr, mask, outputs[0].device, nullptr, 0,
                                             context.stream.get()));
    }

private:
    // [B,H,L,D], or rank 3 [N,L,D] with N playing both batch and heads
    hipattn_sdpa_desc describe(const std::vector<TensorView>& in) const {
        const ov::Shape &q = in[0].shape, &k = in[1].shape, &v = in[2].shape;
        HIP_PLUGIN_ASSERT(k == v, "key " + shape_str(k) + " and value " + shape_str(v) + " differ");
        HIP_PLUGIN_ASSERT(q.size() == k.size(), "query and key ranks differ");
        const size_t r = q.size();
        hipattn_sdpa_desc d{};
        to_hipattn_dtype(type_, d.dtype);
        d.batch = r == 4 ? (int)q[0] : 1;
        d.num_heads_q = (int)q[r - 3];
        d.num_heads_kv = (int)k[r - 3];
        d.len_q = (int)q[r - 2];
        d.len_kv = (int)k[r - 2];
        d.head_dim = (int)q[r - 1];
        HIP_PLUGIN_ASSERT(k[r - 1] == q[r - 1], "head sizes differ: " + shape_str(q) + " vs " + shape_str(k));
        HIP_PLUGIN_ASSERT(r == 3 || k[0] == q[0], "batch sizes differ: " + shape_str(q) + " vs " + shape_str(k));
        d.causal = causal_;
        d.scale = 0.0f;  // 1/sqrt(head_dim) unless the scale input says otherwise
        if (num_inputs_ == 5 && ov::shape_size(in[4].shape) > 0) {
            HIP_PLUGIN_ASSERT(ov::shape_size(in[4].shape) == 1, "scale must hold one value, got " + shape_str(in[4].shape));
            HIP_PLUGIN_ASSERT(in[4].host != nullptr, "scale must be a constant or be set from host memory (it is a launch parameter)");
            d.scale = read_scalar(in[4].host, scale_type_);
            HIP_PLUGIN_ASSERT(d.scale > 0.0f, "scale must be positive");
        }
        return d;
    }

    static float read_scalar(const void* p, const ov::element::Type& t) {
        if (t == ov::element::f32) {
            float x;
            std::memcpy(&x, p, 4);
            return x;
        }
        uint16_t bits;
        std::memcpy(&bits, p, 2);
        if (t == ov::element::bf16) {
            const uint32_t w = (uint32_t)bits << 16;
            float x;
            std::memcpy(&x, &w, 4);
            return x;
        }
        // f16
        const int sign = bits >> 15, exp = (bits >> 10) & 31, man = bits & 1023;
        float x;
        if (exp == 0)
            x = std::ldexp((float)man, -24);
        else if (exp == 31)
            x = man ? NAN : INFINITY;
        else
            x = std::ldexp((float)(man | 1024), exp - 25);
        return sign ? -x : x;
    }

    // numpy broadcast of the mask's shape, right-aligned, against [batch, heads, len_q, len_kv]
    hipattn_mask_desc describe_mask(const std::vector<TensorView>& in, const hipattn_sdpa_desc& d) const {
        const ov::Shape& m = in[3].shape;
        const int64_t full[4] = {d.batch, d.num_heads_q, d.len_q, d.len_kv};
        hipattn_mask_desc md{};
        if (mask_type_ == ov::element::boolean || mask_type_ == ov::element::u8)
            md.dtype = HIPATTN_U8;
        else
            to_hipattn_dtype(mask_type_, md.dtype);
        HIP_PLUGIN_ASSERT(m.size() <= 4, "attention_mask rank " + std::to_string(m.size()));
        int64_t stride = 1;
        for (int ax = 3; ax >= 0; ax--) {
            const int mi = ax - (4 - (int)m.size());
            const int64_t extent = mi >= 0 ? (int64_t)m[mi] : 1;
            HIP_PLUGIN_ASSERT(extent == 1 || extent == full[ax],
                              "attention_mask " + shape_str(m) + " does not broadcast to the scores");
            md.stride[ax] = (extent == 1) ? 0 : stride;
            stride *= extent;
        }
        return md;
    }

    ov::element::Type type_, mask_type_, scale_type_;
    size_t num_inputs_ = 3;
    bool causal_ = false;
};

// Input order of the OpenVINO operator.  score_aggregation_window belongs to the scores output
// (built: the aggregated probabilities a cache-eviction policy reads); the three rotation inputs to the
// cache rotation (built: hipattn_rotate_key_cache ahead of the attention); sinks, the last one, holds one f32
// logit per query head or nothing (built: the term joins the denominators); the three inputs of sparse
// attention are not implemented: they are accepted when they are empty, as exported models carry them,
// and refused when they hold data.
enum PaInput {
    kQuery = 0, kKey, kValue, kKeyCache, kValueCache, kPastLens, kSubsequenceBegins, kBlockIndices,
    kBlockIndicesBegins, kScale, kSlidingWindow, kAlibiSlopes, kMaxContextLen, kPaRequiredInputs,
    kScoreAggregationWindow = kPaRequiredInputs, kRotatedBlockIndices, kRotationDeltas, kRotationTrigLut,
    kXattentionThreshold, kXattentionBlockSize, kXattentionStride, kSinks
};
const char* const kPaOptionalNames[] = {"score_aggregation_window", "rotated_block_indices", "rotation_deltas",
                                        "rotation_trig_lut",        "xattention_threshold",  "xattention_block_size",
                                        "xattention_stride",        "sinks"};

class PagedAttentionOp : public OperationBase {
public:
    PagedAttentionOp(const CreationContext& ctx, const ov::Node& node, IndexCollection&& in, IndexCollection&& out)
        : OperationBase(ctx, node, std::move(in), std::move(out)) {
        const std::string who = "PagedAttentionExtension '" + node.get_friendly_name() + "': ";
        num_inputs_ = node.get_input_size();
        num_outputs_ = node.get_output_size();
        if (num_inputs_ < kPaRequiredInputs)
            HIP_PLUGIN_THROW(who + std::to_string(num_inputs_) + " inputs, at least 13 expected");
        if (num_inputs_ > kPaRequiredInputs + sizeof(kPaOptionalNames) / sizeof(kPaOptionalNames[0]))
            HIP_PLUGIN_THROW(who + std::to_string(num_inputs_) + " inputs: more than this plugin knows of");
        if (num_outputs_ < 1 || num_outputs_ > 2) HIP_PLUGIN_THROW(who + std::to_string(num_outputs_) + " outputs");
        for (size_t i = kRotationTrigLut + 1; i < num_inputs_; i++)
            if (i != kSinks && statically_non_empty(node.get_input_partial_shape(i)))
                HIP_PLUGIN_THROW(who + kPaOptionalNames[i - kPaRequiredInputs] + " holds data: the feature is not supported");
        if (num_inputs_ > kSinks && node.get_input_element_type(kSinks) != ov::element::f32 && !statically_empty(node.get_input_partial_shape(kSinks)))
            HIP_PLUGIN_THROW(who + "sinks must be f32");
        if (num_inputs_ > kRotationTrigLut) {
            for (int i : {kRotatedBlockIndices, kRotationDeltas})
                if (node.get_input_element_type(i) != ov::element::i32 && !statically_empty(node.get_input_partial_shape(i)))
                    HIP_PLUGIN_THROW(who + kPaOptionalNames[i - kPaRequiredInputs] + " must be i32");
            lut_type_ = node.get_input_element_type(kRotationTrigLut);
            if (!is_float(lut_type_) && !statically_empty(node.get_input_partial_shape(kRotationTrigLut)))
                HIP_PLUGIN_THROW(who + "rotation_trig_lut must be f32, f16 or bf16");
        } else if (num_inputs_ > kRotatedBlockIndices) {
            for (size_t i = kRotatedBlockIndices; i < num_inputs_; i++)
                if (statically_non_empty(node.get_input_partial_shape(i)))
                    HIP_PLUGIN_THROW(who + "cache rotation needs rotated_block_indices, rotation_deltas and rotation_trig_lut together");
        }
        if (num_inputs_ > kScoreAggregationWindow && node.get_input_element_type(kScoreAggregationWindow) != ov::element::i32)
            HIP_PLUGIN_THROW(who + "score_aggregation_window must be i32");
        q_type_ = node.get_input_element_type(kQuery);
        kv_type_ = node.get_input_element_type(kKey);
        cache_type_ = node.get_input_element_type(kKeyCache);
        if (node.get_input_element_type(kValue) != kv_type_ || node.get_input_element_type(kValueCache) != cache_type_)
            HIP_PLUGIN_THROW(who + "key/value precisions differ");
        if (!is_float(q_type_) || !is_float(kv_type_)) HIP_PLUGIN_THROW(who + "query/key/value must be f32, f16 or bf16");
        if (!is_float(cache_type_) && cache_type_ != ov::element::u8)
            HIP_PLUGIN_THROW(who + "cache precision " + cache_type_.get_type_name() + " (f32, f16, bf16 or u8 expected)");
        for (int i : {kPastLens, kSubsequenceBegins, kBlockIndices, kBlockIndicesBegins})
            if (node.get_input_element_type(i) != ov::element::i32) HIP_PLUGIN_THROW(who + "index inputs must be i32");
        if (node.get_input_partial_shape(kKeyCache).size() != 4)
            HIP_PLUGIN_THROW(who + "key_cache must be [num_blocks, num_kv_heads, block_size, head_size]");
        // alibi_slopes: empty, or one f32 slope per query head (checked against the head count at run time)
        if (node.get_input_element_type(kAlibiSlopes) != ov::element::f32 && !statically_empty(node.get_input_partial_shape(kAlibiSlopes)))
            HIP_PLUGIN_THROW(who + "alibi_slopes must be f32");
        if (node.get_input_partial_shape(kAlibiSlopes).rank().is_static() && node.get_input_partial_shape(kAlibiSlopes).size() != 1)
            HIP_PLUGIN_THROW(who + "alibi_slopes must be a vector ([0] or [query heads])");
        out1_type_ = num_outputs_ > 1 ? node.get_output_element_type(1) : ov::element::dynamic;
    }

    void MarkOutputUnused(size_t output) override {
        if (output == 1) scores_wanted_ = false;
    }

    // scores: one value per cache position of every sequence, past and new; the output's extent is
    // data (the sum of past_lens), so those must have come from host memory
    std::vector<ov::Shape> InferOutputShapes(const std::vector<TensorView>& in, const InferenceRequestContext&) const override {
        std::vector<ov::Shape> shapes{in.at(kQuery).shape};
        if (num_outputs_ > 1) {
            size_t total = 0;
            if (scores_wanted_ && in[kQuery].shape.at(0) > 0) {
                const TensorView& pl = in[kPastLens];
                HIP_PLUGIN_ASSERT(pl.host != nullptr, "past_lens must be set from host memory when the scores output is used (it sizes that output)");
                HIP_PLUGIN_ASSERT(out1_type_ == ov::element::f32, "the scores output must be f32, not " + out1_type_.get_type_name());
                const int32_t* lens = (const int32_t*)pl.host;
                for (size_t s = 0; s < ov::shape_size(pl.shape); s++) total += (size_t)std::max(lens[s], 0);
                total += in[kQuery].shape[0];
            }
            shapes.push_back(ov::Shape{total});
        }
        return shapes;
    }

    std::vector<size_t> UpdatedInputs() const override { return {kKeyCache, kValueCache}; }
    // launch parameters, and inputs that must be empty: none of them is handed to a kernel
    bool InputIsHostOnly(size_t input) const override {
        return input == kScale || input == kSlidingWindow || input == kMaxContextLen || (input > kRotationTrigLut && input != kSinks);
    }

    // max_context_len is advisory for the attention kernels; only the scores kernels size a grid by it
    bool InputValueShapesLaunch(size_t input) const override {
        return input != kMaxContextLen || (scores_wanted_ && num_outputs_ > 1);
    }

    WorkbufferRequest GetWorkBufferRequest(const std::vector<TensorView>& inputs) const override {
        const hipattn_pa_desc d = describe(inputs);
        size_t bytes = 0;
        HIP_PLUGIN_CHECK(hipattn_paged_attention_workspace_size(&d, &bytes));
        WorkbufferRequest r;
        r.mutable_sizes.push_back(bytes);
        if (scores_wanted_ && num_outputs_ > 1) {
            HIP_PLUGIN_CHECK(hipattn_paged_attention_scores_workspace_size(&d, &bytes));
            r.mutable_sizes.push_back(bytes);
        }
        return r;
    }

    void Execute(const InferenceRequestContext& context, Inputs in, Outputs out, const Workbuffers& wb) const override {
        const hipattn_pa_desc d = describe(in);
        void* ws = wb.mutable_buffers.empty() ? nullptr : wb.mutable_buffers[0];
        const size_t ws_bytes = wb.mutable_sizes.empty() ? 0 : wb.mutable_sizes[0];
        // cache rotation first: the listed key blocks are turned before this step's keys are stored
        if (num_inputs_ > kRotationTrigLut && ov::shape_size(in[kRotatedBlockIndices].shape) > 0) {
            const size_t blocks = ov::shape_size(in[kRotatedBlockIndices].shape);
            const ov::Shape& deltas = in[kRotationDeltas].shape;
            const ov::Shape& lut = in[kRotationTrigLut].shape;
            HIP_PLUGIN_ASSERT(ov::shape_size(deltas) == blocks || ov::shape_size(deltas) == blocks * (size_t)d.block_size,
                              "rotation_deltas must be [rotated blocks, 1] or [rotated blocks, block_size], got " + shape_str(deltas));
            HIP_PLUGIN_ASSERT(ov::shape_size(lut) > 0 && ov::shape_size(lut) % (size_t)d.head_dim == 0,
                              "rotation_trig_lut must be [positions, head_size], got " + shape_str(lut));
            hipattn_dtype lut_dtype = HIPATTN_F32;
            to_hipattn_dtype(lut_type_, lut_dtype);
            HIP_PLUGIN_CHECK(hipattn_rotate_key_cache(&d, in[kKeyCache].device, (const int32_t*)in[kRotatedBlockIndices].device, (int)blocks,
                                                      (const int32_t*)in[kRotationDeltas].device, (int)(ov::shape_size(deltas) / blocks),
                                                      in[kRotationTrigLut].device, lut_dtype, (int)(ov::shape_size(lut) / (size_t)d.head_dim),
                                                      context.stream.get()));
        }
        HIP_PLUGIN_CHECK(hipattn_paged_attention(
            &d, in[kQuery].device, in[kKey].device, in[kValue].device, in[kKeyCache].device, in[kValueCache].device,
            (const int32_t*)in[kPastLens].device, (const int32_t*)in[kSubsequenceBegins].device,
            (const int32_t*)in[kBlockIndices].device, (const int32_t*)in[kBlockIndicesBegins].device, out[0].device, ws,
            ws_bytes, context.stream.get()));
        if (scores_wanted_ && out.size() > 1 && ov::shape_size(out[1].shape) > 0) {
            const int32_t* window = nullptr;
            if (num_inputs_ > kScoreAggregationWindow && ov::shape_size(in[kScoreAggregationWindow].shape) > 0) {
                HIP_PLUGIN_ASSERT(ov::shape_size(in[kScoreAggregationWindow].shape) == (size_t)d.num_seqs,
                                  "score_aggregation_window must hold one value per sequence");
                window = (const int32_t*)in[kScoreAggregationWindow].device;
            }
            HIP_PLUGIN_ASSERT(wb.mutable_buffers.size() > 1, "no scratch for the scores");
            HIP_PLUGIN_CHECK(hipattn_paged_attention_scores(
                &d, in[kQuery].device, in[kKeyCache].device, (const int32_t*)in[kPastLens].device,
                (const int32_t*)in[kSubsequenceBegins].device, (const int32_t*)in[kBlockIndices].device,
                (const int32_t*)in[kBlockIndicesBegins].device, window, (float*)out[1].device,
                (int64_t)ov::shape_size(out[1].shape), wb.mutable_buffers[1], wb.mutable_sizes[1], context.stream.get()));
        }
    }

private:
    template <typename T>
    static T host_scalar(const TensorView& t, const char* what, T dflt, bool required) {
        if (ov::shape_size(t.shape) == 0) {
            HIP_PLUGIN_ASSERT(!required, std::string(what) + " is empty");
            return dflt;
        }
        HIP_PLUGIN_ASSERT(t.host != nullptr, std::string(what) + " must be set from host memory (it sizes the launch)");
        T v;
        std::memcpy(&v, t.host, sizeof(T));
        return v;
    }

    hipattn_pa_desc describe(const std::vector<TensorView>& in) const {
        const ov::Shape& q = in[kQuery].shape;
        const ov::Shape& kc = in[kKeyCache].shape;
        HIP_PLUGIN_ASSERT(q.size() == 2, "query must be [tokens, heads * head_size], got " + shape_str(q));
        HIP_PLUGIN_ASSERT(kc.size() == 4 && in[kValueCache].shape == kc, "key/value cache shapes " + shape_str(kc));
        for (size_t i = kRotationTrigLut + 1; i < num_inputs_; i++)
            HIP_PLUGIN_ASSERT(i == kSinks || ov::shape_size(in[i].shape) == 0,
                              std::string(kPaOptionalNames[i - kPaRequiredInputs]) + " holds data: the feature is not supported");
        if (num_inputs_ > kRotatedBlockIndices && num_inputs_ <= kRotationTrigLut)
            for (size_t i = kRotatedBlockIndices; i < num_inputs_; i++)
                HIP_PLUGIN_ASSERT(ov::shape_size(in[i].shape) == 0, "cache rotation needs rotated_block_indices, rotation_deltas and rotation_trig_lut together");
        hipattn_pa_desc d{};
        to_hipattn_dtype(q_type_, d.q_dtype);
        to_hipattn_dtype(kv_type_, d.kv_dtype);
        to_hipattn_dtype(cache_type_, d.cache_dtype);
        d.out_dtype = d.q_dtype;
        d.num_blocks = (int)kc[0];
        d.num_heads_kv = (int)kc[1];
        d.block_size = (int)kc[2];
        // a u8 cache row carries its scale and zero-point in front of the payload
        d.head_dim = (int)kc[3] - (cache_type_ == ov::element::u8 ? 8 : 0);
        HIP_PLUGIN_ASSERT(d.head_dim > 0 && q[1] % d.head_dim == 0, "query width " + std::to_string(q[1]) +
                                                                        " is not a multiple of head size " +
                                                                        std::to_string(d.head_dim));
        d.num_heads_q = (int)(q[1] / d.head_dim);
        d.num_tokens = (int)q[0];
        HIP_PLUGIN_ASSERT(in[kKey].shape.size() == 2 && in[kKey].shape[0] == q[0] &&
                              in[kKey].shape[1] == (size_t)d.num_heads_kv * d.head_dim && in[kValue].shape == in[kKey].shape,
                          "key/value must be [tokens, kv_heads * head_size], got " + shape_str(in[kKey].shape));
        d.num_seqs = (int)in[kPastLens].shape.at(0);
        HIP_PLUGIN_ASSERT(in[kSubsequenceBegins].shape.at(0) == (size_t)d.num_seqs + 1 &&
                              in[kBlockIndicesBegins].shape.at(0) == (size_t)d.num_seqs + 1,
                          "subsequence_begins / block_indices_begins must have num_sequences + 1 entries");
        d.scale = host_scalar<float>(in[kScale], "scale", 0.0f, false);
        d.sliding_window = host_scalar<int32_t>(in[kSlidingWindow], "sliding_window", 0, false);
        d.max_context_len = host_scalar<int32_t>(in[kMaxContextLen], "max_context_len", 0, false);
        d.flags = 0;  // any split of the tokens over the sequences comes out right without a hint
        d.decode_waves = 0;
        if (ov::shape_size(in[kAlibiSlopes].shape) > 0) {
            HIP_PLUGIN_ASSERT(ov::shape_size(in[kAlibiSlopes].shape) == (size_t)d.num_heads_q,
                              "alibi_slopes must hold one value per query head (" + std::to_string(d.num_heads_q) + "), got " +
                                  shape_str(in[kAlibiSlopes].shape));
            d.alibi_slopes = (const float*)in[kAlibiSlopes].device;
        }
        if (num_inputs_ > kSinks && ov::shape_size(in[kSinks].shape) > 0) {
            HIP_PLUGIN_ASSERT(ov::shape_size(in[kSinks].shape) == (size_t)d.num_heads_q,
                              "sinks must hold one value per query head (" + std::to_string(d.num_heads_q) + "), got " + shape_str(in[kSinks].shape));
            d.sinks = (const float*)in[kSinks].device;
        }
        return d;
    }
    ov::element::Type q_type_, kv_type_, cache_type_, out1_type_, lut_type_ = ov::element::f32;
    size_t num_inputs_ = 0, num_outputs_ = 1;
    bool scores_wanted_ = true;  // until the compiled model says nothing consumes output 1
};

// ReadValue: the variable's device buffer into the output; after a reset, the init_value input (or
// zeros) instead.  The output takes the state's current shape; right after a reset that is the
// init_value's shape, or the variable's shape with dynamic extents at 0.
class ReadValueOp : public OperationBase {
public:
    ReadValueOp(const CreationContext& ctx, const ov::Node& node, IndexCollection&& in, IndexCollection&& out)
        : OperationBase(ctx, node, std::move(in), std::move(out)) {
        auto ext = dynamic_cast<const ov::op::util::VariableExtension*>(&node);
        HIP_PLUGIN_ASSERT(ext != nullptr, "ReadValue without a variable");
        variable_id_ = ext->get_variable_id();
        has_init_ = node.get_input_size() > 0;
    }
    std::vector<ov::Shape> InferOutputShapes(const std::vector<TensorView>& in, const InferenceRequestContext& context) const override {
        auto state = context.variables->get(variable_id_);
        if (state->is_reset_state() && has_init_) return {in.at(0).shape};
        return {state->shape()};
    }
    void Execute(const InferenceRequestContext& context, Inputs in, Outputs out, const Workbuffers&) const override {
        HIP_PLUGIN_ASSERT(context.variables != nullptr, "ReadValue requires a variable context");
        auto state = context.variables->get(variable_id_);
        const size_t bytes = out[0].byte_size();
        if (bytes == 0) return;  // an empty state (the initial KV cache): nothing to copy, nothing to read
        if (state->is_reset_state()) {
            if (has_init_)
                context.stream.transfer(out[0].device, in[0].device, std::min(bytes, in[0].byte_size()));
            else
                context.stream.fill(out[0].device, 0, bytes);
        } else {
            state->read_device_state(context.stream, out[0].device, bytes);
        }
    }

private:
    std::string variable_id_;
    bool has_init_ = false;
};

// Assign: the input becomes the variable's new contents (device to device, grow-only capacity).
class AssignOp : public OperationBase {
public:
    AssignOp(const CreationContext& ctx, const ov::Node& node, IndexCollection&& in, IndexCollection&& out)
        : OperationBase(ctx, node, std::move(in), std::move(out)) {
        auto ext = dynamic_cast<const ov::op::util::VariableExtension*>(&node);
        HIP_PLUGIN_ASSERT(ext != nullptr, "Assign without a variable");
        variable_id_ = ext->get_variable_id();
    }
    std::vector<ov::Shape> InferOutputShapes(const std::vector<TensorView>& in, const InferenceRequestContext&) const override {
        return {in.at(0).shape};
    }
    void Execute(const InferenceRequestContext& context, Inputs in, Outputs, const Workbuffers&) const override {
        HIP_PLUGIN_ASSERT(context.variables != nullptr, "Assign requires a variable context");
        context.variables->get(variable_id_)->update_device_state(context.stream, in[0].device, in[0].shape);
    }
    int InplaceInputOf(size_t) const override { return 0; }

private:
    std::string variable_id_;
};

}  // namespace

}  // namespace hip_gpu
}  // namespace ov

using ov::hip_gpu::AssignOp;
using ov::hip_gpu::ConstantOp;
using ov::hip_gpu::PagedAttentionOp;
using ov::hip_gpu::PassThroughOp;
using ov::hip_gpu::ReadValueOp;
using ov::hip_gpu::SdpaOp;
HIP_OPERATION_REGISTER(PassThroughOp, Parameter)
HIP_OPERATION_REGISTER(PassThroughOp, Result)
HIP_OPERATION_REGISTER(ConstantOp, Constant)
HIP_OPERATION_REGISTER(SdpaOp, ScaledDotProductAttention)
HIP_OPERATION_REGISTER(PagedAttentionOp, PagedAttentionExtension)
HIP_OPERATION_REGISTER(ReadValueOp, ReadValue)
HIP_OPERATION_REGISTER(AssignOp, Assign)
