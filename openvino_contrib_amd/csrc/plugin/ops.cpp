// Operators of the "HIP" plugin: Parameter / Result / Constant pass-throughs and the two attention
// operators, each a thin adapter from node + runtime shapes to one C-ABI call.
//
// SdpaOp stands where the reference lets ScaledDotProductAttentionDecomposition run
// (modules/nvidia_plugin/src/transformer/cuda_graph_transformer.cpp:151-156) and then executes
// MatMulOp / SoftmaxOp / Select / Add / Multiply (src/ops/matmul.cpp:22-75, 185-227,
// src/ops/softmax.cpp:75-147); PagedAttentionOp has no counterpart there.  As in the reference,
// a constructor that throws is how an unsupported node is reported (src/cuda_plugin.cpp:171-188).
#include <cmath>
#include <cstring>

#include "operation.hpp"

namespace hip_plugin {

namespace {

std::string shape_str(const Shape& s) {
    std::string r = "[";
    for (size_t i = 0; i < s.size(); i++) r += (i ? "," : "") + std::to_string(s[i]);
    return r + "]";
}

// Parameter, Result and Constant move no data on the device: the infer request uploads inputs
// before the sequence runs and downloads outputs after it (the reference does those copies inside
// ParameterOp / ResultOp, src/ops/parameter.cpp:24-33, src/ops/result.cpp:28-43).
class PassThroughOp : public OperationBase {
public:
    using OperationBase::OperationBase;
    std::vector<Shape> InferOutputShapes(const std::vector<Shape>& in) const override {
        return in.empty() ? std::vector<Shape>{} : std::vector<Shape>{in[0]};
    }
    void Execute(const InferenceRequestContext&, Inputs, Outputs, const Workbuffers&) const override {}
    int InplaceInputOf(size_t) const override { return input_ids_.empty() ? -1 : 0; }
};

class SdpaOp : public OperationBase {
public:
    SdpaOp(const CreationContext& ctx, const Node& node, IndexCollection&& in, IndexCollection&& out)
        : OperationBase(ctx, node, std::move(in), std::move(out)) {
        if (node.inputs.size() != 3)
            HIP_PLUGIN_THROW("ScaledDotProductAttention '" + node.friendly_name +
                             "': attention_mask / scale inputs are not supported, expected (query, key, value)");
        type_ = node.get_input_element_type(0);
        for (size_t i = 0; i < 3; i++) {
            if (node.get_input_element_type(i) != type_)
                HIP_PLUGIN_THROW("ScaledDotProductAttention '" + node.friendly_name + "': mixed input precisions");
            const size_t rank = node.get_input_partial_shape(i).size();
            if (rank != 3 && rank != 4)
                HIP_PLUGIN_THROW("ScaledDotProductAttention '" + node.friendly_name + "': rank " +
                                 std::to_string(rank) + " inputs (3 or 4 expected)");
        }
        hipattn_dtype dt;
        if (!to_hipattn_dtype(type_, dt) || dt == HIPATTN_U8)
            HIP_PLUGIN_THROW("ScaledDotProductAttention '" + node.friendly_name + "': precision " +
                             element_name(type_) + " (f32, f16 or bf16 expected)");
        causal_ = node.get_bool("causal", false);
    }

    std::vector<Shape> InferOutputShapes(const std::vector<Shape>& in) const override { return {in.at(0)}; }

    void Execute(const InferenceRequestContext& context, Inputs inputs, Outputs outputs,
                 const Workbuffers&) const override {
        const hipattn_sdpa_desc d = describe(inputs);
        HIP_PLUGIN_CHECK(hipattn_sdpa(&d, inputs[0].device, inputs[1].device, inputs[2].device, outputs[0].device,
                                      nullptr, 0, context.stream.get()));
    }

private:
    // [B,H,L,D], or rank 3 [N,L,D] with N playing both batch and heads
    hipattn_sdpa_desc describe(const std::vector<TensorView>& in) const {
        const Shape &q = in[0].shape, &k = in[1].shape, &v = in[2].shape;
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
        d.scale = 0.0f;  // default 1/sqrt(head_dim); the scale input is rejected at construction
        return d;
    }
    ElementType type_;
    bool causal_ = false;
};

// Input order of the OpenVINO operator.
enum PaInput {
    kQuery = 0, kKey, kValue, kKeyCache, kValueCache, kPastLens, kSubsequenceBegins, kBlockIndices,
    kBlockIndicesBegins, kScale, kSlidingWindow, kAlibiSlopes, kMaxContextLen, kPaInputs
};

class PagedAttentionOp : public OperationBase {
public:
    PagedAttentionOp(const CreationContext& ctx, const Node& node, IndexCollection&& in, IndexCollection&& out)
        : OperationBase(ctx, node, std::move(in), std::move(out)) {
        const std::string who = "PagedAttentionExtension '" + node.friendly_name + "': ";
        if (node.inputs.size() < kPaInputs)
            HIP_PLUGIN_THROW(who + std::to_string(node.inputs.size()) + " inputs, at least 13 expected");
        if (node.inputs.size() > kPaInputs)
            HIP_PLUGIN_THROW(who + "score aggregation / cache rotation inputs are not supported");
        q_type_ = node.get_input_element_type(kQuery);
        kv_type_ = node.get_input_element_type(kKey);
        cache_type_ = node.get_input_element_type(kKeyCache);
        if (node.get_input_element_type(kValue) != kv_type_ || node.get_input_element_type(kValueCache) != cache_type_)
            HIP_PLUGIN_THROW(who + "key/value precisions differ");
        auto is_float = [](ElementType t) { return t == ElementType::f32 || t == ElementType::f16 || t == ElementType::bf16; };
        if (!is_float(q_type_) || !is_float(kv_type_)) HIP_PLUGIN_THROW(who + "query/key/value must be f32, f16 or bf16");
        if (!is_float(cache_type_) && cache_type_ != ElementType::u8)
            HIP_PLUGIN_THROW(who + "cache precision " + element_name(cache_type_) + " (f32, f16, bf16 or u8 expected)");
        for (int i : {kPastLens, kSubsequenceBegins, kBlockIndices, kBlockIndicesBegins})
            if (node.get_input_element_type(i) != ElementType::i32) HIP_PLUGIN_THROW(who + "index inputs must be i32");
        if (node.get_input_partial_shape(kKeyCache).size() != 4)
            HIP_PLUGIN_THROW(who + "key_cache must be [num_blocks, num_kv_heads, block_size, head_size]");
        const PartialShape& alibi = node.get_input_partial_shape(kAlibiSlopes);
        if (!(alibi.size() == 1 && alibi[0] == 0)) HIP_PLUGIN_THROW(who + "alibi_slopes are not supported (expected shape [0])");
    }

    std::vector<Shape> InferOutputShapes(const std::vector<Shape>& in) const override { return {in.at(kQuery)}; }

    WorkbufferRequest GetWorkBufferRequest(const std::vector<TensorView>& inputs) const override {
        const hipattn_pa_desc d = describe(inputs);
        size_t bytes = 0;
        HIP_PLUGIN_CHECK(hipattn_paged_attention_workspace_size(&d, &bytes));
        WorkbufferRequest r;
        if (bytes) r.mutable_sizes.push_back(bytes);
        return r;
    }

    void Execute(const InferenceRequestContext& context, Inputs in, Outputs out, const Workbuffers& wb) const override {
        const hipattn_pa_desc d = describe(in);
        void* ws = wb.mutable_buffers.empty() ? nullptr : wb.mutable_buffers[0];
        const size_t ws_bytes = wb.mutable_sizes.empty() ? 0 : wb.mutable_sizes[0];
        HIP_PLUGIN_CHECK(hipattn_paged_attention(
            &d, in[kQuery].device, in[kKey].device, in[kValue].device, in[kKeyCache].device, in[kValueCache].device,
            (const int32_t*)in[kPastLens].device, (const int32_t*)in[kSubsequenceBegins].device,
            (const int32_t*)in[kBlockIndices].device, (const int32_t*)in[kBlockIndicesBegins].device, out[0].device, ws,
            ws_bytes, context.stream.get()));
    }

private:
    template <typename T>
    static T host_scalar(const TensorView& t, const char* what, T dflt, bool required) {
        if (shape_size(t.shape) == 0) {
            HIP_PLUGIN_ASSERT(!required, std::string(what) + " is empty");
            return dflt;
        }
        HIP_PLUGIN_ASSERT(t.host != nullptr, std::string(what) + " must be set from host memory (it sizes the launch)");
        T v;
        std::memcpy(&v, t.host, sizeof(T));
        return v;
    }

    hipattn_pa_desc describe(const std::vector<TensorView>& in) const {
        const Shape& q = in[kQuery].shape;
        const Shape& kc = in[kKeyCache].shape;
        HIP_PLUGIN_ASSERT(q.size() == 2, "query must be [tokens, heads * head_size], got " + shape_str(q));
        HIP_PLUGIN_ASSERT(kc.size() == 4 && in[kValueCache].shape == kc, "key/value cache shapes " + shape_str(kc));
        hipattn_pa_desc d{};
        to_hipattn_dtype(q_type_, d.q_dtype);
        to_hipattn_dtype(kv_type_, d.kv_dtype);
        to_hipattn_dtype(cache_type_, d.cache_dtype);
        d.out_dtype = d.q_dtype;
        d.num_blocks = (int)kc[0];
        d.num_heads_kv = (int)kc[1];
        d.block_size = (int)kc[2];
        // a u8 cache row carries its scale and zero-point in front of the payload
        d.head_dim = (int)kc[3] - (cache_type_ == ElementType::u8 ? 8 : 0);
        HIP_PLUGIN_ASSERT(d.head_dim > 0 && q[1] % d.head_dim == 0, "query width " + std::to_string(q[1]) +
                                                                        " is not a multiple of head size " +
                                                                        std::to_string(d.head_dim));
        d.num_heads_q = (int)(q[1] / d.head_dim);
        d.num_tokens = (int)q[0];
        HIP_PLUGIN_ASSERT(in[kKey].shape.size() == 2 && in[kKey].shape[0] == q[0] &&
                              in[kKey].shape[1] == (int64_t)d.num_heads_kv * d.head_dim && in[kValue].shape == in[kKey].shape,
                          "key/value must be [tokens, kv_heads * head_size], got " + shape_str(in[kKey].shape));
        d.num_seqs = (int)in[kPastLens].shape.at(0);
        HIP_PLUGIN_ASSERT(in[kSubsequenceBegins].shape.at(0) == d.num_seqs + 1 &&
                              in[kBlockIndicesBegins].shape.at(0) == d.num_seqs + 1,
                          "subsequence_begins / block_indices_begins must have num_sequences + 1 entries");
        d.scale = host_scalar<float>(in[kScale], "scale", 0.0f, false);
        d.sliding_window = host_scalar<int32_t>(in[kSlidingWindow], "sliding_window", 0, false);
        d.max_context_len = host_scalar<int32_t>(in[kMaxContextLen], "max_context_len", 0, false);
        d.flags = 0;
        // As many tokens as sequences normally means one token each, and the kernels plan for that
        // without looking; when the lengths came from a host tensor they are looked at here, so that
        // a batch that only resembles a decode step (an empty sequence beside a longer one) is
        // announced as what it is.
        if (d.num_tokens == d.num_seqs && in[kSubsequenceBegins].host != nullptr) {
            const int32_t* begins = static_cast<const int32_t*>(in[kSubsequenceBegins].host);
            for (int s = 0; s < d.num_seqs; s++)
                if (begins[s + 1] - begins[s] != 1) {
                    d.flags |= HIPATTN_PA_ANY_LENGTHS;
                    break;
                }
        }
        d.decode_waves = 0;
        return d;
    }
    ElementType q_type_, kv_type_, cache_type_;
};

}  // namespace

}  // namespace hip_plugin

using hip_plugin::PagedAttentionOp;
using hip_plugin::PassThroughOp;
using hip_plugin::SdpaOp;
HIP_OPERATION_REGISTER(PassThroughOp, Parameter)
HIP_OPERATION_REGISTER(PassThroughOp, Result)
HIP_OPERATION_REGISTER(PassThroughOp, Constant)
HIP_OPERATION_REGISTER(SdpaOp, ScaledDotProductAttention)
HIP_OPERATION_REGISTER(PagedAttentionOp, PagedAttentionExtension)
