// OpenVINO device plugin "MI355X": runs weight-compressed FullyConnected nodes on the GPU through the
// C ABI of libovfcc (include/ovfcc.h).
//
//   ov::Core core;
//   core.register_plugin("/abs/path/libovfcc_plugin.so", "MI355X");
//   auto compiled = core.compile_model(model, "MI355X");      // unchanged ov::Model
//
// What the plugin accepts: models whose Results are MatMuls (transpose_a = false) of a Parameter with a
// weight-decompression subgraph
//     Constant(u4|i4|u8|i8) -> Convert -> [Subtract(zp)] -> Multiply(scale) -> [Reshape] -> [Convert] ->
//     [Transpose] -> [Convert] -> MatMul
// with the constants either output-major ([N, K]: transpose_b = true, or a Transpose node under transpose_b = false)
// or input-major ([K, N]: transpose_b = false and no Transpose node),
// i.e. exactly what ConvertMatMulToFC + ConvertFullyConnectedToFullyConnectedCompressed fold into
// ov::op::internal::FullyConnectedCompressed on the CPU plugin
// (src/plugins/intel_cpu/src/transformations/cpu_opset/common/pass/convert_matmul_to_fc.cpp:47-270,
//  src/common/transformations/src/transformations/op_conversions/convert_fc_to_compressed.cpp:170-225).
// The pattern is matched on the untouched input model, before any folding pass, so the u4/u8 constants
// are still there and no MarkDequantization pass is needed.  Everything else is reported as unsupported by
// query_model (a HETERO device can place it elsewhere) and rejected by compile_model.
//
// The interfaces implemented are ov::IPlugin (src/inference/dev_api/openvino/runtime/iplugin.hpp:74-255),
// ov::ICompiledModel (icompiled_model.hpp:36-190) and ov::ISyncInferRequest (isync_infer_request.hpp:30-175);
// the template plugin (src/plugins/template/src) is the model for which properties to answer.
//
// This file needs OpenVINO's developer headers and libopenvino to build; it is not part of libovfcc.so.
#include <cstring>
#include <istream>
#include <memory>
#include <mutex>
#include <ostream>
#include <sstream>
#include <string>
#include <vector>

#include "openvino/core/model.hpp"
#include "openvino/core/type/float16.hpp"
#include "openvino/op/constant.hpp"
#include "openvino/op/convert.hpp"
#include "openvino/op/matmul.hpp"
#include "openvino/op/multiply.hpp"
#include "openvino/op/parameter.hpp"
#include "openvino/op/reshape.hpp"
#include "openvino/op/result.hpp"
#include "openvino/op/subtract.hpp"
#include "openvino/op/transpose.hpp"
#include "openvino/pass/serialize.hpp"
#include "openvino/runtime/icompiled_model.hpp"
#include "openvino/runtime/internal_properties.hpp"
#include "openvino/runtime/iplugin.hpp"
#include "openvino/runtime/isync_infer_request.hpp"
#include "openvino/runtime/make_tensor.hpp"
#include "openvino/runtime/properties.hpp"
#include "ovfcc.h"

namespace ovfcc_plugin {

[[noreturn]] void throw_last(const char* what) {
    OPENVINO_THROW("ovfcc: ", what, ": ", ovfcc_last_error());
}

// ---- the decompression pattern ------------------------------------------------------------------------

struct CompressedFc {
    std::shared_ptr<ov::op::v0::MatMul> matmul;
    std::shared_ptr<ov::op::v0::Parameter> activations;
    std::shared_ptr<ov::op::v0::Constant> weights, scales, zero_points;  // zero_points may be null
    ovfcc_fc_desc desc{};
    std::vector<ov::float16> scales_f16;  // [N, K/G] ([K/G, N] with OVFCC_W_INPUT_MAJOR)
    std::vector<uint8_t> zp_bytes;        // packed u4 / u8 in OpenVINO order, or one element
};

static std::shared_ptr<ov::op::v0::Constant> constant_behind_convert(const ov::Output<ov::Node>& out) {
    auto node = out.get_node_shared_ptr();
    if (auto cvt = ov::as_type_ptr<ov::op::v0::Convert>(node))
        node = cvt->input_value(0).get_node_shared_ptr();
    return ov::as_type_ptr<ov::op::v0::Constant>(node);
}

static int weight_tag(const ov::element::Type& t) {
    if (t == ov::element::u4) return OVFCC_U4;
    if (t == ov::element::i4) return OVFCC_I4;
    if (t == ov::element::u8) return OVFCC_U8;
    if (t == ov::element::i8) return OVFCC_I8;
    return OVFCC_NONE;
}

// Matches MatMul(Parameter, decompression chain) and fills the C-ABI descriptor.  Mirrors the anchors of
// pattern::op::CompressedWeightsBlock (src/common/transformations/src/transformations/pattern_blocks/
// compressed_weights_block.cpp:31-84) and the shape algebra of combine_groups
// (convert_fc_to_compressed.cpp:42-78): W [N, K] or [N, K/G, G]; scale and zero-point [N, 1], [N, K/G, 1],
// [N], [1] or []; or all of them input-major ([K, N], [K/G, G, N], [K/G, 1, N], ...) under a MatMul with
// transpose_b = false, the form of the reference's decompression tests without transpose_weights
// (src/tests/test_utils/common_test_utils/src/subgraph_builders/weights_decompression_builders.cpp:60-204).
static bool match_compressed_fc(const std::shared_ptr<ov::Node>& node, CompressedFc& fc, std::string& why) {
    auto mm = ov::as_type_ptr<ov::op::v0::MatMul>(node);
    if (!mm)
        return false;
    if (mm->get_transpose_a()) {
        why = "MatMul must have transpose_a = false";
        return false;
    }
    auto param = ov::as_type_ptr<ov::op::v0::Parameter>(mm->input_value(0).get_node_shared_ptr());
    if (!param) {
        why = "activations must come straight from a Parameter";
        return false;
    }
    // walk up from the MatMul's weight input: [Convert] <- [Transpose of the last two axes] <- [Convert] <-
    // [Reshape] <- Multiply
    auto w = mm->input_value(1).get_node_shared_ptr();
    if (auto cvt = ov::as_type_ptr<ov::op::v0::Convert>(w))
        w = cvt->input_value(0).get_node_shared_ptr();
    bool transposed_in_graph = false;
    if (auto tr = ov::as_type_ptr<ov::op::v1::Transpose>(w)) {
        auto order = ov::as_type_ptr<ov::op::v0::Constant>(tr->input_value(1).get_node_shared_ptr());
        if (!order || order->cast_vector<int64_t>() != std::vector<int64_t>{1, 0}) {
            why = "a Transpose on the weight path must swap the two axes of a 2-D constant";
            return false;
        }
        transposed_in_graph = true;
        w = tr->input_value(0).get_node_shared_ptr();
        if (auto cvt = ov::as_type_ptr<ov::op::v0::Convert>(w))
            w = cvt->input_value(0).get_node_shared_ptr();
    }
    // The constants are output-major ([N, K], what FullyConnected wants) when exactly one of transpose_b and the
    // Transpose node turns them; otherwise they are input-major ([K, N]) and the library transposes them once,
    // as the Transpose that ConvertMatMulToFC inserts does in the reference (convert_matmul_to_fc.cpp:47-270).
    const bool input_major = mm->get_transpose_b() == transposed_in_graph;
    if (auto rs = ov::as_type_ptr<ov::op::v1::Reshape>(w))
        w = rs->input_value(0).get_node_shared_ptr();
    auto mul = ov::as_type_ptr<ov::op::v1::Multiply>(w);
    if (!mul) {
        why = "no Multiply(scale) on the weight path";
        return false;
    }
    // one Multiply input is the scale constant, the other Convert(W) or Subtract(Convert(W), zp)
    std::shared_ptr<ov::op::v0::Constant> scale;
    ov::Output<ov::Node> body;
    for (int side = 0; side < 2 && !scale; ++side) {
        auto c = constant_behind_convert(mul->input_value(side));
        if (c && c->get_element_type().is_real()) {
            scale = c;
            body = mul->input_value(1 - side);
        }
    }
    if (!scale) {
        why = "scale is not a floating-point constant";
        return false;
    }
    std::shared_ptr<ov::op::v0::Constant> zp;
    auto body_node = body.get_node_shared_ptr();
    if (auto sub = ov::as_type_ptr<ov::op::v1::Subtract>(body_node)) {
        zp = constant_behind_convert(sub->input_value(1));
        if (!zp) {
            why = "zero-point is not a constant";
            return false;
        }
        body_node = sub->input_value(0).get_node_shared_ptr();
    }
    auto wcvt = ov::as_type_ptr<ov::op::v0::Convert>(body_node);
    auto wconst = wcvt ? ov::as_type_ptr<ov::op::v0::Constant>(wcvt->input_value(0).get_node_shared_ptr()) : nullptr;
    if (!wconst || weight_tag(wconst->get_element_type()) == OVFCC_NONE) {
        why = "weights are not a u4/i4/u8/i8 constant behind a Convert";
        return false;
    }

    const auto& ws = wconst->get_shape();
    int64_t N, K, G;
    if (ws.size() == 2) {
        N = (int64_t)ws[input_major ? 1 : 0];
        K = (int64_t)ws[input_major ? 0 : 1];
        G = K;
    } else if (ws.size() == 3 && !input_major) {
        N = (int64_t)ws[0];
        K = (int64_t)(ws[1] * ws[2]);
        G = (int64_t)ws[2];
    } else if (ws.size() == 3) {
        N = (int64_t)ws[2];
        K = (int64_t)(ws[0] * ws[1]);
        G = (int64_t)ws[1];
    } else {
        why = "weights must be [N, K] or [N, K/G, G] (or [K, N], [K/G, G, N] for a MatMul that does not transpose them)";
        return false;
    }
    const int64_t ng = K / G;
    const size_t scale_count = ov::shape_size(scale->get_shape());
    if (scale_count != (size_t)(N * ng)) {
        if (scale_count == (size_t)N && ng == 1) {
            // per-channel [N] / [N, 1]
        } else {
            why = "scale must hold one value per (channel, group)";
            return false;
        }
    }
    if (mm->get_input_partial_shape(0).rbegin()->is_dynamic() ||
        mm->get_input_partial_shape(0).rbegin()->get_length() != K) {
        why = "last activation dimension must equal K";
        return false;
    }
    const auto act_type = param->get_element_type();
    if (act_type != ov::element::f16 && act_type != ov::element::f32) {
        why = "activations must be f16 (or f32, converted on the host)";
        return false;
    }

    fc.matmul = mm;
    fc.activations = param;
    fc.weights = wconst;
    fc.scales = scale;
    fc.zero_points = zp;
    fc.desc.N = N;
    fc.desc.K = K;
    fc.desc.group_size = G;
    fc.desc.w_type = weight_tag(wconst->get_element_type());
    fc.desc.scale_type = OVFCC_F16;
    fc.desc.bias_type = OVFCC_NONE;
    fc.desc.act_type = OVFCC_F16;
    fc.desc.out_type = mm->get_output_element_type(0) == ov::element::f32 ? OVFCC_F32 : OVFCC_F16;
    fc.desc.flags = input_major ? OVFCC_W_INPUT_MAJOR : 0;
    // scales as f16 in the constant's own order: [N, K/G], or [K/G, N] for input-major constants
    fc.scales_f16.resize((size_t)(N * ng));
    {
        const auto vals = scale->cast_vector<float>();
        for (size_t i = 0; i < fc.scales_f16.size(); ++i)
            fc.scales_f16[i] = ov::float16(vals[i]);
    }
    // zero-points: u4/u8 constants are passed through untouched; real-typed ones (NNCF sometimes stores
    // them as f16) must be integers in 0..255 and become u8
    fc.desc.zp_type = OVFCC_NONE;
    fc.desc.zp_scalar = 0;
    if (zp) {
        const size_t zc = ov::shape_size(zp->get_shape());
        if (zc != 1 && zc != (size_t)(N * ng)) {
            why = "zero-point must be scalar or hold one value per (channel, group)";
            return false;
        }
        fc.desc.zp_scalar = zc == 1 && N * ng != 1;
        const auto zt = zp->get_element_type();
        if (zt == ov::element::u4 || zt == ov::element::u8) {
            fc.desc.zp_type = zt == ov::element::u4 ? OVFCC_U4 : OVFCC_U8;
            fc.zp_bytes.assign(static_cast<const uint8_t*>(zp->get_data_ptr()),
                               static_cast<const uint8_t*>(zp->get_data_ptr()) + zp->get_byte_size());
        } else {
            const auto vals = zp->cast_vector<float>();
            fc.desc.zp_type = OVFCC_U8;
            fc.zp_bytes.resize(vals.size());
            for (size_t i = 0; i < vals.size(); ++i) {
                if (vals[i] < 0 || vals[i] > 255 || vals[i] != (float)(int)vals[i]) {
                    why = "zero-point values must be integers in 0..255";
                    return false;
                }
                fc.zp_bytes[i] = (uint8_t)vals[i];
            }
        }
    }
    if (ovfcc_desc_validate(&fc.desc) != OVFCC_OK) {
        why = ovfcc_last_error();
        return false;
    }
    return true;
}

// Nodes of the decompression chain of a matched MatMul (for query_model)
static void chain_nodes(const CompressedFc& fc, std::vector<std::shared_ptr<ov::Node>>& out) {
    std::vector<std::shared_ptr<ov::Node>> stack{fc.matmul->input_value(1).get_node_shared_ptr()};
    while (!stack.empty()) {
        auto n = stack.back();
        stack.pop_back();
        out.push_back(n);
        for (const auto& in : n->input_values())
            stack.push_back(in.get_node_shared_ptr());
    }
}

// ---- device-resident tensors -------------------------------------------------------------------------------
// The plugin's remote context hands out tensors that live in HBM (src/inference/dev_api/openvino/runtime/
// iremote_context.hpp:24-62, iremote_tensor.hpp:18-78; template: src/plugins/template/src/remote_context.cpp:17-140).
// An infer request whose input and output are such tensors runs without any host copy.

class RemoteTensor : public ov::IRemoteTensor {
public:
    RemoteTensor(std::shared_ptr<const ov::IPlugin> plugin, ovfcc_ctx* ctx, const ov::element::Type& type,
                 const ov::Shape& shape)
        : m_plugin(std::move(plugin)), m_ctx(ctx), m_type(type), m_shape(shape), m_device_name("MI355X") {
        OPENVINO_ASSERT(type.bitwidth() >= 8, "MI355X: remote tensors hold whole-byte element types, got ", type);
        reserve(byte_size_of(shape));
        update_strides();
    }
    ~RemoteTensor() override {
        if (m_ptr)
            ovfcc_device_free(m_ctx, m_ptr);
    }

    const ov::element::Type& get_element_type() const override {
        return m_type;
    }
    const ov::Shape& get_shape() const override {
        return m_shape;
    }
    const ov::Strides& get_strides() const override {
        return m_strides;
    }
    // A larger shape takes a fresh allocation (the old contents are dropped), a smaller one keeps the memory.
    void set_shape(ov::Shape shape) override {
        reserve(byte_size_of(shape));
        m_shape = std::move(shape);
        update_strides();
    }
    const ov::AnyMap& get_properties() const override {
        return m_properties;
    }
    const std::string& get_device_name() const override {
        return m_device_name;
    }
    // Whole-tensor copies only (offsets 0, empty region): what Tensor::copy_to / copy_from of the public API issue.
    void copy_from(const std::shared_ptr<const ov::ITensor>& src, size_t src_offset, size_t dst_offset,
                   const ov::Shape& roi_shape) override {
        OPENVINO_ASSERT(src_offset == 0 && dst_offset == 0 && roi_shape.empty(), "MI355X: region copies are not implemented");
        OPENVINO_ASSERT(src->get_element_type() == m_type && src->is_continuous(),
                        "MI355X: copy_from needs a dense tensor of type ", m_type);
        set_shape(src->get_shape());
        if (auto remote = std::dynamic_pointer_cast<const RemoteTensor>(src)) {
            if (get_byte_size() && ovfcc_memcpy_d2d(m_ctx, m_ptr, remote->device_ptr(), get_byte_size()) != OVFCC_OK)
                throw_last("memcpy_d2d");
        } else if (get_byte_size() && ovfcc_memcpy_h2d(m_ctx, m_ptr, src->data(), get_byte_size()) != OVFCC_OK) {
            throw_last("memcpy_h2d");
        }
    }
    void copy_to(const std::shared_ptr<ov::ITensor>& dst, size_t src_offset, size_t dst_offset,
                 const ov::Shape& roi_shape) const override {
        OPENVINO_ASSERT(src_offset == 0 && dst_offset == 0 && roi_shape.empty(), "MI355X: region copies are not implemented");
        OPENVINO_ASSERT(dst->get_element_type() == m_type, "MI355X: copy_to needs a tensor of type ", m_type);
        if (auto remote = std::dynamic_pointer_cast<RemoteTensor>(dst)) {
            remote->copy_from(std::static_pointer_cast<const ov::ITensor>(shared_from_this_tensor()), 0, 0, {});
            return;
        }
        dst->set_shape(m_shape);
        OPENVINO_ASSERT(dst->is_continuous(), "MI355X: copy_to needs a dense destination");
        if (get_byte_size() && ovfcc_memcpy_d2h(m_ctx, dst->data(), m_ptr, get_byte_size()) != OVFCC_OK)
            throw_last("memcpy_d2h");
    }

    void* device_ptr() const {
        return m_ptr;
    }

private:
    size_t byte_size_of(const ov::Shape& shape) const {
        return ov::shape_size(shape) * m_type.size();
    }
    // copy_to(remote) needs `this` as a shared tensor; a non-owning alias is enough for the duration of the call
    std::shared_ptr<const RemoteTensor> shared_from_this_tensor() const {
        return std::shared_ptr<const RemoteTensor>(std::shared_ptr<const RemoteTensor>{}, this);
    }
    void reserve(size_t bytes) {
        bytes = (std::max<size_t>(bytes, 16) + 15) / 16 * 16;
        if (bytes <= m_capacity)
            return;
        if (m_ptr)
            ovfcc_device_free(m_ctx, m_ptr);
        m_ptr = nullptr;
        m_capacity = 0;
        if (ovfcc_device_malloc(m_ctx, bytes, &m_ptr) != OVFCC_OK)
            throw_last("device_malloc");
        m_capacity = bytes;
        m_properties = {{ov::device::full_name.name(), m_device_name}, {"DEV_MEM_PTR", m_ptr}};
    }
    void update_strides() {
        m_strides.assign(m_shape.size(), 0);
        size_t stride = m_type.size();
        for (size_t d = m_shape.size(); d-- > 0;) {
            m_strides[d] = stride;
            stride *= m_shape[d];
        }
    }

    std::shared_ptr<const ov::IPlugin> m_plugin;  // keeps the device context alive
    ovfcc_ctx* m_ctx;
    ov::element::Type m_type;
    ov::Shape m_shape;
    ov::Strides m_strides;
    std::string m_device_name;
    ov::AnyMap m_properties;
    void* m_ptr = nullptr;
    size_t m_capacity = 0;
};

class RemoteContext : public ov::IRemoteContext {
public:
    RemoteContext(std::shared_ptr<const ov::IPlugin> plugin, ovfcc_ctx* ctx)
        : m_plugin(std::move(plugin)), m_ctx(ctx), m_name("MI355X"),
          m_property{{ov::device::full_name.name(), std::string("AMD Instinct MI355X (gfx950) via ovfcc")}} {}
    const std::string& get_device_name() const override {
        return m_name;
    }
    const ov::AnyMap& get_property() const override {
        return m_property;
    }
    ov::SoPtr<ov::IRemoteTensor> create_tensor(const ov::element::Type& type, const ov::Shape& shape,
                                               const ov::AnyMap&) override {
        return {std::make_shared<RemoteTensor>(m_plugin, m_ctx, type, shape), nullptr};
    }

private:
    std::shared_ptr<const ov::IPlugin> m_plugin;
    ovfcc_ctx* m_ctx;
    std::string m_name;
    ov::AnyMap m_property;
};

// ---- plugin -------------------------------------------------------------------------------------------------

class Plugin;

class CompiledModel : public ov::ICompiledModel {
public:
    struct Node {
        CompressedFc fc;
        ovfcc_weights* weights = nullptr;
        size_t input_index = 0, output_index = 0;
    };

    // node_flags: OVFCC_* flags for every node's descriptor (OVFCC_DYNQUANT_I8 when the caller allows dynamic
    // quantisation); blobs: the repacked nodes of an exported model, in result order, instead of a fresh repack
    CompiledModel(const std::shared_ptr<ov::Model>& model, const std::shared_ptr<const ov::IPlugin>& plugin,
                  ovfcc_ctx* ctx, bool profiling, int node_flags,
                  const std::vector<std::vector<uint8_t>>* blobs = nullptr);
    ~CompiledModel() override {
        for (auto& n : m_nodes)
            ovfcc_weights_destroy(n.weights);
    }

    // Stream layout: magic, node flags, the model as the template plugin stores it (xml and constants from
    // ov::pass::Serialize, each behind its size; src/plugins/template/src/compiled_model.cpp:173-192), then the
    // number of nodes and every node's repacked device image (ovfcc_weights_export) behind its size.
    void export_model(std::ostream& out) const override {
        std::stringstream xml, bin;
        ov::pass::Serialize(xml, bin).run_on_model(m_model);
        const std::string x = xml.str(), b = bin.str();
        auto put = [&out](const void* p, uint64_t n) {
            out.write(reinterpret_cast<const char*>(&n), sizeof(n));
            out.write(static_cast<const char*>(p), static_cast<std::streamsize>(n));
        };
        out.write(kExportMagic, sizeof(kExportMagic));
        const int32_t flags = m_node_flags;
        out.write(reinterpret_cast<const char*>(&flags), sizeof(flags));
        put(x.data(), x.size());
        put(b.data(), b.size());
        const uint64_t count = m_nodes.size();
        out.write(reinterpret_cast<const char*>(&count), sizeof(count));
        for (const auto& n : m_nodes) {
            size_t bytes = 0;
            if (ovfcc_weights_export_size(n.weights, &bytes) != OVFCC_OK)
                throw_last("weights_export_size");
            std::vector<uint8_t> blob(bytes);
            if (ovfcc_weights_export(n.weights, blob.data(), bytes) != OVFCC_OK)
                throw_last("weights_export");
            put(blob.data(), blob.size());
        }
    }
    static constexpr char kExportMagic[8] = {'O', 'V', 'F', 'C', 'C', 'M', '0', '1'};
    std::shared_ptr<const ov::Model> get_runtime_model() const override {
        return m_model;
    }
    void set_property(const ov::AnyMap&) override {
        OPENVINO_THROW_NOT_IMPLEMENTED("MI355X: compiled model has no mutable properties");
    }
    ov::Any get_property(const std::string& name) const override {
        if (name == ov::supported_properties)
            return std::vector<ov::PropertyName>{ov::supported_properties, ov::model_name,
                                                 ov::optimal_number_of_infer_requests, ov::execution_devices,
                                                 ov::enable_profiling};
        if (name == ov::model_name)
            return decltype(ov::model_name)::value_type{m_model->get_friendly_name()};
        if (name == ov::optimal_number_of_infer_requests)
            return decltype(ov::optimal_number_of_infer_requests)::value_type{2};
        if (name == ov::execution_devices)
            return decltype(ov::execution_devices)::value_type{get_plugin()->get_device_name()};
        if (name == ov::enable_profiling)
            return m_profiling;
        OPENVINO_THROW("MI355X: unsupported compiled-model property ", name);
    }
    std::shared_ptr<ov::ISyncInferRequest> create_sync_infer_request() const override;

    const std::vector<Node>& nodes() const {
        return m_nodes;
    }
    ovfcc_ctx* ctx() const {
        return m_ctx;
    }

private:
    std::shared_ptr<ov::Model> m_model;
    std::vector<Node> m_nodes;
    ovfcc_ctx* m_ctx;
    int m_node_flags = 0;
    bool m_profiling;
};

class InferRequest : public ov::ISyncInferRequest {
public:
    explicit InferRequest(const std::shared_ptr<const CompiledModel>& compiled)
        : ov::ISyncInferRequest(compiled), m_compiled(compiled) {
        if (ovfcc_request_create(compiled->ctx(), &m_request) != OVFCC_OK)
            throw_last("request_create");
        // host tensors for every port, as the template plugin does (src/plugins/template/src/sync_infer_request.cpp:94-110)
        for (const auto& port : get_inputs())
            allocate_tensor(port, [port](ov::SoPtr<ov::ITensor>& t) {
                allocate_tensor_impl(t, port.get_element_type(),
                                     port.get_partial_shape().is_dynamic() ? ov::Shape{0} : port.get_shape());
            });
        for (const auto& port : get_outputs())
            allocate_tensor(port, [port](ov::SoPtr<ov::ITensor>& t) {
                allocate_tensor_impl(t, port.get_element_type(),
                                     port.get_partial_shape().is_dynamic() ? ov::Shape{0} : port.get_shape());
            });
    }
    ~InferRequest() override {
        for (auto& b : m_device_staging)
            if (b.ptr)
                ovfcc_device_free(m_compiled->ctx(), b.ptr);
        ovfcc_request_destroy(m_request);
    }

    void infer() override {
        check_tensors();
        m_kernels.clear();
        for (const auto& node : m_compiled->nodes()) {
            auto in = get_tensor(get_inputs()[node.input_index]);
            auto out = get_tensor(get_outputs()[node.output_index]);
            const ov::Shape in_shape = in->get_shape();
            int64_t M = 1;  // 3-D activations flatten to [B*S, K] like the CPU path does
            for (size_t d = 0; d + 1 < in_shape.size(); ++d)
                M *= (int64_t)in_shape[d];
            ov::Shape out_shape = in_shape;
            out_shape.back() = (size_t)node.fc.desc.N;
            out->set_shape(out_shape);  // dynamic M: the output follows the input
            auto rin = std::dynamic_pointer_cast<RemoteTensor>(in._ptr);
            auto rout = std::dynamic_pointer_cast<RemoteTensor>(out._ptr);
            if (rin || rout) {
                // Device-resident tensors: no copy on their side.  A host tensor on the other side goes through a
                // device buffer of the request.
                OPENVINO_ASSERT(in->get_element_type() == ov::element::f16,
                                "MI355X: a device-resident input must be f16, got ", in->get_element_type());
                const size_t x_bytes = (size_t)M * node.fc.desc.K * sizeof(ov::float16);
                const size_t y_bytes = out->get_byte_size();
                void* x_dev = rin ? rin->device_ptr() : device_staging(0, x_bytes);
                void* y_dev = rout ? rout->device_ptr() : device_staging(1, y_bytes);
                if (!rin && x_bytes && ovfcc_memcpy_h2d(m_compiled->ctx(), x_dev, in->data(), x_bytes) != OVFCC_OK)
                    throw_last("memcpy_h2d");
                if (ovfcc_fc_run_device(m_request, node.weights, x_dev, y_dev, M) != OVFCC_OK)
                    throw_last("fc_run_device");
                if (ovfcc_request_sync(m_request) != OVFCC_OK)
                    throw_last("request_sync");
                if (!rout && y_bytes && ovfcc_memcpy_d2h(m_compiled->ctx(), out->data(), y_dev, y_bytes) != OVFCC_OK)
                    throw_last("memcpy_d2h");
            } else {
                const void* x = in->data();
                if (in->get_element_type() == ov::element::f32) {
                    // the device path computes on f16 activations
                    const float* src = static_cast<const float*>(in->data());
                    m_staging.resize((size_t)M * node.fc.desc.K);
                    for (size_t i = 0; i < m_staging.size(); ++i)
                        m_staging[i] = ov::float16(src[i]);
                    x = m_staging.data();
                }
                if (ovfcc_fc_run(m_request, node.weights, x, out->data(), M) != OVFCC_OK)
                    throw_last("fc_run");
            }
            ovfcc_kernel_info info;
            ovfcc_last_kernel_info(m_request, &info);
            m_kernels.push_back(info);
        }
    }

    std::vector<ov::ProfilingInfo> get_profiling_info() const override {
        std::vector<ov::ProfilingInfo> out;
        for (size_t i = 0; i < m_kernels.size(); ++i) {
            ov::ProfilingInfo p;
            p.status = ov::ProfilingInfo::Status::EXECUTED;
            p.node_name = m_compiled->nodes()[i].fc.matmul->get_friendly_name();
            p.node_type = "FullyConnected";
            p.exec_type = m_kernels[i].name;
            out.push_back(p);
        }
        return out;
    }
    std::vector<ov::SoPtr<ov::IVariableState>> query_state() const override {
        return {};
    }

private:
    static void allocate_tensor_impl(ov::SoPtr<ov::ITensor>& tensor, const ov::element::Type& type,
                                     const ov::Shape& shape) {
        if (!tensor || tensor->get_element_type() != type)
            tensor = ov::make_tensor(type, shape);
        else
            tensor->set_shape(shape);
    }

    // device buffer `which` (0 = activations, 1 = outputs) of at least `bytes`, kept and grown across calls
    void* device_staging(int which, size_t bytes) {
        auto& b = m_device_staging[which];
        if (bytes > b.bytes) {
            if (b.ptr)
                ovfcc_device_free(m_compiled->ctx(), b.ptr);
            b.ptr = nullptr, b.bytes = 0;
            if (ovfcc_device_malloc(m_compiled->ctx(), bytes, &b.ptr) != OVFCC_OK)
                throw_last("device_malloc");
            b.bytes = bytes;
        }
        return b.ptr;
    }

    struct DeviceBuffer {
        void* ptr = nullptr;
        size_t bytes = 0;
    };
    std::shared_ptr<const CompiledModel> m_compiled;
    ovfcc_request* m_request = nullptr;
    DeviceBuffer m_device_staging[2];
    std::vector<ov::float16> m_staging;
    std::vector<ovfcc_kernel_info> m_kernels;
};

class Plugin : public ov::IPlugin {
public:
    Plugin() {
        set_device_name("MI355X");
    }
    ~Plugin() override {
        ovfcc_destroy(m_ctx);
    }

    std::shared_ptr<ov::ICompiledModel> compile_model(const std::shared_ptr<const ov::Model>& model,
                                                      const ov::AnyMap& properties) const override {
        bool profiling = m_profiling;
        uint64_t dq_group = m_dq_group;
        for (const auto& kv : properties) {
            if (kv.first == ov::enable_profiling.name())
                profiling = kv.second.as<bool>();
            else if (kv.first == ov::hint::dynamic_quantization_group_size.name())
                dq_group = kv.second.as<uint64_t>();
            else if (!known_hint(kv.first))
                OPENVINO_THROW("MI355X: unsupported property ", kv.first);
        }
        return std::make_shared<CompiledModel>(model->clone(), shared_from_this(), context(), profiling,
                                               dq_group != 0 ? OVFCC_DYNQUANT_I8 : 0);
    }
    std::shared_ptr<ov::ICompiledModel> compile_model(const std::shared_ptr<const ov::Model>& model,
                                                      const ov::AnyMap& properties,
                                                      const ov::SoPtr<ov::IRemoteContext>&) const override {
        return compile_model(model, properties);
    }

    void set_property(const ov::AnyMap& properties) override {
        for (const auto& kv : properties) {
            if (kv.first == ov::enable_profiling.name())
                m_profiling = kv.second.as<bool>();
            else if (kv.first == ov::hint::dynamic_quantization_group_size.name())
                m_dq_group = kv.second.as<uint64_t>();  // non-zero: activations may be quantised per token
            else if (!known_hint(kv.first))
                OPENVINO_THROW("MI355X: unsupported property ", kv.first);
        }
    }

    ov::Any get_property(const std::string& name, const ov::AnyMap&) const override {
        if (name == ov::supported_properties)
            return std::vector<ov::PropertyName>{
                {ov::available_devices.name(), ov::PropertyMutability::RO},
                {ov::supported_properties.name(), ov::PropertyMutability::RO},
                {ov::device::full_name.name(), ov::PropertyMutability::RO},
                {ov::device::architecture.name(), ov::PropertyMutability::RO},
                {ov::device::capabilities.name(), ov::PropertyMutability::RO},
                {ov::device::type.name(), ov::PropertyMutability::RO},
                {ov::range_for_async_infer_requests.name(), ov::PropertyMutability::RO},
                {ov::execution_devices.name(), ov::PropertyMutability::RO},
                {ov::enable_profiling.name(), ov::PropertyMutability::RW},
                {ov::hint::dynamic_quantization_group_size.name(), ov::PropertyMutability::RW},
                {ov::hint::performance_mode.name(), ov::PropertyMutability::RW},
                {ov::hint::inference_precision.name(), ov::PropertyMutability::RW},
                {ov::hint::num_requests.name(), ov::PropertyMutability::RW},
                {ov::num_streams.name(), ov::PropertyMutability::RW},
                {ov::device::id.name(), ov::PropertyMutability::RW},
            };
        // caching_properties tells Core which properties key a cache entry (src/inference/src/dev/plugin.cpp:115-118)
        if (name == ov::internal::supported_properties)
            return decltype(ov::internal::supported_properties)::value_type{
                {ov::internal::caching_properties.name(), ov::PropertyMutability::RO}};
        if (name == ov::internal::caching_properties)
            return std::vector<ov::PropertyName>{ov::device::architecture.name(),
                                                 ov::hint::dynamic_quantization_group_size.name()};
        if (name == ov::hint::dynamic_quantization_group_size)
            return m_dq_group;
        if (name == ov::available_devices)
            return decltype(ov::available_devices)::value_type{"0"};
        if (name == ov::device::full_name)
            return decltype(ov::device::full_name)::value_type{"AMD Instinct MI355X (gfx950) via ovfcc"};
        if (name == ov::device::architecture)
            return decltype(ov::device::architecture)::value_type{"gfx950"};
        if (name == ov::device::type)
            return decltype(ov::device::type)::value_type{ov::device::Type::DISCRETE};
        if (name == ov::device::capabilities)
            return decltype(ov::device::capabilities)::value_type{ov::device::capability::FP16,
                                                                  ov::device::capability::EXPORT_IMPORT};
        if (name == ov::execution_devices)
            return decltype(ov::execution_devices)::value_type{get_device_name()};
        if (name == ov::range_for_async_infer_requests)
            return decltype(ov::range_for_async_infer_requests)::value_type{1, 8, 1};
        if (name == ov::enable_profiling)
            return m_profiling;
        if (name == ov::hint::performance_mode)
            return ov::hint::PerformanceMode::LATENCY;
        if (name == ov::hint::inference_precision)
            return ov::element::f16;
        if (name == ov::hint::num_requests)
            return (uint32_t)0;
        if (name == ov::num_streams)
            return ov::streams::Num(1);
        if (name == ov::device::id)
            return std::string("0");
        OPENVINO_THROW("MI355X: unsupported property ", name);
    }

    // One kind of context: the device's own memory (template: src/plugins/template/src/plugin.cpp:115-124).
    ov::SoPtr<ov::IRemoteContext> create_context(const ov::AnyMap&) const override {
        return {std::make_shared<RemoteContext>(shared_from_this(), context()), nullptr};
    }
    // (Contexts hold no state of their own, so the default one is not cached: a cached context would keep the
    // plugin alive, which it points back to.)
    ov::SoPtr<ov::IRemoteContext> get_default_context(const ov::AnyMap&) const override {
        return {std::make_shared<RemoteContext>(shared_from_this(), context()), nullptr};
    }
    // The reverse of CompiledModel::export_model: the model is read back through Core, the nodes are rebuilt from
    // their device images without repacking (template: src/plugins/template/src/plugin.cpp:230-311).
    std::shared_ptr<ov::ICompiledModel> import_model(std::istream& in, const ov::AnyMap& properties) const override {
        char magic[sizeof(CompiledModel::kExportMagic)];
        in.read(magic, sizeof(magic));
        if (!in || std::memcmp(magic, CompiledModel::kExportMagic, sizeof(magic)) != 0)
            OPENVINO_THROW("MI355X: the stream does not hold a model exported by this plugin");
        int32_t flags = 0;
        in.read(reinterpret_cast<char*>(&flags), sizeof(flags));
        auto get = [&in](std::vector<uint8_t>& v) {
            uint64_t n = 0;
            in.read(reinterpret_cast<char*>(&n), sizeof(n));
            if (!in || n > (uint64_t(1) << 40))
                OPENVINO_THROW("MI355X: damaged model stream");
            v.resize(n);
            in.read(reinterpret_cast<char*>(v.data()), static_cast<std::streamsize>(n));
            if (!in)
                OPENVINO_THROW("MI355X: truncated model stream");
        };
        std::vector<uint8_t> xml, bin;
        get(xml);
        get(bin);
        uint64_t count = 0;
        in.read(reinterpret_cast<char*>(&count), sizeof(count));
        if (!in || count > 65536)
            OPENVINO_THROW("MI355X: damaged model stream");
        std::vector<std::vector<uint8_t>> blobs(count);
        for (auto& b : blobs)
            get(b);
        ov::Tensor weights(ov::element::u8, ov::Shape{bin.size()});
        std::memcpy(weights.data(), bin.data(), bin.size());
        auto model = get_core()->read_model(std::string(xml.begin(), xml.end()), weights);
        bool profiling = m_profiling;
        for (const auto& kv : properties)
            if (kv.first == ov::enable_profiling.name())
                profiling = kv.second.as<bool>();
        return std::make_shared<CompiledModel>(model, shared_from_this(), context(), profiling, flags, &blobs);
    }
    std::shared_ptr<ov::ICompiledModel> import_model(std::istream& in, const ov::SoPtr<ov::IRemoteContext>&,
                                                     const ov::AnyMap& properties) const override {
        return import_model(in, properties);
    }
    std::shared_ptr<ov::ICompiledModel> import_model(const ov::Tensor& blob, const ov::AnyMap& properties) const override {
        std::istringstream in(std::string(static_cast<const char*>(blob.data()), blob.get_byte_size()));
        return import_model(in, properties);
    }
    std::shared_ptr<ov::ICompiledModel> import_model(const ov::Tensor& blob, const ov::SoPtr<ov::IRemoteContext>&,
                                                     const ov::AnyMap& properties) const override {
        return import_model(blob, properties);
    }

    // Supported: each matched MatMul with its whole decompression chain, and the Parameter / Result around it.
    ov::SupportedOpsMap query_model(const std::shared_ptr<const ov::Model>& model, const ov::AnyMap&) const override {
        ov::SupportedOpsMap res;
        for (const auto& node : model->get_ordered_ops()) {
            CompressedFc fc;
            std::string why;
            if (!match_compressed_fc(node, fc, why))
                continue;
            std::vector<std::shared_ptr<ov::Node>> nodes;
            chain_nodes(fc, nodes);
            nodes.push_back(fc.matmul);
            nodes.push_back(fc.activations);
            for (const auto& user : fc.matmul->output(0).get_target_inputs())
                if (ov::is_type<ov::op::v0::Result>(user.get_node()))
                    nodes.push_back(user.get_node()->shared_from_this());
            for (const auto& n : nodes)
                res[n->get_friendly_name()] = get_device_name();
        }
        return res;
    }

private:
    static bool known_hint(const std::string& k) {
        return k == ov::hint::performance_mode.name() || k == ov::hint::inference_precision.name() ||
               k == ov::hint::num_requests.name() || k == ov::num_streams.name() || k == ov::device::id.name() ||
               k == ov::hint::execution_mode.name() || k == ov::hint::model_priority.name() ||
               k == ov::inference_num_threads.name() || k == ov::log::level.name();
    }
    // the device context is created on first use: Core constructs plugins on hosts without the device too
    ovfcc_ctx* context() const {
        std::lock_guard<std::mutex> lock(m_mutex);
        if (!m_ctx && ovfcc_init(0, &m_ctx) != OVFCC_OK)
            throw_last("init");
        return m_ctx;
    }

    mutable std::mutex m_mutex;
    mutable ovfcc_ctx* m_ctx = nullptr;
    bool m_profiling = false;
    uint64_t m_dq_group = 0;  // ov::hint::dynamic_quantization_group_size; 0 = off
};

CompiledModel::CompiledModel(const std::shared_ptr<ov::Model>& model, const std::shared_ptr<const ov::IPlugin>& plugin,
                             ovfcc_ctx* ctx, bool profiling, int node_flags,
                             const std::vector<std::vector<uint8_t>>* blobs)
    : ov::ICompiledModel(model, plugin), m_model(model), m_ctx(ctx), m_node_flags(node_flags), m_profiling(profiling) {
    if (blobs && blobs->size() != model->get_results().size())
        OPENVINO_THROW("MI355X: the imported blob holds ", blobs->size(), " nodes, the model ", model->get_results().size());
    // every Result must be fed by a matched MatMul; every Parameter must feed one
    const auto& results = model->get_results();
    const auto& params = model->get_parameters();
    for (size_t r = 0; r < results.size(); ++r) {
        Node n;
        std::string why = "not a MatMul";
        auto producer = results[r]->input_value(0).get_node_shared_ptr();
        if (!match_compressed_fc(producer, n.fc, why))
            OPENVINO_THROW("MI355X: result ", results[r]->get_friendly_name(),
                           " is not produced by a weight-compressed FullyConnected: ", why,
                           " (use HETERO:MI355X,CPU for the rest of the graph)");
        n.output_index = r;
        for (size_t p = 0; p < params.size(); ++p)
            if (params[p] == n.fc.activations)
                n.input_index = p;
        n.fc.desc.flags |= node_flags;
        if (blobs) {
            // the cached device image; the library checks it against its own descriptor
            if (ovfcc_weights_import(ctx, (*blobs)[r].data(), (*blobs)[r].size(), &n.weights) != OVFCC_OK)
                throw_last("weights_import");
        } else {
            const void* zp = n.fc.zp_bytes.empty() ? nullptr : n.fc.zp_bytes.data();
            if (ovfcc_weights_create(ctx, &n.fc.desc, n.fc.weights->get_data_ptr(), n.fc.scales_f16.data(), zp,
                                     nullptr, &n.weights) != OVFCC_OK)
                throw_last("weights_create");
        }
        // the executed graph shows the same layer type the CPU plugin shows
        // (src/inference/dev_api/openvino/runtime/exec_model_info.hpp:31-73)
        n.fc.matmul->get_rt_info()["layerType"] = std::string("FullyConnected");
        n.fc.matmul->get_rt_info()["primitiveType"] =
            std::string(ovfcc_weights_is_tiled(n.weights) ? "hip_tiled_w" : "hip_plain_w") +
            (n.fc.desc.w_type == OVFCC_U8 || n.fc.desc.w_type == OVFCC_I8 ? "8" : "4");
        m_nodes.push_back(std::move(n));
    }
}

std::shared_ptr<ov::ISyncInferRequest> CompiledModel::create_sync_infer_request() const {
    return std::make_shared<InferRequest>(std::static_pointer_cast<const CompiledModel>(shared_from_this()));
}

}  // namespace ovfcc_plugin

static const ov::Version version = {"ovfcc-0.1", "openvino_mi355x_plugin"};
OV_DEFINE_PLUGIN_CREATE_FUNCTION(ovfcc_plugin::Plugin, version)
