// OpenVINO device plugin "MI355X": runs weight-compressed FullyConnected nodes on the GPU through the
// C ABI of libovfcc (include/ovfcc.h).
//
//   ov::Core core;
//   core.register_plugin("/abs/path/libovfcc_plugin.so", "MI355X");
//   auto compiled = core.compile_model(model, "MI355X");      // unchanged ov::Model
//
// What the plugin accepts: models whose Results are produced by weight-compressed FullyConnected nodes over a
// Parameter, each a MatMul (transpose_a = false) or internal FullyConnected with a weight-decompression subgraph
//     Constant(u4|i4|u8|i8) -> Convert -> [Subtract(zp)] -> Multiply(scale) -> [Reshape] -> [Convert] ->
//     [Transpose] -> [Convert] -> MatMul [-> Add(bias Constant)]
// with the constants either output-major ([N, K]: transpose_b = true, or a Transpose node under transpose_b = false)
// or input-major ([K, N]: transpose_b = false and no Transpose node) -- what ConvertMatMulToFC,
// ConvertFullyConnectedToFullyConnectedCompressed and FullyConnectedBiasFusion fold into
// ov::op::internal::FullyConnectedCompressed on the CPU plugin
// (src/plugins/intel_cpu/src/transformations/cpu_opset/common/pass/convert_matmul_to_fc.cpp:47-270,
//  src/common/transformations/src/transformations/op_conversions/convert_fc_to_compressed.cpp:170-225,
//  src/plugins/intel_cpu/src/transformations/cpu_opset/common/pass/fc_bias_fusion.cpp:32-93).  Two or three such nodes
// of one format over the same Parameter run as one launch (horizontal fusion,
// src/plugins/intel_gpu/src/plugin/transformations/fc_horizontal_fusion.cpp), and Multiply(Swish | Gelu (gate(x)), up(x))
// runs as one node with a gated-linear-unit epilogue.  A mixture-of-experts block in the form the reference's
// Convert3GatherMatmulMoeBlockToMoeOp matches (three GatherMatmul / GatherMatmulCompressed nodes over batched
// compressed constants [E, N, K] or [E, N, K/G, G], the gate activation, the Multiply by the transposed routing
// weights, ReduceSum and Reshape; src/common/transformations/src/transformations/common_optimizations/
// moe_op_fusion.cpp:55-232) whose hidden states, routing weights and expert indices are Parameters runs as one
// ovfcc_moe_device call -- MOECompressed in the executed graph.  A v17::GroupedMatMul over batched compressed constants
// (or the GroupedMatMulCompressed that ConvertGroupedMatMulToGroupedMatMulCompressed makes of it,
// src/common/transformations/src/transformations/op_conversions/convert_grouped_matmul_to_compressed.cpp:25-118) whose
// activations and offsets are Parameters runs as one ovfcc_grouped_matmul_device call, and a GatherMatmul[Compressed]
// outside such a block, over Parameters for activations and indices, as one ovfcc_gather_matmul_device call.  The pattern is matched on the untouched input model, before
// any folding pass, so the u4/u8 constants are still there and no MarkDequantization pass is needed.  Everything
// else is reported as unsupported by query_model (a HETERO device can place it elsewhere) and rejected by
// compile_model.
//
// The interfaces implemented are ov::IPlugin (src/inference/dev_api/openvino/runtime/iplugin.hpp:74-255),
// ov::ICompiledModel (icompiled_model.hpp:36-190) and ov::ISyncInferRequest (isync_infer_request.hpp:30-175);
// the template plugin (src/plugins/template/src) is the model for which properties to answer.
//
// This file needs OpenVINO's developer headers and libopenvino to build; it is not part of libovfcc.so.
#include <atomic>
#include <chrono>
#include <cstring>
#include <istream>
#include <memory>
#include <mutex>
#include <ostream>
#include <sstream>
#include <string>
#include <unordered_map>
#include <vector>

#include "openvino/core/model.hpp"
#include "openvino/core/type/float16.hpp"
#include "openvino/op/constant.hpp"
#include "openvino/op/add.hpp"
#include "openvino/op/convert.hpp"
#include "openvino/op/gelu.hpp"
#include "openvino/op/matmul.hpp"
#include "openvino/op/multiply.hpp"
#include "openvino/op/parameter.hpp"
#include "openvino/op/reduce_sum.hpp"
#include "openvino/op/reshape.hpp"
#include "openvino/op/result.hpp"
#include "openvino/op/slice.hpp"
#include "openvino/op/subtract.hpp"
#include "openvino/op/swish.hpp"
#include "openvino/op/transpose.hpp"
#include "openvino/op/unsqueeze.hpp"
#include "openvino/pass/serialize.hpp"
#include "openvino/runtime/exec_model_info.hpp"
#include "openvino/runtime/icompiled_model.hpp"
#include "openvino/runtime/internal_properties.hpp"
#include "openvino/runtime/iplugin.hpp"
#include "openvino/runtime/isync_infer_request.hpp"
#include "openvino/runtime/make_tensor.hpp"
#include "openvino/runtime/properties.hpp"
#include "ov_ops/fully_connected.hpp"
#include "ov_ops/fully_connected_compressed.hpp"
#include "ov_ops/gather_matmul.hpp"
#include "ov_ops/gather_matmul_compressed.hpp"
#include "ov_ops/grouped_matmul_compressed.hpp"
#include "ovfcc.h"
#include "ovfcc_graph.h"

namespace ovfcc_plugin {

[[noreturn]] void throw_last(const char* what) {
    OPENVINO_THROW("ovfcc: ", what, ": ", ovfcc_last_error());
}

// ---- the model as plain nodes, and what the graph-side entry points make of it --------------------------
// The decisions -- which subgraph is one FullyConnectedCompressed node, how its constants are re-viewed, which bias
// Add folds in, which nodes share a launch -- are taken by libovfcc on a plain description of the model
// (include/ovfcc_graph.h), where they are unit-tested without OpenVINO.  This file only translates: ov::Node ->
// ovfcc_gnode on the way in, the Constants' bytes -> ovfcc_fold_weights_create on the way out.

static int type_tag(const ov::element::Type& t) {
    if (t == ov::element::u4) return OVFCC_U4;
    if (t == ov::element::i4) return OVFCC_I4;
    if (t == ov::element::u8) return OVFCC_U8;
    if (t == ov::element::i8) return OVFCC_I8;
    if (t == ov::element::f16) return OVFCC_F16;
    if (t == ov::element::f32) return OVFCC_F32;
    return OVFCC_TYPE_OTHER;
}

struct ModelGraph {
    std::vector<std::shared_ptr<ov::Node>> ops;  // topological order; index = node id
    std::vector<ovfcc_gnode> nodes;
    std::vector<const void*> constant_data;      // per node: a Constant's bytes (the model keeps them alive), else null
    std::vector<ovfcc_fold> folds;
    std::vector<ovfcc_fused> fused;
    std::vector<ovfcc_moe_fold> moes;  // expert blocks (three GatherMatmul nodes and what joins them)
    // GroupedMatMul[Compressed] nodes over batched compressed constants, and GatherMatmul[Compressed] nodes that
    // are no part of an expert block
    struct Batched {
        ovfcc_gather_fold fold;
        bool gather;
    };
    std::vector<Batched> grouped;
};

static ModelGraph describe(const std::shared_ptr<const ov::Model>& model) {
    ModelGraph g;
    g.ops = model->get_ordered_ops();
    std::unordered_map<const ov::Node*, int> index;
    for (size_t i = 0; i < g.ops.size(); ++i)
        index[g.ops[i].get()] = (int)i;
    g.nodes.resize(g.ops.size());
    g.constant_data.assign(g.ops.size(), nullptr);
    for (size_t i = 0; i < g.ops.size(); ++i) {
        const auto& op = g.ops[i];
        ovfcc_gnode& n = g.nodes[i];
        std::memset(&n, 0, sizeof(n));
        n.n_ints = -1;
        if (ov::is_type<ov::op::v0::Parameter>(op)) n.op = OVFCC_OP_PARAMETER;
        else if (ov::is_type<ov::op::v0::Constant>(op)) n.op = OVFCC_OP_CONSTANT;
        else if (ov::is_type<ov::op::v0::Convert>(op)) n.op = OVFCC_OP_CONVERT;
        else if (ov::is_type<ov::op::v1::Subtract>(op)) n.op = OVFCC_OP_SUBTRACT;
        else if (ov::is_type<ov::op::v1::Multiply>(op)) n.op = OVFCC_OP_MULTIPLY;
        else if (ov::is_type<ov::op::v1::Reshape>(op)) n.op = OVFCC_OP_RESHAPE;
        else if (ov::is_type<ov::op::v1::Transpose>(op)) n.op = OVFCC_OP_TRANSPOSE;
        else if (ov::is_type<ov::op::v0::MatMul>(op)) n.op = OVFCC_OP_MATMUL;
        else if (ov::is_type<ov::op::internal::FullyConnected>(op)) n.op = OVFCC_OP_FULLY_CONNECTED;
        else if (ov::is_type<ov::op::v1::Add>(op)) n.op = OVFCC_OP_ADD;
        else if (ov::is_type<ov::op::v4::Swish>(op)) n.op = OVFCC_OP_SWISH;
        else if (ov::is_type<ov::op::v7::Gelu>(op)) n.op = OVFCC_OP_GELU;
        else if (ov::is_type<ov::op::v0::Result>(op)) n.op = OVFCC_OP_RESULT;
        else if (ov::is_type<ov::op::internal::GatherMatmulCompressed>(op)) n.op = OVFCC_OP_GATHER_MATMUL_COMPRESSED;
        else if (ov::is_type<ov::op::internal::GatherMatmul>(op)) n.op = OVFCC_OP_GATHER_MATMUL;
        else if (ov::is_type<ov::op::internal::GroupedMatMulCompressed>(op)) n.op = OVFCC_OP_GROUPED_MATMUL_COMPRESSED;
        else if (ov::is_type<ov::op::v17::GroupedMatMul>(op)) n.op = OVFCC_OP_GROUPED_MATMUL;
        else if (ov::is_type<ov::op::v0::Unsqueeze>(op)) n.op = OVFCC_OP_UNSQUEEZE;
        else if (ov::is_type<ov::op::v8::Slice>(op)) n.op = OVFCC_OP_SLICE;
        else if (ov::is_type<ov::op::v1::ReduceSum>(op)) n.op = OVFCC_OP_REDUCE_SUM;
        else n.op = OVFCC_OP_OTHER;
        if (op->get_output_size() == 0 || op->get_input_size() > OVFCC_MAX_INPUTS) {
            n.op = OVFCC_OP_OTHER;
            n.rank = -1;
            continue;
        }
        n.type = type_tag(op->get_output_element_type(0));
        const auto& ps = op->get_output_partial_shape(0);
        if (ps.rank().is_dynamic() || ps.size() > OVFCC_MAX_RANK) {
            n.rank = -1;
        } else {
            n.rank = (int32_t)ps.size();
            for (size_t d = 0; d < ps.size(); ++d)
                n.dims[d] = ps[d].is_static() ? ps[d].get_length() : -1;
        }
        n.n_inputs = (int32_t)op->get_input_size();
        for (size_t k = 0; k < op->get_input_size(); ++k)
            n.inputs[k] = index.at(op->get_input_node_ptr(k));
        n.consumers = (int32_t)op->output(0).get_target_inputs().size();
        if (auto mm = ov::as_type_ptr<ov::op::v0::MatMul>(op)) {
            n.transpose_a = mm->get_transpose_a();
            n.transpose_b = mm->get_transpose_b();
        } else if (auto gelu = ov::as_type_ptr<ov::op::v7::Gelu>(op)) {
            n.attr = gelu->get_approximation_mode() == ov::op::GeluApproximationMode::TANH;
        } else if (auto rs = ov::as_type_ptr<ov::op::v1::ReduceSum>(op)) {
            n.attr = rs->get_keep_dims();
        } else if (auto sw = ov::as_type_ptr<ov::op::v4::Swish>(op)) {
            if (sw->get_input_size() != 1)
                n.op = OVFCC_OP_OTHER;  // a beta input: not the beta = 1 form the kernels compute
        } else if (auto c = ov::as_type_ptr<ov::op::v0::Constant>(op)) {
            g.constant_data[i] = c->get_data_ptr();
            // FullyConnected's "no bias" is Constant(dynamic, Shape{0}); small integer constants carry their values
            if (c->get_element_type().is_integral_number() && c->get_element_type().bitwidth() >= 8 &&
                ov::shape_size(c->get_shape()) <= OVFCC_MAX_RANK) {
                const auto vals = c->cast_vector<int64_t>();
                n.n_ints = (int32_t)vals.size();
                for (size_t k = 0; k < vals.size(); ++k)
                    n.ints[k] = vals[k];
            }
        }
    }
    g.folds.resize(g.nodes.size() + 1);
    g.fused.resize(g.nodes.size() + 1);
    int n_folds = 0, n_fused = 0;
    if (ovfcc_fold_model(g.nodes.data(), (int)g.nodes.size(), g.folds.data(), (int)g.folds.size(), &n_folds,
                         g.fused.data(), (int)g.fused.size(), &n_fused) != OVFCC_OK)
        throw_last("fold_model");
    g.folds.resize(n_folds);
    g.fused.resize(n_fused);
    // expert blocks: every node that feeds a Result is tried as the block's root
    for (size_t i = 0; i < g.nodes.size(); ++i) {
        if (g.nodes[i].op != OVFCC_OP_RESULT)
            continue;
        ovfcc_moe_fold m;
        if (ovfcc_fold_moe(g.nodes.data(), (int)g.nodes.size(), g.nodes[i].inputs[0], &m) == OVFCC_OK)
            g.moes.push_back(m);
    }
    // grouped matrix products over batched compressed constants, and routed ones outside expert blocks
    for (size_t i = 0; i < g.nodes.size(); ++i) {
        const int op = g.nodes[i].op;
        ovfcc_gather_fold f;
        if (op == OVFCC_OP_GROUPED_MATMUL || op == OVFCC_OP_GROUPED_MATMUL_COMPRESSED) {
            if (ovfcc_fold_grouped_matmul(g.nodes.data(), (int)g.nodes.size(), (int)i, &f) == OVFCC_OK)
                g.grouped.push_back({f, false});
        } else if (op == OVFCC_OP_GATHER_MATMUL || op == OVFCC_OP_GATHER_MATMUL_COMPRESSED) {
            bool in_block = false;
            for (const auto& m : g.moes)
                in_block = in_block || m.gate.root == (int)i || m.up.root == (int)i || m.down.root == (int)i;
            if (!in_block && ovfcc_fold_gather_matmul(g.nodes.data(), (int)g.nodes.size(), (int)i, &f) == OVFCC_OK)
                g.grouped.push_back({f, true});
        }
    }
    return g;
}

// A matched node, or expert e of a routed / grouped one, created by the library from the Constants' own bytes.
static ovfcc_weights* create_node(ovfcc_ctx* ctx, const ModelGraph& g, const ovfcc_fold& f, int flags) {
    ovfcc_weights* out = nullptr;
    if (ovfcc_fold_weights_create(ctx, g.nodes.data(), (int)g.nodes.size(), &f, g.constant_data.data(), flags, &out) != OVFCC_OK)
        throw_last("fold_weights_create");
    return out;
}

static ovfcc_weights* create_expert(ovfcc_ctx* ctx, const ModelGraph& g, const ovfcc_gather_fold& f, int e, int flags) {
    ovfcc_weights* out = nullptr;
    if (ovfcc_fold_expert_weights_create(ctx, g.nodes.data(), (int)g.nodes.size(), &f, e, g.constant_data.data(), flags,
                                         &out) != OVFCC_OK)
        throw_last("fold_expert_weights_create");
    return out;
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

// One fused node of the compiled model = one kernel launch per inference.
struct Launch {
    struct Output {
        size_t result_index;    // the model output that receives ...
        int64_t column, width;  // ... these columns of the launch's [M, N_out] rows
    };
    ovfcc_weights* weights = nullptr;
    int kind = OVFCC_FUSED_SINGLE;  // enum ovfcc_fused_kind
    size_t input_index = 0;         // the Parameter that holds X
    int64_t K = 0, N_out = 0;
    int out_type = OVFCC_F16;
    std::vector<Output> outputs;    // one (the whole row), or one per horizontally fused part
    std::string name;               // friendly name of the node the launch stands for
    std::vector<std::string> original_names;
    std::string primitive;          // primitiveType of the executed graph
    std::vector<int> folds;         // indices into ModelGraph::folds
};

// One expert block of the compiled model = one ovfcc_moe_device call per inference.
struct MoeLaunch {
    std::vector<ovfcc_weights*> gate_up, down;  // per expert: gate and up with the gated linear unit, down
    size_t hidden_index = 0, routing_index = 0, indices_index = 0;  // the Parameters
    size_t result_index = 0;
    int64_t H = 0;
    int top_k = 0, out_type = OVFCC_F16;
    std::string name;
    std::vector<std::string> original_names;
};

// One GroupedMatMulCompressed node -- a node per group, activations and (in the 2-D x 3-D form) offsets from
// Parameters -- or one GatherMatmulCompressed node outside an expert block: a node per expert, activations
// [1 or top_k, M, K] and indices [M, top_k] from Parameters (offsets_index names the indices then)
struct GroupedLaunch {
    std::vector<ovfcc_weights*> groups;
    size_t a_index = 0, offsets_index = 0, result_index = 0;
    bool with_offsets = false;
    bool gather = false;
    int64_t K = 0, N = 0;
    int out_type = OVFCC_F16;
    std::string name;
    std::vector<std::string> original_names;
};

class CompiledModel : public ov::ICompiledModel {
public:
    // node_flags: OVFCC_* flags for every node's descriptor (OVFCC_DYNQUANT_I8 when the caller allows dynamic
    // quantisation); blobs: the repacked nodes of an exported model, in launch order, instead of a fresh repack
    CompiledModel(const std::shared_ptr<ov::Model>& model, const std::shared_ptr<const ov::IPlugin>& plugin,
                  ovfcc_ctx* ctx, bool profiling, int node_flags,
                  const std::vector<std::vector<uint8_t>>* blobs = nullptr);
    ~CompiledModel() override {
        for (auto& l : m_launches)
            ovfcc_weights_destroy(l.weights);
        for (auto& m : m_moes) {
            for (auto* w : m.gate_up)
                ovfcc_weights_destroy(w);
            for (auto* w : m.down)
                ovfcc_weights_destroy(w);
        }
        for (auto& gm : m_grouped)
            for (auto* w : gm.groups)
                ovfcc_weights_destroy(w);
    }

    // Stream layout: magic, node flags, the model as the template plugin stores it (xml and constants from
    // ov::pass::Serialize, each behind its size; src/plugins/template/src/compiled_model.cpp:173-192), then the
    // number of launches and every launch's repacked device image (ovfcc_weights_export) behind its size.
    void export_model(std::ostream& out) const override {
        OPENVINO_ASSERT(m_moes.empty() && m_grouped.empty(),
                        "MI355X: a model with expert blocks or grouped matrix products is compiled from its constants "
                        "each time (no blob form of batched weights)");
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
        const uint64_t count = m_launches.size();
        out.write(reinterpret_cast<const char*>(&count), sizeof(count));
        for (const auto& l : m_launches) {
            size_t bytes = 0;
            if (ovfcc_weights_export_size(l.weights, &bytes) != OVFCC_OK)
                throw_last("weights_export_size");
            std::vector<uint8_t> blob(bytes);
            if (ovfcc_weights_export(l.weights, blob.data(), bytes) != OVFCC_OK)
                throw_last("weights_export");
            put(blob.data(), blob.size());
        }
    }
    static constexpr char kExportMagic[8] = {'O', 'V', 'F', 'C', 'C', 'M', '0', '2'};

    // The executed graph (src/inference/dev_api/openvino/runtime/exec_model_info.hpp:31-110): one node per launch
    // with the keys the CPU plugin's executed graph carries -- layerType "FullyConnected", primitiveType,
    // originalLayersNames, outputPrecisions, outputLayouts, execOrder and execTimeMcs (the last measured time of the
    // launch, or "not_executed").  A node that stands for one unfused FullyConnected whose constants are
    // output-major is an ov::op::internal::FullyConnectedCompressed over the model's own constants, re-viewed as
    // ConvertFullyConnectedToFullyConnectedCompressed re-views them; fused nodes are ExecutionNodes.
    std::shared_ptr<const ov::Model> get_runtime_model() const override {
        ov::ParameterVector params;
        for (const auto& p : m_model->get_parameters())
            params.push_back(std::make_shared<ov::op::v0::Parameter>(p->get_element_type(), p->get_partial_shape()));
        ov::ResultVector results(m_model->get_results().size());
        for (size_t i = 0; i < m_launches.size(); ++i) {
            const Launch& l = m_launches[i];
            std::shared_ptr<ov::Node> node;
            if (l.kind == OVFCC_FUSED_SINGLE && !(m_graph.folds[(size_t)l.folds[0]].desc.flags & OVFCC_W_INPUT_MAJOR))
                node = compressed_node(m_graph.folds[(size_t)l.folds[0]], params[l.input_index]);
            else
                node = std::make_shared<ov::exec_model_info::ExecutionNode>(ov::OutputVector{params[l.input_index]}, 1);
            node->set_friendly_name(l.name);
            auto& rt = node->get_rt_info();
            std::string names;
            for (const auto& n : l.original_names)
                names += (names.empty() ? "" : ",") + n;
            rt[ov::exec_model_info::LAYER_TYPE] = std::string("FullyConnected");
            rt[ov::exec_model_info::IMPL_TYPE] = l.primitive;
            rt[ov::exec_model_info::ORIGINAL_NAMES] = names;
            rt[ov::exec_model_info::OUTPUT_PRECISIONS] = std::string(l.out_type == OVFCC_F32 ? "f32" : "f16");
            rt[ov::exec_model_info::OUTPUT_LAYOUTS] = std::string("ab");
            rt[ov::exec_model_info::EXECUTION_ORDER] = std::to_string(i);
            const double us = m_last_us[i].load();
            rt[ov::exec_model_info::PERF_COUNTER] = us < 0 ? std::string("not_executed") : std::to_string((long long)us);
            for (const auto& o : l.outputs) {
                results[o.result_index] = std::make_shared<ov::op::v0::Result>(node);
                results[o.result_index]->set_friendly_name(m_model->get_results()[o.result_index]->get_friendly_name());
            }
        }
        for (size_t i = 0; i < m_moes.size(); ++i) {
            const MoeLaunch& m = m_moes[i];
            auto node = std::make_shared<ov::exec_model_info::ExecutionNode>(
                ov::OutputVector{params[m.hidden_index], params[m.routing_index], params[m.indices_index]}, 1);
            node->set_friendly_name(m.name);
            auto& rt = node->get_rt_info();
            std::string names;
            for (const auto& n : m.original_names)
                names += (names.empty() ? "" : ",") + n;
            rt[ov::exec_model_info::LAYER_TYPE] = std::string("MOECompressed");
            rt[ov::exec_model_info::IMPL_TYPE] = std::string("hip_moe_grouped_w4");
            rt[ov::exec_model_info::ORIGINAL_NAMES] = names;
            rt[ov::exec_model_info::OUTPUT_PRECISIONS] = std::string(m.out_type == OVFCC_F32 ? "f32" : "f16");
            rt[ov::exec_model_info::OUTPUT_LAYOUTS] = std::string("ab");
            rt[ov::exec_model_info::EXECUTION_ORDER] = std::to_string(m_launches.size() + i);
            const double us = m_last_us[m_launches.size() + i].load();
            rt[ov::exec_model_info::PERF_COUNTER] = us < 0 ? std::string("not_executed") : std::to_string((long long)us);
            results[m.result_index] = std::make_shared<ov::op::v0::Result>(node);
            results[m.result_index]->set_friendly_name(m_model->get_results()[m.result_index]->get_friendly_name());
        }
        for (size_t i = 0; i < m_grouped.size(); ++i) {
            const GroupedLaunch& gm = m_grouped[i];
            ov::OutputVector ins{params[gm.a_index]};
            if (gm.with_offsets)
                ins.push_back(params[gm.offsets_index]);
            auto node = std::make_shared<ov::exec_model_info::ExecutionNode>(ins, 1);
            node->set_friendly_name(gm.name);
            auto& rt = node->get_rt_info();
            std::string names;
            for (const auto& n : gm.original_names)
                names += (names.empty() ? "" : ",") + n;
            rt[ov::exec_model_info::LAYER_TYPE] = std::string(gm.gather ? "GatherMatmulCompressed" : "GroupedMatMulCompressed");
            rt[ov::exec_model_info::IMPL_TYPE] = std::string("hip_grouped");
            rt[ov::exec_model_info::ORIGINAL_NAMES] = names;
            rt[ov::exec_model_info::OUTPUT_PRECISIONS] = std::string(gm.out_type == OVFCC_F32 ? "f32" : "f16");
            rt[ov::exec_model_info::OUTPUT_LAYOUTS] = std::string(gm.with_offsets && !gm.gather ? "ab" : "abc");
            const size_t order = m_launches.size() + m_moes.size() + i;
            rt[ov::exec_model_info::EXECUTION_ORDER] = std::to_string(order);
            const double us = m_last_us[order].load();
            rt[ov::exec_model_info::PERF_COUNTER] = us < 0 ? std::string("not_executed") : std::to_string((long long)us);
            results[gm.result_index] = std::make_shared<ov::op::v0::Result>(node);
            results[gm.result_index]->set_friendly_name(m_model->get_results()[gm.result_index]->get_friendly_name());
        }
        return std::make_shared<ov::Model>(results, params, m_model->get_friendly_name() + "_executed");
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

    const std::vector<Launch>& launches() const {
        return m_launches;
    }
    const std::vector<MoeLaunch>& moes() const {
        return m_moes;
    }
    const std::vector<GroupedLaunch>& grouped() const {
        return m_grouped;
    }
    ovfcc_ctx* ctx() const {
        return m_ctx;
    }
    void record_time(size_t launch, double us) const {
        m_last_us[launch].store(us);
    }

private:
    // FullyConnectedCompressed over the fold's own constants (output-major), for the executed graph
    std::shared_ptr<ov::Node> compressed_node(const ovfcc_fold& f, const ov::Output<ov::Node>& x) const {
        const auto constant = [this](int id) { return ov::as_type_ptr<ov::op::v0::Constant>(m_graph.ops[(size_t)id]); };
        const auto view = [](const std::shared_ptr<ov::op::v0::Constant>& c, const int64_t v[2]) {
            return v[0] == 0 ? c : std::make_shared<ov::op::v0::Constant>(*c, ov::Shape{(size_t)v[0], (size_t)v[1]});
        };
        std::shared_ptr<ov::Node> bias = f.bias >= 0
                                             ? std::static_pointer_cast<ov::Node>(constant(f.bias))
                                             : std::make_shared<ov::op::v0::Constant>(ov::element::dynamic, ov::Shape{0});
        const auto out_type = f.desc.out_type == OVFCC_F32 ? ov::element::f32 : ov::element::f16;
        auto w = view(constant(f.weights), f.w_view);
        auto s = view(constant(f.scales), f.scale_view);
        if (f.zero_points >= 0)
            return std::make_shared<ov::op::internal::FullyConnectedCompressed>(x, w, bias, s,
                                                                                 view(constant(f.zero_points), f.zp_view),
                                                                                 out_type);
        return std::make_shared<ov::op::internal::FullyConnectedCompressed>(x, w, bias, s, out_type);
    }

    std::shared_ptr<ov::Model> m_model;
    ModelGraph m_graph;
    std::vector<Launch> m_launches;
    std::vector<MoeLaunch> m_moes;
    std::vector<GroupedLaunch> m_grouped;
    mutable std::vector<std::atomic<double>> m_last_us;  // per launch: last measured time, -1 before the first run
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
        m_times_us.clear();
        const auto& launches = m_compiled->launches();
        for (size_t li = 0; li < launches.size(); ++li) {
            const Launch& l = launches[li];
            const auto t0 = std::chrono::steady_clock::now();
            auto in = get_tensor(get_inputs()[l.input_index]);
            const ov::Shape in_shape = in->get_shape();
            int64_t M = 1;  // 3-D activations flatten to [B*S, K] like the CPU path does
            for (size_t d = 0; d + 1 < in_shape.size(); ++d)
                M *= (int64_t)in_shape[d];
            std::vector<ov::SoPtr<ov::ITensor>> outs;
            for (const auto& o : l.outputs) {
                auto out = get_tensor(get_outputs()[o.result_index]);
                ov::Shape out_shape = in_shape;
                out_shape.back() = (size_t)o.width;
                out->set_shape(out_shape);  // dynamic M: the output follows the input
                outs.push_back(out);
            }
            const size_t out_el = l.out_type == OVFCC_F32 ? 4 : 2;
            auto rin = std::dynamic_pointer_cast<RemoteTensor>(in._ptr);
            auto rout = l.outputs.size() == 1 ? std::dynamic_pointer_cast<RemoteTensor>(outs[0]._ptr) : nullptr;
            for (const auto& out : outs)
                OPENVINO_ASSERT(l.outputs.size() == 1 || !std::dynamic_pointer_cast<RemoteTensor>(out._ptr),
                                "MI355X: the outputs of a horizontally fused node must be host tensors");
            if (rin || rout) {
                // Device-resident tensors: no copy on their side.  A host tensor on the other side goes through a
                // device buffer of the request.
                OPENVINO_ASSERT(in->get_element_type() == ov::element::f16,
                                "MI355X: a device-resident input must be f16, got ", in->get_element_type());
                const size_t x_bytes = (size_t)M * l.K * sizeof(ov::float16);
                const size_t y_bytes = (size_t)M * l.N_out * out_el;
                void* x_dev = rin ? rin->device_ptr() : device_staging(0, x_bytes);
                void* y_dev = rout ? rout->device_ptr() : device_staging(1, y_bytes);
                if (!rin && x_bytes && ovfcc_memcpy_h2d(m_compiled->ctx(), x_dev, in->data(), x_bytes) != OVFCC_OK)
                    throw_last("memcpy_h2d");
                if (ovfcc_fc_run_device(m_request, l.weights, x_dev, y_dev, M) != OVFCC_OK)
                    throw_last("fc_run_device");
                if (ovfcc_request_sync(m_request) != OVFCC_OK)
                    throw_last("request_sync");
                if (!rout) {
                    m_y_staging.resize(y_bytes);
                    if (y_bytes && ovfcc_memcpy_d2h(m_compiled->ctx(), m_y_staging.data(), y_dev, y_bytes) != OVFCC_OK)
                        throw_last("memcpy_d2h");
                    scatter_columns(l, outs, M, out_el);
                }
            } else {
                const void* x = in->data();
                if (in->get_element_type() == ov::element::f32) {
                    // the device path computes on f16 activations
                    const float* src = static_cast<const float*>(in->data());
                    m_staging.resize((size_t)M * l.K);
                    for (size_t i = 0; i < m_staging.size(); ++i)
                        m_staging[i] = ov::float16(src[i]);
                    x = m_staging.data();
                }
                if (l.outputs.size() == 1) {
                    if (ovfcc_fc_run(m_request, l.weights, x, outs[0]->data(), M) != OVFCC_OK)
                        throw_last("fc_run");
                } else {
                    m_y_staging.resize((size_t)M * l.N_out * out_el);
                    if (ovfcc_fc_run(m_request, l.weights, x, m_y_staging.data(), M) != OVFCC_OK)
                        throw_last("fc_run");
                    scatter_columns(l, outs, M, out_el);
                }
            }
            ovfcc_kernel_info info;
            ovfcc_last_kernel_info(m_request, &info);
            m_kernels.push_back(info);
            const double us = std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count();
            m_times_us.push_back(us);
            m_compiled->record_time(li, us);
        }
        run_expert_blocks();
        run_grouped_products();
    }

    std::vector<ov::ProfilingInfo> get_profiling_info() const override {
        std::vector<ov::ProfilingInfo> out;
        for (size_t i = 0; i < m_kernels.size(); ++i) {
            ov::ProfilingInfo p;
            p.status = ov::ProfilingInfo::Status::EXECUTED;
            const size_t n_fc = m_compiled->launches().size(), n_moe = m_compiled->moes().size();
            p.node_name = i < n_fc           ? m_compiled->launches()[i].name
                          : i < n_fc + n_moe ? m_compiled->moes()[i - n_fc].name
                                             : m_compiled->grouped()[i - n_fc - n_moe].name;
            p.node_type = i < n_fc           ? "FullyConnected"
                          : i < n_fc + n_moe ? "MOECompressed"
                          : m_compiled->grouped()[i - n_fc - n_moe].gather ? "GatherMatmulCompressed"
                                                                           : "GroupedMatMulCompressed";
            p.exec_type = m_kernels[i].name;
            p.real_time = p.cpu_time = std::chrono::microseconds((long long)m_times_us[i]);
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

    // Expert blocks: hidden states [.., H], routing weights [M, top_k] and indices [M, top_k] in host tensors;
    // staged to the device (f16, f16, int32), one ovfcc_moe_device call, result copied back.
    void run_expert_blocks() {
        const auto& moes = m_compiled->moes();
        for (size_t mi = 0; mi < moes.size(); ++mi) {
            const MoeLaunch& m = moes[mi];
            const auto t0 = std::chrono::steady_clock::now();
            auto hidden = get_tensor(get_inputs()[m.hidden_index]);
            auto routing = get_tensor(get_inputs()[m.routing_index]);
            auto indices = get_tensor(get_inputs()[m.indices_index]);
            auto out = get_tensor(get_outputs()[m.result_index]);
            const ov::Shape in_shape = hidden->get_shape();
            int64_t M = 1;
            for (size_t d = 0; d + 1 < in_shape.size(); ++d)
                M *= (int64_t)in_shape[d];
            out->set_shape(in_shape);
            const size_t pairs = (size_t)M * (size_t)m.top_k;
            OPENVINO_ASSERT(routing->get_size() == pairs && indices->get_size() == pairs,
                            "MI355X: routing weights and indices must hold M x top_k values");
            auto to_half = [this](const ov::SoPtr<ov::ITensor>& t, size_t count) -> const void* {
                if (t->get_element_type() == ov::element::f16)
                    return t->data();
                OPENVINO_ASSERT(t->get_element_type() == ov::element::f32, "MI355X: expected an f16 or f32 tensor");
                const float* src = static_cast<const float*>(t->data());
                m_staging.resize(count);
                for (size_t i = 0; i < count; ++i)
                    m_staging[i] = ov::float16(src[i]);
                return m_staging.data();
            };
            const size_t x_bytes = (size_t)M * m.H * 2, r_bytes = pairs * 2, y_bytes = (size_t)M * m.H * (m.out_type == OVFCC_F32 ? 4 : 2);
            void* x_dev = device_staging(0, x_bytes);
            void* y_dev = device_staging(1, y_bytes);
            void* r_dev = device_staging(2, r_bytes);
            if (x_bytes && ovfcc_memcpy_h2d(m_compiled->ctx(), x_dev, to_half(hidden, (size_t)M * m.H), x_bytes) != OVFCC_OK)
                throw_last("memcpy_h2d");
            if (r_bytes && ovfcc_memcpy_h2d(m_compiled->ctx(), r_dev, to_half(routing, pairs), r_bytes) != OVFCC_OK)
                throw_last("memcpy_h2d");
            std::vector<int32_t> idx(pairs);
            if (indices->get_element_type() == ov::element::i32) {
                std::memcpy(idx.data(), indices->data(), pairs * sizeof(int32_t));
            } else {
                OPENVINO_ASSERT(indices->get_element_type() == ov::element::i64, "MI355X: indices must be i32 or i64");
                const int64_t* src = static_cast<const int64_t*>(indices->data());
                for (size_t i = 0; i < pairs; ++i)
                    idx[i] = (int32_t)src[i];
            }
            if (ovfcc_moe_device(m_request, m.gate_up.data(), m.down.data(), (int)m.gate_up.size(), x_dev, r_dev, idx.data(), M,
                                 m.top_k, y_dev) != OVFCC_OK)
                throw_last("moe_device");
            if (ovfcc_request_sync(m_request) != OVFCC_OK)
                throw_last("request_sync");
            if (y_bytes) {
                if (out->get_element_type() == ov::element::f32 && m.out_type != OVFCC_F32) {
                    m_y_staging.resize(y_bytes);
                    if (ovfcc_memcpy_d2h(m_compiled->ctx(), m_y_staging.data(), y_dev, y_bytes) != OVFCC_OK)
                        throw_last("memcpy_d2h");
                    const auto* h = reinterpret_cast<const ov::float16*>(m_y_staging.data());
                    float* dst = static_cast<float*>(out->data());
                    for (size_t i = 0; i < (size_t)M * m.H; ++i)
                        dst[i] = (float)h[i];
                } else if (ovfcc_memcpy_d2h(m_compiled->ctx(), out->data(), y_dev, y_bytes) != OVFCC_OK) {
                    throw_last("memcpy_d2h");
                }
            }
            ovfcc_kernel_info info;
            ovfcc_last_kernel_info(m_request, &info);
            m_kernels.push_back(info);
            const double us = std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count();
            m_times_us.push_back(us);
            m_compiled->record_time(m_compiled->launches().size() + mi, us);
        }
    }

    // GroupedMatMulCompressed: activations [rows, K] with offsets [G] (cumulative row ends, i32 or i64), or
    // [G, M, K], in host tensors; staged to the device as f16, one ovfcc_grouped_matmul_device call, result copied back.
    void run_grouped_products() {
        const auto& all = m_compiled->grouped();
        for (size_t gi = 0; gi < all.size(); ++gi) {
            const GroupedLaunch& gm = all[gi];
            const auto t0 = std::chrono::steady_clock::now();
            auto a = get_tensor(get_inputs()[gm.a_index]);
            auto out = get_tensor(get_outputs()[gm.result_index]);
            const ov::Shape as = a->get_shape();
            OPENVINO_ASSERT(as.size() == (gm.with_offsets && !gm.gather ? 2u : 3u) && (int64_t)as.back() == gm.K,
                            "MI355X: activations of ", gm.name, " have an unexpected shape");
            const int n_groups = (int)gm.groups.size();
            OPENVINO_ASSERT(gm.gather || gm.with_offsets || (int)as[0] == n_groups,
                            "MI355X: one batch of activations per group");
            const int64_t rows = gm.with_offsets && !gm.gather ? (int64_t)as[0] : (int64_t)as[1];
            int top_k = 0;
            ov::Shape os = as;
            os.back() = (size_t)gm.N;
            std::vector<int32_t> offsets;
            if (gm.with_offsets) {
                auto off = get_tensor(get_inputs()[gm.offsets_index]);
                if (gm.gather) {
                    // indices [M, top_k]; the output is [top_k, M, N]
                    const ov::Shape is = off->get_shape();
                    OPENVINO_ASSERT(is.size() == 2 && (int64_t)is[0] == rows, "MI355X: indices must be [M, top_k]");
                    top_k = (int)is[1];
                    OPENVINO_ASSERT(as[0] == 1 || (int)as[0] == top_k, "MI355X: one batch of activations, or one per selection");
                    os[0] = (size_t)top_k;
                } else {
                    OPENVINO_ASSERT(off->get_size() == (size_t)n_groups, "MI355X: one offset per group");
                }
                offsets.resize(off->get_size());
                if (off->get_element_type() == ov::element::i32) {
                    std::memcpy(offsets.data(), off->data(), offsets.size() * sizeof(int32_t));
                } else {
                    OPENVINO_ASSERT(off->get_element_type() == ov::element::i64, "MI355X: offsets must be i32 or i64");
                    const int64_t* src = static_cast<const int64_t*>(off->data());
                    for (size_t i = 0; i < offsets.size(); ++i)
                        offsets[i] = (int32_t)src[i];
                }
            }
            out->set_shape(os);
            const size_t count = a->get_size(), out_count = out->get_size();
            const size_t x_bytes = count * 2, y_bytes = out_count * (gm.out_type == OVFCC_F32 ? 4 : 2);
            void* x_dev = device_staging(0, x_bytes);
            void* y_dev = device_staging(1, y_bytes);
            const void* x = a->data();
            if (a->get_element_type() != ov::element::f16) {
                OPENVINO_ASSERT(a->get_element_type() == ov::element::f32, "MI355X: expected f16 or f32 activations");
                const float* src = static_cast<const float*>(a->data());
                m_staging.resize(count);
                for (size_t i = 0; i < count; ++i)
                    m_staging[i] = ov::float16(src[i]);
                x = m_staging.data();
            }
            if (x_bytes && ovfcc_memcpy_h2d(m_compiled->ctx(), x_dev, x, x_bytes) != OVFCC_OK)
                throw_last("memcpy_h2d");
            if (gm.gather) {
                if (ovfcc_gather_matmul_device(m_request, gm.groups.data(), n_groups, x_dev, (int)as[0], offsets.data(), rows,
                                               top_k, y_dev) != OVFCC_OK)
                    throw_last("gather_matmul_device");
            } else if (ovfcc_grouped_matmul_device(m_request, gm.groups.data(), n_groups, x_dev,
                                                   gm.with_offsets ? offsets.data() : nullptr, rows, y_dev) != OVFCC_OK) {
                throw_last("grouped_matmul_device");
            }
            if (ovfcc_request_sync(m_request) != OVFCC_OK)
                throw_last("request_sync");
            if (y_bytes) {
                if (out->get_element_type() == ov::element::f32 && gm.out_type != OVFCC_F32) {
                    m_y_staging.resize(y_bytes);
                    if (ovfcc_memcpy_d2h(m_compiled->ctx(), m_y_staging.data(), y_dev, y_bytes) != OVFCC_OK)
                        throw_last("memcpy_d2h");
                    const auto* h = reinterpret_cast<const ov::float16*>(m_y_staging.data());
                    float* dst = static_cast<float*>(out->data());
                    for (size_t i = 0; i < out_count; ++i)
                        dst[i] = (float)h[i];
                } else if (ovfcc_memcpy_d2h(m_compiled->ctx(), out->data(), y_dev, y_bytes) != OVFCC_OK) {
                    throw_last("memcpy_d2h");
                }
            }
            ovfcc_kernel_info info;
            ovfcc_last_kernel_info(m_request, &info);
            m_kernels.push_back(info);
            const double us = std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count();
            m_times_us.push_back(us);
            m_compiled->record_time(m_compiled->launches().size() + m_compiled->moes().size() + gi, us);
        }
    }

    // rows of m_y_staging ([M, N_out]) -> every output's columns (the VariadicSplit after a horizontally fused node)
    void scatter_columns(const Launch& l, const std::vector<ov::SoPtr<ov::ITensor>>& outs, int64_t M, size_t el) {
        for (size_t k = 0; k < l.outputs.size(); ++k) {
            const auto& o = l.outputs[k];
            auto* dst = static_cast<uint8_t*>(outs[k]->data());
            for (int64_t m = 0; m < M; ++m)
                std::memcpy(dst + (size_t)m * o.width * el,
                            m_y_staging.data() + ((size_t)m * l.N_out + (size_t)o.column) * el, (size_t)o.width * el);
        }
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
    DeviceBuffer m_device_staging[3];
    std::vector<ov::float16> m_staging;
    std::vector<uint8_t> m_y_staging;
    std::vector<ovfcc_kernel_info> m_kernels;
    std::vector<double> m_times_us;
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
        bool profiling = m_profiling, dq_asym = m_dq_asym;
        uint64_t dq_group = m_dq_group;
        for (const auto& kv : properties) {
            if (kv.first == ov::enable_profiling.name())
                profiling = kv.second.as<bool>();
            else if (kv.first == ov::hint::dynamic_quantization_group_size.name())
                dq_group = kv.second.as<uint64_t>();
            else if (kv.first == kAsymDynamicQuantization)
                dq_asym = kv.second.as<bool>();
            else if (!known_hint(kv.first))
                OPENVINO_THROW("MI355X: unsupported property ", kv.first);
        }
        return std::make_shared<CompiledModel>(model->clone(), shared_from_this(), context(), profiling,
                                               dq_group == 0 ? 0 : OVFCC_DYNQUANT_I8 | (dq_asym ? OVFCC_DYNQUANT_ASYM : 0));
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
            else if (kv.first == kAsymDynamicQuantization)
                m_dq_asym = kv.second.as<bool>();  // ... as unsigned bytes with a zero-point per token
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
                {kAsymDynamicQuantization, ov::PropertyMutability::RW},
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
                                                 ov::hint::dynamic_quantization_group_size.name(),
                                                 kAsymDynamicQuantization};
        if (name == ov::hint::dynamic_quantization_group_size)
            return m_dq_group;
        if (name == kAsymDynamicQuantization)
            return m_dq_asym;
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

    // Supported: every matched node with its whole decompression chain (bias Add, gate activation and the Multiply
    // of a gated linear unit included), and the Parameter / Results around it.
    ov::SupportedOpsMap query_model(const std::shared_ptr<const ov::Model>& model, const ov::AnyMap&) const override {
        ov::SupportedOpsMap res;
        const ModelGraph g = describe(model);
        auto mark = [&](int id) {
            if (id >= 0)
                res[g.ops[(size_t)id]->get_friendly_name()] = get_device_name();
        };
        auto mark_results_of = [&](int id) {
            for (const auto& user : g.ops[(size_t)id]->output(0).get_target_inputs())
                if (ov::is_type<ov::op::v0::Result>(user.get_node()))
                    res[user.get_node()->get_friendly_name()] = get_device_name();
        };
        for (const auto& u : g.fused) {
            for (int k = 0; k < u.n_parts; ++k) {
                const ovfcc_fold& f = g.folds[(size_t)u.parts[k]];
                for (int c = 0; c < f.n_chain; ++c)
                    mark(f.chain[c]);
                mark(f.matmul);
                mark(f.root);
                if (g.nodes[(size_t)f.activations].op == OVFCC_OP_PARAMETER)
                    mark(f.activations);
                // gate and up of a gated unit feed its Multiply, not a model output
                if (u.kind == OVFCC_FUSED_SINGLE || u.kind == OVFCC_FUSED_CONCAT || (u.kind == OVFCC_FUSED_MLP && k == 2))
                    mark_results_of(f.root);
            }
            if (u.kind == OVFCC_FUSED_GLU || u.kind == OVFCC_FUSED_MLP) {
                // the unit's Multiply: the group's root, or what the down projection of an MLP group reads
                const int mul = u.kind == OVFCC_FUSED_GLU ? u.root : g.folds[(size_t)u.parts[2]].activations;
                mark(mul);
                for (const auto& in : g.ops[(size_t)mul]->input_values())  // the gate's activation node
                    if (ov::is_type<ov::op::v4::Swish>(in.get_node()) || ov::is_type<ov::op::v7::Gelu>(in.get_node()))
                        res[in.get_node()->get_friendly_name()] = get_device_name();
                if (u.kind == OVFCC_FUSED_GLU)
                    mark_results_of(u.root);
            }
        }
        for (const auto& m : g.moes) {
            for (int c = 0; c < m.n_chain; ++c)
                mark(m.chain[c]);
            for (const ovfcc_gather_fold* f : {&m.gate, &m.up, &m.down}) {
                for (int c = 0; c < f->n_chain; ++c)
                    mark(f->chain[c]);
                mark(f->root);
                if (g.ops[(size_t)f->root]->get_input_size() > 3)
                    mark(g.nodes[(size_t)f->root].inputs[3]);  // the empty bias constant
            }
            for (int id : {m.hidden_states, m.routing, m.indices})
                if (g.nodes[(size_t)id].op == OVFCC_OP_PARAMETER)
                    mark(id);
            mark_results_of(m.root);
        }
        for (const auto& b : g.grouped) {
            const ovfcc_gather_fold& f = b.fold;
            for (int c = 0; c < f.n_chain; ++c)
                mark(f.chain[c]);
            mark(f.root);
            if (b.gather && g.ops[(size_t)f.root]->get_input_size() > 3)
                mark(g.nodes[(size_t)f.root].inputs[3]);  // the bias constant, empty or not
            for (int id : {f.activations, f.indices})
                if (id >= 0 && g.nodes[(size_t)id].op == OVFCC_OP_PARAMETER)
                    mark(id);
            mark_results_of(f.root);
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
    // The Intel-GPU plugin's switch for the asymmetric form of that quantisation (ov::intel_gpu::
    // asym_dynamic_quantization, src/plugins/intel_gpu/include/intel_gpu/runtime/internal_properties.hpp:177), by name:
    // its header belongs to that plugin.
    static constexpr const char* kAsymDynamicQuantization = "GPU_ASYM_DYNAMIC_QUANTIZATION";
    bool m_dq_asym = false;
};

CompiledModel::CompiledModel(const std::shared_ptr<ov::Model>& model, const std::shared_ptr<const ov::IPlugin>& plugin,
                             ovfcc_ctx* ctx, bool profiling, int node_flags,
                             const std::vector<std::vector<uint8_t>>* blobs)
    : ov::ICompiledModel(model, plugin), m_model(model), m_graph(describe(model)), m_ctx(ctx), m_node_flags(node_flags),
      m_profiling(profiling) {
    const ModelGraph& g = m_graph;
    const auto& results = model->get_results();
    const auto& params = model->get_parameters();
    std::vector<bool> fed(results.size(), false);
    // the model outputs that read node `id`
    auto results_of = [&](int id) {
        std::vector<size_t> out;
        for (size_t r = 0; r < results.size(); ++r)
            if (results[r]->get_input_node_ptr(0) == g.ops[(size_t)id].get())
                out.push_back(r);
        return out;
    };
    auto create = [&](const ovfcc_fold& f) { return create_node(ctx, g, f, node_flags); };
    auto primitive = [](const ovfcc_weights* w, const ovfcc_fc_desc& d, const char* suffix) {
        return std::string(ovfcc_weights_is_tiled(w) ? "hip_tiled_w" : "hip_plain_w") +
               (d.w_type == OVFCC_U8 || d.w_type == OVFCC_I8 ? "8" : "4") + suffix;
    };
    auto start_launch = [&](const ovfcc_fold& f, int kind) {
        Launch l;
        l.kind = kind;
        l.K = f.desc.K;
        l.out_type = f.desc.out_type;
        OPENVINO_ASSERT(g.nodes[(size_t)f.activations].op == OVFCC_OP_PARAMETER, "MI355X: the activations of ",
                        g.ops[(size_t)f.matmul]->get_friendly_name(),
                        " do not come straight from a Parameter (use HETERO:MI355X,CPU for the rest of the graph)");
        for (size_t p = 0; p < params.size(); ++p)
            if (params[p].get() == g.ops[(size_t)f.activations].get())
                l.input_index = p;
        return l;
    };
    auto add_outputs = [&](Launch& l, int root, int64_t column, int64_t width) {
        const auto rs = results_of(root);
        OPENVINO_ASSERT(!rs.empty(), "MI355X: ", g.ops[(size_t)root]->get_friendly_name(),
                        " feeds no model output (use HETERO:MI355X,CPU for the rest of the graph)");
        for (size_t r : rs) {
            l.outputs.push_back({r, column, width});
            fed[r] = true;
        }
    };
    for (const auto& u : g.fused) {
        const ovfcc_fold& f0 = g.folds[(size_t)u.parts[0]];
        if (u.kind == OVFCC_FUSED_GLU || u.kind == OVFCC_FUSED_MLP) {
            // gate and up with their gated linear unit as one node; with the down projection behind it, one MLP node
            const bool mlp = u.kind == OVFCC_FUSED_MLP;
            const ovfcc_fold& last = g.folds[(size_t)u.parts[mlp ? 2 : 0]];
            Launch l = start_launch(f0, u.kind);
            l.N_out = last.desc.N;
            l.out_type = last.desc.out_type;
            l.name = g.ops[(size_t)u.root]->get_friendly_name();
            l.folds.assign(u.parts, u.parts + u.n_parts);
            add_outputs(l, u.root, 0, l.N_out);
            if (!blobs) {
                ovfcc_weights *gate = create(f0), *up = create(g.folds[(size_t)u.parts[1]]);
                int rc = ovfcc_weights_glu(gate, up, u.glu_type, &l.weights);
                ovfcc_weights_destroy(gate);
                ovfcc_weights_destroy(up);
                if (rc != OVFCC_OK)
                    throw_last("weights_glu");
                if (mlp) {
                    ovfcc_weights *unit = l.weights, *down = create(last);
                    l.weights = nullptr;
                    rc = ovfcc_weights_mlp(unit, down, &l.weights);
                    ovfcc_weights_destroy(unit);
                    ovfcc_weights_destroy(down);
                    if (rc != OVFCC_OK)
                        throw_last("weights_mlp");
                }
            }
            for (int k = 0; k < u.n_parts; ++k)
                l.original_names.push_back(g.ops[(size_t)g.folds[(size_t)u.parts[k]].matmul]->get_friendly_name());
            if (!mlp || last.root != last.matmul)
                l.original_names.push_back(l.name);
            m_launches.push_back(std::move(l));
            continue;
        }
        // horizontally fused siblings share a launch when the library can concatenate them (equal scalar
        // zero-points included); otherwise, like single nodes, each gets its own
        ovfcc_weights* fused_w = nullptr;
        std::vector<ovfcc_weights*> parts;
        if (!blobs)
            for (int k = 0; k < u.n_parts; ++k)
                parts.push_back(create(g.folds[(size_t)u.parts[k]]));
        bool together = u.kind == OVFCC_FUSED_CONCAT;
        if (together && !blobs)
            together = ovfcc_weights_concat(parts.data(), (int)parts.size(), &fused_w) == OVFCC_OK;
        if (together) {
            Launch l = start_launch(f0, OVFCC_FUSED_CONCAT);
            int64_t column = 0;
            for (int k = 0; k < u.n_parts; ++k) {
                const ovfcc_fold& f = g.folds[(size_t)u.parts[k]];
                add_outputs(l, f.root, column, f.desc.N);
                column += f.desc.N;
                l.folds.push_back(u.parts[k]);
                l.original_names.push_back(g.ops[(size_t)f.root]->get_friendly_name());
                l.name += (k ? "+" : "") + g.ops[(size_t)f.root]->get_friendly_name();
            }
            l.N_out = column;
            l.weights = fused_w;
            for (auto* w : parts)
                ovfcc_weights_destroy(w);
            m_launches.push_back(std::move(l));
        } else {
            for (int k = 0; k < u.n_parts; ++k) {
                const ovfcc_fold& f = g.folds[(size_t)u.parts[k]];
                Launch l = start_launch(f, OVFCC_FUSED_SINGLE);
                l.N_out = f.desc.N;
                l.name = g.ops[(size_t)f.root]->get_friendly_name();
                l.folds = {u.parts[k]};
                l.original_names.push_back(g.ops[(size_t)f.matmul]->get_friendly_name());
                if (f.root != f.matmul)
                    l.original_names.push_back(l.name);
                add_outputs(l, f.root, 0, l.N_out);
                l.weights = blobs ? nullptr : parts[(size_t)k];
                m_launches.push_back(std::move(l));
            }
        }
    }
    for (const auto& m : g.moes) {
        OPENVINO_ASSERT(!blobs, "MI355X: a model with expert blocks has no blob form");
        MoeLaunch l;
        auto param_index = [&](int id, const char* what) {
            OPENVINO_ASSERT(g.nodes[(size_t)id].op == OVFCC_OP_PARAMETER, "MI355X: the ", what, " of ",
                            g.ops[(size_t)m.root]->get_friendly_name(),
                            " do not come straight from a Parameter (use HETERO:MI355X,CPU for the rest of the graph)");
            for (size_t p = 0; p < params.size(); ++p)
                if (params[p].get() == g.ops[(size_t)id].get())
                    return p;
            return (size_t)0;
        };
        l.hidden_index = param_index(m.hidden_states, "hidden states");
        l.routing_index = param_index(m.routing, "routing weights");
        l.indices_index = param_index(m.indices, "expert indices");
        const auto rs = results_of(m.root);
        OPENVINO_ASSERT(rs.size() == 1, "MI355X: an expert block must feed exactly one model output");
        l.result_index = rs[0];
        fed[rs[0]] = true;
        l.H = m.gate.desc.K;
        l.top_k = m.gate.top_k;
        OPENVINO_ASSERT(l.top_k > 0, "MI355X: the number of experts per token must be static");
        l.out_type = m.down.desc.out_type;
        l.name = g.ops[(size_t)m.root]->get_friendly_name();
        for (const ovfcc_gather_fold* f : {&m.gate, &m.up, &m.down})
            l.original_names.push_back(g.ops[(size_t)f->root]->get_friendly_name());
        l.original_names.push_back(l.name);
        for (int e = 0; e < m.gate.n_experts; ++e) {
            ovfcc_weights *gate = create_expert(ctx, g, m.gate, e, node_flags), *up = create_expert(ctx, g, m.up, e, node_flags);
            ovfcc_weights* gu = nullptr;
            const int rc = ovfcc_weights_glu(gate, up, m.glu_type, &gu);
            ovfcc_weights_destroy(gate);
            ovfcc_weights_destroy(up);
            if (rc != OVFCC_OK)
                throw_last("weights_glu (expert)");
            l.gate_up.push_back(gu);
            l.down.push_back(create_expert(ctx, g, m.down, e, node_flags));
        }
        m_moes.push_back(std::move(l));
    }
    for (const auto& b : g.grouped) {
        const ovfcc_gather_fold& f = b.fold;
        OPENVINO_ASSERT(!blobs, "MI355X: a model with grouped matrix products has no blob form");
        GroupedLaunch l;
        l.gather = b.gather;
        l.name = g.ops[(size_t)f.root]->get_friendly_name();
        auto param_index = [&](int id, const char* what) {
            OPENVINO_ASSERT(g.nodes[(size_t)id].op == OVFCC_OP_PARAMETER, "MI355X: the ", what, " of ", l.name,
                            " do not come straight from a Parameter (use HETERO:MI355X,CPU for the rest of the graph)");
            for (size_t p = 0; p < params.size(); ++p)
                if (params[p].get() == g.ops[(size_t)id].get())
                    return p;
            return (size_t)0;
        };
        l.a_index = param_index(f.activations, "activations");
        l.with_offsets = f.indices >= 0;
        if (l.with_offsets)
            l.offsets_index = param_index(f.indices, b.gather ? "expert indices" : "offsets");
        const auto rs = results_of(f.root);
        OPENVINO_ASSERT(rs.size() == 1, "MI355X: a grouped or routed matrix product must feed exactly one model output");
        l.result_index = rs[0];
        fed[rs[0]] = true;
        l.K = f.desc.K;
        l.N = f.desc.N;
        l.out_type = f.desc.out_type;
        l.original_names.push_back(l.name);
        for (int e = 0; e < f.n_experts; ++e)
            l.groups.push_back(create_expert(ctx, g, f, e, node_flags));
        m_grouped.push_back(std::move(l));
    }
    for (size_t r = 0; r < results.size(); ++r)
        OPENVINO_ASSERT(fed[r], "MI355X: result ", results[r]->get_friendly_name(),
                        " is not produced by a weight-compressed FullyConnected (use HETERO:MI355X,CPU for the rest "
                        "of the graph)");
    if (blobs) {
        // the cached device images, one per launch in this order; the library checks each against its own descriptor
        OPENVINO_ASSERT(blobs->size() == m_launches.size(), "MI355X: the imported blob holds ", blobs->size(),
                        " nodes, the model compiles to ", m_launches.size());
        for (size_t i = 0; i < m_launches.size(); ++i)
            if (ovfcc_weights_import(ctx, (*blobs)[i].data(), (*blobs)[i].size(), &m_launches[i].weights) != OVFCC_OK)
                throw_last("weights_import");
    }
    for (auto& l : m_launches)
        l.primitive = primitive(l.weights, g.folds[(size_t)l.folds[0]].desc,
                                l.kind == OVFCC_FUSED_MLP   ? "_mlp"
                                : l.kind == OVFCC_FUSED_GLU ? "_glu"
                                                            : (l.kind == OVFCC_FUSED_CONCAT ? "_fused" : ""));
    m_last_us = std::vector<std::atomic<double>>(m_launches.size() + m_moes.size() + m_grouped.size());
    for (auto& t : m_last_us)
        t.store(-1.0);
}

std::shared_ptr<ov::ISyncInferRequest> CompiledModel::create_sync_infer_request() const {
    return std::make_shared<InferRequest>(std::static_pointer_cast<const CompiledModel>(shared_from_this()));
}

}  // namespace ovfcc_plugin

static const ov::Version version = {"ovfcc-0.1", "openvino_mi355x_plugin"};
OV_DEFINE_PLUGIN_CREATE_FUNCTION(ovfcc_plugin::Plugin, version)
