// computation layer of the host mirror (see rg_mirror/computation.h).
#include "rg_mirror/computation.h"
#include "rg_mirror/hip_kernels.h"
#include <unordered_map>

namespace refactor::computation {

    kernel::CollectorBox Operator::candidateKernels(Target) const {
        TODO(detail::cat("Operator \"", name(), "\" lower to kernel not implemented"));
    }

#define RG_OPERATOR_IDS(T, NAME)                                          \
    size_t T::typeId() noexcept {                                         \
        static uint8_t ID = 1;                                            \
        return reinterpret_cast<size_t>(&ID);                             \
    }                                                                     \
    size_t T::opTypeId() const noexcept { return typeId(); }              \
    std::string_view T::name() const noexcept { return NAME; }

    RG_OPERATOR_IDS(RmsNormalization, "RmsNormalization")
    RG_OPERATOR_IDS(Softmax, "Softmax")
    RG_OPERATOR_IDS(MatMulInteger, "MatMulInteger")
    RG_OPERATOR_IDS(DequantizeLinear, "DequantizeLinear")
    RG_OPERATOR_IDS(DynamicQuantizeLinear, "DynamicQuantizeLinear")
    RG_OPERATOR_IDS(Cast, "Cast")
    RG_OPERATOR_IDS(MatMul, "MatMul")
    RG_OPERATOR_IDS(Attention, "Attention")
    RG_OPERATOR_IDS(RotaryEmbedding, "RotaryEmbedding")
    RG_OPERATOR_IDS(Transpose, "Transpose")
    RG_OPERATOR_IDS(Split, "Split")
    RG_OPERATOR_IDS(Concat, "Concat")
    RG_OPERATOR_IDS(Expand, "Expand")
    RG_OPERATOR_IDS(Where, "Where")
    RG_OPERATOR_IDS(Identity, "Identity")
    RG_OPERATOR_IDS(Reshape, "Reshape")
#undef RG_OPERATOR_IDS

    kernel::CollectorBox RmsNormalization::candidateKernels(Target target) const {
        return std::make_unique<kernel::RmsNormalizationCollector>(target, epsilon);
    }
    std::string RmsNormalization::serialize() const { return detail::cat(name(), '(', epsilon, ')'); }

    kernel::CollectorBox Softmax::candidateKernels(Target target) const {
        return std::make_unique<kernel::SoftmaxCollector>(target, axis, causal);
    }
    std::string Softmax::serialize() const {
        return detail::cat(name(), '(', axis, '/', rank, causal ? ", causal)" : ")");
    }

    kernel::CollectorBox MatMulInteger::candidateKernels(Target target) const {
        return std::make_unique<kernel::MatMulIntegerCollector>(target);
    }
    kernel::CollectorBox DequantizeLinear::candidateKernels(Target target) const {
        return std::make_unique<kernel::DequantizeLinearCollector>(target, axis);
    }
    kernel::CollectorBox DynamicQuantizeLinear::candidateKernels(Target target) const {
        return std::make_unique<kernel::DynamicQuantizeLinearCollector>(target);
    }
    kernel::CollectorBox Cast::candidateKernels(Target target) const {
        return std::make_unique<kernel::CastCollector>(target);
    }

    kernel::CollectorBox MatMul::candidateKernels(Target target) const {
        return std::make_unique<kernel::MatMulCollector>(target, alpha, beta, transA, transB);
    }
    std::string MatMul::serialize() const {
        return detail::cat(name(), '(', alpha, ", ", beta, ", ", transA ? 'T' : 'N', ", ", transB ? 'T' : 'N', ')');
    }

    kernel::CollectorBox Attention::candidateKernels(Target target) const {
        return std::make_unique<kernel::AttentionCollector>(target, maxSeqLen);
    }
    std::string Attention::serialize() const { return detail::cat(name(), '(', maxSeqLen, ')'); }

    kernel::CollectorBox Transpose::candidateKernels(Target target) const {
        return std::make_unique<kernel::TransposeCollector>(target, perm);
    }
    std::string Transpose::serialize() const {
        std::string s(name());
        s += "([";
        for (auto p : perm) s += ' ' + std::to_string(p);
        return s + " ])";
    }

    kernel::CollectorBox Split::candidateKernels(Target target) const {
        return std::make_unique<kernel::SplitCollector>(target, axis);
    }
    std::string Split::serialize() const { return detail::cat(name(), '(', axis, ')'); }
    kernel::CollectorBox Concat::candidateKernels(Target target) const {
        return std::make_unique<kernel::ConcatCollector>(target, axis);
    }
    std::string Concat::serialize() const { return detail::cat(name(), '(', axis, ')'); }
    kernel::CollectorBox Expand::candidateKernels(Target target) const {
        return std::make_unique<kernel::ExpandCollector>(target);
    }
    kernel::CollectorBox Where::candidateKernels(Target target) const {
        return std::make_unique<kernel::WhereCollector>(target);
    }

    kernel::CollectorBox RotaryEmbedding::candidateKernels(Target target) const {
        return std::make_unique<kernel::RotaryEmbeddingCollector>(target, theta);
    }
    std::string RotaryEmbedding::serialize() const { return detail::cat(name(), '(', theta, ')'); }

    // RmsNormalizationHip (float) -> DynamicQuantizeLinearHip  ==>  RmsNormalizationQuantizeHip, which keeps the
    // normalised tensor as its first output (it may have further readers) and takes over the three outputs of the
    // quantising node.  Rebuilt from keys like the fusion below.
    struct Lowered {
        graph_topo::GraphTopo topology;
        std::vector<kernel::Node> nodes;
        std::vector<kernel::Edge> edges;
    };
    static Lowered fuseQuantize(Lowered g) {
        using kernel::DynamicQuantizeLinearHip;
        using kernel::RmsNormalizationHip;
        auto &[topology, nodes, edges] = g;
        std::vector<count_t> producer(edges.size(), count_t(-1));
        for (auto [idx, inputs, outputs] : topology)
            for (auto e : outputs) producer[e] = idx;
        std::unordered_map<count_t, count_t> fusedInto;// consumer node -> producer node
        std::unordered_map<count_t, count_t> consumerOf;// producer node -> consumer node
        for (auto [idx, inputs, outputs] : topology) {
            auto const &k = nodes[idx].kernel;
            if (!k || !k->is<DynamicQuantizeLinearHip>() || inputs.size() != 1 || outputs.size() != 3) continue;
            auto const p = producer[inputs[0]];
            if (p == count_t(-1) || consumerOf.count(p) || !nodes[p].kernel || !nodes[p].kernel->is<RmsNormalizationHip>()) continue;
            auto const &rn = static_cast<RmsNormalizationHip const &>(*nodes[p].kernel);
            if (rn.dataType != DataType::F32 || topology.node(p).outputs.size() != 1) continue;
            auto fused = kernel::RmsNormalizationQuantizeHip::build(rn.epsilon, rn.blockCount, rn.blockSize);
            if (!fused) continue;
            nodes[p].kernel = std::move(fused);
            nodes[p].name += "+" + nodes[idx].name;
            fusedInto.emplace(idx, p);
            consumerOf.emplace(p, idx);
        }
        if (fusedInto.empty()) return g;
        graph_topo::Builder<count_t, kernel::Node, count_t, kernel::Edge> builder;
        for (auto [idx, inputs, outputs] : topology) {
            if (fusedInto.count(idx)) continue;
            graph_topo::BuilderNode<count_t> n{{inputs.begin(), inputs.end()}, {outputs.begin(), outputs.end()}};
            if (auto it = consumerOf.find(idx); it != consumerOf.end()) {
                auto const consumer = topology.node(it->second);
                n.outputs.insert(n.outputs.end(), consumer.outputs.begin(), consumer.outputs.end());
            }
            builder.topology.emplace(idx, std::move(n));
            builder.nodes.emplace(idx, std::move(nodes[idx]));
        }
        for (auto e : topology.globalInputs()) builder.globalInputs.push_back(e);
        for (auto e : topology.globalOutputs()) builder.globalOutputs.push_back(e);
        for (count_t e = 0; e < edges.size(); ++e) builder.edges.emplace(e, std::move(edges[e]));
        auto built = builder.build();
        return {std::move(built.topology), std::move(built.nodes), std::move(built.edges)};
    }

    // MatMulIntegerHip -> (int32 edge read once) -> DequantizeLinearHip  ==>  MatMulIntegerDequantizeHip.
    // The graph is rebuilt from keys (old indices) so that the edge numbering stays what GraphTopo
    // promises whatever the position of the scale's producer.
    static kernel::Graph fuseDequantize(graph_topo::GraphTopo topology, std::vector<kernel::Node> nodes,
                                        std::vector<kernel::Edge> edges) {
        using kernel::DequantizeLinearHip;
        using kernel::MatMulIntegerHip;
        std::vector<size_t> readers(edges.size(), 0);
        for (auto e : topology.connections()) ++readers[e];
        std::vector<count_t> producer(edges.size(), count_t(-1));
        for (auto [idx, inputs, outputs] : topology)
            for (auto e : outputs) producer[e] = idx;

        std::unordered_map<count_t, count_t> fusedInto;// consumer node -> producer node
        for (auto [idx, inputs, outputs] : topology) {
            auto const &k = nodes[idx].kernel;
            if (!k || !k->is<DequantizeLinearHip>() || inputs.size() != 2 || outputs.size() != 1) continue;
            auto const &dq = static_cast<DequantizeLinearHip const &>(*k);
            auto const x = inputs[0];
            auto const p = producer[x];
            if (p == count_t(-1) || readers[x] != 1 || !nodes[p].kernel || !nodes[p].kernel->is<MatMulIntegerHip>()) continue;
            auto const &mm = static_cast<MatMulIntegerHip const &>(*nodes[p].kernel);
            if (dq.from != DataType::I32 || dq.withZeroPoint) continue;
            if (dq.perAxis && (dq.inner != 1 || dq.axisLen != mm.info.n)) continue;
            auto const zeroPointInputs = static_cast<dim_t>(topology.node(p).inputs.size() - 2);
            auto fused = kernel::MatMulIntegerDequantizeHip::build(mm.info, zeroPointInputs, dq.perAxis);
            if (!fused) continue;
            nodes[p].kernel = std::move(fused);
            nodes[p].name += "+" + nodes[idx].name;
            fusedInto.emplace(idx, p);
        }
        if (fusedInto.empty()) return kernel::Graph(std::move(topology), std::move(nodes), std::move(edges));

        graph_topo::Builder<count_t, kernel::Node, count_t, kernel::Edge> builder;
        std::unordered_map<count_t, count_t> consumerOf;// producer node -> consumer node
        for (auto [c, p] : fusedInto) consumerOf.emplace(p, c);
        for (auto [idx, inputs, outputs] : topology) {
            if (fusedInto.count(idx)) continue;
            graph_topo::BuilderNode<count_t> n{{inputs.begin(), inputs.end()}, {outputs.begin(), outputs.end()}};
            if (auto it = consumerOf.find(idx); it != consumerOf.end()) {
                auto const consumer = topology.node(it->second);
                n.inputs.push_back(consumer.inputs[1]);// the scale
                n.outputs.assign(consumer.outputs.begin(), consumer.outputs.end());
            }
            builder.topology.emplace(idx, std::move(n));
            builder.nodes.emplace(idx, std::move(nodes[idx]));
        }
        for (auto e : topology.globalInputs()) builder.globalInputs.push_back(e);
        for (auto e : topology.globalOutputs()) builder.globalOutputs.push_back(e);
        for (count_t e = 0; e < edges.size(); ++e) builder.edges.emplace(e, std::move(edges[e]));
        auto g = builder.build();
        return kernel::Graph(std::move(g.topology), std::move(g.nodes), std::move(g.edges));
    }

    Graph::Graph(graph_topo::Graph<Node, Edge> internal) noexcept : _internal(std::move(internal)) {}
    Graph::Graph(graph_topo::GraphTopo topology, std::vector<Node> nodes, std::vector<Edge> edges) noexcept
        : _internal{std::move(topology), std::move(nodes), std::move(edges)} {}

    kernel::Graph Graph::lower(Target target) const {
        auto const &graph = _internal;
        std::vector<kernel::Node> nodes(graph.nodes.size());
        std::vector<kernel::Edge> edges(graph.edges.size());

        std::unordered_map<count_t, count_t> identities;// output edge -> the edge it stands for
        std::vector<std::string> noKernel;
        for (auto [idx, inputs, outputs] : graph.topology) {
            auto const &[op, name] = graph.nodes[idx];
            nodes[idx] = {nullptr, name};
            if (!op) continue;
            if (op->isIdentity()) {
                ASSERT(!inputs.empty() && outputs.size() == 1, "an identity has one output that renames its first input");
                // an input that is itself an identity's output was resolved when that node was visited
                auto source = inputs[0];
                if (auto it = identities.find(source); it != identities.end()) source = it->second;
                identities.emplace(outputs[0], source);
                continue;
            }
            kernel::TensorRefs inputs_, outputs_;
            for (auto e : inputs) inputs_.emplace_back(*graph.edges[e].tensor);
            for (auto e : outputs) outputs_.emplace_back(*graph.edges[e].tensor);
            auto candidates = op->candidateKernels(target)->filter(std::move(inputs_), std::move(outputs_));
            if (candidates.empty()) {
                noKernel.push_back(name);
            } else {
                nodes[idx].kernel = std::move(candidates.front());
            }
        }
        if (!noKernel.empty()) {
            std::string msg = "No kernel selected for ";
            for (auto const &n : noKernel) msg += '"' + n + "\" ";
            RUNTIME_ERROR(msg);
        }
        for (size_t i = 0; i < edges.size(); ++i) {
            auto const &[tensor, name] = graph.edges[i];
            if (!tensor || identities.count(static_cast<count_t>(i))) {
                edges[i] = {nullptr, 0, name};
            } else {
                edges[i] = {tensor->data, tensor->bytesSize(), name};
            }
        }
        auto topology = graph.topology;
        topology.reconnect(identities);
        if (target == Target::Amd) {
            auto g = fuseQuantize({std::move(topology), std::move(nodes), std::move(edges)});
            return fuseDequantize(std::move(g.topology), std::move(g.nodes), std::move(g.edges));
        }
        return kernel::Graph(std::move(topology), std::move(nodes), std::move(edges));
    }

}// namespace refactor::computation
