// computation layer of the host mirror, as far as the hot path needs it: operators that know their
// attributes and name the collector that finds kernels for a target, and the graph of such
// operators that lowers to a kernel::Graph.  Follows
// src/05computation/include/computation/{operator.h:6-47, graph.h:7-35} and
// src/05computation/src/graph.cc:17-78; operator classes as in
// src/05computation/include/computation/operators/{rms_normalization,softmax,mat_mul_integer,
// dequantize_linear,dynamic_quantize_linear,cast,mat_mul,transpose,attention,identity,reshape}.h.
// Differences: Attention has candidateKernels (the reference declares the operator without one, so
// a graph that contains it cannot be lowered there); RotaryEmbedding is new; Softmax carries the
// causal flag and DequantizeLinear the axis that the collectors of this build take; layout
// permutation and serialisation of whole graphs are not part of the path.
#pragma once

#include "rg_mirror/collectors.h"
#include "rg_mirror/graph.h"

namespace refactor::computation {
    using kernel::LayoutType;
    using kernel::Shape;
    using kernel::Tensor;
    using Target = hardware::Device::Type;

    class Operator {
    public:
        virtual ~Operator() = default;
        virtual size_t opTypeId() const = 0;
        virtual std::string_view name() const = 0;
        virtual bool isIdentity() const { return false; }
        // the base throws UnimplementError, like src/05computation/src/operator.cc
        virtual kernel::CollectorBox candidateKernels(Target) const;
        virtual std::string serialize() const { return std::string(name()); }

        template<class T, class... Args> bool is(Args &&...args) const noexcept {
            return this->opTypeId() == T::typeId(std::forward<Args>(args)...);
        }
    };
    using OpBox = std::unique_ptr<Operator>;

#define RG_OPERATOR_COMMON                      \
    static size_t typeId() noexcept;            \
    size_t opTypeId() const noexcept final;     \
    std::string_view name() const noexcept final;

    struct RmsNormalization final : public Operator {
        float epsilon;
        constexpr explicit RmsNormalization(float epsilon_) noexcept : epsilon(epsilon_) {}
        RG_OPERATOR_COMMON
        kernel::CollectorBox candidateKernels(Target) const final;
        std::string serialize() const final;
    };

    struct Softmax final : public Operator {
        uint32_t axis, rank;
        bool causal;
        constexpr Softmax(uint32_t axis_, uint32_t rank_, bool causal_ = false) noexcept
            : axis(axis_), rank(rank_), causal(causal_) {}
        RG_OPERATOR_COMMON
        kernel::CollectorBox candidateKernels(Target) const final;
        std::string serialize() const final;
    };

    struct MatMulInteger final : public Operator {
        RG_OPERATOR_COMMON
        kernel::CollectorBox candidateKernels(Target) const final;
    };

    struct DequantizeLinear final : public Operator {
        int axis;
        constexpr explicit DequantizeLinear(int axis_ = 1) noexcept : axis(axis_) {}
        RG_OPERATOR_COMMON
        kernel::CollectorBox candidateKernels(Target) const final;
    };

    struct DynamicQuantizeLinear final : public Operator {
        RG_OPERATOR_COMMON
        kernel::CollectorBox candidateKernels(Target) const final;
    };

    struct Cast final : public Operator {
        RG_OPERATOR_COMMON
        kernel::CollectorBox candidateKernels(Target) const final;
    };

    struct MatMul final : public Operator {
        float alpha, beta;
        bool transA, transB;
        constexpr MatMul(float alpha_, float beta_, bool transA_, bool transB_) noexcept
            : alpha(alpha_), beta(beta_), transA(transA_), transB(transB_) {}
        RG_OPERATOR_COMMON
        kernel::CollectorBox candidateKernels(Target) const final;
        std::string serialize() const final;
    };

    struct Attention final : public Operator {
        dim_t maxSeqLen;
        constexpr explicit Attention(dim_t maxSeqLen_) noexcept : maxSeqLen(maxSeqLen_) {}
        RG_OPERATOR_COMMON
        kernel::CollectorBox candidateKernels(Target) const final;
        std::string serialize() const final;
    };

    struct Transpose final : public Operator {
        kernel::Permutation perm;
        explicit Transpose(kernel::Permutation perm_) noexcept : perm(std::move(perm_)) {}
        RG_OPERATOR_COMMON
        kernel::CollectorBox candidateKernels(Target) const final;
        std::string serialize() const final;
    };

    // src/05computation/include/computation/operators/{split,concat,expand,where}.h
    struct Split final : public Operator {
        dim_t axis;
        constexpr explicit Split(dim_t axis_) noexcept : axis(axis_) {}
        RG_OPERATOR_COMMON
        kernel::CollectorBox candidateKernels(Target) const final;
        std::string serialize() const final;
    };
    struct Concat final : public Operator {
        dim_t axis;
        constexpr explicit Concat(dim_t axis_) noexcept : axis(axis_) {}
        RG_OPERATOR_COMMON
        kernel::CollectorBox candidateKernels(Target) const final;
        std::string serialize() const final;
    };
    struct Expand final : public Operator {
        RG_OPERATOR_COMMON
        kernel::CollectorBox candidateKernels(Target) const final;
    };
    struct Where final : public Operator {
        RG_OPERATOR_COMMON
        kernel::CollectorBox candidateKernels(Target) const final;
    };

    struct RotaryEmbedding final : public Operator {
        float theta;
        constexpr explicit RotaryEmbedding(float theta_) noexcept : theta(theta_) {}
        RG_OPERATOR_COMMON
        kernel::CollectorBox candidateKernels(Target) const final;
        std::string serialize() const final;
    };

    // The output is the first input under another name or shape: no kernel runs, readers of the
    // output are connected to the input when the graph is lowered.
    struct Identity final : public Operator {
        RG_OPERATOR_COMMON
        bool isIdentity() const noexcept final { return true; }
    };
    struct Reshape final : public Operator {
        RG_OPERATOR_COMMON
        bool isIdentity() const noexcept final { return true; }
    };

#undef RG_OPERATOR_COMMON

    struct Node {
        OpBox op;
        std::string name;
    };

    struct Edge {
        Arc<Tensor> tensor;
        std::string name;
    };

    class Graph {
        graph_topo::Graph<Node, Edge> _internal;

    public:
        explicit Graph(graph_topo::Graph<Node, Edge>) noexcept;
        Graph(graph_topo::GraphTopo, std::vector<Node>, std::vector<Edge>) noexcept;

        // First candidate of every operator's collector; operators without one are collected and
        // reported together ("No kernel selected for ...").  On the AMD target a MatMulInteger whose
        // result is read by one DequantizeLinear only (no zero point, scale per tensor or per index of
        // the last axis) and by nothing else becomes one MatMulIntegerDequantizeHip node: the
        // dequantising node and the int32 edge between the two are gone from the lowered graph.
        kernel::Graph lower(Target) const;
        graph_topo::Graph<Node, Edge> const &internal() const noexcept { return _internal; }
    };

}// namespace refactor::computation
