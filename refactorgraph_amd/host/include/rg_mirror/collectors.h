// Per-operator kernel selectors of the hot path, each with a case for Device::Type::Amd.
// Constructor arguments and filter() contracts follow
// src/04kernel/include/kernel/collectors/{rms_normalization.h, softmax.h, mat_mul_integer.h,
// dequantize_linear.h, attention.h}; RotaryEmbeddingCollector has no counterpart there.
#pragma once

#include "rg_mirror/attributes.h"
#include "rg_mirror/kernel.h"

namespace refactor::kernel {

    struct RmsNormalizationCollector final : public InfoCollector {
        float epsilon;
        constexpr RmsNormalizationCollector(hardware::Device::Type target, float epsilon_) noexcept
            : InfoCollector(target), epsilon(epsilon_) {}
        std::vector<KernelBox> filter(TensorRefs inputs, TensorRefs outputs) const final;
    };

    struct SoftmaxCollector final : public InfoCollector {
        dim_t axis;
        bool causal;// extension: decoder mask over the last two axes (needs axis == rank - 1)
        constexpr SoftmaxCollector(hardware::Device::Type target, dim_t axis_, bool causal_ = false) noexcept
            : InfoCollector(target), axis(axis_), causal(causal_) {}
        std::vector<KernelBox> filter(TensorRefs inputs, TensorRefs outputs) const final;
    };

    struct MatMulIntegerCollector final : public InfoCollector {
        constexpr explicit MatMulIntegerCollector(hardware::Device::Type target) noexcept
            : InfoCollector(target) {}
        std::vector<KernelBox> filter(TensorRefs inputs, TensorRefs outputs) const final;
    };

    struct DequantizeLinearCollector final : public InfoCollector {
        int axis;// used only when the scale has more than one element (ONNX default 1)
        explicit DequantizeLinearCollector(hardware::Device::Type target, int axis_ = 1) noexcept
            : InfoCollector(target), axis(axis_) {}
        std::vector<KernelBox> filter(TensorRefs inputs, TensorRefs outputs) const final;
    };

    // inputs: x float; outputs: y uint8 like x, scale float [], zero point uint8 []
    // (src/04kernel/include/kernel/collectors/dynamic_quantize_linear.h:8-15)
    struct DynamicQuantizeLinearCollector final : public InfoCollector {
        constexpr explicit DynamicQuantizeLinearCollector(hardware::Device::Type target) noexcept
            : InfoCollector(target) {}
        std::vector<KernelBox> filter(TensorRefs inputs, TensorRefs outputs) const final;
    };

    // inputs: A, B [, C]; outputs: Y (src/04kernel/include/kernel/collectors/mat_mul.h:8-18)
    struct MatMulCollector final : public InfoCollector {
        float alpha, beta;
        bool transA, transB;
        constexpr MatMulCollector(hardware::Device::Type target, float alpha_, float beta_, bool transA_,
                                  bool transB_) noexcept
            : InfoCollector(target), alpha(alpha_), beta(beta_), transA(transA_), transB(transB_) {}
        std::vector<KernelBox> filter(TensorRefs inputs, TensorRefs outputs) const final;
    };

    // inputs: x; outputs: y of the requested type, same shape
    // (src/04kernel/include/kernel/collectors/cast.h:8-14)
    struct CastCollector final : public InfoCollector {
        constexpr explicit CastCollector(hardware::Device::Type target) noexcept
            : InfoCollector(target) {}
        std::vector<KernelBox> filter(TensorRefs inputs, TensorRefs outputs) const final;
    };

    // inputs: data; outputs: data with its dimensions permuted
    // (src/04kernel/include/kernel/collectors/transpose.h, src/04kernel/src/collectors/transpose.cc:7-35)
    struct TransposeCollector final : public InfoCollector {
        Permutation perm;
        TransposeCollector(hardware::Device::Type target, Permutation perm_) noexcept
            : InfoCollector(target), perm(std::move(perm_)) {}
        std::vector<KernelBox> filter(TensorRefs inputs, TensorRefs outputs) const final;
    };

    // inputs: data; outputs: its parts along `axis` (src/04kernel/include/kernel/collectors/split.h:8-16)
    struct SplitCollector final : public InfoCollector {
        dim_t axis;
        constexpr SplitCollector(hardware::Device::Type target, dim_t axis_) noexcept
            : InfoCollector(target), axis(axis_) {}
        std::vector<KernelBox> filter(TensorRefs inputs, TensorRefs outputs) const final;
    };

    // inputs: the parts; outputs: them joined along `axis` (src/04kernel/include/kernel/collectors/concat.h:8-16)
    struct ConcatCollector final : public InfoCollector {
        dim_t axis;
        constexpr ConcatCollector(hardware::Device::Type target, dim_t axis_) noexcept
            : InfoCollector(target), axis(axis_) {}
        std::vector<KernelBox> filter(TensorRefs inputs, TensorRefs outputs) const final;
    };

    // inputs: data; outputs: data broadcast to the output's shape (src/04kernel/include/kernel/collectors/expand.h)
    struct ExpandCollector final : public InfoCollector {
        constexpr explicit ExpandCollector(hardware::Device::Type target) noexcept : InfoCollector(target) {}
        std::vector<KernelBox> filter(TensorRefs inputs, TensorRefs outputs) const final;
    };

    // inputs: condition (Bool), x, y; outputs: the selection, broadcast (src/04kernel/include/kernel/collectors/where.h)
    struct WhereCollector final : public InfoCollector {
        constexpr explicit WhereCollector(hardware::Device::Type target) noexcept : InfoCollector(target) {}
        std::vector<KernelBox> filter(TensorRefs inputs, TensorRefs outputs) const final;
    };

    // inputs: query, key, value [, past_seq_len [, k_cache, v_cache]]; outputs: output
    // [, k_cache, v_cache] (src/08-01llm/README.md:29-63).
    struct AttentionCollector final : public InfoCollector {
        dim_t maxSeqLen;
        AttentionCollector(hardware::Device::Type target, dim_t maxSeqLen_) noexcept
            : InfoCollector(target), maxSeqLen(maxSeqLen_) {}
        std::vector<KernelBox> filter(TensorRefs inputs, TensorRefs outputs) const final;
    };

    // inputs: x [batch, seq, heads, dim], positions int64 [batch, seq] or [seq]; outputs: y like x
    struct RotaryEmbeddingCollector final : public InfoCollector {
        float theta;
        constexpr RotaryEmbeddingCollector(hardware::Device::Type target, float theta_) noexcept
            : InfoCollector(target), theta(theta_) {}
        std::vector<KernelBox> filter(TensorRefs inputs, TensorRefs outputs) const final;
    };

}// namespace refactor::kernel
