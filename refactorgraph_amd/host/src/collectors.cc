#include "rg_mirror/collectors.h"
#include "rg_mirror/hip_kernels.h"

// The reference's CPU kernels are not part of this build (the CPU target has no candidates here);
// the Amd case of every collector offers the gfx950 kernel.
namespace refactor::kernel {

    using Target = hardware::Device::Type;

#define ADD(PTR)                                  \
    if (auto ptr = (PTR); ptr) {                  \
        ans.emplace_back(std::move(ptr));         \
    }

    std::vector<KernelBox>
    RmsNormalizationCollector::filter(TensorRefs inputs, TensorRefs) const {
        std::vector<KernelBox> ans;
        switch (_target) {
            case Target::Cpu:
                break;
            case Target::Amd:
                ADD(RmsNormalizationHip::build(epsilon, inputs[0]))
                break;
            default:
                UNREACHABLEX(void, "Unknown target");
        }
        return ans;
    }

    std::vector<KernelBox>
    SoftmaxCollector::filter(TensorRefs inputs, TensorRefs) const {
        auto const &x = inputs[0].get();
        SoftmaxInfo info(x, axis);
        std::vector<KernelBox> ans;
        switch (_target) {
            case Target::Cpu:
                break;
            case Target::Amd: {
                dim_t causalRows = 0;
                if (causal) {
                    // the mask is defined over the last two axes
                    if (x.rank() < 2 || axis + 1 != static_cast<dim_t>(x.rank())) { break; }
                    causalRows = x.shape[x.rank() - 2];
                }
                ADD(SoftmaxHip::build(info, causalRows))
            } break;
            default:
                UNREACHABLEX(void, "Unknown target");
        }
        return ans;
    }

    std::vector<KernelBox>
    MatMulIntegerCollector::filter(TensorRefs inputs, TensorRefs) const {
        MatMulIntegerInfo info(inputs);
        std::vector<KernelBox> ans;
        switch (_target) {
            case Target::Cpu:
                break;
            case Target::Amd:
                ADD(MatMulIntegerHip::build(info))
                break;
            default:
                UNREACHABLEX(void, "Unknown target");
        }
        return ans;
    }

    std::vector<KernelBox>
    DequantizeLinearCollector::filter(TensorRefs inputs, TensorRefs outputs) const {
        std::vector<KernelBox> ans;
        switch (_target) {
            case Target::Cpu:
                break;
            case Target::Amd:
                ADD(DequantizeLinearHip::build(inputs, outputs[0], axis))
                break;
            default:
                UNREACHABLEX(void, "Unknown target");
        }
        return ans;
    }

    std::vector<KernelBox>
    DynamicQuantizeLinearCollector::filter(TensorRefs inputs, TensorRefs outputs) const {
        // src/04kernel/src/collectors/dynamic_quantize_linear.cc:12-33; the reference's kernels
        // take float input and produce uint8 only, which is checked here instead of assumed
        auto const &x = inputs[0].get();
        std::vector<KernelBox> ans;
        switch (_target) {
            case Target::Cpu:
                break;
            case Target::Amd:
                if (x.dataType == DataType::F32 && outputs.size() == 3 &&
                    outputs[0].get().dataType == DataType::U8 && outputs[1].get().dataType == DataType::F32 &&
                    outputs[2].get().dataType == DataType::U8) {
                    ADD(DynamicQuantizeLinearHip::build(x.elementsSize()))
                }
                break;
            default:
                UNREACHABLEX(void, "Unknown target");
        }
        return ans;
    }

    std::vector<KernelBox>
    MatMulCollector::filter(TensorRefs inputs, TensorRefs) const {
        // src/04kernel/src/collectors/mat_mul.cc:12-35
        auto const &a = inputs[0].get();
        auto const &b = inputs[1].get();
        auto info = inputs.size() == 3
                        ? MatMulInfo(a, b, std::make_optional(std::cref(inputs[2].get())), transA, transB, alpha, beta)
                        : MatMulInfo(a, b, std::nullopt, transA, transB, alpha, beta);
        std::vector<KernelBox> ans;
        switch (_target) {
            case Target::Cpu:
                break;
            case Target::Amd:
                ADD(MatMulHip::build(info))
                break;
            default:
                UNREACHABLEX(void, "Unknown target");
        }
        return ans;
    }

    std::vector<KernelBox>
    CastCollector::filter(TensorRefs inputs, TensorRefs outputs) const {
        // src/04kernel/src/collectors/cast.cc:10-33
        auto const &from = inputs[0].get();
        auto const &to = outputs[0].get();
        std::vector<KernelBox> ans;
        switch (_target) {
            case Target::Cpu:
                break;
            case Target::Amd:
                ADD(CastHip::build(from, to))
                break;
            default:
                UNREACHABLEX(void, "Unknown target");
        }
        return ans;
    }

    std::vector<KernelBox>
    TransposeCollector::filter(TensorRefs inputs, TensorRefs) const {
        auto const &data = inputs[0].get();
        std::vector<KernelBox> ans;
        switch (_target) {
            case Target::Cpu:
                break;
            case Target::Amd:
                if (perm.size() == data.shape.size()) { ADD(TransposeHip::build(TransposeInfo(data.dataType, data.shape, perm))) }
                break;
            default:
                UNREACHABLEX(void, "Unknown target");
        }
        return ans;
    }

    std::vector<KernelBox>
    SplitCollector::filter(TensorRefs, TensorRefs outputs) const {
        std::vector<KernelBox> ans;
        switch (_target) {
            case Target::Cpu:
                break;
            case Target::Amd:
                if (!outputs.empty() && axis < outputs[0].get().shape.size()) { ADD(SplitHip::build(SplitInfo(axis, outputs))) }
                break;
            default:
                UNREACHABLEX(void, "Unknown target");
        }
        return ans;
    }

    std::vector<KernelBox>
    ConcatCollector::filter(TensorRefs inputs, TensorRefs) const {
        std::vector<KernelBox> ans;
        switch (_target) {
            case Target::Cpu:
                break;
            case Target::Amd:
                if (!inputs.empty() && axis < inputs[0].get().shape.size()) { ADD(ConcatHip::build(SplitInfo(axis, inputs))) }
                break;
            default:
                UNREACHABLEX(void, "Unknown target");
        }
        return ans;
    }

    std::vector<KernelBox>
    ExpandCollector::filter(TensorRefs inputs, TensorRefs outputs) const {
        std::vector<KernelBox> ans;
        switch (_target) {
            case Target::Cpu:
                break;
            case Target::Amd: {
                // a collector reports "no kernel" for what it cannot take; ExpandInfo's constructor asserts, so the
                // shapes are checked here: right-aligned, every input extent is 1 or the output's
                if (inputs.empty() || outputs.empty()) { break; }
                auto const &in = inputs[0].get().shape;
                auto const &out = outputs[0].get().shape;
                if (in.size() > out.size() || inputs[0].get().dataType != outputs[0].get().dataType) { break; }
                bool broadcasts = true;
                for (size_t i = 0; i < in.size() && broadcasts; ++i) {
                    auto const i_ = in[in.size() - 1 - i], o_ = out[out.size() - 1 - i];
                    broadcasts = i_ == o_ || i_ == 1;
                }
                if (broadcasts) { ADD(ExpandHip::build(ExpandInfo(inputs[0], outputs[0]))) }
            } break;
            default:
                UNREACHABLEX(void, "Unknown target");
        }
        return ans;
    }

    std::vector<KernelBox>
    WhereCollector::filter(TensorRefs inputs, TensorRefs) const {
        std::vector<KernelBox> ans;
        switch (_target) {
            case Target::Cpu:
                break;
            case Target::Amd:
                ADD(WhereHip::build(inputs))
                break;
            default:
                UNREACHABLEX(void, "Unknown target");
        }
        return ans;
    }

    std::vector<KernelBox>
    AttentionCollector::filter(TensorRefs inputs, TensorRefs outputs) const {
        auto const &query = inputs[0].get();
        auto const &key = inputs[1].get();
        std::vector<KernelBox> ans;
        switch (_target) {
            case Target::Cpu:
                break;
            case Target::Amd: {
                AttentionHip::Info info{
                    .dataType = query.dataType,
                    .batch = query.shape[0],
                    .nHead = query.shape[1],
                    .nKVHead = key.shape[1],
                    .pastSeqLen = 0,
                    .seqLen = query.shape[2],
                    .cacheLen = outputs.size() == 1 ? 0 : outputs[1].get().shape[2],
                    .headDim = query.shape[3],
                    .resetCache = inputs.size() == 6,
                    .pastFromInput = inputs.size() > 3,
                    .pastCount = 0,
                };
                if (info.pastFromInput) {
                    // past_seq_len is operator input 3 (after query, key, value); it is read on the
                    // device at run time, a constant value is only recorded for the description
                    auto const &past = inputs[3].get();
                    info.pastCount = static_cast<dim_t>(past.elementsSize());
                    if (past.data) { info.pastSeqLen = static_cast<dim_t>(*past.data->get<int64_t>()); }
                }
                ADD(AttentionHip::build(info))
            } break;
            default:
                UNREACHABLEX(void, "Unknown target");
        }
        return ans;
    }

    std::vector<KernelBox>
    RotaryEmbeddingCollector::filter(TensorRefs inputs, TensorRefs) const {
        std::vector<KernelBox> ans;
        switch (_target) {
            case Target::Cpu:
                break;
            case Target::Amd:
                ADD(RotaryEmbeddingHip::build(theta, inputs[0], inputs[1]))
                break;
            default:
                UNREACHABLEX(void, "Unknown target");
        }
        return ans;
    }

}// namespace refactor::kernel
