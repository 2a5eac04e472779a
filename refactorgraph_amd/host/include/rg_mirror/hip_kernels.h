// The gfx950 kernels behind the collectors: one Kernel subclass per operator, each lowering to
// a Routine that calls one rg_hip_* launcher of include/rg_hip.h on the default stream.
// build() is noexcept and returns nullptr when the kernel does not apply, as the reference's
// CUDA kernels do (e.g. src/04kernel/src/kernels/softmax/cuda_kernel.cc:9-17).
#pragma once

#include "rg_mirror/attributes.h"

namespace refactor::kernel {

    struct RmsNormalizationHip final : public Kernel {
        float epsilon;
        DataType dataType;
        dim_t blockCount, blockSize;

        RmsNormalizationHip(float, DataType, dim_t, dim_t) noexcept;
        static KernelBox build(float epsilon, Tensor const &x) noexcept;
        static size_t typeId() noexcept;
        size_t kernelTypeId() const noexcept final;
        std::string_view description() const noexcept final;
        RoutineWorkspace lower(Resources &) const final;
    };

    // RmsNormalization (float) whose output a DynamicQuantizeLinear reads: both operators' outputs, bit for
    // bit, from two launches instead of three (the normalising launch leaves its output's extrema per
    // workgroup, so its output is read once).  No counterpart in the reference; computation::Graph::lower puts
    // it in place of such a pair.  Inputs: x, w.  Outputs: y (float), yq (uint8), scale, zero point.
    struct RmsNormalizationQuantizeHip final : public Kernel {
        float epsilon;
        dim_t blockCount, blockSize;

        RmsNormalizationQuantizeHip(float, dim_t, dim_t) noexcept;
        static KernelBox build(float epsilon, dim_t blockCount, dim_t blockSize) noexcept;
        static size_t typeId() noexcept;
        size_t kernelTypeId() const noexcept final;
        std::string_view description() const noexcept final;
        RoutineWorkspace lower(Resources &) const final;
    };

    struct SoftmaxHip final : public Kernel {
        SoftmaxInfo info;
        dim_t causalRows;// 0: plain softmax

        SoftmaxHip(SoftmaxInfo, dim_t causalRows) noexcept;
        static KernelBox build(SoftmaxInfo, dim_t causalRows = 0) noexcept;
        static size_t typeId() noexcept;
        size_t kernelTypeId() const noexcept final;
        std::string_view description() const noexcept final;
        RoutineWorkspace lower(Resources &) const final;
    };

    struct MatMulIntegerHip final : public Kernel {
        MatMulIntegerInfo info;

        explicit MatMulIntegerHip(MatMulIntegerInfo) noexcept;
        static KernelBox build(MatMulIntegerInfo) noexcept;
        static size_t typeId() noexcept;
        size_t kernelTypeId() const noexcept final;
        std::string_view description() const noexcept final;
        RoutineWorkspace lower(Resources &) const final;
    };

    // MatMulInteger whose result leaves as float(sum) * scale: what MatMulIntegerHip followed by a
    // DequantizeLinearHip without zero point (scale per tensor, or per index of the last axis)
    // computes, bit for bit, in one kernel and without the int32 tensor.  No counterpart in the
    // reference; computation::Graph::lower puts it in place of such a pair.
    // Inputs: A, B [, a_zero_point [, b_zero_point]], scale.  Output: float [.., m, n].
    struct MatMulIntegerDequantizeHip final : public Kernel {
        MatMulIntegerInfo info;
        dim_t zeroPointInputs;// how many of the optional inputs 2, 3 the operator has
        bool perColumn;

        MatMulIntegerDequantizeHip(MatMulIntegerInfo, dim_t, bool) noexcept;
        static KernelBox build(MatMulIntegerInfo, dim_t zeroPointInputs, bool perColumn) noexcept;
        static size_t typeId() noexcept;
        size_t kernelTypeId() const noexcept final;
        std::string_view description() const noexcept final;
        RoutineWorkspace lower(Resources &) const final;
    };

    struct DequantizeLinearHip final : public Kernel {
        DataType from;
        size_t outer, axisLen, inner;
        bool perAxis, withZeroPoint;

        DequantizeLinearHip(DataType, size_t, size_t, size_t, bool, bool) noexcept;
        // scale with one element: the reference's per-tensor path; with more: one per index of `axis`
        static KernelBox build(TensorRefs const &inputs, Tensor const &output, int axis = 1) noexcept;
        static size_t typeId() noexcept;
        size_t kernelTypeId() const noexcept final;
        std::string_view description() const noexcept final;
        RoutineWorkspace lower(Resources &) const final;
    };

    // mirrors DynamicQuantizeLinearCuda
    // (src/04kernel/src/kernels/dynamic_quantize_linear/cuda_kernel.hh:8-21): float -> uint8
    struct DynamicQuantizeLinearHip final : public Kernel {
        size_t size;

        explicit DynamicQuantizeLinearHip(decltype(size)) noexcept;
        static KernelBox build(decltype(size)) noexcept;
        static size_t typeId() noexcept;
        size_t kernelTypeId() const noexcept final;
        std::string_view description() const noexcept final;
        RoutineWorkspace lower(Resources &) const final;
    };

    // mirrors MatMulCublas (src/04kernel/src/kernels/mat_mul/cublas_kernel.hh): F32, F64, FP16 and,
    // beyond the reference, BF16; no library handle in the resources, the kernels are this library's
    struct MatMulHip final : public Kernel {
        MatMulInfo info;

        explicit MatMulHip(decltype(info)) noexcept;
        static KernelBox build(decltype(info)) noexcept;
        static size_t typeId() noexcept;
        size_t kernelTypeId() const noexcept final;
        std::string_view description() const noexcept final;
        RoutineWorkspace lower(Resources &) const final;
    };

    // mirrors CastCuda (src/04kernel/src/kernels/cast/cuda_kernel.hh:9-23); no run-time compilation:
    // every type pair is a precompiled kernel of the device library
    struct CastHip final : public Kernel {
        DataType from, to;
        size_t size;

        CastHip(decltype(from), decltype(to), decltype(size)) noexcept;
        static KernelBox build(Tensor const &, Tensor const &) noexcept;
        static size_t typeId() noexcept;
        size_t kernelTypeId() const noexcept final;
        std::string_view description() const noexcept final;
        RoutineWorkspace lower(Resources &) const final;
    };

    // mirrors TransposeCuda (src/04kernel/src/kernels/transpose/cuda_kernel.hh)
    struct TransposeHip final : public Kernel {
        TransposeInfo info;

        explicit TransposeHip(TransposeInfo) noexcept;
        static KernelBox build(TransposeInfo) noexcept;
        static size_t typeId() noexcept;
        size_t kernelTypeId() const noexcept final;
        std::string_view description() const noexcept final;
        RoutineWorkspace lower(Resources &) const final;
    };

    // mirror SplitCuda and ConcatCuda (src/04kernel/src/kernels/{split,concat}/cuda_kernel.hh): outputs of
    // Split / inputs of Concat are the parts of the digest, in order
    struct SplitHip final : public Kernel {
        SplitInfo info;
        explicit SplitHip(SplitInfo) noexcept;
        static KernelBox build(SplitInfo) noexcept;
        static size_t typeId() noexcept;
        size_t kernelTypeId() const noexcept final;
        std::string_view description() const noexcept final;
        RoutineWorkspace lower(Resources &) const final;
    };
    struct ConcatHip final : public Kernel {
        SplitInfo info;
        explicit ConcatHip(SplitInfo) noexcept;
        static KernelBox build(SplitInfo) noexcept;
        static size_t typeId() noexcept;
        size_t kernelTypeId() const noexcept final;
        std::string_view description() const noexcept final;
        RoutineWorkspace lower(Resources &) const final;
    };

    // mirrors ExpandCuda (src/04kernel/src/kernels/expand/cuda_kernel.hh); the stride table travels in
    // the kernel arguments, nothing is uploaded at lower() time
    struct ExpandHip final : public Kernel {
        ExpandInfo info;
        explicit ExpandHip(ExpandInfo) noexcept;
        static KernelBox build(ExpandInfo) noexcept;
        static size_t typeId() noexcept;
        size_t kernelTypeId() const noexcept final;
        std::string_view description() const noexcept final;
        RoutineWorkspace lower(Resources &) const final;
    };

    // mirrors WhereCuda (src/04kernel/src/kernels/where/where_cuda.hh): inputs condition (Bool), x, y
    struct WhereHip final : public Kernel {
        DataType dataType;
        Broadcaster broadcaster;
        WhereHip(DataType, Broadcaster) noexcept;
        static KernelBox build(TensorRefs const &inputs) noexcept;
        static size_t typeId() noexcept;
        size_t kernelTypeId() const noexcept final;
        std::string_view description() const noexcept final;
        RoutineWorkspace lower(Resources &) const final;
    };

    struct AttentionHip final : public Kernel {
        // the reference's parameter block (src/04kernel/src/kernels/attention/cuda_kernel.hh:10-14)
        // plus what it leaves to the run time: where past_seq_len comes from
        struct Info {
            DataType dataType;
            dim_t batch, nHead, nKVHead, pastSeqLen, seqLen, cacheLen, headDim;
            bool resetCache;   // 6-input form: copy the input caches into the output caches first
            bool pastFromInput;// inputs[3] holds past_seq_len (read on the device at run time)
            dim_t pastCount;   // its element count: 1 (reference contract) or batch (per row)
        } info;

        explicit AttentionHip(Info) noexcept;
        static KernelBox build(Info) noexcept;
        static size_t typeId() noexcept;
        size_t kernelTypeId() const noexcept final;
        std::string_view description() const noexcept final;
        RoutineWorkspace lower(Resources &) const final;
    };

    struct RotaryEmbeddingHip final : public Kernel {
        DataType dataType;
        dim_t batch, seq, heads, dim;
        bool posPerBatch;
        float theta;

        RotaryEmbeddingHip(DataType, dim_t, dim_t, dim_t, dim_t, bool, float) noexcept;
        static KernelBox build(float theta, Tensor const &x, Tensor const &pos) noexcept;
        static size_t typeId() noexcept;
        size_t kernelTypeId() const noexcept final;
        std::string_view description() const noexcept final;
        RoutineWorkspace lower(Resources &) const final;
    };

    // Per-stream device state kept in Resources, in the way the reference keeps its library
    // handles there (src/04kernel/src/utilities/cuda/cublas_context.cu:18-31): the zeroed ticket
    // counters that let the attention kernel finish in a single launch.
    class HipAttentionState final : public runtime::Resource {
        void *_counters;

    public:
        HipAttentionState();
        ~HipAttentionState();
        HipAttentionState(HipAttentionState const &) = delete;
        static size_t typeId() noexcept;
        static runtime::ResourceBox build();
        size_t resourceTypeId() const noexcept final;
        std::string_view description() const noexcept final;
        void *counters() const noexcept { return _counters; }
    };

}// namespace refactor::kernel
