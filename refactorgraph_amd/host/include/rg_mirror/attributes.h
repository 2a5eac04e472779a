// Shape pre-digestion used by the hot-path collectors.  Semantics follow
// src/04kernel/src/attributes/{softmax_info.cc:6-13, broadcaster.cc:17-105,
// mat_mul_integer_info.cc:5-40, mat_mul_info.cc:5-43, transpose_info.cc:7-126, split_info.cc:5-24,
// expand_info.cc:14-60}.
#pragma once

#include <optional>

#include "rg_mirror/kernel.h"

namespace refactor::kernel {

    // softmax along `axis` of a tensor viewed as [pre, mid, post]
    struct SoftmaxInfo {
        dim_t pre, mid, post;
        DataType type;
        SoftmaxInfo(Tensor const &data, dim_t axis) noexcept;
    };

    // Multidirectional (numpy-style) broadcasting of leading batch dimensions.  Dimensions where
    // every input is 1 are dropped and neighbouring dimensions with the same broadcast pattern
    // are merged; `strides` holds, per merged dimension, one stride per input followed by the
    // output stride.  An empty `strides` means no input is broadcast: locate(k) = k.
    struct Broadcaster {
        std::vector<dim_t> strides;
        dim_t outputsCount, inputsCount;

        explicit Broadcaster(std::vector<std::vector<dim_t>> const &inputShapes);
        explicit Broadcaster(TensorRefs const &inputs);
        void locate(dim_t k, dim_t ans[]) const noexcept;
        bool needBroadcast() const noexcept { return !strides.empty(); }
    };

    // Mirrors src/04kernel/include/kernel/attributes/mat_mul_info.h:9-24.  The reference keeps an
    // ExpandInfo for the bias and expands it into Y before the product; here the bias is read through
    // strides inside the product's epilogue, so the info carries the three strides instead
    // (elements; 0 broadcasts).  `biasSupported` is false for a bias whose batch dimensions are
    // neither all 1 nor the output's (such a bias needs the Expand kernel, which is not built).
    struct MatMulInfo {
        DataType dataType;
        float alpha, beta;
        bool transA, transB;
        dim_t m, k, n;
        bool hasBias, biasSupported;
        size_t biasStrideBatch, biasStrideM, biasStrideN;
        // a bias whose batch dimensions are neither all 1 nor the output's is laid out over [batch..., m, n] first,
        // as the reference does with every bias (src/04kernel/src/kernels/mat_mul/cublas_kernel.cu:26-39):
        // its shape and the output's, for an ExpandInfo; empty when the strides above describe the bias
        std::vector<dim_t> biasExpandFrom, biasExpandTo;
        Broadcaster broadcaster;

        MatMulInfo(Tensor const &, Tensor const &, std::optional<std::reference_wrapper<Tensor const>>,
                   bool, bool, float, float);
        dim_t batch() const noexcept { return broadcaster.outputsCount; }
    };

    // Digest of a transposition (src/04kernel/include/kernel/attributes/transpose_info.h:9-29): the
    // output is blockCount blocks of blockSize bytes; output block i is input block locate(i).
    // Size-1 dimensions are dropped, dimensions that stay neighbours are merged, a last dimension
    // that stays last is folded into the block.  dims are in output order, slowest first.
    using Permutation = std::vector<dim_t>;
    struct TransposeInfo {
        struct Dimension {
            dim_t strideI, strideO;
        };
        std::vector<Dimension> dims;
        dim_t blockSize, blockCount;

        TransposeInfo(DataType, std::vector<dim_t> const &shape, Permutation const &);
        dim_t locate(dim_t) const noexcept;
    };

    // Digest of Split and Concat (src/04kernel/include/kernel/attributes/split_info.h:9-21): the joined
    // tensor is blockCount blocks of `sum` bytes, block i being one segment of every part in turn.
    struct SplitInfo {
        dim_t blockCount, sum;
        std::vector<dim_t> segments;
        SplitInfo(dim_t axis, TensorRefs const &parts);
    };

    // Digest of a one-directional broadcast (src/04kernel/include/kernel/attributes/expand_info.h:9-25):
    // the output is blockCount blocks of blockSize bytes; output block k is input block
    // sum over the strides of (rem / o) * i with rem %= o.  No strides: nothing is broadcast.
    struct ExpandInfo {
        struct Dim {
            dim_t i, o;
            bool operator==(Dim const &rhs) const noexcept { return i == rhs.i && o == rhs.o; }
        };
        std::vector<Dim> strides;
        dim_t blockCount, blockSize;
        ExpandInfo(DataType, std::vector<dim_t> const &input, std::vector<dim_t> const &output);
        ExpandInfo(Tensor const &input, Tensor const &output);
    };

    struct MatMulIntegerInfo {
        struct Input {
            bool withZeroPoint,// a zero-point tensor is present and not a constant of all zeros
                signed_,       // the zero point's dtype is I8 (the reference reads the operand so)
                scalar;        // one element; otherwise one per (batch, row) of the operand
            Input(TensorRefs const &, size_t i) noexcept;
        };
        Input a, b;
        dim_t m, k, n;
        Broadcaster broadcaster;

        explicit MatMulIntegerInfo(TensorRefs const &inputs) noexcept;
        dim_t batch() const noexcept { return broadcaster.outputsCount; }
    };

}// namespace refactor::kernel
