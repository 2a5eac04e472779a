// Shape pre-digestion used by the hot-path collectors.  Semantics follow
// src/04kernel/src/attributes/{softmax_info.cc:6-13, broadcaster.cc:17-105,
// mat_mul_integer_info.cc:5-40}.
#pragma once

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
