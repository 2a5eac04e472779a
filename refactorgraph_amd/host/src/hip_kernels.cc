#include "rg_mirror/hip_kernels.h"
#include "rg_mirror/stream.h"
#include "rg_hip.h"
#include <cmath>

// A failing launcher raises a RUNTIME_ERROR with the library's message; the reference's
// library-backed kernels abort instead (src/04kernel/src/utilities/cuda/cublas_context.hh:7-12),
// an exception keeps a host process that embeds the runtime alive.
#define HIP_CALL(CALL)                                                                                \
    if (auto status_ = (CALL); status_ != 0) {                                                        \
        RUNTIME_ERROR(::refactor::detail::cat("rg_hip failed on \"" #CALL "\" with \"",               \
                                              rg_hip_error_string(status_), "\" (", status_, ")"));   \
    }

namespace refactor::kernel {

    // the stream the routines of this Resources enqueue on: the default stream (like the reference's
    // routines) unless the runtime::Stream has put a HipStream there to record a graph
    static void *streamOf(Resources &res) noexcept {
        auto *s = res.fetch<runtime::HipStream>();
        return s ? s->handle() : nullptr;
    }

    template<class T> static size_t idOf() noexcept {
        static uint8_t ID = 1;
        return reinterpret_cast<size_t>(&ID);
    }

    // ------------------------------------------------------------------ RmsNormalization

    using RN = RmsNormalizationHip;
    RN::RmsNormalizationHip(float epsilon_, DataType dataType_, dim_t blockCount_, dim_t blockSize_) noexcept
        : Kernel(), epsilon(epsilon_), dataType(dataType_), blockCount(blockCount_), blockSize(blockSize_) {}

    KernelBox RN::build(float epsilon, Tensor const &x) noexcept {
        if (!x.dataType.isFloat() || x.shape.empty()) { return nullptr; }
        dim_t blockSize = x.shape.back(), blockCount = 1;
        for (size_t i = 0; i + 1 < x.shape.size(); ++i) { blockCount *= x.shape[i]; }
        return std::make_unique<RN>(epsilon, x.dataType, blockCount, blockSize);
    }
    size_t RN::typeId() noexcept { return idOf<RN>(); }
    size_t RN::kernelTypeId() const noexcept { return typeId(); }
    std::string_view RN::description() const noexcept { return "Performing rms normalization on AMD gfx950"; }
    RoutineWorkspace RN::lower(Resources &) const {
        return [epsilon = epsilon, code = static_cast<int>(dataType.internal), rows = blockCount, cols = blockSize]//
            (Resources &res, void *, void const *const *inputs, void *const *outputs) {
                HIP_CALL(rg_hip_rms_norm(outputs[0], inputs[0], inputs[1], rows, cols, epsilon, code, streamOf(res)));
            };
    }

    using RNQ = RmsNormalizationQuantizeHip;
    RNQ::RmsNormalizationQuantizeHip(float epsilon_, dim_t blockCount_, dim_t blockSize_) noexcept
        : Kernel(), epsilon(epsilon_), blockCount(blockCount_), blockSize(blockSize_) {}
    KernelBox RNQ::build(float epsilon, dim_t blockCount, dim_t blockSize) noexcept {
        if (rg_hip_rms_norm_quantize_workspace(blockCount, blockSize) == 0) { return nullptr; }
        return std::make_unique<RNQ>(epsilon, blockCount, blockSize);
    }
    size_t RNQ::typeId() noexcept { return idOf<RNQ>(); }
    size_t RNQ::kernelTypeId() const noexcept { return typeId(); }
    std::string_view RNQ::description() const noexcept {
        return "Performing rms normalization with dynamic quantization of its output on AMD gfx950";
    }
    RoutineWorkspace RNQ::lower(Resources &) const {
        auto const bytes = rg_hip_rms_norm_quantize_workspace(blockCount, blockSize);
        auto routine = [epsilon = epsilon, rows = blockCount, cols = blockSize, bytes]//
            (Resources &res, void *workspace, void const *const *inputs, void *const *outputs) {
                HIP_CALL(rg_hip_rms_norm_quantize(static_cast<uint8_t *>(outputs[1]), static_cast<float *>(outputs[2]),
                                                  static_cast<uint8_t *>(outputs[3]), static_cast<float *>(outputs[0]),
                                                  static_cast<float const *>(inputs[0]), static_cast<float const *>(inputs[1]),
                                                  rows, cols, epsilon, workspace, bytes, streamOf(res)));
            };
        return RoutineWorkspace(std::move(routine), bytes);
    }

    // ------------------------------------------------------------------ Softmax

    using SM = SoftmaxHip;
    SM::SoftmaxHip(SoftmaxInfo info_, dim_t causalRows_) noexcept : Kernel(), info(info_), causalRows(causalRows_) {}
    KernelBox SM::build(SoftmaxInfo info, dim_t causalRows) noexcept {
        if (!info.type.isFloat()) { return nullptr; }
        if (causalRows && (info.post != 1 || info.pre % causalRows != 0 || info.mid < causalRows)) { return nullptr; }
        return std::make_unique<SM>(info, causalRows);
    }
    size_t SM::typeId() noexcept { return idOf<SM>(); }
    size_t SM::kernelTypeId() const noexcept { return typeId(); }
    std::string_view SM::description() const noexcept { return "Performing Softmax on AMD gfx950"; }
    RoutineWorkspace SM::lower(Resources &) const {
        return [info = info, causalRows = causalRows](Resources &res, void *, void const *const *inputs, void *const *outputs) {
            HIP_CALL(rg_hip_softmax(outputs[0], inputs[0], info.pre, info.mid, info.post,
                                    static_cast<int>(info.type.internal), causalRows, streamOf(res)));
        };
    }

    // ------------------------------------------------------------------ MatMulInteger

    using MMI = MatMulIntegerHip;
    MMI::MatMulIntegerHip(MatMulIntegerInfo info_) noexcept : Kernel(), info(std::move(info_)) {}
    KernelBox MMI::build(MatMulIntegerInfo info) noexcept { return std::make_unique<MMI>(std::move(info)); }
    size_t MMI::typeId() noexcept { return idOf<MMI>(); }
    size_t MMI::kernelTypeId() const noexcept { return typeId(); }
    std::string_view MMI::description() const noexcept { return "Performing MatMulInteger with int8 MFMA on AMD gfx950"; }
    RoutineWorkspace MMI::lower(Resources &) const {
        unsigned flags = 0;
        if (info.a.scalar) { flags |= RG_MMI_A_ZP_SCALAR; }
        if (info.b.scalar) { flags |= RG_MMI_B_ZP_SCALAR; }
        // operand matrix of every output batch, resolved once here
        std::vector<uint32_t> aIndex, bIndex;
        if (info.broadcaster.needBroadcast()) {
            aIndex.resize(info.batch());
            bIndex.resize(info.batch());
            for (dim_t i = 0; i < info.batch(); ++i) {
                dim_t at[2];
                info.broadcaster.locate(i, at);
                aIndex[i] = at[0];
                bIndex[i] = at[1];
            }
        }
        // zero points are subtracted while the tiles are staged: the workspace the reference
        // needs for adjusted copies (m*k [+ k*n] bytes per batch) is not needed here
        auto const workspace = rg_hip_matmul_integer_workspace(info.batch(), info.m, info.k, info.n, flags);
        auto routine = [info = info, flags, aIndex = std::move(aIndex), bIndex = std::move(bIndex)]//
            (Resources &res, void *workspace, void const *const *inputs, void *const *outputs) {
                // inputs: A, B [, a_zero_point [, b_zero_point]]; an elided (constant zero) or absent
                // zero point is passed as null
                void const *aZp = info.a.withZeroPoint ? inputs[2] : nullptr;
                void const *bZp = info.b.withZeroPoint ? inputs[3] : nullptr;
                HIP_CALL(rg_hip_matmul_integer(
                    static_cast<int32_t *>(outputs[0]), inputs[0], inputs[1], aZp, bZp, flags,
                    info.batch(), info.m, info.k, info.n,
                    aIndex.empty() ? nullptr : aIndex.data(), bIndex.empty() ? nullptr : bIndex.data(),
                    workspace, streamOf(res)));
            };
        return {std::move(routine), workspace};
    }

    // ------------------------------------------------------------------ Transpose

    TransposeHip::TransposeHip(TransposeInfo info_) noexcept : Kernel(), info(std::move(info_)) {}
    KernelBox TransposeHip::build(TransposeInfo info) noexcept {
        return info.dims.size() <= 8 ? std::make_unique<TransposeHip>(std::move(info)) : nullptr;
    }
    size_t TransposeHip::typeId() noexcept { return idOf<TransposeHip>(); }
    size_t TransposeHip::kernelTypeId() const noexcept { return typeId(); }
    std::string_view TransposeHip::description() const noexcept { return "Performing transpose operation on AMD gfx950"; }
    RoutineWorkspace TransposeHip::lower(Resources &) const {
        std::vector<uint32_t> strideI, strideO;
        for (auto [i, o] : info.dims) {
            strideI.push_back(i);
            strideO.push_back(o);
        }
        return [strideI = std::move(strideI), strideO = std::move(strideO), blockSize = info.blockSize,
                blockCount = info.blockCount](Resources &res, void *, void const *const *inputs, void *const *outputs) {
            HIP_CALL(rg_hip_transpose(outputs[0], inputs[0], strideI.data(), strideO.data(), strideI.size(), blockSize,
                                      blockCount, streamOf(res)));
        };
    }

    // ------------------------------------------------------------------ Split / Concat / Expand / Where

    SplitHip::SplitHip(SplitInfo info_) noexcept : Kernel(), info(std::move(info_)) {}
    KernelBox SplitHip::build(SplitInfo info) noexcept { return std::make_unique<SplitHip>(std::move(info)); }
    size_t SplitHip::typeId() noexcept { return idOf<SplitHip>(); }
    size_t SplitHip::kernelTypeId() const noexcept { return typeId(); }
    std::string_view SplitHip::description() const noexcept { return "Performing split operation on AMD gfx950"; }
    RoutineWorkspace SplitHip::lower(Resources &) const {
        return [info = this->info](Resources &res, void *, void const *const *inputs, void *const *outputs) {
            HIP_CALL(rg_hip_split(outputs, inputs[0], info.segments.data(), info.segments.size(), info.blockCount, info.sum,
                                  streamOf(res)));
        };
    }

    ConcatHip::ConcatHip(SplitInfo info_) noexcept : Kernel(), info(std::move(info_)) {}
    KernelBox ConcatHip::build(SplitInfo info) noexcept { return std::make_unique<ConcatHip>(std::move(info)); }
    size_t ConcatHip::typeId() noexcept { return idOf<ConcatHip>(); }
    size_t ConcatHip::kernelTypeId() const noexcept { return typeId(); }
    std::string_view ConcatHip::description() const noexcept { return "Performing concat operation on AMD gfx950"; }
    RoutineWorkspace ConcatHip::lower(Resources &) const {
        return [info = this->info](Resources &res, void *, void const *const *inputs, void *const *outputs) {
            HIP_CALL(rg_hip_concat(outputs[0], inputs, info.segments.data(), info.segments.size(), info.blockCount, info.sum,
                                   streamOf(res)));
        };
    }

    ExpandHip::ExpandHip(ExpandInfo info_) noexcept : Kernel(), info(std::move(info_)) {}
    KernelBox ExpandHip::build(ExpandInfo info) noexcept {
        return info.strides.size() <= 8 ? std::make_unique<ExpandHip>(std::move(info)) : nullptr;
    }
    size_t ExpandHip::typeId() noexcept { return idOf<ExpandHip>(); }
    size_t ExpandHip::kernelTypeId() const noexcept { return typeId(); }
    std::string_view ExpandHip::description() const noexcept { return "Performing expand operation on AMD gfx950"; }
    RoutineWorkspace ExpandHip::lower(Resources &) const {
        std::vector<uint32_t> strideI, strideO;
        for (auto [i, o] : info.strides) {
            strideI.push_back(i);
            strideO.push_back(o);
        }
        return [strideI = std::move(strideI), strideO = std::move(strideO), blockSize = info.blockSize,
                blockCount = info.blockCount](Resources &res, void *, void const *const *inputs, void *const *outputs) {
            HIP_CALL(rg_hip_expand(outputs[0], inputs[0], strideI.data(), strideO.data(), strideI.size(), blockSize, blockCount,
                                   streamOf(res)));
        };
    }

    WhereHip::WhereHip(DataType dataType_, Broadcaster b) noexcept : Kernel(), dataType(dataType_), broadcaster(std::move(b)) {}
    KernelBox WhereHip::build(TensorRefs const &inputs) noexcept {
        if (inputs.size() != 3 || inputs[1].get().dataType != inputs[2].get().dataType) { return nullptr; }
        auto const size = inputs[1].get().dataType.size();
        if (size != 1 && size != 2 && size != 4 && size != 8) { return nullptr; }
        Broadcaster b(inputs);
        if (b.strides.size() / 4 > 8) { return nullptr; }
        return std::make_unique<WhereHip>(inputs[1].get().dataType, std::move(b));
    }
    size_t WhereHip::typeId() noexcept { return idOf<WhereHip>(); }
    size_t WhereHip::kernelTypeId() const noexcept { return typeId(); }
    std::string_view WhereHip::description() const noexcept { return "Performing where operation on AMD gfx950"; }
    RoutineWorkspace WhereHip::lower(Resources &) const {
        return [strides = broadcaster.strides, count = broadcaster.outputsCount,
                eleSize = dataType.size()](Resources &res, void *, void const *const *inputs, void *const *outputs) {
            HIP_CALL(rg_hip_where(outputs[0], inputs[0], inputs[1], inputs[2], strides.data(), strides.size() / 4, count, eleSize,
                                  streamOf(res)));
        };
    }

    // ------------------------------------------------------------------ MatMulInteger + DequantizeLinear

    using MMD = MatMulIntegerDequantizeHip;
    MMD::MatMulIntegerDequantizeHip(MatMulIntegerInfo info_, dim_t zeroPointInputs_, bool perColumn_) noexcept
        : Kernel(), info(std::move(info_)), zeroPointInputs(zeroPointInputs_), perColumn(perColumn_) {}
    KernelBox MMD::build(MatMulIntegerInfo info, dim_t zeroPointInputs, bool perColumn) noexcept {
        return zeroPointInputs <= 2 ? std::make_unique<MMD>(std::move(info), zeroPointInputs, perColumn) : nullptr;
    }
    size_t MMD::typeId() noexcept { return idOf<MMD>(); }
    size_t MMD::kernelTypeId() const noexcept { return typeId(); }
    std::string_view MMD::description() const noexcept {
        return "Performing MatMulInteger with a dequantising epilogue on AMD gfx950";
    }
    RoutineWorkspace MMD::lower(Resources &) const {
        unsigned flags = 0;
        if (info.a.scalar) { flags |= RG_MMI_A_ZP_SCALAR; }
        if (info.b.scalar) { flags |= RG_MMI_B_ZP_SCALAR; }
        std::vector<uint32_t> aIndex, bIndex;
        if (info.broadcaster.needBroadcast()) {
            aIndex.resize(info.batch());
            bIndex.resize(info.batch());
            for (dim_t i = 0; i < info.batch(); ++i) {
                dim_t at[2];
                info.broadcaster.locate(i, at);
                aIndex[i] = at[0];
                bIndex[i] = at[1];
            }
        }
        auto const workspace = rg_hip_matmul_integer_workspace(info.batch(), info.m, info.k, info.n, flags);
        auto routine = [info = info, flags, scaleAt = 2 + zeroPointInputs, perColumn = perColumn,
                        aIndex = std::move(aIndex), bIndex = std::move(bIndex)]//
            (Resources &res, void *workspacePtr, void const *const *inputs, void *const *outputs) {
                void const *aZp = info.a.withZeroPoint ? inputs[2] : nullptr;
                void const *bZp = info.b.withZeroPoint ? inputs[3] : nullptr;
                HIP_CALL(rg_hip_matmul_integer_dequantize(
                    static_cast<float *>(outputs[0]), inputs[0], inputs[1], aZp, bZp, flags,
                    info.batch(), info.m, info.k, info.n,
                    aIndex.empty() ? nullptr : aIndex.data(), bIndex.empty() ? nullptr : bIndex.data(),
                    static_cast<float const *>(inputs[scaleAt]), perColumn ? 1 : 0, workspacePtr, streamOf(res)));
            };
        return {std::move(routine), workspace};
    }

    // ------------------------------------------------------------------ DequantizeLinear

    using DQ = DequantizeLinearHip;
    DQ::DequantizeLinearHip(DataType from_, size_t outer_, size_t axisLen_, size_t inner_, bool perAxis_,
                            bool withZeroPoint_) noexcept
        : Kernel(), from(from_), outer(outer_), axisLen(axisLen_), inner(inner_), perAxis(perAxis_),
          withZeroPoint(withZeroPoint_) {}
    KernelBox DQ::build(TensorRefs const &inputs, Tensor const &output, int axis) noexcept {
        auto const &x = inputs[0].get();
        auto const &scale = inputs[1].get();
        if (output.dataType != DataType::F32 || scale.dataType != DataType::F32) { return nullptr; }
        switch (x.dataType) {
            case DataType::U8: case DataType::I8: case DataType::U16: case DataType::I16: case DataType::I32:
                break;
            default:
                return nullptr;
        }
        auto const withZp = inputs.size() > 2;
        if (withZp && inputs[2].get().dataType != x.dataType) { return nullptr; }
        auto const scales = scale.elementsSize();
        if (withZp && inputs[2].get().elementsSize() != scales) { return nullptr; }
        if (scales == 1) { return std::make_unique<DQ>(x.dataType, 1, 1, x.elementsSize(), false, withZp); }
        // one scale per index of `axis`
        auto const rank = static_cast<int>(x.rank());
        if (axis < 0) { axis += rank; }
        if (axis < 0 || axis >= rank || x.shape[axis] != scales) { return nullptr; }
        size_t outer = 1, inner = 1;
        for (int i = 0; i < axis; ++i) { outer *= x.shape[i]; }
        for (int i = axis + 1; i < rank; ++i) { inner *= x.shape[i]; }
        return std::make_unique<DQ>(x.dataType, outer, scales, inner, true, withZp);
    }
    size_t DQ::typeId() noexcept { return idOf<DQ>(); }
    size_t DQ::kernelTypeId() const noexcept { return typeId(); }
    std::string_view DQ::description() const noexcept { return "Performing dequantize linear on AMD gfx950"; }
    RoutineWorkspace DQ::lower(Resources &) const {
        return [*this](Resources &res, void *, void const *const *inputs, void *const *outputs) {
            HIP_CALL(rg_hip_dequantize_linear(static_cast<float *>(outputs[0]), inputs[0],
                                              static_cast<float const *>(inputs[1]),
                                              withZeroPoint ? inputs[2] : nullptr, outer, axisLen, inner,
                                              static_cast<int>(from.internal), perAxis ? 1 : 0, streamOf(res)));
        };
    }

    // ------------------------------------------------------------------ DynamicQuantizeLinear

    using DQL = DynamicQuantizeLinearHip;
    DQL::DynamicQuantizeLinearHip(decltype(size) size_) noexcept : Kernel(), size(size_) {}
    KernelBox DQL::build(decltype(size) size) noexcept {
        return size > 0 ? std::make_unique<DQL>(size) : nullptr;
    }
    size_t DQL::typeId() noexcept { return idOf<DQL>(); }
    size_t DQL::kernelTypeId() const noexcept { return typeId(); }
    std::string_view DQL::description() const noexcept { return "Performing dynamic quantize linear on AMD gfx950"; }
    RoutineWorkspace DQL::lower(Resources &) const {
        auto const workspace = rg_hip_dynamic_quantize_linear_workspace(size);
        auto routine = [size = size, workspace](Resources &res, void *workspacePtr, void const *const *inputs,
                                                void *const *outputs) {
            HIP_CALL(rg_hip_dynamic_quantize_linear(static_cast<uint8_t *>(outputs[0]),
                                                    static_cast<float *>(outputs[1]),
                                                    static_cast<uint8_t *>(outputs[2]),
                                                    static_cast<float const *>(inputs[0]), size, workspacePtr,
                                                    workspace, streamOf(res)));
        };
        return {std::move(routine), workspace};
    }

    // ------------------------------------------------------------------ MatMul

    MatMulHip::MatMulHip(decltype(info) info_) noexcept : Kernel(), info(std::move(info_)) {}
    KernelBox MatMulHip::build(decltype(info) info) noexcept {
        // src/04kernel/src/kernels/mat_mul/cublas_kernel.cc:9-20 accepts F32, F64, FP16
        auto const dt = info.dataType;
        if (dt != DataType::F32 && dt != DataType::F64 && dt != DataType::FP16 && dt != DataType::BF16) { return nullptr; }
        if (info.hasBias && !info.biasSupported) { return nullptr; }
        return std::make_unique<MatMulHip>(std::move(info));
    }
    size_t MatMulHip::typeId() noexcept { return idOf<MatMulHip>(); }
    size_t MatMulHip::kernelTypeId() const noexcept { return typeId(); }
    std::string_view MatMulHip::description() const noexcept { return "Performing MatMul with MFMA on AMD gfx950"; }
    RoutineWorkspace MatMulHip::lower(Resources &) const {
        std::vector<uint32_t> aIndex, bIndex;
        if (info.broadcaster.needBroadcast()) {
            aIndex.resize(info.batch());
            bIndex.resize(info.batch());
            for (dim_t i = 0; i < info.batch(); ++i) {
                dim_t at[2];
                info.broadcaster.locate(i, at);
                aIndex[i] = at[0];
                bIndex[i] = at[1];
            }
        }
        if (!info.biasExpandFrom.empty()) {
            // The bias broadcasts over some batch dimensions only: Expand lays it out over [batch..., m, n] in the
            // workspace and the product reads it from there, one element per output.  (The reference expands into Y
            // and lets the library update Y in place; here tiles of ragged shapes overlap, so Y cannot be both.)
            ExpandInfo const e(info.dataType, info.biasExpandFrom, info.biasExpandTo);
            std::vector<uint32_t> strideI, strideO;
            for (auto [i, o] : e.strides) {
                strideI.push_back(i);
                strideO.push_back(o);
            }
            auto const bytes = static_cast<size_t>(e.blockSize) * e.blockCount;
            auto routine = [info = info, aIndex = std::move(aIndex), bIndex = std::move(bIndex), strideI = std::move(strideI),
                            strideO = std::move(strideO), blockSize = e.blockSize, blockCount = e.blockCount]//
                (Resources &res, void *workspace, void const *const *inputs, void *const *outputs) {
                    HIP_CALL(rg_hip_expand(workspace, inputs[2], strideI.data(), strideO.data(), strideI.size(), blockSize,
                                           blockCount, streamOf(res)));
                    HIP_CALL(rg_hip_matmul(outputs[0], inputs[0], inputs[1], workspace,
                                           static_cast<int>(info.dataType.internal), info.transA, info.transB, info.alpha,
                                           info.beta, info.batch(), info.m, info.k, info.n,
                                           aIndex.empty() ? nullptr : aIndex.data(), bIndex.empty() ? nullptr : bIndex.data(),
                                           info.biasStrideBatch, info.biasStrideM, info.biasStrideN, streamOf(res)));
                };
            return RoutineWorkspace(std::move(routine), bytes);
        }
        // A workspace where the library has a use for one (few rows against weights kept as [k, n]: sums of shares
        // of k meet there); its contents never need preparing, so any range of the stack will do.
        auto const bytes = rg_hip_matmul_workspace(static_cast<int>(info.dataType.internal), info.transA, info.transB,
                                                   info.batch(), info.m, info.k, info.n);
        auto routine = [info = info, aIndex = std::move(aIndex), bIndex = std::move(bIndex), bytes]//
            (Resources &res, void *workspace, void const *const *inputs, void *const *outputs) {
                HIP_CALL(rg_hip_matmul_ws(outputs[0], inputs[0], inputs[1], info.hasBias ? inputs[2] : nullptr,
                                          static_cast<int>(info.dataType.internal), info.transA, info.transB, info.alpha,
                                          info.beta, info.batch(), info.m, info.k, info.n,
                                          aIndex.empty() ? nullptr : aIndex.data(), bIndex.empty() ? nullptr : bIndex.data(),
                                          info.biasStrideBatch, info.biasStrideM, info.biasStrideN, bytes ? workspace : nullptr, bytes,
                                          streamOf(res)));
            };
        return RoutineWorkspace(std::move(routine), bytes);
    }

    // ------------------------------------------------------------------ Cast

    CastHip::CastHip(decltype(from) from_, decltype(to) to_, decltype(size) size_) noexcept
        : Kernel(), from(from_), to(to_), size(size_) {}
    KernelBox CastHip::build(Tensor const &from, Tensor const &to) noexcept {
        auto castable = [](DataType t) {
            return t.isCpuNumberic() || t == DataType::Bool || t == DataType::FP16 || t == DataType::BF16;
        };
        if (!castable(from.dataType) || !castable(to.dataType)) { return nullptr; }
        if (from.elementsSize() != to.elementsSize()) { return nullptr; }
        return std::make_unique<CastHip>(from.dataType, to.dataType, from.elementsSize());
    }
    size_t CastHip::typeId() noexcept { return idOf<CastHip>(); }
    size_t CastHip::kernelTypeId() const noexcept { return typeId(); }
    std::string_view CastHip::description() const noexcept { return "Performing cast operation on AMD gfx950"; }
    RoutineWorkspace CastHip::lower(Resources &) const {
        return [from = from, to = to, size = size](Resources &res, void *, void const *const *inputs, void *const *outputs) {
            HIP_CALL(rg_hip_cast(outputs[0], inputs[0], size, static_cast<int>(from.internal),
                                 static_cast<int>(to.internal), streamOf(res)));
        };
    }

    // ------------------------------------------------------------------ Attention

    HipAttentionState::HipAttentionState() : _counters(nullptr) {
        auto const bytes = rg_hip_attention_kvcache_state_bytes();
        HIP_CALL(rg_hip_malloc(&_counters, bytes));
        std::vector<uint8_t> zeros(bytes, 0);
        HIP_CALL(rg_hip_memcpy_h2d(_counters, zeros.data(), bytes));
    }
    HipAttentionState::~HipAttentionState() { rg_hip_free(_counters); }
    size_t HipAttentionState::typeId() noexcept { return idOf<HipAttentionState>(); }
    runtime::ResourceBox HipAttentionState::build() { return std::make_unique<HipAttentionState>(); }
    size_t HipAttentionState::resourceTypeId() const noexcept { return typeId(); }
    std::string_view HipAttentionState::description() const noexcept { return "Attention ticket counters on AMD gfx950"; }

    using AT = AttentionHip;
    AT::AttentionHip(Info info_) noexcept : Kernel(), info(info_) {}
    KernelBox AT::build(Info info) noexcept {
        if (info.dataType != DataType::FP16 && info.dataType != DataType::BF16) { return nullptr; }
        if (info.headDim != 64 && info.headDim != 80 && info.headDim != 96 && info.headDim != 128) { return nullptr; }
        if (info.nKVHead == 0 || info.nHead % info.nKVHead != 0) { return nullptr; }
        if (info.cacheLen && info.cacheLen < info.seqLen) { return nullptr; }
        if (info.pastFromInput && info.pastCount != 1 && info.pastCount != info.batch) { return nullptr; }
        return std::make_unique<AT>(info);
    }
    size_t AT::typeId() noexcept { return idOf<AT>(); }
    size_t AT::kernelTypeId() const noexcept { return typeId(); }
    std::string_view AT::description() const noexcept { return "Performing multihead attention on AMD gfx950"; }
    RoutineWorkspace AT::lower(Resources &res) const {
        // created here, at lowering, so that no allocation happens in the routine
        res.fetchOrStore<HipAttentionState>();
        auto const workspace = rg_hip_attention_kvcache_workspace(info.batch, info.nHead, info.nKVHead, info.seqLen,
                                                                  info.cacheLen, info.headDim);
        auto const scale = 1.0f / std::sqrt(static_cast<float>(info.headDim));
        auto routine = [info = info, workspace, scale]//
            (Resources &res, void *ws, void const *const *inputs, void *const *outputs) {
                auto *state = res.fetchOrStore<HipAttentionState>();
                // inputs: query, key, value [, past_seq_len [, k_cache, v_cache]]
                // outputs: output [, k_cache, v_cache]; with 4 inputs the output caches are the
                // persistent ones the history already lives in, with 6 they start as copies of the inputs
                void *kCache = info.cacheLen ? outputs[1] : nullptr;
                void *vCache = info.cacheLen ? outputs[2] : nullptr;
                if (info.resetCache && kCache) {
                    auto const bytes = static_cast<size_t>(info.batch) * info.nKVHead * info.cacheLen * info.headDim *
                                       info.dataType.size();
                    if (inputs[4] != kCache) { HIP_CALL(rg_hip_memcpy_d2d_async(kCache, inputs[4], bytes, streamOf(res))); }
                    if (inputs[5] != vCache) { HIP_CALL(rg_hip_memcpy_d2d_async(vCache, inputs[5], bytes, streamOf(res))); }
                }
                auto const *past = info.pastFromInput ? static_cast<int64_t const *>(inputs[3]) : nullptr;
                HIP_CALL(rg_hip_attention_kvcache(
                    outputs[0], inputs[0], inputs[1], inputs[2], kCache, vCache, past,
                    info.pastCount == info.batch && info.batch > 1 ? 1 : 0,
                    info.batch, info.nHead, info.nKVHead, info.seqLen, info.cacheLen, info.headDim, scale,
                    static_cast<int>(info.dataType.internal), ws, workspace, state->counters(), streamOf(res)));
            };
        return {std::move(routine), workspace};
    }

    // ------------------------------------------------------------------ RotaryEmbedding

    using RE = RotaryEmbeddingHip;
    RE::RotaryEmbeddingHip(DataType dataType_, dim_t batch_, dim_t seq_, dim_t heads_, dim_t dim_, bool posPerBatch_,
                           float theta_) noexcept
        : Kernel(), dataType(dataType_), batch(batch_), seq(seq_), heads(heads_), dim(dim_),
          posPerBatch(posPerBatch_), theta(theta_) {}
    KernelBox RE::build(float theta, Tensor const &x, Tensor const &pos) noexcept {
        if (x.rank() != 4 || pos.dataType != DataType::I64) { return nullptr; }
        if (x.dataType != DataType::FP16 && x.dataType != DataType::BF16 && x.dataType != DataType::F32) { return nullptr; }
        if (x.shape[3] % 2 != 0 || x.shape[3] > 512) { return nullptr; }
        bool perBatch;
        if (pos.rank() == 2 && pos.shape[0] == x.shape[0] && pos.shape[1] == x.shape[1]) perBatch = true;
        else if (pos.rank() == 1 && pos.shape[0] == x.shape[1]) perBatch = false;
        else return nullptr;
        return std::make_unique<RE>(x.dataType, x.shape[0], x.shape[1], x.shape[2], x.shape[3], perBatch, theta);
    }
    size_t RE::typeId() noexcept { return idOf<RE>(); }
    size_t RE::kernelTypeId() const noexcept { return typeId(); }
    std::string_view RE::description() const noexcept { return "Performing rotary embedding on AMD gfx950"; }
    RoutineWorkspace RE::lower(Resources &) const {
        return [*this](Resources &res, void *, void const *const *inputs, void *const *outputs) {
            HIP_CALL(rg_hip_rope(outputs[0], inputs[0], static_cast<int64_t const *>(inputs[1]), posPerBatch ? 1 : 0,
                                 batch, seq, heads, dim, theta, static_cast<int>(dataType.internal), streamOf(res)));
        };
    }

}// namespace refactor::kernel
