// kernel layer core of the host mirror: Kernel, InfoCollector, kernel::Tensor and the constant
// Blob.  Follows src/04kernel/include/kernel/{kernel.h:12-23, collector.h:10-20, tensor.h:12-30,
// blob.hh, layout.h} with std::vector where the reference uses absl::InlinedVector.
#pragma once

#include "rg_mirror/hardware.h"
#include "rg_mirror/runtime.h"
#include <functional>

namespace refactor::kernel {

    using runtime::Resources;
    using runtime::Routine;
    using RoutineWorkspace = runtime::Node;

    class Kernel {
    public:
        virtual ~Kernel() = default;
        virtual size_t kernelTypeId() const = 0;
        virtual std::string_view description() const = 0;
        // the base throws UnimplementError, like src/04kernel/src/kernel.cc:5-7
        virtual RoutineWorkspace lower(Resources &) const;

        template<class T, class... Args>
        bool is(Args &&...args) const noexcept {
            return this->kernelTypeId() == T::typeId(std::forward<Args>(args)...);
        }
    };
    using KernelBox = std::unique_ptr<Kernel>;

    // Host memory initialised once; a Tensor that carries one is a compile-time constant.
    class Blob {
        void *_ptr;
        explicit Blob(size_t);

    public:
        Blob(Blob const &) = delete;
        ~Blob();
        static std::pair<Arc<Blob>, void *> share(size_t);
        operator void const *() const noexcept { return _ptr; }
        template<class T> T const *get() const noexcept { return reinterpret_cast<T const *>(_ptr); }
    };

    struct LayoutType {
        enum : uint8_t { NCHW, NHWC, Others } internal;
        constexpr LayoutType(decltype(internal) i) noexcept : internal(i) {}
        constexpr operator decltype(internal)() const noexcept { return internal; }
    };

    using Shape = std::vector<dim_t>;
    using Strides = std::vector<dim_t>;

    struct Tensor {
        DataType dataType;
        Shape shape;
        LayoutType layout;
        Arc<Blob> data;

        Tensor(DataType, Shape, LayoutType, Arc<Blob>) noexcept;
        static Arc<Tensor> share(DataType, Shape, LayoutType = LayoutType::Others, Arc<Blob> = nullptr) noexcept;

        int64_t rank() const;
        size_t elementsSize() const;
        size_t bytesSize() const;
        Strides strides() const;
        void *malloc();
        void free();
    };
    using TensorRefs = std::vector<std::reference_wrapper<Tensor const>>;

    class InfoCollector {
    protected:
        hardware::Device::Type _target;
        constexpr explicit InfoCollector(hardware::Device::Type target) : _target(target) {}

    public:
        virtual ~InfoCollector() = default;
        // candidates in preference order; the caller takes the first
        // (src/05computation/src/graph.cc:47-52)
        virtual std::vector<KernelBox> filter(TensorRefs inputs, TensorRefs outputs) const = 0;
    };
    using CollectorBox = std::unique_ptr<InfoCollector>;

}// namespace refactor::kernel
