#include "rg_mirror/kernel.h"
#include <cstdlib>
#include <numeric>

namespace refactor::kernel {

    RoutineWorkspace Kernel::lower(Resources &) const {
        TODO(detail::cat("lower not implemented for ", description()));
    }

    Blob::Blob(size_t bytes) : _ptr(std::malloc(bytes ? bytes : 1)) {}
    Blob::~Blob() { std::free(_ptr); }
    std::pair<Arc<Blob>, void *> Blob::share(size_t bytes) {
        auto blob = Arc<Blob>(new Blob(bytes));
        auto ptr = blob->_ptr;
        return {std::move(blob), ptr};
    }

    Tensor::Tensor(DataType dataType_, Shape shape_, LayoutType layout_, Arc<Blob> data_) noexcept
        : dataType(dataType_), shape(std::move(shape_)), layout(layout_), data(std::move(data_)) {}

    Arc<Tensor> Tensor::share(DataType dataType, Shape shape, LayoutType layout, Arc<Blob> data) noexcept {
        return std::make_shared<Tensor>(dataType, std::move(shape), layout, std::move(data));
    }

    int64_t Tensor::rank() const { return static_cast<int64_t>(shape.size()); }
    size_t Tensor::elementsSize() const {
        return std::accumulate(shape.begin(), shape.end(), size_t(1), std::multiplies<size_t>());
    }
    size_t Tensor::bytesSize() const { return dataType.size() * elementsSize(); }
    Strides Tensor::strides() const {
        Strides ans(shape.size());
        dim_t run = 1;
        for (auto i = shape.size(); i-- > 0;) {
            ans[i] = run;
            run *= shape[i];
        }
        return ans;
    }
    void *Tensor::malloc() {
        auto [blob, ptr] = Blob::share(bytesSize());
        data = std::move(blob);
        return ptr;
    }
    void Tensor::free() { data = nullptr; }

}// namespace refactor::kernel
