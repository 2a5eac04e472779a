// runtime layer of the host mirror: the Routine signature every kernel lowers to and the
// per-stream Resources map.  Follows src/03runtime/include/runtime/{stream.h:10-22,
// resource.h:10-45}; the graph-walking Stream is in rg_mirror/stream.h.
#pragma once

#include "rg_mirror/common.h"
#include <functional>
#include <unordered_map>

namespace refactor::runtime {

    class Resource {
    public:
        virtual ~Resource() = default;
        virtual size_t resourceTypeId() const = 0;
        virtual std::string_view description() const = 0;
        bool is(size_t id) const noexcept { return resourceTypeId() == id; }
    };
    using ResourceBox = std::unique_ptr<Resource>;

    // Type-id keyed, owning, not thread-safe (one per Stream).
    class Resources {
        std::unordered_map<size_t, ResourceBox> _internal;

    public:
        Resource *fetch(size_t) noexcept;
        Resource *fetchOrStore(ResourceBox) noexcept;
        Resource *fetchOrStore(size_t, std::function<ResourceBox()>);

        template<class T> T *fetch() noexcept { return dynamic_cast<T *>(fetch(T::typeId())); }
        template<class T> T *fetchOrStore(ResourceBox r) noexcept {
            return dynamic_cast<T *>(fetchOrStore(std::move(r)));
        }
        template<class T, class... Args> T *fetchOrStore(Args &&...args) {
            return dynamic_cast<T *>(fetchOrStore(
                T::typeId(), [&]() -> ResourceBox { return T::build(std::forward<Args>(args)...); }));
        }
    };

    // (resources, workspace, inputs, outputs): raw device addresses in operator order; work is
    // enqueued on the default stream and nothing is synchronised.
    using Routine = std::function<void(Resources &, void *, void const *const *, void *const *)>;

    void emptyRoutine(Resources &, void *, void const *const *, void *const *);

    struct Node {
        Routine routine;
        size_t workspaceOffset;// a size when returned by Kernel::lower, an offset once allocated

        template<class T>
        Node(T &&r, size_t wso = 0) noexcept : routine(std::forward<T>(r)), workspaceOffset(wso) {}
    };

}// namespace refactor::runtime
