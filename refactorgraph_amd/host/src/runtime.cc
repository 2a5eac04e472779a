#include "rg_mirror/runtime.h"

namespace refactor::runtime {

    Resource *Resources::fetch(size_t id) noexcept {
        auto it = _internal.find(id);
        return it == _internal.end() ? nullptr : it->second.get();
    }
    Resource *Resources::fetchOrStore(ResourceBox resource) noexcept {
        auto id = resource->resourceTypeId();
        return _internal.try_emplace(id, std::move(resource)).first->second.get();
    }
    Resource *Resources::fetchOrStore(size_t id, std::function<ResourceBox()> make) {
        auto it = _internal.find(id);
        if (it == _internal.end()) { it = _internal.emplace(id, make()).first; }
        return it->second.get();
    }

    void emptyRoutine(Resources &, void *, void const *const *, void *const *) {}

}// namespace refactor::runtime
