#include "rg_mirror/hardware.h"
#include "rg_hip.h"
#include <cstdlib>
#include <cstring>
#include <iterator>
#include <utility>

#define HIP_ASSERT(CALL)                                                                              \
    if (auto status_ = (CALL); status_ != 0) {                                                        \
        RUNTIME_ERROR(::refactor::detail::cat("hip failed on \"" #CALL "\" with \"",                  \
                                              rg_hip_error_string(status_), "\" (", status_, ")"));   \
    }

namespace refactor::hardware {

    // ------------------------------------------------------------------ CPU memory

    void *CpuMemory::malloc(size_t bytes) { return std::malloc(bytes); }
    void CpuMemory::free(void *ptr) { std::free(ptr); }
    void *CpuMemory::copyHD(void *dst, void const *src, size_t bytes) const { return std::memcpy(dst, src, bytes); }
    void *CpuMemory::copyDH(void *dst, void const *src, size_t bytes) const { return std::memcpy(dst, src, bytes); }
    void *CpuMemory::copyDD(void *dst, void const *src, size_t bytes) const { return std::memcpy(dst, src, bytes); }

    // ------------------------------------------------------------------ AMD memory

    void *AmdMemory::malloc(size_t bytes) {
        void *ptr = nullptr;
        HIP_ASSERT(rg_hip_malloc(&ptr, bytes));
        return ptr;
    }
    void AmdMemory::free(void *ptr) { HIP_ASSERT(rg_hip_free(ptr)); }
    void *AmdMemory::copyHD(void *dst, void const *src, size_t bytes) const {
        HIP_ASSERT(rg_hip_memcpy_h2d(dst, src, bytes));
        return dst;
    }
    void *AmdMemory::copyDH(void *dst, void const *src, size_t bytes) const {
        HIP_ASSERT(rg_hip_memcpy_d2h(dst, src, bytes));
        return dst;
    }
    void *AmdMemory::copyDD(void *dst, void const *src, size_t bytes) const {
        HIP_ASSERT(rg_hip_memcpy_d2d(dst, src, bytes));
        return dst;
    }

    // ------------------------------------------------------------------ offset planning

    OffsetCalculator::OffsetCalculator(size_t alignment, bool) : _alignment(alignment ? alignment : 1) {}

    size_t OffsetCalculator::alloc(size_t bytes) {
        auto const need = alignBytes(bytes, _alignment);
        if (need == 0) return _peak;// nothing to place
        _used += need;
        auto best = _freeByOffset.end();
        for (auto it = _freeByOffset.begin(); it != _freeByOffset.end(); ++it)
            if (it->second >= need && (best == _freeByOffset.end() || it->second < best->second)) best = it;
        if (best != _freeByOffset.end()) {
            auto const [offset, size] = *best;
            _freeByOffset.erase(best);
            if (size > need) _freeByOffset.emplace(offset + need, size - need);
            return offset;
        }
        if (!_freeByOffset.empty()) {
            auto last = std::prev(_freeByOffset.end());
            if (last->first + last->second == _peak) {// too small, but it can grow with the range
                auto const offset = last->first;
                _freeByOffset.erase(last);
                _peak = offset + need;
                return offset;
            }
        }
        auto const offset = _peak;
        _peak += need;
        return offset;
    }

    void OffsetCalculator::free(size_t offset, size_t bytes) {
        auto size = alignBytes(bytes, _alignment);
        if (size == 0) return;
        _used -= size;
        auto next = _freeByOffset.lower_bound(offset);
        if (next != _freeByOffset.begin()) {
            auto prev = std::prev(next);
            ASSERT(prev->first + prev->second <= offset, "double free");
            if (prev->first + prev->second == offset) {
                offset = prev->first;
                size += prev->second;
                _freeByOffset.erase(prev);
            }
        }
        if (next != _freeByOffset.end()) {
            ASSERT(offset + size <= next->first, "double free");
            if (offset + size == next->first) {
                size += next->second;
                _freeByOffset.erase(next);
            }
        }
        _freeByOffset.emplace(offset, size);
    }

    // ------------------------------------------------------------------ pool

    MemPool::MemPool(Arc<Memory> parent, size_t memPoolSize, size_t alignment)
        : _parent(std::move(parent)),
          _memPoolSize(memPoolSize),
          _alignment(alignment ? alignment : 1),
          _ptr(_parent->malloc(memPoolSize)),
          _freeByOffset{{0, memPoolSize}},
          _ptrToBlobsize{} {}

    MemPool::~MemPool() { _parent->free(_ptr); }

    void *MemPool::malloc(size_t bytes) {
        if (bytes == 0) { return nullptr; }
        auto const need = (bytes + _alignment - 1) / _alignment * _alignment;
        // best fit: the smallest free range that holds the request; ties go to the lowest offset
        auto best = _freeByOffset.end();
        for (auto it = _freeByOffset.begin(); it != _freeByOffset.end(); ++it) {
            if (it->second >= need && (best == _freeByOffset.end() || it->second < best->second)) { best = it; }
        }
        ASSERT(best != _freeByOffset.end(), "out of memory");
        auto const offset = best->first, have = best->second;
        _freeByOffset.erase(best);
        if (have > need) { _freeByOffset.emplace(offset + need, have - need); }
        void *ans = static_cast<uint8_t *>(_ptr) + offset;
        _ptrToBlobsize.emplace(ans, need);
        return ans;
    }

    void MemPool::free(void *ptr) {
        if (!ptr) { return; }
        auto it = _ptrToBlobsize.find(ptr);
        ASSERT(it != _ptrToBlobsize.end(), "invalid ptr");
        size_t offset = static_cast<uint8_t *>(ptr) - static_cast<uint8_t *>(_ptr), bytes = it->second;
        _ptrToBlobsize.erase(it);
        // merge with the free ranges that touch this one
        auto next = _freeByOffset.lower_bound(offset);
        if (next != _freeByOffset.end() && next->first == offset + bytes) {
            bytes += next->second;
            next = _freeByOffset.erase(next);
        }
        if (next != _freeByOffset.begin()) {
            auto prev = std::prev(next);
            if (prev->first + prev->second == offset) {
                offset = prev->first;
                bytes += prev->second;
                _freeByOffset.erase(prev);
            }
        }
        _freeByOffset.emplace(offset, bytes);
    }

    void *MemPool::copyHD(void *dst, void const *src, size_t bytes) const { return _parent->copyHD(dst, src, bytes); }
    void *MemPool::copyDH(void *dst, void const *src, size_t bytes) const { return _parent->copyDH(dst, src, bytes); }
    void *MemPool::copyDD(void *dst, void const *src, size_t bytes) const { return _parent->copyDD(dst, src, bytes); }

    // ------------------------------------------------------------------ device + blob

    Device::Blob::Blob(Device *device, size_t size) : _device(device), _ptr(nullptr), _size(size) {
        _device->setContext();
        _ptr = _device->_mem->malloc(size);
    }
    Device::Blob::~Blob() {
        _device->setContext();
        _device->_mem->free(std::exchange(_ptr, nullptr));
    }
    void Device::Blob::copyFromHost(void const *ptr) const { copyFromHost(ptr, _size); }
    void Device::Blob::copyFromHost(void const *ptr, size_t size) const {
        ASSERT(size <= _size, "size too large");
        _device->setContext();
        _device->_mem->copyHD(_ptr, ptr, size);
    }
    void Device::Blob::copyToHost(void *ptr) const { copyToHost(ptr, _size); }
    void Device::Blob::copyToHost(void *ptr, size_t size) const {
        ASSERT(size <= _size, "size too large");
        _device->setContext();
        _device->_mem->copyDH(ptr, _ptr, size);
    }
    void Device::Blob::copyFrom(Blob const &rhs) const { copyFrom(rhs, rhs._size); }
    void Device::Blob::copyFrom(Blob const &rhs, size_t size) const {
        ASSERT(size <= rhs._size && size <= _size, "size too large");
        if (_device->_mem == rhs._device->_mem) {
            _device->setContext();
            _device->_mem->copyDD(_ptr, rhs._ptr, size);
        } else if (rhs._device->type() == Device::Type::Cpu) {
            copyFromHost(rhs._ptr, size);
        } else {
            std::vector<uint8_t> staging(size);
            rhs.copyToHost(staging.data(), size);
            copyFromHost(staging.data(), size);
        }
    }
    void Device::Blob::copyTo(Blob const &rhs) const { rhs.copyFrom(*this); }
    void Device::Blob::copyTo(Blob const &rhs, size_t size) const { rhs.copyFrom(*this, size); }

    Device::Device(int32_t card, Arc<Memory> mem) : _card(card), _mem(std::move(mem)) {}
    void Device::setContext() const {}
    Arc<Device::Blob> Device::malloc(size_t size) { return Arc<Blob>(new Blob(this, size)); }
    void Device::copyOut(void *host, void const *deviceAddress, size_t bytes) const {
        setContext();
        _mem->copyDH(host, deviceAddress, bytes);
    }
    Arc<Device::Blob> Device::absorb(Arc<Blob> &&blob) {
        if (blob->_device == this) { return std::move(blob); }
        if (blob->_device->_mem == _mem) {
            blob->_device = this;
            return std::move(blob);
        }
        auto moved = malloc(blob->_size);
        moved->copyFrom(*blob);
        return moved;
    }

    Cpu::Cpu() : Device(0, std::make_shared<CpuMemory>()) {}

    static Arc<Memory> amdMemory(int32_t card, size_t poolBytes) {
        int count = 0;
        HIP_ASSERT(rg_hip_device_count(&count));
        ASSERT(0 <= card && card < count, "Invalid card id: ", card);
        HIP_ASSERT(rg_hip_set_device(card));
        size_t free = 0, total = 0;
        HIP_ASSERT(rg_hip_mem_info(&free, &total));
        auto const size = poolBytes ? poolBytes : free / 10 * 9;
        constexpr size_t alignment = 256;
        return std::make_shared<MemPool>(std::make_shared<AmdMemory>(), size, alignment);
    }

    Amd::Amd(int32_t card, size_t poolBytes) : Device(card, amdMemory(card, poolBytes)) {}
    void Amd::setContext() const { HIP_ASSERT(rg_hip_set_device(_card)); }

    // ------------------------------------------------------------------ device manager

    namespace device {
        static std::unordered_map<int32_t, std::unordered_map<int32_t, Arc<Device>>> &registry() {
            static std::unordered_map<int32_t, std::unordered_map<int32_t, Arc<Device>>> devices;
            return devices;
        }
        static Arc<Device> cpu() {
            static auto instance = std::make_shared<Cpu>();
            return instance;
        }

        Arc<Device> fetch(Device::Type type) {
            if (type == Device::Type::Cpu) { return cpu(); }
            auto &all = registry();
            if (auto kind = all.find(static_cast<int32_t>(type)); kind != all.end() && !kind->second.empty()) {
                return kind->second.begin()->second;
            }
            return init(type, 0, "");
        }
        Arc<Device> fetch(Device::Type type, int32_t card) {
            if (type == Device::Type::Cpu) { return cpu(); }
            auto &all = registry();
            if (auto kind = all.find(static_cast<int32_t>(type)); kind != all.end()) {
                if (auto it = kind->second.find(card); it != kind->second.end()) { return it->second; }
            }
            return nullptr;
        }
        Arc<Device> init(Device::Type type, int32_t card, std::string_view args) {
            if (auto device = fetch(type, card); device) { return device; }
            size_t pool = 0;
            if (auto at = args.find("pool="); at != std::string_view::npos) {
                pool = std::strtoull(std::string(args.substr(at + 5)).c_str(), nullptr, 10);
            }
            Arc<Device> device;
            switch (type) {
                case Device::Type::Amd:
                    device = std::make_shared<Amd>(card, pool);
                    break;
                default:
                    // the Nvidia / Mlu / Kunlun backends of the reference are not part of this build
                    device = UNREACHABLEX(Arc<Device>, "device type ", static_cast<int>(type), " is not built");
            }
            return registry()[static_cast<int32_t>(type)].emplace(card, std::move(device)).first->second;
        }
        void sync(Device::Type type) {
            if (type == Device::Type::Amd) { HIP_ASSERT(rg_hip_sync()); }
        }
    }// namespace device

}// namespace refactor::hardware
