// hardware layer of the host mirror: Memory backends, the best-fit MemPool, Device / Blob and
// the device manager, with a new Device::Type::Amd next to the reference's targets.
// Interfaces follow src/02hardware/include/hardware/{memory.h:8-16, mem_pool.h:10-27,
// device.h:9-59, device_manager.h:8-10}; the AMD device talks to the GPU only through the C ABI
// of include/rg_hip.h (the reference's NVIDIA backend calls the CUDA runtime directly,
// src/02hardware/src/devices/nvidia/{device.cc,memory.cc}).
#pragma once

#include "rg_mirror/common.h"
#include <map>
#include <unordered_map>

namespace refactor::hardware {

    class Memory {
    public:
        virtual ~Memory() = default;
        virtual void *malloc(size_t) = 0;
        virtual void free(void *) = 0;
        virtual void *copyHD(void *dst, void const *src, size_t bytes) const = 0;
        virtual void *copyDH(void *dst, void const *src, size_t bytes) const = 0;
        virtual void *copyDD(void *dst, void const *src, size_t bytes) const = 0;
    };

    class CpuMemory final : public Memory {
    public:
        void *malloc(size_t) final;
        void free(void *) final;
        void *copyHD(void *dst, void const *src, size_t bytes) const final;
        void *copyDH(void *dst, void const *src, size_t bytes) const final;
        void *copyDD(void *dst, void const *src, size_t bytes) const final;
    };

    // hipMalloc / hipFree / hipMemcpy through rg_hip_*; failures become RUNTIME_ERRORs.
    class AmdMemory final : public Memory {
    public:
        void *malloc(size_t) final;
        void free(void *) final;
        void *copyHD(void *dst, void const *src, size_t bytes) const final;
        void *copyDH(void *dst, void const *src, size_t bytes) const final;
        void *copyDD(void *dst, void const *src, size_t bytes) const final;
    };

    // One slab taken from `parent` at construction, carved by a best-fit free list whose
    // neighbouring free ranges are merged on free().  Every returned pointer is `alignment`
    // aligned relative to the slab.  Exhaustion is a RUNTIME_ERROR ("out of memory").
    class MemPool final : public Memory {
        Arc<Memory> _parent;
        size_t _memPoolSize, _alignment;
        void *_ptr;
        std::map<size_t, size_t> _freeByOffset;            // offset -> bytes
        std::unordered_map<void *, size_t> _ptrToBlobsize;// live blocks (aligned size)

    public:
        MemPool(Arc<Memory> parent, size_t memPoolSize, size_t alignment);
        ~MemPool();
        MemPool(MemPool const &) = delete;

        void *malloc(size_t bytes) final;
        void free(void *ptr) final;
        void *copyHD(void *dst, void const *src, size_t bytes) const final;
        void *copyDH(void *dst, void const *src, size_t bytes) const final;
        void *copyDD(void *dst, void const *src, size_t bytes) const final;
    };

    // smallest multiple of `alignment` that is >= bytes (src/02hardware/include/hardware/functions.h)
    constexpr size_t alignBytes(size_t bytes, size_t alignment) noexcept {
        return alignment ? (bytes + alignment - 1) / alignment * alignment : bytes;
    }

    // Plans offsets inside one range that only grows at its end: alloc() takes the smallest free
    // block that fits (lowest offset among equals), else lengthens the free block that touches
    // the end, else appends; free() merges neighbours.  peak() is the range the plan needs.
    // Behaviour of src/02hardware/src/mem_offset_calculator.cc:28-117 (without its tracing).
    class OffsetCalculator {
        size_t _used = 0, _peak = 0, _alignment;
        std::map<size_t, size_t> _freeByOffset;// offset -> bytes

    public:
        explicit OffsetCalculator(size_t alignment, bool trace = false);
        size_t alloc(size_t bytes);
        void free(size_t offset, size_t bytes);
        size_t peak() const noexcept { return _peak; }
        size_t used() const noexcept { return _used; }
    };

    class Device {
    public:
        enum class Type : int32_t {
            Cpu,
            Nvidia,
            Mlu,
            Kunlun,
            Amd,// gfx950 through librg_hip.so
        };

    protected:
        int32_t _card;
        Arc<Memory> _mem;
        Device(int32_t card, Arc<Memory> mem);

    public:
        class Blob {
            friend class Device;
            Device *_device;
            void *_ptr;
            size_t _size;
            Blob(Device *device, size_t);

        public:
            ~Blob();
            Blob(Blob const &) = delete;
            void copyFromHost(void const *) const;
            void copyFromHost(void const *, size_t) const;
            void copyToHost(void *) const;
            void copyToHost(void *, size_t) const;
            void copyFrom(Blob const &) const;
            void copyFrom(Blob const &, size_t) const;
            void copyTo(Blob const &) const;
            void copyTo(Blob const &, size_t) const;
            constexpr size_t size() const noexcept { return _size; }
            constexpr void *get() const noexcept { return _ptr; }
            template<class T> constexpr T *get() const noexcept { return static_cast<T *>(_ptr); }
            constexpr operator void *() const noexcept { return get(); }
            constexpr operator bool() const noexcept { return get(); }
        };

        virtual ~Device() = default;
        virtual Type type() const noexcept = 0;
        virtual void setContext() const;

        Arc<Blob> malloc(size_t);
        Arc<Blob> absorb(Arc<Blob> &&);
        // device address -> host memory, blocking (what Executor::trace reads node results with; the
        // reference has kernel::cuda::copyOut for it, src/04kernel/cuda/src/functions.cu:17-21)
        void copyOut(void *host, void const *deviceAddress, size_t bytes) const;
    };

    class Cpu final : public Device {
    public:
        Cpu();
        Type type() const noexcept final { return Type::Cpu; }
    };

    // One MI355X card.  The constructor selects the card and reserves 90 % of its free memory
    // in a MemPool aligned to 256 bytes (so 128-bit vector access is legal on every blob).
    // `poolBytes` overrides the reservation (0 = default), e.g. for tests.
    class Amd final : public Device {
    public:
        explicit Amd(int32_t card, size_t poolBytes = 0);
        Type type() const noexcept final { return Type::Amd; }
        void setContext() const final;
    };

    namespace device {
        Arc<Device> fetch(Device::Type);
        Arc<Device> fetch(Device::Type, int32_t card);
        // args: "pool=<bytes>" limits the AMD device's pool; anything else is ignored.
        Arc<Device> init(Device::Type, int32_t card, std::string_view args);
        // blocking wait for the work queued on the current AMD device (Executor::bench's sync)
        void sync(Device::Type);
    }// namespace device

}// namespace refactor::hardware
