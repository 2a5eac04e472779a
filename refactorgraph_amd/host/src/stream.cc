// runtime::Stream of the host mirror (see rg_mirror/stream.h).
#include "rg_mirror/stream.h"
#include "rg_hip.h"

#define HIP_ASSERT(CALL)                                                                              \
    if (auto status_ = (CALL); status_ != 0) {                                                        \
        RUNTIME_ERROR(::refactor::detail::cat("hip failed on \"" #CALL "\" with \"",                  \
                                              rg_hip_error_string(status_), "\" (", status_, ")"));   \
    }

namespace refactor::runtime {

    Stream::Stream(Resources resources, size_t stackBytes, graph_topo::GraphTopo topology, std::vector<Node> nodes,
                   std::vector<Edge> edges, Arc<hardware::Device> device)
        : _device(std::move(device)),
          _stack(_device->malloc(stackBytes)),
          _resources(std::move(resources)),
          _graph{std::move(topology), std::move(nodes), std::move(edges)} {
        ASSERT(_graph.nodes.size() == _graph.topology.nodeCount(), "one runtime node per topology node");
        ASSERT(_graph.edges.size() == _graph.topology.edgeCount(), "one runtime edge per topology edge");
    }

    HipStream::HipStream() : _handle(nullptr) { HIP_ASSERT(rg_hip_stream_create(&_handle)); }
    HipStream::~HipStream() { rg_hip_stream_destroy(_handle); }
    size_t HipStream::typeId() noexcept {
        static uint8_t ID = 1;
        return reinterpret_cast<size_t>(&ID);
    }
    ResourceBox HipStream::build() { return std::make_unique<HipStream>(); }
    size_t HipStream::resourceTypeId() const noexcept { return typeId(); }
    std::string_view HipStream::description() const noexcept { return "HIP stream the routines enqueue on"; }

    Stream::Stream(Stream &&o) noexcept
        : _device(std::move(o._device)), _stack(std::move(o._stack)), _resources(std::move(o._resources)),
          _graph(std::move(o._graph)), _recorded(std::exchange(o._recorded, nullptr)),
          _recordedData(std::move(o._recordedData)) {}
    Stream &Stream::operator=(Stream &&o) noexcept {
        if (this != &o) {
            dropRecording();
            _device = std::move(o._device);
            _stack = std::move(o._stack);
            _resources = std::move(o._resources);
            _graph = std::move(o._graph);
            _recorded = std::exchange(o._recorded, nullptr);
            _recordedData = std::move(o._recordedData);
        }
        return *this;
    }
    Stream::~Stream() { dropRecording(); }

    void Stream::dropRecording() noexcept {
        if (_recorded) {
            rg_hip_sync();// a replay may still be running
            rg_hip_graph_destroy(std::exchange(_recorded, nullptr));
        }
        _recordedData.clear();
    }

    Arc<hardware::Device::Blob> Stream::setData(count_t edge, size_t bytes) {
        dropRecording();
        return _graph.edges.at(edge).blob = _device->malloc(bytes);
    }
    void Stream::setData(count_t edge, Arc<hardware::Device::Blob> blob) {
        dropRecording();
        _graph.edges.at(edge).blob = std::move(blob);
    }
    void Stream::setData(count_t edge, void const *hostData, size_t bytes) {
        dropRecording();
        auto blob = _device->malloc(bytes);
        blob->copyFromHost(hostData, bytes);
        _graph.edges.at(edge).blob = std::move(blob);
    }
    Arc<hardware::Device::Blob> Stream::getData(count_t edge) const { return _graph.edges.at(edge).blob; }
    bool Stream::copyData(count_t edge, void *hostData, size_t bytes) const {
        auto const &blob = _graph.edges.at(edge).blob;
        if (!blob) return false;
        blob->copyToHost(hostData, bytes);
        return true;
    }

    template<class F> void Stream::walk(F &&visit) {
        auto *stack = _stack->get<uint8_t>();
        std::vector<void *> addresses;
        auto address = [&](count_t e) -> void * {
            auto const &edge = _graph.edges[e];
            return edge.blob ? edge.blob->get() : stack + edge.stackOffset;
        };
        for (auto [idx, inputs, outputs] : _graph.topology) {
            addresses.clear();
            for (auto e : inputs) addresses.push_back(address(e));
            for (auto e : outputs) addresses.push_back(address(e));
            auto const *in = const_cast<void const *const *>(addresses.data());
            auto *const *out = addresses.data() + inputs.size();
            auto const &node = _graph.nodes[idx];
            _device->setContext();
            auto const t0 = std::chrono::steady_clock::now();
            node.routine(_resources, stack + node.workspaceOffset, in, out);
            visit(idx, in, out, t0);
        }
    }

    void Stream::run() {
        walk([](count_t, void const *const *, void *const *, std::chrono::steady_clock::time_point) {});
    }

    std::vector<std::chrono::nanoseconds> Stream::bench(void (*sync)()) {
        std::vector<std::chrono::nanoseconds> ans(_graph.nodes.size());
        walk([&](count_t idx, void const *const *, void *const *, std::chrono::steady_clock::time_point t0) {
            if (sync) sync();
            ans[idx] = std::chrono::steady_clock::now() - t0;
        });
        return ans;
    }

    void Stream::record() {
        ASSERT(_device->type() == hardware::Device::Type::Amd, "only a stream on the AMD device records HIP graphs");
        dropRecording();
        auto *own = _resources.fetchOrStore<HipStream>();
        run();// everything that initialises itself on first use has done so before the recording
        HIP_ASSERT(rg_hip_stream_sync(own->handle()));
        HIP_ASSERT(rg_hip_graph_begin(own->handle()));
        try {
            run();
        } catch (...) {
            void *broken = nullptr;
            rg_hip_graph_end(own->handle(), &broken);
            rg_hip_graph_destroy(broken);
            throw;
        }
        HIP_ASSERT(rg_hip_graph_end(own->handle(), &_recorded));
        _recordedData.push_back(_stack);
        for (auto const &e : _graph.edges)
            if (e.blob) _recordedData.push_back(e.blob);
    }

    void Stream::replay() {
        ASSERT(_recorded, "nothing recorded (record() first; setData discards a recording)");
        _device->setContext();
        HIP_ASSERT(rg_hip_graph_launch(_recorded, _resources.fetch<HipStream>()->handle()));
    }

    void Stream::trace(std::function<void(count_t, void const *const *, void const *const *)> record) {
        walk([&](count_t idx, void const *const *in, void *const *out, std::chrono::steady_clock::time_point) {
            record(idx, in, const_cast<void const *const *>(out));
        });
    }

}// namespace refactor::runtime
