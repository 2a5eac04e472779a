// The graph-walking executor of the host mirror: a topology of lowered kernels (runtime::Node)
// and data edges, run in order on one device.  Follows
// src/03runtime/include/runtime/stream.h:24-52 and src/03runtime/src/stream.cc:6-98: an edge is
// either a blob of its own (global inputs and outputs, constants) or a range of the stream's
// stack, a node's workspace is a range of the same stack, and a routine receives raw device
// addresses in operator order.  Nothing is synchronised by run(); bench() and trace() are the
// per-node variants the reference's Executor::bench / Executor::trace are built on.
#pragma once

#include "rg_mirror/graph_topo.h"
#include "rg_mirror/hardware.h"
#include "rg_mirror/runtime.h"
#include <chrono>

namespace refactor::runtime {

    struct Edge {
        Arc<hardware::Device::Blob> blob;// null: the edge lives in the stack at stackOffset
        size_t stackOffset;
        std::string name;
    };

    // A HIP stream of its own in a Resources: while it is there, the AMD kernels' routines enqueue on
    // it instead of on the default stream (which cannot record a graph).  Created with default
    // flags and priority, so it stays ordered with the blocking copies of Device::Blob.
    class HipStream final : public Resource {
        void *_handle;

    public:
        HipStream();
        ~HipStream();
        HipStream(HipStream const &) = delete;
        static size_t typeId() noexcept;
        static ResourceBox build();
        size_t resourceTypeId() const noexcept final;
        std::string_view description() const noexcept final;
        void *handle() const noexcept { return _handle; }
    };

    class Stream {
        Arc<hardware::Device> _device;
        Arc<hardware::Device::Blob> _stack;
        Resources _resources;
        graph_topo::Graph<Node, Edge> _graph;
        void *_recorded = nullptr;                             // executable HIP graph of one run()
        std::vector<Arc<hardware::Device::Blob>> _recordedData;// the blobs its addresses point into
        void dropRecording() noexcept;

        // calls `visit(nodeIdx, inputs, outputs)` after each routine
        template<class F> void walk(F &&visit);

    public:
        Stream(Resources, size_t stackBytes, graph_topo::GraphTopo, std::vector<Node>, std::vector<Edge>,
               Arc<hardware::Device>);
        Stream(Stream &&) noexcept;
        Stream &operator=(Stream &&) noexcept;
        Stream(Stream const &) = delete;
        ~Stream();

        graph_topo::Graph<Node, Edge> const &graph() const noexcept { return _graph; }
        Arc<hardware::Device> const &device() const noexcept { return _device; }
        Arc<hardware::Device::Blob> setData(count_t edge, size_t bytes);
        void setData(count_t edge, Arc<hardware::Device::Blob>);
        void setData(count_t edge, void const *hostData, size_t bytes);
        Arc<hardware::Device::Blob> getData(count_t edge) const;
        // false if the edge has no blob of its own (stack edges cannot be read back)
        bool copyData(count_t edge, void *hostData, size_t bytes) const;

        void run();
        // host time of every node including `sync()` (null: enqueue time only), by node index
        std::vector<std::chrono::nanoseconds> bench(void (*sync)());
        void trace(std::function<void(count_t, void const *const *, void const *const *)> record);

        // AMD device only, no counterpart in the reference.  record() runs the graph once eagerly and
        // then records one run() of it — every launch of every routine — into an executable HIP graph;
        // replay() enqueues that whole graph with one call and does not wait for it.  The recording
        // holds the addresses of the moment: new contents go into the existing blobs
        // (getData(i)->copyFromHost), and anything that gives an edge another blob (setData) discards
        // the recording, after which replay() is an error until record() is called again.
        void record();
        bool recorded() const noexcept { return _recorded != nullptr; }
        void replay();
    };

}// namespace refactor::runtime
