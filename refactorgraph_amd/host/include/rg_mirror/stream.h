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

    class Stream {
        Arc<hardware::Device> _device;
        Arc<hardware::Device::Blob> _stack;
        Resources _resources;
        graph_topo::Graph<Node, Edge> _graph;

        // calls `visit(nodeIdx, inputs, outputs)` after each routine
        template<class F> void walk(F &&visit);

    public:
        Stream(Resources, size_t stackBytes, graph_topo::GraphTopo, std::vector<Node>, std::vector<Edge>,
               Arc<hardware::Device>);

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
    };

}// namespace refactor::runtime
