// From a graph of kernels to a runnable Stream.  Follows
// src/04kernel/include/kernel/{graph.h:8-46, allocators.h} and src/04kernel/src/{graph.cc:21-84,
// allocators/flat_allocator.cpp:6-43, allocators/reusable_allocator.cpp:6-59}: every kernel is
// lowered once, an Allocator turns edge sizes and workspace sizes into offsets of one stack,
// constants are uploaded (once per device and blob), global outputs get blobs of their own.
#pragma once

#include "rg_mirror/kernel.h"
#include "rg_mirror/stream.h"

namespace refactor::kernel {

    struct Node {
        KernelBox kernel;// null: nothing to run (runtime::emptyRoutine)
        std::string name;
    };

    struct Edge {
        Arc<Blob> data;// constant contents, or null
        size_t size;   // bytes
        std::string name;
    };

    struct AllocScheme {
        size_t stack;
        std::vector<runtime::Node> nodes;// workspace sizes replaced by stack offsets
        std::vector<runtime::Edge> edges;// stackOffset: an offset, SIZE_MAX (not on the stack: global input,
                                         // constant, unused) or SIZE_MAX - 1 (global output: gets a blob)
    };

    using Allocator = AllocScheme (*)(graph_topo::GraphTopo const &, std::vector<runtime::Node>,
                                      std::vector<Edge> const &, size_t alignBytes);

    // every produced edge and every workspace gets a range of its own
    AllocScheme flatAllocate(graph_topo::GraphTopo const &, std::vector<runtime::Node>, std::vector<Edge> const &, size_t);
    // ranges are handed back once their last reader has run and are used again (hardware::OffsetCalculator)
    AllocScheme reusableAllocate(graph_topo::GraphTopo const &, std::vector<runtime::Node>, std::vector<Edge> const &, size_t);

    struct Graph {
        using _N = Node;
        using _E = Edge;
        using _G = graph_topo::Graph<_N, _E>;

        _G _internal;

        Graph(graph_topo::GraphTopo, std::vector<_N>, std::vector<_E>) noexcept;
        // Offsets are aligned to 32 bytes (src/04kernel/src/graph.cc:49), to 256 on the AMD device, whose
        // kernels use 128-bit accesses and whose pool is aligned the same way.
        runtime::Stream lower(Arc<hardware::Device>, Allocator) const;
    };

}// namespace refactor::kernel
