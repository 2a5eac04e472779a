// kernel::Graph::lower and the two stack allocators (see rg_mirror/graph.h).
#include "rg_mirror/graph.h"
#include <map>
#include <unordered_set>
#include <utility>

namespace refactor::kernel {

    namespace {
        constexpr size_t OFF_STACK = SIZE_MAX, GLOBAL_OUTPUT = SIZE_MAX - 1;

        // how often every edge is read (by nodes or as a global output)
        std::vector<size_t> readers(graph_topo::GraphTopo const &topology, size_t edges) {
            std::vector<size_t> rc(edges, 0);
            for (auto e : topology.connections()) ++rc.at(e);
            return rc;
        }
    }// namespace

    AllocScheme flatAllocate(graph_topo::GraphTopo const &topology, std::vector<runtime::Node> nodes,
                             std::vector<Edge> const &edges, size_t alignBytes) {
        auto const rc = readers(topology, edges.size());
        auto const globalOutputs_ = topology.globalOutputs();
        std::unordered_set<count_t> globalOutputs(globalOutputs_.begin(), globalOutputs_.end());
        std::vector<runtime::Edge> edges_(edges.size(), runtime::Edge{nullptr, OFF_STACK, {}});
        size_t size = 0;
        for (auto [idx, inputs, outputs] : topology) {
            for (auto e : outputs) {
                if (!rc[e]) continue;// nobody reads it: stays off the stack
                if (globalOutputs.count(e)) {
                    edges_[e].stackOffset = GLOBAL_OUTPUT;
                } else {
                    edges_[e].stackOffset = size;
                    size += hardware::alignBytes(edges[e].size, alignBytes);
                }
            }
            if (auto &node = nodes[idx]; node.workspaceOffset) {
                auto const bytes = std::exchange(node.workspaceOffset, size);
                size += hardware::alignBytes(bytes, alignBytes);
            }
        }
        return {size, std::move(nodes), std::move(edges_)};
    }

    AllocScheme reusableAllocate(graph_topo::GraphTopo const &topology, std::vector<runtime::Node> nodes,
                                 std::vector<Edge> const &edges, size_t alignBytes) {
        auto rc = readers(topology, edges.size());
        auto const globalOutputs_ = topology.globalOutputs();
        std::unordered_set<count_t> globalOutputs(globalOutputs_.begin(), globalOutputs_.end());
        std::vector<runtime::Edge> edges_(edges.size(), runtime::Edge{nullptr, OFF_STACK, {}});
        hardware::OffsetCalculator calculator(alignBytes);
        for (auto [idx, inputs, outputs] : topology) {
            for (auto e : outputs) {
                if (globalOutputs.count(e)) {
                    edges_[e].stackOffset = GLOBAL_OUTPUT;
                } else {
                    edges_[e].stackOffset = calculator.alloc(edges[e].size);
                }
            }
            // the workspace is live only while this node runs: outputs and inputs stay allocated around it
            if (auto &node = nodes[idx]; node.workspaceOffset) {
                auto const bytes = node.workspaceOffset;
                node.workspaceOffset = calculator.alloc(bytes);
                calculator.free(node.workspaceOffset, bytes);
            }
            for (auto e : outputs)
                if (!rc[e] && edges_[e].stackOffset < GLOBAL_OUTPUT) calculator.free(edges_[e].stackOffset, edges[e].size);
            for (auto e : inputs) {
                ASSERT(rc[e], "an edge is released more often than it is read");
                if (!--rc[e] && edges_[e].stackOffset < GLOBAL_OUTPUT) calculator.free(edges_[e].stackOffset, edges[e].size);
            }
        }
        return {calculator.peak(), std::move(nodes), std::move(edges_)};
    }

    Graph::Graph(graph_topo::GraphTopo topology, std::vector<_N> nodes, std::vector<_E> edges) noexcept
        : _internal{std::move(topology), std::move(nodes), std::move(edges)} {}

    runtime::Stream Graph::lower(Arc<hardware::Device> device, Allocator allocator) const {
        device->setContext();
        runtime::Resources res;

        std::vector<runtime::Node> nodes;
        nodes.reserve(_internal.nodes.size());
        for (auto const &node : _internal.nodes) {
            if (node.kernel) {
                nodes.emplace_back(node.kernel->lower(res));
            } else {
                nodes.emplace_back(runtime::emptyRoutine);
            }
        }

        auto const align = device->type() == hardware::Device::Type::Amd ? size_t(256) : size_t(32);
        auto [stack, nodes_, edges_] = allocator(_internal.topology, std::move(nodes), _internal.edges, align);

        // A constant is uploaded once per (device, host blob) and shared by every stream lowered
        // afterwards; the entry goes away with the last stream that uses it.  The map is looked up by
        // address, so an entry also remembers whose addresses these were: a host blob or device that
        // was freed and whose address has been reused since does not match, and the constant is
        // uploaded again (the reference keys by the shared pointers themselves, which keeps every
        // constant ever lowered alive).  Single-threaded like the rest of the lowering.
        struct Uploaded {
            std::weak_ptr<hardware::Device> device;
            std::weak_ptr<Blob> host;
            std::weak_ptr<hardware::Device::Blob> copy;
        };
        static std::map<std::pair<hardware::Device *, Blob const *>, Uploaded> uploaded;
        std::erase_if(uploaded, [](auto const &kv) { return kv.second.copy.expired(); });
        auto const sameOwner = [](auto const &weak, auto const &shared) {
            return !weak.owner_before(shared) && !shared.owner_before(weak);
        };

        for (size_t i = 0; i < edges_.size(); ++i) {
            auto const &edge = _internal.edges[i];
            edges_[i].name = edge.name;
            if (edge.data) {
                auto &slot = uploaded[{device.get(), edge.data.get()}];
                auto blob = slot.copy.lock();
                if (!blob || !sameOwner(slot.device, device) || !sameOwner(slot.host, edge.data)) {
                    blob = device->malloc(edge.size);
                    blob->copyFromHost(edge.data->get<void>(), edge.size);
                    slot = Uploaded{device, edge.data, blob};
                }
                edges_[i].blob = std::move(blob);
            } else if (edges_[i].stackOffset == GLOBAL_OUTPUT) {
                edges_[i].blob = device->malloc(edge.size);
            }
        }
        return runtime::Stream(std::move(res), stack, _internal.topology, std::move(nodes_), std::move(edges_),
                               std::move(device));
    }

}// namespace refactor::kernel
