// Graph topology container of the host mirror: which edges every node reads and writes, in an
// order in which the nodes can run.  Public surface follows
// src/01graph_topo/include/graph_topo/{container.h:8-77, builder.hpp:9-100}:
//   * edges are numbered: global inputs first, then per node (in node order) the edges only that
//     node reads ("local" edges, e.g. constants) followed by the edges it writes;
//   * iterating a GraphTopo yields (node index, input edge indices, output edge range);
//   * connections() lists the global outputs' edges first, then every node's inputs.
// The storage here is prefix-sum (CSR) tables, so a node is reachable by index in O(1) where the
// reference walks its iterator; Builder orders nodes deterministically (by key) where the
// reference follows hash-map order.
#pragma once

#include "rg_mirror/common.h"
#include <algorithm>
#include <iterator>
#include <map>
#include <set>
#include <unordered_map>

namespace refactor {

    using count_t = uint32_t;

    // [begin_, end_) of contiguous values
    template<class T> struct slice_t {
        T const *begin_, *end_;
        bool empty() const noexcept { return end_ == begin_; }
        size_t size() const noexcept { return static_cast<size_t>(end_ - begin_); }
        T const &operator[](size_t i) const noexcept { return begin_[i]; }
        T const &at(size_t i) const {
            ASSERT(i < size(), "Index out of range");
            return begin_[i];
        }
        T const *begin() const noexcept { return begin_; }
        T const *end() const noexcept { return end_; }
    };

    // the integers [begin_, end_)
    template<class T = size_t> struct range_t {
        T begin_, end_;
        struct Iterator {
            using iterator_category = std::forward_iterator_tag;
            using value_type = T;
            using difference_type = std::ptrdiff_t;
            using pointer = T const *;
            using reference = T;
            T v;
            T operator*() const noexcept { return v; }
            Iterator &operator++() noexcept { return ++v, *this; }
            Iterator operator++(int) noexcept { return Iterator{v++}; }
            bool operator!=(Iterator const &o) const noexcept { return v != o.v; }
            bool operator==(Iterator const &o) const noexcept { return v == o.v; }
        };
        bool empty() const noexcept { return end_ == begin_; }
        size_t size() const noexcept { return static_cast<size_t>(end_ - begin_); }
        T operator[](size_t i) const noexcept { return begin_ + static_cast<T>(i); }
        T at(size_t i) const {
            ASSERT(i < size(), "Index out of range");
            return (*this)[i];
        }
        Iterator begin() const noexcept { return {begin_}; }
        Iterator end() const noexcept { return {end_}; }
    };
    template<class T = size_t> range_t<T> range0_(T end) { return {0, end}; }

}// namespace refactor

namespace refactor::graph_topo {

    class GraphTopo {
        count_t _lenIn = 0, _lenOut = 0;
        std::vector<count_t> _connections;// global outputs, then the inputs of node 0, 1, ...
        std::vector<count_t> _inputBegin; // per node (+1): first of its inputs in _connections
        std::vector<count_t> _edgeBegin;  // per node (+1): its first own edge (local edges, then outputs)
        std::vector<count_t> _localCount; // per node: edges only it reads

    public:
        struct NodeRef {
            count_t idx;
            slice_t<count_t> inputs;
            range_t<count_t> outputs;
        };

        class Iterator {
            GraphTopo const *_g;
            count_t _idx;

        public:
            Iterator(GraphTopo const &g, count_t idx) noexcept : _g(&g), _idx(idx) {}
            bool operator==(Iterator const &o) const noexcept { return _idx == o._idx; }
            bool operator!=(Iterator const &o) const noexcept { return _idx != o._idx; }
            bool operator<(Iterator const &o) const noexcept { return _idx < o._idx; }
            Iterator &operator++() noexcept { return ++_idx, *this; }
            Iterator operator++(int) noexcept { return Iterator(*_g, _idx++); }
            NodeRef operator*() const { return _g->node(_idx); }
        };

        GraphTopo() : GraphTopo(0, 0) {}
        GraphTopo(count_t lenIn, count_t lenOut);
        // Appends a node (callers append in an order in which the nodes can run): the edge indices it
        // reads, how many of them nobody else produces (they are numbered now, before its outputs) and
        // how many edges it writes.  Returns the range of its outputs.
        range_t<count_t> pushNode(std::vector<count_t> const &inputs, count_t localEdges, count_t outputs);
        void setGlobalOutput(count_t i, count_t edge);
        // Every reader (node input or global output) of an edge that is a key of `map` reads the mapped
        // edge instead; returns how many connections changed
        // (src/01graph_topo/src/inplace_modifier.cc:92-101, there a separate InplaceModifier).
        size_t reconnect(std::unordered_map<count_t, count_t> const &map);

        NodeRef node(count_t idx) const;
        Iterator begin() const noexcept { return Iterator(*this, 0); }
        Iterator end() const noexcept { return Iterator(*this, static_cast<count_t>(nodeCount())); }
        size_t globalInputsCount() const noexcept { return _lenIn; }
        size_t globalOutputsCount() const noexcept { return _lenOut; }
        size_t nodeCount() const noexcept { return _localCount.size(); }
        size_t edgeCount() const noexcept { return _edgeBegin.back(); }
        range_t<count_t> globalInputs() const noexcept { return {0, _lenIn}; }
        slice_t<count_t> globalOutputs() const noexcept { return {_connections.data(), _connections.data() + _lenOut}; }
        slice_t<count_t> connections() const noexcept {
            return {_connections.data(), _connections.data() + _connections.size()};
        }
        // first edge index that belongs to node `idx` (its local edges start there)
        count_t firstEdgeOf(count_t idx) const { return _edgeBegin.at(idx); }
        count_t localEdgesOf(count_t idx) const { return _localCount.at(idx); }

        std::string toString() const;
    };

    template<class Node, class Edge>
    struct Graph {
        GraphTopo topology;
        std::vector<Node> nodes;
        std::vector<Edge> edges;
    };

    template<class EdgeKey>
    struct BuilderNode {
        std::vector<EdgeKey> inputs, outputs;
    };

    // Keys -> indices.  A node is placed once every input it has is either numbered already or
    // produced by nobody (then it becomes one of the node's local edges); among the nodes that
    // can be placed, the one with the smallest key goes first.  A cycle is a RUNTIME_ERROR.
    template<class NodeKey, class Node, class EdgeKey, class Edge>
    struct Builder {
        std::map<NodeKey, BuilderNode<EdgeKey>> topology;
        std::vector<EdgeKey> globalInputs, globalOutputs;
        std::map<NodeKey, Node> nodes;
        std::map<EdgeKey, Edge> edges;

        Graph<Node, Edge> build() {
            Graph<Node, Edge> ans{
                GraphTopo(static_cast<count_t>(globalInputs.size()), static_cast<count_t>(globalOutputs.size())), {}, {}};
            std::map<EdgeKey, count_t> index;
            auto number = [&](EdgeKey const &key) {
                index[key] = static_cast<count_t>(ans.edges.size());
                if (auto it = edges.find(key); it != edges.end()) {
                    ans.edges.emplace_back(std::move(it->second));
                } else {
                    ans.edges.emplace_back();
                }
            };
            std::set<EdgeKey> produced(globalInputs.begin(), globalInputs.end());
            for (auto const &[key, n] : topology) produced.insert(n.outputs.begin(), n.outputs.end());
            for (auto const &key : globalInputs) number(key);

            std::set<NodeKey> placed;
            while (placed.size() < topology.size()) {
                bool progress = false;
                for (auto const &[key, n] : topology) {
                    if (placed.count(key)) continue;
                    std::vector<EdgeKey> local;
                    bool ready = true;
                    for (auto const &e : n.inputs) {
                        if (index.count(e)) continue;
                        if (produced.count(e)) {
                            ready = false;
                            break;
                        }
                        if (std::find(local.begin(), local.end(), e) == local.end()) local.push_back(e);
                    }
                    if (!ready) continue;
                    for (auto const &e : local) number(e);
                    for (auto const &e : n.outputs) number(e);
                    std::vector<count_t> inputs;
                    inputs.reserve(n.inputs.size());
                    for (auto const &e : n.inputs) inputs.push_back(index.at(e));
                    ans.topology.pushNode(inputs, static_cast<count_t>(local.size()), static_cast<count_t>(n.outputs.size()));
                    ans.nodes.emplace_back(std::move(nodes.at(key)));
                    placed.insert(key);
                    progress = true;
                    break;// smallest ready key first, then look again from the start
                }
                if (!progress) RUNTIME_ERROR("graph_topo::Builder: the nodes cannot be ordered (cycle)");
            }
            for (size_t i = 0; i < globalOutputs.size(); ++i)
                ans.topology.setGlobalOutput(static_cast<count_t>(i), index.at(globalOutputs[i]));
            return ans;
        }
    };

}// namespace refactor::graph_topo
