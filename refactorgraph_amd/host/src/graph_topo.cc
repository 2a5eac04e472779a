// GraphTopo storage: prefix tables over the nodes (see rg_mirror/graph_topo.h).
#include "rg_mirror/graph_topo.h"

namespace refactor::graph_topo {

    GraphTopo::GraphTopo(count_t lenIn, count_t lenOut)
        : _lenIn(lenIn), _lenOut(lenOut), _connections(lenOut, 0), _inputBegin{lenOut}, _edgeBegin{lenIn} {}

    range_t<count_t> GraphTopo::pushNode(std::vector<count_t> const &inputs, count_t localEdges, count_t outputs) {
        auto const firstOwn = _edgeBegin.back(), firstOutput = firstOwn + localEdges;
        for (auto e : inputs) ASSERT(e < firstOutput, "a node reads an edge that is numbered after its own");
        _connections.insert(_connections.end(), inputs.begin(), inputs.end());
        _inputBegin.push_back(static_cast<count_t>(_connections.size()));
        _edgeBegin.push_back(firstOutput + outputs);
        _localCount.push_back(localEdges);
        return {firstOutput, firstOutput + outputs};
    }

    void GraphTopo::setGlobalOutput(count_t i, count_t edge) {
        ASSERT(i < _lenOut, "no such global output");
        ASSERT(edge < edgeCount(), "no such edge");
        _connections[i] = edge;
    }

    size_t GraphTopo::reconnect(std::unordered_map<count_t, count_t> const &map) {
        size_t changed = 0;
        for (auto &c : _connections)
            if (auto it = map.find(c); it != map.end()) {
                c = it->second;
                ++changed;
            }
        return changed;
    }

    GraphTopo::NodeRef GraphTopo::node(count_t idx) const {
        ASSERT(idx < nodeCount(), "no such node");
        auto const *c = _connections.data();
        return {
            idx,
            {c + _inputBegin[idx], c + _inputBegin[idx + 1]},
            {_edgeBegin[idx] + _localCount[idx], _edgeBegin[idx + 1]},
        };
    }

    std::string GraphTopo::toString() const {
        std::ostringstream os;
        auto list = [&](auto const &xs) {
            for (auto x : xs) os << ' ' << x;
        };
        os << "inputs:";
        list(globalInputs());
        os << '\n';
        for (auto [idx, inputs, outputs] : *this) {
            os << "node " << idx << ":";
            list(inputs);
            os << " ->";
            list(outputs);
            os << '\n';
        }
        os << "outputs:";
        list(globalOutputs());
        os << '\n';
        return os.str();
    }

}// namespace refactor::graph_topo
