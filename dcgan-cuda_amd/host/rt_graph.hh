// Runtime graph: owns the rt::Node instructions and orders them for execution
// (reference: src/runtime/graph.hh:15-58, src/runtime/nodes-list.hh:10-24).
#pragma once

#include <iosfwd>
#include <vector>

#include "node.hh"

namespace rt
{

class Graph
{
public:
    Graph() = default;
    ~Graph();
    Graph(const Graph&) = delete;
    Graph& operator=(const Graph&) = delete;

    // Takes ownership of the node.
    void add(Node* node);
    // Removes (and deletes) the node and, recursively, every node that consumes it.
    void remove(Node* node);
    const std::vector<Node*>& nodes() const { return nodes_; }

    // Every node `vals` depend on (themselves included), each after all of its predecessors.
    // Throws std::runtime_error on a cycle.
    std::vector<Node*> topological_sort(const std::vector<Node*>& vals) const;

private:
    std::vector<Node*> nodes_;
};

// An ordered instruction list without the OP_NOP placeholders; preds()[i] holds the positions
// of the instructions that instruction i waits for (placeholders are looked through).
class NodesList
{
public:
    explicit NodesList(const std::vector<Node*>& nodes);

    std::size_t size() const { return nodes_.size(); }
    const std::vector<Node*>& nodes() const { return nodes_; }
    const std::vector<std::vector<std::size_t>>& preds() const { return preds_; }

private:
    std::vector<Node*> nodes_;
    std::vector<std::vector<std::size_t>> preds_;
};

std::ostream& operator<<(std::ostream& os, const NodesList& list);

}  // namespace rt
