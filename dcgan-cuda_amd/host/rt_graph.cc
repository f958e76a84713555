#include "rt_graph.hh"

#include <algorithm>
#include <map>
#include <ostream>
#include <stdexcept>
#include <unordered_map>
#include <unordered_set>

namespace rt
{

Graph::~Graph()
{
    for (Node* n : nodes_)
        delete n;
}

void Graph::add(Node* node)
{
    if (!node)
        throw std::runtime_error("rt::Graph::add: null node");
    nodes_.push_back(node);
}

void Graph::remove(Node* node)
{
    auto it = std::find(nodes_.begin(), nodes_.end(), node);
    if (it == nodes_.end())
        return;
    nodes_.erase(it);
    for (Node* p : node->preds)
        p->succs.erase(std::remove(p->succs.begin(), p->succs.end(), node), p->succs.end());
    const std::vector<Node*> consumers = node->succs;  // remove() edits node->succs
    for (Node* s : consumers)
        remove(s);
    delete node;
}

std::vector<Node*> Graph::topological_sort(const std::vector<Node*>& vals) const
{
    // Depth-first post-order over the predecessor edges: linear time, and the order of `vals`
    // and of each node's operands decides ties, so the schedule is deterministic.
    std::vector<Node*> order;
    std::unordered_map<Node*, int> state;  // 1 = on the stack, 2 = emitted
    std::vector<std::pair<Node*, std::size_t>> stack;
    for (Node* root : vals)
    {
        if (!root || state[root] == 2)
            continue;
        stack.emplace_back(root, 0);
        state[root] = 1;
        while (!stack.empty())
        {
            auto& [n, next] = stack.back();
            if (next < n->preds.size())
            {
                Node* p = n->preds[next++];
                const int st = state[p];
                if (st == 1)
                    throw std::runtime_error("Topological sort failed");
                if (st == 0)
                {
                    state[p] = 1;
                    stack.emplace_back(p, 0);
                }
            }
            else
            {
                state[n] = 2;
                order.push_back(n);
                stack.pop_back();
            }
        }
    }
    return order;
}

namespace
{
void real_preds(Node* n, std::vector<Node*>& out)
{
    for (Node* p : n->preds)
    {
        if (p->type == Node::OP_NOP)
            real_preds(p, out);
        else
            out.push_back(p);
    }
}
}  // namespace

NodesList::NodesList(const std::vector<Node*>& nodes)
{
    std::unordered_map<Node*, std::size_t> pos;
    for (Node* n : nodes)
        if (n->type != Node::OP_NOP)
        {
            pos[n] = nodes_.size();
            nodes_.push_back(n);
        }
    for (Node* n : nodes_)
    {
        std::vector<Node*> ps;
        real_preds(n, ps);
        std::vector<std::size_t> idx;
        for (Node* p : ps)
        {
            auto it = pos.find(p);
            if (it == pos.end())
                throw std::runtime_error("rt::NodesList: predecessor missing from the list");
            idx.push_back(it->second);
        }
        preds_.push_back(std::move(idx));
    }
}

std::ostream& operator<<(std::ostream& os, const NodesList& list)
{
    std::map<const dbl_t*, std::string> names;
    auto name = [&](const dbl_t* p) -> std::string {
        if (!p)
            return "-";
        auto it = names.find(p);
        if (it == names.end())
            it = names.emplace(p, "t" + std::to_string(names.size())).first;
        return it->second;
    };
    for (std::size_t i = 0; i < list.size(); ++i)
    {
        const Node* n = list.nodes()[i];
        os << i << ": " << Node::name_of(n->type) << " (" << name(n->in1) << ", " << name(n->in2) << ", "
           << name(n->in3) << ") -> " << name(n->out1) << "  after {";
        for (std::size_t p : list.preds()[i])
            os << ' ' << p;
        os << " }\n";
    }
    return os;
}

}  // namespace rt
