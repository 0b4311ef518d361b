// Directed graph over layer indices for DAGModel (the interface the reference's include/small/utils/Graph.hpp
// offers its model classes: vertices are 0..n-1, edges keep insertion order, which fixes the order of a
// layer's inputs).
#pragma once

#include <algorithm>
#include <cstddef>
#include <deque>
#include <stdexcept>
#include <vector>

namespace small
{

class Graph
{
public:
    typedef size_t VertexID;

    Graph() {}

    size_t get_num_nodes() const { return m_out.size(); }

    void add_vertex(VertexID v)
    {
        if (v >= m_out.size())
        {
            m_out.resize(v + 1);
            m_in.resize(v + 1);
        }
    }

    void add_edge(VertexID src, VertexID dst)
    {
        add_vertex(std::max(src, dst));
        m_out[src].push_back(dst);
        m_in[dst].push_back(src);
    }

    std::vector<VertexID> const &out_neighbors(VertexID v) const { return m_out.at(v); }
    std::vector<VertexID> const &in_neighbors(VertexID v) const { return m_in.at(v); }

    std::vector<VertexID> sources() const
    {
        std::vector<VertexID> r;
        for (VertexID v = 0; v < m_in.size(); ++v)
            if (m_in[v].empty()) r.push_back(v);
        return r;
    }

    std::vector<VertexID> sinks() const
    {
        std::vector<VertexID> r;
        for (VertexID v = 0; v < m_out.size(); ++v)
            if (m_out[v].empty()) r.push_back(v);
        return r;
    }

    // widest breadth-first level reached from root (Graph.hpp:120-154 of the reference; sizes the buffer pool)
    size_t max_width(VertexID root) const
    {
        size_t width = 1;
        std::vector<char> seen(get_num_nodes(), 0);
        std::vector<VertexID> level{root}, next;
        seen[root] = 1;
        while (!level.empty())
        {
            next.clear();
            for (VertexID u : level)
                for (VertexID v : m_out[u])
                    if (!seen[v]) { seen[v] = 1; next.push_back(v); }
            level.swap(next);
            width = std::max(width, level.size());
        }
        return width;
    }

    // An order in which every vertex follows all its predecessors.  Layer graphs are built in file order with
    // edges pointing forward, so ascending index order is kept whenever it is valid (Kahn's algorithm that
    // always takes the smallest ready vertex); a cycle raises std::invalid_argument.
    std::deque<VertexID> topological_sort() const
    {
        const size_t n = get_num_nodes();
        std::vector<size_t> pending(n);
        std::vector<VertexID> ready;
        for (VertexID v = 0; v < n; ++v)
        {
            pending[v] = m_in[v].size();
            if (pending[v] == 0) ready.push_back(v);
        }
        std::deque<VertexID> order;
        while (!ready.empty())
        {
            auto it = std::min_element(ready.begin(), ready.end());
            const VertexID u = *it;
            ready.erase(it);
            order.push_back(u);
            for (VertexID v : m_out[u])
                if (--pending[v] == 0) ready.push_back(v);
        }
        if (order.size() != n) throw std::invalid_argument("Graph::topological_sort ERROR: the graph has a cycle.");
        return order;
    }

private:
    std::vector<std::vector<VertexID>> m_out, m_in;
};

} // namespace small
