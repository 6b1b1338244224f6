// Dependency graph of buffers and its cache traces.
//
// Same results as the reference's OptGraph / GraphTranslator
// (src/modules/graph/opt_graph.rs:8-44, opt_graph/optimize.rs:7-129,
// graph_translator.rs:9-58), computed from per-node consumer lists instead of
// rescanning all later nodes for every question.
#pragma once

#include <algorithm>
#include <cstddef>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "core.hpp"

namespace custos {

struct Node {
    size_t idx = 0;
    std::vector<size_t> deps;
    size_t len = 0;
    bool skip = false;  // set by Buffer::checkpoint(): never part of a trace
    bool is_leaf() const { return deps.empty(); }
};

// Nodes whose buffers could share one allocation: `cache_idx` first, then the
// chain that follows it.
struct CacheTrace {
    size_t cache_idx = 0;
    std::vector<size_t> use_cache_idxs;
    bool operator==(const CacheTrace& o) const {
        return cache_idx == o.cache_idx && use_cache_idxs == o.use_cache_idxs;
    }
};

class OptGraph {
   public:
    std::vector<Node> nodes;

    size_t add_leaf(size_t len) { return add_node(len, {}); }

    size_t add_node(size_t len, std::vector<size_t> deps) {
        const size_t idx = nodes.size();
        consumers_.emplace_back();
        // one entry per consumer even when it names the node twice (deps: [c, c])
        std::vector<size_t> uniq = deps;
        std::sort(uniq.begin(), uniq.end());
        uniq.erase(std::unique(uniq.begin(), uniq.end()), uniq.end());
        for (size_t d : uniq)
            if (d < idx) consumers_[d].push_back(idx);
        nodes.push_back(Node{idx, std::move(deps), len, false});
        return idx;
    }

    const Node& node(size_t idx) const { return nodes[idx]; }

    // A node starts or continues a shared allocation only while at most one
    // later node of the same length reads it (optimize.rs:110-129).
    bool is_path_optimizable(const Node& check_at) const {
        if (check_at.is_leaf()) return false;
        size_t same_len = 0;
        for (size_t c : consumers_[check_at.idx])
            if (nodes[c].len == check_at.len && ++same_len > 1) return false;
        return true;
    }

    // The chain after `trace_at`: repeatedly the first later node that is not
    // skipped, reads the current node and has the start's length; the first
    // node that is itself not optimizable still joins, then the chain ends
    // (optimize.rs:57-88).
    std::vector<size_t> trace_cache_path_raw(const Node& trace_at) const {
        std::vector<size_t> trace;
        if (!is_path_optimizable(trace_at)) return trace;
        size_t idx = trace_at.idx;
        for (;;) {
            size_t next = nodes.size();
            for (size_t c : consumers_[idx]) {  // ascending node order
                if (nodes[c].skip || nodes[c].len != trace_at.len) continue;
                next = c;
                break;
            }
            if (next == nodes.size()) break;
            idx = next;
            trace.push_back(idx);
            if (!is_path_optimizable(nodes[idx])) break;
        }
        return trace;
    }

    // Disjoint traces over all non-leaf nodes in node order (optimize.rs:19-53).
    std::vector<CacheTrace> cache_traces() const {
        std::vector<CacheTrace> traces;
        std::unordered_set<size_t> visited;
        for (const Node& node : nodes) {
            if (node.is_leaf() || node.skip || visited.count(node.idx)) continue;
            std::vector<size_t> raw = trace_cache_path_raw(node);
            if (raw.empty()) continue;
            CacheTrace t;
            t.cache_idx = node.idx;
            for (size_t idx : raw)
                if (visited.insert(idx).second) t.use_cache_idxs.push_back(idx);
            traces.push_back(std::move(t));
        }
        return traces;
    }

   private:
    std::vector<std::vector<size_t>> consumers_;  // later nodes reading node i, ascending
};

// Buffer id <-> node index <-> lazy cursor (graph_translator.rs:9-58).
struct GraphTranslator {
    std::unordered_map<UniqueId, size_t> buf_id_to_idx;
    std::unordered_map<size_t, UniqueId> idx_to_buf_id;
    std::unordered_map<size_t, UniqueId> idx_to_cursor;
    size_t next_idx = 0;
    OptGraph opt_graph;

    void add_leaf(size_t len) {
        opt_graph.add_leaf(len);
        next_idx = opt_graph.nodes.size();
    }

    void add_node(size_t len, const std::vector<Id>& deps) {
        std::vector<size_t> idxs;
        for (const Id& id : deps) {
            auto it = buf_id_to_idx.find(id.id);
            if (it == buf_id_to_idx.end()) throw Error(DeviceError::GraphOptimization);
            idxs.push_back(it->second);
        }
        opt_graph.add_node(len, std::move(idxs));
        next_idx = opt_graph.nodes.size();
    }

    std::vector<CacheTrace> to_cursor_cache_traces(const std::vector<CacheTrace>& traces) const {
        std::vector<CacheTrace> out;
        for (const CacheTrace& t : traces) {
            CacheTrace c;
            c.cache_idx = static_cast<size_t>(idx_to_cursor.at(t.cache_idx));
            for (size_t i : t.use_cache_idxs) c.use_cache_idxs.push_back(static_cast<size_t>(idx_to_cursor.at(i)));
            out.push_back(std::move(c));
        }
        return out;
    }
};

}  // namespace custos
