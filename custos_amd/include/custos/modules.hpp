// The module stack: Base, Cached, Lazy, Graph, Autograd.
//
// Modules compose at compile time, `HIP<Autograd<Graph<Lazy<Base>>>>`, like the
// reference's (src/modules/{base,cached,lazy,graph,autograd}.rs).  Every module
// implements the same set of "features" and passes what it does not handle to
// the module it wraps (`modules`), as the reference does with its pass-down
// macros in src/features.rs.
#pragma once

#include <algorithm>
#include <cstddef>
#include <functional>
#include <memory>
#include <typeindex>
#include <vector>

#include "buffer.hpp"
#include "core.hpp"
#include "opt_graph.hpp"

namespace custos {

struct Operation {
    std::vector<Id> arg_ids;
    // looks its arguments up by id in `buffers`; `device` points to the concrete device
    std::function<void(Buffers& buffers, void* device)> op;
    // unary op hint (src/op_hint.rs): type-erased UnaryHint<T> + its element type
    OpHintKind hint_kind = OpHintKind::None;
    std::shared_ptr<void> unary_hint;
    std::type_index hint_type = std::type_index(typeid(void));
    // expression hint of any arity (type-erased ExprHint<T>): which arguments the
    // expression reads, in operand order, and which one it writes
    std::shared_ptr<void> expr_hint;
    std::type_index expr_type = std::type_index(typeid(void));
    std::vector<int> in_args;
    int out_arg = -1;
    // text of the expression a fused operation computes, over markers a, b, c, d
    std::string fused_source;

    static Operation no_op() {
        Operation o;
        o.op = [](Buffers&, void*) {};
        return o;
    }
};

struct AnyOpHint {
    OpHintKind kind = OpHintKind::None;
    std::shared_ptr<void> unary;
    std::type_index type = std::type_index(typeid(void));
};

struct AnyExprHint {
    std::shared_ptr<void> hint;
    std::type_index type = std::type_index(typeid(void));
    std::vector<int> in_args;
    int out_arg = -1;
};

template <class T>
AnyOpHint erase_hint(OpHint<T> h) {
    return AnyOpHint{h.kind, std::static_pointer_cast<void>(h.unary), std::type_index(typeid(T))};
}

class Tape;
class Gradients;
struct AutogradState;

// ---------------------------------------------------------------------------
// Base: runs operations immediately, allocates on retrieve (src/modules/base.rs)
// ---------------------------------------------------------------------------
struct Base {
    template <class D>
    void setup(D&) {}
    // called by the device's destructor while it can still free memory
    template <class D>
    void teardown(D&) {}

    // `Retrieve::retrieve`: a fresh zeroed allocation (base.rs:103-130); not zero-filled
    // when the caller is an operation that overwrites all of it right away
    template <class T, class D>
    Buffer<T, D> retrieve(D& dev, size_t len, const std::vector<Id>&, const std::vector<bool>&) {
        cursor_++;
        uint64_t ptr = dev.alloc_raw(len * sizeof(T), /*zeroed=*/!dev.output_hint(), len);
        return Buffer<T, D>::from_parts(&dev, ptr, len, Id{ptr, len}, AllocFlag::None);
    }
    template <class T, class D>
    void on_new_buffer(D&, const Buffer<T, D>&) {}
    void on_drop_buffer(Id) {}
    void on_release_cached(uint64_t) {}

    // Base never records (base.rs:53-62): the device calls the closure directly.
    template <class D>
    void add_op(D& dev, Operation&& op) {
        Buffers none;
        op.op(none, &dev);
    }
    size_t ops_count() const { return 0; }
    void set_lazy_enabled(bool) {}
    bool is_lazy_enabled() const { return false; }
    void set_op_hint(AnyOpHint) {}
    void set_expr_hint(AnyExprHint) {}
    template <class D>
    void elementwise_fusing(D&, const GraphTranslator*, const std::vector<UniqueId>&) {}
    template <class D>
    void exec_now(D&, size_t, size_t) {}
    template <class D>
    void run(D&) {}

    template <class T, class D>
    Buffer<T, D> replace_buf(D&, const Buffer<T, D>& b) {
        return b.shallow();
    }
    void set_checkpoint_buffer(Id) {}

    template <class D>
    void optimize_mem_graph(D&, const GraphTranslator*) {}
    template <class D>
    void unary_fusing(D&, const GraphTranslator*) {}

    void add_grad_fn(Operation&&) {}
    void set_grad_enabled(bool) {}
    bool is_grad_enabled() const { return false; }
    AutogradState* autograd() { return nullptr; }
    void set_requires_grad(Id, bool) {}
    bool requires_grad_of(Id) const { return false; }

    size_t cursor() const { return cursor_; }
    void set_cursor(size_t c) { cursor_ = c; }
    Buffers* buffers() { return nullptr; }
    uint64_t lazy_version() const { return 0; }

   private:
    size_t cursor_ = 0;
};

// ---------------------------------------------------------------------------
// Lazy: records operations, defers allocation (src/modules/lazy.rs)
// ---------------------------------------------------------------------------
template <class Mods, class T = float>
struct Lazy {
    Mods modules;
    Buffers buffers_;                // id -> shallow copy: user buffers and lazily allocated ones
    std::vector<Operation> graph;    // LazyGraph::operations

    template <class D>
    void setup(D& dev) {
        dev.lazy_setup();
        modules.setup(dev);
    }
    template <class D>
    void teardown(D& dev) {
        for (auto& kv : buffers_)
            if (kv.second.module_owned && kv.second.ptr) dev.free_raw(kv.second.ptr);
        buffers_.clear();
        graph.clear();
        modules.teardown(dev);
    }

    // No allocation: an id (the cursor) and a note to allocate later (lazy.rs:325-387).
    template <class U, class D>
    Buffer<U, D> retrieve(D& dev, size_t len, const std::vector<Id>&, const std::vector<bool>&) {
        Id id{static_cast<UniqueId>(cursor_), len};
        alloc_later_.push_back(Pending{id, std::type_index(typeid(U)), sizeof(U)});
        cursor_++;
        return Buffer<U, D>::from_parts(&dev, 0, len, id, AllocFlag::Lazy);
    }

    template <class U, class D>
    void on_new_buffer(D& dev, const Buffer<U, D>& b) {
        buffers_[b.id().id] = AnyBuf{b.ptr(), b.len(), std::type_index(typeid(U)), false, sizeof(U)};
        modules.on_new_buffer(dev, b);
    }
    void on_drop_buffer(Id id) {
        auto it = buffers_.find(id.id);
        if (it != buffers_.end() && !it->second.module_owned) {
            buffers_.erase(it);
            version_++;  // recorded operations that name it must fail at the next run
        }
        modules.on_drop_buffer(id);
    }
    void on_release_cached(uint64_t ptr) { modules.on_release_cached(ptr); }

    template <class D>
    void add_op(D& dev, Operation&& op) {
        if (enabled_) {
            graph.push_back(std::move(op));
            version_++;
        } else {
            Buffers* b = &buffers_;
            op.op(*b, &dev);
        }
    }
    size_t ops_count() const { return graph.size(); }
    void set_lazy_enabled(bool e) { enabled_ = e; }
    bool is_lazy_enabled() const { return enabled_; }

    // Tags the last recorded operation (lazy.rs:136-143).
    void set_op_hint(AnyOpHint h) {
        if (!enabled_ || graph.empty()) return;
        graph.back().hint_kind = h.kind;
        graph.back().unary_hint = std::move(h.unary);
        graph.back().hint_type = h.type;
    }

    void set_expr_hint(AnyExprHint h) {
        if (!enabled_ || graph.empty()) return;
        graph.back().expr_hint = std::move(h.hint);
        graph.back().expr_type = h.type;
        graph.back().in_args = std::move(h.in_args);
        graph.back().out_arg = h.out_arg;
    }

    // Runs and drains operations [begin, end) now (lazy.rs:145-162, lazy_graph.rs:93-104).
    template <class D>
    void exec_now(D& dev, size_t begin, size_t end) {
        alloc_later(dev);
        end = std::min(end, graph.size());
        begin = std::min(begin, end);
        std::vector<Operation> drained(std::make_move_iterator(graph.begin() + begin),
                                       std::make_move_iterator(graph.begin() + end));
        graph.erase(graph.begin() + begin, graph.begin() + end);
        version_++;
        for (auto& op : drained) op.op(buffers_, &dev);
    }

    // alloc_later -> call_lazily -> device.run() (lazy.rs:190-198).  The device
    // decides how the recorded sequence is executed (directly, or captured into
    // a graph once and replayed while `version` stays the same).
    template <class D>
    void run(D& dev) {
        alloc_later(dev);
        dev.lazy_run(version_, [this, &dev] { call_lazily(dev); });
        modules.run(dev);
    }

    template <class D>
    void call_lazily(D& dev) {
        for (auto& op : graph) op.op(buffers_, &dev);
    }

    // Allocates every lazily retrieved buffer that has no memory yet (lazy.rs:173-179).
    template <class D>
    void alloc_later(D& dev) {
        for (const Pending& p : alloc_later_) alloc_one(dev, p);
        alloc_later_.clear();
    }

    template <class U, class D>
    Buffer<U, D> replace_buf(D& dev, const Buffer<U, D>& b) {
        auto it = buffers_.find(b.id().id);
        if (it == buffers_.end()) return modules.template replace_buf<U>(dev, b);
        if (it->second.type != std::type_index(typeid(U))) throw Error(DeviceError::TypeMismatch);
        return Buffer<U, D>::from_parts(&dev, it->second.ptr, it->second.len, b.id(), AllocFlag::Wrapper,
                                        b.requires_grad());
    }
    void set_checkpoint_buffer(Id id) { modules.set_checkpoint_buffer(id); }

    // One allocation per cache trace, shared by all its buffers
    // (lazy/optimization.rs:4-44).  Buffers outside every trace get their own.
    template <class D>
    void optimize_mem_graph(D& dev, const GraphTranslator* gt) {
        if (!gt) throw Error(DeviceError::MissingCacheTraces);
        const std::vector<CacheTrace> traces = gt->opt_graph.cache_traces();
        std::vector<Pending> pending;
        pending.swap(alloc_later_);
        for (const Pending& p : pending) {
            for (const CacheTrace& t : traces) {
                auto head = gt->idx_to_buf_id.find(t.cache_idx);
                if (head == gt->idx_to_buf_id.end()) throw Error(DeviceError::GraphOptimization);
                if (head->second != p.id.id) continue;
                alloc_one(dev, p);
                AnyBuf shared = buffers_.at(p.id.id);
                shared.module_owned = false;
                for (size_t use : t.use_cache_idxs) {
                    auto use_id = gt->idx_to_buf_id.find(use);
                    if (use_id == gt->idx_to_buf_id.end()) throw Error(DeviceError::GraphOptimization);
                    // a buffer of another element type keeps an allocation of its own, as in the
                    // Cached module (cached.rs:430-441); the reference's Lazy aliases it anyway and
                    // the run then fails (opt_graph/optimize.rs:659-690)
                    bool same_type = true;
                    for (const Pending& q : pending)
                        if (q.id.id == use_id->second) same_type = q.type == p.type;
                    if (!same_type) continue;
                    buffers_[use_id->second] = shared;
                    allocated_ids_.insert(use_id->second);
                }
            }
        }
        for (const Pending& p : pending) alloc_one(dev, p);  // not the head of any trace
        version_++;
    }

    // Replaces every maximal run of hinted unary operations inside a cache
    // trace by one fused operation (lazy/optimization.rs:46-96,
    // src/devices/fusing.rs:41-92).  Unlike the reference, operations of a
    // trace that carry no unary hint are left alone, and a trace may hold
    // several runs.
    template <class D>
    void unary_fusing(D& dev, const GraphTranslator* gt) {
        if (!gt) throw Error(DeviceError::MissingCacheTraces);
        // producing operation of every buffer id
        std::unordered_map<UniqueId, size_t> producer;
        for (size_t i = 0; i < graph.size(); i++)
            if (graph[i].hint_kind == OpHintKind::Unary && graph[i].arg_ids.size() == 2)
                producer[graph[i].arg_ids[0].id] = i;  // apply_fn records (out, in)

        for (const CacheTrace& t : gt->opt_graph.cache_traces()) {
            std::vector<size_t> node_idxs{t.cache_idx};
            node_idxs.insert(node_idxs.end(), t.use_cache_idxs.begin(), t.use_cache_idxs.end());
            std::vector<size_t> run;  // operation indices of the current run
            auto flush = [&] {
                if (run.size() >= 2) fuse_run(dev, run);
                run.clear();
            };
            for (size_t node : node_idxs) {
                auto bid = gt->idx_to_buf_id.find(node);
                if (bid == gt->idx_to_buf_id.end()) throw Error(DeviceError::GraphOptimization);
                auto p = producer.find(bid->second);
                const bool unary = p != producer.end() && graph[p->second].hint_type == std::type_index(typeid(T));
                if (!unary) {
                    flush();
                    continue;
                }
                const size_t op_idx = p->second;
                // the run continues only if this op reads what the previous one wrote
                if (!run.empty() && graph[op_idx].arg_ids[1].id != graph[run.back()].arg_ids[0].id) flush();
                run.push_back(op_idx);
            }
            flush();
        }
    }

    // Fuses element-wise operations of any arity across operations: an operation
    // whose only reader is another hinted operation is inlined into that reader,
    // repeatedly, so `t = a*b; u = t+c; y = sqrt(abs(u))*0.3` becomes one
    // three-operand kernel that moves 16 bytes per element instead of 32.
    // (The reference fuses unary chains only; unary chains are the one-operand
    // case of this.)  An operation is inlined only if its output
    //   - was retrieved lazily (not a buffer the user filled),
    //   - is read by exactly one recorded operation and is not in `keep` (the
    //     Autograd module lists what its gradient functions read),
    //   - is not a checkpoint, has the reader's length,
    //   - and none of its own operands is written between it and the reader;
    // the fused operation takes the reader's place and may have at most four
    // distinct operand buffers.  Intermediates are never computed (they keep the
    // zeros of their allocation), as with unary fusing.
    template <class D>
    void elementwise_fusing(D& dev, const GraphTranslator* gt, const std::vector<UniqueId>& keep) {
        if (!gt) throw Error(DeviceError::MissingCacheTraces);
        const std::type_index tt(typeid(T));
        const size_t n_ops = graph.size();
        auto hinted = [&](size_t i) { return graph[i].expr_hint && graph[i].expr_type == tt && graph[i].out_arg >= 0; };

        // readers of every buffer id; producers of lazily retrieved outputs
        std::unordered_map<UniqueId, int> readers;
        std::unordered_map<UniqueId, size_t> producer;
        for (size_t i = 0; i < n_ops; i++) {
            if (hinted(i)) {
                for (int a : graph[i].in_args) readers[graph[i].arg_ids[a].id]++;
                const Id out = graph[i].arg_ids[graph[i].out_arg];
                if (producer.count(out.id)) readers[out.id] += 2;  // written twice: leave it alone
                producer[out.id] = i;
            } else {
                for (const Id& id : graph[i].arg_ids) readers[id.id] += 2;  // unknown use: never inline
            }
        }
        for (UniqueId id : keep) readers[id] += 2;  // e.g. what gradient functions will read

        auto skipped = [&](UniqueId id) {
            auto it = gt->buf_id_to_idx.find(id);
            return it != gt->buf_id_to_idx.end() && gt->opt_graph.nodes[it->second].skip;
        };
        auto written_between = [&](const std::vector<Id>& leaves, size_t from, size_t to) {
            for (size_t j = from + 1; j < to; j++) {
                if (graph[j].arg_ids.empty()) continue;
                for (size_t a = 0; a < graph[j].arg_ids.size(); a++) {
                    if (hinted(j) && static_cast<int>(a) != graph[j].out_arg) continue;  // only reads it
                    for (const Id& leaf : leaves)
                        if (graph[j].arg_ids[a].id == leaf.id) return true;
                }
            }
            return false;
        };

        std::vector<std::unique_ptr<FusedExpr<T>>> exprs(n_ops);
        std::vector<bool> absorbed(n_ops, false);
        for (size_t i = 0; i < n_ops; i++) {
            if (!hinted(i)) continue;
            auto e = std::make_unique<FusedExpr<T>>();
            typename FusedExpr<T>::Item item;
            item.hint = std::static_pointer_cast<ExprHint<T>>(graph[i].expr_hint);
            auto leaf_index = [&](FusedExpr<T>& fe, Id id) {
                for (size_t k = 0; k < fe.leaves.size(); k++)
                    if (fe.leaves[k].id == id.id) return static_cast<int>(k);
                fe.leaves.push_back(id);
                return static_cast<int>(fe.leaves.size()) - 1;
            };
            for (int a : graph[i].in_args) item.inputs.push_back(leaf_index(*e, graph[i].arg_ids[a]));
            e->items.push_back(std::move(item));
            e->root = 0;
            const Id out = graph[i].arg_ids[graph[i].out_arg];

            // inline producers of leaves until nothing changes
            bool changed = true;
            while (changed) {
                changed = false;
                for (size_t k = 0; k < e->leaves.size() && !changed; k++) {
                    const Id leaf = e->leaves[k];
                    auto p = producer.find(leaf.id);
                    if (p == producer.end() || p->second >= i || absorbed[p->second] || !exprs[p->second]) continue;
                    if (!allocated_lazily(leaf.id) || readers[leaf.id] != 1 || skipped(leaf.id) || leaf.len != out.len) continue;
                    const FusedExpr<T>& pe = *exprs[p->second];
                    if (written_between(pe.leaves, p->second, i)) continue;
                    // distinct operand buffers after the merge
                    // (the producer's operands take the place of the inlined one)
                    std::vector<Id> merged;
                    auto push_unique = [&merged](const Id& id) {
                        for (const Id& m : merged)
                            if (m.id == id.id) return;
                        merged.push_back(id);
                    };
                    for (size_t q = 0; q < e->leaves.size(); q++) {
                        if (q != k) push_unique(e->leaves[q]);
                        else
                            for (const Id& pl : pe.leaves) push_unique(pl);
                    }
                    if (merged.size() > 4) continue;
                    // rebuild: items of the producer first, then ours, leaves re-indexed
                    auto fused = std::make_unique<FusedExpr<T>>();
                    auto remap_leaf = [&](Id id) {
                        for (size_t q = 0; q < merged.size(); q++)
                            if (merged[q].id == id.id) return static_cast<int>(q);
                        return -1;
                    };
                    fused->leaves = merged;
                    const int p_off = 0, own_off = static_cast<int>(pe.items.size());
                    for (const auto& it : pe.items) {
                        typename FusedExpr<T>::Item ni{it.hint, {}};
                        for (int in : it.inputs) ni.inputs.push_back(in >= 0 ? remap_leaf(pe.leaves[in]) : ~(~in + p_off));
                        fused->items.push_back(std::move(ni));
                    }
                    for (const auto& it : e->items) {
                        typename FusedExpr<T>::Item ni{it.hint, {}};
                        for (int in : it.inputs) {
                            if (in < 0) ni.inputs.push_back(~(~in + own_off));
                            else if (static_cast<size_t>(in) == k) ni.inputs.push_back(~(pe.root + p_off));
                            else ni.inputs.push_back(remap_leaf(e->leaves[in]));
                        }
                        fused->items.push_back(std::move(ni));
                    }
                    fused->root = e->root + own_off;
                    absorbed[p->second] = true;
                    e = std::move(fused);
                    changed = true;
                }
            }
            exprs[i] = std::move(e);
        }

        for (size_t i = 0; i < n_ops; i++) {
            if (absorbed[i]) {
                graph[i] = Operation::no_op();
                continue;
            }
            if (!exprs[i] || exprs[i]->items.size() < 2) continue;
            std::shared_ptr<FusedExpr<T>> fe(std::move(exprs[i]));
            const Id out_id = graph[i].arg_ids[graph[i].out_arg];
            Operation fused;
            fused.arg_ids.push_back(out_id);
            for (const Id& l : fe->leaves) fused.arg_ids.push_back(l);
            fused.hint_kind = OpHintKind::UnaryFused;
            fused.fused_source = fe->to_cl_source({"a", "b", "c", "d"});
            auto fn = dev.template elementwise_fuse_op<T>(fe);
            fused.op = [fe, out_id, fn](Buffers& bufs, void* devp) {
                D& d = *static_cast<D*>(devp);
                auto view = [&](Id id) {
                    auto it = bufs.find(id.id);
                    if (it == bufs.end() || it->second.ptr == 0) throw Error(DeviceError::InvalidLazyBuf);
                    if (it->second.type != std::type_index(typeid(T))) throw Error(DeviceError::TypeMismatch);
                    return Buffer<T, D>::from_parts(&d, it->second.ptr, it->second.len, id, AllocFlag::Wrapper);
                };
                Buffer<T, D> out = view(out_id);
                std::vector<Buffer<T, D>> ins;
                for (const Id& l : fe->leaves) ins.push_back(view(l));
                fn(out, ins, d);
            };
            graph[i] = std::move(fused);
        }
        version_++;
    }

    bool allocated_lazily(UniqueId id) const {
        if (allocated_ids_.count(id)) return true;
        for (const Pending& p : alloc_later_)
            if (p.id.id == id) return true;
        return false;
    }

    void add_grad_fn(Operation&& op) { modules.add_grad_fn(std::move(op)); }
    void set_grad_enabled(bool e) { modules.set_grad_enabled(e); }
    bool is_grad_enabled() const { return modules.is_grad_enabled(); }
    AutogradState* autograd() { return modules.autograd(); }
    void set_requires_grad(Id id, bool v) { modules.set_requires_grad(id, v); }
    bool requires_grad_of(Id id) const { return modules.requires_grad_of(id); }

    size_t cursor() const { return cursor_; }
    void set_cursor(size_t c) { cursor_ = c; }
    Buffers* buffers() { return &buffers_; }
    uint64_t lazy_version() const { return version_; }

   private:
    struct Pending {
        Id id;
        std::type_index type;
        size_t elem_size;
    };

    template <class D>
    void alloc_one(D& dev, const Pending& p) {
        if (allocated_ids_.count(p.id.id)) return;
        // lazy ids count up from 0, buffers with data use their address: both
        // live in one table (lazy.rs:347-357)
        if (buffers_.count(p.id.id)) throw Error(DeviceError::IdCollision);
        uint64_t ptr = dev.alloc_raw(p.id.len * p.elem_size, /*zeroed=*/true, p.id.len);
        buffers_[p.id.id] = AnyBuf{ptr, p.id.len, p.type, true, p.elem_size};
        allocated_ids_.insert(p.id.id);
    }

    template <class D>
    void fuse_run(D& dev, const std::vector<size_t>& run) {
        std::vector<std::shared_ptr<UnaryHint<T>>> hints;
        for (size_t i : run) hints.push_back(std::static_pointer_cast<UnaryHint<T>>(graph[i].unary_hint));
        const Id out_id = graph[run.back()].arg_ids[0];
        const Id in_id = graph[run.front()].arg_ids[1];
        Operation fused;
        fused.arg_ids = {out_id, in_id};
        fused.hint_kind = OpHintKind::UnaryFused;
        auto fused_fn = dev.template unary_fuse_op<T>(std::move(hints));
        fused.op = [out_id, in_id, fused_fn](Buffers& bufs, void* devp) {
            D& d = *static_cast<D*>(devp);
            auto out = bufs.find(out_id.id);
            auto in = bufs.find(in_id.id);
            if (out == bufs.end() || in == bufs.end()) throw Error(DeviceError::InvalidLazyBuf);
            if (out->second.type != std::type_index(typeid(T)) || in->second.type != std::type_index(typeid(T)))
                throw Error(DeviceError::TypeMismatch);
            Buffer<T, D> o = Buffer<T, D>::from_parts(&d, out->second.ptr, out->second.len, out_id, AllocFlag::Wrapper);
            Buffer<T, D> i = Buffer<T, D>::from_parts(&d, in->second.ptr, in->second.len, in_id, AllocFlag::Wrapper);
            fused_fn(o, i, d);
        };
        // the fused operation takes the place of the first one (fusing.rs:55,
        // optimization.rs:88-90); the others become no-ops
        for (size_t i : run) graph[i] = Operation::no_op();
        graph[run.front()] = std::move(fused);
        version_++;
    }

    std::vector<Pending> alloc_later_;
    std::unordered_set<UniqueId> allocated_ids_;
    size_t cursor_ = 0;
    bool enabled_ = true;
    uint64_t version_ = 1;
};

// ---------------------------------------------------------------------------
// Cached: the n-th retrieve of an epoch returns the allocation the n-th
// retrieve of the previous epoch made (src/modules/cached.rs:22-255).
// ---------------------------------------------------------------------------
// The key is the cursor, which counts retrieves and which the caller rewinds
// with `device.range(..)` at the start of every epoch (src/range.rs:9-62).  The
// module owns the allocations; a retrieved buffer is a handle with
// `AllocFlag::Cached` that reports its drop, so that the module knows which
// allocations are in use.  `optimize_mem_graph` lets all buffers of a cache
// trace share the allocation of the trace's first buffer (cached.rs:415-446)
// and frees the ones they had.
template <class Mods>
struct Cached {
    Mods modules;

    template <class D>
    void setup(D& dev) {
        modules.setup(dev);
    }
    template <class D>
    void teardown(D& dev) {
        std::unordered_set<uint64_t> freed;
        for (auto& kv : cache_)
            if (kv.second.ptr && freed.insert(kv.second.ptr).second) dev.free_raw(kv.second.ptr);
        cache_.clear();
        live_.clear();
        modules.teardown(dev);
    }

    template <class U, class D>
    Buffer<U, D> retrieve(D& dev, size_t len, const std::vector<Id>& parents, const std::vector<bool>& rg) {
        const UniqueId key = static_cast<UniqueId>(cursor_);
        auto it = cache_.find(key);
        if (it == cache_.end()) {
            Buffer<U, D> fresh = modules.template retrieve<U>(dev, len, parents, rg);
            fresh.set_flag(AllocFlag::Cached);  // cached.rs:203: the module frees it, not the handle
            it = cache_.emplace(key, AnyBuf{fresh.ptr(), len, std::type_index(typeid(U)), true, sizeof(U)}).first;
            live_[fresh.ptr()]++;
            cursor_++;
            return fresh;
        }
        // The reference keys its default cache by the cursor alone and trusts the
        // caller to repeat the same sequence of retrieves; here a retrieve that
        // does not fit what the cursor position holds is an error.
        if (it->second.type != std::type_index(typeid(U))) throw Error(DeviceError::TypeMismatch);
        if (it->second.len != len) throw Error(DeviceError::ShapeLengthMismatch);
        cursor_++;
        live_[it->second.ptr]++;
        return Buffer<U, D>::from_parts(&dev, it->second.ptr, len, Id{it->second.ptr, len}, AllocFlag::Cached);
    }

    template <class U, class D>
    void on_new_buffer(D& dev, const Buffer<U, D>& b) {
        modules.on_new_buffer(dev, b);
    }
    void on_drop_buffer(Id id) { modules.on_drop_buffer(id); }
    void on_release_cached(uint64_t ptr) {
        auto it = live_.find(ptr);
        if (it != live_.end() && it->second > 0) it->second--;
    }

    template <class D>
    void add_op(D& dev, Operation&& op) {
        modules.add_op(dev, std::move(op));
    }
    size_t ops_count() const { return modules.ops_count(); }
    void set_lazy_enabled(bool e) { modules.set_lazy_enabled(e); }
    bool is_lazy_enabled() const { return modules.is_lazy_enabled(); }
    void set_op_hint(AnyOpHint h) { modules.set_op_hint(std::move(h)); }
    void set_expr_hint(AnyExprHint h) { modules.set_expr_hint(std::move(h)); }
    template <class D>
    void exec_now(D& dev, size_t b, size_t e) {
        modules.exec_now(dev, b, e);
    }
    template <class D>
    void run(D& dev) {
        modules.run(dev);
    }
    template <class U, class D>
    Buffer<U, D> replace_buf(D& dev, const Buffer<U, D>& b) {
        return modules.template replace_buf<U>(dev, b);
    }
    void set_checkpoint_buffer(Id id) { modules.set_checkpoint_buffer(id); }

    // cached.rs:415-446, on cursor positions instead of node indices
    // (graph_translator.rs:45-57).  Buffers of another element type or length keep
    // their own allocation.  Fails if a handle to an allocation that would be
    // replaced is still alive.
    template <class D>
    void optimize_mem_graph(D& dev, const GraphTranslator* gt) {
        if (!gt) throw Error(DeviceError::MissingCacheTraces);
        const std::vector<CacheTrace> traces = gt->to_cursor_cache_traces(gt->opt_graph.cache_traces());
        for (const CacheTrace& t : traces) {
            auto head = cache_.find(static_cast<UniqueId>(t.cache_idx));
            if (head == cache_.end()) throw Error(DeviceError::GraphOptimization);
            for (size_t use : t.use_cache_idxs) {
                auto u = cache_.find(static_cast<UniqueId>(use));
                if (u == cache_.end()) throw Error(DeviceError::GraphOptimization);
                if (u->second.ptr == head->second.ptr) continue;
                if (u->second.type != head->second.type || u->second.len != head->second.len) continue;
                if (live_[u->second.ptr] > 0) throw Error(DeviceError::CachedInUse);
            }
        }
        for (const CacheTrace& t : traces) {
            const AnyBuf shared = cache_.at(static_cast<UniqueId>(t.cache_idx));
            for (size_t use : t.use_cache_idxs) {
                AnyBuf& u = cache_.at(static_cast<UniqueId>(use));
                if (u.ptr == shared.ptr || u.type != shared.type || u.len != shared.len) continue;
                const uint64_t old = u.ptr;
                u = shared;
                bool still_used = false;
                for (const auto& kv : cache_) still_used = still_used || kv.second.ptr == old;
                if (!still_used) {
                    dev.free_raw(old);
                    live_.erase(old);
                }
            }
        }
        modules.optimize_mem_graph(dev, gt);
    }
    // cached.rs:448-455
    template <class D>
    void unary_fusing(D&, const GraphTranslator*) {
        throw Error(DeviceError::UnaryFusingUnsupported);
    }
    template <class D>
    void elementwise_fusing(D&, const GraphTranslator*, const std::vector<UniqueId>&) {
        throw Error(DeviceError::UnaryFusingUnsupported);
    }

    void add_grad_fn(Operation&& op) { modules.add_grad_fn(std::move(op)); }
    void set_grad_enabled(bool e) { modules.set_grad_enabled(e); }
    bool is_grad_enabled() const { return modules.is_grad_enabled(); }
    AutogradState* autograd() { return modules.autograd(); }
    void set_requires_grad(Id id, bool v) { modules.set_requires_grad(id, v); }
    bool requires_grad_of(Id id) const { return modules.requires_grad_of(id); }

    // cached.rs:257-267: the module has a cursor of its own
    size_t cursor() const { return cursor_; }
    void set_cursor(size_t c) { cursor_ = c; }
    Buffers* buffers() { return modules.buffers(); }
    uint64_t lazy_version() const { return modules.lazy_version(); }

    size_t cached_allocations() const {
        std::unordered_set<uint64_t> distinct;
        for (const auto& kv : cache_) distinct.insert(kv.second.ptr);
        return distinct.size();
    }

   private:
    std::unordered_map<UniqueId, AnyBuf> cache_;   // cursor position -> allocation
    std::unordered_map<uint64_t, size_t> live_;    // address -> handles given out and not dropped yet
    size_t cursor_ = 0;
};

// ---------------------------------------------------------------------------
// Graph: dependency DAG built at every retrieve (src/modules/graph.rs)
// ---------------------------------------------------------------------------
template <class Mods, class T = float>
struct Graph {
    Mods modules;
    GraphTranslator graph_trans;

    template <class D>
    void setup(D& dev) {
        modules.setup(dev);
    }
    template <class D>
    void teardown(D& dev) {
        modules.teardown(dev);
    }

    template <class U, class D>
    Buffer<U, D> retrieve(D& dev, size_t len, const std::vector<Id>& parents, const std::vector<bool>& rg) {
        Buffer<U, D> data = modules.template retrieve<U>(dev, len, parents, rg);
        // the inner module bumped the cursor (graph.rs:172-177)
        const UniqueId cursor = static_cast<UniqueId>(modules.cursor()) - 1;
        if (!contains_ids_.insert(cursor).second) return data;
        const size_t next_idx = graph_trans.next_idx;
        graph_trans.buf_id_to_idx[data.id().id] = next_idx;
        graph_trans.idx_to_buf_id[next_idx] = data.id().id;
        graph_trans.idx_to_cursor[next_idx] = cursor;
        graph_trans.add_node(len, parents);
        return data;
    }

    // A buffer created with data is a leaf (graph.rs:115-127).
    template <class U, class D>
    void on_new_buffer(D& dev, const Buffer<U, D>& b) {
        graph_trans.buf_id_to_idx[b.id().id] = graph_trans.next_idx;
        graph_trans.add_leaf(b.len());
        modules.on_new_buffer(dev, b);
    }
    void on_drop_buffer(Id id) { modules.on_drop_buffer(id); }
    void on_release_cached(uint64_t ptr) { modules.on_release_cached(ptr); }

    template <class D>
    void add_op(D& dev, Operation&& op) {
        modules.add_op(dev, std::move(op));
    }
    size_t ops_count() const { return modules.ops_count(); }
    void set_lazy_enabled(bool e) { modules.set_lazy_enabled(e); }
    bool is_lazy_enabled() const { return modules.is_lazy_enabled(); }
    void set_op_hint(AnyOpHint h) { modules.set_op_hint(std::move(h)); }
    void set_expr_hint(AnyExprHint h) { modules.set_expr_hint(std::move(h)); }
    template <class D>
    void exec_now(D& dev, size_t b, size_t e) {
        modules.exec_now(dev, b, e);
    }
    template <class D>
    void run(D& dev) {
        modules.run(dev);
    }
    template <class U, class D>
    Buffer<U, D> replace_buf(D& dev, const Buffer<U, D>& b) {
        return modules.template replace_buf<U>(dev, b);
    }
    // graph.rs:255-259
    void set_checkpoint_buffer(Id id) {
        auto it = graph_trans.buf_id_to_idx.find(id.id);
        if (it == graph_trans.buf_id_to_idx.end()) throw Error(DeviceError::GraphOptimization);
        graph_trans.opt_graph.nodes[it->second].skip = true;
    }

    // graph.rs:79-113: hand the own translator down unless one was given
    template <class D>
    void optimize_mem_graph(D& dev, const GraphTranslator* gt) {
        modules.optimize_mem_graph(dev, gt ? gt : &graph_trans);
    }
    template <class D>
    void unary_fusing(D& dev, const GraphTranslator* gt) {
        modules.unary_fusing(dev, gt ? gt : &graph_trans);
    }
    template <class D>
    void elementwise_fusing(D& dev, const GraphTranslator* gt, const std::vector<UniqueId>& keep) {
        modules.elementwise_fusing(dev, gt ? gt : &graph_trans, keep);
    }

    void add_grad_fn(Operation&& op) { modules.add_grad_fn(std::move(op)); }
    void set_grad_enabled(bool e) { modules.set_grad_enabled(e); }
    bool is_grad_enabled() const { return modules.is_grad_enabled(); }
    AutogradState* autograd() { return modules.autograd(); }
    void set_requires_grad(Id id, bool v) { modules.set_requires_grad(id, v); }
    bool requires_grad_of(Id id) const { return modules.requires_grad_of(id); }
    size_t cursor() const { return modules.cursor(); }
    void set_cursor(size_t c) { modules.set_cursor(c); }
    Buffers* buffers() { return modules.buffers(); }
    uint64_t lazy_version() const { return modules.lazy_version(); }

   private:
    std::unordered_set<UniqueId> contains_ids_;
};

// ---------------------------------------------------------------------------
// Autograd: tape of gradient functions + gradient buffers
// (src/modules/autograd.rs, autograd/tape.rs, autograd/gradients.rs)
// ---------------------------------------------------------------------------
struct AutogradState {
    std::vector<Operation> tape;                       // Tape::lazy_graph
    Buffers grads;                                     // Gradients::grads_pool, keyed by buffer id
    Buffers no_grads_pool;                             // buffers by id when no module below keeps them
    std::unordered_map<UniqueId, bool> buf_requires_grad;
    bool enabled = true;
};

template <class Mods>
struct Autograd {
    Mods modules;
    AutogradState state;

    template <class D>
    void setup(D& dev) {
        modules.setup(dev);
    }
    template <class D>
    void teardown(D& dev) {
        for (auto& kv : state.grads)
            if (kv.second.ptr) dev.free_raw(kv.second.ptr);
        state.grads.clear();
        state.tape.clear();
        modules.teardown(dev);
    }

    // requires_grad propagates from the parents (autograd.rs:110-136)
    template <class U, class D>
    Buffer<U, D> retrieve(D& dev, size_t len, const std::vector<Id>& parents, const std::vector<bool>& rg) {
        const bool requires_grad = std::any_of(rg.begin(), rg.end(), [](bool b) { return b; });
        Buffer<U, D> data = modules.template retrieve<U>(dev, len, parents, rg);
        state.buf_requires_grad[data.id().id] = requires_grad;
        data.set_requires_grad_flag(requires_grad);
        register_no_grad_buf(data);
        return data;
    }
    template <class U, class D>
    void on_new_buffer(D& dev, const Buffer<U, D>& b) {
        state.buf_requires_grad[b.id().id] = b.requires_grad();
        register_no_grad_buf(b);
        modules.on_new_buffer(dev, b);
    }
    void on_drop_buffer(Id id) {
        state.no_grads_pool.erase(id.id);
        modules.on_drop_buffer(id);
    }
    void on_release_cached(uint64_t ptr) { modules.on_release_cached(ptr); }

    template <class D>
    void add_op(D& dev, Operation&& op) {
        modules.add_op(dev, std::move(op));
    }
    size_t ops_count() const { return modules.ops_count(); }
    void set_lazy_enabled(bool e) { modules.set_lazy_enabled(e); }
    bool is_lazy_enabled() const { return modules.is_lazy_enabled(); }
    void set_op_hint(AnyOpHint h) { modules.set_op_hint(std::move(h)); }
    void set_expr_hint(AnyExprHint h) { modules.set_expr_hint(std::move(h)); }
    template <class D>
    void exec_now(D& dev, size_t b, size_t e) {
        modules.exec_now(dev, b, e);
    }
    template <class D>
    void run(D& dev) {
        modules.run(dev);
    }
    template <class U, class D>
    Buffer<U, D> replace_buf(D& dev, const Buffer<U, D>& b) {
        Buffer<U, D> r = modules.template replace_buf<U>(dev, b);
        r.set_requires_grad_flag(requires_grad_of(b.id()) || b.requires_grad());
        return r;
    }
    void set_checkpoint_buffer(Id id) { modules.set_checkpoint_buffer(id); }
    template <class D>
    void optimize_mem_graph(D& dev, const GraphTranslator* gt) {
        modules.optimize_mem_graph(dev, gt);
    }
    template <class D>
    void unary_fusing(D& dev, const GraphTranslator* gt) {
        modules.unary_fusing(dev, gt);
    }
    // buffers the gradient functions on the tape will read must stay computed
    template <class D>
    void elementwise_fusing(D& dev, const GraphTranslator* gt, const std::vector<UniqueId>& keep) {
        std::vector<UniqueId> all = keep;
        for (const Operation& g : state.tape)
            for (const Id& id : g.arg_ids) all.push_back(id.id);
        modules.elementwise_fusing(dev, gt, all);
    }

    // autograd.rs:245-256
    void add_grad_fn(Operation&& op) {
        if (state.enabled) state.tape.push_back(std::move(op));
    }
    void set_grad_enabled(bool e) { state.enabled = e; }
    bool is_grad_enabled() const { return state.enabled; }
    AutogradState* autograd() { return &state; }
    void set_requires_grad(Id id, bool v) { state.buf_requires_grad[id.id] = v; }
    bool requires_grad_of(Id id) const {
        auto it = state.buf_requires_grad.find(id.id);
        return it != state.buf_requires_grad.end() && it->second;
    }

    size_t cursor() const { return modules.cursor(); }
    void set_cursor(size_t c) { modules.set_cursor(c); }
    // buffers by id for the gradient functions: the Lazy module's table when
    // there is one, else the pool kept here (autograd.rs:60-75)
    Buffers* buffers() {
        Buffers* below = modules.buffers();
        return below ? below : &state.no_grads_pool;
    }
    uint64_t lazy_version() const { return modules.lazy_version(); }

   private:
    template <class U, class D>
    void register_no_grad_buf(const Buffer<U, D>& b) {
        if (modules.buffers() != nullptr || !b.has_data()) return;
        state.no_grads_pool.emplace(b.id().id, AnyBuf{b.ptr(), b.len(), std::type_index(typeid(U)), false, sizeof(U)});
    }
};

}  // namespace custos
