// Recording and graph construction: dependency levels from address-range
// conflicts, merging of equal launches, explicit hipGraph nodes, replay
// (include/custos_hip.h).
#include <algorithm>
#include <array>
#include <cstring>
#include <queue>
#include <set>

#include "runtime.hpp"

namespace custos_hip {

namespace {

// ---- building a graph from the recorded work ----
//
// The recorded list is not replayed launch by launch.  Every node gets a
// dependency level: one more than the highest level among earlier nodes whose
// memory it conflicts with (read-after-write, write-after-read or
// write-after-write on overlapping address ranges).  Nodes of one level are
// independent of each other, so kernel launches of one level that use the same
// kernel are merged into ONE grid that walks a table of operand addresses
// (equal lengths: segment = block / tiles per segment; different lengths: a
// block map names segment and tile of every workgroup).  1024 small buffers
// with three operations each become three kernel nodes instead of 3072.  The
// merged nodes are then ordered as one chain in level order (the default: a
// dependency between branches of a graph costs several times what a node of a
// chain costs, and an element-wise launch of any size fills the chip alone), by
// an edge per dependency, or by joins between levels.

constexpr uint64_t kChunkShift = 21;  // conflict search buckets of 2 MiB
// A launch of more tiles than this is not merged with launches of other lengths:
// it fills the chip by itself, and the block map would grow with it.
constexpr unsigned long long kRaggedMaxTiles = 16384;
// A node counts as a producer if one of this many levels after it reads what it writes.
constexpr size_t kLookAheadLevels = 8;
// A chain follows the recording (instead of the levels) if one of its launches touches this much.
constexpr unsigned long long kFollowRecordingFromBytes = 8ull << 20;

// Earlier accesses are kept once per distinct (range, mode) with the highest level seen, so
// a program that runs over the same buffers many times keeps the search lists as short as
// a single pass does; the lists hang off the 2 MiB address chunks a range touches.
//
// With `edges`, every node also gets the recorded nodes it has to wait for (`deps`).  An entry
// then names the nodes a later conflicting access must follow: for a written range its last
// writer (earlier writers of the same range precede it already), for a read range the readers
// since the last write that covered it.  A write that covers an entry entirely takes over from
// it: whatever conflicts with the entry later conflicts with that write too.
void assign_levels(std::vector<RecNode>& nodes, bool edges) {
    struct Seen {
        uint64_t begin, end;
        bool write;
        int level;
        std::vector<uint32_t> users;
    };
    struct Key {
        uint64_t begin, end;
        bool write;
        bool operator==(const Key& o) const { return begin == o.begin && end == o.end && write == o.write; }
    };
    struct KeyHash {
        size_t operator()(const Key& k) const {
            uint64_t h = (k.begin * 0x9e3779b97f4a7c15ull) ^ (k.end + (k.write ? 0x7f4a7c15ull : 0));
            return static_cast<size_t>(h ^ (h >> 29));
        }
    };
    std::vector<Seen> seen;
    std::unordered_map<Key, uint32_t, KeyHash> known;
    std::unordered_map<uint64_t, std::vector<uint32_t>> buckets;
    std::vector<uint32_t> covered;
    int highest = -1;  // highest level so far
    int fence = -1;    // level of the last node with unknown memory use
    for (size_t index = 0; index < nodes.size(); index++) {
        RecNode& node = nodes[index];
        node.deps.clear();
        int level = fence + 1;
        if (node.type == RecNode::Source) {
            // unknown reads and writes: after everything before, before everything after
            node.level = fence = highest = highest + 1;
            continue;
        }
        covered.clear();
        for (const Access& a : node.acc) {
            if (a.end <= a.begin) continue;
            for (uint64_t c = a.begin >> kChunkShift; c <= (a.end - 1) >> kChunkShift; c++) {
                auto it = buckets.find(c);
                if (it == buckets.end()) continue;
                for (uint32_t si : it->second) {
                    const Seen& s = seen[si];
                    if (!edges && s.level < level) continue;  // cannot raise the level any more
                    if (!a.write && !s.write) continue;       // two reads never conflict
                    if (!(a.begin < s.end && s.begin < a.end)) continue;
                    level = std::max(level, s.level + 1);
                    if (!edges) continue;
                    node.deps.insert(node.deps.end(), s.users.begin(), s.users.end());
                    if (a.write && a.begin <= s.begin && s.end <= a.end && !s.users.empty()) covered.push_back(si);
                }
            }
        }
        node.level = level;
        highest = std::max(highest, level);
        if (edges) {
            std::sort(node.deps.begin(), node.deps.end());
            node.deps.erase(std::unique(node.deps.begin(), node.deps.end()), node.deps.end());
            for (uint32_t si : covered) seen[si].users.clear();
        }
        for (const Access& a : node.acc) {
            if (a.end <= a.begin) continue;
            auto [slot, fresh] = known.try_emplace(Key{a.begin, a.end, a.write}, static_cast<uint32_t>(seen.size()));
            if (!fresh) {
                Seen& s = seen[slot->second];
                s.level = std::max(s.level, level);
                if (edges && (s.users.empty() || s.users.back() != index)) s.users.push_back(static_cast<uint32_t>(index));
                continue;
            }
            seen.push_back({a.begin, a.end, a.write, level, {}});
            if (edges) seen.back().users.push_back(static_cast<uint32_t>(index));
            for (uint64_t c = a.begin >> kChunkShift; c <= (a.end - 1) >> kChunkShift; c++) buckets[c].push_back(slot->second);
        }
    }
}

// ---- joining producers with their consumers ----
//
// A recorded apply launch whose output a later apply launch reads element for element (the
// same address and length) is joined with that launch: ONE kernel evaluates both expressions
// per element, stores both results where the two launches stored them, and hands the first
// result to the second expression in a register instead of through memory.  `t = a * b;
// u = t + c; y = f(u)` becomes one launch that reads a, b, c and writes t, u, y: 24 instead of
// 32 bytes per f32 element, one launch instead of three.  Every buffer still receives exactly
// the value the separate launches gave it (the value handed on is the stored one, rounded to
// the storage type), so nothing a caller can observe changes.
//
// What may be joined.  Both are apply or unary-gradient launches of generated kernels (a
// gradient launch is the expression `g + (o * f'(x))` stored to g) with the same element type,
// length and alignment phase.  The consumer reads at least one output of the producer.
// Every address range of the one that the other also touches, one of them writing, is the
// SAME range (same address): the fused kernel handles element i of every operand in one
// lane, all loads before all stores, so equal ranges behave as in the separate launches and
// disjoint ones do not matter, but a range shifted against another would be read or written
// by another lane at another time.  And nothing recorded between the two conflicts with the
// producer (reads what it writes, writes what it reads or writes): the joined launch takes the
// consumer's place in the recording.  Joined launches are producers and consumers in turn.
//
// Two launches that only READ a common input (the forward launch of an operation and its
// gradient launch both read x) are joined under the same conditions: the earlier one commutes
// with everything up to the later one, and the joined kernel loads the common input once.

struct ChainBuild {
    // per stage: the kernel of its launch (whose expression it evaluates), where each variable of
    // that expression comes from (ChainStage::source), and where the launch stored its result
    std::vector<const custos_hip_kernel*> stage_kernel;
    std::vector<std::vector<int>> source;
    std::vector<uint64_t> stage_ptr;
    std::vector<uint64_t> ext;  // input pointers of the kernel to be
    size_t size() const { return stage_kernel.size(); }
};

// The last stage that writes `ptr`, or -1.
int writer_of(const ChainBuild& c, uint64_t ptr) {
    for (size_t s = c.stage_ptr.size(); s-- > 0;)
        if (c.stage_ptr[s] == ptr) return static_cast<int>(s);
    return -1;
}

int input_index(ChainBuild* c, uint64_t ptr) {
    for (size_t i = 0; i < c->ext.size(); i++)
        if (c->ext[i] == ptr) return static_cast<int>(i);
    c->ext.push_back(ptr);
    return static_cast<int>(c->ext.size()) - 1;
}

size_t distinct_outputs(const ChainBuild& c) {
    size_t n = 0;
    for (size_t s = 0; s < c.stage_ptr.size(); s++) n += writer_of(c, c.stage_ptr[s]) == static_cast<int>(s);
    return n;
}

bool fusable_kernel(const RecNode& n) {
    if (n.type != RecNode::Kernel || !n.k->spec.auto_unroll) return false;
    if (n.k->spec.kind != Kind::Apply && n.k->spec.kind != Kind::UnaryGrad) return false;
    return n.k->spec.tuning.blocks_per_cu <= 0;
}

// What a recorded launch evaluates per element, as an expression over its pointers: an apply
// launch its own expression over its inputs; a unary-gradient launch `g + (o * f'(x))` over
// (x, g, o) = (lhs, lhs_grad, out_grad), the product rounded before the sum like in its own kernel
// (src/devices/cpu_stack_ops.rs:27-29), stored to g.
Expr stage_expr(const custos_hip_kernel* k) {
    Expr e = k->spec.expr;
    if (k->spec.kind != Kind::UnaryGrad) return e;
    Node g, o, prod, sum;
    g.op = o.op = Op::Var;
    g.var = 1;
    o.var = 2;
    const int derivative = e.root, first = static_cast<int>(e.nodes.size());
    prod.op = Op::Mul;
    prod.a = first + 1;  // o
    prod.b = derivative;
    sum.op = Op::Add;
    sum.a = first;       // g
    sum.b = first + 2;   // o * f'(x)
    e.nodes.insert(e.nodes.end(), {g, o, prod, sum});
    e.root = first + 3;
    e.n_vars = 3;
    return e;
}

ChainBuild chain_of(const RecNode& n) {
    ChainBuild c;
    std::vector<int> source;
    if (n.k->spec.kind == Kind::UnaryGrad) {
        // (x, g, o) in the order of the launch's pointers; g is read and written
        for (size_t v = 0; v < 3; v++) source.push_back(input_index(&c, n.ptrs[v]));
        c.stage_ptr.push_back(n.ptrs[1]);
    } else {
        for (int v = 0; v < n.k->spec.expr.n_vars; v++) source.push_back(input_index(&c, n.ptrs[static_cast<size_t>(v)]));
        c.stage_ptr.push_back(n.ptrs.back());
    }
    c.source.push_back(std::move(source));
    c.stage_kernel.push_back(n.k);
    return c;
}

// `producer` followed by `consumer` as one chain (which takes `producer`'s place), or false if
// they may not be joined (`producer` is left as it was).  The consumer reads what the producer
// wrote -- or, with `sharing`, the two only read a common input, which the joined kernel then
// loads once.
bool join_chains(ChainBuild& producer, const ChainBuild& consumer, uint64_t bytes, bool sharing, ChainBuild* joined) {
    // every range of the one against every range of the other, one of them written: equal or disjoint
    auto clash = [&](uint64_t p, uint64_t q) { return p != q && p < q + bytes && q < p + bytes; };
    for (uint64_t w : producer.stage_ptr) {
        for (uint64_t q : consumer.ext)
            if (clash(w, q)) return false;
        for (uint64_t q : consumer.stage_ptr)
            if (clash(w, q)) return false;
    }
    for (uint64_t w : consumer.stage_ptr)
        for (uint64_t p : producer.ext)
            if (clash(w, p)) return false;
    bool related = false;
    for (uint64_t q : consumer.ext)
        related = related || writer_of(producer, q) >= 0 ||
                  (sharing && std::find(producer.ext.begin(), producer.ext.end(), q) != producer.ext.end());
    if (!related) return false;
    // the limits of one kernel, before anything is moved
    size_t inputs = producer.ext.size(), outputs = 0;
    for (uint64_t q : consumer.ext)
        inputs += writer_of(producer, q) < 0 && std::find(producer.ext.begin(), producer.ext.end(), q) == producer.ext.end();
    for (size_t s = 0; s < producer.size(); s++)
        outputs += writer_of(producer, producer.stage_ptr[s]) == static_cast<int>(s) && writer_of(consumer, producer.stage_ptr[s]) < 0;
    outputs += distinct_outputs(consumer);
    if (producer.size() + consumer.size() > static_cast<size_t>(kMaxChainStages) || inputs > static_cast<size_t>(kMaxChainInputs) ||
        outputs > static_cast<size_t>(kMaxChainOutputs))
        return false;
    const int shift = static_cast<int>(producer.size());
    ChainBuild c = std::move(producer);
    // what an input pointer of the consumer becomes: the stored value of the producer's stage
    // that wrote that memory last, or an input pointer of the joined kernel
    std::vector<int> mapped;
    for (uint64_t q : consumer.ext) {
        const int w = writer_of(c, q);
        mapped.push_back(w >= 0 ? -(1 + w) : input_index(&c, q));
    }
    for (size_t s = 0; s < consumer.size(); s++) {
        std::vector<int> source = consumer.source[s];
        for (int& from : source) from = from >= 0 ? mapped[static_cast<size_t>(from)] : from - shift;
        c.source.push_back(std::move(source));
        c.stage_ptr.push_back(consumer.stage_ptr[s]);
        c.stage_kernel.push_back(consumer.stage_kernel[s]);
    }
    *joined = std::move(c);
    return true;
}

// The recording `nodes` with producers joined into their consumers (see above), in `fused`.
// The kernels of the joined launches are only named here (handles from the cache, or new ones);
// the graph build compiles the entry point it replays each of them through, and hands back in
// `refused` those it could not get (time budget spent, compilation failed): their chains stay
// the launches they were recorded as (`left_unjoined` counts those launches).
int32_t fuse_producers(custos_hip_device* dev, const std::vector<RecNode>& nodes, bool share_reads,
                       const std::set<const custos_hip_kernel*>& refused, std::vector<RecNode>* fused_out, size_t* fused_away,
                       size_t* left_unjoined) {
    *fused_away = 0;
    *left_unjoined = 0;
    fused_out->clear();
    struct Candidate {
        size_t at;  // index into `out`
        ChainBuild chain;
        std::vector<Access> acc;
        bool open;
    };
    std::vector<RecNode> out;
    std::vector<char> dead;
    std::vector<int32_t> cand_at;  // per entry of `out`: its candidate (whose chain it stands for), or -1
    std::vector<Candidate> cands;
    std::unordered_map<uint64_t, std::vector<uint32_t>> buckets;
    size_t closed_below = 0;  // every candidate with a lower id is closed (a kernel with unknown memory use came by)
    size_t joined_launches = 0;
    std::vector<uint32_t> hits, sharers;
    for (const RecNode& node : nodes) {
        if (node.type == RecNode::Source) {
            closed_below = cands.size();
            out.push_back(node);
            dead.push_back(0);
            cand_at.push_back(-1);
            continue;
        }
        // open candidates this node conflicts with, and those that read exactly what it reads
        hits.clear();
        sharers.clear();
        for (const Access& a : node.acc) {
            if (a.end <= a.begin) continue;
            for (uint64_t c = a.begin >> kChunkShift; c <= (a.end - 1) >> kChunkShift; c++) {
                auto it = buckets.find(c);
                if (it == buckets.end()) continue;
                std::vector<uint32_t>& ids = it->second;
                size_t kept = 0;
                for (uint32_t id : ids) {
                    if (id < closed_below || !cands[id].open) continue;  // dropped from the list
                    ids[kept++] = id;
                    bool conflict = false, same_read = false;
                    for (const Access& b : cands[id].acc) {
                        conflict = conflict || ((a.write || b.write) && a.begin < b.end && b.begin < a.end);
                        same_read = same_read || (!a.write && !b.write && a.begin == b.begin && a.end == b.end);
                    }
                    if (conflict) hits.push_back(id);
                    else if (same_read && share_reads) sharers.push_back(id);
                }
                ids.resize(kept);
            }
        }
        std::sort(hits.begin(), hits.end());
        hits.erase(std::unique(hits.begin(), hits.end()), hits.end());
        const bool fusable = fusable_kernel(node);
        ChainBuild chain;
        if (fusable) chain = chain_of(node);
        const uint64_t bytes = node.n * (fusable ? dtype_size(node.k->spec.dtype) : 1);
        for (uint32_t id : hits) {
            Candidate& p = cands[id];
            p.open = false;  // joined or not, nothing later may be joined with it
            if (!fusable) continue;
            const RecNode& pn = out[p.at];
            if (pn.k->spec.dtype != node.k->spec.dtype || pn.n != node.n || pn.head != node.head || pn.n_vec != node.n_vec ||
                pn.k->spec.tuning.block_threads != node.k->spec.tuning.block_threads)
                continue;
            ChainBuild joined;
            if (!join_chains(p.chain, chain, bytes, /*sharing=*/false, &joined)) continue;
            chain = std::move(joined);
            dead[p.at] = 1;
            joined_launches++;
        }
        // then the candidate that only shares an input with it (it stays open if it cannot be
        // joined).  Only if there is exactly one: an input that several open launches read is a
        // common operand (a bias, a mask), not a sign that those launches belong together.
        std::sort(sharers.begin(), sharers.end());
        sharers.erase(std::unique(sharers.begin(), sharers.end()), sharers.end());
        sharers.erase(std::remove_if(sharers.begin(), sharers.end(),
                                     [&](uint32_t id) { return !cands[id].open || std::binary_search(hits.begin(), hits.end(), id); }),
                      sharers.end());
        if (sharers.size() != 1) sharers.clear();
        for (uint32_t id : sharers) {
            Candidate& p = cands[id];
            if (!fusable) continue;
            const RecNode& pn = out[p.at];
            if (pn.k->spec.dtype != node.k->spec.dtype || pn.n != node.n || pn.head != node.head || pn.n_vec != node.n_vec ||
                pn.k->spec.tuning.block_threads != node.k->spec.tuning.block_threads)
                continue;
            ChainBuild joined;
            if (!join_chains(p.chain, chain, bytes, /*sharing=*/true, &joined)) continue;
            chain = std::move(joined);
            p.open = false;
            dead[p.at] = 1;
            joined_launches++;
        }
        out.push_back(node);
        dead.push_back(0);
        cand_at.push_back(-1);
        if (!fusable) continue;
        Candidate c;
        c.at = out.size() - 1;
        c.open = true;
        for (uint64_t p : chain.ext) c.acc.push_back({p, p + bytes, false});
        for (size_t s = 0; s < chain.stage_ptr.size(); s++)
            if (writer_of(chain, chain.stage_ptr[s]) == static_cast<int>(s))
                c.acc.push_back({chain.stage_ptr[s], chain.stage_ptr[s] + bytes, true});
        for (const Access& a : c.acc)
            for (uint64_t ch = a.begin >> kChunkShift; ch <= (a.end - 1) >> kChunkShift; ch++)
                buckets[ch].push_back(static_cast<uint32_t>(cands.size()));
        cand_at.back() = static_cast<int32_t>(cands.size());
        c.chain = std::move(chain);
        cands.push_back(std::move(c));
    }
    if (joined_launches == 0) return CUSTOS_HIP_OK;
    // kernels of the chains; the nodes take their final form
    std::vector<RecNode> fused;
    // chains of the same launches wired the same way share a kernel: looked up once per shape
    std::map<std::vector<uint64_t>, custos_hip_kernel*> kernel_of_shape;
    for (size_t i = 0; i < out.size(); i++) {
        if (dead[i]) continue;
        RecNode node = std::move(out[i]);
        static const ChainBuild single;
        const ChainBuild& chain = cand_at[i] >= 0 ? cands[static_cast<size_t>(cand_at[i])].chain : single;
        if (chain.size() > 1) {
            std::vector<int> out_of(chain.size(), -1);
            std::vector<uint64_t> outs;
            for (size_t s = 0; s < chain.size(); s++) {
                if (writer_of(chain, chain.stage_ptr[s]) != static_cast<int>(s)) continue;
                out_of[s] = static_cast<int>(outs.size());
                outs.push_back(chain.stage_ptr[s]);
            }
            std::vector<uint64_t> shape = {chain.ext.size(), outs.size()};
            for (size_t s = 0; s < chain.size(); s++) {
                // (handles of one code differ in the values of their literal parameters only)
                shape.push_back(reinterpret_cast<uint64_t>(chain.stage_kernel[s]->code ? chain.stage_kernel[s]->code : chain.stage_kernel[s]));
                shape.push_back(static_cast<uint64_t>(static_cast<int64_t>(out_of[s])));
                for (int from : chain.source[s]) shape.push_back(static_cast<uint64_t>(static_cast<int64_t>(from)));
            }
            auto known = kernel_of_shape.find(shape);
            if (known == kernel_of_shape.end()) {
                custos_hip_kernel* k = nullptr;
                std::vector<ChainStage> stages(chain.size());
                for (size_t s = 0; s < chain.size(); s++) {
                    const custos_hip_kernel* sk = chain.stage_kernel[s];
                    stages[s].expr = stage_expr(sk);
                    stages[s].source = chain.source[s];
                    stages[s].out = out_of[s];
                    // a literal is in the chain's code, or one of its launch parameters, as it is for
                    // the launch's own kernel (the nodes a gradient stage adds hold no literals)
                    if (sk->spec.consts.n_params > 0) {
                        stages[s].slot = sk->spec.consts.slot;
                        stages[s].slot.resize(stages[s].expr.nodes.size(), -1);
                        stages[s].n_params = sk->spec.consts.n_params;
                        stages[s].param_bytes = sk->spec.consts.bytes.size();
                    }
                }
                Tuning tuning = node.k->spec.tuning;
                tuning.unroll = 0;  // (only kernels whose vectors per thread were left open are joined)
                // a shape without a kernel (one that cannot be generated, one the build refused) stays
                // the launches it was recorded as
                if (chain_kernel(dev, node.k->spec.dtype, std::move(stages), static_cast<int>(chain.ext.size()),
                                 static_cast<int>(outs.size()), tuning, &k) != CUSTOS_HIP_OK ||
                    refused.count(k))
                    k = nullptr;
                known = kernel_of_shape.emplace(std::move(shape), k).first;
            }
            custos_hip_kernel* const k = known->second;
            if (!k) {
                // the chain's launches again, in the order of its stages
                *left_unjoined += chain.size();
                const uint64_t bytes = node.n * dtype_size(node.k->spec.dtype);
                for (size_t s = 0; s < chain.size(); s++) {
                    RecNode single = node;
                    single.k = const_cast<custos_hip_kernel*>(chain.stage_kernel[s]);
                    single.ptrs.clear();
                    single.acc.clear();
                    single.const_bytes.clear();
                    for (int from : chain.source[s]) single.ptrs.push_back(from >= 0 ? chain.ext[static_cast<size_t>(from)] : chain.stage_ptr[static_cast<size_t>(-from - 1)]);
                    if (single.k->spec.kind != Kind::UnaryGrad) single.ptrs.push_back(chain.stage_ptr[s]);
                    for (size_t p = 0; p < single.ptrs.size(); p++) {
                        const bool written = single.k->spec.kind == Kind::UnaryGrad ? p == 1 : p + 1 == single.ptrs.size();
                        single.acc.push_back({single.ptrs[p], single.ptrs[p] + bytes, written});
                    }
                    fused.push_back(std::move(single));
                }
                continue;
            }
            const uint64_t bytes = node.n * dtype_size(node.k->spec.dtype);
            node.const_bytes.clear();
            for (const custos_hip_kernel* sk : chain.stage_kernel)
                node.const_bytes.insert(node.const_bytes.end(), sk->spec.consts.bytes.begin(), sk->spec.consts.bytes.end());
            node.k = k;
            node.ptrs = chain.ext;
            node.ptrs.insert(node.ptrs.end(), outs.begin(), outs.end());
            node.acc.clear();
            for (uint64_t p : chain.ext) node.acc.push_back({p, p + bytes, false});
            for (uint64_t p : outs) node.acc.push_back({p, p + bytes, true});
        }
        fused.push_back(std::move(node));
    }
    *fused_away = nodes.size() - fused.size();
    *fused_out = std::move(fused);
    return CUSTOS_HIP_OK;
}

bool batchable(const RecNode& n) {
    if (n.type != RecNode::Kernel || n.head != 0 || n.k->spec.kind == Kind::Source) return false;
    for (uint64_t p : n.ptrs)
        if (p & 15) return false;
    return true;
}

// One node of the graph to be: a recorded piece of work, or several launches merged.
struct Planned {
    std::vector<size_t> members;  // indices into the recorded list; more than one = one merged launch
    bool ragged = false;          // members differ in length
    size_t table_offset = 0;      // in u64 entries
    size_t map_offset = 0;        // ragged: start of the block map, in u64 entries
    size_t blocks = 0;            // ragged: workgroups
    custos_hip_kernel* kern = nullptr;  // kernels: the kernel of the (first) member
    ResolvedShape shape;                // kernels: vectors per thread and cache policy that suit the bytes the
                                        // node touches; whether it walks its tiles against the previous such node
    bool feeds_later = false;           // single launches: one of the next levels reads what it writes
};

// The entry point a planned kernel node is replayed through.
EntrySet entry_of(const Planned& p) {
    return p.members.size() == 1 ? EntrySet::Single : p.ragged ? EntrySet::Ragged : EntrySet::Batched;
}

// Tiles of one segment of a merged launch (merged launches keep the workgroup size the kernel was compiled for).
unsigned long long tiles_of(const custos_hip_kernel* k, const RecNode& n, int unroll) {
    const unsigned long long tile_vecs = static_cast<unsigned long long>(k->spec.tuning.block_threads) * unroll;
    return std::max(1ull, (n.n_vec + tile_vecs - 1) / tile_vecs);
}

// Whether a recorded piece of work reads the operand behind one of its accesses (the gradient
// operand of a unary-gradient kernel is read and written).
bool reads_operand(const RecNode& n, const Access& a) {
    return !a.write || (n.type == RecNode::Kernel && n.k->spec.kind == Kind::UnaryGrad);
}

// The traffic of one level's nodes, for the launch shapes of the levels after it.
void record_level(const std::vector<RecNode>& nodes, const std::vector<size_t>& of_level, RecentTraffic* history) {
    std::vector<Access> all;
    for (size_t i : of_level)
        if (nodes[i].type != RecNode::Source) all.insert(all.end(), nodes[i].acc.begin(), nodes[i].acc.end());
    unsigned long long bytes = 0;
    for (const Access& a : all) bytes += a.end - a.begin;
    if (bytes > kTrafficBeyondBytes) history->record(all);
}

// The nodes of one dependency level: launches of one kernel (or of one code with different
// literal values) are merged -- equal lengths into a `_batched` grid, different lengths into a
// `_ragged` one --, everything else stays single.
std::vector<Planned> group_level(const custos_hip_device* dev, const std::vector<RecNode>& nodes,
                                 const std::vector<size_t>& of_level) {
    std::vector<Planned> out;
    // candidates for merging, grouped by code in first-seen order
    std::vector<std::pair<custos_hip_kernel*, std::vector<size_t>>> groups;
    for (size_t i : of_level) {
        if (dev->batching && batchable(nodes[i])) {
            auto g = std::find_if(groups.begin(), groups.end(), [&](const auto& kv) { return kv.first == nodes[i].k->code; });
            if (g == groups.end()) {
                groups.push_back({nodes[i].k->code, {}});
                g = groups.end() - 1;
            }
            g->second.push_back(i);
        } else {
            out.emplace_back();
            out.back().members.push_back(i);
        }
    }
    for (auto& g : groups) {
        bool uniform = true;
        for (size_t i : g.second) uniform = uniform && nodes[i].n == nodes[g.second[0]].n;
        if (uniform) {
            // equal lengths: one grid, segment = block / tiles per segment
            std::vector<std::pair<unsigned long long, Planned>> by_n;
            for (size_t i : g.second) {
                auto it = std::find_if(by_n.begin(), by_n.end(), [&](const auto& kv) { return kv.first == nodes[i].n; });
                if (it == by_n.end()) {
                    by_n.push_back({nodes[i].n, Planned{}});
                    it = by_n.end() - 1;
                }
                it->second.members.push_back(i);
            }
            for (auto& kv : by_n) out.push_back(std::move(kv.second));
            continue;
        }
        // different lengths: one grid with a block map; a launch that fills the chip on its
        // own stays a launch of its own
        Planned merged;
        for (size_t i : g.second) {
            if (tiles_of(nodes[i].k, nodes[i], 2) > kRaggedMaxTiles) {
                out.emplace_back();
                out.back().members.push_back(i);
            } else {
                merged.members.push_back(i);
            }
        }
        merged.ragged = merged.members.size() > 1;
        if (!merged.members.empty()) out.push_back(std::move(merged));
    }
    return out;
}

// What the launches around a (merged) kernel node say about it: the levels before it (`history`),
// and whether one of the levels after it reads what it writes (`later_reads`).
CacheHint hint_for(const std::vector<RecNode>& nodes, const Planned& p, const RecentTraffic& history,
                   const std::vector<const std::vector<Access>*>& later_reads) {
    std::vector<Access> all, reads;
    bool feeds_later = false;
    for (size_t i : p.members)
        for (const Access& a : nodes[i].acc) {
            all.push_back(a);
            if (reads_operand(nodes[i], a)) reads.push_back(a);
            if (!a.write) continue;
            for (const std::vector<Access>* level : later_reads)
                for (const Access& r : *level) feeds_later = feeds_later || (r.begin < a.end && a.begin < r.end);
        }
    return history.classify(reads, all, feeds_later);
}

// Table rows of a merged launch: per member its operand addresses, for a ragged launch its
// length, then its literal parameters padded to whole words; after the rows of a ragged
// launch the block map (segment << 32 | tile per workgroup).
void append_tables(const std::vector<RecNode>& nodes, Planned* p, std::vector<uint64_t>* host_table) {
    p->table_offset = host_table->size();
    for (size_t member : p->members) {
        for (uint64_t ptr : nodes[member].ptrs) host_table->push_back(ptr);
        if (p->ragged) host_table->push_back(nodes[member].n);
        const std::vector<unsigned char>& values = literal_values(nodes[member]);
        for (size_t at = 0; at < values.size(); at += 8) {
            uint64_t word = 0;
            std::memcpy(&word, values.data() + at, std::min<size_t>(8, values.size() - at));
            host_table->push_back(word);
        }
    }
    if (!p->ragged) return;
    p->map_offset = host_table->size();
    for (size_t seg = 0; seg < p->members.size(); seg++) {
        const unsigned long long tiles = tiles_of(p->kern, nodes[p->members[seg]], p->shape.unroll);
        for (unsigned long long t = 0; t < tiles; t++) host_table->push_back(static_cast<uint64_t>(seg) << 32 | t);
    }
    p->blocks = host_table->size() - p->map_offset;
}

// Plans one level: merging, the launch shape of every kernel node, the tables of the merged
// launches (appended to `host_table`); then the level's traffic joins `history`.
std::vector<Planned> plan_level(custos_hip_device* dev, const std::vector<RecNode>& nodes,
                                const std::vector<size_t>& of_level, RecentTraffic* history,
                                const std::vector<const std::vector<Access>*>& later_reads,
                                std::vector<uint64_t>* host_table) {
    std::vector<Planned> out = group_level(dev, nodes, of_level);
    for (Planned& p : out) {
        const RecNode& first = nodes[p.members[0]];
        if (first.type == RecNode::Kernel) {
            // the launch shape follows the bytes the (merged) launch touches and the launches around it
            p.kern = first.k;
            unsigned long long touched = 0;
            for (const Access& a : first.acc) touched += a.end - a.begin;
            if (p.members.size() == 1 && touched > kTrafficBeyondBytes) {
                // one large launch: decided as for a launch issued directly, with what the graph knows on
                // top (whether one of the next levels reads what it writes)
                if (touched >= kHintFromBytes)
                    for (const Access& a : first.acc)
                        for (const std::vector<Access>* level : later_reads)
                            for (const Access& r : *level)
                                p.feeds_later = p.feeds_later || (a.write && r.begin < a.end && a.begin < r.end);
                RecentTraffic before = *history;  // (the level's traffic joins the history below, once)
                p.shape = shape_of_launch(dev, first.k, first.acc, &before, p.feeds_later);
            } else {
                unsigned long long footprint = 0;
                for (size_t i : p.members) footprint += nodes[i].ptrs.size() * nodes[i].n * dtype_size(nodes[i].k->spec.dtype);
                CacheHint hint = CacheHint::Unknown;
                unsigned long long working_set = 0;
                if (footprint >= kHintFromBytes) {
                    hint = hint_for(nodes, p, *history, later_reads);
                    dev->hinted[static_cast<int>(hint)]++;
                }
                if (footprint > kTrafficBeyondBytes) {
                    std::vector<Access> all;
                    for (size_t i : p.members) all.insert(all.end(), nodes[i].acc.begin(), nodes[i].acc.end());
                    working_set = history->working_set_with(all);
                }
                p.shape = resolve_shape(dev, first.k, footprint, hint, working_set);
                dev->last_shape[0] = p.shape.unroll, dev->last_shape[1] = p.shape.nontemporal, dev->last_shape[2] = p.shape.alternate;
                dev->last_shape[3] = p.shape.block;
            }
        }
        if (p.members.size() > 1) append_tables(nodes, &p, host_table);
    }
    record_level(nodes, of_level, history);
    return out;
}

std::vector<unsigned char> value(const void* p, size_t n) {
    const unsigned char* c = static_cast<const unsigned char*>(p);
    return std::vector<unsigned char>(c, c + n);
}

// A planned node in launchable form: function, launch shape, argument values.  `rev` is the
// direction bit of a generated kernel's mode word; `table` the device address of the graph's tables.
int32_t lower_node(custos_hip_device* dev, const std::vector<RecNode>& nodes, const Planned& p, uint64_t table,
                   unsigned long long rev, LoweredNode* out) {
    const RecNode& first = nodes[p.members[0]];
    LoweredNode ln;
    if (first.type == RecNode::Copy) {
        ln.is_copy = true;
        ln.dst = first.ptrs[0];
        ln.src = first.ptrs[1];
        ln.bytes = first.bytes;
    } else if (first.type == RecNode::Source) {
        ln.args = first.arg_values;
        ln.func = reinterpret_cast<void*>(first.k->fns[0]);
        ln.grid = dim3(first.grid3[0], first.grid3[1], first.grid3[2]);
        ln.block = dim3(first.block3[0], first.block3[1], first.block3[2]);
        ln.shared_mem = first.shared_mem;
    } else if (first.type == RecNode::Fill) {
        const unsigned long long a0 = first.bytes, a1 = first.head, a2 = first.n_vec;
        ln.args = {value(&first.ptrs[0], 8), value(&a0, 8), value(&a1, 8), value(&a2, 8)};
        for (uint32_t word : first.pattern) ln.args.push_back(value(&word, 4));
        ln.func = first.pattern.empty() ? fill_zero_kernel() : fill_pattern_kernel();
        ln.module_fn = false;
        ln.grid = dim3(fill_grid(dev, first.n_vec));
        ln.block = dim3(fill_block());
    } else {
        ln.block = dim3(static_cast<unsigned int>(p.shape.block));
        // (compiled by now: build_graph asked for the entry point of every planned node)
        hipFunction_t fn = nullptr;
        int32_t rc = entry_point(dev, p.kern, entry_of(p), &fn);
        if (rc != CUSTOS_HIP_OK) return rc;
        ln.func = reinterpret_cast<void*>(fn);
        if (p.members.size() == 1) {
            for (uint64_t ptr : first.ptrs) ln.args.push_back(value(&ptr, 8));
            const unsigned long long a0 = first.n, a1 = first.head, a2 = first.n_vec;
            ln.args.push_back(value(&a0, 8));
            ln.args.push_back(value(&a1, 8));
            ln.args.push_back(value(&a2, 8));
            ln.grid = dim3(launch_grid(dev, p.kern, first.n, first.n_vec, p.shape));
            // what a replay as plain launches needs to choose the shape again (replay_graph)
            unsigned long long touched = 0;
            for (const Access& a : first.acc) touched += a.end - a.begin;
            if (touched > kTrafficBeyondBytes && p.kern->spec.auto_unroll) {
                ln.kern = p.kern;
                ln.n = first.n, ln.head = first.head, ln.n_vec = first.n_vec;
                ln.acc = first.acc;
                ln.feeds_later = p.feeds_later;
            }
        } else if (p.ragged) {
            if (p.blocks > (1ull << 31) - 1)
                return set_error(dev, CUSTOS_HIP_ERR_TOO_LARGE, "a merged launch would need more than 2^31 workgroups");
            const uint64_t rows = table + p.table_offset * sizeof(uint64_t);
            const uint64_t map = table + p.map_offset * sizeof(uint64_t);
            ln.args = {value(&rows, 8), value(&map, 8)};
            ln.grid = dim3(static_cast<unsigned int>(p.blocks));
        } else {
            const unsigned long long tiles_per_seg = tiles_of(p.kern, first, p.shape.unroll);
            const unsigned long long blocks = tiles_per_seg * p.members.size();
            if (blocks > (1ull << 31) - 1)
                return set_error(dev, CUSTOS_HIP_ERR_TOO_LARGE, "a batched launch would need more than 2^31 workgroups");
            const uint64_t rows = table + p.table_offset * sizeof(uint64_t);
            const unsigned long long a0 = first.n, a1 = first.n_vec;
            ln.args = {value(&rows, 8), value(&a0, 8), value(&a1, 8), value(&tiles_per_seg, 8)};
            ln.grid = dim3(static_cast<unsigned int>(blocks));
        }
        // a generated entry point ends with the block of literal parameters (if the
        // expression has any) and the direction
        // (a merged launch reads them from its table rows instead)
        if (first.k->spec.consts.n_params > 0 && p.members.size() == 1) ln.args.push_back(literal_values(first));
        const unsigned long long mode = p.members.size() == 1
                                            ? single_launch_mode(p.kern, first.n, first.head, first.n_vec, p.shape, rev != 0)
                                            : launch_mode(p.shape.unroll, p.shape.nontemporal, rev != 0, p.shape.block);
        ln.args.push_back(value(&mode, 8));
        ln.mode_arg = static_cast<int>(ln.args.size()) - 1;
        if (p.shape.alternate) ln.rev_arg = ln.mode_arg;
    }
    *out = std::move(ln);
    return CUSTOS_HIP_OK;
}

// Everything that decides what a recording does, word by word: two recordings with equal
// signatures build equal graphs.  (A kernel handle stands for its code and its literal values.)
std::vector<uint64_t> signature(const std::vector<RecNode>& nodes) {
    std::vector<uint64_t> sig;
    sig.reserve(nodes.size() * 10);
    for (const RecNode& n : nodes) {
        sig.push_back(static_cast<uint64_t>(n.type));
        sig.push_back(reinterpret_cast<uint64_t>(n.k));
        sig.insert(sig.end(), {n.n, n.head, n.n_vec, n.bytes, static_cast<uint64_t>(n.ptrs.size())});
        sig.insert(sig.end(), n.ptrs.begin(), n.ptrs.end());
        sig.push_back(n.pattern.size());
        sig.insert(sig.end(), n.pattern.begin(), n.pattern.end());
        if (n.type != RecNode::Source) continue;
        for (int d = 0; d < 3; d++) sig.push_back(static_cast<uint64_t>(n.grid3[d]) << 32 | n.block3[d]);
        sig.push_back(n.shared_mem);
        sig.push_back(n.arg_values.size());
        for (const auto& value : n.arg_values) {
            sig.push_back(value.size());
            for (size_t at = 0; at < value.size(); at += 8) {
                uint64_t word = 0;
                std::memcpy(&word, value.data() + at, std::min<size_t>(8, value.size() - at));
                sig.push_back(word);
            }
        }
    }
    return sig;
}

// What every node of the graph to be waits for, as indices into the nodes in level order.
// Level joins: a node waits for the whole level before it (`join_levels`).  Per-node edges: a
// node waits for the nodes that hold the recorded work its members conflict with; a node with
// unknown memory use waits for everything before it that nothing waits for yet, and everything
// after it waits for it, directly or through a node that does.
std::vector<std::vector<uint32_t>> node_edges(const std::vector<RecNode>& nodes, const std::vector<std::vector<Planned>>& plan) {
    std::vector<uint32_t> planned_of(nodes.size(), 0);
    uint32_t id = 0;
    for (const auto& level : plan)
        for (const Planned& p : level) {
            for (size_t m : p.members) planned_of[m] = id;
            id++;
        }
    std::vector<std::vector<uint32_t>> waits(id);
    std::vector<char> waited_for(id, 0);
    int64_t fence = -1;  // the last node with unknown memory use
    id = 0;
    for (const auto& level : plan)
        for (const Planned& p : level) {
            std::vector<uint32_t>& w = waits[id];
            if (nodes[p.members[0]].type == RecNode::Source) {
                for (uint32_t q = fence < 0 ? 0 : static_cast<uint32_t>(fence); q < id; q++)
                    if (!waited_for[q]) w.push_back(q);
                fence = id;
            } else {
                for (size_t m : p.members)
                    for (uint32_t d : nodes[m].deps) w.push_back(planned_of[d]);
                std::sort(w.begin(), w.end());
                w.erase(std::unique(w.begin(), w.end()), w.end());
                if (fence >= 0) {
                    // everything before the fence precedes it; the fence itself is waited for
                    // unless a node that follows it is
                    w.erase(w.begin(), std::lower_bound(w.begin(), w.end(), static_cast<uint32_t>(fence)));
                    if (w.empty()) w.push_back(static_cast<uint32_t>(fence));
                }
            }
            for (uint32_t q : w) waited_for[q] = 1;
            id++;
        }
    return waits;
}

// One chain has to put the nodes in SOME order that respects their dependencies.  Level by
// level is one; it interleaves independent chains, so that a chain over large buffers finds
// nothing of its own left in the caches when its next launch comes.  This order follows the
// recording instead: among the nodes whose dependencies are out, the one whose first launch
// was recorded first.  A program recorded chain by chain replays chain by chain, one recorded
// level by level stays as it is, and so do merged launches (their first members were recorded
// in level order).  Returns the recorded work of every node, in that order.
std::vector<std::vector<size_t>> stages_in_recording_order(const custos_hip_device* dev, const std::vector<RecNode>& nodes,
                                                           const std::vector<std::vector<size_t>>& by_level) {
    std::vector<std::vector<Planned>> groups;
    for (const auto& of_level : by_level) groups.push_back(group_level(dev, nodes, of_level));
    const std::vector<std::vector<uint32_t>> waits = node_edges(nodes, groups);
    std::vector<const Planned*> flat;
    for (const auto& level : groups)
        for (const Planned& p : level) flat.push_back(&p);
    std::vector<std::vector<uint32_t>> followers(flat.size());
    std::vector<uint32_t> pending(flat.size(), 0);
    for (uint32_t id = 0; id < flat.size(); id++) {
        pending[id] = static_cast<uint32_t>(waits[id].size());
        for (uint32_t q : waits[id]) followers[q].push_back(id);
    }
    auto first_recorded = [&](uint32_t id) { return *std::min_element(flat[id]->members.begin(), flat[id]->members.end()); };
    typedef std::pair<size_t, uint32_t> Ready;  // (first recorded member, node)
    std::priority_queue<Ready, std::vector<Ready>, std::greater<Ready>> ready;
    for (uint32_t id = 0; id < flat.size(); id++)
        if (pending[id] == 0) ready.push({first_recorded(id), id});
    std::vector<std::vector<size_t>> stages;
    while (!ready.empty()) {
        const uint32_t id = ready.top().second;
        ready.pop();
        stages.push_back(flat[id]->members);
        for (uint32_t f : followers[id])
            if (--pending[f] == 0) ready.push({first_recorded(f), f});
    }
    return stages;
}

// Brute-force check of a built graph's ordering, independent of how the edges were found: every
// two recorded pieces of work that touch overlapping memory, one of them writing (or one of
// them with unknown memory use), must sit in different nodes with a path from the earlier one's
// node to the later one's.  Quadratic in the recorded work; for tests.
bool ordering_holds(const std::vector<RecNode>& nodes, const std::vector<std::vector<Planned>>& plan,
                    const std::vector<std::vector<uint32_t>>& waits) {
    std::vector<uint32_t> planned_of(nodes.size(), 0);
    uint32_t count = 0;
    for (const auto& level : plan)
        for (const Planned& p : level) {
            for (size_t m : p.members) planned_of[m] = count;
            count++;
        }
    // reach[b][a]: node a runs before node b.  Nodes only wait for nodes made before them.
    std::vector<std::vector<char>> reach(count, std::vector<char>(count, 0));
    for (uint32_t b = 0; b < count; b++)
        for (uint32_t a : waits[b]) {
            if (a >= b) return false;
            reach[b][a] = 1;
            for (uint32_t c = 0; c < a; c++) reach[b][c] = reach[b][c] | reach[a][c];
        }
    auto conflict = [](const RecNode& x, const RecNode& y) {
        if (x.type == RecNode::Source || y.type == RecNode::Source) return true;
        for (const Access& a : x.acc)
            for (const Access& b : y.acc)
                if ((a.write || b.write) && a.begin < b.end && b.begin < a.end && a.begin < a.end && b.begin < b.end) return true;
        return false;
    };
    for (size_t j = 0; j < nodes.size(); j++)
        for (size_t i = 0; i < j; i++)
            if (conflict(nodes[i], nodes[j]) && !reach[planned_of[j]][planned_of[i]]) return false;
    return true;
}

// The waits of level joins, in the form node_edges gives: everything of the level before.
std::vector<std::vector<uint32_t>> level_waits(const std::vector<std::vector<Planned>>& plan) {
    std::vector<std::vector<uint32_t>> waits;
    uint32_t first_of_previous = 0, first_of_this = 0;
    for (const auto& level : plan) {
        for (size_t k = 0; k < level.size(); k++) {
            waits.emplace_back();
            for (uint32_t q = first_of_previous; q < first_of_this; q++) waits.back().push_back(q);
        }
        first_of_previous = first_of_this;
        first_of_this += static_cast<uint32_t>(level.size());
    }
    return waits;
}

// Issues one lowered node on `stream` (a replay as plain launches; the recording pass of
// instantiate_chain).
hipError_t issue_node(LoweredNode& ln, hipStream_t stream) {
    if (ln.is_copy)
        return hipMemcpyAsync(reinterpret_cast<void*>(ln.dst), reinterpret_cast<const void*>(ln.src), ln.bytes,
                              hipMemcpyDeviceToDevice, stream);
    void* argv[24];
    std::vector<void*> more;
    void** args = argv;
    if (ln.args.size() > 24) {
        more.resize(ln.args.size());
        args = more.data();
    }
    for (size_t i = 0; i < ln.args.size(); i++) args[i] = ln.args[i].data();
    if (ln.module_fn)
        return hipModuleLaunchKernel(static_cast<hipFunction_t>(ln.func), ln.grid.x, ln.grid.y, ln.grid.z, ln.block.x, ln.block.y,
                                     ln.block.z, ln.shared_mem, stream, args, nullptr);
    return hipLaunchKernel(ln.func, ln.grid, ln.block, args, ln.shared_mem, stream);
}

// One chain as an instantiated hipGraph: the nodes are launched, in the chain's order, on a
// stream of their own that is in capture mode, which is how the runtime takes kernels of
// run-time compiled modules into a graph (hipModuleLaunchKernel with their hipFunction_t; the
// `func` of hipGraphAddKernelNode's parameters is documented as a host function, and handing it
// a hipFunction_t, which the runtime happens to accept, ended a traced run inside
// hipGraphLaunch).  Relaxed mode: other threads with devices of their own keep allocating.
int32_t instantiate_chain(custos_hip_device* dev, custos_hip_graph* g, std::vector<std::vector<LoweredNode>>& lowered) {
    hipStream_t recording = nullptr;
    HIP_TRY(dev, hipStreamCreateWithFlags(&recording, hipStreamNonBlocking));
    hipError_t e = hipStreamBeginCapture(recording, hipStreamCaptureModeRelaxed);
    size_t issued = 0;
    for (auto& level : lowered)
        for (LoweredNode& ln : level) {
            if (e != hipSuccess) break;
            e = issue_node(ln, recording);
            issued++;
        }
    hipGraph_t captured = nullptr;
    const hipError_t ended = hipStreamEndCapture(recording, &captured);  // (also after a failure: it closes the capture)
    (void)hipStreamDestroy(recording);
    if (e == hipSuccess) e = ended;
    if (e != hipSuccess) {
        if (captured) (void)hipGraphDestroy(captured);
        return hip_fail(dev, e, "recording a chain of launches into a hipGraph");
    }
    g->graph = captured;
    g->edges = issued ? issued - 1 : 0;
    HIP_TRY(dev, hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0));
    return CUSTOS_HIP_OK;
}

// The plan as an instantiated hipGraph.  With level joins the nodes of a level sit side by side
// behind one empty node that waits for the level before (instead of |previous| x |level|
// edges); with per-node edges (`waits`) every node follows exactly what it conflicts with.
int32_t instantiate(custos_hip_device* dev, custos_hip_graph* g, std::vector<std::vector<LoweredNode>>& lowered,
                    const std::vector<std::vector<uint32_t>>* waits) {
    HIP_TRY(dev, hipGraphCreate(&g->graph, 0));
    std::vector<hipGraphNode_t> prev;  // level joins: what the nodes of the current level wait for
    std::vector<hipGraphNode_t> all;   // per-node edges: every node made so far
    for (auto& level : lowered) {
        std::vector<hipGraphNode_t> deps = prev;
        if (!waits && deps.size() > 1) {
            hipGraphNode_t join;
            HIP_TRY(dev, hipGraphAddEmptyNode(&join, g->graph, deps.data(), deps.size()));
            g->edges += deps.size();
            deps = {join};
        }
        std::vector<hipGraphNode_t> made;
        for (LoweredNode& ln : level) {
            if (waits) {
                deps.clear();
                for (uint32_t q : (*waits)[all.size()]) deps.push_back(all[q]);
            }
            hipGraphNode_t node;
            if (ln.is_copy) {
                HIP_TRY(dev, hipGraphAddMemcpyNode1D(&node, g->graph, deps.data(), deps.size(),
                                                     reinterpret_cast<void*>(ln.dst),
                                                     reinterpret_cast<const void*>(ln.src), ln.bytes,
                                                     hipMemcpyDeviceToDevice));
            } else {
                std::vector<void*> args;
                for (auto& v : ln.args) args.push_back(v.data());
                hipKernelNodeParams kp{};
                kp.func = ln.func;
                kp.gridDim = ln.grid;
                kp.blockDim = ln.block;
                kp.sharedMemBytes = ln.shared_mem;
                kp.kernelParams = args.data();
                kp.extra = nullptr;
                HIP_TRY(dev, hipGraphAddKernelNode(&node, g->graph, deps.data(), deps.size(), &kp));
            }
            g->edges += deps.size();
            made.push_back(node);
            all.push_back(node);
        }
        prev = std::move(made);
    }
    HIP_TRY(dev, hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0));
    return CUSTOS_HIP_OK;
}

}  // namespace

int32_t build_graph(custos_hip_device* dev, custos_hip_graph* g) {
    g->recorded = dev->recorded.size();
    g->signature = signature(dev->recorded);
    g->built_with = {dev->batching ? 1u : 0u, static_cast<uint64_t>(dev->graph_edges), dev->direct_replay_max,
                     dev->fusing ? 1u : 0u};
    const bool serial = dev->graph_edges == CUSTOS_HIP_GRAPH_EDGES_CHAIN || dev->graph_edges == CUSTOS_HIP_GRAPH_EDGES_CHAIN_BY_LEVEL;

    // Plan, then get the entry point every planned kernel node is replayed through.  The kernels
    // of joined launches are new code that nothing but this graph asked for: they are compiled
    // while the build has spent less than its budget on them, and a chain whose kernel the build
    // does not get (budget, a compilation that fails) goes back to the launches it was recorded
    // as -- the recording is then joined and planned again without it (once or twice: what was
    // compiled on the way is cached).
    std::vector<RecNode> joined;
    std::set<const custos_hip_kernel*> refused;
    uint64_t spent_on_joined_ns = 0;
    std::vector<std::vector<Planned>> plan;
    std::vector<uint64_t> host_table;
    const std::vector<RecNode>* planned_from = nullptr;
    for (;;) {
        std::vector<RecNode>* use = &dev->recorded;
        g->fused_away = g->unjoined = 0;
        if (dev->fusing) {
            const std::string error_before = dev->last_error;
            if (fuse_producers(dev, dev->recorded, /*share_reads=*/true, refused, &joined, &g->fused_away, &g->unjoined) == CUSTOS_HIP_OK &&
                g->fused_away > 0)
                use = &joined;
            else
                g->fused_away = 0;
            dev->last_error = error_before;
        }
        std::vector<RecNode>& nodes = *use;
        // The order of a chain only matters where a launch is large enough for the caches to matter;
        // a recording of small launches keeps the level order and the cheaper analysis.
        bool follow_recording = false;
        if (dev->graph_edges == CUSTOS_HIP_GRAPH_EDGES_CHAIN)
            for (const RecNode& n : nodes) {
                unsigned long long touched = 0;
                for (const Access& a : n.acc) touched += a.end - a.begin;
                follow_recording = follow_recording || touched >= kFollowRecordingFromBytes;
            }
        assign_levels(nodes, dev->graph_edges == CUSTOS_HIP_GRAPH_EDGES_PER_NODE || follow_recording);
        int max_level = -1;
        for (const RecNode& n : nodes) max_level = std::max(max_level, n.level);
        g->levels = static_cast<size_t>(max_level + 1);

        plan.clear();
        host_table.clear();
        std::vector<std::vector<size_t>> by_level(static_cast<size_t>(max_level + 1));
        for (size_t i = 0; i < nodes.size(); i++) by_level[static_cast<size_t>(nodes[i].level)].push_back(i);
        // One chain: from here on a "level" is one node, in the order the chain will have.
        if (follow_recording) by_level = stages_in_recording_order(dev, nodes, by_level);
        // A graph is built to be replayed: its first levels follow its last ones, so the traffic
        // history starts with one pass over the whole graph.
        RecentTraffic history;
        for (const auto& of_level : by_level) record_level(nodes, of_level, &history);
        // what every level reads, for the producers in the levels before it (the levels after the
        // last one are the first ones of the next replay)
        std::vector<std::vector<Access>> level_reads(by_level.size());
        for (size_t level = 0; level < by_level.size(); level++)
            for (size_t i : by_level[level])
                for (const Access& a : nodes[i].acc)
                    if (nodes[i].type != RecNode::Source && reads_operand(nodes[i], a)) level_reads[level].push_back(a);
        for (size_t level = 0; level < by_level.size(); level++) {
            std::vector<const std::vector<Access>*> later_reads;
            for (size_t ahead = 1; ahead <= kLookAheadLevels && ahead <= by_level.size(); ahead++)
                later_reads.push_back(&level_reads[(level + ahead) % by_level.size()]);
            plan.push_back(plan_level(dev, nodes, by_level[level], &history, later_reads, &host_table));
        }
        planned_from = use;

        bool plan_again = false;
        for (const auto& level : plan)
            for (const Planned& p : level) {
                if (!p.kern) continue;
                custos_hip_kernel* owner = p.kern->code ? p.kern->code : p.kern;
                const EntrySet which = entry_of(p);
                if (owner->fns[static_cast<int>(which)] || refused.count(owner)) continue;
                hipFunction_t fn = nullptr;
                if (owner->spec.kind != Kind::Chain) {
                    // (a kernel made while the device was recording, or its first merged launch)
                    int32_t rc = entry_point(dev, owner, which, &fn);
                    if (rc != CUSTOS_HIP_OK) return rc;
                    continue;
                }
                if (spent_on_joined_ns >= dev->fusing_budget_ms * 1000000ull) {
                    refused.insert(owner);
                    if (g->unjoined_reason.empty())
                        g->unjoined_reason = "the build's time budget for compiling kernels of joined launches (" +
                                             std::to_string(dev->fusing_budget_ms) + " ms) was spent";
                    plan_again = true;
                    continue;
                }
                const uint64_t before = dev->compile_ns;
                const std::string error_before = dev->last_error;
                const int32_t rc = entry_point(dev, owner, which, &fn);
                spent_on_joined_ns += dev->compile_ns - before;
                if (rc != CUSTOS_HIP_OK) {
                    refused.insert(owner);
                    g->unjoined_reason = dev->last_error;
                    dev->last_error = error_before;
                    plan_again = true;
                }
            }
        if (!plan_again) break;
    }
    std::vector<RecNode>& nodes = *const_cast<std::vector<RecNode>*>(planned_from);

    if (!host_table.empty()) {
        HIP_TRY(dev, hipMalloc(&g->table, host_table.size() * sizeof(uint64_t)));
        // (in stream order on the compute stream, where every launch of the graph follows)
        int32_t rc = send_to_device(dev, reinterpret_cast<uint64_t>(g->table), host_table.data(), host_table.size() * sizeof(uint64_t));
        if (rc != CUSTOS_HIP_OK) return rc;
    }

    std::vector<std::vector<LoweredNode>> lowered(plan.size());
    unsigned long long parity = 0;
    size_t total = 0;
    bool chain = true;
    for (size_t level = 0; level < plan.size(); level++) {
        for (const Planned& p : plan[level]) {
            // a node that alternates runs against the direction of the one before it
            const unsigned long long rev = p.shape.alternate ? (parity ^= 1) : 0;
            LoweredNode ln;
            int32_t rc = lower_node(dev, nodes, p, reinterpret_cast<uint64_t>(g->table), rev, &ln);
            if (rc != CUSTOS_HIP_OK) return rc;
            if (!ln.is_copy) {
                g->kernel_nodes++;
                const RecNode& first = nodes[p.members[0]];
                if (first.type == RecNode::Fill) g->node_names.push_back(first.pattern.empty() ? "custos_fill_zero" : "custos_fill_pattern");
                else if (first.type == RecNode::Source) g->node_names.push_back(first.k->spec.name);
                else g->node_names.push_back(p.kern->spec.name + (p.members.size() == 1 ? "" : p.ragged ? "_ragged" : "_batched"));
            }
            lowered[level].push_back(std::move(ln));
            total++;
        }
        chain = chain && lowered[level].size() == 1;
    }

    // In one chain every order that follows the levels is a valid one, so a short graph of any
    // shape can be replayed as plain launches.
    if ((chain || serial) && total <= dev->direct_replay_max) {
        for (auto& level : lowered)
            for (LoweredNode& ln : level) g->direct.push_back(std::move(ln));
        // With an odd number of alternating nodes the first one of the next replay would
        // run in the direction of the last one of this replay: flip them all every replay.
        size_t alternating = 0;
        for (const LoweredNode& ln : g->direct) alternating += ln.rev_arg >= 0;
        g->flip_each_replay = alternating % 2 == 1;
        return CUSTOS_HIP_OK;
    }
    std::vector<std::vector<uint32_t>> waits;
    if (dev->graph_edges == CUSTOS_HIP_GRAPH_EDGES_PER_NODE) {
        waits = node_edges(nodes, plan);
    } else if (serial) {
        waits.resize(total);
        for (uint32_t id = 1; id < total; id++) waits[id].push_back(id - 1);
    } else {
        waits = level_waits(plan);
    }
    if (dev->graph_verify) {
        if (nodes.size() > 8192) return set_error(dev, CUSTOS_HIP_ERR_TOO_LARGE, "recording too long for the brute-force ordering check");
        if (!ordering_holds(nodes, plan, waits))
            return set_error(dev, CUSTOS_HIP_ERR_GRAPH_ORDER, "built graph does not order two conflicting pieces of recorded work");
    }
    if (serial) return instantiate_chain(dev, g, lowered);
    return instantiate(dev, g, lowered, dev->graph_edges == CUSTOS_HIP_GRAPH_EDGES_LEVEL_JOINS ? nullptr : &waits);
}

int32_t replay_graph(custos_hip_device* dev, custos_hip_graph* g) {
    dev->graph_since_wait = g;
    dev->graphs_since_wait++;
    if (g->exec) {
        HIP_TRY(dev, hipGraphLaunch(g->exec, dev->stream));
        return CUSTOS_HIP_OK;
    }
    for (LoweredNode& ln : g->direct) {
        if (ln.kern) {
            // A large launch of a short recording is a plain launch like any other: its shape follows
            // what ran before it on this device (the rest of the recording, the replay before, whatever
            // the caller launched in between), as for a launch issued directly.
            const ResolvedShape shape = shape_of_launch(dev, ln.kern, ln.acc, &dev->recent, ln.feeds_later);
            const unsigned long long mode =
                single_launch_mode(ln.kern, ln.n, ln.head, ln.n_vec, shape, shape.alternate && (dev->launch_parity ^= 1));
            std::memcpy(ln.args[static_cast<size_t>(ln.mode_arg)].data(), &mode, 8);
            ln.grid = dim3(launch_grid(dev, ln.kern, ln.n, ln.n_vec, shape));
            ln.block = dim3(static_cast<unsigned int>(shape.block));
        } else if (ln.rev_arg >= 0 && g->flip_each_replay) {
            ln.args[ln.rev_arg][0] ^= 1;
        }
        HIP_TRY(dev, issue_node(ln, dev->stream));
    }
    return CUSTOS_HIP_OK;
}

void stop_matching(custos_hip_device* dev) {
    if (!dev->matching) return;
    dev->matching = false;
    dev->recorded.assign(dev->previous_recorded.begin(), dev->previous_recorded.begin() + static_cast<std::ptrdiff_t>(dev->matched));
}

// After a graph was built from `recorded`, or found to be the graph of the same recording:
// the recording is kept for the comparison with the next one (unless it is very long).
static void keep_recording_of(custos_hip_device* dev, custos_hip_graph* g) {
    constexpr size_t kKeepUpTo = 1u << 16;
    if (dev->recorded.size() <= kKeepUpTo) {
        dev->previous_recorded = std::move(dev->recorded);
        dev->previous_graph = g;
    } else {
        dev->previous_recorded.clear();
        dev->previous_graph = nullptr;
    }
    dev->recorded.clear();
}

void destroy_graph(custos_hip_graph* g) {
    if (g->exec) (void)hipGraphExecDestroy(g->exec);
    if (g->graph) (void)hipGraphDestroy(g->graph);
    if (g->table) (void)hipFree(g->table);
    delete g;
}

}  // namespace custos_hip

using namespace custos_hip;

extern "C" {

// ---- capture / replay ----

int32_t custos_hip_capture_begin(custos_hip_device* dev) {
    REQUIRE_DEV(dev);
    if (dev->capturing) return set_error(dev, CUSTOS_HIP_ERR_CAPTURE_STATE, "the device is already recording");
    // The recorded list starts empty.  Allocation, reads and writes stay legal while
    // recording: they execute at once, outside the compute stream's order, and are not part
    // of the graph; the first of them waits for the work that is in flight now
    // (drain_before_immediate_work).  Recording itself launches nothing, and a replay of
    // the graph is ordered on the compute stream behind that work, so beginning takes no wait.
    dev->recorded.clear();
    dev->capturing = true;
    dev->undrained_at_capture = true;
    dev->matching = dev->previous_graph != nullptr && !dev->previous_recorded.empty();
    dev->matched = 0;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_capture_end(custos_hip_device* dev, custos_hip_graph** graph) {
    REQUIRE_DEV(dev);
    if (!graph) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "graph out pointer is null");
    *graph = nullptr;
    if (!dev->capturing) return set_error(dev, CUSTOS_HIP_ERR_CAPTURE_STATE, "the device is not recording");
    dev->capturing = false;
    stop_matching(dev);
    custos_hip_graph* g = new custos_hip_graph;
    int32_t rc = build_graph(dev, g);
    if (rc != CUSTOS_HIP_OK) {
        dev->recorded.clear();
        destroy_graph(g);
        return rc;
    }
    keep_recording_of(dev, g);
    dev->graphs_built++;
    dev->graphs.push_back(g);
    *graph = g;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_capture_end_reuse(custos_hip_device* dev, custos_hip_graph* previous, custos_hip_graph** graph) {
    REQUIRE_DEV(dev);
    if (!graph) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "graph out pointer is null");
    *graph = nullptr;
    if (!dev->capturing) return set_error(dev, CUSTOS_HIP_ERR_CAPTURE_STATE, "the device is not recording");
    if (previous && std::find(dev->graphs.begin(), dev->graphs.end(), previous) == dev->graphs.end())
        return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "the previous graph does not belong to this device");
    const std::array<uint64_t, 4> settings = {dev->batching ? 1u : 0u, static_cast<uint64_t>(dev->graph_edges),
                                              dev->direct_replay_max, dev->fusing ? 1u : 0u};
    // the whole recording repeated, launch for launch, the one `previous` stands for
    if (previous && dev->matching && dev->previous_graph == previous && dev->matched == dev->previous_recorded.size() &&
        previous->built_with == settings) {
        dev->capturing = false;
        dev->matching = false;
        dev->reused_while_recording++;
        *graph = previous;
        return CUSTOS_HIP_OK;
    }
    stop_matching(dev);
    if (previous && previous->built_with == settings && previous->signature == signature(dev->recorded)) {
        dev->capturing = false;
        keep_recording_of(dev, previous);
        dev->reused_by_comparison++;
        *graph = previous;
        return CUSTOS_HIP_OK;
    }
    return custos_hip_capture_end(dev, graph);
}

int32_t custos_hip_capture_stats(custos_hip_device* dev, uint64_t* reused_while_recording, uint64_t* reused_by_comparison,
                                 uint64_t* built) {
    REQUIRE_DEV(dev);
    if (reused_while_recording) *reused_while_recording = dev->reused_while_recording;
    if (reused_by_comparison) *reused_by_comparison = dev->reused_by_comparison;
    if (built) *built = dev->graphs_built;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_set_graph_batching(custos_hip_device* dev, int32_t enabled) {
    REQUIRE_DEV(dev);
    dev->batching = enabled != 0;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_set_graph_fusing(custos_hip_device* dev, int32_t enabled) {
    REQUIRE_DEV(dev);
    if (enabled < 0) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "negative value");
    dev->fusing = enabled != 0;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_set_graph_fusing_budget(custos_hip_device* dev, uint32_t milliseconds) {
    REQUIRE_DEV(dev);
    dev->fusing_budget_ms = milliseconds;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_graph_unjoined(custos_hip_graph* graph, size_t* launches, const char** reason) {
    if (!graph || !launches) return set_error(nullptr, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "null argument");
    *launches = graph->unjoined;
    if (reason) *reason = graph->unjoined_reason.c_str();
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_set_graph_direct_replay(custos_hip_device* dev, int32_t max_nodes) {
    REQUIRE_DEV(dev);
    if (max_nodes < 0) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "max_nodes is negative");
    dev->direct_replay_max = static_cast<size_t>(max_nodes);
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_set_graph_edges(custos_hip_device* dev, int32_t mode) {
    REQUIRE_DEV(dev);
    if (mode < CUSTOS_HIP_GRAPH_EDGES_LEVEL_JOINS || mode > CUSTOS_HIP_GRAPH_EDGES_CHAIN_BY_LEVEL)
        return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "unknown graph edge mode");
    dev->graph_edges = mode;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_set_graph_verify(custos_hip_device* dev, int32_t enabled) {
    REQUIRE_DEV(dev);
    dev->graph_verify = enabled != 0;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_graph_edge_count(custos_hip_graph* graph, size_t* edges) {
    if (!graph || !edges) return CUSTOS_HIP_ERR_INVALID_ARGUMENT;
    *edges = graph->edges;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_is_capturing(custos_hip_device* dev, int32_t* capturing) {
    REQUIRE_DEV(dev);
    if (!capturing) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "capturing is null");
    *capturing = dev->capturing ? 1 : 0;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_graph_launch(custos_hip_device* dev, custos_hip_graph* graph) {
    REQUIRE_DEV(dev);
    if (!graph) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "graph is null");
    if (dev->capturing) return set_error(dev, CUSTOS_HIP_ERR_CAPTURE_STATE, "cannot replay while recording");
    return replay_graph(dev, graph);
}

int32_t custos_hip_graph_node_count(custos_hip_graph* graph, size_t* kernel_nodes) {
    if (!graph || !kernel_nodes) return set_error(nullptr, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "null argument");
    *kernel_nodes = graph->kernel_nodes;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_graph_node_kernel(custos_hip_graph* graph, size_t node, const char** name) {
    if (!graph || !name) return set_error(nullptr, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "null argument");
    if (node >= graph->node_names.size()) return set_error(nullptr, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "no such kernel node");
    *name = graph->node_names[node].c_str();
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_graph_fused_launches(custos_hip_graph* graph, size_t* launches) {
    if (!graph || !launches) return set_error(nullptr, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "null argument");
    *launches = graph->fused_away;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_graph_stats(custos_hip_graph* graph, size_t* recorded, size_t* kernel_nodes, size_t* levels) {
    if (!graph) return set_error(nullptr, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "graph is null");
    if (recorded) *recorded = graph->recorded;
    if (kernel_nodes) *kernel_nodes = graph->kernel_nodes;
    if (levels) *levels = graph->levels;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_graph_destroy(custos_hip_device* dev, custos_hip_graph* graph) {
    REQUIRE_DEV(dev);
    if (!graph) return CUSTOS_HIP_OK;
    auto it = std::find(dev->graphs.begin(), dev->graphs.end(), graph);
    if (it == dev->graphs.end()) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "graph does not belong to this device");
    dev->graphs.erase(it);
    if (dev->previous_graph == graph) {
        dev->previous_graph = nullptr;
        dev->previous_recorded.clear();
    }
    if (dev->graph_since_wait == graph) {
        dev->graph_since_wait = nullptr;
        dev->launches_since_wait = true;  // the pending work is no longer that of one known graph
    }
    HIP_TRY(dev, hipStreamSynchronize(dev->stream));
    destroy_graph(graph);
    return CUSTOS_HIP_OK;
}

}  // extern "C"
