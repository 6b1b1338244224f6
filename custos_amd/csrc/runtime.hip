// C ABI of the MI355X element-wise backend: device handle, memory, run-time
// compiled expression kernels, launches, graph capture/replay.
// Interface and reference citations: include/custos_hip.h.
#include <hip/hip_runtime.h>
#include <hip/hiprtc.h>

#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cstdio>
#include <fstream>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/custos_hip.h"
#include "expr.hpp"
#include "kernel_gen.hpp"

using namespace custos_hip;

struct custos_hip_kernel {
    KernelSpec spec;
    hipModule_t module = nullptr;
    hipFunction_t fn = nullptr;
    hipFunction_t fn_batched = nullptr;
};

struct custos_hip_graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    void* table = nullptr;    // operand address tables of the batched nodes (device memory)
    size_t kernel_nodes = 0;  // kernel nodes in the instantiated graph
    size_t recorded = 0;      // launches, clears and copies that were recorded
    size_t levels = 0;        // dependency levels
};

// One recorded piece of work (while the device is recording, nothing is launched).
struct Access {
    uint64_t begin, end;
    bool write;
};
struct RecNode {
    enum Type { Kernel, Fill, Copy, Source } type = Kernel;
    custos_hip_kernel* k = nullptr;
    std::vector<uint64_t> ptrs;  // kernel: operand addresses in parameter order; fill: {ptr}; copy: {dst, src}
    unsigned long long n = 0, head = 0, n_vec = 0, bytes = 0;
    unsigned int grid = 1;
    std::vector<Access> acc;
    int level = 0;
    // Source: launch shape and a copy of the argument values.  What such a kernel
    // reads and writes is unknown, so it orders itself against everything.
    unsigned int grid3[3] = {1, 1, 1}, block3[3] = {1, 1, 1}, shared_mem = 0;
    std::vector<std::vector<unsigned char>> arg_values;
};

struct custos_hip_device {
    int idx = 0;
    hipStream_t stream = nullptr;    // compute stream: every launch, in call order
    hipStream_t transfer = nullptr;  // copies that must not be recorded while capturing
    hipEvent_t t0 = nullptr, t1 = nullptr;
    hipDeviceProp_t props{};
    std::string arch;
    Tuning tuning;
    bool capturing = false;          // recording: launches, clears and copies go to `recorded`
    bool batching = true;            // merge equal independent launches of a level into one grid
    std::vector<RecNode> recorded;
    uint64_t compiles = 0, hits = 0, disk_hits = 0;
    std::string last_error;
    std::unordered_map<uint64_t, std::vector<std::unique_ptr<custos_hip_kernel>>> cache;
    std::vector<custos_hip_graph*> graphs;
};

namespace {

thread_local std::string g_last_error;

int32_t set_error(custos_hip_device* dev, int32_t code, const std::string& msg) {
    (dev ? dev->last_error : g_last_error) = msg;
    return code;
}

int32_t hip_fail(custos_hip_device* dev, hipError_t e, const char* what) {
    // clear the sticky "last error" of the runtime so it is not reported twice
    (void)hipGetLastError();
    return set_error(dev, static_cast<int32_t>(e),
                     std::string(what) + ": " + hipGetErrorName(e) + " (" + hipGetErrorString(e) + ")");
}

#define HIP_TRY(dev, call)                                   \
    do {                                                     \
        hipError_t e__ = (call);                             \
        if (e__ != hipSuccess) return hip_fail(dev, e__, #call); \
    } while (0)

#define REQUIRE_DEV(dev)                                                                    \
    do {                                                                                    \
        if (!(dev)) return set_error(nullptr, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "device handle is null"); \
        HIP_TRY(dev, hipSetDevice((dev)->idx));                                             \
    } while (0)

// ---- zero fill: 16-byte stores over the aligned body, bytes at the edges ----

__global__ void __launch_bounds__(256) custos_fill_zero(unsigned char* p, unsigned long long bytes,
                                                        unsigned long long head,
                                                        unsigned long long n_vec) {
    typedef unsigned int u4 __attribute__((ext_vector_type(4)));
    u4* v = reinterpret_cast<u4*>(p + head);
    const unsigned long long gid = (unsigned long long)blockIdx.x * 256 + threadIdx.x;
    const unsigned long long n_threads = (unsigned long long)gridDim.x * 256;
    const u4 z = {0u, 0u, 0u, 0u};
    for (unsigned long long i = gid; i < n_vec; i += n_threads) v[i] = z;
    if (gid < head) p[gid] = 0;
    for (unsigned long long i = head + n_vec * 16 + gid; i < bytes; i += n_threads) p[i] = 0;
}

unsigned int fill_grid(custos_hip_device* dev, unsigned long long n_vec) {
    unsigned long long want = (n_vec + 255) / 256;
    // 8 vectors per thread at most: enough workgroups to fill the chip, not one per 4 KiB
    unsigned long long cap = static_cast<unsigned long long>(dev->props.multiProcessorCount) * 64;
    unsigned long long g = std::max(1ull, std::min(want, std::max(cap, (want + 7) / 8)));
    return static_cast<unsigned int>(std::min(g, 1ull << 22));
}

int32_t launch_fill_zero(custos_hip_device* dev, uint64_t dptr, size_t bytes, hipStream_t stream) {
    unsigned long long head = (16 - (dptr & 15)) & 15;
    if (head > bytes) head = bytes;
    unsigned long long n_vec = (bytes - head) / 16;
    if (dev->capturing && stream == dev->stream) {
        RecNode node;
        node.type = RecNode::Fill;
        node.ptrs = {dptr};
        node.bytes = bytes;
        node.head = head;
        node.n_vec = n_vec;
        node.acc = {{dptr, dptr + bytes, true}};
        dev->recorded.push_back(std::move(node));
        return CUSTOS_HIP_OK;
    }
    unsigned int grid = fill_grid(dev, n_vec);
    hipLaunchKernelGGL(custos_fill_zero, dim3(grid), dim3(256), 0, stream,
                       reinterpret_cast<unsigned char*>(dptr), static_cast<unsigned long long>(bytes),
                       head, n_vec);
    HIP_TRY(dev, hipGetLastError());
    return CUSTOS_HIP_OK;
}

// ---- hiprtc ----

int32_t compile_to_code_object(custos_hip_device* dev, const KernelSpec& spec,
                               const std::string& arch, std::vector<char>* code) {
    hiprtcProgram prog = nullptr;
    hiprtcResult r = hiprtcCreateProgram(&prog, spec.source.c_str(), "custos_kernel.hip", 0, nullptr, nullptr);
    if (r != HIPRTC_SUCCESS)
        return set_error(dev, CUSTOS_HIP_ERR_COMPILE, std::string("hiprtcCreateProgram: ") + hiprtcGetErrorString(r));
    std::vector<std::string> opts = hiprtc_options(arch);
    std::vector<const char*> copts;
    for (const std::string& o : opts) copts.push_back(o.c_str());
    r = hiprtcCompileProgram(prog, static_cast<int>(copts.size()), copts.data());
    if (r != HIPRTC_SUCCESS) {
        size_t log_size = 0;
        hiprtcGetProgramLogSize(prog, &log_size);
        std::string log(log_size, '\0');
        if (log_size) hiprtcGetProgramLog(prog, &log[0]);
        hiprtcDestroyProgram(&prog);
        return set_error(dev, CUSTOS_HIP_ERR_COMPILE,
                         std::string("hiprtcCompileProgram: ") + hiprtcGetErrorString(r) + "\n" + log +
                             "\n--- source ---\n" + spec.source);
    }
    size_t size = 0;
    hiprtcGetCodeSize(prog, &size);
    code->resize(size);
    hiprtcGetCode(prog, code->data());
    hiprtcDestroyProgram(&prog);
    return CUSTOS_HIP_OK;
}

// ---- code objects on disk ----
//
// With CUSTOS_HIP_KERNEL_CACHE_DIR set, every compiled code object is stored as
// <dir>/<key>-<arch>-<hiprtc version>.co together with the source it was built
// from; a later process loads it instead of compiling when the stored source is
// identical (the 64-bit key alone is not trusted).

std::string cache_file(const KernelSpec& spec, const std::string& arch) {
    const char* dir = std::getenv("CUSTOS_HIP_KERNEL_CACHE_DIR");
    if (!dir || !*dir) return "";
    int major = 0, minor = 0;
    (void)hiprtcVersion(&major, &minor);
    std::string a = arch;
    for (char& c : a)
        if (c == ':' || c == '/' || c == '+') c = '_';
    char key[17];
    std::snprintf(key, sizeof key, "%016llx", static_cast<unsigned long long>(spec.hash));
    return std::string(dir) + "/" + key + "-" + a + "-" + std::to_string(major) + "." + std::to_string(minor) + ".co";
}

// the text hiprtc compiles: generated kernels start with a comment line that
// spells the expression as the caller wrote it; it is not part of the identity
std::string source_identity(const KernelSpec& spec) {
    if (spec.kind == Kind::Source) return spec.name + "\n" + spec.source;
    return spec.source.substr(spec.source.find('\n') + 1);
}

bool load_cached_code(const KernelSpec& spec, const std::string& arch, std::vector<char>* code) {
    const std::string path = cache_file(spec, arch);
    if (path.empty()) return false;
    std::ifstream f(path, std::ios::binary);
    if (!f) return false;
    char magic[8] = {0};
    uint64_t src_len = 0, code_len = 0;
    f.read(magic, 8);
    f.read(reinterpret_cast<char*>(&src_len), 8);
    if (!f || std::memcmp(magic, "CUSTOSC1", 8) != 0 || src_len > (1u << 26)) return false;
    std::string src(src_len, '\0');
    f.read(&src[0], static_cast<std::streamsize>(src_len));
    f.read(reinterpret_cast<char*>(&code_len), 8);
    if (!f || src != source_identity(spec) || code_len == 0 || code_len > (1u << 28)) return false;
    code->resize(code_len);
    f.read(code->data(), static_cast<std::streamsize>(code_len));
    return static_cast<bool>(f);
}

void store_cached_code(const KernelSpec& spec, const std::string& arch, const std::vector<char>& code) {
    const std::string path = cache_file(spec, arch);
    if (path.empty()) return;
    (void)mkdir(std::getenv("CUSTOS_HIP_KERNEL_CACHE_DIR"), 0777);
    const std::string tmp = path + ".tmp" + std::to_string(static_cast<long>(getpid()));
    {
        std::ofstream f(tmp, std::ios::binary | std::ios::trunc);
        if (!f) return;
        const std::string src = source_identity(spec);
        const uint64_t src_len = src.size(), code_len = code.size();
        f.write("CUSTOSC1", 8);
        f.write(reinterpret_cast<const char*>(&src_len), 8);
        f.write(src.data(), static_cast<std::streamsize>(src_len));
        f.write(reinterpret_cast<const char*>(&code_len), 8);
        f.write(code.data(), static_cast<std::streamsize>(code_len));
        if (!f) {
            std::remove(tmp.c_str());
            return;
        }
    }
    if (std::rename(tmp.c_str(), path.c_str()) != 0) std::remove(tmp.c_str());
}

bool markers_from_c(const char* const* markers, int32_t n, std::vector<std::string>* out) {
    if (!markers || n < 1 || n > 4) return false;
    for (int i = 0; i < n; i++) {
        if (!markers[i] || !markers[i][0]) return false;
        out->push_back(markers[i]);
    }
    return true;
}

int32_t spec_from_c(custos_hip_device* dev, int32_t kind, int32_t dtype, const char* src,
                    const char* const* markers, int32_t n_markers, const Tuning& tuning,
                    KernelSpec* spec) {
    if (!src) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "expression source is null");
    if (kind != CUSTOS_HIP_KIND_APPLY && kind != CUSTOS_HIP_KIND_UNARY_GRAD)
        return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "unknown kernel kind");
    if (!dtype_valid(dtype)) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "unknown element type");
    std::vector<std::string> m;
    if (!markers_from_c(markers, n_markers, &m))
        return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "1 to 4 non-empty markers are required");
    ParseError err;
    if (!build_kernel_spec(static_cast<Kind>(kind), static_cast<DType>(dtype), src, m, tuning, spec, &err))
        return set_error(dev, err.code ? err.code : CUSTOS_HIP_ERR_EXPR_SYNTAX, err.message);
    return CUSTOS_HIP_OK;
}

Tuning tuning_from_c(const custos_hip_tuning* t) {
    if (!t) return normalize_tuning(0, 0, 0, 0);
    return normalize_tuning(t->block_threads, t->unroll, t->blocks_per_cu, t->nontemporal);
}

int32_t copy_out_string(const std::string& s, char* buf, size_t cap, size_t* needed) {
    if (needed) *needed = s.size() + 1;
    if (buf && cap) {
        size_t n = std::min(cap - 1, s.size());
        std::memcpy(buf, s.data(), n);
        buf[n] = '\0';
    }
    return CUSTOS_HIP_OK;
}

struct Range {
    uint64_t ptr;
    bool written;
};

// Checks operand addresses and computes how the element range splits into a
// scalar head, 16-byte vectors and a scalar tail.
int32_t plan_launch(custos_hip_device* dev, const custos_hip_kernel* k, const std::vector<Range>& ops,
                    size_t n, unsigned long long* head, unsigned long long* n_vec, unsigned int* grid) {
    const size_t es = dtype_size(k->spec.dtype);
    if (n > (1ull << 40)) return set_error(dev, CUSTOS_HIP_ERR_TOO_LARGE, "more than 2^40 elements");
    const uint64_t bytes = static_cast<uint64_t>(n) * es;
    for (const Range& r : ops) {
        if (r.ptr == 0) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "null device pointer");
        if (r.ptr % es) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "device pointer is not aligned to the element size");
    }
    for (const Range& w : ops) {
        if (!w.written) continue;
        for (const Range& r : ops) {
            if (&r == &w || r.ptr == w.ptr) continue;
            if (r.ptr < w.ptr + bytes && w.ptr < r.ptr + bytes)
                return set_error(dev, CUSTOS_HIP_ERR_BAD_OVERLAP,
                                 "the output range partially overlaps an input range");
        }
    }
    bool same_phase = true;
    for (const Range& r : ops) same_phase = same_phase && (r.ptr & 15) == (ops[0].ptr & 15);
    unsigned long long h = 0, nv = 0;
    if (same_phase) {
        h = ((16 - (ops[0].ptr & 15)) & 15) / es;
        if (h > n) h = n;
        nv = (n - h) / k->spec.vec_elems;
    }
    const Tuning& t = k->spec.tuning;
    const unsigned long long tile_vecs = static_cast<unsigned long long>(t.block_threads) * t.unroll;
    unsigned long long tiles = (nv + tile_vecs - 1) / tile_vecs;
    unsigned long long scalar = n - nv * k->spec.vec_elems;
    const unsigned long long cus = static_cast<unsigned long long>(dev->props.multiProcessorCount);
    unsigned long long scalar_blocks = std::min((scalar + t.block_threads - 1) / t.block_threads, cus * 32);
    if (t.blocks_per_cu > 0) tiles = std::min(tiles, cus * t.blocks_per_cu);
    unsigned long long g = std::max(1ull, std::max(tiles, scalar_blocks));
    g = std::min(g, 1ull << 22);
    *head = h;
    *n_vec = nv;
    *grid = static_cast<unsigned int>(g);
    return CUSTOS_HIP_OK;
}

// Launches the kernel over one set of operands, or records the launch while
// the device is recording.  `ops` are the operand addresses in the order of the
// kernel's pointer parameters.
int32_t launch_or_record(custos_hip_device* dev, custos_hip_kernel* k, const std::vector<Range>& ops, size_t n) {
    unsigned long long head, n_vec, count = n;
    unsigned int grid;
    int32_t rc = plan_launch(dev, k, ops, n, &head, &n_vec, &grid);
    if (rc != CUSTOS_HIP_OK) return rc;
    if (dev->capturing) {
        RecNode node;
        node.type = RecNode::Kernel;
        node.k = k;
        node.n = n;
        node.head = head;
        node.n_vec = n_vec;
        node.grid = grid;
        const uint64_t bytes = static_cast<uint64_t>(n) * dtype_size(k->spec.dtype);
        for (const Range& r : ops) {
            node.ptrs.push_back(r.ptr);
            // (the gradient operand of a unary-gradient kernel is read and written;
            // a write access already orders it against every other access)
            node.acc.push_back({r.ptr, r.ptr + bytes, r.written});
        }
        dev->recorded.push_back(std::move(node));
        return CUSTOS_HIP_OK;
    }
    uint64_t ptrs[8];
    std::vector<void*> args;
    for (size_t i = 0; i < ops.size(); i++) {
        ptrs[i] = ops[i].ptr;
        args.push_back(&ptrs[i]);
    }
    args.push_back(&count);
    args.push_back(&head);
    args.push_back(&n_vec);
    HIP_TRY(dev, hipModuleLaunchKernel(k->fn, grid, 1, 1, static_cast<unsigned int>(k->spec.tuning.block_threads),
                                       1, 1, 0, dev->stream, args.data(), nullptr));
    return CUSTOS_HIP_OK;
}

// ---- building a graph from the recorded work ----
//
// The recorded list is not replayed launch by launch.  Every node gets a
// dependency level: one more than the highest level among earlier nodes whose
// memory it conflicts with (read-after-write, write-after-read or
// write-after-write on overlapping address ranges).  Nodes of one level are
// independent of each other, so they run side by side in the graph, and kernel
// launches of one level that use the same kernel over the same length are
// merged into ONE grid that walks a table of operand addresses.  1024 small
// buffers with three operations each become three kernel nodes instead of
// 3072.

constexpr uint64_t kChunkShift = 21;  // conflict search buckets of 2 MiB

void assign_levels(std::vector<RecNode>& nodes) {
    struct Seen {
        uint64_t begin, end;
        bool write;
        int level;
    };
    std::vector<Seen> seen;
    std::unordered_map<uint64_t, std::vector<uint32_t>> buckets;
    int highest = -1;  // highest level so far
    int fence = -1;    // level of the last node with unknown memory use
    for (RecNode& node : nodes) {
        int level = fence + 1;
        if (node.type == RecNode::Source) {
            // unknown reads and writes: after everything before, before everything after
            node.level = fence = highest = highest + 1;
            continue;
        }
        for (const Access& a : node.acc) {
            if (a.end <= a.begin) continue;
            for (uint64_t c = a.begin >> kChunkShift; c <= (a.end - 1) >> kChunkShift; c++) {
                auto it = buckets.find(c);
                if (it == buckets.end()) continue;
                for (uint32_t si : it->second) {
                    const Seen& s = seen[si];
                    if (s.level < level) continue;        // cannot raise the level any more
                    if (!a.write && !s.write) continue;   // two reads never conflict
                    if (a.begin < s.end && s.begin < a.end) level = s.level + 1;
                }
            }
        }
        node.level = level;
        highest = std::max(highest, level);
        for (const Access& a : node.acc) {
            if (a.end <= a.begin) continue;
            const uint32_t idx = static_cast<uint32_t>(seen.size());
            seen.push_back({a.begin, a.end, a.write, level});
            for (uint64_t c = a.begin >> kChunkShift; c <= (a.end - 1) >> kChunkShift; c++) buckets[c].push_back(idx);
        }
    }
}

bool batchable(const RecNode& n) {
    if (n.type != RecNode::Kernel || n.head != 0 || !n.k->fn_batched) return false;
    for (uint64_t p : n.ptrs)
        if (p & 15) return false;
    return true;
}

int32_t build_graph(custos_hip_device* dev, custos_hip_graph* g) {
    std::vector<RecNode>& nodes = dev->recorded;
    assign_levels(nodes);
    int max_level = -1;
    for (const RecNode& n : nodes) max_level = std::max(max_level, n.level);
    g->recorded = nodes.size();
    g->levels = static_cast<size_t>(max_level + 1);

    // plan: per level, either single nodes or batches of node indices
    struct Planned {
        std::vector<size_t> members;  // indices into `nodes`; more than one = batched launch
        size_t table_offset = 0;      // in u64 entries
    };
    std::vector<std::vector<Planned>> plan(static_cast<size_t>(max_level + 1));
    std::vector<uint64_t> host_table;
    for (int level = 0; level <= max_level; level++) {
        std::vector<Planned>& out = plan[level];
        // batches keyed by (kernel, n), in first-seen order
        std::vector<std::pair<std::pair<custos_hip_kernel*, unsigned long long>, size_t>> keys;
        for (size_t i = 0; i < nodes.size(); i++) {
            if (nodes[i].level != level) continue;
            if (dev->batching && batchable(nodes[i])) {
                const auto key = std::make_pair(nodes[i].k, nodes[i].n);
                size_t slot = out.size();
                for (const auto& kv : keys)
                    if (kv.first == key) slot = kv.second;
                if (slot == out.size()) {
                    keys.push_back({key, slot});
                    out.emplace_back();
                }
                out[slot].members.push_back(i);
            } else {
                out.emplace_back();
                out.back().members.push_back(i);
            }
        }
        for (Planned& p : out) {
            if (p.members.size() < 2) continue;
            p.table_offset = host_table.size();
            for (size_t i : p.members)
                for (uint64_t ptr : nodes[i].ptrs) host_table.push_back(ptr);
        }
    }
    if (!host_table.empty()) {
        HIP_TRY(dev, hipMalloc(&g->table, host_table.size() * sizeof(uint64_t)));
        HIP_TRY(dev, hipMemcpy(g->table, host_table.data(), host_table.size() * sizeof(uint64_t), hipMemcpyHostToDevice));
    }

    HIP_TRY(dev, hipGraphCreate(&g->graph, 0));
    std::vector<hipGraphNode_t> prev;  // what the nodes of the current level wait for
    for (int level = 0; level <= max_level; level++) {
        std::vector<hipGraphNode_t> deps = prev;
        if (deps.size() > 1) {  // one join node instead of |prev| x |level| edges
            hipGraphNode_t join;
            HIP_TRY(dev, hipGraphAddEmptyNode(&join, g->graph, deps.data(), deps.size()));
            deps = {join};
        }
        std::vector<hipGraphNode_t> made;
        for (const Planned& p : plan[level]) {
            const RecNode& first = nodes[p.members[0]];
            hipGraphNode_t node;
            if (first.type == RecNode::Copy) {
                HIP_TRY(dev, hipGraphAddMemcpyNode1D(&node, g->graph, deps.data(), deps.size(),
                                                     reinterpret_cast<void*>(first.ptrs[0]),
                                                     reinterpret_cast<const void*>(first.ptrs[1]), first.bytes,
                                                     hipMemcpyDeviceToDevice));
                made.push_back(node);
                continue;
            }
            hipKernelNodeParams kp{};
            kp.sharedMemBytes = 0;
            kp.extra = nullptr;
            std::vector<void*> args;
            uint64_t ptrs[8];
            unsigned long long a0, a1, a2, a3;
            if (first.type == RecNode::Source) {
                for (const auto& v : first.arg_values) args.push_back(const_cast<unsigned char*>(v.data()));
                kp.func = reinterpret_cast<void*>(first.k->fn);
                kp.gridDim = dim3(first.grid3[0], first.grid3[1], first.grid3[2]);
                kp.blockDim = dim3(first.block3[0], first.block3[1], first.block3[2]);
                kp.sharedMemBytes = first.shared_mem;
            } else if (first.type == RecNode::Fill) {
                ptrs[0] = first.ptrs[0];
                a0 = first.bytes, a1 = first.head, a2 = first.n_vec;
                args = {&ptrs[0], &a0, &a1, &a2};
                kp.func = reinterpret_cast<void*>(custos_fill_zero);
                kp.gridDim = dim3(fill_grid(dev, first.n_vec));
                kp.blockDim = dim3(256);
            } else if (p.members.size() == 1) {
                for (size_t i = 0; i < first.ptrs.size(); i++) {
                    ptrs[i] = first.ptrs[i];
                    args.push_back(&ptrs[i]);
                }
                a0 = first.n, a1 = first.head, a2 = first.n_vec;
                args.push_back(&a0);
                args.push_back(&a1);
                args.push_back(&a2);
                kp.func = reinterpret_cast<void*>(first.k->fn);
                kp.gridDim = dim3(first.grid);
                kp.blockDim = dim3(static_cast<unsigned int>(first.k->spec.tuning.block_threads));
            } else {
                const Tuning& t = first.k->spec.tuning;
                const unsigned long long tile_vecs = static_cast<unsigned long long>(t.block_threads) * t.unroll;
                a3 = std::max(1ull, (first.n_vec + tile_vecs - 1) / tile_vecs);  // tiles per segment
                const unsigned long long blocks = a3 * p.members.size();
                if (blocks > (1ull << 31) - 1)
                    return set_error(dev, CUSTOS_HIP_ERR_TOO_LARGE, "a batched launch would need more than 2^31 workgroups");
                ptrs[0] = reinterpret_cast<uint64_t>(g->table) + p.table_offset * sizeof(uint64_t);
                a0 = first.n, a1 = first.n_vec;
                args = {&ptrs[0], &a0, &a1, &a3};
                kp.func = reinterpret_cast<void*>(first.k->fn_batched);
                kp.gridDim = dim3(static_cast<unsigned int>(blocks));
                kp.blockDim = dim3(static_cast<unsigned int>(t.block_threads));
            }
            kp.kernelParams = args.data();
            HIP_TRY(dev, hipGraphAddKernelNode(&node, g->graph, deps.data(), deps.size(), &kp));
            g->kernel_nodes++;
            made.push_back(node);
        }
        prev = std::move(made);
    }
    HIP_TRY(dev, hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0));
    return CUSTOS_HIP_OK;
}

// Code object from the disk cache or from hiprtc, loaded as a module; entry point looked up.
int32_t build_module(custos_hip_device* dev, custos_hip_kernel* k) {
    std::vector<char> code;
    bool from_disk = load_cached_code(k->spec, dev->arch, &code);
    if (from_disk && hipModuleLoadData(&k->module, code.data()) != hipSuccess) {
        (void)hipGetLastError();  // a stale or damaged file: compile instead
        k->module = nullptr;
        from_disk = false;
    }
    if (!from_disk) {
        int32_t rc = compile_to_code_object(dev, k->spec, dev->arch, &code);
        if (rc != CUSTOS_HIP_OK) return rc;
        HIP_TRY(dev, hipModuleLoadData(&k->module, code.data()));
        store_cached_code(k->spec, dev->arch, code);
        dev->compiles++;
    } else {
        dev->disk_hits++;
    }
    hipError_t e = hipModuleGetFunction(&k->fn, k->module, k->spec.name.c_str());
    if (e != hipSuccess) {
        (void)hipModuleUnload(k->module);
        k->module = nullptr;
        return hip_fail(dev, e, "hipModuleGetFunction");
    }
    return CUSTOS_HIP_OK;
}

void destroy_graph(custos_hip_graph* g) {
    if (g->exec) (void)hipGraphExecDestroy(g->exec);
    if (g->graph) (void)hipGraphDestroy(g->graph);
    if (g->table) (void)hipFree(g->table);
    delete g;
}

}  // namespace

extern "C" {

int32_t custos_hip_device_count(int32_t* count) {
    if (!count) return set_error(nullptr, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "count is null");
    int c = 0;
    hipError_t e = hipGetDeviceCount(&c);
    if (e != hipSuccess) {
        *count = 0;
        return hip_fail(nullptr, e, "hipGetDeviceCount");
    }
    *count = c;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_chosen_device_idx(void) {
    const char* v = std::getenv("CUSTOS_HIP_DEVICE_IDX");
    if (!v || !*v) return 0;
    char* end = nullptr;
    long idx = std::strtol(v, &end, 10);
    if (*end != '\0' || idx < 0) return 0;
    return static_cast<int32_t>(idx);
}

int32_t custos_hip_device_create(int32_t idx, custos_hip_device** out) {
    if (!out) return set_error(nullptr, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "out handle is null");
    *out = nullptr;
    int count = 0;
    HIP_TRY(nullptr, hipGetDeviceCount(&count));
    if (idx < 0 || idx >= count)
        return set_error(nullptr, CUSTOS_HIP_ERR_INVALID_DEVICE_INDEX,
                         "device index " + std::to_string(idx) + " out of range: " + std::to_string(count) + " device(s)");
    std::unique_ptr<custos_hip_device> dev(new custos_hip_device);
    dev->idx = idx;
    HIP_TRY(nullptr, hipSetDevice(idx));
    HIP_TRY(nullptr, hipGetDeviceProperties(&dev->props, idx));
    dev->arch = dev->props.gcnArchName;
    dev->tuning = normalize_tuning(0, 0, 0, 0);
    HIP_TRY(nullptr, hipStreamCreateWithFlags(&dev->stream, hipStreamNonBlocking));
    HIP_TRY(nullptr, hipStreamCreateWithFlags(&dev->transfer, hipStreamNonBlocking));
    HIP_TRY(nullptr, hipEventCreate(&dev->t0));
    HIP_TRY(nullptr, hipEventCreate(&dev->t1));
    *out = dev.release();
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_device_destroy(custos_hip_device* dev) {
    if (!dev) return CUSTOS_HIP_OK;
    (void)hipSetDevice(dev->idx);
    (void)hipStreamSynchronize(dev->stream);
    (void)hipStreamSynchronize(dev->transfer);
    for (custos_hip_graph* g : dev->graphs) destroy_graph(g);
    for (auto& bucket : dev->cache)
        for (auto& k : bucket.second)
            if (k->module) (void)hipModuleUnload(k->module);
    (void)hipEventDestroy(dev->t0);
    (void)hipEventDestroy(dev->t1);
    (void)hipStreamDestroy(dev->stream);
    (void)hipStreamDestroy(dev->transfer);
    delete dev;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_get_device_info(custos_hip_device* dev, custos_hip_device_info* info) {
    REQUIRE_DEV(dev);
    if (!info) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "info is null");
    std::memset(info, 0, sizeof *info);
    std::snprintf(info->name, sizeof info->name, "%s", dev->props.name);
    std::snprintf(info->arch, sizeof info->arch, "%s", dev->props.gcnArchName);
    info->compute_units = dev->props.multiProcessorCount;
    info->wavefront_size = dev->props.warpSize;
    info->clock_khz = dev->props.clockRate;
    info->memory_clock_khz = dev->props.memoryClockRate;
    info->memory_bus_bits = dev->props.memoryBusWidth;
    info->l2_bytes = dev->props.l2CacheSize;
    info->total_memory = dev->props.totalGlobalMem;
    return CUSTOS_HIP_OK;
}

const char* custos_hip_last_error(custos_hip_device* dev) {
    return dev ? dev->last_error.c_str() : g_last_error.c_str();
}

int32_t custos_hip_sync(custos_hip_device* dev) {
    REQUIRE_DEV(dev);
    if (dev->capturing)
        return set_error(dev, CUSTOS_HIP_ERR_CAPTURE_STATE, "cannot wait for a stream that is recording");
    HIP_TRY(dev, hipStreamSynchronize(dev->stream));
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_set_tuning(custos_hip_device* dev, const custos_hip_tuning* tuning) {
    REQUIRE_DEV(dev);
    dev->tuning = tuning_from_c(tuning);
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_get_tuning(custos_hip_device* dev, custos_hip_tuning* tuning) {
    REQUIRE_DEV(dev);
    if (!tuning) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "tuning is null");
    tuning->block_threads = dev->tuning.block_threads;
    tuning->unroll = dev->tuning.unroll;
    tuning->blocks_per_cu = dev->tuning.blocks_per_cu;
    tuning->nontemporal = dev->tuning.nontemporal;
    return CUSTOS_HIP_OK;
}

// ---- memory ----

int32_t custos_hip_alloc(custos_hip_device* dev, size_t bytes, int32_t flags, uint64_t* dptr) {
    REQUIRE_DEV(dev);
    if (!dptr) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "dptr is null");
    *dptr = 0;
    if (bytes == 0) return set_error(dev, CUSTOS_HIP_ERR_ZERO_LENGTH_BUFFER, "zero length buffers are not supported");
    void* p = nullptr;
    HIP_TRY(dev, hipMalloc(&p, bytes));
    uint64_t addr = reinterpret_cast<uint64_t>(p);
    if (flags != CUSTOS_HIP_ALLOC_UNINIT) {
        // While recording, the fill must run now and not become part of the graph.
        hipStream_t s = dev->capturing ? dev->transfer : dev->stream;
        int32_t rc = launch_fill_zero(dev, addr, bytes, s);
        if (rc == CUSTOS_HIP_OK && dev->capturing) {
            hipError_t e = hipStreamSynchronize(dev->transfer);
            if (e != hipSuccess) rc = hip_fail(dev, e, "hipStreamSynchronize(transfer)");
        }
        if (rc != CUSTOS_HIP_OK) {
            (void)hipFree(p);
            return rc;
        }
    }
    *dptr = addr;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_free(custos_hip_device* dev, uint64_t dptr) {
    REQUIRE_DEV(dev);
    if (dptr == 0) return CUSTOS_HIP_OK;
    // work that still uses the range must finish first
    if (!dev->capturing) HIP_TRY(dev, hipStreamSynchronize(dev->stream));
    HIP_TRY(dev, hipFree(reinterpret_cast<void*>(dptr)));
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_write(custos_hip_device* dev, uint64_t dst, const void* src, size_t bytes) {
    REQUIRE_DEV(dev);
    if (bytes == 0) return CUSTOS_HIP_OK;
    if (!dst || !src) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "null pointer");
    if (dev->capturing) {
        HIP_TRY(dev, hipMemcpyAsync(reinterpret_cast<void*>(dst), src, bytes, hipMemcpyHostToDevice, dev->transfer));
        HIP_TRY(dev, hipStreamSynchronize(dev->transfer));
        return CUSTOS_HIP_OK;
    }
    HIP_TRY(dev, hipMemcpyAsync(reinterpret_cast<void*>(dst), src, bytes, hipMemcpyHostToDevice, dev->stream));
    // the caller may reuse `src` right away
    HIP_TRY(dev, hipStreamSynchronize(dev->stream));
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_read(custos_hip_device* dev, void* dst, uint64_t src, size_t bytes) {
    REQUIRE_DEV(dev);
    if (bytes == 0) return CUSTOS_HIP_OK;
    if (!dst || !src) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "null pointer");
    if (!dev->capturing) HIP_TRY(dev, hipStreamSynchronize(dev->stream));
    HIP_TRY(dev, hipMemcpyAsync(dst, reinterpret_cast<const void*>(src), bytes, hipMemcpyDeviceToHost, dev->transfer));
    HIP_TRY(dev, hipStreamSynchronize(dev->transfer));
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_copy(custos_hip_device* dev, uint64_t dst, uint64_t src, size_t bytes) {
    REQUIRE_DEV(dev);
    if (bytes == 0) return CUSTOS_HIP_OK;
    if (!dst || !src) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "null pointer");
    if (dev->capturing) {
        RecNode node;
        node.type = RecNode::Copy;
        node.ptrs = {dst, src};
        node.bytes = bytes;
        node.acc = {{dst, dst + bytes, true}, {src, src + bytes, false}};
        dev->recorded.push_back(std::move(node));
        return CUSTOS_HIP_OK;
    }
    HIP_TRY(dev, hipMemcpyAsync(reinterpret_cast<void*>(dst), reinterpret_cast<const void*>(src), bytes,
                                hipMemcpyDeviceToDevice, dev->stream));
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_clear(custos_hip_device* dev, uint64_t dptr, size_t bytes) {
    REQUIRE_DEV(dev);
    if (bytes == 0) return CUSTOS_HIP_OK;
    if (!dptr) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "null pointer");
    return launch_fill_zero(dev, dptr, bytes, dev->stream);
}

// ---- expression kernels ----

int32_t custos_hip_expr_compile(custos_hip_device* dev, int32_t kind, int32_t dtype, const char* src,
                                const char* const* markers, int32_t n_markers,
                                custos_hip_kernel** kernel) {
    REQUIRE_DEV(dev);
    if (!kernel) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "kernel out pointer is null");
    *kernel = nullptr;
    std::unique_ptr<custos_hip_kernel> k(new custos_hip_kernel);
    int32_t rc = spec_from_c(dev, kind, dtype, src, markers, n_markers, dev->tuning, &k->spec);
    if (rc != CUSTOS_HIP_OK) return rc;

    auto& bucket = dev->cache[k->spec.hash];
    for (auto& cached : bucket) {
        // the generated text starts with the caller's spelling of the expression
        // as a comment; compare what is compiled, i.e. everything after it
        const std::string& a = cached->spec.source;
        const std::string& b = k->spec.source;
        if (a.compare(a.find('\n'), std::string::npos, b, b.find('\n'), std::string::npos) == 0) {
            dev->hits++;
            *kernel = cached.get();
            return CUSTOS_HIP_OK;
        }
    }
    rc = build_module(dev, k.get());
    if (rc != CUSTOS_HIP_OK) return rc;
    // the second entry point of the module: many equal launches in one grid
    if (hipModuleGetFunction(&k->fn_batched, k->module, (k->spec.name + "_batched").c_str()) != hipSuccess) {
        (void)hipGetLastError();
        k->fn_batched = nullptr;
    }
    *kernel = k.get();
    bucket.push_back(std::move(k));
    return CUSTOS_HIP_OK;
}

// ---- caller-written kernels (src/devices/cuda/kernel_cache.rs:39-61, kernel_launch.rs:81-163) ----

int32_t custos_hip_source_compile(custos_hip_device* dev, const char* src, const char* fn_name,
                                  custos_hip_kernel** kernel) {
    REQUIRE_DEV(dev);
    if (!kernel) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "kernel out pointer is null");
    *kernel = nullptr;
    if (!src || !fn_name || !*fn_name) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "source or function name is null");
    std::unique_ptr<custos_hip_kernel> k(new custos_hip_kernel);
    k->spec.kind = Kind::Source;
    k->spec.name = fn_name;
    k->spec.source = src;
    k->spec.hash = fnv1a64(fn_name, std::strlen(fn_name), fnv1a64(src, std::strlen(src), fnv1a64("custos-source-v1", 16)));
    auto& bucket = dev->cache[k->spec.hash];
    for (auto& cached : bucket) {
        if (cached->spec.kind == Kind::Source && cached->spec.name == k->spec.name && cached->spec.source == k->spec.source) {
            dev->hits++;
            *kernel = cached.get();
            return CUSTOS_HIP_OK;
        }
    }
    int32_t rc = build_module(dev, k.get());
    if (rc != CUSTOS_HIP_OK) return rc;
    *kernel = k.get();
    bucket.push_back(std::move(k));
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_source_launch(custos_hip_device* dev, custos_hip_kernel* kernel, const uint32_t* grid,
                                 const uint32_t* block, uint32_t shared_mem_bytes, void* const* params,
                                 const size_t* param_sizes, int32_t n_params) {
    REQUIRE_DEV(dev);
    if (!kernel || !grid || !block || n_params < 0 || (n_params > 0 && (!params || !param_sizes)))
        return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "null argument");
    if (kernel->spec.kind != Kind::Source)
        return set_error(dev, CUSTOS_HIP_ERR_KIND_MISMATCH, "kernel was not compiled from caller-written source");
    for (int i = 0; i < 3; i++)
        if (grid[i] == 0 || block[i] == 0) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "grid and block dimensions must be positive");
    if (static_cast<uint64_t>(block[0]) * block[1] * block[2] > 1024)
        return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "more than 1024 threads per workgroup");
    if (dev->capturing) {
        RecNode node;
        node.type = RecNode::Source;
        node.k = kernel;
        for (int i = 0; i < 3; i++) node.grid3[i] = grid[i], node.block3[i] = block[i];
        node.shared_mem = shared_mem_bytes;
        for (int i = 0; i < n_params; i++) {
            const unsigned char* p = static_cast<const unsigned char*>(params[i]);
            node.arg_values.emplace_back(p, p + param_sizes[i]);
        }
        dev->recorded.push_back(std::move(node));
        return CUSTOS_HIP_OK;
    }
    std::vector<void*> args(params, params + n_params);
    HIP_TRY(dev, hipModuleLaunchKernel(kernel->fn, grid[0], grid[1], grid[2], block[0], block[1], block[2],
                                       shared_mem_bytes, dev->stream, args.data(), nullptr));
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_source_launch1d(custos_hip_device* dev, custos_hip_kernel* kernel, size_t len,
                                   void* const* params, const size_t* param_sizes, int32_t n_params) {
    REQUIRE_DEV(dev);
    if (!kernel) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "null kernel");
    if (kernel->spec.kind != Kind::Source)
        return set_error(dev, CUSTOS_HIP_ERR_KIND_MISMATCH, "kernel was not compiled from caller-written source");
    if (len == 0) return CUSTOS_HIP_OK;
    // block size from the occupancy calculator, grid = ceil(len / block) (kernel_launch.rs:141-151)
    int min_grid = 0, block_size = 0;
    HIP_TRY(dev, hipModuleOccupancyMaxPotentialBlockSize(&min_grid, &block_size, kernel->fn, 0, 0));
    if (block_size <= 0) block_size = 256;
    const uint64_t blocks = (len + static_cast<size_t>(block_size) - 1) / static_cast<size_t>(block_size);
    if (blocks > 0x7fffffffull) return set_error(dev, CUSTOS_HIP_ERR_TOO_LARGE, "more workgroups than a one-dimensional grid holds");
    const uint32_t grid[3] = {static_cast<uint32_t>(blocks), 1, 1};
    const uint32_t block[3] = {static_cast<uint32_t>(block_size), 1, 1};
    return custos_hip_source_launch(dev, kernel, grid, block, 0, params, param_sizes, n_params);
}

const char* custos_hip_kernel_source(const custos_hip_kernel* kernel) {
    return kernel ? kernel->spec.source.c_str() : "";
}

const char* custos_hip_kernel_name(const custos_hip_kernel* kernel) {
    return kernel ? kernel->spec.name.c_str() : "";
}

uint64_t custos_hip_kernel_hash(const custos_hip_kernel* kernel) { return kernel ? kernel->spec.hash : 0; }

int32_t custos_hip_kernel_arity(const custos_hip_kernel* kernel) {
    return kernel ? kernel->spec.expr.n_vars : 0;
}

int32_t custos_hip_cache_stats(custos_hip_device* dev, uint64_t* compiles, uint64_t* hits) {
    REQUIRE_DEV(dev);
    if (compiles) *compiles = dev->compiles;
    if (hits) *hits = dev->hits;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_cache_disk_hits(custos_hip_device* dev, uint64_t* disk_hits) {
    REQUIRE_DEV(dev);
    if (disk_hits) *disk_hits = dev->disk_hits;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_expr_emit(int32_t kind, int32_t dtype, const char* src, const char* const* markers,
                             int32_t n_markers, const custos_hip_tuning* tuning, char* buf, size_t cap,
                             size_t* needed, uint64_t* hash) {
    KernelSpec spec;
    int32_t rc = spec_from_c(nullptr, kind, dtype, src, markers, n_markers, tuning_from_c(tuning), &spec);
    if (rc != CUSTOS_HIP_OK) return rc;
    if (hash) *hash = spec.hash;
    return copy_out_string(spec.source, buf, cap, needed);
}

int32_t custos_hip_expr_build_code_object(int32_t kind, int32_t dtype, const char* src,
                                          const char* const* markers, int32_t n_markers,
                                          const custos_hip_tuning* tuning, size_t* code_size) {
    KernelSpec spec;
    int32_t rc = spec_from_c(nullptr, kind, dtype, src, markers, n_markers, tuning_from_c(tuning), &spec);
    if (rc != CUSTOS_HIP_OK) return rc;
    std::vector<char> code;
    rc = compile_to_code_object(nullptr, spec, "gfx950", &code);
    if (rc != CUSTOS_HIP_OK) return rc;
    if (code_size) *code_size = code.size();
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_expr_canonical(const char* src, const char* const* markers, int32_t n_markers,
                                  char* buf, size_t cap, size_t* needed) {
    if (!src) return set_error(nullptr, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "expression source is null");
    std::vector<std::string> m;
    if (!markers_from_c(markers, n_markers, &m))
        return set_error(nullptr, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "1 to 4 non-empty markers are required");
    Expr e;
    ParseError err;
    if (!parse_expr(src, m, &e, &err)) return set_error(nullptr, err.code, err.message);
    return copy_out_string(to_cl_source(e, m), buf, cap, needed);
}

// ---- launches ----

int32_t custos_hip_apply_fn_n(custos_hip_device* dev, custos_hip_kernel* kernel, const uint64_t* ins,
                              int32_t n_ins, uint64_t out, size_t n) {
    REQUIRE_DEV(dev);
    if (!kernel || !ins) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "null kernel or operand list");
    if (kernel->spec.kind != Kind::Apply)
        return set_error(dev, CUSTOS_HIP_ERR_KIND_MISMATCH, "kernel was not compiled as an apply kernel");
    if (n_ins != kernel->spec.expr.n_vars)
        return set_error(dev, CUSTOS_HIP_ERR_ARITY_MISMATCH,
                         "kernel takes " + std::to_string(kernel->spec.expr.n_vars) + " operand(s), got " + std::to_string(n_ins));
    if (n == 0) return CUSTOS_HIP_OK;
    std::vector<Range> ops;
    for (int i = 0; i < n_ins; i++) ops.push_back({ins[i], false});
    ops.push_back({out, true});
    return launch_or_record(dev, kernel, ops, n);
}

int32_t custos_hip_apply_fn(custos_hip_device* dev, custos_hip_kernel* kernel, uint64_t x, uint64_t out, size_t n) {
    return custos_hip_apply_fn_n(dev, kernel, &x, 1, out, n);
}

int32_t custos_hip_apply_fn2(custos_hip_device* dev, custos_hip_kernel* kernel, uint64_t lhs, uint64_t rhs,
                             uint64_t out, size_t n) {
    uint64_t ins[2] = {lhs, rhs};
    return custos_hip_apply_fn_n(dev, kernel, ins, 2, out, n);
}

int32_t custos_hip_add_unary_grad(custos_hip_device* dev, custos_hip_kernel* kernel, uint64_t lhs,
                                  uint64_t lhs_grad, uint64_t out_grad, size_t n) {
    REQUIRE_DEV(dev);
    if (!kernel) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "null kernel");
    if (kernel->spec.kind != Kind::UnaryGrad)
        return set_error(dev, CUSTOS_HIP_ERR_KIND_MISMATCH, "kernel was not compiled as a unary-gradient kernel");
    if (n == 0) return CUSTOS_HIP_OK;
    std::vector<Range> ops = {{lhs, false}, {lhs_grad, true}, {out_grad, false}};
    return launch_or_record(dev, kernel, ops, n);
}

// ---- capture / replay ----

int32_t custos_hip_capture_begin(custos_hip_device* dev) {
    REQUIRE_DEV(dev);
    if (dev->capturing) return set_error(dev, CUSTOS_HIP_ERR_CAPTURE_STATE, "the device is already recording");
    // Earlier eager work must be complete before anything recorded can run, and
    // the recorded list starts empty.  Allocation, reads and writes stay legal
    // while recording: they execute at once and are not part of the graph.
    HIP_TRY(dev, hipStreamSynchronize(dev->stream));
    dev->recorded.clear();
    dev->capturing = true;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_capture_end(custos_hip_device* dev, custos_hip_graph** graph) {
    REQUIRE_DEV(dev);
    if (!graph) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "graph out pointer is null");
    *graph = nullptr;
    if (!dev->capturing) return set_error(dev, CUSTOS_HIP_ERR_CAPTURE_STATE, "the device is not recording");
    dev->capturing = false;
    custos_hip_graph* g = new custos_hip_graph;
    int32_t rc = build_graph(dev, g);
    dev->recorded.clear();
    if (rc != CUSTOS_HIP_OK) {
        destroy_graph(g);
        return rc;
    }
    dev->graphs.push_back(g);
    *graph = g;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_set_graph_batching(custos_hip_device* dev, int32_t enabled) {
    REQUIRE_DEV(dev);
    dev->batching = enabled != 0;
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
    HIP_TRY(dev, hipGraphLaunch(graph->exec, dev->stream));
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_graph_node_count(custos_hip_graph* graph, size_t* kernel_nodes) {
    if (!graph || !kernel_nodes) return set_error(nullptr, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "null argument");
    *kernel_nodes = graph->kernel_nodes;
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
    HIP_TRY(dev, hipStreamSynchronize(dev->stream));
    destroy_graph(graph);
    return CUSTOS_HIP_OK;
}

// ---- timing ----

int32_t custos_hip_timer_begin(custos_hip_device* dev) {
    REQUIRE_DEV(dev);
    if (dev->capturing) return set_error(dev, CUSTOS_HIP_ERR_CAPTURE_STATE, "cannot time a recording stream");
    HIP_TRY(dev, hipEventRecord(dev->t0, dev->stream));
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_timer_end(custos_hip_device* dev, double* ms) {
    REQUIRE_DEV(dev);
    if (!ms) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "ms is null");
    if (dev->capturing) return set_error(dev, CUSTOS_HIP_ERR_CAPTURE_STATE, "cannot time a recording stream");
    HIP_TRY(dev, hipEventRecord(dev->t1, dev->stream));
    HIP_TRY(dev, hipEventSynchronize(dev->t1));
    float f = 0.f;
    HIP_TRY(dev, hipEventElapsedTime(&f, dev->t0, dev->t1));
    *ms = f;
    return CUSTOS_HIP_OK;
}

}  // extern "C"
