// Internal declarations shared by the translation units of libcustos_hip.so:
// the handle types behind the C ABI, error helpers, and the functions that
// cross file boundaries.  Interface and reference citations: include/custos_hip.h.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hiprtc.h>

#include <array>
#include <cstdint>
#include <map>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/custos_hip.h"
#include "expr.hpp"
#include "kernel_gen.hpp"

struct custos_hip_kernel {
    custos_hip::KernelSpec spec;
    // One module and entry point per EntrySet (single launch; equal launches in one grid;
    // launches of different lengths in one grid), each compiled and loaded when it is first
    // needed (custos_hip::entry_point).  Only the kernel that owns the code loads modules; a
    // caller-written kernel has the first one only.
    hipModule_t modules[custos_hip::kEntrySets] = {nullptr, nullptr, nullptr};
    hipFunction_t fns[custos_hip::kEntrySets] = {nullptr, nullptr, nullptr};
    std::string expr_src;  // the expression as the caller spelt it
    // the request custos_hip_expr_compile answered with this handle last (kind, dtype, and the device's
    // compile settings then, by their epoch): a recording that repeats the one before asks again
    int32_t request_kind = -1, request_dtype = -1;
    uint64_t request_epoch = ~0ull;
    std::vector<std::string> markers;
    // Handles for the same code with other values of the literal parameters, by those
    // values: they share this kernel's modules (their own stay null) and differ
    // in `spec.consts.bytes`, `spec.expr` and `expr_src`.  `code` points at the kernel that
    // owns the module (itself for the owner).
    std::map<std::string, std::unique_ptr<custos_hip_kernel>> siblings;
    custos_hip_kernel* code = nullptr;
};

// An address range an operand of a launch covers, and whether the launch writes it.
struct Access {
    uint64_t begin, end;
    bool write;
};

// A graph node in launchable form: function, shape and a copy of the argument values.
struct LoweredNode {
    bool is_copy = false;
    uint64_t dst = 0, src = 0;  // copy
    size_t bytes = 0;
    void* func = nullptr;       // kernel: hipFunction_t of a module, or the host handle of a library kernel
    bool module_fn = true;
    dim3 grid{1, 1, 1}, block{1, 1, 1};
    unsigned int shared_mem = 0;
    std::vector<std::vector<unsigned char>> args;
    int rev_arg = -1;  // index of the mode word (bit 0 = direction) of a node that alternates, else -1
    int mode_arg = -1;  // index of the mode word of a generated kernel
    // A single launch of more than kTrafficBeyondBytes, for a replay as plain launches, which chooses
    // the launch shape like a launch issued directly (`kern` is null for every other node):
    custos_hip_kernel* kern = nullptr;
    unsigned long long n = 0, head = 0, n_vec = 0;
    std::vector<Access> acc;
    bool feeds_later = false;
};

struct custos_hip_graph {
    // A short chain (every level one node, at most direct_replay_max nodes) is
    // replayed by issuing its nodes on the compute stream: stream order is exactly
    // its dependency order, and a handful of launches cost less than a graph launch.
    // Everything else is an instantiated hipGraph.
    std::vector<LoweredNode> direct;
    bool flip_each_replay = false;  // direct replay: alternating nodes change direction every replay
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    void* table = nullptr;    // operand address tables of the batched nodes (device memory)
    size_t kernel_nodes = 0;  // kernel nodes in the instantiated graph
    size_t recorded = 0;      // launches, clears and copies that were recorded
    size_t levels = 0;        // dependency levels
    size_t edges = 0;         // dependency edges of the instantiated graph (joins included)
    // what the graph was built from: the recording, word by word, and the device's graph settings
    // (merging, edge mode, direct replay limit) -- see custos_hip_capture_end_reuse
    std::vector<uint64_t> signature;
    std::array<uint64_t, 4> built_with{};
    size_t fused_away = 0;    // recorded launches that became stages of a later launch's kernel
    size_t unjoined = 0;      // recorded launches that would have been joined, had the build got their kernel
    std::string unjoined_reason;  // why not: the time budget, or the compiler's message
    std::vector<std::string> node_names;  // entry point of every kernel node, in the order of the chain / the levels
    // how long the last wait took that waited for one launch of this graph and nothing else
    uint64_t last_wait_ns = 0;
};

// One recorded piece of work (while the device is recording, nothing is launched).
struct RecNode {
    enum Type { Kernel, Fill, Copy, Source } type = Kernel;
    custos_hip_kernel* k = nullptr;
    std::vector<uint64_t> ptrs;  // kernel: operand addresses in parameter order; fill: {ptr}; copy: {dst, src}
    unsigned long long n = 0, head = 0, n_vec = 0, bytes = 0;
    std::vector<uint32_t> pattern;  // fill: the 16 bytes that repeat; empty = zeros
    std::vector<unsigned char> const_bytes;  // chain kernel: this launch's values of the literal parameters
                                             // (every other generated kernel carries them in its handle)
    std::vector<Access> acc;
    int level = 0;
    std::vector<uint32_t> deps;  // recorded nodes this one has to follow (filled when a graph is built with per-node edges)
    // Source: launch shape and a copy of the argument values.  What such a kernel
    // reads and writes is unknown, so it orders itself against everything.
    unsigned int grid3[3] = {1, 1, 1}, block3[3] = {1, 1, 1}, shared_mem = 0;
    std::vector<std::vector<unsigned char>> arg_values;
};

// The address ranges of the last few launches, from which a launch learns whether it reads
// what one of them wrote and how much was touched since (see CacheHint).
// Launches up to kTrafficBeyondBytes are not tracked (their kernels are shorter than a launch
// call, and they keep the small-launch shape whatever came before); whether a launch is part of
// a chain is asked from kHintFromBytes on, the smallest launch whose shape could follow from it.
constexpr unsigned long long kHintFromBytes = 64ull << 20;
constexpr unsigned long long kTrafficBeyondBytes = 8ull << 20;
class RecentTraffic {
   public:
    // Whether one of the recorded launches wrote something in `reads`.
    bool wrote_any_of(const std::vector<Access>& reads) const;
    // Whether the launch recorded last wrote something in `ranges`.
    bool last_wrote_any_of(const std::vector<Access>& ranges) const;
    // Whether the launch recorded last read (and did not write) all of `range`.
    bool last_read_all_of(const Access& range) const;
    // Distinct bytes touched by the recorded launches and by `all` together.
    unsigned long long working_set_with(const std::vector<Access>& all) const;
    void record(const std::vector<Access>& all);
    // The hint for a launch that reads `reads` and touches `all`; `feeds_later`: it is known
    // that a launch soon after it reads what it writes.
    custos_hip::CacheHint classify(const std::vector<Access>& reads, const std::vector<Access>& all,
                                   bool feeds_later = false) const;

   private:
    std::vector<std::vector<Access>> launches_;  // oldest first, at most 8, each merged and sorted
};

// The operand checks of a merged launch over `n_sets` rows of `n_ptrs` device addresses, every
// operand `bytes` long, operand number `written` of a row being the one the launch writes:
// addresses non-null and 16-byte aligned, no partial overlap between a row's output and its inputs
// (the same address is fine), and no row writes memory that another row reads or writes.
// Linear in the number of operands: all operands have one length L, so two of them overlap exactly
// when their addresses are less than L apart.  With memory cut into pieces of L bytes, at most one
// written operand may start in a piece (two would overlap), and whatever overlaps a written operand
// starts in its piece or a neighbouring one: the written operands go into a hash table by piece,
// and every operand looks into three pieces.  The table is sized once (`reserve`) and reused by a
// stamp per check, so a check allocates nothing.
namespace custos_hip {
struct OperandSetChecker {
    struct Slot {
        uint64_t piece, begin;
        uint32_t set, stamp;
    };
    std::vector<Slot> slots;  // a power of two, at least twice the rows of a check
    uint32_t stamp = 0;
    void reserve(size_t max_sets);
    // 0, or CUSTOS_HIP_ERR_INVALID_ARGUMENT / CUSTOS_HIP_ERR_BAD_OVERLAP with `*why` set
    int32_t check(const uint64_t* operands, int n_ptrs, size_t n_sets, int written, uint64_t bytes, const char** why);
};
}  // namespace custos_hip

struct custos_hip_device {
    int idx = 0;
    hipStream_t stream = nullptr;    // compute stream: every launch, in call order
    hipStream_t transfer = nullptr;  // copies that must not be recorded while capturing
    hipEvent_t t0 = nullptr, t1 = nullptr;
    std::vector<hipEvent_t> marks;   // custos_hip_timer_mark: an event per index, created on first use
    hipDeviceProp_t props{};
    std::string arch;
    custos_hip::Tuning tuning;
    bool capturing = false;          // recording: launches, clears and copies go to `recorded`
    // A caller that records the same program before every run (the reference's Lazy module does,
    // src/modules/lazy.rs:190-197): the recording `previous_graph` was built from is kept, and while
    // a new recording repeats it launch for launch (`matching`, `matched` launches so far) nothing
    // is stored; the first launch that differs copies the part that matched into `recorded` and
    // recording goes on as usual.  custos_hip_capture_end_reuse then hands `previous_graph` back
    // without comparing anything when the whole recording matched.
    std::vector<RecNode> previous_recorded;
    custos_hip_graph* previous_graph = nullptr;
    bool matching = false;
    size_t matched = 0;
    uint64_t reused_while_recording = 0, reused_by_comparison = 0, graphs_built = 0;  // how recordings ended (custos_hip_capture_stats)
    bool undrained_at_capture = false;  // work was (possibly) in flight on the compute stream when the recording
                                        // began and nothing has waited for it since (drain_before_immediate_work)
    int32_t literal_policy = 0;      // CUSTOS_HIP_LITERALS_*
    bool eq_as_cpu_eval = false;     // custos_hip_set_eq_policy: `eq` compiled as `<=`
    // per shared-form key: how many distinct texts of that structure were compiled or looked up
    std::unordered_map<uint64_t, uint32_t> value_sets_seen;
    RecentTraffic recent;            // of the launches issued directly (not recorded)
    uint64_t hinted[4] = {0, 0, 0, 0};  // launches and graph nodes of at least kHintFromBytes by CacheHint
    int32_t last_shape[4] = {0, 0, 0, 0};  // vectors per thread, cache policy, alternating, workgroup size: of the generated kernel
                                        // launched or planned into a graph last (custos_hip_last_launch_shape)
    size_t direct_replay_max = 4;    // longest chain replayed as plain launches instead of a hipGraph
    bool graph_verify = false;       // built graphs are checked by brute force against the recorded conflicts
    int32_t graph_edges = CUSTOS_HIP_GRAPH_EDGES_CHAIN;  // how built graphs order their nodes
    // allocation pool: freed blocks by rounded size; every block this handle allocated and has not
    // returned to the driver, by address
    std::unordered_map<size_t, std::vector<void*>> pool;
    struct Block {
        size_t bytes = 0;     // rounded size
        bool pooled = false;  // in `pool` (freed by the caller), else handed out
        int32_t slab = -1;    // index into `slabs` of the allocation the block was cut from, or -1: an allocation of its own
    };
    // Small blocks are cut from larger allocations ("slabs"), which are zero-filled once when they
    // are made: a program that allocates thousands of small buffers pays one driver allocation and
    // one fill launch per slab instead of per buffer.  A slab goes back to the driver when every
    // block cut from it has (a freed block first waits in the pool like any other).
    struct Slab {
        uint64_t base = 0;
        size_t bytes = 0, used = 0;  // `used`: bytes cut off so far
        size_t blocks = 0;           // blocks cut from it that have not gone back to the driver
    };
    std::vector<Slab> slabs;         // (entries of released slabs stay, with base 0)
    int32_t open_slab = -1;          // the slab blocks are being cut from
    std::unordered_map<uint64_t, Block> block_bytes;
    size_t pooled_bytes = 0, pool_limit = 0;
    uint64_t pool_reused = 0, pool_allocated = 0;
    custos_hip_kernel* identity_u32 = nullptr;  // copies run through these
    custos_hip_kernel* identity_u8 = nullptr;
    uint32_t* done_flag = nullptr;  // pinned host word the compute stream writes sequence numbers to
    void* done_flag_dev = nullptr;  // its device address
    uint32_t done_seq = 0;
    // What the next wait waits for, and how long the last one took (the poll window of a wait
    // follows the work, see wait_compute_stream_now in device.hip): graph launches and other
    // work issued on the compute stream since the last wait.
    uint64_t last_wait_ns = 0;
    custos_hip_graph* graph_since_wait = nullptr;
    uint32_t graphs_since_wait = 0;
    bool launches_since_wait = false;
    unsigned long long* scratch_table = nullptr;  // this device's copy of the library's static operand table
    // work area of the operand checks of custos_hip_apply_fn_many_noalloc (made when the handle
    // is created: that call may not allocate, on the host either)
    custos_hip::OperandSetChecker noalloc_checker;
    // The calls that passed those checks last (their addresses, kept in room reserved at creation,
    // replaced in turn): a serving loop calls with the same few tables again and again, and a call
    // identical to one of them passes without the checks.  `noalloc_in_table`: the entry whose
    // rows the GPU's table still holds (nobody rewrote it since), or -1; a call identical to that
    // one launches without sending its rows again.
    struct CheckedCall {
        const custos_hip_kernel* kernel = nullptr;
        size_t n = 0;
        std::vector<uint64_t> operands;
    };
    std::array<CheckedCall, 4> noalloc_checked;
    size_t noalloc_next = 0;
    int noalloc_in_table = -1;
    unsigned char* read_stage = nullptr;  // pinned host memory short reads (first slot) and writes are staged in
    uint64_t read_stage_dev = 0;          // its device address
    uint64_t waits_begun = 0, waits_done = 0;  // waits for the compute stream, numbered
    size_t write_slot = 0;                     // next staging slot of a short write
    std::array<uint64_t, 16> write_slot_issued{};  // per slot: `waits_begun` when its last launch was issued
    std::array<bool, 16> write_slot_used{};
    unsigned long long launch_parity = 0;  // direction of the last launch that alternates
    bool batching = true;            // merge equal independent launches of a level into one grid
    bool fusing = true;              // a recorded apply launch is joined with the apply launches that read what it wrote
    uint64_t fusing_budget_ms = 1000;  // a graph build starts compiling kernels of joined launches while it has spent
                                       // less than this on them
    std::vector<RecNode> recorded;
    uint64_t compiles = 0, hits = 0, disk_hits = 0;  // translation units compiled; cache hits; units loaded from disk
    uint64_t compile_ns = 0;                          // time spent in hiprtc so far
    std::string last_error;
    std::unordered_map<uint64_t, std::vector<std::unique_ptr<custos_hip_kernel>>> cache;
    // expression exactly as the caller spelt it (with kind, type, markers, tuning) -> kernel:
    // a repeated call is answered without parsing (what the (source, name) map of
    // src/devices/cuda/kernel_cache.rs:45-49 does for the reference)
    std::unordered_map<std::string, custos_hip_kernel*> by_text;
    uint64_t compile_epoch = 0;  // advanced by every setting that changes what a text compiles to (tuning, eq and literal policy)
    std::vector<custos_hip_graph*> graphs;
};

namespace custos_hip {

// Stores the message for custos_hip_last_error (per device, or per thread when
// there is no device) and returns `code`.
int32_t set_error(custos_hip_device* dev, int32_t code, const std::string& msg);
// The same for a failed HIP runtime call; clears the runtime's sticky error.
int32_t hip_fail(custos_hip_device* dev, hipError_t e, const char* what);
const std::string& thread_last_error();

#define HIP_TRY(dev, call)                                   \
    do {                                                     \
        hipError_t e__ = (call);                             \
        if (e__ != hipSuccess) return hip_fail(dev, e__, #call); \
    } while (0)

// Every entry point makes the handle's GPU the calling thread's current device -- unless the
// process sees a single GPU, which is then every thread's current device anyway (the call costs
// 0.06 us, a twentieth of what an eager launch costs the host).
extern bool g_single_gpu;  // set when a handle is created
#define REQUIRE_DEV(dev)                                                                    \
    do {                                                                                    \
        if (!(dev)) return set_error(nullptr, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "device handle is null"); \
        if (!custos_hip::g_single_gpu) HIP_TRY(dev, hipSetDevice((dev)->idx));              \
    } while (0)

// An operand of a launch: device address and whether the kernel writes it.
struct Range {
    uint64_t ptr;
    bool written;
};

// launch shape from the C struct; unset fields take the defaults
inline Tuning tuning_from_c(const custos_hip_tuning* t) {
    if (!t) return normalize_tuning(0, 0, 0, 0, 0);
    return normalize_tuning(t->block_threads, t->unroll, t->blocks_per_cu, t->nontemporal, t->direction);
}

// device.hip
hipError_t wait_compute_stream(custos_hip_device* dev);
// Ends the comparison with the previous recording (see custos_hip_device::matching): what matched
// so far becomes the beginning of `recorded`.  Called before anything is appended to `recorded`.
void stop_matching(custos_hip_device* dev);
// While the device compares: whether this launch is the next one of the previous recording (then
// it is counted and nothing else has to be done for it).
inline bool repeats_previous_launch(custos_hip_device* dev, const custos_hip_kernel* k, const uint64_t* ins, int n_ins, uint64_t out,
                                    size_t n) {
    if (dev->matched >= dev->previous_recorded.size()) return false;
    const RecNode& was = dev->previous_recorded[dev->matched];
    if (was.type != RecNode::Kernel || was.k != k || was.n != n || was.ptrs.size() != static_cast<size_t>(n_ins) + 1 ||
        was.ptrs[static_cast<size_t>(n_ins)] != out)
        return false;
    for (int i = 0; i < n_ins; i++)
        if (was.ptrs[static_cast<size_t>(i)] != ins[i]) return false;
    dev->matched++;
    return true;
}
int32_t send_to_device(custos_hip_device* dev, uint64_t dst, const void* src, size_t bytes);
hipError_t drain_before_immediate_work(custos_hip_device* dev);
unsigned int fill_grid(custos_hip_device* dev, unsigned long long n_vec);
unsigned int fill_block();
// device-to-device copy, launched or recorded: the identity kernel, or the runtime's copy
int32_t launch_copy(custos_hip_device* dev, uint64_t dst, uint64_t src, size_t bytes);  // threads per workgroup of the zero-fill kernel
int32_t launch_fill_zero(custos_hip_device* dev, uint64_t dptr, size_t bytes, hipStream_t stream);
void* fill_pattern_kernel();  // the same for a fill with a repeated value
void* fill_zero_kernel();  // host handle of the zero-fill kernel, for graph kernel nodes

// jit.cpp
int32_t compile_to_code_object(custos_hip_device* dev, const KernelSpec& spec, const std::string& arch,
                               std::vector<char>* code, EntrySet which = EntrySet::Single);
// The entry point `which` of `k`, compiled (or loaded from the disk cache) and looked up on first
// use.  Kernels made while the device records are not compiled until a graph build or a launch
// asks for the entry point it uses.
int32_t entry_point(custos_hip_device* dev, custos_hip_kernel* k, EntrySet which, hipFunction_t* fn);
// The kernel of the expression `x` over `dtype` elements (compiled once per device).
int32_t identity_kernel(custos_hip_device* dev, DType dtype, custos_hip_kernel** out);
// How a launch of `k` that touches `footprint_bytes` runs: vectors per thread and cache policy
// from the bytes touched and from what is known about the launches around it (`hint`), unless
// the caller pinned them (the vectors per thread when the kernel was compiled, cache policy and
// direction in the device's tuning now).  `alternate`: the launch walks its tiles against the
// direction of the previous such launch.
struct ResolvedShape {
    int unroll = 2;
    int nontemporal = 0;
    bool alternate = false;
    int block = 128;  // threads per workgroup of this launch
};
// `revisits`: the launch touches memory the launch before it wrote (see preferred_shape).
ResolvedShape resolve_shape(const custos_hip_device* dev, const custos_hip_kernel* k, unsigned long long footprint_bytes,
                            CacheHint hint = CacheHint::Unknown, unsigned long long working_set_bytes = 0, bool revisits = true, int keep_inputs = 0);
// The shape of ONE launch of `k` over the operand ranges `acc`, from the launches before it
// (`history`, which the launch then joins) and from whether a launch soon after it reads what it
// writes (`feeds_later`); counts the hint in the device's statistics.  The same decision for a
// launch issued directly, a node of a graph being built, and a node of a short recording that is
// replayed as plain launches.
ResolvedShape shape_of_launch(custos_hip_device* dev, const custos_hip_kernel* k, const std::vector<Access>& acc,
                              RecentTraffic* history, bool feeds_later);

// jit.cpp: the kernel handle for a chain of apply expressions (cached; compiled when an entry point is asked for).
int32_t chain_kernel(custos_hip_device* dev, DType dtype, std::vector<ChainStage> stages, int n_ext, int n_outs,
                     const Tuning& tuning, custos_hip_kernel** out);
// The mode word of a single launch of `k` over n elements (n_vec vectors after `head` scalar
// elements) in the given shape.
inline uint64_t single_launch_mode(const custos_hip_kernel* k, unsigned long long n, unsigned long long head,
                                   unsigned long long n_vec, const ResolvedShape& shape, bool rev) {
    const unsigned long long tile_vecs = static_cast<unsigned long long>(shape.block) * shape.unroll;
    const bool edges = head > 0 || head + n_vec * static_cast<unsigned long long>(k->spec.vec_elems) < n;
    return custos_hip::launch_mode(shape.unroll, shape.nontemporal, rev, shape.block, (n_vec + tile_vecs - 1) / tile_vecs, edges);
}
// The values of a recorded launch's literal parameters.
inline const std::vector<unsigned char>& literal_values(const RecNode& n) {
    return n.k->spec.kind == custos_hip::Kind::Chain ? n.const_bytes : n.k->spec.consts.bytes;
}
// launch.cpp
int32_t launch_or_record(custos_hip_device* dev, custos_hip_kernel* k, const std::vector<Range>& ops, size_t n);
// Workgroups of a single launch of `k` over n_vec vectors and n elements in the given shape.
unsigned int launch_grid(const custos_hip_device* dev, const custos_hip_kernel* k, unsigned long long n,
                         unsigned long long n_vec, const ResolvedShape& shape);

// graph.cpp
int32_t replay_graph(custos_hip_device* dev, custos_hip_graph* g);
int32_t build_graph(custos_hip_device* dev, custos_hip_graph* g);
void destroy_graph(custos_hip_graph* g);

}  // namespace custos_hip
