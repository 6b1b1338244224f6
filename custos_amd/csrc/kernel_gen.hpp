// Generates the HIP source of one element-wise kernel from an expression.
//
// Replaces the format!() kernel strings of the reference
// (src/devices/cuda/ops.rs:154-166,214-226, src/devices/cuda/fusing.rs:27-39):
// instead of one thread per element with 4-byte accesses, every lane moves
// 16-byte vectors, `unroll` of them per tile, all loads of a tile issued before
// the first store.
#pragma once

#include <cstdint>
#include <string>
#include <vector>

#include "expr.hpp"

namespace custos_hip {

enum class Kind : int32_t {
    Apply = 0,
    UnaryGrad = 1,
    Source = 2,  // caller-written kernel source
    Chain = 3,   // several apply expressions in one kernel, every one with its own output (made when a graph is built)
};

struct Tuning {
    // Launch shape of the generated kernels.  Workgroups of 64 or 128 threads
    // sustain 3-5 % more than 256..1024-thread workgroups in interleaved,
    // repeated timing on MI355X (many small workgroups keep the memory channels
    // evenly loaded); persistent grids were 5-20 % slower.  The other three
    // knobs are chosen per launch from the bytes it touches (preferred_shape)
    // unless the caller fixes them.
    int block_threads = 128;
    int unroll = 0;         // 16-byte vectors per thread and tile; 0: chosen per launch (2, or 1 with one-wavefront workgroups)
    int blocks_per_cu = 0;  // <= 0: one tile per workgroup
    int nontemporal = -1;   // bit 0 loads, bit 1 stores, 64 stores written through at once; -1: chosen per
                            // launch.  Read from the device's tuning when a launch is issued or a graph built.
    int direction = 0;      // 1: tiles first to last; 2: every launch the other way round; 0: chosen per launch
    // Not a shape, but it travels the same way: `eq` nodes are compiled as `<=`, which is what the
    // reference's CPU device evaluates for them (src/two_way_ops/ops/cmps.rs:135), instead of `==`,
    // which is what the reference's GPU kernels compute.
    bool eq_as_leq = false;
};

// What suits a launch that touches `footprint_bytes` (all operands together)
// through `n_operands` pointers.
struct LaunchShape {
    int unroll;
    int nontemporal;
    bool alternate;  // walk the tiles in the direction opposite to the previous launch
    int block = 0;   // threads per workgroup; 0: the most the kernel was compiled for
};
// What is known about a launch from the address ranges of the launches around it.  A launch
// that reads what one of the last few launches wrote (or whose output one of the next few
// reads) is part of a chain; what suits it depends on whether everything those launches touch
// stays in the memory-side cache (256 MiB).
enum class CacheHint {
    Unknown,   // not part of a chain: the launch shape follows the bytes the launch touches
    Crowded,   // not part of a chain, but the launches around it touch more than the cache holds
    Resident,  // the chain's working set fits the cache: temporal accesses
    Streams,   // it does not: stream past the cache
};
constexpr unsigned long long kCacheWorkingSet = 256ull << 20;
// `working_set_bytes`: distinct bytes touched by the launch and the last few launches before it
// together (0 = not known: the launch's own bytes count).
constexpr unsigned long long kL2WorkingSet = 32ull << 20;  // what the eight L2s hold together
// `revisits`: the launch touches memory that the launch before it wrote (the same launch repeated,
// a consumer of the last launch); `n_written`: how many of its operands it writes.
LaunchShape preferred_shape(unsigned long long footprint_bytes, int n_operands, CacheHint hint = CacheHint::Unknown,
                            unsigned long long working_set_bytes = 0, bool revisits = true, int n_written = 1, int keep_inputs = 0);

// The last argument of every generated entry point: how this launch runs the kernel.  Nothing
// of it is compiled in, so one kernel per expression serves every launch size.
//   bit 0      the tiles are walked from the last to the first
//   bit 1, 2   non-temporal loads, non-temporal stores
//   bits 3..6  input 0..3 is loaded with temporal accesses although bit 1 is set: the memory-side cache is
//              to keep that input (the launch after this one reads it again) and nothing else
//   bit 7      stores are written through to device scope at once instead of lingering in an L2
//   bits 8..11 vectors per thread (only read by kernels whose launch shape was left open)
//   bits 13,14 threads per workgroup as 64 << bits (likewise)
//   bit 12     (single-launch entry point) the range has scalar elements: a head before the first
//              16-byte boundary or a tail after the last whole vector
//   bits 16..  (single-launch entry point) the number of tiles of the vector range
// The last two spare every workgroup of a launch the arithmetic that finds them out again: the
// host knows them.
// `nontemporal` as in Tuning: bit 0 loads, bit 1 stores, kStoresWriteThrough the write-through stores;
// bits kKeepInputShift.. (library's choice only): the inputs that keep temporal loads.
constexpr int kStoresWriteThrough = 64;
constexpr int kKeepInputShift = 8, kKeepInputMask = 15;
inline uint64_t launch_mode(int unroll, int nontemporal, bool rev, int block_threads, uint64_t n_tiles = 0,
                            bool scalar_edges = true) {
    const uint64_t log2_waves = block_threads >= 512 ? 3 : block_threads >= 256 ? 2 : block_threads >= 128 ? 1 : 0;
    return (rev ? 1u : 0u) | static_cast<uint64_t>(nontemporal & 3) << 1 |
           static_cast<uint64_t>((nontemporal >> kKeepInputShift) & kKeepInputMask) << 3 |
           static_cast<uint64_t>((nontemporal & kStoresWriteThrough) ? 1 : 0) << 7 | static_cast<uint64_t>(unroll & 15) << 8 |
           (scalar_edges ? 1u << 12 : 0u) | log2_waves << 13 | n_tiles << 16;
}

// Fills unset (zero) fields with the defaults and clamps to legal values
// (`nontemporal` and `direction` as in custos_hip_tuning).
Tuning normalize_tuning(int block_threads, int unroll, int blocks_per_cu, int nontemporal, int direction);

// One expression of a chain kernel.  A chain stands for apply launches that were recorded one
// after the other, the later ones reading what the earlier ones wrote: every stage computes its
// expression, stores the result where its launch stored it, and a later stage that read that
// memory takes the value as it was stored (rounded to the storage type) from a register.
struct ChainStage {
    Expr expr;
    std::vector<int> source;  // per variable of `expr`: index of an input pointer of the kernel, or
                              // -(1 + s) for the stored value of stage s
    int out = -1;             // which output pointer of the kernel receives the value; -1: none, a
                              // later stage writes the same memory
    std::vector<int> slot;    // per node of `expr`: the literal is launch parameter `slot` of this stage, or
                              // -1 (ConstPlan::slot of the launch's own kernel); empty: every literal in the code
    int n_params = 0;         // launch parameters of this stage; in the kernel's block they follow those of the
                              // stages before it
    size_t param_bytes = 0;   // their size (n_params values of the compute type)
};
constexpr int kMaxChainStages = 8, kMaxChainInputs = 8, kMaxChainOutputs = 6;

// A generated kernel has three entry points, each in a translation unit of its own (the
// per-element function and the tile function repeat in all three) that is compiled when it is
// first needed: a transcendental expression is expanded eight or nine times per entry point,
// and most kernels are only ever launched through one of them.
enum class EntrySet : int {
    Single = 0,   // `<name>`: one launch over one set of operands
    Batched = 1,  // `<name>_batched`: many operand sets of equal length in one grid
    Ragged = 2,   // `<name>_ragged`: many operand sets of different lengths in one grid
};
constexpr int kEntrySets = 3;
inline const char* entry_suffix(EntrySet which) {
    return which == EntrySet::Single ? "" : which == EntrySet::Batched ? "_batched" : "_ragged";
}

struct KernelSpec {
    Kind kind = Kind::Apply;
    DType dtype = DType::F32;
    Expr expr;                       // Apply, UnaryGrad
    std::vector<ChainStage> stages;  // Chain
    int n_ext = 0, n_outs = 0;       // Chain: input and output pointers (inputs first)
    std::string chain_text;          // Chain: the stages spelt out, literal values included
    Tuning tuning;             // as compiled: workgroup size, grid kind, most vectors per thread
    bool auto_unroll = false;  // the caller left the launch shape open: the kernel holds the tile functions for
                               // 2 and for 1 vectors per thread, and every launch names its vectors per thread
                               // and its workgroup size (64 threads, or `tuning.block_threads`) in its mode word
    ConstPlan consts;          // literals that are launch parameters, and this text's values for them
    int n_literals = 0;        // literals in the expression, parameters or not
    std::vector<uint64_t> code_literals;  // values of the literals that stay in the code, in node order
    std::vector<std::string> markers;     // operand names, for the text
    uint64_t hash = 0;   // cache key: expression without the parameter values, dtype, kind, tuning
    std::string name;    // entry point: custos_<kind>_<dtype>_<hash>, unique per kernel so
                         // that profiler output tells the kernels apart
    std::string source[3];  // the kernel's translation units by EntrySet (each empty until emit_kernel_source)
    int vec_elems = 4;   // elements per 16-byte vector
};

// Parses, hashes and emits. On failure returns false and fills `err`.
// `literals_in_code`: the kernel for exactly these literal values (the compiler sees them);
// else the form shared by all expressions that differ only in literal values, which takes
// them as launch parameters (ConstPlan).
// `with_source = false` stops before the text is generated (enough for a cache lookup).
bool build_kernel_spec(Kind kind, DType dtype, const std::string& src,
                       const std::vector<std::string>& markers, const Tuning& tuning,
                       bool literals_in_code, KernelSpec* out, ParseError* err, bool with_source = true);
// The same for a chain kernel; a stage's literals are in the code or launch parameters as they are
// for the kernel of the stage's own launch.
bool build_chain_spec(DType dtype, std::vector<ChainStage> stages, int n_ext, int n_outs, const Tuning& tuning,
                      KernelSpec* out, ParseError* err, bool with_source = true);
// Pointer parameters of a generated kernel's single-launch entry point (= the width of a table
// row of a merged launch, before the literal parameters).
int kernel_pointers(const KernelSpec& k);
// Generates `k->source[which]` (which also finds node / element type combinations that cannot be
// compiled, such as a transcendental node over integers).
bool emit_kernel_source(KernelSpec* k, ParseError* err, EntrySet which = EntrySet::Single);
// Whether two specs describe the same translation unit, without looking at the text: kind,
// element type, launch shape, expression structure and the literals that stay in the code.
bool same_code(const KernelSpec& a, const KernelSpec& b);

// Options handed to hiprtc for every kernel.
std::vector<std::string> hiprtc_options(const std::string& arch);

}  // namespace custos_hip
