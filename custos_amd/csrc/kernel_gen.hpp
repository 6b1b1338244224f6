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

enum class Kind : int32_t { Apply = 0, UnaryGrad = 1, Source = 2 /* caller-written kernel source */ };

struct Tuning {
    // Defaults from interleaved, repeated timing of the fused f32 chain at 2^28
    // elements on MI355X: workgroups of 64 or 128 threads with 2 vectors per
    // thread sustain 3-5 % more than 256..1024-thread workgroups or other unroll
    // factors (many small workgroups keep the memory channels evenly loaded);
    // streaming (non-temporal) loads and stores add another 1-2 %; persistent
    // grids were 5-20 % slower.
    int block_threads = 128;
    int unroll = 2;
    int blocks_per_cu = 0;  // <= 0: one tile per workgroup
    int nontemporal = 3;    // bit 0 loads, bit 1 stores
};

// Fills unset (zero) fields with the defaults and clamps to legal values.
Tuning normalize_tuning(int block_threads, int unroll, int blocks_per_cu, int nontemporal);

struct KernelSpec {
    Kind kind = Kind::Apply;
    DType dtype = DType::F32;
    Expr expr;
    Tuning tuning;
    uint64_t hash = 0;   // cache key: expression, dtype, kind, tuning
    std::string name;    // entry point: custos_<kind>_<dtype>_<hash>, unique per kernel so
                         // that profiler output tells the kernels apart
    std::string source;  // complete translation unit
    int vec_elems = 4;   // elements per 16-byte vector
};

// Parses, hashes and emits. On failure returns false and fills `err`.
bool build_kernel_spec(Kind kind, DType dtype, const std::string& src,
                       const std::vector<std::string>& markers, const Tuning& tuning,
                       KernelSpec* out, ParseError* err);

// Options handed to hiprtc for every kernel.
std::vector<std::string> hiprtc_options(const std::string& arch);

}  // namespace custos_hip
