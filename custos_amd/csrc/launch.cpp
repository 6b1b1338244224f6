// Launches of generated and caller-written kernels: operand checks, the split
// into scalar head / 16-byte vectors / scalar tail, and recording while the
// device records (include/custos_hip.h).
#include <algorithm>
#include <cstdlib>
#include <cstring>

#include "runtime.hpp"

// ---- RecentTraffic ----

namespace {

constexpr size_t kTrafficDepth = 8;  // launches looked back at

// Sorted, non-overlapping ranges covering the same addresses; `write` = any writer.
std::vector<Access> merged(std::vector<Access> ranges) {
    std::sort(ranges.begin(), ranges.end(), [](const Access& a, const Access& b) { return a.begin < b.begin; });
    std::vector<Access> out;
    for (const Access& r : ranges) {
        if (r.end <= r.begin) continue;
        if (!out.empty() && r.begin <= out.back().end) {
            out.back().end = std::max(out.back().end, r.end);
            out.back().write = out.back().write || r.write;
        } else {
            out.push_back(r);
        }
    }
    return out;
}

unsigned long long total_bytes(const std::vector<Access>& sorted_disjoint) {
    unsigned long long bytes = 0;
    for (const Access& r : sorted_disjoint) bytes += r.end - r.begin;
    return bytes;
}

}  // namespace

bool RecentTraffic::wrote_any_of(const std::vector<Access>& reads) const {
    for (const std::vector<Access>& launch : launches_)
        for (const Access& w : launch) {
            if (!w.write) continue;
            for (const Access& r : reads)
                if (r.begin < w.end && w.begin < r.end) return true;
        }
    return false;
}

bool RecentTraffic::last_read_all_of(const Access& range) const {
    if (launches_.empty()) return false;
    for (const Access& was : launches_.back())
        if (!was.write && was.begin <= range.begin && range.end <= was.end) return true;
    return false;
}

bool RecentTraffic::last_wrote_any_of(const std::vector<Access>& ranges) const {
    if (launches_.empty()) return false;
    for (const Access& w : launches_.back()) {
        if (!w.write) continue;
        for (const Access& r : ranges)
            if (r.begin < w.end && w.begin < r.end) return true;
    }
    return false;
}

unsigned long long RecentTraffic::working_set_with(const std::vector<Access>& all) const {
    std::vector<Access> touched = all;
    for (const std::vector<Access>& launch : launches_) touched.insert(touched.end(), launch.begin(), launch.end());
    return total_bytes(merged(std::move(touched)));
}

custos_hip::CacheHint RecentTraffic::classify(const std::vector<Access>& reads, const std::vector<Access>& all,
                                              bool feeds_later) const {
    const bool fits = working_set_with(all) <= custos_hip::kCacheWorkingSet;
    if (!feeds_later && !wrote_any_of(reads)) return fits ? custos_hip::CacheHint::Unknown : custos_hip::CacheHint::Crowded;
    return fits ? custos_hip::CacheHint::Resident : custos_hip::CacheHint::Streams;
}

void RecentTraffic::record(const std::vector<Access>& all) {
    if (launches_.size() == kTrafficDepth) launches_.erase(launches_.begin());
    // written and read ranges are merged separately, so that the writer flag stays exact
    std::vector<Access> reads, writes;
    for (const Access& a : all) (a.write ? writes : reads).push_back(a);
    std::vector<Access> launch = merged(std::move(writes));
    const std::vector<Access> r = merged(std::move(reads));
    launch.insert(launch.end(), r.begin(), r.end());
    launches_.push_back(std::move(launch));
}

namespace custos_hip {

namespace {

// Checks operand addresses and computes how the element range splits into a
// scalar head, 16-byte vectors and a scalar tail.
int32_t plan_launch(custos_hip_device* dev, const custos_hip_kernel* k, const std::vector<Range>& ops,
                    size_t n, unsigned long long* head, unsigned long long* n_vec) {
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
    *head = h;
    *n_vec = nv;
    return CUSTOS_HIP_OK;
}

}  // namespace

unsigned int launch_grid(const custos_hip_device* dev, const custos_hip_kernel* k, unsigned long long n,
                         unsigned long long n_vec, const ResolvedShape& shape) {
    const Tuning& t = k->spec.tuning;
    const unsigned long long block = static_cast<unsigned long long>(shape.block);
    const unsigned long long tile_vecs = block * shape.unroll;
    unsigned long long tiles = (n_vec + tile_vecs - 1) / tile_vecs;
    const unsigned long long scalar = n - n_vec * k->spec.vec_elems;
    const unsigned long long cus = static_cast<unsigned long long>(dev->props.multiProcessorCount);
    const unsigned long long scalar_blocks = std::min((scalar + block - 1) / block, cus * 32);
    if (t.blocks_per_cu > 0) tiles = std::min(tiles, cus * t.blocks_per_cu);
    unsigned long long g = std::max(1ull, std::max(tiles, scalar_blocks));
    return static_cast<unsigned int>(std::min(g, 1ull << 22));
}

// Launches the kernel over one set of operands, or records the launch while
// the device is recording.  `ops` are the operand addresses in the order of the
// kernel's pointer parameters.
int32_t launch_or_record(custos_hip_device* dev, custos_hip_kernel* k, const std::vector<Range>& ops, size_t n) {
    if (dev->capturing && dev->matching && dev->matched < dev->previous_recorded.size()) {
        // (launches that do not come through custos_hip_apply_fn_n, which compares by itself: copies)
        const RecNode& was = dev->previous_recorded[dev->matched];
        bool same = was.type == RecNode::Kernel && was.k == k && was.n == n && was.ptrs.size() == ops.size();
        for (size_t i = 0; same && i < ops.size(); i++) same = was.ptrs[i] == ops[i].ptr;
        if (same) {
            dev->matched++;
            return CUSTOS_HIP_OK;
        }
    }
    unsigned long long head = 0, n_vec = 0, count = n;
    int32_t rc = plan_launch(dev, k, ops, n, &head, &n_vec);
    if (rc != CUSTOS_HIP_OK) return rc;
    if (dev->capturing) {
        stop_matching(dev);
        RecNode node;
        node.type = RecNode::Kernel;
        node.k = k;
        node.n = n;
        node.head = head;
        node.n_vec = n_vec;
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
    // (compiled when custos_hip_expr_compile returned, unless the device was recording then)
    hipFunction_t fn = nullptr;
    rc = entry_point(dev, k, EntrySet::Single, &fn);
    if (rc != CUSTOS_HIP_OK) return rc;
    // the launch shape that suits the bytes this launch touches and what the launches just
    // before it left in the caches
    const uint64_t bytes = static_cast<uint64_t>(n) * dtype_size(k->spec.dtype);
    std::vector<Access> acc;
    for (const Range& r : ops) acc.push_back({r.ptr, r.ptr + bytes, r.written});
    const ResolvedShape shape = shape_of_launch(dev, k, acc, &dev->recent, /*feeds_later=*/false);
    const unsigned int grid = launch_grid(dev, k, n, n_vec, shape);
    unsigned long long mode = single_launch_mode(k, n, head, n_vec, shape, shape.alternate && (dev->launch_parity ^= 1));
    uint64_t ptrs[8];
    std::vector<void*> args;
    for (size_t i = 0; i < ops.size(); i++) {
        ptrs[i] = ops[i].ptr;
        args.push_back(&ptrs[i]);
    }
    args.push_back(&count);
    args.push_back(&head);
    args.push_back(&n_vec);
    // the expression's literals that are launch parameters: one block by value
    if (k->spec.consts.n_params > 0) args.push_back(k->spec.consts.bytes.data());
    args.push_back(&mode);
    dev->launches_since_wait = true;
    HIP_TRY(dev, hipModuleLaunchKernel(fn, grid, 1, 1, static_cast<unsigned int>(shape.block), 1, 1, 0, dev->stream, args.data(),
                                       nullptr));
    return CUSTOS_HIP_OK;
}

ResolvedShape shape_of_launch(custos_hip_device* dev, const custos_hip_kernel* k, const std::vector<Access>& acc,
                              RecentTraffic* history, bool feeds_later) {
    unsigned long long footprint = 0;
    for (const Access& a : acc) footprint += a.end - a.begin;
    CacheHint hint = CacheHint::Unknown;
    unsigned long long working_set = 0;
    bool revisits = true;
    int keep_inputs = 0;
    if (footprint > kTrafficBeyondBytes) {
        if (footprint >= kHintFromBytes) {
            std::vector<Access> reads;
            // (the gradient operand of a unary-gradient kernel is read and written)
            for (const Access& a : acc)
                if (!a.write || k->spec.kind == Kind::UnaryGrad) reads.push_back(a);
            hint = history->classify(reads, acc, feeds_later);
            dev->hinted[static_cast<int>(hint)]++;
        }
        // what the launches before it leave to this one: the L2s to a small launch, the
        // memory-side cache to a large one
        working_set = history->working_set_with(acc);
        revisits = history->last_wrote_any_of(acc);
        // Inputs (the first four pointers can be named) that this launch only reads and that the
        // launch before it read as well, while nothing that launch wrote is touched: they are what
        // the memory-side cache can still hold of that launch, and what the launch after this one
        // is likely to read again -- if they are no more than twice what that cache holds.
        if (!revisits) {
            unsigned long long kept = 0;
            for (size_t i = 0; i < acc.size() && i < 4; i++) {
                if (acc[i].write || !history->last_read_all_of(acc[i])) continue;
                bool also_written = false;
                for (const Access& w : acc) also_written = also_written || (w.write && w.begin < acc[i].end && acc[i].begin < w.end);
                if (also_written) continue;
                keep_inputs |= 1 << i;
                kept += acc[i].end - acc[i].begin;
            }
            if (kept > 2 * kCacheWorkingSet) keep_inputs = 0;
        }
        history->record(acc);
    }
    const ResolvedShape shape = resolve_shape(dev, k, footprint, hint, working_set, revisits, keep_inputs);
    dev->last_shape[0] = shape.unroll, dev->last_shape[1] = shape.nontemporal, dev->last_shape[2] = shape.alternate;
    dev->last_shape[3] = shape.block;
    return shape;
}

}  // namespace custos_hip

using namespace custos_hip;

extern "C" {

// ---- launches ----

int32_t custos_hip_apply_fn_n(custos_hip_device* dev, custos_hip_kernel* kernel, const uint64_t* ins,
                              int32_t n_ins, uint64_t out, size_t n) {
    // (the same launch as in the recording before: it passed every check then, and nothing is
    // asked of the runtime for it, so the device need not be made current either)
    if (dev && dev->matching && kernel && ins && n_ins >= 0 && repeats_previous_launch(dev, kernel, ins, n_ins, out, n))
        return CUSTOS_HIP_OK;
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

int32_t custos_hip_last_launch_shape(custos_hip_device* dev, int32_t* unroll, int32_t* nontemporal, int32_t* alternate) {
    REQUIRE_DEV(dev);
    if (unroll) *unroll = dev->last_shape[0];
    if (nontemporal) *nontemporal = dev->last_shape[1];
    if (alternate) *alternate = dev->last_shape[2];
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_launch_hint_stats(custos_hip_device* dev, uint64_t* unrelated, uint64_t* resident, uint64_t* streaming) {
    REQUIRE_DEV(dev);
    if (unrelated) *unrelated = dev->hinted[static_cast<int>(CacheHint::Unknown)] + dev->hinted[static_cast<int>(CacheHint::Crowded)];
    if (resident) *resident = dev->hinted[static_cast<int>(CacheHint::Resident)];
    if (streaming) *streaming = dev->hinted[static_cast<int>(CacheHint::Streams)];
    return CUSTOS_HIP_OK;
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
    if (dev && dev->matching && kernel) {
        const uint64_t first_two[2] = {lhs, lhs_grad};
        if (repeats_previous_launch(dev, kernel, first_two, 2, out_grad, n)) return CUSTOS_HIP_OK;
    }
    REQUIRE_DEV(dev);
    if (!kernel) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "null kernel");
    if (kernel->spec.kind != Kind::UnaryGrad)
        return set_error(dev, CUSTOS_HIP_ERR_KIND_MISMATCH, "kernel was not compiled as a unary-gradient kernel");
    if (n == 0) return CUSTOS_HIP_OK;
    std::vector<Range> ops = {{lhs, false}, {lhs_grad, true}, {out_grad, false}};
    return launch_or_record(dev, kernel, ops, n);
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
        if (dev->matching && dev->matched < dev->previous_recorded.size()) {
            const RecNode& was = dev->previous_recorded[dev->matched];
            bool same = was.type == RecNode::Source && was.k == kernel && was.shared_mem == shared_mem_bytes &&
                        was.arg_values.size() == static_cast<size_t>(n_params);
            for (int i = 0; same && i < 3; i++) same = was.grid3[i] == grid[i] && was.block3[i] == block[i];
            for (int i = 0; same && i < n_params; i++) {
                const auto& value = was.arg_values[static_cast<size_t>(i)];
                same = params[i] && value.size() == param_sizes[i] && std::memcmp(value.data(), params[i], param_sizes[i]) == 0;
            }
            if (same) {
                dev->matched++;
                return CUSTOS_HIP_OK;
            }
        }
        stop_matching(dev);
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
    dev->launches_since_wait = true;
    HIP_TRY(dev, hipModuleLaunchKernel(kernel->fns[0], grid[0], grid[1], grid[2], block[0], block[1], block[2],
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
    HIP_TRY(dev, hipModuleOccupancyMaxPotentialBlockSize(&min_grid, &block_size, kernel->fns[0], 0, 0));
    if (block_size <= 0) block_size = 256;
    const uint64_t blocks = (len + static_cast<size_t>(block_size) - 1) / static_cast<size_t>(block_size);
    if (blocks > 0x7fffffffull) return set_error(dev, CUSTOS_HIP_ERR_TOO_LARGE, "more workgroups than a one-dimensional grid holds");
    const uint32_t grid[3] = {static_cast<uint32_t>(blocks), 1, 1};
    const uint32_t block[3] = {static_cast<uint32_t>(block_size), 1, 1};
    return custos_hip_source_launch(dev, kernel, grid, block, 0, params, param_sizes, n_params);
}

}  // extern "C"
