// `HIP<Mods>`: the MI355X device, over the C ABI of libcustos_hip.so.
//
// Takes the place of `CUDA<Mods>` in user code: `HIP<Lazy<Graph<Base>>>` for
// `CUDA<Lazy<Graph<Base>>>`.  Mirrors src/devices/cuda/cuda.rs:22-165 (device,
// Alloc), src/devices/cuda/ops.rs:17-234 (Read/Write/Clear, ApplyFunction,
// UnaryGrad), src/devices/cuda/fusing.rs:3-51 (UnaryFusing) and
// src/devices/cuda/lazy.rs:31-72 (LazySetup / LazyRun).  Everything a kernel
// computes happens in the library; nothing is evaluated on the host.
#pragma once

#include <array>
#include <cstdint>
#include <cstring>
#include <functional>
#include <memory>
#include <string>
#include <type_traits>
#include <vector>

#include "../../../include/custos_hip.h"
#include "device.hpp"

namespace custos {

// `CDatatype` (src/devices/cdatatype.rs:3-62): element types the kernels know.
template <class T>
struct HipDType;
#define CUSTOS_HIP_DTYPE(T, V)                         \
    template <>                                        \
    struct HipDType<T> {                               \
        static constexpr int32_t value = V;            \
    };
CUSTOS_HIP_DTYPE(float, CUSTOS_HIP_F32)
CUSTOS_HIP_DTYPE(double, CUSTOS_HIP_F64)
CUSTOS_HIP_DTYPE(int32_t, CUSTOS_HIP_I32)
CUSTOS_HIP_DTYPE(int64_t, CUSTOS_HIP_I64)
CUSTOS_HIP_DTYPE(uint8_t, CUSTOS_HIP_U8)
CUSTOS_HIP_DTYPE(int8_t, CUSTOS_HIP_I8)
CUSTOS_HIP_DTYPE(int16_t, CUSTOS_HIP_I16)
CUSTOS_HIP_DTYPE(uint16_t, CUSTOS_HIP_U16)
CUSTOS_HIP_DTYPE(uint32_t, CUSTOS_HIP_U32)
CUSTOS_HIP_DTYPE(uint64_t, CUSTOS_HIP_U64)
#undef CUSTOS_HIP_DTYPE

// 16-bit floats (custos/half.hpp): f32 compute and one rounding in the kernels for
// f16 / bf16, every node rounded for the *_pernode types.
template <>
struct HipDType<f16> {
    static constexpr int32_t value = CUSTOS_HIP_F16;
};
template <>
struct HipDType<bf16> {
    static constexpr int32_t value = CUSTOS_HIP_BF16;
};
template <>
struct HipDType<f16_pernode> {
    static constexpr int32_t value = CUSTOS_HIP_F16_PERNODE;
};
template <>
struct HipDType<bf16_pernode> {
    static constexpr int32_t value = CUSTOS_HIP_BF16_PERNODE;
};

template <class Mods>
class HIP : public Device<HIP<Mods>, Mods> {
   public:
    using Self = HIP<Mods>;

    // `HIP::<Mods>::new(idx)` (src/devices/cuda/cuda.rs:53-67): creates the
    // device state, then lets the modules set up (Lazy calls `lazy_setup`).
    explicit HIP(int idx = custos_hip_chosen_device_idx()) {
        int32_t rc = custos_hip_device_create(idx, &dev_);
        if (rc != CUSTOS_HIP_OK) throw Error(DeviceError::Backend, rc, custos_hip_last_error(nullptr));
        this->modules.setup(*this);
    }
    HIP(const HIP&) = delete;
    HIP& operator=(const HIP&) = delete;
    ~HIP() {
        // module-owned allocations go first, while the device handle is alive
        this->modules.teardown(*this);
        if (graph_) custos_hip_graph_destroy(dev_, graph_);
        custos_hip_device_destroy(dev_);
    }

    custos_hip_device* handle() const { return dev_; }
    void sync() { check(custos_hip_sync(dev_)); }

    // ---- raw memory (Alloc / Read / WriteBuf / ClearBuf) ----
    uint64_t alloc_raw(size_t bytes, bool zeroed, size_t /*len*/) {
        uint64_t p = 0;
        check(custos_hip_alloc(dev_, bytes, zeroed ? CUSTOS_HIP_ALLOC_ZEROED : CUSTOS_HIP_ALLOC_UNINIT, &p));
        return p;
    }
    void free_raw(uint64_t ptr) {
        if (dev_) custos_hip_free(dev_, ptr);
    }
    void read_raw(void* dst, uint64_t src, size_t bytes) { check(custos_hip_read(dev_, dst, src, bytes)); }
    void write_raw(uint64_t dst, const void* src, size_t bytes) { check(custos_hip_write(dev_, dst, src, bytes)); }
    void clear_raw(uint64_t ptr, size_t bytes) { check(custos_hip_clear(dev_, ptr, bytes)); }
    void fill_raw(uint64_t ptr, size_t bytes, const void* value, size_t value_bytes) {
        check(custos_hip_fill(dev_, ptr, bytes, value, value_bytes));
    }
    void copy_raw(uint64_t dst, uint64_t src, size_t bytes) { check(custos_hip_copy(dev_, dst, src, bytes)); }

    // ---- launches ----

    // `try_cu_apply_fn_mut` (src/devices/cuda/ops.rs:144-177): print the
    // expression with the marker, fetch the kernel, launch.
    template <class T, class F>
    void apply_fn_impl(const Buffer<T, Self>& x, Buffer<T, Self>& out, F f) {
        const std::string src = to_cl_source(f(Resolve<T>::with_marker("x")));
        custos_hip_kernel* k = compile(CUSTOS_HIP_KIND_APPLY, HipDType<T>::value, src, {"x"});
        check(custos_hip_apply_fn(dev_, k, x.ptr(), out.ptr(), x.len()));
    }

    // Two-operand expression `f(lhs, rhs)` (src/two_way_ops/mod.rs:96-104,172-193).
    template <class T, class F>
    void apply_fn2_impl(const Buffer<T, Self>& lhs, const Buffer<T, Self>& rhs, Buffer<T, Self>& out, F f) {
        const std::string src = to_cl_source(f(Resolve<T>::with_marker("x"), Resolve<T>::with_marker("y")));
        custos_hip_kernel* k = compile(CUSTOS_HIP_KIND_APPLY, HipDType<T>::value, src, {"x", "y"});
        check(custos_hip_apply_fn2(dev_, k, lhs.ptr(), rhs.ptr(), out.ptr(), lhs.len()));
    }

    // `try_cu_add_unary_grad` (src/devices/cuda/ops.rs:201-234)
    template <class T, class F>
    void add_unary_grad_impl(const Buffer<T, Self>& lhs, Buffer<T, Self>& lhs_grad, const Buffer<T, Self>& out_grad, F f) {
        const std::string src = to_cl_source(f(Resolve<T>::with_marker("x")));
        custos_hip_kernel* k = compile(CUSTOS_HIP_KIND_UNARY_GRAD, HipDType<T>::value, src, {"x"});
        check(custos_hip_add_unary_grad(dev_, k, lhs.ptr(), lhs_grad.ptr(), out_grad.ptr(), lhs.len()));
    }

    // `UnaryFusing::unary_fuse_op` (src/devices/cuda/fusing.rs:8-50): one kernel
    // for the whole chain; the fused body is `operations_to_fused_src`.
    template <class T>
    std::function<void(Buffer<T, Self>&, const Buffer<T, Self>&, Self&)> unary_fuse_op(
        std::vector<std::shared_ptr<UnaryHint<T>>> ops_to_fuse) {
        return [ops = std::move(ops_to_fuse)](Buffer<T, Self>& out, const Buffer<T, Self>& buf, Self& dev) {
            if (ops.empty()) return;
            const std::string src = operations_to_fused_src<T>(ops);
            custos_hip_kernel* k = dev.compile(CUSTOS_HIP_KIND_APPLY, HipDType<T>::value, src, {"x"});
            dev.check(custos_hip_apply_fn(dev.dev_, k, buf.ptr(), out.ptr(), buf.len()));
        };
    }

    // The operation `Lazy::elementwise_fusing` puts in place of several hinted
    // operations: one kernel over up to four operand buffers.
    template <class T>
    std::function<void(Buffer<T, Self>&, const std::vector<Buffer<T, Self>>&, Self&)> elementwise_fuse_op(
        std::shared_ptr<FusedExpr<T>> expr) {
        return [expr](Buffer<T, Self>& out, const std::vector<Buffer<T, Self>>& ins, Self& dev) {
            static const char* const names[] = {"a", "b", "c", "d"};
            std::vector<std::string> markers;
            std::vector<const char*> cmarkers;
            for (size_t i = 0; i < ins.size(); i++) markers.push_back(names[i]);
            for (size_t i = 0; i < ins.size(); i++) cmarkers.push_back(names[i]);
            const std::string src = expr->to_cl_source(markers);
            custos_hip_kernel* k = nullptr;
            dev.check(custos_hip_expr_compile(dev.dev_, CUSTOS_HIP_KIND_APPLY, HipDType<T>::value, src.c_str(),
                                              cmarkers.data(), static_cast<int32_t>(cmarkers.size()), &k));
            uint64_t ptrs[4];
            for (size_t i = 0; i < ins.size(); i++) ptrs[i] = ins[i].ptr();
            dev.check(custos_hip_apply_fn_n(dev.dev_, k, ptrs, static_cast<int32_t>(ins.size()), out.ptr(), out.len()));
        };
    }

    // ---- caller-written kernels ----

    // `device.launch_kernel(src, fn_name, grid, block, shared_mem, args)` and
    // `device.launch_kernel1d(len, src, fn_name, args)` (src/devices/cuda/cuda_device.rs:85-112).
    // Buffers pass their device address, numbers pass by value (`AsCudaCvoidPtr`,
    // src/devices/cuda/kernel_launch.rs:29-77).
    template <class... Args>
    void launch_kernel(const std::string& src, const char* fn_name, const uint32_t (&grid)[3], const uint32_t (&block)[3],
                       uint32_t shared_mem_bytes, const Args&... args) {
        custos_hip_kernel* k = nullptr;
        check(custos_hip_source_compile(dev_, src.c_str(), fn_name, &k));
        KernelArgs<sizeof...(Args)> packed(args...);
        check(custos_hip_source_launch(dev_, k, grid, block, shared_mem_bytes, packed.ptrs, packed.sizes,
                                       static_cast<int32_t>(sizeof...(Args))));
    }
    template <class... Args>
    void launch_kernel1d(size_t len, const std::string& src, const char* fn_name, const Args&... args) {
        custos_hip_kernel* k = nullptr;
        check(custos_hip_source_compile(dev_, src.c_str(), fn_name, &k));
        KernelArgs<sizeof...(Args)> packed(args...);
        check(custos_hip_source_launch1d(dev_, k, len, packed.ptrs, packed.sizes, static_cast<int32_t>(sizeof...(Args))));
    }

    // ---- Lazy hooks ----

    // `LazySetup::lazy_setup`.  The reference starts stream capture here and
    // keeps it open until the first run (src/devices/cuda/lazy.rs:59-72); this
    // device records only while the operations of a run are replayed, so that
    // allocation and eager work never land in the graph.
    void lazy_setup() {}

    // `LazyRun::run` (src/devices/cuda/lazy.rs:31-49): the first run of a given
    // operation list records it into a graph and instantiates it; every run
    // launches the graph once.  `version` changes whenever the recorded
    // operations change; then the graph is rebuilt.  The wait that ends the
    // reference's run is deferred to whatever next looks at the results (see
    // `set_run_waits`).
    template <class Replay>
    void lazy_run(uint64_t version, Replay replay) {
        if (!graph_ || graph_version_ != version) {
            if (graph_) {
                check(custos_hip_graph_destroy(dev_, graph_));
                graph_ = nullptr;
            }
            check(custos_hip_capture_begin(dev_));
            try {
                replay();
            } catch (...) {
                custos_hip_graph* dropped = nullptr;
                if (custos_hip_capture_end(dev_, &dropped) == CUSTOS_HIP_OK && dropped)
                    custos_hip_graph_destroy(dev_, dropped);
                throw;
            }
            check(custos_hip_capture_end(dev_, &graph_));
            graph_version_ = version;
            graph_builds_++;
        }
        check(custos_hip_graph_launch(dev_, graph_));
        if (run_waits_) check(custos_hip_sync(dev_));
    }

    // The reference's run returns after the stream has drained
    // (src/devices/cuda/lazy.rs:42-43).  Here a run returns once its graph is queued on
    // the device's one compute stream, and the wait is taken by whatever looks at the
    // results next: `read` (and everything built on it: `read_to_vec`, serialisation,
    // `Display`), `sync`, dropping the device; a `write` into a buffer of the program is a
    // copy on the same stream behind the run (it waits only for its own host range);
    // dropping a buffer returns its block to a pool whose reuse is ordered on that stream
    // too, or waits before the block goes back to the driver; re-recording a changed
    // program waits before its first allocation or transfer.  Device memory cannot be
    // reached from the host except through these calls, so a program sees the same values
    // whether the wait sits in `run` or there; what moves is the time `run` itself takes
    // and the call that reports a failure of the device (an error of the launch itself --
    // a dropped buffer, a rejected graph -- is still thrown by `run`).  Runs that follow
    // each other without looking at results queue back to back: a small program then costs
    // its kernels, not kernels + completion signal + wake-up + launch latency per run.
    // `set_run_waits(true)` restores the wait inside every run.
    void set_run_waits(bool waits) { run_waits_ = waits; }
    bool run_waits() const { return run_waits_; }

    // how often a run had to (re)record its graph, and the kernels in it
    uint64_t graph_builds() const { return graph_builds_; }
    size_t graph_kernel_nodes() const {
        size_t n = 0;
        if (graph_) custos_hip_graph_node_count(graph_, &n);
        return n;
    }

    // Launch shape of the generated kernels; zero fields are left to the library, which
    // chooses them per launch from the bytes it touches.
    void set_tuning(const custos_hip_tuning& tuning) { check(custos_hip_set_tuning(dev_, &tuning)); }
    // How literal values reach kernels (CUSTOS_HIP_LITERALS_*): by default the first set of values of an
    // expression is compiled in, later sets are launch parameters of one shared kernel.
    void set_literal_policy(int32_t policy) { check(custos_hip_set_literal_policy(dev_, policy)); }
    // What `eq` computes in kernels compiled from now on: `==` (CUSTOS_HIP_EQ_EXACT, the default, like the
    // reference's GPU kernels) or `<=` (CUSTOS_HIP_EQ_AS_CPU_EVAL, what the reference's CPU device evaluates).
    void set_eq_policy(int32_t policy) { check(custos_hip_set_eq_policy(dev_, policy)); }
    // (hiprtc compilations, cache hits) so far
    std::pair<uint64_t, uint64_t> cache_stats() const {
        uint64_t compiles = 0, hits = 0;
        custos_hip_cache_stats(dev_, &compiles, &hits);
        return {compiles, hits};
    }
    // Launches and graph nodes of 64 MiB and more so far: {not part of a chain, chain that stays in the
    // memory-side cache, chain that streams}.
    std::array<uint64_t, 3> launch_hint_stats() const {
        std::array<uint64_t, 3> s{};
        custos_hip_launch_hint_stats(dev_, &s[0], &s[1], &s[2]);
        return s;
    }
    // Longest recorded chain that is replayed as plain launches instead of a graph launch.
    void set_graph_direct_replay(int32_t max_nodes) { check(custos_hip_set_graph_direct_replay(dev_, max_nodes)); }
    // How built graphs order their nodes: CUSTOS_HIP_GRAPH_EDGES_LEVEL_JOINS, _PER_NODE or _CHAIN.
    void set_graph_edges(int32_t mode) { check(custos_hip_set_graph_edges(dev_, mode)); }
    // Whether a lazy run joins recorded apply launches with the apply launches that read their
    // output into one kernel (default: yes; every buffer still receives the same values).
    void set_graph_fusing(bool enabled) { check(custos_hip_set_graph_fusing(dev_, enabled ? 1 : 0)); }
    // How long the first run of a program may spend compiling kernels of joined launches (default 1000 ms);
    // what it does not get within that replays as the launches that were recorded.
    void set_graph_fusing_budget(uint32_t milliseconds) { check(custos_hip_set_graph_fusing_budget(dev_, milliseconds)); }
    // Recorded launches of the current graph that would have been joined, had the build got their kernel, and why not.
    std::pair<size_t, std::string> graph_unjoined() const {
        size_t launches = 0;
        const char* reason = "";
        if (graph_) custos_hip_graph_unjoined(graph_, &launches, &reason);
        return {launches, reason ? reason : ""};
    }
    // (hiprtc translation units compiled so far, milliseconds spent in them)
    std::pair<uint64_t, double> compile_stats() const {
        uint64_t units = 0;
        double ms = 0;
        custos_hip_compile_stats(dev_, &units, &ms);
        return {units, ms};
    }

    custos_hip_kernel* compile(int32_t kind, int32_t dtype, const std::string& src,
                               std::initializer_list<const char*> markers) {
        std::vector<const char*> m(markers);
        custos_hip_kernel* k = nullptr;
        check(custos_hip_expr_compile(dev_, kind, dtype, src.c_str(), m.data(), static_cast<int32_t>(m.size()), &k));
        return k;
    }

    void check(int32_t rc) {
        if (rc != CUSTOS_HIP_OK) throw Error(DeviceError::Backend, rc, custos_hip_last_error(dev_));
    }

   private:
    // argument values laid out for the launch call: 8 bytes of storage each
    template <size_t N>
    struct KernelArgs {
        uint64_t storage[N ? N : 1] = {};
        void* ptrs[N ? N : 1] = {};
        size_t sizes[N ? N : 1] = {};
        template <class... A>
        explicit KernelArgs(const A&... a) {
            size_t i = 0;
            (put(i++, a), ...);
        }
        template <class T>
        void put(size_t i, const Buffer<T, Self>& b) {
            storage[i] = b.ptr();
            ptrs[i] = &storage[i];
            sizes[i] = sizeof(uint64_t);
        }
        template <class V, class = std::enable_if_t<std::is_arithmetic_v<V>>>
        void put(size_t i, const V& v) {
            static_assert(sizeof(V) <= sizeof(uint64_t), "kernel argument too large");
            std::memcpy(&storage[i], &v, sizeof(V));
            ptrs[i] = &storage[i];
            sizes[i] = sizeof(V);
        }
    };

    custos_hip_device* dev_ = nullptr;
    custos_hip_graph* graph_ = nullptr;
    uint64_t graph_version_ = 0;
    uint64_t graph_builds_ = 0;
    bool run_waits_ = false;
};

}  // namespace custos
