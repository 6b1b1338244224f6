// Device handle, memory, zero fill and timing of the C ABI (include/custos_hip.h).
#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <thread>

#include "runtime.hpp"
#include "scratch_order.hpp"

namespace custos_hip {

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

const std::string& thread_last_error() { return g_last_error; }

bool g_single_gpu = false;

constexpr size_t kStagedReadMax = 64u << 10;  // reads and writes up to this size go through pinned staging memory
constexpr size_t kSignalledReadMax = 4u << 10;  // reads up to this size: the copy kernel also writes the wait's completion word
constexpr size_t kWriteSlots = 16;            // staging slots of short writes (the first slot of the block is the read's)

// Operand table of custos_hip_apply_fn_many_noalloc: device memory that belongs to the
// library's code object, so the entry point never allocates.  Every GPU the library runs on
// holds its own copy (64 KiB) at its own address until the process ends; `scratch` itself is
// only the host-side name of the symbol, the address on device d is g_scratch_ptr[d], looked
// up once per device when the first handle on that device is created.
constexpr size_t kScratchWords = 8192;
static __device__ __align__(256) unsigned long long scratch[kScratchWords];
constexpr int kMaxDevices = 64;
static unsigned long long* g_scratch_ptr[kMaxDevices];
// All handles on a GPU share that GPU's table, each launching on a stream of its own: an event
// per GPU orders calls through different handles (who waits and who records: ScratchOrder).  The
// mutex covers the look-up, and in the entry point everything from the wait to the event record,
// so that calls from several threads take turns.
static hipEvent_t g_scratch_event[kMaxDevices];
static ScratchOrder g_scratch_order[kMaxDevices];
static std::mutex g_scratch_mutex;
static_assert(kScratchWords * sizeof(unsigned long long) <= kStagedReadMax, "the table travels through one staging slot");

// With device `idx` current: the address of that device's copy of `scratch` (and, made with
// it, the event that orders the table's users).
static hipError_t scratch_address(int idx, unsigned long long** out) {
    if (idx < 0 || idx >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[idx]) {
        void* p = nullptr;
        hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        hipEvent_t event = nullptr;
        e = hipEventCreateWithFlags(&event, hipEventDisableTiming);
        if (e != hipSuccess) return e;
        g_scratch_event[idx] = event;
        g_scratch_ptr[idx] = static_cast<unsigned long long*>(p);
    }
    *out = g_scratch_ptr[idx];
    if (g_scratch_order[idx].handle_created()) {
        const auto* last_user = static_cast<const custos_hip_device*>(g_scratch_order[idx].last_user);
        hipError_t e = hipEventRecord(g_scratch_event[idx], last_user->stream);
        if (e != hipSuccess) {
            g_scratch_order[idx].handle_not_created();
            return e;
        }
    }
    return hipSuccess;
}

// Waits for the compute stream.  The blocking wait of the runtime takes about 9 us to
// notice that a job has finished -- three times the job itself for a small replayed
// graph, and a gap in front of the next launch for a large one.  So the stream writes a
// sequence number into pinned host memory behind the work, and the host polls that word.
// How long it polls follows the work: the wait remembers how long the last wait for the
// same work took (per graph when exactly the launch of a graph is waited for, else per
// stream).  A graph launch predicted to take milliseconds is slept through up to half a
// millisecond before its predicted end; the rest is polled with a pause instruction, for at least 2 ms
// and at least twice the prediction.  Only work that outlasts that window -- work nothing
// predicted -- ends in the blocking wait, where 9 us no longer matter.
static inline void cpu_pause() {
#if defined(__x86_64__) || defined(__i386__)
    __builtin_ia32_pause();
#else
    std::this_thread::yield();
#endif
}

// Polls the completion word until it holds `seq` (see above for how long).
static hipError_t poll_completion_word(custos_hip_device* dev, uint32_t seq) {
    using clock = std::chrono::steady_clock;
    using std::chrono::nanoseconds;
    custos_hip_graph* const graph = dev->graphs_since_wait == 1 && !dev->launches_since_wait ? dev->graph_since_wait : nullptr;
    const uint64_t predicted_ns = graph && graph->last_wait_ns ? graph->last_wait_ns : dev->last_wait_ns;
    const uint64_t window_ns = std::min<uint64_t>(std::max<uint64_t>(2000000, 2 * predicted_ns), 50000000);
    const auto start = clock::now();
    volatile uint32_t* flag = dev->done_flag;
    hipError_t result = hipSuccess;
    bool done = *flag == seq;
    // (only a prediction for exactly this work is slept on: a wrong one would add latency)
    if (graph && graph->last_wait_ns > 2000000) {
        const auto sleep_until = start + nanoseconds(graph->last_wait_ns - 500000);
        while (!done && clock::now() < sleep_until) {
            std::this_thread::sleep_for(std::min<nanoseconds>(nanoseconds(1000000), sleep_until - clock::now()));
            done = *flag == seq;
        }
    }
    for (unsigned spins = 0; !done; spins++) {
        cpu_pause();
        done = *flag == seq;
        if (!done && (spins & 63) == 63 && clock::now() - start > nanoseconds(window_ns)) {
            result = hipStreamSynchronize(dev->stream);
            break;
        }
    }
    const uint64_t took = static_cast<uint64_t>(std::chrono::duration_cast<nanoseconds>(clock::now() - start).count());
    dev->last_wait_ns = took;
    if (graph) graph->last_wait_ns = took;
    dev->graph_since_wait = nullptr;
    dev->graphs_since_wait = 0;
    dev->launches_since_wait = false;
    return result;
}

static hipError_t wait_compute_stream_now(custos_hip_device* dev) {
    if (!dev->done_flag) return hipStreamSynchronize(dev->stream);
    const uint32_t seq = ++dev->done_seq;
    hipError_t e = hipStreamWriteValue32(dev->stream, dev->done_flag_dev, seq, 0);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return hipStreamSynchronize(dev->stream);
    }
    return poll_completion_word(dev, seq);
}

// `waits_begun` / `waits_done` number the waits: work issued while `waits_begun` was w has
// finished once `waits_done` is above w (what the staging slots of short writes go by).
hipError_t wait_compute_stream(custos_hip_device* dev) {
    const uint64_t mine = ++dev->waits_begun;
    hipError_t e = wait_compute_stream_now(dev);
    if (e == hipSuccess) dev->waits_done = mine;
    return e;
}

// Recording begins without a wait (custos_hip_capture_begin), so that a caller who records
// right after launching a graph does not drain the stream between two runs.  What still runs
// at once while the device records -- allocation with its zero fill, reads, writes, a free
// that goes back to the driver -- uses the transfer stream or the driver, outside the compute
// stream's order: the first of them takes the wait for the work that was in flight when the
// recording began (nothing is launched on the compute stream while recording, so one wait is
// enough).
hipError_t drain_before_immediate_work(custos_hip_device* dev) {
    if (!dev->undrained_at_capture) return hipSuccess;
    hipError_t e = wait_compute_stream(dev);
    if (e == hipSuccess) dev->undrained_at_capture = false;
    return e;
}

// ---- zero fill: 16-byte stores over the aligned body, bytes at the edges ----
//
// Tiles of 128 threads x 2 vectors, one tile per workgroup: 6.56 TB/s over 1 GiB and
// 6.66 over 64 MiB on MI355X, against 5.6 / 6.5 for 256-thread workgroups that loop
// over 8 vectors per thread, 5.9-6.0 for one vector per thread, and 6.4-6.6 for
// hipMemsetAsync (which may not be recorded into graphs here).

constexpr unsigned int kFillBlock = 128, kFillUnroll = 2;

__global__ void __launch_bounds__(kFillBlock) custos_fill_zero(unsigned char* p, unsigned long long bytes,
                                                               unsigned long long head,
                                                               unsigned long long n_vec) {
    typedef unsigned int u4 __attribute__((ext_vector_type(4)));
    u4* v = reinterpret_cast<u4*>(p + head);
    const u4 z = {0u, 0u, 0u, 0u};
    const unsigned long long tile_vecs = (unsigned long long)kFillBlock * kFillUnroll;
    const unsigned long long n_tiles = (n_vec + tile_vecs - 1) / tile_vecs;
    for (unsigned long long tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
#pragma unroll
        for (unsigned int u = 0; u < kFillUnroll; u++) {
            const unsigned long long i = tile * tile_vecs + (unsigned long long)u * kFillBlock + threadIdx.x;
            if (i < n_vec) v[i] = z;
        }
    }
    const unsigned long long gid = (unsigned long long)blockIdx.x * kFillBlock + threadIdx.x;
    const unsigned long long n_threads = (unsigned long long)gridDim.x * kFillBlock;
    if (gid < head) p[gid] = 0;
    for (unsigned long long i = head + n_vec * 16 + gid; i < bytes; i += n_threads) p[i] = 0;
}

// The same walk with a 16-byte pattern instead of zeros (a value of 1, 2, 4, 8 or 16 bytes
// repeated): byte k of the pattern belongs at addresses that are k modulo 16, which is what
// the aligned body stores; the bytes at the edges pick theirs by address.
__device__ __forceinline__ unsigned char pattern_byte(unsigned int w0, unsigned int w1, unsigned int w2, unsigned int w3,
                                                      unsigned long long address) {
    const unsigned int k = static_cast<unsigned int>(address & 15);
    const unsigned int word = k < 4 ? w0 : k < 8 ? w1 : k < 12 ? w2 : w3;
    return static_cast<unsigned char>(word >> ((k & 3) * 8));
}

__global__ void __launch_bounds__(kFillBlock) custos_fill_pattern(unsigned char* p, unsigned long long bytes,
                                                                  unsigned long long head, unsigned long long n_vec,
                                                                  unsigned int w0, unsigned int w1, unsigned int w2,
                                                                  unsigned int w3) {
    typedef unsigned int u4 __attribute__((ext_vector_type(4)));
    u4* v = reinterpret_cast<u4*>(p + head);
    const u4 pattern = {w0, w1, w2, w3};
    const unsigned long long tile_vecs = (unsigned long long)kFillBlock * kFillUnroll;
    const unsigned long long n_tiles = (n_vec + tile_vecs - 1) / tile_vecs;
    for (unsigned long long tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
#pragma unroll
        for (unsigned int u = 0; u < kFillUnroll; u++) {
            const unsigned long long i = tile * tile_vecs + (unsigned long long)u * kFillBlock + threadIdx.x;
            if (i < n_vec) v[i] = pattern;
        }
    }
    const unsigned long long gid = (unsigned long long)blockIdx.x * kFillBlock + threadIdx.x;
    const unsigned long long n_threads = (unsigned long long)gridDim.x * kFillBlock;
    const unsigned long long base = reinterpret_cast<unsigned long long>(p);
    if (gid < head) p[gid] = pattern_byte(w0, w1, w2, w3, base + gid);
    for (unsigned long long i = head + n_vec * 16 + gid; i < bytes; i += n_threads)
        p[i] = pattern_byte(w0, w1, w2, w3, base + i);
}

// Short copies between device memory and pinned host memory (the staging of short reads and
// writes): source and destination at the same 16-byte phase, 16-byte vectors over the aligned
// body, bytes at the edges.  Compiled with the library, so that a first read or write does
// not wait for a run-time compilation.
__global__ void __launch_bounds__(kFillBlock) custos_stage_copy(unsigned char* dst, const unsigned char* src,
                                                                unsigned long long bytes, unsigned long long head,
                                                                unsigned long long n_vec) {
    typedef unsigned int u4 __attribute__((ext_vector_type(4)));
    u4* d = reinterpret_cast<u4*>(dst + head);
    const u4* s = reinterpret_cast<const u4*>(src + head);
    const unsigned long long gid = (unsigned long long)blockIdx.x * kFillBlock + threadIdx.x;
    const unsigned long long n_threads = (unsigned long long)gridDim.x * kFillBlock;
    for (unsigned long long i = gid; i < n_vec; i += n_threads) d[i] = s[i];
    if (gid < head) dst[gid] = src[gid];
    for (unsigned long long i = head + n_vec * 16 + gid; i < bytes; i += n_threads) dst[i] = src[i];
}

// The same copy by ONE workgroup that writes the completion word of the wait itself when it is
// done (a few KiB at most: what a caller reads back between launches is a loss value, a
// handful of parameters).  The word is written behind the data: all copies of the workgroup,
// a fence to system scope, then the store, which travels the same way to host memory as the data.
__global__ void __launch_bounds__(kFillBlock) custos_stage_copy_and_signal(unsigned char* dst, const unsigned char* src,
                                                                           unsigned long long bytes, unsigned long long head,
                                                                           unsigned long long n_vec, unsigned int* word,
                                                                           unsigned int seq) {
    typedef unsigned int u4 __attribute__((ext_vector_type(4)));
    u4* d = reinterpret_cast<u4*>(dst + head);
    const u4* s = reinterpret_cast<const u4*>(src + head);
    for (unsigned long long i = threadIdx.x; i < n_vec; i += kFillBlock) d[i] = s[i];
    if (threadIdx.x < head) dst[threadIdx.x] = src[threadIdx.x];
    for (unsigned long long i = head + n_vec * 16 + threadIdx.x; i < bytes; i += kFillBlock) dst[i] = src[i];
    __threadfence_system();
    __syncthreads();
    if (threadIdx.x == 0) __hip_atomic_store(word, seq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

// `dst` and `src` at the same 16-byte phase; runs on the compute stream, never recorded.
static int32_t launch_stage_copy(custos_hip_device* dev, uint64_t dst, uint64_t src, size_t bytes) {
    unsigned long long head = (16 - (dst & 15)) & 15;
    if (head > bytes) head = bytes;
    const unsigned long long n_vec = (bytes - head) / 16;
    const unsigned int grid = static_cast<unsigned int>(std::max(1ull, (n_vec + kFillBlock - 1) / kFillBlock));
    dev->launches_since_wait = true;
    hipLaunchKernelGGL(custos_stage_copy, dim3(grid), dim3(kFillBlock), 0, dev->stream,
                       reinterpret_cast<unsigned char*>(dst), reinterpret_cast<const unsigned char*>(src),
                       static_cast<unsigned long long>(bytes), head, n_vec);
    HIP_TRY(dev, hipGetLastError());
    return CUSTOS_HIP_OK;
}

// A short write costs the runtime about 14 us, most of it the wait that lets the caller
// reuse `src`.  Up to 64 KiB the data is copied into a pinned staging slot (at the
// destination's 16-byte phase) and a copy kernel moves it from there, in stream
// order and without a wait; a slot is reused once a wait that began after its launch has
// finished, and a seventeenth write in a row without one waits first.
// Needs the staging memory, at most kStagedReadMax bytes, and a device that is not recording.
// The next staging slot, free to be filled: host address and device address of its byte 0 at
// the 16-byte phase of `dst`.
static int32_t staging_slot(custos_hip_device* dev, uint64_t dst, unsigned char** host, uint64_t* device) {
    const size_t slot = dev->write_slot;
    static_assert(kWriteSlots == std::tuple_size<decltype(dev->write_slot_issued)>::value, "one entry per slot");
    if (dev->write_slot_used[slot] && dev->waits_done <= dev->write_slot_issued[slot])
        HIP_TRY(dev, wait_compute_stream(dev));
    const size_t offset = (kStagedReadMax + 16) * (1 + slot) + (dst & 15);
    *host = dev->read_stage + offset;
    *device = dev->read_stage_dev + offset;
    return CUSTOS_HIP_OK;
}

// Launches the copy of `bytes` bytes from the slot staging_slot handed out to `dst`.
static int32_t staging_slot_send(custos_hip_device* dev, uint64_t dst, uint64_t slot_device, size_t bytes) {
    int32_t rc = launch_stage_copy(dev, dst, slot_device, bytes);
    if (rc != CUSTOS_HIP_OK) return rc;
    const size_t slot = dev->write_slot;
    dev->write_slot_issued[slot] = dev->waits_begun;
    dev->write_slot_used[slot] = true;
    dev->write_slot = (slot + 1) % kWriteSlots;
    return CUSTOS_HIP_OK;
}

int32_t staged_write(custos_hip_device* dev, uint64_t dst, const void* src, size_t bytes) {
    unsigned char* host = nullptr;
    uint64_t device = 0;
    int32_t rc = staging_slot(dev, dst, &host, &device);
    if (rc != CUSTOS_HIP_OK) return rc;
    std::memcpy(host, src, bytes);
    return staging_slot_send(dev, dst, device, bytes);
}

// Host data the library itself sends (the operand table of a graph): in stream order through the
// staging slots when the device has them and the data is small -- the runtime's synchronous copy
// costs 9 ms the first time a process uses it, more than the rest of a small graph's build --
// else with that copy.  `src` may be reused when this returns.
int32_t send_to_device(custos_hip_device* dev, uint64_t dst, const void* src, size_t bytes) {
    constexpr size_t kThroughSlotsMax = 1u << 20;
    if (!dev->read_stage || bytes > kThroughSlotsMax) {
        HIP_TRY(dev, hipMemcpy(reinterpret_cast<void*>(dst), src, bytes, hipMemcpyHostToDevice));
        return CUSTOS_HIP_OK;
    }
    for (size_t done = 0; done < bytes; done += kStagedReadMax) {
        int32_t rc = staged_write(dev, dst + done, static_cast<const unsigned char*>(src) + done, std::min(kStagedReadMax, bytes - done));
        if (rc != CUSTOS_HIP_OK) return rc;
    }
    return CUSTOS_HIP_OK;
}

unsigned int fill_grid(custos_hip_device* dev, unsigned long long n_vec) {
    (void)dev;
    const unsigned long long tile_vecs = (unsigned long long)kFillBlock * kFillUnroll;
    const unsigned long long tiles = (n_vec + tile_vecs - 1) / tile_vecs;
    return static_cast<unsigned int>(std::max(1ull, std::min(tiles, 1ull << 22)));
}

// ---- device-to-device copy ----
//
// A copy is the identity expression: it runs through the generated kernel for `x`
// over 4-byte (or 1-byte) elements and so gets the launch shape, the recording and the
// merging of every other launch; the runtime's hipMemcpyAsync moves 1 GiB at 5.06 TB/s
// on MI355X, the identity kernel at 6.4-6.8 TB/s.  Only byte-granular ranges whose
// source and destination sit at different 16-byte phases go through the runtime.

int32_t launch_copy(custos_hip_device* dev, uint64_t dst, uint64_t src, size_t bytes) {
    const bool words = ((dst | src | bytes) & 3) == 0;
    if (!words && ((dst ^ src) & 15) != 0) {
        if (dev->capturing) {
            stop_matching(dev);
            RecNode node;
            node.type = RecNode::Copy;
            node.ptrs = {dst, src};
            node.bytes = bytes;
            node.acc = {{dst, dst + bytes, true}, {src, src + bytes, false}};
            dev->recorded.push_back(std::move(node));
            return CUSTOS_HIP_OK;
        }
        dev->launches_since_wait = true;
        HIP_TRY(dev, hipMemcpyAsync(reinterpret_cast<void*>(dst), reinterpret_cast<const void*>(src), bytes,
                                    hipMemcpyDeviceToDevice, dev->stream));
        return CUSTOS_HIP_OK;
    }
    custos_hip_kernel* k = nullptr;
    int32_t rc = identity_kernel(dev, words ? DType::U32 : DType::U8, &k);
    if (rc != CUSTOS_HIP_OK) return rc;
    return launch_or_record(dev, k, {{src, false}, {dst, true}}, words ? bytes / 4 : bytes);
}

// `pattern`: null for zeros, else the 16 bytes that repeat from any 16-byte boundary on.
int32_t launch_fill(custos_hip_device* dev, uint64_t dptr, size_t bytes, hipStream_t stream, const uint32_t* pattern) {
    unsigned long long head = (16 - (dptr & 15)) & 15;
    if (head > bytes) head = bytes;
    unsigned long long n_vec = (bytes - head) / 16;
    if (dev->capturing && stream == dev->stream) {
        if (dev->matching && dev->matched < dev->previous_recorded.size()) {
            const RecNode& was = dev->previous_recorded[dev->matched];
            const bool same_pattern = pattern ? was.pattern.size() == 4 && std::memcmp(was.pattern.data(), pattern, 16) == 0 : was.pattern.empty();
            if (was.type == RecNode::Fill && was.ptrs[0] == dptr && was.bytes == bytes && same_pattern) {
                dev->matched++;
                return CUSTOS_HIP_OK;
            }
        }
        stop_matching(dev);
        RecNode node;
        node.type = RecNode::Fill;
        node.ptrs = {dptr};
        node.bytes = bytes;
        node.head = head;
        node.n_vec = n_vec;
        if (pattern) node.pattern.assign(pattern, pattern + 4);
        node.acc = {{dptr, dptr + bytes, true}};
        dev->recorded.push_back(std::move(node));
        return CUSTOS_HIP_OK;
    }
    unsigned int grid = fill_grid(dev, n_vec);
    if (stream == dev->stream) dev->launches_since_wait = true;
    if (pattern)
        hipLaunchKernelGGL(custos_fill_pattern, dim3(grid), dim3(kFillBlock), 0, stream,
                           reinterpret_cast<unsigned char*>(dptr), static_cast<unsigned long long>(bytes), head, n_vec,
                           pattern[0], pattern[1], pattern[2], pattern[3]);
    else
        hipLaunchKernelGGL(custos_fill_zero, dim3(grid), dim3(kFillBlock), 0, stream,
                           reinterpret_cast<unsigned char*>(dptr), static_cast<unsigned long long>(bytes),
                           head, n_vec);
    HIP_TRY(dev, hipGetLastError());
    return CUSTOS_HIP_OK;
}

int32_t launch_fill_zero(custos_hip_device* dev, uint64_t dptr, size_t bytes, hipStream_t stream) {
    return launch_fill(dev, dptr, bytes, stream, nullptr);
}

void* fill_zero_kernel() { return reinterpret_cast<void*>(custos_fill_zero); }
void* fill_pattern_kernel() { return reinterpret_cast<void*>(custos_fill_pattern); }
unsigned int fill_block() { return kFillBlock; }

}  // namespace custos_hip

using namespace custos_hip;

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
    g_single_gpu = count == 1;
    if (idx < 0 || idx >= count)
        return set_error(nullptr, CUSTOS_HIP_ERR_INVALID_DEVICE_INDEX,
                         "device index " + std::to_string(idx) + " out of range: " + std::to_string(count) + " device(s)");
    // the deleter also releases what was created before a later step failed
    auto drop = [](custos_hip_device* d) {
        if (d->t0) (void)hipEventDestroy(d->t0);
        if (d->t1) (void)hipEventDestroy(d->t1);
        if (d->stream) (void)hipStreamDestroy(d->stream);
        if (d->transfer) (void)hipStreamDestroy(d->transfer);
        if (d->done_flag) (void)hipHostFree(d->done_flag);
        delete d;
    };
    std::unique_ptr<custos_hip_device, decltype(drop)> dev(new custos_hip_device, drop);
    dev->idx = idx;
    HIP_TRY(nullptr, hipSetDevice(idx));
    HIP_TRY(nullptr, hipGetDeviceProperties(&dev->props, idx));
    dev->arch = dev->props.gcnArchName;
    dev->tuning = normalize_tuning(0, 0, 0, 0, 0);
    HIP_TRY(nullptr, hipStreamCreateWithFlags(&dev->stream, hipStreamNonBlocking));
    HIP_TRY(nullptr, hipStreamCreateWithFlags(&dev->transfer, hipStreamNonBlocking));
    HIP_TRY(nullptr, hipEventCreate(&dev->t0));
    HIP_TRY(nullptr, hipEventCreate(&dev->t1));
    dev->pool_limit = dev->props.totalGlobalMem / 4;
    // (optional: without it only the allocation-free merged launch is unavailable)
    if (scratch_address(idx, &dev->scratch_table) != hipSuccess) {
        (void)hipGetLastError();
        dev->scratch_table = nullptr;
    }
    dev->noalloc_checker.reserve(kScratchWords / 2);  // so that the entry point that may not allocate finds its room
    for (auto& call : dev->noalloc_checked) call.operands.reserve(kScratchWords);
    // completion word for short waits (pinned, mapped host memory); optional
    void* flag = nullptr;
    if (hipHostMalloc(&flag, 64, hipHostMallocMapped) == hipSuccess) {
        void* flag_dev = nullptr;
        if (hipHostGetDevicePointer(&flag_dev, flag, 0) == hipSuccess) {
            dev->done_flag = static_cast<uint32_t*>(flag);
            dev->done_flag_dev = flag_dev;
            *dev->done_flag = 0;
            // staging for short reads, next to it (optional as well)
            void* stage = nullptr;
            void* stage_dev = nullptr;
            if (hipHostMalloc(&stage, (kStagedReadMax + 16) * (1 + kWriteSlots), hipHostMallocMapped) == hipSuccess) {
                if (hipHostGetDevicePointer(&stage_dev, stage, 0) == hipSuccess) {
                    dev->read_stage = static_cast<unsigned char*>(stage);
                    dev->read_stage_dev = reinterpret_cast<uint64_t>(stage_dev);
                } else {
                    (void)hipGetLastError();
                    (void)hipHostFree(stage);
                }
            } else {
                (void)hipGetLastError();
            }
        } else {
            (void)hipGetLastError();
            (void)hipHostFree(flag);
        }
    } else {
        (void)hipGetLastError();
    }
    *out = dev.release();
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_device_destroy(custos_hip_device* dev) {
    if (!dev) return CUSTOS_HIP_OK;
    (void)hipSetDevice(dev->idx);
    (void)hipStreamSynchronize(dev->stream);
    (void)hipStreamSynchronize(dev->transfer);
    if (dev->idx >= 0 && dev->idx < kMaxDevices) {
        // (its launches have finished: the next user of the table need not wait for this handle)
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        if (dev->scratch_table) g_scratch_order[dev->idx].handle_destroyed(dev);
    }
    for (custos_hip_graph* g : dev->graphs) destroy_graph(g);
    // every block of this handle goes back to the driver, pooled or still held by the caller
    for (auto& kv : dev->block_bytes)
        if (kv.second.slab < 0) (void)hipFree(reinterpret_cast<void*>(kv.first));
    for (const custos_hip_device::Slab& slab : dev->slabs)
        if (slab.base) (void)hipFree(reinterpret_cast<void*>(slab.base));
    for (auto& bucket : dev->cache)
        for (auto& k : bucket.second)
            for (hipModule_t module : k->modules)
                if (module) (void)hipModuleUnload(module);
    (void)hipEventDestroy(dev->t0);
    (void)hipEventDestroy(dev->t1);
    for (hipEvent_t mark : dev->marks)
        if (mark) (void)hipEventDestroy(mark);
    (void)hipStreamDestroy(dev->stream);
    (void)hipStreamDestroy(dev->transfer);
    if (dev->done_flag) (void)hipHostFree(dev->done_flag);
    if (dev->read_stage) (void)hipHostFree(dev->read_stage);
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
    return dev ? dev->last_error.c_str() : thread_last_error().c_str();
}

int32_t custos_hip_sync(custos_hip_device* dev) {
    REQUIRE_DEV(dev);
    // While the device records nothing new reaches the compute stream: the wait is for the
    // work that was in flight when the recording began.
    if (dev->capturing) {
        HIP_TRY(dev, drain_before_immediate_work(dev));
        return CUSTOS_HIP_OK;
    }
    HIP_TRY(dev, wait_compute_stream(dev));
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_set_tuning(custos_hip_device* dev, const custos_hip_tuning* tuning) {
    REQUIRE_DEV(dev);
    dev->tuning = tuning_from_c(tuning);
    dev->compile_epoch++;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_get_tuning(custos_hip_device* dev, custos_hip_tuning* tuning) {
    REQUIRE_DEV(dev);
    if (!tuning) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "tuning is null");
    tuning->block_threads = dev->tuning.block_threads;
    tuning->unroll = dev->tuning.unroll;
    tuning->blocks_per_cu = dev->tuning.blocks_per_cu;
    tuning->nontemporal = dev->tuning.nontemporal < 0 ? 0 : dev->tuning.nontemporal == 0 ? -1 : dev->tuning.nontemporal;
    tuning->direction = dev->tuning.direction;
    return CUSTOS_HIP_OK;
}

// ---- memory ----

// Sizes are rounded so that buffers of similar length share pool entries:
// 512 B steps below 1 MiB, 2 MiB steps above (hipMalloc hands out 2 MiB
// granules for large blocks anyway).
static size_t pool_size_class(size_t bytes) {
    const size_t step = bytes < (1u << 20) ? 512 : (2u << 20);
    return (bytes + step - 1) / step * step;
}

constexpr size_t kSlabBytes = 4u << 20;        // blocks of up to kSlabBlockMax bytes are cut from allocations of this size
constexpr size_t kSlabBlockMax = 256u << 10;

// A block whose registry entry was `block` goes back to the driver (the work that used it has
// finished): an allocation of its own at once, a block of a slab together with the slab's last one.
static void give_back(custos_hip_device* dev, uint64_t addr, const custos_hip_device::Block& block) {
    if (block.slab < 0) {
        (void)hipFree(reinterpret_cast<void*>(addr));
        return;
    }
    custos_hip_device::Slab& slab = dev->slabs[static_cast<size_t>(block.slab)];
    if (--slab.blocks > 0) return;
    (void)hipFree(reinterpret_cast<void*>(slab.base));
    slab = custos_hip_device::Slab{};
    if (dev->open_slab == block.slab) dev->open_slab = -1;
}

static void release_pool(custos_hip_device* dev) {
    (void)hipStreamSynchronize(dev->stream);
    for (auto& kv : dev->pool)
        for (void* p : kv.second) {
            const uint64_t addr = reinterpret_cast<uint64_t>(p);
            const custos_hip_device::Block block = dev->block_bytes[addr];
            dev->block_bytes.erase(addr);
            give_back(dev, addr, block);
        }
    dev->pool.clear();
    dev->pooled_bytes = 0;
}

// A new block of `rounded` bytes cut from the open slab, or from a new one (zero-filled as a
// whole: `*zeroed` tells the caller that the block needs no fill of its own).  0 when no slab
// could be made; the caller then allocates the block by itself.
static uint64_t cut_from_slab(custos_hip_device* dev, size_t rounded, bool* zeroed) {
    *zeroed = false;
    if (dev->open_slab < 0 || dev->slabs[static_cast<size_t>(dev->open_slab)].used + rounded > kSlabBytes) {
        void* base = nullptr;
        if (hipMalloc(&base, kSlabBytes) != hipSuccess) {
            (void)hipGetLastError();
            return 0;
        }
        // (zeros once, in the order every other fill of an allocation has: the compute stream, or,
        // while the device records, the transfer stream and a wait)
        hipStream_t s = dev->capturing ? dev->transfer : dev->stream;
        int32_t rc = launch_fill_zero(dev, reinterpret_cast<uint64_t>(base), kSlabBytes, s);
        if (rc == CUSTOS_HIP_OK && dev->capturing && hipStreamSynchronize(dev->transfer) != hipSuccess) rc = CUSTOS_HIP_ERR_INVALID_ARGUMENT;
        if (rc != CUSTOS_HIP_OK) {
            (void)hipGetLastError();
            (void)hipFree(base);
            return 0;
        }
        // (the slab that was open keeps its blocks and goes when the last of them does; the entry of
        // a slab that is gone is used again)
        custos_hip_device::Slab slab;
        slab.base = reinterpret_cast<uint64_t>(base);
        slab.bytes = kSlabBytes;
        size_t index = 0;
        while (index < dev->slabs.size() && dev->slabs[index].base != 0) index++;
        if (index == dev->slabs.size()) dev->slabs.push_back(slab);
        else dev->slabs[index] = slab;
        dev->open_slab = static_cast<int32_t>(index);
    }
    custos_hip_device::Slab& slab = dev->slabs[static_cast<size_t>(dev->open_slab)];
    const uint64_t addr = slab.base + slab.used;
    slab.used += rounded;
    slab.blocks++;
    *zeroed = true;
    return addr;
}

int32_t custos_hip_alloc(custos_hip_device* dev, size_t bytes, int32_t flags, uint64_t* dptr) {
    REQUIRE_DEV(dev);
    if (!dptr) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "dptr is null");
    *dptr = 0;
    if (bytes == 0) return set_error(dev, CUSTOS_HIP_ERR_ZERO_LENGTH_BUFFER, "zero length buffers are not supported");
    const size_t rounded = pool_size_class(bytes);
    void* p = nullptr;
    bool already_zero = false;  // a block newly cut from a slab: the slab was zero-filled when it was made
    if (dev->capturing && flags != CUSTOS_HIP_ALLOC_UNINIT) HIP_TRY(dev, drain_before_immediate_work(dev));
    auto pooled = dev->pool.find(rounded);
    if (pooled != dev->pool.end() && !pooled->second.empty()) {
        p = pooled->second.back();
        pooled->second.pop_back();
        dev->pooled_bytes -= rounded;
        dev->pool_reused++;
        dev->block_bytes[reinterpret_cast<uint64_t>(p)].pooled = false;
    } else {
        bool zeroed = false;
        const uint64_t cut = rounded <= kSlabBlockMax ? cut_from_slab(dev, rounded, &zeroed) : 0;
        if (cut) {
            p = reinterpret_cast<void*>(cut);
            dev->block_bytes[cut] = {rounded, false, dev->open_slab};
            already_zero = zeroed;
        } else {
            hipError_t e = hipMalloc(&p, rounded);
            if (e != hipSuccess && dev->pooled_bytes > 0) {
                (void)hipGetLastError();
                release_pool(dev);  // the pool may hold what this allocation needs
                e = hipMalloc(&p, rounded);
            }
            if (e != hipSuccess) return hip_fail(dev, e, "hipMalloc");
            dev->block_bytes[reinterpret_cast<uint64_t>(p)] = {rounded, false, -1};
        }
        dev->pool_allocated++;
    }
    uint64_t addr = reinterpret_cast<uint64_t>(p);
    if (flags != CUSTOS_HIP_ALLOC_UNINIT && !already_zero) {
        // While recording, the fill must run now and not become part of the graph.
        hipStream_t s = dev->capturing ? dev->transfer : dev->stream;
        int32_t rc = launch_fill_zero(dev, addr, bytes, s);
        if (rc == CUSTOS_HIP_OK && dev->capturing) {
            hipError_t e = hipStreamSynchronize(dev->transfer);
            if (e != hipSuccess) rc = hip_fail(dev, e, "hipStreamSynchronize(transfer)");
        }
        if (rc != CUSTOS_HIP_OK) {
            const custos_hip_device::Block block = dev->block_bytes[addr];
            dev->block_bytes.erase(addr);
            give_back(dev, addr, block);
            return rc;
        }
    }
    *dptr = addr;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_free(custos_hip_device* dev, uint64_t dptr) {
    REQUIRE_DEV(dev);
    if (dptr == 0) return CUSTOS_HIP_OK;
    auto known = dev->block_bytes.find(dptr);
    if (known == dev->block_bytes.end())
        return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "not the address of a block this device handle allocated");
    if (known->second.pooled)
        return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "the block was freed already");
    if (dev->pooled_bytes + known->second.bytes <= dev->pool_limit) {
        // Reuse is ordered on the compute stream behind whatever still uses the block.
        // (A recorded graph that names the address must not be replayed after this,
        // exactly as after a real free.)
        known->second.pooled = true;
        dev->pool[known->second.bytes].push_back(reinterpret_cast<void*>(dptr));
        dev->pooled_bytes += known->second.bytes;
        return CUSTOS_HIP_OK;
    }
    const custos_hip_device::Block block = known->second;
    dev->block_bytes.erase(known);
    // work that still uses the range must finish first
    if (!dev->capturing) HIP_TRY(dev, hipStreamSynchronize(dev->stream));
    else HIP_TRY(dev, drain_before_immediate_work(dev));
    give_back(dev, dptr, block);
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_set_pool_limit(custos_hip_device* dev, size_t limit_bytes) {
    REQUIRE_DEV(dev);
    dev->pool_limit = limit_bytes;
    if (dev->pooled_bytes > limit_bytes) release_pool(dev);
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_pool_trim(custos_hip_device* dev) {
    REQUIRE_DEV(dev);
    release_pool(dev);
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_pool_stats(custos_hip_device* dev, size_t* pooled_bytes, uint64_t* reused, uint64_t* allocated) {
    REQUIRE_DEV(dev);
    if (pooled_bytes) *pooled_bytes = dev->pooled_bytes;
    if (reused) *reused = dev->pool_reused;
    if (allocated) *allocated = dev->pool_allocated;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_write(custos_hip_device* dev, uint64_t dst, const void* src, size_t bytes) {
    REQUIRE_DEV(dev);
    if (bytes == 0) return CUSTOS_HIP_OK;
    if (!dst || !src) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "null pointer");
    if (dev->capturing) {
        HIP_TRY(dev, drain_before_immediate_work(dev));
        HIP_TRY(dev, hipMemcpyAsync(reinterpret_cast<void*>(dst), src, bytes, hipMemcpyHostToDevice, dev->transfer));
        HIP_TRY(dev, hipStreamSynchronize(dev->transfer));
        return CUSTOS_HIP_OK;
    }
    if (dev->read_stage && bytes <= kStagedReadMax) return staged_write(dev, dst, src, bytes);
    HIP_TRY(dev, hipMemcpyAsync(reinterpret_cast<void*>(dst), src, bytes, hipMemcpyHostToDevice, dev->stream));
    // the caller may reuse `src` right away
    HIP_TRY(dev, hipStreamSynchronize(dev->stream));
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_read(custos_hip_device* dev, void* dst, uint64_t src, size_t bytes) {
    REQUIRE_DEV(dev);
    if (bytes == 0) return CUSTOS_HIP_OK;
    if (!dst || !src) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "null pointer");
    // Not recording: the copy is ordered on the compute stream behind the work that produces
    // the data, one wait in all.  While recording nothing is in flight there, and the copy must
    // not become part of the recording: it goes through the transfer stream.
    // A short read costs the runtime about 20 us whatever its size.  Up to 64 KiB a copy
    // kernel stores the data into pinned host memory instead (at the source's 16-byte phase, so
    // that it moves whole vectors), and the host waits on the completion word: 4 bytes in
    // about 8 us.
    if (!dev->capturing && dev->read_stage && bytes <= kStagedReadMax) {
        const uint64_t phase = src & 15;
        if (bytes <= kSignalledReadMax) {
            // one dispatch instead of two: the copy's one workgroup ends with the completion word
            unsigned long long head = (16 - phase) & 15;
            if (head > bytes) head = bytes;
            const unsigned long long n_vec = (bytes - head) / 16;
            const uint64_t mine = ++dev->waits_begun;
            const uint32_t seq = ++dev->done_seq;
            hipLaunchKernelGGL(custos_stage_copy_and_signal, dim3(1), dim3(kFillBlock), 0, dev->stream,
                               reinterpret_cast<unsigned char*>(dev->read_stage_dev + phase), reinterpret_cast<const unsigned char*>(src),
                               static_cast<unsigned long long>(bytes), head, n_vec, static_cast<unsigned int*>(dev->done_flag_dev), seq);
            HIP_TRY(dev, hipGetLastError());
            HIP_TRY(dev, poll_completion_word(dev, seq));
            dev->waits_done = mine;
            std::memcpy(dst, dev->read_stage + phase, bytes);
            return CUSTOS_HIP_OK;
        }
        int32_t rc = launch_stage_copy(dev, dev->read_stage_dev + phase, src, bytes);
        if (rc != CUSTOS_HIP_OK) return rc;
        HIP_TRY(dev, wait_compute_stream(dev));
        std::memcpy(dst, dev->read_stage + phase, bytes);
        return CUSTOS_HIP_OK;
    }
    hipStream_t s = dev->capturing ? dev->transfer : dev->stream;
    if (dev->capturing) HIP_TRY(dev, drain_before_immediate_work(dev));
    HIP_TRY(dev, hipMemcpyAsync(dst, reinterpret_cast<const void*>(src), bytes, hipMemcpyDeviceToHost, s));
    HIP_TRY(dev, hipStreamSynchronize(s));
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_copy(custos_hip_device* dev, uint64_t dst, uint64_t src, size_t bytes) {
    REQUIRE_DEV(dev);
    if (bytes == 0) return CUSTOS_HIP_OK;
    if (!dst || !src) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "null pointer");
    return launch_copy(dev, dst, src, bytes);
}

int32_t custos_hip_clear(custos_hip_device* dev, uint64_t dptr, size_t bytes) {
    REQUIRE_DEV(dev);
    if (bytes == 0) return CUSTOS_HIP_OK;
    if (!dptr) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "null pointer");
    return launch_fill_zero(dev, dptr, bytes, dev->stream);
}

int32_t custos_hip_fill(custos_hip_device* dev, uint64_t dptr, size_t bytes, const void* value, size_t value_bytes) {
    REQUIRE_DEV(dev);
    if (bytes == 0) return CUSTOS_HIP_OK;
    if (!dptr || !value) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "null pointer");
    if (value_bytes == 0 || value_bytes > 16 || (value_bytes & (value_bytes - 1)) != 0)
        return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "a fill value has 1, 2, 4, 8 or 16 bytes");
    if (dptr % value_bytes != 0 || bytes % value_bytes != 0)
        return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "address and length of a fill are multiples of the value's size");
    unsigned char repeated[16];
    for (size_t k = 0; k < 16; k++) repeated[k] = static_cast<const unsigned char*>(value)[k % value_bytes];
    uint32_t pattern[4];
    std::memcpy(pattern, repeated, 16);
    const bool zeros = (pattern[0] | pattern[1] | pattern[2] | pattern[3]) == 0;
    return launch_fill(dev, dptr, bytes, dev->stream, zeros ? nullptr : pattern);
}

// ---- many launches of one kernel in one grid, without any allocation ----

}  // extern "C"

namespace custos_hip {

void OperandSetChecker::reserve(size_t max_sets) {
    size_t size = 16;
    while (size < 2 * max_sets) size *= 2;
    if (slots.size() < size) {
        slots.assign(size, Slot{0, 0, 0, 0});
        stamp = 0;
    }
}

int32_t OperandSetChecker::check(const uint64_t* operands, int n_ptrs, size_t n_sets, int written, uint64_t bytes, const char** why) {
    if (slots.size() < 2 || slots.size() < 2 * n_sets || bytes == 0 || written < 0 || written >= n_ptrs) {
        *why = "operand check called outside its limits";
        return CUSTOS_HIP_ERR_INVALID_ARGUMENT;
    }
    if (++stamp == 0) {  // (after 2^32 checks: every slot looks empty again)
        for (Slot& slot : slots) slot.stamp = 0;
        stamp = 1;
    }
    const size_t mask = slots.size() - 1;
    int shift = 64;
    for (size_t size = slots.size(); size > 1; size /= 2) shift--;
    auto home = [&](uint64_t piece) { return static_cast<size_t>((piece * 0x9e3779b97f4a7c15ull) >> shift); };
    // the rows one by one, and the written operand of each into the table
    for (size_t s = 0; s < n_sets; s++) {
        const uint64_t* row = operands + s * static_cast<size_t>(n_ptrs);
        const uint64_t out = row[written];
        for (int i = 0; i < n_ptrs; i++) {
            if (row[i] == 0) {
                *why = "null device pointer";
                return CUSTOS_HIP_ERR_INVALID_ARGUMENT;
            }
            if (row[i] & 15) {
                *why = "operands of a merged launch are 16-byte aligned";
                return CUSTOS_HIP_ERR_INVALID_ARGUMENT;
            }
            if (row[i] > UINT64_MAX - bytes) {
                *why = "an operand range wraps around the address space";
                return CUSTOS_HIP_ERR_INVALID_ARGUMENT;
            }
        }
        for (int i = 0; i < n_ptrs; i++)
            if (i != written && row[i] != out && row[i] < out + bytes && out < row[i] + bytes) {
                *why = "the output range partially overlaps an input range";
                return CUSTOS_HIP_ERR_BAD_OVERLAP;
            }
        const uint64_t piece = out / bytes;
        size_t at = home(piece);
        for (; slots[at].stamp == stamp; at = (at + 1) & mask)
            if (slots[at].piece == piece) {  // two written operands less than their length apart
                *why = "an operand set writes memory that another operand set uses";
                return CUSTOS_HIP_ERR_BAD_OVERLAP;
            }
        slots[at] = Slot{piece, out, static_cast<uint32_t>(s), stamp};
    }
    // every operand against the written operands of the other rows around it
    for (size_t s = 0; s < n_sets; s++) {
        const uint64_t* row = operands + s * static_cast<size_t>(n_ptrs);
        for (int i = 0; i < n_ptrs; i++) {
            const uint64_t a = row[i], piece = a / bytes;
            for (uint64_t p = piece == 0 ? 0 : piece - 1; p <= piece + 1; p++)
                for (size_t at = home(p); slots[at].stamp == stamp; at = (at + 1) & mask) {
                    if (slots[at].piece != p) continue;
                    const uint64_t w = slots[at].begin;
                    if (slots[at].set != s && w < a + bytes && a < w + bytes) {
                        *why = "an operand set writes memory that another operand set uses";
                        return CUSTOS_HIP_ERR_BAD_OVERLAP;
                    }
                    break;  // (one written operand per piece)
                }
        }
    }
    return CUSTOS_HIP_OK;
}

}  // namespace custos_hip

extern "C" {

int32_t custos_hip_check_operand_sets(const uint64_t* operands, int32_t operands_per_set, size_t n_sets, int32_t written,
                                      uint64_t bytes) {
    if (!operands || operands_per_set < 1 || written < 0 || written >= operands_per_set || bytes == 0)
        return CUSTOS_HIP_ERR_INVALID_ARGUMENT;
    if (n_sets == 0) return CUSTOS_HIP_OK;
    OperandSetChecker checker;
    checker.reserve(n_sets);
    const char* why = "";
    return checker.check(operands, operands_per_set, n_sets, written, bytes, &why);
}

int32_t custos_hip_apply_fn_many_noalloc(custos_hip_device* dev, custos_hip_kernel* kernel, const uint64_t* operands,
                                         int32_t operands_per_set, size_t n_sets, size_t n) {
    REQUIRE_DEV(dev);
    if (!kernel || !operands) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "null kernel or operand table");
    if (kernel->spec.kind == Kind::Source)
        return set_error(dev, CUSTOS_HIP_ERR_KIND_MISMATCH, "a caller-written kernel has no entry point for merged launches");
    // (loading code allocates: the entry point must be there already)
    const custos_hip_kernel* owner = kernel->code ? kernel->code : kernel;
    const hipFunction_t fn = owner->fns[static_cast<int>(EntrySet::Batched)];
    if (!fn)
        return set_error(dev, CUSTOS_HIP_ERR_NOT_PREPARED,
                         "the kernel's entry point for merged launches is not loaded: call custos_hip_kernel_prepare_merged "
                         "where allocation is allowed");
    if (dev->capturing)
        return set_error(dev, CUSTOS_HIP_ERR_CAPTURE_STATE, "the allocation-free merged launch cannot be recorded");
    const int n_ptrs = kernel->spec.kind == Kind::UnaryGrad ? 3 : kernel->spec.expr.n_vars + 1;
    if (operands_per_set != n_ptrs)
        return set_error(dev, CUSTOS_HIP_ERR_ARITY_MISMATCH,
                         "kernel takes " + std::to_string(n_ptrs) + " addresses per operand set, got " + std::to_string(operands_per_set));
    if (n_sets == 0 || n == 0) return CUSTOS_HIP_OK;
    if (!dev->read_stage || !dev->scratch_table)
        return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "the device handle has no staging memory for the operand table");
    if (n > (1ull << 40)) return set_error(dev, CUSTOS_HIP_ERR_TOO_LARGE, "more than 2^40 elements");
    const std::vector<unsigned char>& values = kernel->spec.consts.bytes;
    const size_t const_words = (values.size() + 7) / 8;
    const size_t row_words = static_cast<size_t>(n_ptrs) + const_words;
    if (n_sets > kScratchWords / row_words)
        return set_error(dev, CUSTOS_HIP_ERR_TOO_LARGE,
                         "the static operand table holds " + std::to_string(kScratchWords / row_words) + " operand sets of this kernel (" +
                             std::to_string(kScratchWords * 8) + " bytes), got " + std::to_string(n_sets));
    // Operand checks on the host, before anything is launched: aligned, no partial overlap
    // inside a set (`out == in` exactly is fine), and no set writes what another set touches.
    // Their work area was made when the handle was created.  A serving loop calls
    // with the same few tables again and again: the calls that passed last are kept, and a call
    // identical to one of them passes again without the checks.
    const uint64_t bytes = static_cast<uint64_t>(n) * dtype_size(kernel->spec.dtype);
    const size_t n_words = n_sets * static_cast<size_t>(n_ptrs);
    int known = -1;
    for (size_t c = 0; c < dev->noalloc_checked.size() && known < 0; c++) {
        const auto& call = dev->noalloc_checked[c];
        if (call.kernel == kernel && call.n == n && call.operands.size() == n_words &&
            std::memcmp(call.operands.data(), operands, n_words * 8) == 0)
            known = static_cast<int>(c);
    }
    if (known < 0) {
        const int written = kernel->spec.kind == Kind::UnaryGrad ? 1 : n_ptrs - 1;
        const char* why = "";
        const int32_t checked = dev->noalloc_checker.check(operands, n_ptrs, n_sets, written, bytes, &why);
        if (checked != CUSTOS_HIP_OK) return set_error(dev, checked, why);
        known = static_cast<int>(dev->noalloc_next);
        dev->noalloc_next = (dev->noalloc_next + 1) % dev->noalloc_checked.size();
        if (dev->noalloc_in_table == known) dev->noalloc_in_table = -1;
        auto& call = dev->noalloc_checked[static_cast<size_t>(known)];
        call.operands.assign(operands, operands + n_words);  // (within the reserved room: nothing is allocated)
        call.kernel = kernel;
        call.n = n;
    }
    const ResolvedShape shape = resolve_shape(dev, kernel, static_cast<unsigned long long>(n_sets) * n_ptrs * bytes);
    const unsigned long long count = n, n_vec = n / static_cast<unsigned long long>(kernel->spec.vec_elems);
    const unsigned long long tile_vecs = static_cast<unsigned long long>(shape.block) * shape.unroll;
    unsigned long long tiles_per_seg = std::max(1ull, (n_vec + tile_vecs - 1) / tile_vecs);
    if (tiles_per_seg * n_sets > (1ull << 31) - 1)
        return set_error(dev, CUSTOS_HIP_ERR_TOO_LARGE, "a merged launch would need more than 2^31 workgroups");

    // From here to the event record one caller at a time per process: the table has one copy per GPU.
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    // The launch of another handle may still be reading the table: this stream's work from here
    // on waits for it.  (The launches of this handle are ordered by its stream.)
    ScratchOrder& order = g_scratch_order[dev->idx];
    if (order.must_wait(dev)) HIP_TRY(dev, hipStreamWaitEvent(dev->stream, g_scratch_event[dev->idx], 0));
    // Table rows as the `_batched` entry point reads them (addresses, then the literal
    // parameters), written straight into a pinned staging slot; the library's copy kernel moves
    // them into the table on the compute stream, behind the previous call's launch.  Not needed
    // when the table still holds the rows of an identical call of this handle.
    const uint64_t table_dev = reinterpret_cast<uint64_t>(dev->scratch_table);
    if (!(dev->noalloc_in_table == known && order.still_holds_rows_of(dev))) {
        dev->noalloc_in_table = -1;
        unsigned char* slot_host = nullptr;
        uint64_t slot_dev = 0;
        int32_t rc = staging_slot(dev, table_dev, &slot_host, &slot_dev);
        if (rc != CUSTOS_HIP_OK) return rc;
        uint64_t* table = reinterpret_cast<uint64_t*>(slot_host);  // (the table is 256-byte aligned: phase 0)
        for (size_t s = 0; s < n_sets; s++) {
            uint64_t* row = table + s * row_words;
            std::memcpy(row, operands + s * static_cast<size_t>(n_ptrs), static_cast<size_t>(n_ptrs) * 8);
            for (size_t w = 0; w < const_words; w++) {
                uint64_t word = 0;
                std::memcpy(&word, values.data() + w * 8, std::min<size_t>(8, values.size() - w * 8));
                row[n_ptrs + w] = word;
            }
        }
        rc = staging_slot_send(dev, table_dev, slot_dev, n_sets * row_words * 8);
        if (rc != CUSTOS_HIP_OK) return rc;
    }
    unsigned long long mode = launch_mode(shape.unroll, shape.nontemporal, false, shape.block);
    uint64_t table_arg = table_dev;
    unsigned long long count_arg = count, n_vec_arg = n_vec;
    void* args[] = {&table_arg, &count_arg, &n_vec_arg, &tiles_per_seg, &mode};
    dev->launches_since_wait = true;
    HIP_TRY(dev, hipModuleLaunchKernel(fn, static_cast<unsigned int>(tiles_per_seg * n_sets), 1, 1,
                                       static_cast<unsigned int>(shape.block), 1, 1, 0, dev->stream, args, nullptr));
    if (order.launched(dev)) HIP_TRY(dev, hipEventRecord(g_scratch_event[dev->idx], dev->stream));
    dev->noalloc_in_table = known;
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_kernel_prepare_merged(custos_hip_device* dev, custos_hip_kernel* kernel) {
    REQUIRE_DEV(dev);
    if (!kernel) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "null kernel");
    hipFunction_t fn = nullptr;
    return entry_point(dev, kernel, EntrySet::Batched, &fn);
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

// Numbered marks for per-step timing: an event per index, created on first use.
int32_t custos_hip_timer_mark(custos_hip_device* dev, uint32_t index) {
    REQUIRE_DEV(dev);
    if (index >= 4096) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "timer marks are numbered 0..4095");
    if (dev->capturing) return set_error(dev, CUSTOS_HIP_ERR_CAPTURE_STATE, "cannot time a recording stream");
    if (dev->marks.size() <= index) dev->marks.resize(index + 1, nullptr);
    if (!dev->marks[index]) HIP_TRY(dev, hipEventCreate(&dev->marks[index]));
    HIP_TRY(dev, hipEventRecord(dev->marks[index], dev->stream));
    return CUSTOS_HIP_OK;
}

int32_t custos_hip_timer_between(custos_hip_device* dev, uint32_t first, uint32_t second, double* ms) {
    REQUIRE_DEV(dev);
    if (!ms) return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "ms is null");
    if (first >= dev->marks.size() || second >= dev->marks.size() || !dev->marks[first] || !dev->marks[second])
        return set_error(dev, CUSTOS_HIP_ERR_INVALID_ARGUMENT, "a timer mark that was never recorded");
    HIP_TRY(dev, hipEventSynchronize(dev->marks[second]));
    float f = 0.f;
    HIP_TRY(dev, hipEventElapsedTime(&f, dev->marks[first], dev->marks[second]));
    *ms = f;
    return CUSTOS_HIP_OK;
}

}  // extern "C"
