/*
 * custos_hip.h -- C ABI of the MI355X (gfx950) element-wise backend for custos.
 *
 * This is the boundary a custos `HIP<Mods>` device binds through FFI.  It
 * covers what the reference's CUDA device reaches through its own driver
 * wrappers (src/devices/cuda/api/ffi.rs:165-264, api/nvrtc/ffi.rs:36-54) for
 * the element-wise path: device memory, expression kernels compiled at run
 * time, the three launches (apply / two-operand apply / unary gradient) and
 * graph capture + replay for `Lazy`.
 *
 * Conventions
 *   - every function returns a status: 0 on success, a HIP error number
 *     (hipError_t, 1..9999) or a library code (>= 10000, see below).
 *     `custos_hip_last_error` returns a message for the last failure.
 *   - handles are opaque; a device handle and everything created from it is
 *     used by one thread at a time (the reference's devices are `!Sync`:
 *     RefCell state in src/devices/cuda/cuda_device.rs:14-29).
 *   - device pointers are `uint64_t` addresses, so a buffer id can be the
 *     address as in src/devices/cuda/cuda_ptr.rs:44-49.  Sub-ranges of an
 *     allocation (address + offset) are accepted wherever a pointer is.
 *   - all work is issued on the device handle's compute stream, in call order.
 */
#ifndef CUSTOS_HIP_H
#define CUSTOS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct custos_hip_device custos_hip_device;
typedef struct custos_hip_kernel custos_hip_kernel;
typedef struct custos_hip_graph custos_hip_graph;

/* Library status codes (HIP's own error numbers stay below 10000). */
enum custos_hip_status {
    CUSTOS_HIP_OK = 0,
    CUSTOS_HIP_ERR_INVALID_ARGUMENT = 10001,
    /* zero-byte allocation: src/devices/cuda/api/cuda.rs:69-71,
     * DeviceError::ZeroLengthBuffer (src/error.rs) */
    CUSTOS_HIP_ERR_ZERO_LENGTH_BUFFER = 10002,
    /* device index out of range: src/devices/cuda/api/cuda.rs:36-39 */
    CUSTOS_HIP_ERR_INVALID_DEVICE_INDEX = 10003,
    CUSTOS_HIP_ERR_EXPR_SYNTAX = 10010,      /* expression text does not follow the grammar */
    CUSTOS_HIP_ERR_EXPR_UNKNOWN_MARKER = 10011,
    CUSTOS_HIP_ERR_EXPR_UNSUPPORTED = 10012, /* node not defined for the element type */
    CUSTOS_HIP_ERR_COMPILE = 10020,          /* hiprtc rejected the generated kernel */
    CUSTOS_HIP_ERR_KIND_MISMATCH = 10030,    /* kernel launched through the wrong entry point */
    CUSTOS_HIP_ERR_ARITY_MISMATCH = 10031,
    CUSTOS_HIP_ERR_NOT_PREPARED = 10032,     /* an entry point that may not load code was called before the code was loaded */
    CUSTOS_HIP_ERR_CAPTURE_STATE = 10040,    /* begin while capturing / end while not / op illegal in capture */
    CUSTOS_HIP_ERR_GRAPH_ORDER = 10041,      /* the ordering check of a built graph failed (custos_hip_set_graph_verify) */
    CUSTOS_HIP_ERR_BAD_OVERLAP = 10050,      /* output partially overlaps an input */
    CUSTOS_HIP_ERR_TOO_LARGE = 10060
};

/* Element types: the reference's CDatatype list (src/devices/cdatatype.rs:7-62).
 * F16 / BF16 are storage types: values are widened to f32, the whole expression
 * is computed in f32 and rounded once (nearest even) at the store. */
enum custos_hip_dtype {
    CUSTOS_HIP_F32 = 0,
    CUSTOS_HIP_F64 = 1,
    CUSTOS_HIP_I32 = 2,
    CUSTOS_HIP_I64 = 3,
    CUSTOS_HIP_F16 = 4,
    CUSTOS_HIP_BF16 = 5,
    CUSTOS_HIP_U8 = 6,
    CUSTOS_HIP_I8 = 7,
    CUSTOS_HIP_I16 = 8,
    CUSTOS_HIP_U16 = 9,
    CUSTOS_HIP_U32 = 10,
    CUSTOS_HIP_U64 = 11,
    /* The same storage as F16 / BF16, but every node of the expression is rounded to the
     * storage type (constants included), the product of the gradient kernel too: what the
     * reference's `half` arithmetic computes on the CPU and native half arithmetic on a GPU
     * (src/number.rs:487-676, src/devices/cdatatype.rs:53-62). */
    CUSTOS_HIP_F16_PERNODE = 12,
    CUSTOS_HIP_BF16_PERNODE = 13
};

/* Kernel kinds. */
enum custos_hip_kind {
    /* out[i] = f(in0[i], .., in{k-1}[i]), k = number of markers (1..4).
     * One marker: `applyFn` (src/devices/cuda/ops.rs:144-177) and, when the
     * source is a statement list "x = ..;\n x = ..;\n", the fused unary chain
     * (src/devices/cuda/fusing.rs:21-48, src/devices/fusing.rs:4-19).
     * Two markers: the two-operand expressions of src/two_way_ops/mod.rs:96-104. */
    CUSTOS_HIP_KIND_APPLY = 0,
    /* lhs_grad[i] += out_grad[i] * f(lhs[i]): `addUnaryGrad`
     * (src/devices/cuda/ops.rs:201-234). One marker. */
    CUSTOS_HIP_KIND_UNARY_GRAD = 1
};

/* Allocation flags. */
enum custos_hip_alloc_flags {
    CUSTOS_HIP_ALLOC_ZEROED = 0,  /* like CPU alloc (src/devices/cpu/cpu_ptr.rs:74-85) */
    CUSTOS_HIP_ALLOC_UNINIT = 1   /* like CUDAPtr::new (src/devices/cuda/cuda_ptr.rs:21-30) */
};

typedef struct custos_hip_device_info {
    char name[128];
    char arch[64];           /* e.g. "gfx950:sramecc+:xnack-" */
    int32_t compute_units;
    int32_t wavefront_size;
    int32_t clock_khz;
    int32_t memory_clock_khz;
    int32_t memory_bus_bits;
    int32_t l2_bytes;
    uint64_t total_memory;
} custos_hip_device_info;

/* Launch shape knobs of the generated kernels.  Zero fields keep the default.
 * `block_threads`, `unroll` and `blocks_per_cu` are compiled into a kernel (part of its cache
 * key: they apply to kernels compiled while they are set); `nontemporal` and `direction` are
 * arguments of every launch and apply to launches issued, and graphs built, while they are set. */
typedef struct custos_hip_tuning {
    int32_t block_threads;   /* threads per workgroup (multiple of 64), default 128 */
    int32_t unroll;          /* 16-byte vectors per thread per tile; 0 (default): the kernel holds the
                                code for 2 and for 1, chosen per launch from the bytes it touches */
    int32_t blocks_per_cu;   /* > 0: persistent grid of CUs*blocks_per_cu workgroups that
                                stride over the tiles; <= 0 (default): one tile per workgroup */
    int32_t nontemporal;     /* bit 0: non-temporal loads, bit 1: non-temporal stores, 64: stores are
                                written through to device scope at once; -1 = all off;
                                0 (default): chosen per launch from the bytes it touches */
    int32_t direction;       /* 1: tiles from the first to the last; 2: every launch walks them the
                                other way round than the launch before, so that it starts on what
                                the caches still hold; 0 (default): chosen per launch */
} custos_hip_tuning;

/* ---- device (src/devices/cuda/cuda.rs:53-67, cuda_device.rs:31-128) ---- */

int32_t custos_hip_device_count(int32_t *count);
/* Creates the handle: selects device `idx`, creates the compute stream.
 * The reference reads the index from CUSTOS_CU_DEVICE_IDX
 * (src/devices/cuda/mod.rs:35-42); callers here may read CUSTOS_HIP_DEVICE_IDX
 * with custos_hip_chosen_device_idx. */
int32_t custos_hip_device_create(int32_t idx, custos_hip_device **dev);
int32_t custos_hip_device_destroy(custos_hip_device *dev);
int32_t custos_hip_chosen_device_idx(void);
int32_t custos_hip_get_device_info(custos_hip_device *dev, custos_hip_device_info *info);
/* Message of the last failed call on `dev`; with dev == NULL, of the last
 * failed call of this thread that had no device (create, emit). */
const char *custos_hip_last_error(custos_hip_device *dev);
/* Blocks until the compute stream is idle (Stream::sync, src/devices/cuda/api/cuda.rs).
 * While the device records, nothing new reaches the stream: the wait is then for the work
 * that was in flight when the recording began. */
int32_t custos_hip_sync(custos_hip_device *dev);
int32_t custos_hip_set_tuning(custos_hip_device *dev, const custos_hip_tuning *tuning);
int32_t custos_hip_get_tuning(custos_hip_device *dev, custos_hip_tuning *tuning);

/* ---- memory (src/devices/cuda/cuda.rs:114-138, cuda_ptr.rs:21-77, ops.rs:17-117) ---- */

/* Alloc::alloc.  bytes == 0 fails with ZERO_LENGTH_BUFFER. */
int32_t custos_hip_alloc(custos_hip_device *dev, size_t bytes, int32_t flags, uint64_t *dptr);
/* Drop of an owning CUDAPtr (src/devices/cuda/cuda_ptr.rs:64-77). 0 is ignored.
 * The block goes back to the device's pool (below) without waiting for the
 * stream: every later use of the address is ordered behind the work that still
 * reads or writes it, because all device work of a handle runs on one stream. */
int32_t custos_hip_free(custos_hip_device *dev, uint64_t dptr);
/* Freed blocks are kept, by rounded size, and handed out again by custos_hip_alloc
 * instead of going through hipFree / hipMalloc (tens of microseconds and a device-wide
 * wait each; the reference's CUDA device pays cuMemAlloc / cuMemFree per buffer,
 * src/devices/cuda/api/cuda.rs:60-78).  `limit_bytes` bounds what the pool holds; 0
 * switches pooling off and releases what is held.  Default: a quarter of the device's
 * memory.  When hipMalloc fails the pool is released and the allocation retried. */
int32_t custos_hip_set_pool_limit(custos_hip_device *dev, size_t limit_bytes);
/* Releases every pooled block to the driver (waits for the stream). */
int32_t custos_hip_pool_trim(custos_hip_device *dev);
/* Bytes held in the pool, allocations served from it, allocations that went to hipMalloc. */
int32_t custos_hip_pool_stats(custos_hip_device *dev, size_t *pooled_bytes, uint64_t *reused,
                              uint64_t *allocated);
/* WriteBuf::write: host -> device, ordered on the compute stream; the host
 * range may be reused as soon as the call returns. Up to 64 KiB the data is copied
 * into one of 16 pinned staging slots and a copy kernel moves it from there without a
 * wait (3.4 us per write instead of the 14 us of a copy through the runtime and the wait
 * that frees the host range). */
int32_t custos_hip_write(custos_hip_device *dev, uint64_t dst, const void *src, size_t bytes);
/* Read::read: waits for the compute stream unless it is capturing, then copies
 * device -> host and waits for the copy (src/devices/cuda/ops.rs:32-48). Up to 64 KiB
 * a copy kernel stores the data into pinned host memory behind the work and the host
 * polls the completion word (10 us per read instead of 21). */
int32_t custos_hip_read(custos_hip_device *dev, void *dst, uint64_t src, size_t bytes);
/* WriteBuf::write_buf / CopySlice / CloneBuf: device -> device
 * (src/devices/cuda/ops.rs:66-117).  Runs as the identity expression through the
 * generated kernels; ranges that overlap partly are rejected (CUSTOS_HIP_ERR_BAD_OVERLAP). */
int32_t custos_hip_copy(custos_hip_device *dev, uint64_t dst, uint64_t src, size_t bytes);
/* ClearBuf::clear / ZeroGrad::zero_grad (`cu_clear`, src/devices/cuda/mod.rs:59-74).
 * Implemented as a fill kernel, so it may be captured into a graph. */
int32_t custos_hip_clear(custos_hip_device *dev, uint64_t dptr, size_t bytes);
/* Fills `bytes` bytes with one value of `value_bytes` (1, 2, 4, 8 or 16) bytes repeated;
 * address and length are multiples of `value_bytes`. What `Buffer::backward` needs for its
 * seed of ones: the reference builds the ones on the host and writes them to the device
 * (src/buffer/impl_autograd.rs:37-56, src/modules/autograd/tape.rs:67-83), N elements over
 * the host link for every backward pass; this is one store-only kernel at memory speed,
 * and it can be recorded like a clear. */
int32_t custos_hip_fill(custos_hip_device *dev, uint64_t dptr, size_t bytes, const void *value, size_t value_bytes);

/* ---- expression kernels (src/devices/cuda/kernel_cache.rs:10-73, source.rs:21-66) ---- */

/*
 * Compiles (or fetches from the cache) the kernel for one expression.
 *
 * `src` is the text custos' `ToCLSource` produces (src/two_way_ops/ops.rs,
 * ops/unary.rs, ops/cmps.rs), e.g. "((x * 2.0) + 1.0)", "pow((x * 3.0), (y + 1.0))",
 * "-(tan(x))", or a fused body "x = sin(x);\nx = (x * 2.0);\n"
 * (src/devices/fusing.rs:4-19).  `markers[k]` is the name the caller gave to
 * operand k (`Resolve::marker`, src/two_way_ops/resolve.rs:25-30); an index
 * suffix as in "x[idx]" is part of the name.
 * Numeric literals take the element type (a "2.0" in an f32 expression is the
 * f32 2.0), nothing is contracted into fma and no fast-math is applied, so
 * + - * / compare min max abs neg are bit-identical to the CPU device.
 * Kernels are cached per device by (expression structure, dtype, kind,
 * tuning): the same expression is compiled once.
 * Literal values need not cost a compilation each: a closure such as
 * `|x| x.mul(lr)` prints a new text for every value of `lr`
 * (src/two_way_ops/resolve.rs:131-141), and the reference compiles every distinct
 * text (src/devices/cuda/kernel_cache.rs:45-61).  Here the first set of values an
 * expression is seen with is compiled into the code; when the same expression
 * arrives with other values, a form that takes the literals as launch parameters
 * ("(x * c0)") is compiled once, and every further set of values is a handle on that
 * code carrying its own values.  Literals that always stay in the code: the divisor
 * of an integer division, and every literal of an expression with more than 32 of
 * them.  Results do not depend on which way a literal travels
 * (custos_hip_set_literal_policy pins one).
 * The kernel handle stays valid until the device is destroyed; a handle per distinct
 * set of values is kept (about 1 KiB each).
 */
int32_t custos_hip_expr_compile(custos_hip_device *dev, int32_t kind, int32_t dtype,
                                const char *src, const char *const *markers, int32_t n_markers,
                                custos_hip_kernel **kernel);
/* Generated HIP source of a kernel, the name of its entry point (what a
 * profiler lists: custos_<kind>_<dtype>_<key>), its 64-bit cache key and arity. */
const char *custos_hip_kernel_source(const custos_hip_kernel *kernel);
const char *custos_hip_kernel_name(const custos_hip_kernel *kernel);
uint64_t custos_hip_kernel_hash(const custos_hip_kernel *kernel);
int32_t custos_hip_kernel_arity(const custos_hip_kernel *kernel);
/* The kernel a launch of `kernel` over `n` elements runs: always `kernel` itself.  (One kernel
 * per expression serves every launch size: vectors per thread, cache policy and direction are
 * arguments of the launch, so nothing is compiled after custos_hip_expr_compile has returned --
 * the reference compiles once per text too, src/devices/cuda/kernel_cache.rs:39-61.) */
int32_t custos_hip_kernel_launched_as(custos_hip_device *dev, custos_hip_kernel *kernel, size_t n,
                                      custos_hip_kernel **variant);
/* How literal values reach a kernel (see custos_hip_expr_compile). */
#define CUSTOS_HIP_LITERALS_ADAPTIVE 0      /* in the code for the first set of values, parameters after */
#define CUSTOS_HIP_LITERALS_IN_CODE 1       /* every distinct set of values is compiled (the reference's way) */
#define CUSTOS_HIP_LITERALS_AS_PARAMETERS 2 /* always the shared form */
int32_t custos_hip_set_literal_policy(custos_hip_device *dev, int32_t policy);
/* What an `eq` node of expressions compiled from now on computes.  The reference disagrees with
 * itself: its GPU kernels are the text "(a == b)" (src/two_way_ops/ops/cmps.rs:117-130), its CPU
 * device evaluates `a <= b` (cmps.rs:135).  Default: `==`, like every GPU backend of the
 * reference; AS_CPU_EVAL compiles `<=`, so that results equal CPU<Base>'s for `eq` as well. */
#define CUSTOS_HIP_EQ_EXACT 0
#define CUSTOS_HIP_EQ_AS_CPU_EVAL 1
int32_t custos_hip_set_eq_policy(custos_hip_device *dev, int32_t policy);
/* Number of hiprtc compilations / cache hits since the device was created. */
int32_t custos_hip_cache_stats(custos_hip_device *dev, uint64_t *compiles, uint64_t *hits);

/* Disk cache: with the environment variable CUSTOS_HIP_KERNEL_CACHE_DIR set, code
 * objects are stored there (keyed by cache key, device architecture and hiprtc
 * version, verified against the stored source) and loaded by later processes
 * instead of compiling.  `*disk_hits` counts kernels loaded that way. */
int32_t custos_hip_cache_disk_hits(custos_hip_device *dev, uint64_t *disk_hits);

/* Caller-written kernels: `KernelCache::kernel` + `launch_kernel` / `launch_kernel1d`
 * (src/devices/cuda/kernel_cache.rs:39-61, kernel_launch.rs:81-163,
 * cuda_device.rs:85-112).  `src` is HIP source containing `extern "C" __global__
 * void <fn_name>(...)`; it is compiled once per (source, name) and cached.
 * `params[i]` points to the value of argument i (a device address is passed as a
 * pointer to the uint64_t holding it, like `AsCudaCvoidPtr`), `param_sizes[i]` is
 * its size in bytes.  While recording, the argument values are copied and the
 * launch becomes a graph node ordered after all earlier and before all later
 * work (its memory use is unknown). */
int32_t custos_hip_source_compile(custos_hip_device *dev, const char *src, const char *fn_name,
                                  custos_hip_kernel **kernel);
int32_t custos_hip_source_launch(custos_hip_device *dev, custos_hip_kernel *kernel,
                                 const uint32_t *grid, const uint32_t *block,
                                 uint32_t shared_mem_bytes, void *const *params,
                                 const size_t *param_sizes, int32_t n_params);
/* One-dimensional launch over `len` work items: workgroup size from the occupancy
 * calculator, grid = ceil(len / workgroup size). */
int32_t custos_hip_source_launch1d(custos_hip_device *dev, custos_hip_kernel *kernel, size_t len,
                                   void *const *params, const size_t *param_sizes,
                                   int32_t n_params);

/* Host-only helpers (no GPU needed): parse + emit the HIP source of a kernel
 * into `buf` (`*needed` = bytes including the terminator), and run the hiprtc
 * compilation for gfx950 without loading the result (`*code_size` = bytes). */
int32_t custos_hip_expr_emit(int32_t kind, int32_t dtype, const char *src,
                             const char *const *markers, int32_t n_markers,
                             const custos_hip_tuning *tuning, char *buf, size_t cap,
                             size_t *needed, uint64_t *hash);
/* The same for the form shared by all expressions that differ from `src` only in literal
 * values (literals as launch parameters, see custos_hip_expr_constants). */
int32_t custos_hip_expr_emit_shared(int32_t kind, int32_t dtype, const char *src,
                                    const char *const *markers, int32_t n_markers,
                                    const custos_hip_tuning *tuning, char *buf, size_t cap,
                                    size_t *needed, uint64_t *hash);
int32_t custos_hip_expr_build_code_object(int32_t kind, int32_t dtype, const char *src,
                                          const char *const *markers, int32_t n_markers,
                                          const custos_hip_tuning *tuning, size_t *code_size);
/* Launches of 64 MiB and more (issued directly, or nodes of built graphs) so far, by what the
 * address ranges of the launches around them told: not part of a chain; part of a chain -- it
 * reads what one of the last eight launches wrote, or in a graph one of the next levels reads
 * what it writes -- whose working set stays in the 256 MiB memory-side cache; part of a chain
 * whose working set does not.  (Only the last kind changes a launch shape: a two-pointer launch
 * of 256 to 768 MiB keeps its stores temporal when it is part of a streaming chain.) */
int32_t custos_hip_launch_hint_stats(custos_hip_device *dev, uint64_t *unrelated, uint64_t *resident,
                                     uint64_t *streaming);
/* Host-only: the launch shape the library picks for a launch that touches `footprint_bytes`
 * (all operands together) through `n_operands` pointers, for the knobs left at 0 in
 * custos_hip_tuning: vectors per thread, the `nontemporal` bits, and whether the launch
 * walks its tiles against the direction of the previous one -- for a launch that is not part
 * of a chain (see custos_hip_launch_hint_stats) and comes after nothing: a launch of more than
 * 8 and up to 32 MiB (what the eight L2s hold together) keeps temporal accesses only if it and
 * the up to eight tracked launches (or graph levels) before it touch no more than those 32 MiB
 * together; otherwise it streams like a larger one.  And a launch of 256 to 768 MiB through two
 * pointers streams its stores past the memory-side cache as well when those launches touched
 * other memory too. */
/* The same with everything else the choice depends on: how many of the operands the launch
 * writes (`n_written`: a kernel that writes through at least two pointers more than it reads
 * through, and touches 128 MiB or more, takes temporal loads and non-temporal stores written
 * through at once, so that the cache keeps its input and not its outputs), the distinct bytes the
 * launch and the launches before it touch together (`working_set_bytes`, 0 = unknown), and
 * what it has in common with the launch before it (`revisits`: 1 = it touches memory that launch
 * wrote; 0 = nothing of that: a launch of more than 32 MiB then runs as one-wavefront workgroups
 * with one vector per thread, and `block_threads` receives 64, else 0 for the workgroup size the
 * kernel was compiled for; 2 = nothing that launch wrote, and its first input is something that
 * launch read as well (`y = f(x)` into another buffer every time; a gradient launch behind the
 * forward launch of the same x): as for 0, with the direction alternating and everything streaming
 * past the memory-side cache but that input, which is loaded with temporal accesses -- reported in
 * `nontemporal` as 256 << i for input i on top of the bits of custos_hip_tuning). */
int32_t custos_hip_preferred_shape_of(uint64_t footprint_bytes, int32_t n_operands, int32_t n_written,
                                      uint64_t working_set_bytes, int32_t revisits, int32_t *unroll,
                                      int32_t *nontemporal, int32_t *alternate, int32_t *block_threads);
int32_t custos_hip_preferred_shape(uint64_t footprint_bytes, int32_t n_operands, int32_t *unroll,
                                   int32_t *nontemporal, int32_t *alternate);
/* The shape of the generated kernel that was launched directly, or planned into a graph by
 * custos_hip_capture_end, last on this device (same three values; all 0 before the first).
 * `nontemporal` may carry 256 << i on top of the bits of custos_hip_tuning: input i of the launch
 * keeps temporal loads although bit 0 is set, because the launch before it read that input too
 * and the memory-side cache is left to it (see custos_hip_preferred_shape_of).
 * No counterpart in the reference, whose launches have one shape. */
int32_t custos_hip_last_launch_shape(custos_hip_device *dev, int32_t *unroll, int32_t *nontemporal,
                                     int32_t *alternate);
/* Canonical re-print of an expression in the reference's ToCLSource format. */
int32_t custos_hip_expr_canonical(const char *src, const char *const *markers, int32_t n_markers,
                                  char *buf, size_t cap, size_t *needed);
/* Host-only: the values of the literals of `src` that the shared form of its kernel takes
 * as launch parameters, in the order c0, c1, ... of the generated text, each in the type the
 * expression is computed in (f32 for the 16-bit float types, else the element type).
 * `*n_params` = how many, `*needed` = their bytes; copied to `buf` if `cap` suffices. */
int32_t custos_hip_expr_constants(int32_t dtype, const char *src, const char *const *markers,
                                  int32_t n_markers, void *buf, size_t cap, size_t *needed,
                                  int32_t *n_params);

/* ---- launches ---- */

/* ApplyFunction::apply_fn body: out[i] = f(x[i]), i < n  (src/devices/cuda/ops.rs:126-177).
 * `out == x` (exact alias) is allowed; partial overlap is rejected. */
int32_t custos_hip_apply_fn(custos_hip_device *dev, custos_hip_kernel *kernel, uint64_t x,
                            uint64_t out, size_t n);
/* Two-operand expression: out[i] = f(lhs[i], rhs[i]). */
int32_t custos_hip_apply_fn2(custos_hip_device *dev, custos_hip_kernel *kernel, uint64_t lhs,
                             uint64_t rhs, uint64_t out, size_t n);
/* k-operand expression (k = kernel arity, 1..4). */
int32_t custos_hip_apply_fn_n(custos_hip_device *dev, custos_hip_kernel *kernel,
                              const uint64_t *ins, int32_t n_ins, uint64_t out, size_t n);
/* UnaryGrad::add_unary_grad body: lhs_grad[i] += out_grad[i] * f(lhs[i])
 * (src/devices/cuda/ops.rs:186-234), evaluated as g + (o * d), two roundings. */
int32_t custos_hip_add_unary_grad(custos_hip_device *dev, custos_hip_kernel *kernel, uint64_t lhs,
                                  uint64_t lhs_grad, uint64_t out_grad, size_t n);

/* No counterpart in the reference.  For callers that cannot allocate where they launch: tight
 * serving loops, harnesses that forbid hipMalloc, code that runs between the begin and the end
 * of a stream capture on ANOTHER stream (this call launches on the library's own stream, cannot
 * be recorded itself, and may wait for a staging slot).
 * What it does is what a recording of `n_sets` independent launches of `kernel` does when it is
 * built and replayed (custos_hip_capture_end merges them into one grid whose operand addresses
 * sit in a device table that the graph allocates): ONE grid over `n_sets` operand sets of `n`
 * elements each, but with the table in a static device array of the library (64 KiB per GPU,
 * held until the process ends) instead of an allocation.  This call never calls hipMalloc or
 * hipFree, compiles or loads no code and allocates nothing on the host heap: the kernel's entry
 * point for merged launches must have been loaded before, where allocation is allowed, with
 * custos_hip_kernel_prepare_merged (else CUSTOS_HIP_ERR_NOT_PREPARED).
 * `operands`: `n_sets` rows of `operands_per_set` device addresses in the order of the
 * kernel's pointer parameters (apply kernel: the inputs, then the output; unary-gradient kernel:
 * lhs, lhs_grad, out_grad), every address 16-byte aligned.  A row may name its output as one of
 * its inputs (exact alias); partial overlap inside a row, and a row that writes what another row
 * uses, are rejected (CUSTOS_HIP_ERR_BAD_OVERLAP).
 * Limit: n_sets * (operands_per_set + ceil(bytes of the kernel's literal parameters / 8)) <= 8192
 * table words, else CUSTOS_HIP_ERR_TOO_LARGE (2048 sets of a three-operand kernel).  Not legal
 * while the device records (CUSTOS_HIP_ERR_CAPTURE_STATE).
 * All calls on one GPU share that GPU's table, which keeps the rows of the last call (nothing in
 * it has to start at zero: every row a launch reads is rewritten by its call -- except that a
 * call identical to the handle's last one, kernel, length and addresses, finds its rows still in
 * the table when no other handle used it in between, and launches without sending them again or
 * repeating the operand checks).  Calls through one
 * device handle are ordered by its compute stream; a call through another handle on the same GPU
 * makes its stream wait for the launch of the table's last user before it rewrites the table
 * (one event per GPU, made when the first handle on that GPU is created), and calls from several
 * threads take turns. */
int32_t custos_hip_apply_fn_many_noalloc(custos_hip_device *dev, custos_hip_kernel *kernel,
                                         const uint64_t *operands, int32_t operands_per_set,
                                         size_t n_sets, size_t n);
/* The operand checks of custos_hip_apply_fn_many_noalloc by themselves, on the host (no device is
 * touched): `n_sets` rows of `operands_per_set` addresses, every operand `bytes` long, operand
 * number `written` of a row the one a launch writes.  0, CUSTOS_HIP_ERR_INVALID_ARGUMENT (a null
 * or unaligned address) or CUSTOS_HIP_ERR_BAD_OVERLAP.  No counterpart in the reference. */
int32_t custos_hip_check_operand_sets(const uint64_t *operands, int32_t operands_per_set, size_t n_sets,
                                      int32_t written, uint64_t bytes);
/* Compiles (or takes from the caches) and loads the entry point of `kernel` for merged launches
 * of equal length.  A generated kernel has three entry points -- one launch; many launches of
 * equal length in one grid; many launches of different lengths in one grid -- each a translation
 * unit of its own that is built when it is first needed: custos_hip_expr_compile builds the
 * first (the reference compiles one function per text too, src/devices/cuda/kernel_cache.rs:39-61),
 * a graph build the ones its nodes use, this call the second.  No counterpart in the reference. */
int32_t custos_hip_kernel_prepare_merged(custos_hip_device *dev, custos_hip_kernel *kernel);

/* ---- lazy run: capture once, replay (src/devices/cuda/lazy.rs:10-72) ---- */

/* LazySetup::lazy_setup: from here on launches/clears/copies are recorded, not run.
 * Allocation, reads and writes stay legal while recording and execute at once.
 * Takes no wait: work launched before (a graph of the run before, say) may still be in
 * flight; the first allocation, read, write or custos_hip_sync during the recording waits
 * for it, and a replay of the recorded graph is ordered behind it on the compute stream. */
int32_t custos_hip_capture_begin(custos_hip_device *dev);
/* Ends recording and instantiates an executable graph (LazyCudaGraph::new).
 * The graph is built from the recorded work, not replayed launch by launch:
 * launches that read what an earlier launch wrote are joined with it into one
 * kernel (custos_hip_set_graph_fusing), the work is sorted into dependency levels
 * (work of one level touches no common memory), and launches of one level that use
 * the same kernel are merged into one grid, whatever their lengths (1024 buffers x 3
 * operations replay as ONE kernel node; 3 with the joining switched off). How the
 * nodes are ordered: custos_hip_set_graph_edges. */
int32_t custos_hip_capture_end(custos_hip_device *dev, custos_hip_graph **graph);
/* capture_end for a caller that records the same program before every run (the reference's
 * Lazy::run calls every recorded operation again before each launch of its graph,
 * src/modules/lazy.rs:190-197, src/devices/cuda/lazy.rs:31-49): ends recording, and if the
 * recording is, launch for launch and address for address, the one `previous` was built from
 * (and the graph settings have not changed), hands back `previous` itself and builds nothing.
 * Otherwise a new graph is built as by capture_end; `previous` (may be null) is left alone and
 * stays the caller's to destroy.  The device keeps the recording its last graph stands for and
 * compares every launch, clear and copy of the next recording with it as it is recorded; while
 * they repeat it nothing is stored, and a recording that repeated all of it is recognised here
 * without any comparison (custos_hip_capture_stats). */
int32_t custos_hip_capture_end_reuse(custos_hip_device *dev, custos_hip_graph *previous, custos_hip_graph **graph);
/* How the recordings of this device ended so far.  `reused_while_recording`: calls of
 * custos_hip_capture_end_reuse that handed `previous` back because every launch of the recording
 * repeated the recording before it -- the device compares while it records and stores nothing, so
 * a caller that records the same program before every run pays a comparison per launch (0.02 us)
 * instead of a recorded launch (0.18 us); `reused_by_comparison`: handed back after the finished
 * recording was compared with the one `previous` was built from; `built`: graphs built.  Any
 * pointer may be null.  No counterpart in the reference. */
int32_t custos_hip_capture_stats(custos_hip_device *dev, uint64_t *reused_while_recording,
                                 uint64_t *reused_by_comparison, uint64_t *built);
/* Switches the merging of equal independent launches off (0) or on (default):
 * with it off every recorded launch becomes its own kernel node. */
int32_t custos_hip_set_graph_batching(custos_hip_device *dev, int32_t enabled);
/* Switches the joining of producers with their consumers off (0) or on (default).  With it on, a
 * recorded apply or unary-gradient launch whose output a later recorded apply or unary-gradient
 * launch reads element for element (same address, length and element type; a gradient launch
 * counts as the expression `lhs_grad + (out_grad * f'(lhs))` stored to lhs_grad) becomes one
 * kernel with that launch (so do two such launches that only read a common input, which is then
 * loaded once): both expressions
 * are evaluated per element, both results are stored where the two launches stored them, and
 * the second expression takes the first result -- as it was stored, rounded to the storage type
 * -- from a register.  `t = a * b; u = t + c; y = f(u)` replays as one launch that reads a, b, c
 * and writes t, u, y.  Every buffer receives exactly what the separate launches gave it.  Only
 * launches whose address ranges are pairwise equal or disjoint are joined, and only if nothing
 * recorded between them touches what the earlier one reads or writes; a joined launch is
 * producer and consumer in turn (up to 8 expressions, 8 inputs and 6 outputs per kernel).  A
 * literal is part of the joined kernel's code or one of its launch parameters as it is for the
 * launch's own kernel, so expressions that keep arriving with new values share their joined
 * kernels as they share their own.  The
 * kernels are compiled when the graph is built, within a time budget
 * (custos_hip_set_graph_fusing_budget); launches whose joined kernel is neither cached nor
 * compiled within it, or does not compile, replay as they were recorded
 * (custos_hip_graph_unjoined).  No counterpart in the reference, whose captured
 * graphs replay launch by launch (src/devices/cuda/lazy.rs:31-49). */
int32_t custos_hip_set_graph_fusing(custos_hip_device *dev, int32_t enabled);
/* How long a graph build may spend compiling kernels of joined launches (default 1000 ms): a
 * compilation starts only while less than that has been spent on them in this build, so 0 means
 * that only kernels from the caches are used.  A compilation takes 0.2-0.5 s the first time a
 * machine sees the kernel and about 0.03 s afterwards (the compiler library's own cache). */
int32_t custos_hip_set_graph_fusing_budget(custos_hip_device *dev, uint32_t milliseconds);
/* Recorded launches of `graph` that the build would have joined with others but left as they were
 * recorded, because their joined kernel was not compiled within the budget or did not compile;
 * `reason` (may be null) receives a text that lives as long as the graph: empty, the budget, or
 * the compiler's message. */
int32_t custos_hip_graph_unjoined(custos_hip_graph *graph, size_t *launches, const char **reason);
/* hiprtc compilations so far (translation units: a kernel has up to three, see
 * custos_hip_kernel_prepare_merged) and the time spent in them.  No counterpart in the reference. */
int32_t custos_hip_compile_stats(custos_hip_device *dev, uint64_t *units, double *milliseconds);
/* The entry point kernel node `node` (0 .. kernel_nodes-1, in replay order) of a built graph
 * launches, as a profiler lists it; the string lives as long as the graph.  No counterpart in
 * the reference. */
int32_t custos_hip_graph_node_kernel(custos_hip_graph *graph, size_t node, const char **name);
/* Recorded launches of a built graph that became part of a later launch's kernel. */
int32_t custos_hip_graph_fused_launches(custos_hip_graph *graph, size_t *launches);
/* Host-only: the source of the kernel that joins `n_stages` expressions (for tests and
 * inspection; nothing is launched).  `stage_srcs[s]` is an expression over the variables v0 ..
 * v{stage_vars[s]-1}; `sources` lists, stage after stage, where each variable comes from: the
 * index of an input pointer (0 .. n_inputs-1), or -(1 + t) for the stored value of stage t < s;
 * `stage_outs[s]` is the output pointer (0 .. n_outputs-1) that receives the stage's value, or -1
 * if a later stage writes the same memory.  `literals_as_parameters`: the literals are launch
 * parameters of the kernel (what a stage gets whose own kernel takes them that way, see
 * custos_hip_expr_compile) instead of part of its code.  With `code_size` the source is also
 * compiled for gfx950 and the size of the code object returned. */
int32_t custos_hip_chain_emit(int32_t dtype, const char *const *stage_srcs, const int32_t *stage_vars,
                              int32_t n_stages, const int32_t *sources, const int32_t *stage_outs,
                              int32_t n_inputs, int32_t n_outputs, int32_t literals_as_parameters,
                              char *buf, size_t cap, size_t *needed, size_t *code_size);
/* A recording that comes out as a plain chain (every dependency level one node, or any
 * recording under CUSTOS_HIP_GRAPH_EDGES_CHAIN) of at most `max_nodes` nodes is replayed by
 * issuing its nodes on the compute stream instead of launching an instantiated graph: for a
 * handful of launches that is cheaper than a graph launch. Default 4; 0 always instantiates a graph. Applies to later capture_end calls. */
int32_t custos_hip_set_graph_direct_replay(custos_hip_device *dev, int32_t max_nodes);
/* How a built graph orders its nodes (results are the same in every mode; applies to later
 * capture_end calls). The reference's stream capture serialises the recorded launches one by
 * one: src/devices/cuda/lazy.rs:10-29.
 * LEVEL_JOINS: the nodes of a dependency level sit side by side and wait for the whole level
 *   before them through one empty join node.
 * PER_NODE: every node waits only for the nodes whose memory it conflicts with (read-after-write,
 *   write-after-read, write-after-write on overlapping ranges), so independent chains do not wait
 *   for each other; a caller-written kernel still orders itself against everything.
 * CHAIN (default): the (merged) nodes form one chain; nothing runs side by side.
 *   An element-wise launch of any size worth it fills the chip by itself, and on this runtime a
 *   dependency between branches of a graph costs several times what a node of a chain costs:
 *   measured 1.3 to 4.7 times faster than LEVEL_JOINS and up to 2.2 times faster than PER_NODE
 *   on graphs of 16 to 768 nodes; only independent chains of launches that stream hundreds of
 *   MiB each replayed 3 % faster with PER_NODE. A graph of at most
 *   custos_hip_set_graph_direct_replay nodes is then replayed as plain launches.
 * CHAIN_BY_LEVEL: one chain, always level by level. CHAIN differs from it only for recordings
 *   with launches of 8 MiB and more: there the chain follows the recording where the
 *   dependencies allow (among the nodes that are ready, the one recorded first), so that a
 *   program recorded chain by chain over large buffers also replays chain by chain and finds its
 *   data in the caches, instead of streaming every buffer from memory at every level. */
enum custos_hip_graph_edges {
    CUSTOS_HIP_GRAPH_EDGES_LEVEL_JOINS = 0,
    CUSTOS_HIP_GRAPH_EDGES_PER_NODE = 1,
    CUSTOS_HIP_GRAPH_EDGES_CHAIN = 2,
    CUSTOS_HIP_GRAPH_EDGES_CHAIN_BY_LEVEL = 3
};
int32_t custos_hip_set_graph_edges(custos_hip_device *dev, int32_t mode);
/* With `enabled`, capture_end checks every graph it builds by brute force before instantiating it:
 * any two recorded pieces of work that touch overlapping memory, one of them writing, must be in
 * different nodes joined by a path; otherwise CUSTOS_HIP_ERR_GRAPH_ORDER. Quadratic in the
 * recorded work (at most 8192 recorded pieces); meant for tests. No counterpart in the
 * reference, whose captured graphs are serial by construction. */
int32_t custos_hip_set_graph_verify(custos_hip_device *dev, int32_t enabled);
/* Dependency edges of an instantiated graph, joins included (0 for a directly replayed chain).
 * No counterpart in the reference. */
int32_t custos_hip_graph_edge_count(custos_hip_graph *graph, size_t *edges);
int32_t custos_hip_is_capturing(custos_hip_device *dev, int32_t *capturing);
/* LazyCudaGraph::launch on the compute stream.  No wait: launches queue behind each other in
 * call order, and custos_hip_read, custos_hip_write, custos_hip_sync, a free that returns memory
 * to the driver, custos_hip_graph_destroy and custos_hip_device_destroy are ordered behind them or
 * wait for them.  The reference waits after every launch (src/devices/cuda/lazy.rs:42-43); a
 * caller who wants that calls custos_hip_sync. */
int32_t custos_hip_graph_launch(custos_hip_device *dev, custos_hip_graph *graph);
int32_t custos_hip_graph_node_count(custos_hip_graph *graph, size_t *kernel_nodes);
/* Recorded pieces of work, kernel nodes in the instantiated graph, dependency levels. */
int32_t custos_hip_graph_stats(custos_hip_graph *graph, size_t *recorded, size_t *kernel_nodes,
                               size_t *levels);
int32_t custos_hip_graph_destroy(custos_hip_device *dev, custos_hip_graph *graph);

/* ---- timing on the compute stream (bench support) ---- */

int32_t custos_hip_timer_begin(custos_hip_device *dev);
/* Records the end event, waits for it, returns milliseconds since timer_begin. */
int32_t custos_hip_timer_end(custos_hip_device *dev, double *ms);

/* Per-step timing: records mark number `index` (0..4095) on the compute stream, behind the work
 * issued so far; `timer_between` waits for mark `second` and returns the milliseconds from mark
 * `first` to it.  A mark between every two steps of a loop gives every step's own duration
 * (median, minimum) without a wait inside the loop. */
int32_t custos_hip_timer_mark(custos_hip_device *dev, uint32_t index);
int32_t custos_hip_timer_between(custos_hip_device *dev, uint32_t first, uint32_t second, double *ms);

#ifdef __cplusplus
}
#endif
#endif
