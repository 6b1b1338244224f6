"""`HIP` device over the C ABI with the call contract of custos' device traits.

Mirrors, for the element-wise path, what `CUDA<Base>` offers in the reference:
`buffer` / `read` / `write` / `clear` (src/devices/cuda/ops.rs:17-117),
`apply_fn` (src/unary.rs:7-28, src/devices/cuda/ops.rs:119-141),
`add_unary_grad` (src/unary.rs:31-58, src/devices/cuda/ops.rs:179-199), the
fused unary op (src/devices/cuda/fusing.rs:3-51) and graph capture / replay
(src/devices/cuda/lazy.rs:10-72).  All arithmetic happens in the HIP kernels.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import capi
from .expr import Resolve, _wrap, fused_source


def _np_dtype(dtype: str):
    return np.dtype(capi.DTYPES[dtype][1])


def _same_shape(first, *others):
    """Operands of one launch have one length and one element type: a shorter one would be read
    or written beyond its end on the device (`None` entries, an output still to allocate, pass)."""
    for other in others:
        if other is None:
            continue
        if other.len != first.len or other.dtype != first.dtype:
            raise ValueError(f"operands differ in length or element type: {first.len} x {first.dtype} "
                             f"and {other.len} x {other.dtype}")


class Buffer:
    """A device allocation of `len` elements (`Buffer<T, HIP>` with `CUDAPtr`-like
    base: address, length, ownership flag -- src/devices/cuda/cuda_ptr.rs:7-15)."""

    def __init__(self, device: "HIP", ptr: int, length: int, dtype: str, owned: bool = True):
        self.device = device
        self.ptr = ptr
        self.len = length
        self.dtype = dtype
        self.owned = owned

    def __len__(self):
        return self.len

    @property
    def id(self) -> int:
        return self.ptr

    @property
    def nbytes(self) -> int:
        return self.len * _np_dtype(self.dtype).itemsize

    def read(self) -> np.ndarray:
        return self.device.read(self)

    def write(self, data) -> None:
        self.device.write(self, data)

    def clear(self) -> None:
        self.device.clear(self)

    def slice(self, start: int, stop: int) -> "Buffer":
        """Non-owning view of elements [start, stop)."""
        if not (0 <= start <= stop <= self.len):
            raise IndexError("slice out of range")
        item = _np_dtype(self.dtype).itemsize
        return Buffer(self.device, self.ptr + start * item, stop - start, self.dtype, owned=False)

    def free(self) -> None:
        if self.owned and self.ptr and self.device is not None and self.device.handle:
            self.device._check(self.device.lib.custos_hip_free(self.device.handle, self.ptr))
        self.ptr = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Graph:
    """An instantiated, replayable capture (`LazyCudaGraph`, src/devices/cuda/lazy.rs:10-29)."""

    def __init__(self, device: "HIP", handle):
        self.device = device
        self.handle = handle

    def launch(self) -> None:
        self.device._check(self.device.lib.custos_hip_graph_launch(self.device.handle, self.handle))

    @property
    def kernel_nodes(self) -> int:
        n = C.c_size_t(0)
        self.device._check(self.device.lib.custos_hip_graph_node_count(self.handle, C.byref(n)))
        return n.value

    def stats(self):
        """(recorded pieces of work, kernel nodes in the graph, dependency levels)"""
        a, b, c = C.c_size_t(0), C.c_size_t(0), C.c_size_t(0)
        self.device._check(self.device.lib.custos_hip_graph_stats(self.handle, C.byref(a), C.byref(b), C.byref(c)))
        return a.value, b.value, c.value

    def kernel_names(self):
        """Entry points of the graph's kernel nodes in replay order, as a profiler lists them."""
        names = []
        for i in range(self.kernel_nodes):
            name = C.c_char_p()
            self.device._check(self.device.lib.custos_hip_graph_node_kernel(self.handle, i, C.byref(name)))
            names.append(name.value.decode())
        return names

    @property
    def fused_launches(self) -> int:
        """Recorded launches that became part of a later launch's kernel."""
        n = C.c_size_t(0)
        self.device._check(self.device.lib.custos_hip_graph_fused_launches(self.handle, C.byref(n)))
        return n.value

    def unjoined(self):
        """(recorded launches the build would have joined but left as recorded, reason): the time budget of
        the build, or the compiler's message."""
        n, why = C.c_size_t(0), C.c_char_p()
        self.device._check(self.device.lib.custos_hip_graph_unjoined(self.handle, C.byref(n), C.byref(why)))
        return n.value, (why.value or b"").decode()

    def edge_count(self) -> int:
        """Dependency edges of the instantiated graph, joins included (0 for a directly replayed chain)."""
        e = C.c_size_t(0)
        self.device._check(self.device.lib.custos_hip_graph_edge_count(self.handle, C.byref(e)))
        return e.value

    def destroy(self) -> None:
        if self.handle and self.device.handle:
            self.device._check(self.device.lib.custos_hip_graph_destroy(self.device.handle, self.handle))
        self.handle = None


class HIP:
    """`HIP::<Base>::new(idx)`: eager execution, plain allocation."""

    def __init__(self, idx: int | None = None):
        self.lib = capi.load_library()
        self.handle = None
        if idx is None:
            idx = self.lib.custos_hip_chosen_device_idx()
        h = C.c_void_p()
        capi.check(self.lib.custos_hip_device_create(idx, C.byref(h)))
        self.handle = h

    # -- plumbing --
    def _check(self, rc: int) -> None:
        capi.check(rc, self.handle)

    def close(self) -> None:
        if self.handle:
            self.lib.custos_hip_device_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def info(self) -> capi.DeviceInfo:
        info = capi.DeviceInfo()
        self._check(self.lib.custos_hip_get_device_info(self.handle, C.byref(info)))
        return info

    def sync(self) -> None:
        self._check(self.lib.custos_hip_sync(self.handle))

    def set_tuning(self, block_threads=0, unroll=0, blocks_per_cu=0, nontemporal=0, direction=0) -> None:
        """Launch shape of generated kernels; 0 leaves a knob to the library (`custos_hip_tuning`)."""
        t = capi.Tuning(block_threads, unroll, blocks_per_cu, nontemporal, direction)
        self._check(self.lib.custos_hip_set_tuning(self.handle, C.byref(t)))

    def set_pool_limit(self, limit_bytes: int) -> None:
        """Bytes of freed blocks the device keeps for reuse (0 switches the pool off)."""
        self._check(self.lib.custos_hip_set_pool_limit(self.handle, limit_bytes))

    def pool_trim(self) -> None:
        self._check(self.lib.custos_hip_pool_trim(self.handle))

    def pool_stats(self):
        """(bytes held in the pool, allocations served from it, allocations that went to hipMalloc)"""
        a, b, c = C.c_size_t(0), C.c_uint64(0), C.c_uint64(0)
        self._check(self.lib.custos_hip_pool_stats(self.handle, C.byref(a), C.byref(b), C.byref(c)))
        return a.value, b.value, c.value

    def cache_stats(self):
        a, b = C.c_uint64(0), C.c_uint64(0)
        self._check(self.lib.custos_hip_cache_stats(self.handle, C.byref(a), C.byref(b)))
        return a.value, b.value

    # -- Alloc / Read / WriteBuf / ClearBuf --
    def alloc(self, length: int, dtype: str = "f32", zeroed: bool = True) -> Buffer:
        ptr = C.c_uint64(0)
        nbytes = length * _np_dtype(dtype).itemsize
        flags = capi.ALLOC_ZEROED if zeroed else capi.ALLOC_UNINIT
        self._check(self.lib.custos_hip_alloc(self.handle, nbytes, flags, C.byref(ptr)))
        return Buffer(self, ptr.value, length, dtype)

    def buffer(self, data, dtype: str = "f32") -> Buffer:
        """`device.buffer([...])` / `Buffer::from((&device, slice))`."""
        arr = np.ascontiguousarray(data, dtype=_np_dtype(dtype))
        buf = self.alloc(arr.size, dtype, zeroed=False)
        self.write(buf, arr)
        return buf

    def write(self, buf: Buffer, data) -> None:
        arr = np.ascontiguousarray(data, dtype=_np_dtype(buf.dtype))
        if arr.size != buf.len:
            raise ValueError(f"write of {arr.size} elements into a buffer of {buf.len}")
        self._check(self.lib.custos_hip_write(self.handle, buf.ptr, arr.ctypes.data_as(C.c_void_p), arr.nbytes))

    def read(self, buf: Buffer) -> np.ndarray:
        out = np.empty(buf.len, dtype=_np_dtype(buf.dtype))
        self._check(self.lib.custos_hip_read(self.handle, out.ctypes.data_as(C.c_void_p), buf.ptr, out.nbytes))
        return out

    def clear(self, buf: Buffer) -> None:
        self._check(self.lib.custos_hip_clear(self.handle, buf.ptr, buf.nbytes))

    def fill(self, buf: Buffer, value) -> None:
        """Every element of `buf` set to `value` on the device."""
        item = np.asarray(value, dtype=_np_dtype(buf.dtype)).reshape(1)
        self._check(self.lib.custos_hip_fill(self.handle, buf.ptr, buf.nbytes, item.ctypes.data_as(C.c_void_p), item.itemsize))

    def copy(self, dst: Buffer, src: Buffer) -> None:
        if dst.nbytes != src.nbytes:
            raise ValueError("size mismatch")
        self._check(self.lib.custos_hip_copy(self.handle, dst.ptr, src.ptr, src.nbytes))

    # -- kernels --
    def compile(self, kind: int, dtype: str, src: str, markers=("x",)):
        arr, n = capi.c_markers(list(markers))
        k = C.c_void_p()
        self._check(self.lib.custos_hip_expr_compile(self.handle, kind, capi.DTYPES[dtype][0], src.encode(), arr, n, C.byref(k)))
        return k

    def kernel_source(self, kernel) -> str:
        return self.lib.custos_hip_kernel_source(kernel).decode()

    def kernel_name(self, kernel, n: int | None = None) -> str:
        """Entry point name; with `n`, of the variant a launch over n elements runs."""
        if n is not None:
            v = C.c_void_p()
            self._check(self.lib.custos_hip_kernel_launched_as(self.handle, kernel, n, C.byref(v)))
            kernel = v
        return self.lib.custos_hip_kernel_name(kernel).decode()

    def apply_fn(self, buf: Buffer, f, out: Buffer | None = None) -> Buffer:
        """`device.apply_fn(&buf, |x| ...)`: out[i] = f(buf[i]) in a new buffer."""
        _same_shape(buf, out)
        src = _wrap(f(Resolve("x"))).to_cl_source(buf.dtype)
        kernel = self.compile(capi.KIND_APPLY, buf.dtype, src, ("x",))
        if out is None:
            out = self.alloc(buf.len, buf.dtype, zeroed=False)
        self._check(self.lib.custos_hip_apply_fn(self.handle, kernel, buf.ptr, out.ptr, buf.len))
        return out

    def apply_fn2(self, lhs: Buffer, rhs: Buffer, f, out: Buffer | None = None) -> Buffer:
        """Two-operand expression: out[i] = f(lhs[i], rhs[i])."""
        _same_shape(lhs, rhs, out)
        src = _wrap(f(Resolve("x", 0), Resolve("y", 1))).to_cl_source(lhs.dtype)
        kernel = self.compile(capi.KIND_APPLY, lhs.dtype, src, ("x", "y"))
        if out is None:
            out = self.alloc(lhs.len, lhs.dtype, zeroed=False)
        self._check(self.lib.custos_hip_apply_fn2(self.handle, kernel, lhs.ptr, rhs.ptr, out.ptr, lhs.len))
        return out

    def apply_fn_n(self, ins, f, out: Buffer | None = None) -> Buffer:
        """k-operand expression (k <= 4) over markers a, b, c, d."""
        _same_shape(*ins, out)
        names = ("a", "b", "c", "d")[: len(ins)]
        src = _wrap(f(*[Resolve(n, i) for i, n in enumerate(names)])).to_cl_source(ins[0].dtype)
        kernel = self.compile(capi.KIND_APPLY, ins[0].dtype, src, names)
        if out is None:
            out = self.alloc(ins[0].len, ins[0].dtype, zeroed=False)
        ptrs = (C.c_uint64 * len(ins))(*[b.ptr for b in ins])
        self._check(self.lib.custos_hip_apply_fn_n(self.handle, kernel, ptrs, len(ins), out.ptr, ins[0].len))
        return out

    def apply_fn_many_noalloc(self, kernel, operand_sets, n: int) -> None:
        """One grid over many operand sets of `n` elements each, the operand table in the library's
        static device array: no allocation anywhere on the way.  `operand_sets`: per set the
        buffers (or addresses) in the order of the kernel's pointer parameters."""
        rows = [[b.ptr if isinstance(b, Buffer) else int(b) for b in row] for row in operand_sets]
        per_set = len(rows[0]) if rows else 0
        if any(len(r) != per_set for r in rows):
            raise ValueError("operand sets differ in their number of operands")
        for row, given in zip(rows, operand_sets):
            for b in given:
                if isinstance(b, Buffer) and b.len < n:
                    raise ValueError(f"operand of {b.len} elements in a launch over {n}")
        flat = (C.c_uint64 * max(1, len(rows) * per_set))(*[p for r in rows for p in r])
        self._check(self.lib.custos_hip_apply_fn_many_noalloc(self.handle, kernel, flat, per_set, len(rows), n))

    def fused_apply_fn(self, buf: Buffer, ops, out: Buffer | None = None) -> Buffer:
        """The op `unary_fuse_op` returns: all `ops` applied in sequence in one kernel."""
        _same_shape(buf, out)
        src = fused_source(ops, buf.dtype)
        kernel = self.compile(capi.KIND_APPLY, buf.dtype, src, ("x",))
        if out is None:
            out = self.alloc(buf.len, buf.dtype, zeroed=False)
        self._check(self.lib.custos_hip_apply_fn(self.handle, kernel, buf.ptr, out.ptr, buf.len))
        return out

    def add_unary_grad(self, lhs: Buffer, lhs_grad: Buffer, out_grad: Buffer, lhs_grad_fn) -> None:
        """`device.add_unary_grad(&lhs, &mut lhs_grad, &out_grad, |x| ...)`."""
        _same_shape(lhs, lhs_grad, out_grad)
        src = _wrap(lhs_grad_fn(Resolve("x"))).to_cl_source(lhs.dtype)
        kernel = self.compile(capi.KIND_UNARY_GRAD, lhs.dtype, src, ("x",))
        self._check(self.lib.custos_hip_add_unary_grad(self.handle, kernel, lhs.ptr, lhs_grad.ptr, out_grad.ptr, lhs.len))

    # -- caller-written kernels (`launch_kernel` / `launch_kernel1d`, src/devices/cuda/cuda_device.rs:85-112) --
    def _source_args(self, args):
        """Buffers pass their device address, ctypes values and numpy scalars pass with their own
        width (`np.uint64(n)` for an `unsigned long long` parameter), Python ints become c_int32 and
        Python floats c_float (`AsCudaCvoidPtr`, src/devices/cuda/kernel_launch.rs:29-77)."""
        vals = []
        for a in args:
            if isinstance(a, Buffer):
                vals.append(C.c_uint64(a.ptr))
            elif isinstance(a, C._SimpleCData):
                vals.append(a)
            elif isinstance(a, np.generic) and not isinstance(a, np.bool_):
                vals.append(np.ctypeslib.as_ctypes_type(a.dtype)(a.item()))
            elif isinstance(a, (bool, int, np.bool_)):
                vals.append(C.c_int32(int(a)))
            else:
                vals.append(C.c_float(float(a)))
        ptrs = (C.c_void_p * len(vals))(*[C.cast(C.pointer(v), C.c_void_p) for v in vals])
        sizes = (C.c_size_t * len(vals))(*[C.sizeof(v) for v in vals])
        return vals, ptrs, sizes

    def compile_source(self, src: str, fn_name: str):
        k = C.c_void_p()
        self._check(self.lib.custos_hip_source_compile(self.handle, src.encode(), fn_name.encode(), C.byref(k)))
        return k

    def launch_kernel(self, src: str, fn_name: str, grid, block, shared_mem_bytes: int, args) -> None:
        k = self.compile_source(src, fn_name)
        vals, ptrs, sizes = self._source_args(args)
        g = (C.c_uint32 * 3)(*grid)
        b = (C.c_uint32 * 3)(*block)
        self._check(self.lib.custos_hip_source_launch(self.handle, k, g, b, shared_mem_bytes, ptrs, sizes, len(vals)))

    def launch_kernel1d(self, length: int, src: str, fn_name: str, args) -> None:
        k = self.compile_source(src, fn_name)
        vals, ptrs, sizes = self._source_args(args)
        self._check(self.lib.custos_hip_source_launch1d(self.handle, k, length, ptrs, sizes, len(vals)))

    def disk_cache_hits(self) -> int:
        v = C.c_uint64(0)
        self._check(self.lib.custos_hip_cache_disk_hits(self.handle, C.byref(v)))
        return v.value

    # -- capture / replay --
    def capture_begin(self) -> None:
        self._check(self.lib.custos_hip_capture_begin(self.handle))

    def capture_end(self) -> Graph:
        g = C.c_void_p()
        self._check(self.lib.custos_hip_capture_end(self.handle, C.byref(g)))
        return Graph(self, g)

    def capture_end_reuse(self, previous: Graph | None) -> Graph:
        """capture_end that hands back `previous` itself when the recording is the one it was built from."""
        g = C.c_void_p()
        self._check(self.lib.custos_hip_capture_end_reuse(self.handle, previous.handle if previous else None, C.byref(g)))
        if previous is not None and g.value == previous.handle.value:
            return previous
        return Graph(self, g)

    def capture_stats(self):
        """(recordings that repeated the one before and were recognised while recording, recordings
        recognised by comparison afterwards, graphs built)."""
        a, b, c = C.c_uint64(), C.c_uint64(), C.c_uint64()
        self._check(self.lib.custos_hip_capture_stats(self.handle, C.byref(a), C.byref(b), C.byref(c)))
        return a.value, b.value, c.value

    def set_graph_batching(self, enabled: bool) -> None:
        self._check(self.lib.custos_hip_set_graph_batching(self.handle, 1 if enabled else 0))

    def set_eq_policy(self, policy: int) -> None:
        """What `eq` nodes compiled from now on compute: capi.EQ_EXACT (`==`, the reference's GPU kernels) or
        capi.EQ_AS_CPU_EVAL (`<=`, what the reference's CPU device evaluates)."""
        self._check(self.lib.custos_hip_set_eq_policy(self.handle, int(policy)))

    def set_graph_fusing(self, enabled) -> None:
        """Whether a graph build joins recorded launches with the launches that read their output."""
        self._check(self.lib.custos_hip_set_graph_fusing(self.handle, int(bool(enabled))))

    def set_graph_fusing_budget(self, milliseconds: int) -> None:
        """How long a graph build may spend compiling kernels of joined launches (default 1000 ms; 0: only
        kernels from the caches)."""
        self._check(self.lib.custos_hip_set_graph_fusing_budget(self.handle, int(milliseconds)))

    def prepare_merged(self, kernel) -> None:
        """Compiles and loads the kernel's entry point for many launches of equal length in one grid."""
        self._check(self.lib.custos_hip_kernel_prepare_merged(self.handle, kernel))

    def compile_stats(self):
        """(translation units compiled by hiprtc so far, milliseconds spent in them)."""
        units, ms = C.c_uint64(0), C.c_double(0)
        self._check(self.lib.custos_hip_compile_stats(self.handle, C.byref(units), C.byref(ms)))
        return units.value, ms.value

    def launch_hint_stats(self):
        """(not part of a chain, chain that stays in the memory-side cache, chain that streams) counts of
        the launches and graph nodes of 64 MiB and more so far."""
        a, b, c = C.c_uint64(0), C.c_uint64(0), C.c_uint64(0)
        self._check(self.lib.custos_hip_launch_hint_stats(self.handle, C.byref(a), C.byref(b), C.byref(c)))
        return a.value, b.value, c.value

    def last_launch_shape(self):
        """(vectors per thread, cache-policy bits, alternating) of the generated kernel launched, or
        planned into a graph, last."""
        u, nt, alt = C.c_int32(0), C.c_int32(0), C.c_int32(0)
        self._check(self.lib.custos_hip_last_launch_shape(self.handle, C.byref(u), C.byref(nt), C.byref(alt)))
        return u.value, nt.value, bool(alt.value)

    def set_literal_policy(self, policy: int) -> None:
        """How literal values reach kernels: capi.LITERALS_ADAPTIVE (default), _IN_CODE, _AS_PARAMETERS."""
        self._check(self.lib.custos_hip_set_literal_policy(self.handle, policy))

    def set_graph_direct_replay(self, max_nodes: int) -> None:
        self._check(self.lib.custos_hip_set_graph_direct_replay(self.handle, max_nodes))

    def set_graph_edges(self, mode: int) -> None:
        """How built graphs order their nodes: capi.GRAPH_EDGES_LEVEL_JOINS, _PER_NODE or _CHAIN."""
        self._check(self.lib.custos_hip_set_graph_edges(self.handle, int(mode)))

    def set_graph_verify(self, enabled: bool) -> None:
        """capture_end checks the ordering of every graph it builds by brute force (for tests)."""
        self._check(self.lib.custos_hip_set_graph_verify(self.handle, 1 if enabled else 0))

    def is_capturing(self) -> bool:
        v = C.c_int32(0)
        self._check(self.lib.custos_hip_is_capturing(self.handle, C.byref(v)))
        return bool(v.value)

    # -- timing --
    def timer_begin(self) -> None:
        self._check(self.lib.custos_hip_timer_begin(self.handle))

    def timer_end(self) -> float:
        ms = C.c_double(0)
        self._check(self.lib.custos_hip_timer_end(self.handle, C.byref(ms)))
        return ms.value

    def timer_mark(self, index: int) -> None:
        """Records mark `index` (0..4095) on the compute stream behind the work issued so far."""
        self._check(self.lib.custos_hip_timer_mark(self.handle, index))

    def timer_between(self, first: int, second: int) -> float:
        """Milliseconds from mark `first` to mark `second` (waits for the second)."""
        ms = C.c_double(0)
        self._check(self.lib.custos_hip_timer_between(self.handle, first, second, C.byref(ms)))
        return ms.value
