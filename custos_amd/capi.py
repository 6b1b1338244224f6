"""ctypes binding of include/custos_hip.h.  Loading fails loudly: there is no
fallback implementation of any entry point."""
from __future__ import annotations

import ctypes as C
import os

KIND_APPLY = 0
KIND_UNARY_GRAD = 1

ALLOC_ZEROED = 0
ALLOC_UNINIT = 1

# name -> (custos_hip_dtype value, numpy dtype string of the storage)
DTYPES = {
    "f32": (0, "float32"),
    "f64": (1, "float64"),
    "i32": (2, "int32"),
    "i64": (3, "int64"),
    "f16": (4, "float16"),
    "bf16": (5, "uint16"),
    "u8": (6, "uint8"),
    "i8": (7, "int8"),
    "i16": (8, "int16"),
    "u16": (9, "uint16"),
    "u32": (10, "uint32"),
    "u64": (11, "uint64"),
    "f16_pernode": (12, "float16"),
    "bf16_pernode": (13, "uint16"),
}

EQ_EXACT, EQ_AS_CPU_EVAL = 0, 1
ERR_INVALID_ARGUMENT = 10001
ERR_ZERO_LENGTH_BUFFER = 10002
ERR_INVALID_DEVICE_INDEX = 10003
ERR_EXPR_SYNTAX = 10010
ERR_EXPR_UNKNOWN_MARKER = 10011
ERR_EXPR_UNSUPPORTED = 10012
ERR_COMPILE = 10020
ERR_KIND_MISMATCH = 10030
ERR_ARITY_MISMATCH = 10031
ERR_NOT_PREPARED = 10032
ERR_CAPTURE_STATE = 10040
ERR_GRAPH_ORDER = 10041
ERR_BAD_OVERLAP = 10050
ERR_TOO_LARGE = 10060

GRAPH_EDGES_LEVEL_JOINS, GRAPH_EDGES_PER_NODE, GRAPH_EDGES_CHAIN, GRAPH_EDGES_CHAIN_BY_LEVEL = 0, 1, 2, 3


class CustosHipError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"custos-hip error {code}: {message}")
        self.code = code
        self.message = message


class DeviceInfo(C.Structure):
    _fields_ = [
        ("name", C.c_char * 128),
        ("arch", C.c_char * 64),
        ("compute_units", C.c_int32),
        ("wavefront_size", C.c_int32),
        ("clock_khz", C.c_int32),
        ("memory_clock_khz", C.c_int32),
        ("memory_bus_bits", C.c_int32),
        ("l2_bytes", C.c_int32),
        ("total_memory", C.c_uint64),
    ]


class Tuning(C.Structure):
    _fields_ = [
        ("block_threads", C.c_int32),
        ("unroll", C.c_int32),
        ("blocks_per_cu", C.c_int32),
        ("nontemporal", C.c_int32),
        ("direction", C.c_int32),
    ]


def lib_path() -> str:
    return os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libcustos_hip.so")


_P = C.c_void_p
_PP = C.POINTER(C.c_void_p)
_STRS = C.POINTER(C.c_char_p)

# every exported function: name -> (restype, argtypes).  tests check this list
# against the header and against the symbols of the built library.
PROTOTYPES = {
    "custos_hip_device_count": (C.c_int32, [C.POINTER(C.c_int32)]),
    "custos_hip_device_create": (C.c_int32, [C.c_int32, _PP]),
    "custos_hip_device_destroy": (C.c_int32, [_P]),
    "custos_hip_chosen_device_idx": (C.c_int32, []),
    "custos_hip_get_device_info": (C.c_int32, [_P, C.POINTER(DeviceInfo)]),
    "custos_hip_last_error": (C.c_char_p, [_P]),
    "custos_hip_sync": (C.c_int32, [_P]),
    "custos_hip_set_tuning": (C.c_int32, [_P, C.POINTER(Tuning)]),
    "custos_hip_get_tuning": (C.c_int32, [_P, C.POINTER(Tuning)]),
    "custos_hip_alloc": (C.c_int32, [_P, C.c_size_t, C.c_int32, C.POINTER(C.c_uint64)]),
    "custos_hip_set_pool_limit": (C.c_int32, [_P, C.c_size_t]),
    "custos_hip_pool_trim": (C.c_int32, [_P]),
    "custos_hip_pool_stats": (C.c_int32, [_P, C.POINTER(C.c_size_t), C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "custos_hip_free": (C.c_int32, [_P, C.c_uint64]),
    "custos_hip_write": (C.c_int32, [_P, C.c_uint64, C.c_void_p, C.c_size_t]),
    "custos_hip_read": (C.c_int32, [_P, C.c_void_p, C.c_uint64, C.c_size_t]),
    "custos_hip_capture_stats": (C.c_int32, [_P, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "custos_hip_check_operand_sets": (C.c_int32, [C.POINTER(C.c_uint64), C.c_int32, C.c_size_t, C.c_int32, C.c_uint64]),
    "custos_hip_copy": (C.c_int32, [_P, C.c_uint64, C.c_uint64, C.c_size_t]),
    "custos_hip_clear": (C.c_int32, [_P, C.c_uint64, C.c_size_t]),
    "custos_hip_expr_compile": (C.c_int32, [_P, C.c_int32, C.c_int32, C.c_char_p, _STRS, C.c_int32, _PP]),
    "custos_hip_kernel_source": (C.c_char_p, [_P]),
    "custos_hip_kernel_name": (C.c_char_p, [_P]),
    "custos_hip_kernel_hash": (C.c_uint64, [_P]),
    "custos_hip_preferred_shape": (C.c_int32, [C.c_uint64, C.c_int32, C.POINTER(C.c_int32), C.POINTER(C.c_int32), C.POINTER(C.c_int32)]),
    "custos_hip_preferred_shape_of": (C.c_int32, [C.c_uint64, C.c_int32, C.c_int32, C.c_uint64, C.c_int32, C.POINTER(C.c_int32),
                                                  C.POINTER(C.c_int32), C.POINTER(C.c_int32), C.POINTER(C.c_int32)]),
    "custos_hip_set_graph_fusing": (C.c_int32, [_P, C.c_int32]),
    "custos_hip_graph_node_kernel": (C.c_int32, [_P, C.c_size_t, C.POINTER(C.c_char_p)]),
    "custos_hip_graph_fused_launches": (C.c_int32, [_P, C.POINTER(C.c_size_t)]),
    "custos_hip_chain_emit": (C.c_int32, [C.c_int32, C.POINTER(C.c_char_p), C.POINTER(C.c_int32), C.c_int32, C.POINTER(C.c_int32),
                                          C.POINTER(C.c_int32), C.c_int32, C.c_int32, C.c_int32, C.c_char_p, C.c_size_t,
                                          C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]),
    "custos_hip_last_launch_shape": (C.c_int32, [_P, C.POINTER(C.c_int32), C.POINTER(C.c_int32), C.POINTER(C.c_int32)]),
    "custos_hip_kernel_launched_as": (C.c_int32, [_P, _P, C.c_size_t, C.POINTER(C.c_void_p)]),
    "custos_hip_kernel_arity": (C.c_int32, [_P]),
    "custos_hip_cache_stats": (C.c_int32, [_P, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "custos_hip_cache_disk_hits": (C.c_int32, [_P, C.POINTER(C.c_uint64)]),
    "custos_hip_source_compile": (C.c_int32, [_P, C.c_char_p, C.c_char_p, _PP]),
    "custos_hip_source_launch": (C.c_int32, [_P, _P, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.c_uint32,
                                             C.POINTER(C.c_void_p), C.POINTER(C.c_size_t), C.c_int32]),
    "custos_hip_source_launch1d": (C.c_int32, [_P, _P, C.c_size_t, C.POINTER(C.c_void_p), C.POINTER(C.c_size_t), C.c_int32]),
    "custos_hip_expr_emit": (C.c_int32, [C.c_int32, C.c_int32, C.c_char_p, _STRS, C.c_int32, C.POINTER(Tuning),
                                         C.c_char_p, C.c_size_t, C.POINTER(C.c_size_t), C.POINTER(C.c_uint64)]),
    "custos_hip_expr_emit_shared": (C.c_int32, [C.c_int32, C.c_int32, C.c_char_p, _STRS, C.c_int32, C.POINTER(Tuning),
                                                C.c_char_p, C.c_size_t, C.POINTER(C.c_size_t), C.POINTER(C.c_uint64)]),
    "custos_hip_set_literal_policy": (C.c_int32, [_P, C.c_int32]),
    "custos_hip_set_eq_policy": (C.c_int32, [_P, C.c_int32]),
    "custos_hip_launch_hint_stats": (C.c_int32, [_P, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "custos_hip_expr_build_code_object": (C.c_int32, [C.c_int32, C.c_int32, C.c_char_p, _STRS, C.c_int32,
                                                      C.POINTER(Tuning), C.POINTER(C.c_size_t)]),
    "custos_hip_expr_canonical": (C.c_int32, [C.c_char_p, _STRS, C.c_int32, C.c_char_p, C.c_size_t,
                                              C.POINTER(C.c_size_t)]),
    "custos_hip_expr_constants": (C.c_int32, [C.c_int32, C.c_char_p, _STRS, C.c_int32, C.c_void_p, C.c_size_t,
                                              C.POINTER(C.c_size_t), C.POINTER(C.c_int32)]),
    "custos_hip_apply_fn": (C.c_int32, [_P, _P, C.c_uint64, C.c_uint64, C.c_size_t]),
    "custos_hip_apply_fn2": (C.c_int32, [_P, _P, C.c_uint64, C.c_uint64, C.c_uint64, C.c_size_t]),
    "custos_hip_apply_fn_n": (C.c_int32, [_P, _P, C.POINTER(C.c_uint64), C.c_int32, C.c_uint64, C.c_size_t]),
    "custos_hip_apply_fn_many_noalloc": (C.c_int32, [_P, _P, C.POINTER(C.c_uint64), C.c_int32, C.c_size_t, C.c_size_t]),
    "custos_hip_kernel_prepare_merged": (C.c_int32, [_P, _P]),
    "custos_hip_set_graph_fusing_budget": (C.c_int32, [_P, C.c_uint32]),
    "custos_hip_graph_unjoined": (C.c_int32, [_P, C.POINTER(C.c_size_t), C.POINTER(C.c_char_p)]),
    "custos_hip_compile_stats": (C.c_int32, [_P, C.POINTER(C.c_uint64), C.POINTER(C.c_double)]),
    "custos_hip_fill": (C.c_int32, [_P, C.c_uint64, C.c_size_t, C.c_void_p, C.c_size_t]),
    "custos_hip_add_unary_grad": (C.c_int32, [_P, _P, C.c_uint64, C.c_uint64, C.c_uint64, C.c_size_t]),
    "custos_hip_capture_begin": (C.c_int32, [_P]),
    "custos_hip_capture_end": (C.c_int32, [_P, _PP]),
    "custos_hip_capture_end_reuse": (C.c_int32, [_P, _P, _PP]),
    "custos_hip_is_capturing": (C.c_int32, [_P, C.POINTER(C.c_int32)]),
    "custos_hip_graph_launch": (C.c_int32, [_P, _P]),
    "custos_hip_graph_node_count": (C.c_int32, [_P, C.POINTER(C.c_size_t)]),
    "custos_hip_graph_stats": (C.c_int32, [_P, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]),
    "custos_hip_set_graph_batching": (C.c_int32, [_P, C.c_int32]),
    "custos_hip_set_graph_direct_replay": (C.c_int32, [_P, C.c_int32]),
    "custos_hip_set_graph_edges": (C.c_int32, [_P, C.c_int32]),
    "custos_hip_set_graph_verify": (C.c_int32, [_P, C.c_int32]),
    "custos_hip_graph_edge_count": (C.c_int32, [_P, C.POINTER(C.c_size_t)]),
    "custos_hip_graph_destroy": (C.c_int32, [_P, _P]),
    "custos_hip_timer_begin": (C.c_int32, [_P]),
    "custos_hip_timer_end": (C.c_int32, [_P, C.POINTER(C.c_double)]),
    "custos_hip_timer_mark": (C.c_int32, [_P, C.c_uint32]),
    "custos_hip_timer_between": (C.c_int32, [_P, C.c_uint32, C.c_uint32, C.POINTER(C.c_double)]),
}

_lib = None


def load_library():
    """Loads libcustos_hip.so from the package's `lib/` folder (built in-tree by
    `__graft_entry__.build()` / `make -C custos_amd/csrc`)."""
    global _lib
    if _lib is not None:
        return _lib
    path = lib_path()
    if not os.path.exists(path):
        raise ImportError(
            f"{path} is missing: build it with `make -C custos_amd/csrc` "
            "(or `python -c 'import __graft_entry__ as g; g.build()'`). There is no fallback."
        )
    lib = C.CDLL(path)
    for name, (restype, argtypes) in PROTOTYPES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def c_markers(markers):
    arr = (C.c_char_p * len(markers))(*[m.encode() for m in markers])
    return arr, len(markers)


def last_error(dev_handle) -> str:
    msg = load_library().custos_hip_last_error(dev_handle)
    return msg.decode(errors="replace") if msg else ""


def check(rc: int, dev_handle=None):
    if rc != 0:
        raise CustosHipError(rc, last_error(dev_handle))


def preferred_shape(footprint_bytes: int, n_operands: int):
    """(vectors per thread, nontemporal bits, alternates direction) for such a launch."""
    u, nt, alt = C.c_int32(0), C.c_int32(0), C.c_int32(0)
    check(load_library().custos_hip_preferred_shape(footprint_bytes, n_operands, C.byref(u), C.byref(nt), C.byref(alt)))
    return u.value, nt.value, bool(alt.value)


def preferred_shape_of(footprint_bytes: int, n_operands: int, n_written: int = 1, working_set_bytes: int = 0, revisits=True):
    """(vectors per thread, nontemporal bits, alternates direction, threads per workgroup or 0) with everything
    the choice depends on.  `revisits`: True / 1 = touches what the launch before wrote, False / 0 = has nothing
    in common with it, 2 = its first input is something that launch read, and it touches nothing that launch wrote."""
    u, nt, alt, block = C.c_int32(0), C.c_int32(0), C.c_int32(0), C.c_int32(0)
    check(load_library().custos_hip_preferred_shape_of(footprint_bytes, n_operands, n_written, working_set_bytes, int(revisits),
                                                       C.byref(u), C.byref(nt), C.byref(alt), C.byref(block)))
    return u.value, nt.value, bool(alt.value), block.value


LITERALS_ADAPTIVE, LITERALS_IN_CODE, LITERALS_AS_PARAMETERS = 0, 1, 2


def expr_emit(kind: int, dtype: str, src: str, markers, tuning: Tuning | None = None, shared: bool = False):
    """Host-only: generated HIP source and cache key of a kernel: the one for exactly these
    literal values, or (`shared`) the form that takes the literals as launch parameters."""
    lib = load_library()
    emit = lib.custos_hip_expr_emit_shared if shared else lib.custos_hip_expr_emit
    arr, n = c_markers(markers)
    needed = C.c_size_t(0)
    h = C.c_uint64(0)
    t = C.byref(tuning) if tuning is not None else None
    check(emit(kind, DTYPES[dtype][0], src.encode(), arr, n, t, None, 0, C.byref(needed), C.byref(h)))
    buf = C.create_string_buffer(needed.value)
    check(emit(kind, DTYPES[dtype][0], src.encode(), arr, n, t, buf, needed.value, None, None))
    return buf.value.decode(), h.value


def chain_emit(dtype: str, stages, n_inputs: int, n_outputs: int, compile_it: bool = False, literals_as_parameters: bool = False):
    """Host-only: source (and, with `compile_it`, the gfx950 code size) of the kernel that joins several
    expressions.  `stages`: (source text over v0.., [where each variable comes from], output index or -1)."""
    lib = load_library()
    srcs = (C.c_char_p * len(stages))(*[s[0].encode() for s in stages])
    n_vars = (C.c_int32 * len(stages))(*[len(s[1]) for s in stages])
    flat = [v for s in stages for v in s[1]]
    sources = (C.c_int32 * len(flat))(*flat)
    outs = (C.c_int32 * len(stages))(*[s[2] for s in stages])
    needed, size = C.c_size_t(0), C.c_size_t(0)
    args = (DTYPES[dtype][0], srcs, n_vars, len(stages), sources, outs, n_inputs, n_outputs, 1 if literals_as_parameters else 0)
    check(lib.custos_hip_chain_emit(*args, None, 0, C.byref(needed), C.byref(size) if compile_it else None))
    buf = C.create_string_buffer(needed.value)
    check(lib.custos_hip_chain_emit(*args, buf, needed.value, None, None))
    return buf.value.decode(), size.value


def expr_build_code_object(kind: int, dtype: str, src: str, markers, tuning: Tuning | None = None) -> int:
    """Host-only: runs hiprtc for gfx950 on the generated kernel, returns the code object size."""
    lib = load_library()
    arr, n = c_markers(markers)
    size = C.c_size_t(0)
    t = C.byref(tuning) if tuning is not None else None
    check(lib.custos_hip_expr_build_code_object(kind, DTYPES[dtype][0], src.encode(), arr, n, t, C.byref(size)))
    return size.value


def expr_constants(dtype: str, src: str, markers):
    """The literals of `src` that its kernel takes as launch parameters (c0, c1, ...), as a
    numpy array of the type the expression is computed in."""
    import numpy as np
    lib = load_library()
    arr, n = c_markers(markers)
    needed, count = C.c_size_t(0), C.c_int32(0)
    check(lib.custos_hip_expr_constants(DTYPES[dtype][0], src.encode(), arr, n, None, 0, C.byref(needed), C.byref(count)))
    compute = {"f16": "f32", "bf16": "f32", "f16_pernode": "f32", "bf16_pernode": "f32"}.get(dtype, dtype)
    np_type = {"f32": np.float32, "f64": np.float64, "i32": np.int32, "i64": np.int64, "u8": np.uint8, "i8": np.int8,
               "i16": np.int16, "u16": np.uint16, "u32": np.uint32, "u64": np.uint64}[compute]
    out = np.zeros(count.value, dtype=np_type)
    if needed.value:
        check(lib.custos_hip_expr_constants(DTYPES[dtype][0], src.encode(), arr, n, out.ctypes.data, out.nbytes, None, None))
    return out


def expr_canonical(src: str, markers) -> str:
    lib = load_library()
    arr, n = c_markers(markers)
    needed = C.c_size_t(0)
    check(lib.custos_hip_expr_canonical(src.encode(), arr, n, None, 0, C.byref(needed)))
    buf = C.create_string_buffer(needed.value)
    check(lib.custos_hip_expr_canonical(src.encode(), arr, n, buf, needed.value, None))
    return buf.value.decode()
