"""MI355X (gfx950) element-wise backend for custos: Python binding of the C ABI.

The product is `lib/libcustos_hip.so` (sources in `csrc/`, interface in
`include/custos_hip.h`).  This package is the thin host-side layer the tests
and the benchmark use: a ctypes binding, a mirror of custos' `Combiner`
expression vocabulary that prints the reference's `to_cl_source` text, and a
small `HIP` device class with the `apply_fn` / `add_unary_grad` call contract.
There is no CPU fallback: every operation fails if the library is missing.
"""
from .expr import Resolve, Expr, Const, to_marker, to_val  # noqa: F401
from .capi import (  # noqa: F401
    CustosHipError,
    DTYPES,
    KIND_APPLY,
    KIND_UNARY_GRAD,
    lib_path,
    load_library,
)
from .device import HIP, Buffer, Graph  # noqa: F401
