"""ctypes binding of librk.so -- the only route from the host mirror to the kernels.

There is no fallback: if the shared library has not been built, importing this module raises
(build it with ``python amdgpu.jl_amd/build.py`` or ``__graft_entry__.build()``).
The prototypes below restate ``include/rk.h``; ``tests/test_abi_cpu.py`` checks that every symbol
the header declares is exported.
"""
from __future__ import annotations

import ctypes as C
import os

# PyTorch supplies device memory and streams on this side of the ABI, and it ships its own HIP
# runtime (libamdhip64.so.7).  It must be in the process BEFORE librk.so is opened so that the
# loader binds librk.so to that same runtime instance; two runtimes in one process do not share
# devices or streams.  (A Julia host binds librk.so to the runtime AMDGPU.jl already loaded.)
import torch  # noqa: F401  (import order matters)

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("RK_LIBRARY") or os.path.join(HERE, "librk.so")      # RK_LIBRARY: another build of the same ABI

RK_MAX_DIMS = 8
RK_MAX_OPERANDS = 8
RK_MAX_PROGRAM = 48

# status codes
RK_SUCCESS = 0
RK_ERR_INVALID_ARGUMENT = 10001
RK_ERR_UNSUPPORTED = 10002
RK_ERR_WORKSPACE = 10003
RK_ERR_DIMENSION = 10004
RK_ERR_TOO_LARGE = 10005
RK_ERR_WAIT = 10006
RK_STATIC_SCRATCH_BYTES = 16 << 20

# rk_dtype
RK_F32, RK_F64, RK_I32, RK_I64, RK_U8, RK_U32, RK_U64, RK_F16, RK_I16, RK_I8, RK_U16 = range(11)
# rk_map
RK_MAP_IDENTITY, RK_MAP_ABS2, RK_MAP_ABS = range(3)
RK_MAP_MAX_TOKENS, RK_MAP_MAX_CONSTS = 16, 4
# rk_op
RK_OP_ADD, RK_OP_MUL, RK_OP_MAX, RK_OP_MIN, RK_OP_AND, RK_OP_OR, RK_OP_XOR = range(7)
# rk_opkind
RK_KIND_MAPREDUCE, RK_KIND_FINDMINMAX, RK_KIND_ACCUMULATE, RK_KIND_FINDALL = range(4)
# rk_bc_token
(RK_BC_ADD, RK_BC_SUB, RK_BC_MUL, RK_BC_DIV, RK_BC_MAX, RK_BC_MIN, RK_BC_POW, RK_BC_FMA) = range(32, 40)
(RK_BC_NEG, RK_BC_ABS, RK_BC_ABS2, RK_BC_SQRT, RK_BC_EXP, RK_BC_LOG, RK_BC_SIN, RK_BC_COS, RK_BC_TANH,
 RK_BC_INV, RK_BC_IDENTITY) = range(64, 75)
(RK_BC_LT, RK_BC_LE, RK_BC_GT, RK_BC_GE, RK_BC_EQ, RK_BC_NE, RK_BC_AND, RK_BC_OR) = range(96, 104)
RK_BC_IFELSE = 112
(RK_BC_NOT, RK_BC_ISODD, RK_BC_ISEVEN, RK_BC_ISNAN, RK_BC_WRAP_I32, RK_BC_WRAP_U32, RK_BC_ROUND_F16,
 RK_BC_WRAP_I8, RK_BC_WRAP_U8, RK_BC_WRAP_I16, RK_BC_WRAP_U16) = range(128, 139)


class RkOperand(C.Structure):
    _fields_ = [
        ("ptr", C.c_void_p),
        ("dtype", C.c_int32),
        ("ndim", C.c_int32),
        ("shape", C.c_int64 * RK_MAX_DIMS),
        ("scalar_f", C.c_double),
        ("scalar_i", C.c_int64),
        ("strided", C.c_int32),
        ("reserved", C.c_int32),
        ("strides", C.c_int64 * RK_MAX_DIMS),
    ]


class RkProgram(C.Structure):
    _fields_ = [
        ("compute", C.c_int32),
        ("n_operands", C.c_int32),
        ("operands", RkOperand * RK_MAX_OPERANDS),
        ("n_tokens", C.c_int32),
        ("tokens", C.c_int32 * RK_MAX_PROGRAM),
    ]


class RkMapProgram(C.Structure):
    _fields_ = [
        ("n_tokens", C.c_int32),
        ("tokens", C.c_int32 * RK_MAP_MAX_TOKENS),
        ("n_consts", C.c_int32),
        ("const_f", C.c_double * RK_MAP_MAX_CONSTS),
        ("const_i", C.c_int64 * RK_MAP_MAX_CONSTS),
    ]


_I64P = C.POINTER(C.c_int64)

PROTOTYPES = {
    "rk_version": (C.c_int32, []),
    "rk_status_string": (C.c_char_p, [C.c_int32]),
    "rk_workspace_bytes": (C.c_size_t, [C.c_int, C.c_int, C.c_int, _I64P, C.c_uint32]),
    "rk_workspace_init": (C.c_int32, [C.c_void_p, C.c_size_t, C.c_void_p]),
    "rk_set_wait_budget": (C.c_int64, [C.c_int64]),
    "rk_workspace_status": (C.c_int32, [C.c_void_p, C.c_size_t, C.c_void_p]),
    "rk_sort_status": (C.c_int32, [C.c_void_p, C.c_size_t, C.c_void_p]),
    "rk_accumulate_static_status": (C.c_int32, [C.c_void_p]),
    "rk_mapreduce": (C.c_int32, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_int, _I64P, C.c_uint32,
                                 C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "rk_mapreduce_strided": (C.c_int32, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_int, _I64P, _I64P, C.c_uint32,
                                         C.c_void_p, _I64P, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "rk_accumulate_strided": (C.c_int32, [C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_int, _I64P, _I64P, _I64P, C.c_int,
                                          C.c_int32, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "rk_mapreduce_program": (C.c_int32, [C.POINTER(RkMapProgram), C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_int, _I64P, C.c_uint32,
                                         C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "rk_findminmax": (C.c_int32, [C.c_int32, C.c_int, C.c_void_p, C.c_int, _I64P, C.c_uint32,
                                  C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "rk_findminmax_strided": (C.c_int32, [C.c_int32, C.c_int, C.c_void_p, C.c_int, _I64P, _I64P, C.c_uint32,
                                          C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "rk_accumulate": (C.c_int32, [C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_int, _I64P, C.c_int,
                                  C.c_int32, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "rk_accumulate_static": (C.c_int32, [C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_int, _I64P, C.c_int,
                                         C.c_int32, C.c_void_p, C.c_void_p]),
    "rk_broadcast": (C.c_int32, [C.POINTER(RkProgram), C.c_void_p, C.c_int, C.c_int, _I64P, C.c_void_p]),
    "rk_broadcast_strided": (C.c_int32, [C.POINTER(RkProgram), C.c_void_p, C.c_int, C.c_int, _I64P, _I64P, C.c_void_p]),
    "rk_volumerhs_f32": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_float, C.c_void_p, C.c_int64,
                                     C.c_void_p]),
    "rk_findall_scatter": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, _I64P, C.c_void_p]),
    "rk_gather_slices": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_int64, C.c_int64, C.c_int64, C.c_void_p]),
    "rk_sort_tmp_bytes": (C.c_size_t, [C.c_int, C.c_int64, C.c_int32]),
    "rk_sort": (C.c_int32, [C.c_int, C.c_void_p, C.c_int64, C.c_int32, C.c_void_p, C.c_size_t, C.c_void_p]),
    "rk_sortperm": (C.c_int32, [C.c_int, C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_void_p, C.c_size_t, C.c_void_p]),
    "rk_permutedims": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, _I64P, C.POINTER(C.c_int32), C.c_void_p]),
    "rk_reverse": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, _I64P, C.c_uint32, C.c_void_p]),
    "rk_findall": (C.c_int32, [C.c_void_p, C.c_int, _I64P, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
}


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: the HIP kernels have not been built. "
            "Run `python amdgpu.jl_amd/build.py` (needs hipcc). There is no CPU fallback.")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in PROTOTYPES.items():
        fn = getattr(lib, name)      # AttributeError if the library does not export it
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


class RKError(RuntimeError):
    """Non-zero status from librk.so (the analogue of the reference's HIPError, src/hip/error.jl:143-147)."""

    def __init__(self, status: int, where: str = ""):
        self.status = int(status)
        msg = lib.rk_status_string(self.status)
        text = msg.decode() if msg else "?"
        super().__init__(f"{where + ': ' if where else ''}rk status {self.status}: {text}")


class DimensionMismatch(RKError, ValueError):
    """Julia's DimensionMismatch."""


class UnsupportedError(RKError, NotImplementedError):
    """The request is legal Julia but the library declines it: an operation outside the enumerated native set, an
    extent beyond what the kernels index (RK_ERR_TOO_LARGE), a workspace the call cannot use (RK_ERR_WORKSPACE).
    A binding inside AMDGPU.jl answers all three by running the stock method; this mirror has no stock method, so
    it raises the one exception type a caller catches to take another path.  `status` tells the three apart."""


class WaitError(RKError):
    """RK_ERR_WAIT: a kernel gave up a bounded wait, so the results of that call are meaningless.  Raised where the
    mirror synchronises anyway (``Array(x)``, a scalar fetch); the workspace has been prepared again by then."""


DECLINED = (RK_ERR_UNSUPPORTED, RK_ERR_TOO_LARGE, RK_ERR_WORKSPACE)


def check(status: int, where: str = "") -> None:
    if status == RK_SUCCESS:
        return
    if status == RK_ERR_DIMENSION:
        raise DimensionMismatch(status, where)
    if status in DECLINED:
        raise UnsupportedError(status, where)
    if status == RK_ERR_WAIT:
        raise WaitError(status, where)
    raise RKError(status, where)


def shape_array(shape):
    n = len(shape)
    arr = (C.c_int64 * max(n, 1))(*[int(s) for s in shape])
    return arr
