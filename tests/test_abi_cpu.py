"""CPU-only checks of the C ABI: librk.so loads, exports every symbol include/rk.h declares, and rejects
bad arguments with status codes before touching the GPU (no compute call is made here)."""
import ctypes as C
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "rk.h")


@pytest.fixture(scope="module")
def L(rk):
    from amdgpu_jl_amd import _lib
    return _lib


def _declared_symbols():
    text = open(HEADER).read()
    return re.findall(r"RK_API\s+[\w\s\*]+?\b(rk_\w+)\s*\(", text)


def test_header_symbols_are_exported_and_bound(L):
    names = _declared_symbols()
    assert len(names) >= 10 and len(set(names)) == len(names)
    raw = C.CDLL(L.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), f"librk.so does not export {n}"
        assert n in L.PROTOTYPES, f"the ctypes binding lacks {n}"
    assert set(L.PROTOTYPES) == set(names)


def test_only_c_abi_symbols_are_public(L):
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", L.LIB_PATH], capture_output=True, text=True, check=True).stdout
    public = {l.split()[-1] for l in out.splitlines() if " T " in l}
    assert {s for s in public if s.startswith("rk_")} == set(_declared_symbols())
    assert not [s for s in public if "rk" in s and not s.startswith("rk_") and not s.startswith("_")]


def test_header_constants_match_binding(L):
    text = open(HEADER).read()
    for name in ("RK_ERR_INVALID_ARGUMENT", "RK_ERR_UNSUPPORTED", "RK_ERR_WORKSPACE", "RK_ERR_DIMENSION", "RK_ERR_TOO_LARGE", "RK_ERR_WAIT"):
        assert int(re.search(name + r"\s*=\s*(\d+)", text).group(1)) == getattr(L, name)
    assert int(re.search(r"#define RK_MAX_DIMS (\d+)", text).group(1)) == L.RK_MAX_DIMS
    assert int(re.search(r"#define RK_MAX_OPERANDS (\d+)", text).group(1)) == L.RK_MAX_OPERANDS
    assert int(re.search(r"#define RK_MAX_PROGRAM (\d+)", text).group(1)) == L.RK_MAX_PROGRAM
    assert int(re.search(r"#define RK_VERSION (\d+)", text).group(1)) == L.lib.rk_version()
    assert int(re.search(r"RK_BC_ADD = (\d+)", text).group(1)) == L.RK_BC_ADD
    assert int(re.search(r"RK_BC_NEG = (\d+)", text).group(1)) == L.RK_BC_NEG


def test_status_strings(L):
    assert L.lib.rk_status_string(0) == b"RK_SUCCESS"
    for code in (L.RK_ERR_INVALID_ARGUMENT, L.RK_ERR_UNSUPPORTED, L.RK_ERR_WORKSPACE, L.RK_ERR_DIMENSION, L.RK_ERR_TOO_LARGE, L.RK_ERR_WAIT):
        assert L.lib.rk_status_string(code).startswith(b"RK_ERR_")
    assert L.lib.rk_status_string(424242) == b"unknown rk status"


def test_mapreduce_argument_validation(L):
    sh = L.shape_array((10,))
    one = C.c_void_p(0x1000)                  # never dereferenced: validation fails first
    f = L.lib.rk_mapreduce
    assert f(0, 0, L.RK_F32, L.RK_F32, None, 1, sh, 1, None, None, None, 0, None) == L.RK_ERR_INVALID_ARGUMENT   # null arrays
    assert f(0, 9, L.RK_F32, L.RK_F32, one, 1, sh, 1, one, None, None, 0, None) == L.RK_ERR_INVALID_ARGUMENT     # bad op
    assert f(7, 0, L.RK_F32, L.RK_F32, one, 1, sh, 1, one, None, None, 0, None) == L.RK_ERR_INVALID_ARGUMENT     # bad map
    assert f(0, 0, 99, L.RK_F32, one, 1, sh, 1, one, None, None, 0, None) == L.RK_ERR_INVALID_ARGUMENT           # bad dtype
    assert f(0, 0, L.RK_F32, L.RK_F32, one, 9, sh, 1, one, None, None, 0, None) == L.RK_ERR_INVALID_ARGUMENT     # ndim > 8
    assert f(0, 0, L.RK_F32, L.RK_F32, one, 1, L.shape_array((-1,)), 1, one, None, None, 0, None) == L.RK_ERR_INVALID_ARGUMENT
    assert f(0, 0, L.RK_F32, L.RK_I32, one, 1, sh, 1, one, None, None, 0, None) == L.RK_ERR_UNSUPPORTED           # Float32 -> Int32
    assert f(0, 0, L.RK_I16, L.RK_F32, one, 1, sh, 1, one, None, None, 0, None) == L.RK_ERR_UNSUPPORTED           # Int16 -> Float32
    assert f(0, 0, L.RK_I8, L.RK_I32, one, 1, sh, 1, one, None, None, 0, None) == L.RK_ERR_UNSUPPORTED            # Int8 sums widen to Int64 only
    # zero-length input: success without launching (src/kernels/mapreduce.jl:91), even with null pointers
    assert f(0, 0, L.RK_F32, L.RK_F32, None, 1, L.shape_array((0,)), 1, None, None, None, 0, None) == L.RK_SUCCESS
    # a reduction that needs partials but has no workspace
    big = L.shape_array((1 << 24,))
    assert f(0, 0, L.RK_F32, L.RK_F32, one, 1, big, 1, one, None, None, 0, None) == L.RK_ERR_WORKSPACE
    assert f(0, 0, L.RK_F32, L.RK_F32, one, 1, big, 1, one, None, C.c_void_p(0x1001), 1 << 30, None) == L.RK_ERR_WORKSPACE   # misaligned


def test_findminmax_and_accumulate_validation(L):
    sh = L.shape_array((4, 4))
    one = C.c_void_p(0x1000)
    g = L.lib.rk_findminmax
    assert g(1, L.RK_F32, None, 2, sh, 1, one, one, None, 0, None) == L.RK_ERR_INVALID_ARGUMENT
    assert g(1, L.RK_F32, one, 2, sh, 1, None, None, None, 0, None) == L.RK_ERR_INVALID_ARGUMENT      # no output requested
    assert g(1, 99, one, 2, sh, 1, one, one, None, 0, None) == L.RK_ERR_INVALID_ARGUMENT                # no such element type
    assert g(1, L.RK_F32, None, 2, L.shape_array((0, 4)), 1, None, None, None, 0, None) == L.RK_SUCCESS
    gs = L.lib.rk_findminmax_strided
    tr = L.shape_array((4, 1))                                   # a 4 x 4 transpose: strides (4, 1)
    assert gs(1, L.RK_F32, None, 2, sh, tr, 1, one, one, None, 0, None) == L.RK_ERR_INVALID_ARGUMENT
    assert gs(1, L.RK_F32, one, 2, sh, tr, 1, None, None, None, 0, None) == L.RK_ERR_INVALID_ARGUMENT
    assert gs(1, L.RK_F32, one, 2, sh, L.shape_array((2, 8)), 1, one, one, None, 0, None) == L.RK_ERR_UNSUPPORTED     # a view with gaps
    assert gs(1, L.RK_F32, one, 2, sh, tr, 3, one, one, None, 0, None) == L.RK_ERR_UNSUPPORTED    # dims=: of a transpose: the first of equal winners differs
    assert gs(1, L.RK_F32, None, 2, L.shape_array((0, 4)), tr, 1, None, None, None, 0, None) == L.RK_SUCCESS
    a = L.lib.rk_accumulate
    assert a(0, L.RK_F32, L.RK_F32, None, one, 2, sh, 1, 1, None, None, 0, None) == L.RK_ERR_INVALID_ARGUMENT
    assert a(0, L.RK_F32, L.RK_F32, one, one, 2, sh, 0, 1, None, None, 0, None) == L.RK_ERR_INVALID_ARGUMENT   # dim is 1-based
    assert a(7, L.RK_F32, L.RK_F32, one, one, 2, sh, 1, 1, None, None, 0, None) == L.RK_ERR_INVALID_ARGUMENT   # no such operator
    assert a(L.RK_OP_XOR, L.RK_F32, L.RK_F32, one, one, 2, sh, 1, 1, None, None, 0, None) == L.RK_ERR_UNSUPPORTED        # bitwise: integers only
    m = L.lib.rk_mapreduce
    assert m(0, L.RK_OP_AND, L.RK_I32, L.RK_I32, one, 2, sh, 1, one, None, None, 0, None) == L.RK_ERR_UNSUPPORTED        # and in scans only
    assert a(2, L.RK_F32, L.RK_F32, one, one, 2, sh, 1, 0, None, None, 0, None) == L.RK_ERR_INVALID_ARGUMENT   # exclusive max needs init
    assert a(0, L.RK_F32, L.RK_F64, one, C.c_void_p(0x3000), 2, sh, 1, 1, None, None, 0, None) == L.RK_ERR_UNSUPPORTED
    for narrow in (L.RK_I8, L.RK_I16, L.RK_U16, L.RK_F16):                      # narrow scans are native, but only into their own type
        assert a(0, narrow, L.RK_I32, one, C.c_void_p(0x3000), 2, sh, 1, 1, None, None, 0, None) == L.RK_ERR_UNSUPPORTED
        assert a(0, narrow, narrow, one, C.c_void_p(0x3000), 2, L.shape_array((0, 4)), 1, 1, None, None, 0, None) == L.RK_SUCCESS
    assert a(0, L.RK_U8, L.RK_I64, one, one, 2, sh, 1, 1, None, None, 0, None) == L.RK_ERR_INVALID_ARGUMENT    # aliasing with different sizes
    assert a(0, L.RK_F32, L.RK_F32, None, None, 1, L.shape_array((0,)), 1, 1, None, None, 0, None) == L.RK_SUCCESS
    # a look-back scan without workspace
    assert a(0, L.RK_I32, L.RK_I32, one, C.c_void_p(0x2000), 1, L.shape_array((1 << 24,)), 1, 1, None, None, 0, None) == L.RK_ERR_WORKSPACE


def _prog(L, tokens, operands, compute=None):
    p = L.RkProgram()
    p.compute = L.RK_F32 if compute is None else compute
    p.n_operands = len(operands)
    for k, (ptr, dt, shape) in enumerate(operands):
        p.operands[k].ptr = ptr
        p.operands[k].dtype = dt
        p.operands[k].ndim = len(shape)
        for d, n in enumerate(shape):
            p.operands[k].shape[d] = n
    p.n_tokens = len(tokens)
    for i, t in enumerate(tokens):
        p.tokens[i] = t
    return p


def test_broadcast_program_validation(L):
    b = L.lib.rk_broadcast
    sh = L.shape_array((4, 3))
    dest = C.c_void_p(0x1000)
    arr = lambda *s: (0x2000, L.RK_F32, s)
    assert b(None, dest, L.RK_F32, 2, sh, None) == L.RK_ERR_INVALID_ARGUMENT
    ok_ops = [arr(4, 3), arr(4, 3)]
    assert b(_prog(L, [0, 1], ok_ops), dest, L.RK_F32, 2, sh, None) == L.RK_ERR_INVALID_ARGUMENT              # two values left
    assert b(_prog(L, [0, L.RK_BC_ADD], ok_ops), dest, L.RK_F32, 2, sh, None) == L.RK_ERR_INVALID_ARGUMENT    # stack underflow
    assert b(_prog(L, [0, 5, L.RK_BC_ADD], ok_ops), dest, L.RK_F32, 2, sh, None) == L.RK_ERR_INVALID_ARGUMENT  # operand 5 missing
    assert b(_prog(L, [0, 1, 999], ok_ops), dest, L.RK_F32, 2, sh, None) == L.RK_ERR_INVALID_ARGUMENT          # unknown token
    assert b(_prog(L, [0, 1, L.RK_BC_ADD], ok_ops, compute=L.RK_I32), dest, L.RK_F32, 2, sh, None) == L.RK_ERR_UNSUPPORTED
    assert b(_prog(L, [0, 1, L.RK_BC_ADD], [arr(4, 3), arr(3, 3)]), dest, L.RK_F32, 2, sh, None) == L.RK_ERR_DIMENSION
    assert b(_prog(L, [0, 1, L.RK_BC_ADD], [arr(4, 3), arr(4, 3, 2)]), dest, L.RK_F32, 2, sh, None) == L.RK_ERR_DIMENSION
    assert b(_prog(L, [0, 1, L.RK_BC_ADD], ok_ops), None, L.RK_F32, 2, sh, None) == L.RK_ERR_INVALID_ARGUMENT  # null dest
    deep = [0] * 9 + [L.RK_BC_ADD] * 8
    assert b(_prog(L, deep, ok_ops), dest, L.RK_F32, 2, sh, None) == L.RK_ERR_UNSUPPORTED                     # stack deeper than 8
    assert b(_prog(L, [0, L.RK_BC_ISODD], ok_ops), dest, L.RK_U8, 2, sh, None) == L.RK_ERR_UNSUPPORTED        # isodd in a Float32 program
    assert b(_prog(L, [0, 1, L.RK_BC_IFELSE], ok_ops), dest, L.RK_F32, 2, sh, None) == L.RK_ERR_INVALID_ARGUMENT   # ifelse pops three
    assert b(_prog(L, [0, 1, L.RK_BC_ADD], [arr(0, 3), arr(0, 3)]), None, L.RK_F32, 2, L.shape_array((0, 3)), None) == L.RK_SUCCESS


def test_mapreduce_program_validation(L):
    m = L.lib.rk_mapreduce_program
    sh = L.shape_array((4, 3))
    A, R = C.c_void_p(0x1000), C.c_void_p(0x2000)

    def prog(tokens, n_consts=1):
        p = L.RkMapProgram()
        p.n_tokens = len(tokens)
        for i, t in enumerate(tokens):
            p.tokens[i] = t
        p.n_consts = n_consts
        return p
    plus1 = [0, 1, L.RK_BC_ADD]
    assert m(None, L.RK_OP_ADD, L.RK_F32, L.RK_F32, A, 2, sh, 1, R, None, None, 0, None) == L.RK_ERR_INVALID_ARGUMENT
    assert m(prog([]), L.RK_OP_ADD, L.RK_F32, L.RK_F32, A, 2, sh, 1, R, None, None, 0, None) == L.RK_ERR_INVALID_ARGUMENT
    assert m(prog(plus1, 5), L.RK_OP_ADD, L.RK_F32, L.RK_F32, A, 2, sh, 1, R, None, None, 0, None) == L.RK_ERR_INVALID_ARGUMENT
    assert m(prog([0, 2, L.RK_BC_ADD]), L.RK_OP_ADD, L.RK_F32, L.RK_F32, A, 2, sh, 1, R, None, None, 0, None) == L.RK_ERR_INVALID_ARGUMENT   # constant 2 missing
    assert m(prog([0, L.RK_BC_ADD]), L.RK_OP_ADD, L.RK_F32, L.RK_F32, A, 2, sh, 1, R, None, None, 0, None) == L.RK_ERR_INVALID_ARGUMENT      # stack underflow
    assert m(prog([0, 1]), L.RK_OP_ADD, L.RK_F32, L.RK_F32, A, 2, sh, 1, R, None, None, 0, None) == L.RK_ERR_INVALID_ARGUMENT                # two values left
    assert m(prog(plus1), 7, L.RK_F32, L.RK_F32, A, 2, sh, 1, R, None, None, 0, None) == L.RK_ERR_INVALID_ARGUMENT
    deep = [0, 0, 0, 0, 0] + [L.RK_BC_ADD] * 4
    assert m(prog(deep), L.RK_OP_ADD, L.RK_F32, L.RK_F32, A, 2, sh, 1, R, None, None, 0, None) == L.RK_ERR_UNSUPPORTED      # value stack deeper than 4
    assert m(prog([0, L.RK_BC_SQRT]), L.RK_OP_ADD, L.RK_I64, L.RK_I64, A, 2, sh, 1, R, None, None, 0, None) == L.RK_ERR_UNSUPPORTED   # sqrt(Int) is a Float64
    assert m(prog([0, L.RK_BC_ISODD]), L.RK_OP_ADD, L.RK_F32, L.RK_I64, A, 2, sh, 1, R, None, None, 0, None) == L.RK_ERR_UNSUPPORTED
    assert m(prog(plus1), L.RK_OP_ADD, L.RK_F32, L.RK_F64, A, 2, sh, 1, R, None, None, 0, None) == L.RK_ERR_UNSUPPORTED     # no such type pair
    assert m(prog(plus1), L.RK_OP_ADD, L.RK_F32, L.RK_F32, None, 2, sh, 1, R, None, None, 0, None) == L.RK_ERR_INVALID_ARGUMENT
    assert m(prog(plus1), L.RK_OP_ADD, L.RK_F32, L.RK_F32, None, 2, L.shape_array((0, 3)), 1, None, None, None, 0, None) == L.RK_SUCCESS   # mapreduce.jl:91


def test_volumerhs_and_scatter_validation(L):
    v = L.lib.rk_volumerhs_f32
    one = C.c_void_p(0x1000)
    assert v(None, one, one, 9.81, one, 10, None) == L.RK_ERR_INVALID_ARGUMENT
    assert v(one, one, one, 9.81, one, -1, None) == L.RK_ERR_INVALID_ARGUMENT
    assert v(None, None, None, 9.81, None, 0, None) == L.RK_SUCCESS
    s = L.lib.rk_findall_scatter
    assert s(None, one, one, 1, L.shape_array((5,)), None) == L.RK_ERR_INVALID_ARGUMENT
    assert s(None, None, None, 1, L.shape_array((0,)), None) == L.RK_SUCCESS
    assert s(one, one, one, 9, L.shape_array((5,)), None) == L.RK_ERR_INVALID_ARGUMENT
    two = C.c_void_p(0x2000)
    r = L.lib.rk_reverse
    assert r(None, one, 4, 1, L.shape_array((5,)), 1, None) == L.RK_ERR_INVALID_ARGUMENT
    assert r(one, one, 3, 1, L.shape_array((5,)), 1, None) == L.RK_ERR_UNSUPPORTED
    assert r(one, one, 4, 9, L.shape_array((5,)), 1, None) == L.RK_ERR_INVALID_ARGUMENT
    assert r(C.c_void_p(0x1002), one, 4, 1, L.shape_array((5,)), 1, None) == L.RK_ERR_INVALID_ARGUMENT   # misaligned for the element
    assert r(None, None, 4, 1, L.shape_array((0,)), 1, None) == L.RK_SUCCESS
    assert r(one, one, 4, 2, L.shape_array((5, 1)), 2, None) == L.RK_SUCCESS          # reverse! of an extent of 1: nothing to do
    pm = L.lib.rk_permutedims
    i32 = lambda *v: (C.c_int32 * len(v))(*v)
    assert pm(one, two, 4, 2, L.shape_array((5, 6)), i32(2, 2), None) == L.RK_ERR_INVALID_ARGUMENT     # not a permutation
    assert pm(one, two, 4, 2, L.shape_array((5, 6)), i32(0, 1), None) == L.RK_ERR_INVALID_ARGUMENT
    assert pm(one, one, 4, 2, L.shape_array((5, 6)), i32(2, 1), None) == L.RK_ERR_INVALID_ARGUMENT     # in place is not defined
    assert pm(one, two, 5, 2, L.shape_array((5, 6)), i32(2, 1), None) == L.RK_ERR_UNSUPPORTED
    assert pm(None, None, 4, 2, L.shape_array((0, 6)), i32(2, 1), None) == L.RK_SUCCESS
    so, sp, tb = L.lib.rk_sort, L.lib.rk_sortperm, L.lib.rk_sort_tmp_bytes
    big = C.c_void_p(0x10000)
    assert so(L.RK_F32, None, 10, 0, big, 1 << 30, None) == L.RK_ERR_INVALID_ARGUMENT
    assert so(L.RK_U8, one, 10, 0, big, 1 << 30, None) == L.RK_ERR_UNSUPPORTED
    assert so(99, one, 10, 0, big, 1 << 30, None) == L.RK_ERR_INVALID_ARGUMENT
    assert so(L.RK_F32, one, -1, 0, big, 1 << 30, None) == L.RK_ERR_INVALID_ARGUMENT
    assert so(L.RK_F32, one, 10, 0, None, 0, None) == L.RK_ERR_WORKSPACE
    assert so(L.RK_F32, one, 10, 0, big, 16, None) == L.RK_ERR_WORKSPACE
    assert so(L.RK_F32, one, 1 << 31, 0, big, 1 << 40, None) == L.RK_ERR_TOO_LARGE
    assert so(L.RK_F32, None, 0, 0, None, 0, None) == L.RK_SUCCESS
    assert sp(L.RK_I64, one, None, 10, 0, big, 1 << 30, None) == L.RK_ERR_INVALID_ARGUMENT
    n = 1 << 20
    assert tb(L.RK_F32, n, 0) >= 4 * n and tb(L.RK_F32, n, 1) >= 16 * n and tb(L.RK_F32, n, 0) < 5 * n
    assert tb(L.RK_I64, n, 0) >= 8 * n and tb(L.RK_I16, n, 0) >= 2 * n and tb(L.RK_U8, n, 0) == 256
    ga = L.lib.rk_gather_slices
    assert ga(None, one, two, 4, 3, 5, 7, None) == L.RK_ERR_INVALID_ARGUMENT
    assert ga(one, one, two, 3, 3, 5, 7, None) == L.RK_ERR_UNSUPPORTED
    assert ga(one, one, two, 4, -1, 5, 7, None) == L.RK_ERR_INVALID_ARGUMENT
    assert ga(None, None, None, 4, 3, 0, 7, None) == L.RK_SUCCESS
    f = L.lib.rk_findall
    assert f(None, 1, L.shape_array((5,)), one, None, two, 16 << 20, None) == L.RK_ERR_INVALID_ARGUMENT
    assert f(one, 1, L.shape_array((5,)), None, None, two, 16 << 20, None) == L.RK_ERR_INVALID_ARGUMENT
    assert f(one, 9, L.shape_array((5,)), one, None, two, 16 << 20, None) == L.RK_ERR_INVALID_ARGUMENT
    assert f(one, 1, L.shape_array((-5,)), one, None, two, 16 << 20, None) == L.RK_ERR_INVALID_ARGUMENT
    assert f(one, 1, L.shape_array((5,)), one, None, None, 0, None) == L.RK_ERR_WORKSPACE
    assert f(None, 1, L.shape_array((0,)), None, None, None, 0, None) == L.RK_SUCCESS


def test_workspace_queries(L):
    wb = L.lib.rk_workspace_bytes
    base = wb(L.RK_KIND_MAPREDUCE, L.RK_F32, 1, L.shape_array((1 << 20,)), 1)
    assert base % 256 == 0 and base <= (16 << 20)          # RK_WORKSPACE_DEFAULT serves it
    small = wb(L.RK_KIND_ACCUMULATE, L.RK_I32, 1, L.shape_array((1000,)), 1)
    big = wb(L.RK_KIND_ACCUMULATE, L.RK_I32, 1, L.shape_array((1 << 27,)), 1)
    assert small == base and big > base and big <= (16 << 20)
    assert wb(L.RK_KIND_ACCUMULATE, L.RK_F32, 2, L.shape_array((4096, 16384)), 1) == base     # lines fit one tile: no descriptors
    assert wb(L.RK_KIND_FINDALL, L.RK_U8, 1, L.shape_array((1 << 31,)), 0) <= (16 << 20)
    assert wb(L.RK_KIND_FINDALL, L.RK_U8, 1, L.shape_array((1 << 26,)), 0) > base
    assert wb(L.RK_KIND_ACCUMULATE, 99, 1, None, 0) == base                                    # bad arguments: the generic minimum
    wi = L.lib.rk_workspace_init
    assert wi(None, 1 << 24, None) == L.RK_ERR_INVALID_ARGUMENT
    assert wi(C.c_void_p(0x1001), 1 << 24, None) == L.RK_ERR_WORKSPACE
    assert wi(C.c_void_p(0x1000), 1024, None) == L.RK_ERR_WORKSPACE


def test_strided_entry_points_reject_what_is_not_permuted_dense(L):
    ws, A, R = C.c_void_p(0x10000000), C.c_void_p(0x20000000), C.c_void_p(0x30000000)
    shp = L.shape_array((40, 30))
    for strides in ((1, 80), (2, 80), (1, 20), (-1, 40), (0, 1), (1, 1)):          # gaps, steps, overlap, reversal, repetition
        st = L.lib.rk_mapreduce_strided(L.RK_MAP_IDENTITY, L.RK_OP_ADD, L.RK_F32, L.RK_F32, A, 2, shp, L.shape_array(strides), 1, R, None,
                                        None, ws, 16 << 20, None)
        assert st == L.RK_ERR_UNSUPPORTED, strides
        st = L.lib.rk_accumulate_strided(L.RK_OP_ADD, L.RK_F32, L.RK_F32, A, R, 2, shp, L.shape_array(strides), L.shape_array(strides), 1, 1,
                                         None, ws, 16 << 20, None)
        assert st == L.RK_ERR_UNSUPPORTED, strides
    # input and output of a scan laid out differently
    st = L.lib.rk_accumulate_strided(L.RK_OP_ADD, L.RK_F32, L.RK_F32, A, R, 2, shp, L.shape_array((30, 1)), None, 1, 1, None, ws, 16 << 20, None)
    assert st == L.RK_ERR_UNSUPPORTED
    assert L.lib.rk_mapreduce_strided(L.RK_MAP_IDENTITY, L.RK_OP_ADD, L.RK_F32, L.RK_F32, None, 2, shp, None, 1, R, None, None, ws, 16 << 20,
                                      None) == L.RK_ERR_INVALID_ARGUMENT
    assert L.lib.rk_mapreduce_strided(L.RK_MAP_IDENTITY, L.RK_OP_ADD, L.RK_F32, L.RK_F32, None, 1, L.shape_array((0,)), None, 1, None, None, None,
                                      None, 0, None) == 0


def test_long_outer_extents_are_not_rejected(L):
    """Shapes whose outer extent exceeds 65535 (the y / z limit of a grid) pass validation and planning: with no device
    the call then stops at the launch with a HIP error, never with RK_ERR_TOO_LARGE.  Only meaningful -- and only safe,
    the pointers are made up -- on a machine without a GPU; the GPU suite runs the same shapes on real arrays."""
    import torch
    if torch.cuda.device_count() > 0:
        pytest.skip("a device is present: the same shapes run for real in tests/test_large_gpu.py")
    ws, A, R = C.c_void_p(0x10000000), C.c_void_p(0x20000000), C.c_void_p(0x30000000)
    for shape in ((64, 2, 70000), (64, 5, 70000), (100, 3, 111848), (256, 2, 65536)):
        for dt in (L.RK_F32, L.RK_F64, L.RK_I32):
            st = L.lib.rk_mapreduce(L.RK_MAP_IDENTITY, L.RK_OP_ADD, dt, dt, A, 3, L.shape_array(shape), 2, R, None, ws, 16 << 20, None)
            assert 0 < st < 10000, (shape, dt, st)                      # a hipError_t: no device
        st = L.lib.rk_findminmax(1, L.RK_F32, A, 3, L.shape_array(shape), 2, R, None, ws, 16 << 20, None)
        assert 0 < st < 10000, (shape, st)
    for shape in ((64, 64, 70000), (1000, 3, 112625), (2048, 4, 100000)):
        st = L.lib.rk_accumulate(L.RK_OP_ADD, L.RK_F32, L.RK_F32, A, R, 3, L.shape_array(shape), 2, 1, None, ws, 16 << 20, None)
        assert 0 < st < 10000, (shape, st)
    # a U8 -> I64 scan is sized by its OUTPUT type: two descriptor words per tile
    shp = L.shape_array((1 << 27,))
    assert L.lib.rk_workspace_bytes(L.RK_KIND_ACCUMULATE, L.RK_I64, 1, shp, 1) > L.lib.rk_workspace_bytes(L.RK_KIND_ACCUMULATE, L.RK_I32, 1, shp, 1)


def test_host_mirror_rules_without_gpu(rk):
    """Host-side logic of the mirror that needs no device: eltype rules, broadcast shapes, program flattening."""
    assert rk.reduce_eltype("add_sum", np.int32) == np.int64 and rk.reduce_eltype("add", np.int32) == np.int32
    assert rk.accumulate_eltype("add", np.bool_) == np.int64 and rk.accumulate_eltype("add", np.int32) == np.int32
    from amdgpu_jl_amd import broadcast as B
    assert B.broadcast_shape((2, 3), (2,)) == (2, 3)
    with pytest.raises(rk.DimensionMismatch):
        B.broadcast_shape((2, 3), (3,))
    a = np.float32(0.5)
    toks = B._compile(a * B.lazy(1.0) + B.lazy(2.0) * B.exp(B.lazy(3.0)))[1]
    from amdgpu_jl_amd import _lib as L
    assert toks == [0, 1, L.RK_BC_MUL, 2, 3, L.RK_BC_EXP, L.RK_BC_MUL, L.RK_BC_ADD]
    with pytest.raises(rk.UnsupportedError):
        B.broadcasted("besselj", 1.0)
    # a NumPy Float32 scalar on the left keeps its type (0.5f0 .* x computes in Float32, not Float64)
    assert B._compile(np.float32(0.5) * B.lazy(np.float32(2.0)))[2] == np.float32
    assert B._compile(0.5 * B.lazy(np.float32(2.0)))[2] == np.float64
    # Julia's promotion, not NumPy's: Int64 with Float32 is Float32; Int32 with UInt32 is UInt32
    assert B.promote_type(np.int64, np.float32) == np.float32 and B.promote_type(np.int32, np.uint32) == np.uint32
    assert B.promote_type(np.bool_, np.int32) == np.int32 and B.promote_type(np.int64, np.uint32) == np.int64
    # closures of mapreduce(f, op, A) traced on a symbolic element: tokens, constants, eltype of f(x), compute type
    toks, consts, elt, comp = B.compile_map(lambda x: x + 1, np.float32)
    assert toks == [0, 1, L.RK_BC_ADD] and consts == [1] and elt == np.float32 and comp == np.float32
    toks, consts, elt, comp = B.compile_map(lambda x: x + 1, np.int32)
    assert elt == np.int64 and comp == np.int64 and toks == [0, 1, L.RK_BC_ADD]
    toks, consts, elt, comp = B.compile_map(lambda x: x * x > 0, np.int32)          # the comparison needs the wrapped square
    assert elt == np.bool_ and toks == [0, 0, L.RK_BC_MUL, L.RK_BC_WRAP_I32, 1, L.RK_BC_GT]
    toks, _, elt, _ = B.compile_map(lambda x: x * x, np.int32)                      # and so does a widening reduction
    assert elt == np.int32 and toks == [0, 0, L.RK_BC_MUL, L.RK_BC_WRAP_I32]
    assert B.compile_map(lambda x: B.isodd(x), np.int64)[2] == np.bool_
    assert B.compile_map(lambda x: x, np.float64)[0] == [0]
    with pytest.raises(rk.UnsupportedError):
        B.compile_map(lambda x: B.isodd(x), np.float32)
    assert B._compile(B.lazy(np.float32(1)) > B.lazy(2))[4] == np.bool_


def test_declined_statuses_raise_the_fallback_exception(L):
    """Out-of-set operations, extents beyond the kernels' indexing and unusable workspaces are all `declined`: the one
    exception a caller catches to take another path (the Julia binding runs the stock method for the same three)."""
    for code in (L.RK_ERR_UNSUPPORTED, L.RK_ERR_TOO_LARGE, L.RK_ERR_WORKSPACE):
        with pytest.raises(L.UnsupportedError) as e:
            L.check(code, "probe")
        assert e.value.status == code
    for code in (L.RK_ERR_INVALID_ARGUMENT, L.RK_ERR_WAIT):
        with pytest.raises(L.RKError) as e:
            L.check(code, "probe")
        assert not isinstance(e.value, L.UnsupportedError)
    with pytest.raises(L.DimensionMismatch):
        L.check(L.RK_ERR_DIMENSION, "probe")
