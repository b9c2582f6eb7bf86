"""TEST INFRASTRUCTURE ONLY: runs the reference's OWN generated C kernels
(oracle/_ref/libmegcc_ref.so, built by `make -C oracle ref` from /root/reference) on host arrays.

The calling sequence is the one the reference's unit-test proxy uses
(compiler/test/kernel/common/src/cc_proxy.cpp:125-255): S_workspace -> allocate -> three-phase
S_init (count, describe, transform; runtime/src/init.c:94-131) -> swap the processed weight in by
name -> S(inputs, outputs, workspace, opt=NULL).
"""
import ctypes as C
import os
import subprocess

import numpy as np

from megcc_amd import abi

_HERE = os.path.dirname(os.path.abspath(__file__))
_PATH = os.path.join(_HERE, "_ref", "libmegcc_ref.so")
_LIB = None


def build():
    subprocess.check_call(["make", "-s", "-C", _HERE, "ref"])


def available():
    return os.path.exists(_PATH)


def lib():
    global _LIB
    if _LIB is None:
        _LIB = C.CDLL(_PATH)
    return _LIB


def has(symbol):
    return available() and hasattr(lib(), symbol)


def run(symbol, inputs, outputs):
    """inputs/outputs: lists of abi.Tensor over host memory. Returns nothing; outputs are
    written in place."""
    L = lib()
    kern = getattr(L, symbol)
    kern.argtypes = abi.KERNEL_ARGS
    kern.restype = C.c_int
    keep = []
    inputs = list(inputs)

    ws = abi.Workspace()
    ws_fn = getattr(L, symbol + "_workspace", None)
    size = C.c_size_t(0)
    if ws_fn is not None:
        ws_fn.argtypes = abi.WORKSPACE_ARGS
        ws_fn.restype = C.c_int
        st = ws_fn(abi.tensor_array(inputs), len(inputs), 1, C.byref(size))
        assert st == 0, "%s_workspace -> %d" % (symbol, st)
    # some GI kernels assert on a non-NULL workspace pointer they never use
    ws_buf = np.zeros(max(int(size.value), 64), np.uint8)
    keep.append(ws_buf)
    ws.ptr = ws_buf.ctypes.data
    ws.size = int(size.value)

    init_fn = getattr(L, symbol + "_init", None)
    if init_fn is not None:
        init_fn.argtypes = abi.INIT_ARGS
        init_fn.restype = C.c_int
        n_out = C.c_int(0)
        st = init_fn(abi.tensor_array(inputs), len(inputs), None, C.byref(n_out), None)
        assert st == 0
        if n_out.value:
            assert n_out.value == 1
            w = abi.Tensor()
            st = init_fn(abi.tensor_array(inputs), len(inputs), C.byref(w), None, None)
            assert st == 0
            nelem = 1
            for i in range(w.layout.nr_dim):
                nelem *= w.layout.dims[i]
            buf = np.zeros(nelem * abi.np_dtype(w.dtype.type_enum).itemsize, np.uint8)
            keep.append(buf)
            w.ptr = buf.ctypes.data
            st = init_fn(abi.tensor_array(inputs), len(inputs), C.byref(w), C.byref(n_out), None)
            assert st == 0
            for i, t in enumerate(inputs):
                if t.name == w.name:
                    inputs[i] = w
    st = kern(abi.tensor_array(inputs), len(inputs), abi.tensor_array(outputs), len(outputs),
              C.byref(ws), None)
    assert st == 0, "%s -> %d" % (symbol, st)


_MEMPLAN_PATH = os.path.join(_HERE, "_ref", "libmegcc_ref_memplan.so")
_MEMPLAN = None


def memplan_available():
    return os.path.exists(_MEMPLAN_PATH)


def plan_memory(begin, end, size, alignment=1):
    """The reference's own StaticMemAlloc (PUSHDOWN) on these requests, through
    oracle/ref_memplan.cpp. Returns (offsets, arena_bytes, lower_bound). The reference aborts the
    process on requests it rejects (begin >= end, alignment not a power of two)."""
    global _MEMPLAN
    if _MEMPLAN is None:
        _MEMPLAN = C.CDLL(_MEMPLAN_PATH)
    arrs = [np.ascontiguousarray(a, dtype=np.uint64) for a in (begin, end, size)]
    n = len(arrs[0])
    off = np.zeros(max(n, 1), np.uint64)
    total, bound = C.c_size_t(0), C.c_size_t(0)
    ptr = lambda a: a.ctypes.data_as(C.POINTER(C.c_size_t))
    st = _MEMPLAN.ref_plan_memory(
        C.c_size_t(n), ptr(arrs[0]), ptr(arrs[1]), ptr(arrs[2]), C.c_size_t(alignment), ptr(off),
        C.byref(total), C.byref(bound))
    assert st == 0
    return off[:n].astype(np.int64), int(total.value), int(bound.value)


_TINY_DUMP = os.path.join(_HERE, "_ref", "ref_tiny_dump")


def tiny_dump_available():
    return os.path.exists(_TINY_DUMP)


def tiny_dump(path):
    """What the reference's generated FlatBuffers reader sees in the `.tiny` file at `path`
    (oracle/ref_tiny_dump.c), as text."""
    return subprocess.run([_TINY_DUMP, path], check=True, capture_output=True, text=True).stdout
