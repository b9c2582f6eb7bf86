"""ctypes front-end of libmegcc_gfx950.so: prototypes, device buffers, and a helper that runs one
operator through the uniform kernel ABI (workspace -> three-phase init -> kernel), the calling
sequence of the TinyNN runtime (runtime/src/init.c:29-131, runtime/src/vm/op.c:67-172)."""
import ctypes as C
import os

import numpy as np

from . import LIB_PATH, abi  # noqa: F401

_lib = None


class MegccError(RuntimeError):
    pass


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise MegccError(
                "%s is missing: run `python -c 'import __graft_entry__ as g; g.build()'` "
                "(there is no CPU fallback)" % LIB_PATH)
        L = C.CDLL(LIB_PATH)
        kern = abi.KERNEL_ARGS
        L.megcc_gfx950_conv2d.argtypes = [C.POINTER(abi.ConvAttr)] + kern
        L.megcc_gfx950_conv2d_init.argtypes = [C.POINTER(abi.ConvAttr)] + abi.INIT_ARGS
        L.megcc_gfx950_conv2d_workspace.argtypes = [C.POINTER(abi.ConvAttr)] + abi.WORKSPACE_ARGS
        L.megcc_gfx950_conv2d_noalloc.argtypes = [C.POINTER(abi.ConvAttr)] + kern[:4] + kern[5:]
        L.megcc_gfx950_matmul.argtypes = [C.POINTER(abi.MatMulAttr)] + kern
        L.megcc_gfx950_matmul_workspace.argtypes = [C.POINTER(abi.MatMulAttr)] + abi.WORKSPACE_ARGS
        L.megcc_gfx950_pooling.argtypes = [C.POINTER(abi.PoolAttr)] + kern
        L.megcc_gfx950_elemwise_multitype.argtypes = [C.POINTER(C.c_int)] + kern
        L.megcc_gfx950_elemwise.argtypes = [C.POINTER(C.c_int)] + kern
        L.megcc_gfx950_typecvt.argtypes = kern
        L.megcc_gfx950_reduce.argtypes = [C.POINTER(abi.ReduceAttr)] + kern
        L.megcc_gfx950_relayout.argtypes = kern
        L.megcc_gfx950_concat.argtypes = [C.POINTER(C.c_int)] + kern
        L.megcc_gfx950_resize.argtypes = [C.POINTER(abi.ResizeAttr)] + kern
        L.megcc_gfx950_fused_elemwise.argtypes = [C.POINTER(abi.FusedElemwiseAttr)] + kern
        L.megcc_gfx950_parse_symbol.argtypes = [C.c_char_p, C.POINTER(abi.KernelDesc)]
        L.megcc_gfx950_call.argtypes = [C.POINTER(abi.KernelDesc)] + kern
        L.megcc_gfx950_call_init.argtypes = [C.POINTER(abi.KernelDesc)] + abi.INIT_ARGS
        L.megcc_gfx950_call_workspace.argtypes = [C.POINTER(abi.KernelDesc)] + abi.WORKSPACE_ARGS
        L.megcc_gfx950_init_device.argtypes = [C.POINTER(abi.Device)]
        L.megcc_gfx950_malloc.argtypes = [C.c_size_t]
        L.megcc_gfx950_malloc.restype = C.c_void_p
        L.megcc_gfx950_free.argtypes = [C.c_void_p]
        L.megcc_gfx950_free.restype = None
        L.megcc_gfx950_memcpy_h2d.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        L.megcc_gfx950_memcpy_d2h.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        L.megcc_gfx950_memset.argtypes = [C.c_void_p, C.c_int, C.c_size_t]
        L.megcc_gfx950_wait.argtypes = []
        L.megcc_gfx950_stream.argtypes = []
        L.megcc_gfx950_stream.restype = C.c_void_p
        L.megcc_gfx950_last_error.argtypes = []
        L.megcc_gfx950_last_error.restype = C.c_char_p
        L.megcc_gfx950_last_kernel.argtypes = []
        L.megcc_gfx950_last_kernel.restype = C.c_char_p
        L.megcc_gfx950_set_option.argtypes = [C.c_char_p, C.c_int]
        L.megcc_gfx950_model_create.argtypes = []
        L.megcc_gfx950_model_create.restype = C.c_void_p
        L.megcc_gfx950_model_destroy.argtypes = [C.c_void_p]
        L.megcc_gfx950_model_destroy.restype = None
        dims = C.POINTER(C.c_uint32)
        L.megcc_gfx950_model_add_tensor.argtypes = [C.c_void_p, C.c_char_p, C.c_int, dims, C.c_int, C.c_float]
        L.megcc_gfx950_model_add_weight.argtypes = [C.c_void_p, C.c_char_p, C.c_int, dims, C.c_int, C.c_float, C.c_void_p]
        L.megcc_gfx950_model_add_alias.argtypes = [C.c_void_p, C.c_char_p, C.c_int, C.c_int, dims]
        L.megcc_gfx950_model_add_view.argtypes = [C.c_void_p, C.c_char_p, C.c_int, C.c_int, dims,
                                                  C.POINTER(C.c_int), C.c_size_t]
        ints = C.POINTER(C.c_int)
        L.megcc_gfx950_model_add_opr.argtypes = [C.c_void_p, C.c_char_p, ints, C.c_int, ints, C.c_int]
        L.megcc_gfx950_model_add_opr_desc.argtypes = [C.c_void_p, C.POINTER(abi.KernelDesc), C.c_char_p,
                                                      ints, C.c_int, ints, C.c_int]
        L.megcc_gfx950_model_mark_io.argtypes = [C.c_void_p, C.c_int, C.c_int]
        L.megcc_gfx950_model_finalize.argtypes = [C.c_void_p]
        L.megcc_gfx950_model_arena_bytes.argtypes = [C.c_void_p]
        L.megcc_gfx950_model_arena_bytes.restype = C.c_size_t
        L.megcc_gfx950_model_tensor_ptr.argtypes = [C.c_void_p, C.c_int]
        L.megcc_gfx950_model_tensor_ptr.restype = C.c_void_p
        L.megcc_gfx950_model_set_input.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_size_t]
        L.megcc_gfx950_model_get_output.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_size_t]
        L.megcc_gfx950_model_forward.argtypes = [C.c_void_p]
        L.megcc_gfx950_model_join.argtypes = [C.c_void_p]
        L.megcc_gfx950_model_get_output_async.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_size_t]
        L.megcc_gfx950_model_nr_opr.argtypes = [C.c_void_p]
        L.megcc_gfx950_model_run_opr.argtypes = [C.c_void_p, C.c_int]
        L.megcc_gfx950_model_load.argtypes = [C.c_void_p, C.c_size_t, C.POINTER(C.c_void_p)]
        L.megcc_gfx950_tiny_describe.argtypes = [C.c_void_p, C.c_size_t, C.c_char_p, C.c_size_t,
                                                 C.POINTER(C.c_size_t)]
        sizes = C.POINTER(C.c_size_t)
        L.megcc_gfx950_plan_memory.argtypes = [
            C.c_size_t, sizes, sizes, sizes, C.c_size_t, sizes, sizes, sizes]
        _lib = L
    return _lib


EXPORTS = [
    "megcc_gfx950_conv2d", "megcc_gfx950_conv2d_init", "megcc_gfx950_conv2d_workspace",
    "megcc_gfx950_conv2d_noalloc",
    "megcc_gfx950_matmul", "megcc_gfx950_matmul_workspace", "megcc_gfx950_pooling",
    "megcc_gfx950_elemwise_multitype", "megcc_gfx950_elemwise", "megcc_gfx950_typecvt",
    "megcc_gfx950_softmax", "megcc_gfx950_softmax_max_columns",
    "megcc_gfx950_dw_pool_add", "megcc_gfx950_dw_pool_add_supported",
    "megcc_gfx950_pw_dw", "megcc_gfx950_pw_dw_supported",
    "megcc_gfx950_reduce", "megcc_gfx950_relayout", "megcc_gfx950_concat", "megcc_gfx950_resize", "megcc_gfx950_fused_elemwise",
    "megcc_gfx950_parse_symbol", "megcc_gfx950_call",
    "megcc_gfx950_call_init", "megcc_gfx950_call_workspace", "megcc_gfx950_init_device",
    "megcc_gfx950_malloc", "megcc_gfx950_free", "megcc_gfx950_memcpy_h2d",
    "megcc_gfx950_memcpy_d2h", "megcc_gfx950_memset", "megcc_gfx950_wait",
    "megcc_gfx950_stream", "megcc_gfx950_last_error", "megcc_gfx950_last_kernel",
    "megcc_gfx950_set_option", "megcc_gfx950_requant_affine",
    "megcc_gfx950_model_create", "megcc_gfx950_model_destroy", "megcc_gfx950_model_add_tensor",
    "megcc_gfx950_model_add_weight", "megcc_gfx950_model_add_alias", "megcc_gfx950_model_add_view",
    "megcc_gfx950_model_add_opr", "megcc_gfx950_model_add_opr_desc",
    "megcc_gfx950_model_mark_io", "megcc_gfx950_model_finalize", "megcc_gfx950_model_arena_bytes",
    "megcc_gfx950_model_set_plan", "megcc_gfx950_model_nr_kernel", "megcc_gfx950_model_launch_mode",
    "megcc_gfx950_model_tensor_ptr", "megcc_gfx950_model_set_input",
    "megcc_gfx950_model_get_output", "megcc_gfx950_model_forward", "megcc_gfx950_model_join", "megcc_gfx950_model_nr_tail_kernel", "megcc_gfx950_model_get_output_async", "megcc_gfx950_model_nr_opr",
    "megcc_gfx950_model_run_opr", "megcc_gfx950_plan_memory", "megcc_gfx950_model_load",
    "megcc_gfx950_tiny_describe",
]


def check(status, what=""):
    if status != abi.SUCCESS:
        raise MegccError("%s: TinyNNStatus %d: %s" % (
            what, status, lib().megcc_gfx950_last_error().decode()))


def plan_memory(begin, end, size, alignment=1):
    """Static memory plan (host code only): interval i lives during time steps
    [begin[i], end[i]) and needs size[i] bytes. Returns (offsets, arena_bytes, lower_bound), the
    result of the reference's StaticMemAlloc PUSHDOWN solver on the same requests
    (compiler/lib/Dialect/Kernel/Transforms/migrate/static_mem_alloc.h:26,
    Transforms/StaticMemoryPlanning.cpp:34-96)."""
    arrs = [np.ascontiguousarray(a, dtype=np.uint64) for a in (begin, end, size)]
    n = len(arrs[0])
    assert all(len(a) == n for a in arrs)
    off = np.zeros(max(n, 1), np.uint64)
    total, bound = C.c_size_t(0), C.c_size_t(0)
    ptr = lambda a: a.ctypes.data_as(C.POINTER(C.c_size_t))
    check(lib().megcc_gfx950_plan_memory(
        n, ptr(arrs[0]), ptr(arrs[1]), ptr(arrs[2]), alignment, ptr(off),
        C.byref(total), C.byref(bound)), "plan_memory")
    return off[:n].astype(np.int64), int(total.value), int(bound.value)


def tiny_describe(data):
    """Text listing of a `.tiny` model file (bytes): one line per weight, tensor, instruction."""
    data = bytes(data)
    need = C.c_size_t(0)
    check(lib().megcc_gfx950_tiny_describe(data, len(data), None, 0, C.byref(need)), "tiny_describe")
    buf = C.create_string_buffer(need.value)
    check(lib().megcc_gfx950_tiny_describe(data, len(data), buf, need.value, None), "tiny_describe")
    return buf.value.decode(errors="replace")


class DeviceBuffer:
    """HBM allocation made through the Device.malloc hook of the library."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        self.ptr = lib().megcc_gfx950_malloc(max(self.nbytes, 1))
        if not self.ptr:
            raise MegccError("device malloc of %d bytes failed" % self.nbytes)

    @classmethod
    def from_array(cls, arr):
        arr = np.ascontiguousarray(arr)
        buf = cls(arr.nbytes)
        if arr.nbytes:
            check(lib().megcc_gfx950_memcpy_h2d(buf.ptr, arr.ctypes.data, arr.nbytes), "h2d")
            check(lib().megcc_gfx950_wait(), "wait")
        return buf

    def to_array(self, shape, dtype):
        out = np.empty(shape, dtype)
        assert out.nbytes <= self.nbytes
        if out.nbytes:
            check(lib().megcc_gfx950_memcpy_d2h(out.ctypes.data, self.ptr, out.nbytes), "d2h")
        return out

    def fill(self, value):
        check(lib().megcc_gfx950_memset(self.ptr, value, self.nbytes), "memset")

    def free(self):
        if self.ptr:
            lib().megcc_gfx950_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def wait():
    check(lib().megcc_gfx950_wait(), "wait")


def last_kernel():
    """which kernel variant this thread's most recent operator call selected"""
    return lib().megcc_gfx950_last_kernel().decode()


def requant_affine(act, s_src, s_flt, s_dst):
    """(c, d) of the one-multiply-add requantisation the host proved exact for these scales, or None"""
    c, d = C.c_float(), C.c_float()
    f = lib().megcc_gfx950_requant_affine
    f.argtypes = [C.c_int, C.c_float, C.c_float, C.c_float, C.POINTER(C.c_float), C.POINTER(C.c_float)]
    f.restype = C.c_int
    return (c.value, d.value) if f(act, s_src, s_flt, s_dst, C.byref(c), C.byref(d)) else None


def set_option(name, value):
    """kernel-selection override (megcc_gfx950_set_option)"""
    check(lib().megcc_gfx950_set_option(name.encode(), int(value)), "set_option " + name)


def parse_symbol(symbol):
    desc = abi.KernelDesc()
    check(lib().megcc_gfx950_parse_symbol(symbol.encode(), C.byref(desc)), "parse_symbol " + symbol)
    return desc


class PreparedOp:
    """One operator instance: device tensors, the processed weight from the init protocol, ready
    to be launched repeatedly (what one `Opr` instruction of the TinyNN VM holds)."""

    def __init__(self, desc, in_specs, out_specs):
        L = lib()
        self.desc = desc
        self.keep = []
        self.in_tensors = []
        for s in in_specs:
            buf = DeviceBuffer.from_array(s.array)
            self.keep.append(buf)
            self.in_tensors.append(abi.make_tensor(
                buf.ptr + s.offset * s.array.itemsize, s.shape, s.type_enum, s.scale, s.name,
                s.strides))
        self.out_bufs, self.out_tensors, self.out_specs = [], [], out_specs
        for s in out_specs:
            buf = DeviceBuffer(s.nbytes)
            buf.fill(0x5A)  # poison: an element the kernel fails to write shows up in the compare
            self.out_bufs.append(buf)
            self.out_tensors.append(abi.make_tensor(
                buf.ptr + s.offset * abi.np_dtype(s.type_enum).itemsize, s.shape, s.type_enum,
                s.scale, s.name, s.strides))
        # workspace
        size = C.c_size_t(0)
        ins = abi.tensor_array(self.in_tensors)
        check(L.megcc_gfx950_call_workspace(C.byref(desc), ins, len(self.in_tensors), 1,
                                            C.byref(size)), "workspace")
        self.ws = abi.Workspace()
        self.ws_buf = DeviceBuffer(size.value) if size.value else None
        self.ws.ptr = self.ws_buf.ptr if self.ws_buf else None
        self.ws.size = size.value
        # three-phase init
        n_out = C.c_int(0)
        check(L.megcc_gfx950_call_init(C.byref(desc), ins, len(self.in_tensors), None,
                                       C.byref(n_out), None), "init(count)")
        self.n_processed = n_out.value
        if n_out.value:
            assert n_out.value == 1
            w = abi.Tensor()
            check(L.megcc_gfx950_call_init(C.byref(desc), ins, len(self.in_tensors), C.byref(w),
                                           None, None), "init(describe)")
            nbytes = abi.np_dtype(w.dtype.type_enum).itemsize
            for i in range(w.layout.nr_dim):
                nbytes *= w.layout.dims[i]
            wbuf = DeviceBuffer(nbytes)
            self.keep.append(wbuf)
            w.ptr = wbuf.ptr
            check(L.megcc_gfx950_call_init(C.byref(desc), ins, len(self.in_tensors), C.byref(w),
                                           C.byref(n_out), None), "init(transform)")
            for i, t in enumerate(self.in_tensors):
                if t.name == w.name:
                    self.in_tensors[i] = w
        self.ins = abi.tensor_array(self.in_tensors)
        self.outs = abi.tensor_array(self.out_tensors)

    def launch(self):
        check(lib().megcc_gfx950_call(C.byref(self.desc), self.ins, len(self.in_tensors), self.outs,
                                      len(self.out_tensors), C.byref(self.ws), None), "kernel")

    def launch_noalloc(self):
        """the same convolution through megcc_gfx950_conv2d_noalloc: no workspace argument, the
        library's static scratch array instead"""
        assert self.desc.kind == abi.KERN_CONV
        check(lib().megcc_gfx950_conv2d_noalloc(
            C.byref(self.desc.attr.conv), self.ins, len(self.in_tensors), self.outs,
            len(self.out_tensors), None), "conv2d_noalloc")

    def poison_outputs(self):
        for buf in self.out_bufs:
            buf.fill(0x5A)

    def result(self, i=0):
        s = self.out_specs[i]
        return self.out_bufs[i].to_array(s.storage, abi.np_dtype(s.type_enum))


def run_symbol(symbol, in_specs, out_specs):
    """Run the operator the reference calls `symbol` once and fetch its (first) output."""
    op = PreparedOp(parse_symbol(symbol), in_specs, out_specs)
    op.launch()
    return op.result()


class Model:
    """Python handle of the in-memory model runtime (megcc_gfx950_model_*)."""

    def __init__(self):
        self.h = lib().megcc_gfx950_model_create()
        if not self.h:
            raise MegccError("model_create failed: " + lib().megcc_gfx950_last_error().decode())
        self.shapes = {}

    @classmethod
    def load(cls, data, shapes=None):
        """Model from the bytes of a `.tiny` file (megcc_gfx950_model_load). Tensor ids are the
        file's tensor_pool indices; `shapes` = {id: (shape, dtype enum)} for the tensors get()
        will be asked for."""
        self = cls.__new__(cls)
        self.h = None
        self.shapes = dict(shapes or {})
        data = bytes(data)
        h = C.c_void_p()
        check(lib().megcc_gfx950_model_load(data, len(data), C.byref(h)), "model_load")
        self.h = h.value
        return self

    @staticmethod
    def _dims(shape):
        return (C.c_uint32 * len(shape))(*[int(d) for d in shape])

    def _remember(self, tid, shape, type_enum, what):
        if tid < 0:
            raise MegccError("%s failed: %s" % (what, lib().megcc_gfx950_last_error().decode()))
        self.shapes[tid] = (tuple(shape), type_enum)
        return tid

    def tensor(self, name, shape, type_enum, scale=1.0):
        tid = lib().megcc_gfx950_model_add_tensor(self.h, name.encode(), len(shape), self._dims(shape),
                                                  type_enum, scale)
        return self._remember(tid, shape, type_enum, "add_tensor")

    def weight(self, name, array, type_enum, scale=1.0):
        array = np.ascontiguousarray(array)
        tid = lib().megcc_gfx950_model_add_weight(self.h, name.encode(), array.ndim,
                                                  self._dims(array.shape), type_enum, scale,
                                                  array.ctypes.data)
        return self._remember(tid, array.shape, type_enum, "add_weight")

    def alias(self, name, of, shape):
        tid = lib().megcc_gfx950_model_add_alias(self.h, name.encode(), of, len(shape), self._dims(shape))
        return self._remember(tid, shape, self.shapes[of][1], "add_alias")

    def view(self, name, of, shape, strides, offset=0):
        """strided window into tensor `of`: element strides, first element `offset` elements in"""
        es = abi.np_dtype(self.shapes[of][1]).itemsize
        tid = lib().megcc_gfx950_model_add_view(
            self.h, name.encode(), of, len(shape), self._dims(shape),
            (C.c_int * len(shape))(*[int(s) for s in strides]), C.c_size_t(offset * es))
        return self._remember(tid, shape, self.shapes[of][1], "add_view")

    def opr(self, symbol, inputs, outputs):
        ins = (C.c_int * len(inputs))(*inputs)
        outs = (C.c_int * len(outputs))(*outputs)
        check(lib().megcc_gfx950_model_add_opr(self.h, symbol.encode(), ins, len(inputs), outs,
                                               len(outputs)), "add_opr " + symbol)

    def opr_desc(self, desc, name, inputs, outputs):
        """operator given as a filled KernelDesc (fused elementwise chains have no symbol that
        determines them)"""
        ins = (C.c_int * len(inputs))(*inputs)
        outs = (C.c_int * len(outputs))(*outputs)
        check(lib().megcc_gfx950_model_add_opr_desc(self.h, C.byref(desc), name.encode(), ins,
                                                    len(inputs), outs, len(outputs)), "add_opr_desc " + name)

    def mark_input(self, tid):
        check(lib().megcc_gfx950_model_mark_io(self.h, tid, 0), "mark_io")

    def mark_output(self, tid):
        check(lib().megcc_gfx950_model_mark_io(self.h, tid, 1), "mark_io")

    def set_plan(self, offsets, arena_bytes):
        """the compiler's static memory plan: byte offset per tensor id (entries of weights, inputs
        and views are ignored) and the arena size; finalize() then keeps it instead of planning"""
        L = lib()
        L.megcc_gfx950_model_set_plan.argtypes = [C.c_void_p, C.POINTER(C.c_size_t), C.c_int, C.c_size_t]
        arr = (C.c_size_t * len(offsets))(*[int(o) for o in offsets])
        check(L.megcc_gfx950_model_set_plan(self.h, arr, len(offsets), int(arena_bytes)), "set_plan")

    def finalize(self):
        check(lib().megcc_gfx950_model_finalize(self.h), "finalize")

    @property
    def nr_kernel(self):
        """kernels one forward launches (an operator chain run as one kernel counts once)"""
        L = lib()
        L.megcc_gfx950_model_nr_kernel.argtypes = [C.c_void_p]
        return L.megcc_gfx950_model_nr_kernel(self.h)

    @property
    def nr_tail_kernel(self):
        """how many of those kernels run on the second stream under plain launches (they overlap the
        next forward's first kernels)"""
        L = lib()
        L.megcc_gfx950_model_nr_tail_kernel.argtypes = [C.c_void_p]
        return L.megcc_gfx950_model_nr_tail_kernel(self.h)

    def launch_mode(self):
        """(mode, eager_ms, graph_ms): 1 = graph replay, -1 = one launch per kernel, 0 = undecided"""
        L = lib()
        L.megcc_gfx950_model_launch_mode.argtypes = [C.c_void_p, C.POINTER(C.c_float), C.POINTER(C.c_float)]
        e, g = C.c_float(), C.c_float()
        mode = L.megcc_gfx950_model_launch_mode(self.h, C.byref(e), C.byref(g))
        return mode, e.value, g.value

    @property
    def arena_bytes(self):
        return lib().megcc_gfx950_model_arena_bytes(self.h)

    @property
    def nr_opr(self):
        return lib().megcc_gfx950_model_nr_opr(self.h)

    def set_input(self, tid, array):
        array = np.ascontiguousarray(array)
        check(lib().megcc_gfx950_model_set_input(self.h, tid, array.ctypes.data, array.nbytes), "set_input")

    def forward(self):
        check(lib().megcc_gfx950_model_forward(self.h), "forward")

    def join(self):
        """orders the library stream behind everything forward() has launched (the last operators of
        a forward may run on a second stream)"""
        check(lib().megcc_gfx950_model_join(self.h), "join")

    def run_opr(self, index):
        check(lib().megcc_gfx950_model_run_opr(self.h, index), "run_opr")

    def get(self, tid):
        shape, type_enum = self.shapes[tid]
        out = np.empty(shape, abi.np_dtype(type_enum))
        check(lib().megcc_gfx950_model_get_output(self.h, tid, out.ctypes.data, out.nbytes), "get_output")
        return out

    def get_async(self, tid, out):
        """enqueues the copy of tensor `tid` into the array `out` behind the forward that produced it;
        the bytes are there after wait()"""
        shape, type_enum = self.shapes[tid]
        assert out.shape == tuple(shape) and out.dtype == abi.np_dtype(type_enum) and out.flags["C_CONTIGUOUS"]
        check(lib().megcc_gfx950_model_get_output_async(self.h, tid, out.ctypes.data, out.nbytes), "get_output_async")

    def close(self):
        if self.h:
            lib().megcc_gfx950_model_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
