"""ctypes mirror of include/megcc_gfx950.h.

The struct layouts are the TinyNN runtime's (runtime/src/data_struct.h:12-59, device.h:8-21,
tinynn.h:7-54), so the same Python objects can be handed to libmegcc_gfx950.so (device pointers)
and, in the tests, to the reference's generated C kernels (host pointers).
"""
import ctypes as C

import numpy as np

MAX_DIM = 7

# TinyNNStatus
SUCCESS = 0
ERROR_NULL_PTR = 1
ERROR_OUT_OF_RANGE = 4
ERROR_NO_FOUND = 5
ERROR_NO_IMPLEMENT = 6
ERROR_UNSUPPORTED_DTYPE_TYPE = 11
ERROR_INVALID_LAYOUT = 12

# TinyNNDType
FLOAT, FLOAT16, INT, INT8, INT16, UINT8 = 0, 1, 2, 3, 4, 5
QINT8, QINT32, QUINT8 = 100, 101, 102

# MegccFormat / MegccSparse / MegccNonline
FMT_NCHW, FMT_NCHW44, FMT_NCHW_NCHW44 = 0, 1, 2
DENSE, GROUP = 0, 1
IDENTITY, RELU, H_SWISH, SIGMOID = 0, 1, 2, 3
NONLINE_NAMES = {IDENTITY: "IDENTITY", RELU: "RELU", H_SWISH: "H_SWISH", SIGMOID: "SIGMOID"}
# MegccPoolMode
POOL_MAX, POOL_AVERAGE, POOL_AVERAGE_COUNT_EXCLUDE_PADDING = 0, 1, 2
POOL_NAMES = {0: "MAX", 1: "AVERAGE", 2: "AVERAGE_COUNT_EXCLUDE_PADDING"}
# MegccMultiTypeMode
Q_ADD, Q_FUSE_ADD_RELU, Q_MUL, Q_RELU = 0, 1, 2, 3
MULTITYPE_NAMES = {0: "QADD", 1: "QFUSE_ADD_RELU", 2: "QMUL", 3: "QRELU"}
# MegccElemwiseMode
EW_RELU, EW_EXP, EW_SIGMOID, EW_H_SWISH, EW_NEGATE = 0, 1, 2, 3, 4
EW_ADD, EW_SUB, EW_MUL, EW_TRUE_DIV, EW_MAX, EW_MIN, EW_FUSE_ADD_RELU = 16, 17, 18, 19, 20, 21, 22
EW_MODES = {"RELU": 0, "EXP": 1, "SIGMOID": 2, "H_SWISH": 3, "NEGATE": 4, "ADD": 16, "SUB": 17,
            "MUL": 18, "TRUE_DIV": 19, "MAX": 20, "MIN": 21, "FUSE_ADD_RELU": 22}
# MegccReduceMode
REDUCE_SUM, REDUCE_MEAN, REDUCE_MAX, REDUCE_MIN, REDUCE_PRODUCT, REDUCE_SUM_SQR = 0, 1, 2, 3, 4, 5
REDUCE_MODES = {"SUM": 0, "MEAN": 1, "MAX": 2, "MIN": 3, "PRODUCT": 4, "SUM_SQR": 5}
# MegccKernelKind
KERN_CONV, KERN_MATMUL, KERN_POOLING, KERN_ELEMWISE_MULTITYPE = 1, 2, 3, 4
KERN_ELEMWISE, KERN_TYPECVT, KERN_REDUCE = 5, 6, 7
KERN_RELAYOUT, KERN_CONCAT, KERN_RESIZE, KERN_FUSED_ELEMWISE, KERN_SOFTMAX = 8, 9, 10, 11, 12
KERN_DW_POOL_ADD = 13
KERN_PW_DW = 14
IMODE_NEAREST, IMODE_LINEAR = 0, 1


class Device(C.Structure):
    _fields_ = [
        ("alignment", C.c_int),
        ("device_type", C.c_int),
        ("malloc", C.CFUNCTYPE(C.c_void_p, C.c_size_t)),
        ("free", C.CFUNCTYPE(None, C.c_void_p)),
    ]


class RuntimeOpt(C.Structure):
    _fields_ = [("device", C.POINTER(Device))]


class DTypeParam(C.Structure):
    _fields_ = [("scale", C.c_float), ("zero_point", C.c_uint8)]


class DType(C.Structure):
    _fields_ = [("type_enum", C.c_int), ("param", DTypeParam)]


class Layout(C.Structure):
    _fields_ = [
        ("nr_dim", C.c_int),
        ("dims", C.c_uint32 * MAX_DIM),
        ("stride", C.c_int * MAX_DIM),
        ("format", C.c_int),
    ]


class Tensor(C.Structure):
    _fields_ = [
        ("name", C.c_char_p),
        ("dtype", DType),
        ("layout", Layout),
        ("ptr", C.c_void_p),
        ("offset", C.c_size_t),
        ("use_count", C.c_int),
        ("is_weight", C.c_int),
        ("is_dynamic", C.c_int),
        ("checksum", C.c_uint32),
        ("size", C.c_size_t),
        ("is_shared", C.c_int),
        ("is_input", C.c_int),
    ]


class Workspace(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("size", C.c_size_t), ("offset", C.c_size_t)]


class ConvAttr(C.Structure):
    _fields_ = [
        ("kernel_h", C.c_uint32), ("kernel_w", C.c_uint32),
        ("stride_h", C.c_uint32), ("stride_w", C.c_uint32),
        ("pad_h", C.c_uint32), ("pad_w", C.c_uint32),
        ("dilate_h", C.c_uint32), ("dilate_w", C.c_uint32),
        ("format", C.c_int), ("sparse", C.c_int), ("nonline", C.c_int),
        ("with_bias", C.c_int),
    ]


class PoolAttr(C.Structure):
    _fields_ = [
        ("window_h", C.c_uint32), ("window_w", C.c_uint32),
        ("stride_h", C.c_uint32), ("stride_w", C.c_uint32),
        ("pad_h", C.c_uint32), ("pad_w", C.c_uint32),
        ("format", C.c_int), ("mode", C.c_int),
    ]


class MatMulAttr(C.Structure):
    _fields_ = [("transpose_a", C.c_int), ("transpose_b", C.c_int)]


class ReduceAttr(C.Structure):
    _fields_ = [("mode", C.c_int), ("axis", C.c_int)]


class ResizeAttr(C.Structure):
    _fields_ = [("format", C.c_int), ("imode", C.c_int)]


FUSED_MAX_STEPS, FUSED_MAX_INPUTS = 16, 8
# modes that exist only as steps of a fused elementwise chain (MegccElemwiseMode)
FUSED_ONLY_MODES = {"ABS": 5, "LOG": 6, "SILU": 7, "ROUND": 8, "LT": 23, "LEQ": 24, "EQ": 25,
                    "FLOOR_DIV": 26, "FUSE_ADD_SIGMOID": 27, "FUSE_ADD_TANH": 28,
                    "FUSE_MUL_ADD3": 32, "FUSE_MUL_ADD4": 33}


class FusedStep(C.Structure):
    _fields_ = [("mode", C.c_int), ("nr_arg", C.c_int), ("arg", C.c_int * 4)]


class FusedElemwiseAttr(C.Structure):
    _fields_ = [("nr_input", C.c_int), ("nr_step", C.c_int), ("step", FusedStep * FUSED_MAX_STEPS)]


def parse_fused_modes(modes, nr_input):
    """["I0,I1,ADD,O0", "O0,I2,MUL,D", ...] -> [(mode enum, [value numbers])]: the naming of
    compiler/test/kernel/opr/common/fused_elemwise.cpp:67-95 (I<k> input k, O<j> result of step j,
    the last step's result is the output whatever it is called)."""
    prog = []
    for j, text in enumerate(modes):
        parts = text.split(",")
        names, mode = parts[:-2], parts[-2]
        args = []
        for nm in names:
            k = int(nm[1:])
            assert (nm[0] == "I" and k < nr_input) or (nm[0] == "O" and k < j), text
            args.append(k if nm[0] == "I" else nr_input + k)
        enum = EW_MODES[mode] if mode in EW_MODES else FUSED_ONLY_MODES[mode]
        prog.append((enum, args))
    return prog


def fused_attr(prog, nr_input):
    a = FusedElemwiseAttr()
    a.nr_input, a.nr_step = nr_input, len(prog)
    for j, (mode, args) in enumerate(prog):
        a.step[j].mode, a.step[j].nr_arg = mode, len(args)
        for i, v in enumerate(args):
            a.step[j].arg[i] = v
    return a


class DwPoolAddAttr(C.Structure):
    _fields_ = [("conv", ConvAttr), ("pool", PoolAttr), ("mode", C.c_int), ("mid_scale", C.c_float)]


class PwDwAttr(C.Structure):
    _fields_ = [("pw", ConvAttr), ("dw", ConvAttr), ("mid_scale", C.c_float)]


class _KernelAttrUnion(C.Union):
    _fields_ = [
        ("conv", ConvAttr), ("matmul", MatMulAttr), ("pool", PoolAttr),
        ("multitype", C.c_int), ("elemwise", C.c_int), ("reduce", ReduceAttr),
        ("concat_axis", C.c_int), ("resize", ResizeAttr), ("fused", FusedElemwiseAttr),
        ("dw_pool_add", DwPoolAddAttr), ("pw_dw", PwDwAttr),
    ]


class KernelDesc(C.Structure):
    _fields_ = [("kind", C.c_int), ("attr", _KernelAttrUnion)]


_NP_OF = {
    FLOAT: np.float32, INT: np.int32, INT8: np.int8, INT16: np.int16, UINT8: np.uint8,
    QINT8: np.int8, QINT32: np.int32, QUINT8: np.uint8,
}


def np_dtype(type_enum):
    return np.dtype(_NP_OF[type_enum])


def contiguous_strides(shape):
    strides, s = [], 1
    for d in reversed(shape):
        strides.append(s)
        s *= int(d)
    return list(reversed(strides))


def make_tensor(ptr, shape, type_enum, scale=1.0, name=b"t", strides=None):
    """A Tensor whose ptr is `ptr` (host or device address, an int)."""
    t = Tensor()
    t.name = name
    t.dtype.type_enum = type_enum
    t.dtype.param.scale = scale
    t.dtype.param.zero_point = 0
    t.layout.nr_dim = len(shape)
    st = strides if strides is not None else contiguous_strides(shape)
    for i, d in enumerate(shape):
        t.layout.dims[i] = int(d)
        t.layout.stride[i] = int(st[i])
    t.layout.format = 0
    t.ptr = ptr
    n = 1
    for d in shape:
        n *= int(d)
    t.size = n * np_dtype(type_enum).itemsize
    return t


def host_tensor(arr, type_enum, scale=1.0, name=b"t", shape=None, strides=None, offset=0):
    """Tensor over a C-contiguous numpy array (kept alive by the caller). With `shape`, a view
    into it: `strides` and `offset` (where the view's first element lies) count elements."""
    assert arr.flags["C_CONTIGUOUS"]
    return make_tensor(arr.ctypes.data + offset * arr.itemsize,
                       arr.shape if shape is None else shape, type_enum, scale, name, strides)


def tensor_array(tensors):
    arr = (C.POINTER(Tensor) * len(tensors))()
    for i, t in enumerate(tensors):
        arr[i] = C.pointer(t)
    return arr


KERNEL_ARGS = [
    C.POINTER(C.POINTER(Tensor)), C.c_int, C.POINTER(C.POINTER(Tensor)), C.c_int,
    C.POINTER(Workspace), C.POINTER(RuntimeOpt),
]
INIT_ARGS = [
    C.POINTER(C.POINTER(Tensor)), C.c_int, C.POINTER(Tensor), C.POINTER(C.c_int),
    C.POINTER(RuntimeOpt),
]
WORKSPACE_ARGS = [C.POINTER(C.POINTER(Tensor)), C.c_int, C.c_int, C.POINTER(C.c_size_t)]
