"""TEST INFRASTRUCTURE ONLY: numpy front-end of oracle/liboracle_port.so (oracle_port.c).

Importable from tests/, bench.py's cpu_baseline leg and __graft_entry__.smoke() only.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

FMT_NCHW, FMT_NCHW44, FMT_NCHW_NCHW44 = 0, 1, 2


def build():
    subprocess.check_call(["make", "-s", "-C", _HERE, "port"])


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "liboracle_port.so")
        if not os.path.exists(path):
            build()
        _LIB = C.CDLL(path)
    return _LIB


def set_threads(n):
    lib().orc_set_threads(int(n))


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def conv_out_hw(ih, iw, fh, fw, sh, sw, ph, pw, dh=1, dw=1):
    oh = (ih + 2 * ph - (dh * (fh - 1) + 1)) // sh + 1
    ow = (iw + 2 * pw - (dw * (fw - 1) + 1)) // sw + 1
    return oh, ow


def _conv_dims(src, flt_fmt, groups, oc):
    if src.ndim == 5:
        n, c4, ih, iw, _ = src.shape
        return n, c4 * 4, ih, iw
    n, c, ih, iw = src.shape
    return n, c, ih, iw


def conv(src, flt, bias, fmt, groups, oc, fh, fw, stride, pad, dilate, act, scales=None):
    """src/flt/bias as laid out by the reference (NCHW or NCHW44 arrays); returns dst in the
    reference's layout. scales = (src, flt, dst) for qsi8, None for f32."""
    n, ic, ih, iw = _conv_dims(src, fmt, groups, oc)
    sh, sw = stride
    ph, pw = pad
    dh, dw = dilate
    oh, ow = conv_out_hw(ih, iw, fh, fw, sh, sw, ph, pw, dh, dw)
    dst_shape = (n, oc, oh, ow) if fmt == FMT_NCHW else (n, oc // 4, oh, ow, 4)
    L = lib()
    if scales is not None:
        dst = np.empty(dst_shape, np.int8)
        L.orc_conv_q8(
            _p(src), _p(flt), _p(bias), _p(dst), fmt, groups, n, ic, ih, iw, oc, oh, ow, fh, fw,
            sh, sw, ph, pw, dh, dw, act, C.c_float(scales[0]), C.c_float(scales[1]),
            C.c_float(scales[2]))
    else:
        dst = np.empty(dst_shape, np.float32)
        L.orc_conv_f32(
            _p(src), _p(flt), _p(bias), _p(dst), fmt, groups, n, ic, ih, iw, oc, oh, ow, fh, fw,
            sh, sw, ph, pw, dh, dw, act)
    return dst


def matmul_f32(a, b, trans_a=False, trans_b=False):
    m = a.shape[1] if trans_a else a.shape[0]
    k = a.shape[0] if trans_a else a.shape[1]
    n = b.shape[0] if trans_b else b.shape[1]
    c = np.empty((m, n), np.float32)
    lib().orc_matmul_f32(_p(a), _p(b), _p(c), m, n, k, a.shape[1], b.shape[1], n,
                         int(trans_a), int(trans_b))
    return c


def pool_q8(src, fmt, mode, window, stride, pad):
    if fmt == FMT_NCHW44:
        n, c4, ih, iw, _ = src.shape
        c = c4 * 4
    else:
        n, c, ih, iw = src.shape
    oh = (ih + 2 * pad[0] - window[0]) // stride[0] + 1
    ow = (iw + 2 * pad[1] - window[1]) // stride[1] + 1
    dst = np.empty((n, c // 4, oh, ow, 4) if fmt == FMT_NCHW44 else (n, c, oh, ow), np.int8)
    lib().orc_pool_q8(_p(src), _p(dst), fmt, mode, n, c, ih, iw, oh, ow, window[0], window[1],
                      stride[0], stride[1], pad[0], pad[1])
    return dst


def _bcast(a, b):
    if b is None or a.shape == b.shape:
        return 0, 1, 1
    if b.size == 1:
        return 1, 1, 1
    if b.ndim == a.ndim and b.size == b.shape[1] == a.shape[1]:
        inner = 1
        for d in a.shape[2:]:
            inner *= d
        return 2, a.shape[1], inner
    if b.ndim == 1 and b.shape[0] == a.shape[-1]:
        return 2, a.shape[-1], 1
    if a.ndim == 2 and b.ndim == 2 and b.shape == (a.shape[0], 1):
        return 2, a.shape[0], a.shape[1]
    raise ValueError("unsupported broadcast %s vs %s" % (a.shape, b.shape))


def multitype_q8(a, b, mode, s0, s1, sd):
    dst = np.empty(a.shape, np.int8)
    bc, c, inner = _bcast(a, b)
    lib().orc_multitype_q8(_p(a), _p(b), _p(dst), mode, C.c_size_t(a.size), bc, c,
                           C.c_size_t(inner), C.c_float(s0), C.c_float(s1), C.c_float(sd))
    return dst


def elemwise_f32(a, b, mode):
    """f32 Elemwise over the broadcast of a and b (right-aligned shapes, extent 1 stretches:
    numpy's own rule materialises the operands, the per-element expressions are the C port's)."""
    if b is None:
        shape = a.shape
    else:
        shape = np.broadcast_shapes(a.shape, b.shape)
        a = np.ascontiguousarray(np.broadcast_to(a, shape))
        b = np.ascontiguousarray(np.broadcast_to(b, shape))
    dst = np.empty(shape, np.float32)
    lib().orc_elemwise_f32(_p(a), _p(b), _p(dst), mode, C.c_size_t(dst.size), 0, 1, C.c_size_t(1))
    return dst


def typecvt(src, src_kind, dst_kind, src_scale=1.0, dst_scale=1.0):
    L = lib()
    n = C.c_size_t(src.size)
    if (src_kind, dst_kind) == ("f32", "qsi8"):
        dst = np.empty(src.shape, np.int8)
        L.orc_typecvt_f32_q8(_p(src), _p(dst), n, C.c_float(dst_scale))
    elif (src_kind, dst_kind) == ("qsi8", "f32"):
        dst = np.empty(src.shape, np.float32)
        L.orc_typecvt_q8_f32(_p(src), _p(dst), n, C.c_float(src_scale))
    elif (src_kind, dst_kind) == ("qsi8", "qsi8"):
        dst = np.empty(src.shape, np.int8)
        L.orc_typecvt_q8_q8(_p(src), _p(dst), n, C.c_float(src_scale), C.c_float(dst_scale))
    elif (src_kind, dst_kind) == ("qsi32", "qsi8"):
        dst = np.empty(src.shape, np.int8)
        L.orc_typecvt_q32_q8(_p(src), _p(dst), n, C.c_float(src_scale), C.c_float(dst_scale))
    else:
        raise ValueError((src_kind, dst_kind))
    return dst


def reduce_f32(src, mode, axis):
    a = int(np.prod(src.shape[:axis], dtype=np.int64))
    b = src.shape[axis]
    c = int(np.prod(src.shape[axis + 1:], dtype=np.int64))
    shape = list(src.shape)
    shape[axis] = 1
    dst = np.empty(shape, np.float32)
    lib().orc_reduce_f32(_p(src), _p(dst), mode, a, b, c)
    return dst


def relayout(src, src_off, src_shape, src_strides, dst, dst_off, dst_shape, dst_strides):
    """dst view <- src view; `src`/`dst` are flat-able dense arrays, offsets/strides count
    elements. Writes into `dst` in place."""
    assert src.dtype == dst.dtype and src.flags["C_CONTIGUOUS"] and dst.flags["C_CONTIGUOUS"]
    i64 = lambda v: np.ascontiguousarray(v, dtype=np.int64)
    sd, ss, dd, ds = i64(src_shape), i64(src_strides), i64(dst_shape), i64(dst_strides)
    es = src.itemsize
    lib().orc_relayout(
        C.c_void_p(src.ctypes.data + src_off * es), len(sd), _p(sd), _p(ss),
        C.c_void_p(dst.ctypes.data + dst_off * es), len(dd), _p(dd), _p(ds), es)


def concat(arrays, axis):
    shape = list(arrays[0].shape)
    shape[axis] = sum(a.shape[axis] for a in arrays)
    dst = np.empty(shape, arrays[0].dtype)
    outer = int(np.prod(shape[:axis], dtype=np.int64))
    inner = int(np.prod(shape[axis + 1:], dtype=np.int64))
    arrays = [np.ascontiguousarray(a) for a in arrays]
    ptrs = (C.c_void_p * len(arrays))(*[a.ctypes.data for a in arrays])
    lens = np.array([a.shape[axis] for a in arrays], np.int64)
    lib().orc_concat(ptrs, _p(lens), len(arrays), _p(dst), C.c_int64(outer), C.c_int64(inner),
                     dst.itemsize)
    return dst


def resize(src, out_hw, imode, nchw44=False, src_strides=None, src_shape=None):
    """f32 Resize. `src` dense [N,C,H,W] / [N,C/4,H,W,4]; for NEAREST the source may be a
    strided NCHW view of a dense buffer (`src_shape`, `src_strides` in elements)."""
    oh, ow = out_hw
    shape = tuple(src_shape) if src_shape is not None else src.shape
    n, c, ih, iw = shape[:4]
    src = np.ascontiguousarray(src, dtype=np.float32)
    if imode == "LINEAR":
        assert src_strides is None
        dst = np.empty((n, c, oh, ow, 4) if nchw44 else (n, c, oh, ow), np.float32)
        lib().orc_resize_linear_f32(_p(src), _p(dst), n, c * 4 if nchw44 else c, ih, iw, oh, ow,
                                    1 if nchw44 else 0)
        return dst
    assert imode == "NEAREST" and not nchw44
    st = src_strides if src_strides is not None else (c * ih * iw, ih * iw, iw, 1)
    dst = np.empty((n, c, oh, ow), np.float32)
    lib().orc_resize_nearest_f32(_p(src), _p(dst), n, c, ih, iw, oh, ow,
                                 *[C.c_int64(int(v)) for v in st])
    return dst


def fused_elemwise(prog, arrays, types, out_shape):
    """prog: list of (mode, [value numbers]); arrays: the f32 inputs; types: 0 VECTOR, 1 SCALAR,
    2 [1,C,1,1], 3 [1,C,1,1,4] per input."""
    flat = np.zeros((len(prog), 6), np.int32)
    for j, (mode, args) in enumerate(prog):
        flat[j, 0], flat[j, 1] = mode, len(args)
        flat[j, 2:2 + len(args)] = args
    arrays = [np.ascontiguousarray(a, dtype=np.float32) for a in arrays]
    ptrs = (C.c_void_p * len(arrays))(*[a.ctypes.data for a in arrays])
    ty = np.asarray(types, np.int32)
    dst = np.empty(out_shape, np.float32)
    n = int(np.prod(out_shape, dtype=np.int64))
    dims1 = out_shape[1] if len(out_shape) >= 2 else 1
    stride1 = int(np.prod(out_shape[2:], dtype=np.int64)) if len(out_shape) >= 2 else 1
    lib().orc_fused_elemwise_f32(_p(flat), len(arrays), len(prog), ptrs, _p(ty), _p(dst),
                                 C.c_size_t(n), C.c_size_t(stride1), C.c_size_t(dims1))
    return dst
