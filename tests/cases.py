"""Operator test cases shared by the CPU (oracle) and GPU (parity) tests.

A case knows (1) the reference kernel symbol MegCC would generate for it, (2) how to draw seeded
inputs in the reference's layouts, (3) how to evaluate it on the CPU port (oracle/port.py) and on
the reference's generated C (oracle/ref.py), and (4) the Tensor list the uniform kernel ABI takes.
The GPU side (tests/gpu_util.py) consumes the same description.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from megcc_amd import abi  # noqa: E402
from oracle import port, ref  # noqa: E402

FMT_NAME = {abi.FMT_NCHW: "NCHW", abi.FMT_NCHW44: "NCHW44", abi.FMT_NCHW_NCHW44: "NCHW_NCHW44"}


def rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


def _op(shape, dtype, scale=None):
    """operand text of oracle/ref_kernels.spec: dims|dtype|scale"""
    return "o:%s|%s|%s" % ("x".join(str(int(d)) for d in shape), dtype,
                           "" if scale is None else repr(float(scale)))


class TensorSpec:
    """name, numpy array (inputs) or shape (outputs), TinyNN dtype enum, scale.
    A strided view is given by `strides` and `offset` (elements; offset = where the view's first
    element lies) into a dense buffer: `array` itself for an input, a buffer of shape `storage`
    for an output (the whole buffer comes back as the result)."""

    def __init__(self, name, shape, type_enum, scale=1.0, array=None, strides=None, offset=0,
                 storage=None):
        self.name, self.shape, self.type_enum, self.scale, self.array = (
            name, tuple(shape), type_enum, scale, array)
        self.strides, self.offset = strides, offset
        self.storage = tuple(storage) if storage is not None else self.shape

    @property
    def nbytes(self):
        return int(np.prod(self.storage, dtype=np.int64)) * abi.np_dtype(self.type_enum).itemsize


class ConvCase:
    def __init__(self, fmt, sparse, n, ic, ih, iw, oc, k, stride=1, pad=0, act=abi.IDENTITY,
                 dtype="qsi8", scales=(0.02, 0.01, 0.05), bias=True, dilate=1,
                 src_range=(-128, 127), flt_range=(-127, 127), bias_range=(-1000, 1000)):
        self.fmt, self.sparse = fmt, sparse
        self.n, self.ic, self.ih, self.iw, self.oc = n, ic, ih, iw, oc
        self.fh = self.fw = k
        self.sh = self.sw = stride
        self.ph = self.pw = pad
        self.dh = self.dw = dilate
        self.act, self.dtype, self.scales, self.bias = act, dtype, scales, bias
        self.src_range, self.flt_range, self.bias_range = src_range, flt_range, bias_range
        self.groups = ic if sparse == abi.GROUP else 1
        if sparse == abi.GROUP:
            assert ic == oc, "only channel-wise GROUP cases are described here"
        self.oh, self.ow = port.conv_out_hw(ih, iw, k, k, stride, stride, pad, pad, dilate, dilate)

    def __repr__(self):
        return "%s[n%d c%d->%d %dx%d %s]" % (self.symbol(), self.n, self.ic, self.oc, self.ih,
                                             self.iw, "x".join("%g" % s for s in self.scales))

    # -- shapes in the reference's layouts (BareMetal/ConvKernel.cpp:48-113) -------------------
    def src_shape(self):
        if self.fmt == abi.FMT_NCHW44:
            return (self.n, self.ic // 4, self.ih, self.iw, 4)
        return (self.n, self.ic, self.ih, self.iw)

    def dst_shape(self):
        if self.fmt == abi.FMT_NCHW:
            return (self.n, self.oc, self.oh, self.ow)
        return (self.n, self.oc // 4, self.oh, self.ow, 4)

    def flt_shape(self):
        k = self.fh
        if self.fmt == abi.FMT_NCHW:
            if self.sparse == abi.GROUP:
                return (self.groups, 1, 1, k, k)
            return (self.oc, self.ic, k, k)
        if self.fmt == abi.FMT_NCHW_NCHW44:
            return (self.oc // 4, k, k, self.ic, 4)
        if self.sparse == abi.GROUP:
            return (self.groups // 4, 1, 1, k, k, 4)
        return (self.oc // 4, self.ic // 4, k, k, 4, 4)

    def bias_shape(self):
        if self.fmt == abi.FMT_NCHW:
            return (1, self.oc, 1, 1)
        return (1, self.oc // 4, 1, 1, 4)

    def symbol(self):
        """ConvImpl::GetKernelSymbol, BareMetal/ConvKernel.cpp:144-176 (GI_ prefix and suffix
        order of GeneralIntrinsic/ConvKernel/Fp32Im2col.cpp for the f32 NCHW dense case)."""
        q = self.dtype == "qsi8"
        io = "qsi8qsi8qsi32qsi8" if q else "f32f32f32f32"
        if not self.bias:
            io = "qsi8qsi8qsi8" if q else "f32f32f32"
        s = "kernel_conv2d_%dx%d_%s_%s_p%dx%d_s%dx%d_d%dx%d_%s" % (
            self.fh, self.fw, FMT_NAME[self.fmt], "GROUP" if self.sparse == abi.GROUP else "DENSE",
            self.ph, self.pw, self.sh, self.sw, self.dh, self.dw, io)
        if self.bias:
            s += "_bias"
        if self.act != abi.IDENTITY:
            s += "_" + abi.NONLINE_NAMES[self.act]
        return s

    def spec_line(self):
        """the attribute bag the reference compiler hands to KernelGen for this operator
        (compiler/test/kernel/common/src/cc_fill_attr.cpp:253-274), in ref_dump's text form"""
        q = self.dtype == "qsi8"
        sd, bd = ("qsi8", "qsi32") if q else ("f32", "f32")
        ss, fs, ds = self.scales if q else (None, None, None)
        src_shape = self.src_shape()
        a = ["ConvKernel", "format=s:" + ("NCHW" if self.fmt == abi.FMT_NCHW else "NCHW44"),
             "sparse=s:" + ("GROUP" if self.sparse == abi.GROUP else "DENSE"),
             "mode=s:CROSS_CORRELATION", "nonlineMode=s:" + abi.NONLINE_NAMES[self.act],
             "kernel_h=u:%d" % self.fh, "kernel_w=u:%d" % self.fw, "stride_h=u:%d" % self.sh,
             "stride_w=u:%d" % self.sw, "pad_h=u:%d" % self.ph, "pad_w=u:%d" % self.pw,
             "dilate_h=u:%d" % self.dh, "dilate_w=u:%d" % self.dw,
             "nr_operands=i:%d" % (4 if self.bias else 3),
             "operand:0=" + _op(src_shape, sd, ss), "operand:1=" + _op(self.flt_shape(), sd, fs)]
        if self.bias:
            a.append("operand:2=" + _op(self.bias_shape(), bd, ss * fs if q else None))
        a.append("operand:%d=%s" % (3 if self.bias else 2, _op(self.dst_shape(), sd, ds)))
        return " ".join(a)

    def attr(self):
        return abi.ConvAttr(self.fh, self.fw, self.sh, self.sw, self.ph, self.pw, self.dh, self.dw,
                            self.fmt, self.sparse, self.act, int(self.bias))

    def gen(self, seed=0):
        r = rng(seed)
        if self.dtype == "qsi8":
            src = r.integers(self.src_range[0], self.src_range[1] + 1, self.src_shape()).astype(np.int8)
            flt = r.integers(self.flt_range[0], self.flt_range[1] + 1, self.flt_shape()).astype(np.int8)
            b = r.integers(self.bias_range[0], self.bias_range[1] + 1, self.bias_shape()).astype(np.int32)
        else:
            src = r.uniform(-1, 1, self.src_shape()).astype(np.float32)
            flt = r.uniform(-1, 1, self.flt_shape()).astype(np.float32)
            b = r.uniform(-0.1, 0.1, self.bias_shape()).astype(np.float32)
        return {"src": src, "flt": flt, "bias": b if self.bias else None}

    def specs(self, arrays):
        q = self.dtype == "qsi8"
        ss, fs, ds = self.scales if q else (1.0, 1.0, 1.0)
        ins = [TensorSpec(b"src", self.src_shape(), abi.QINT8 if q else abi.FLOAT, ss, arrays["src"]),
               TensorSpec(b"flt", self.flt_shape(), abi.QINT8 if q else abi.FLOAT, fs, arrays["flt"])]
        if self.bias:
            ins.append(TensorSpec(b"bias", self.bias_shape(), abi.QINT32 if q else abi.FLOAT,
                                  float(np.float32(ss) * np.float32(fs)), arrays["bias"]))
        outs = [TensorSpec(b"dst", self.dst_shape(), abi.QINT8 if q else abi.FLOAT, ds)]
        return ins, outs

    def run_port(self, arrays):
        return port.conv(arrays["src"], arrays["flt"], arrays["bias"], self.fmt, self.groups,
                         self.oc, self.fh, self.fw, (self.sh, self.sw), (self.ph, self.pw),
                         (self.dh, self.dw), self.act,
                         self.scales if self.dtype == "qsi8" else None)

    def ops(self):
        return 2 * self.n * self.oc * self.oh * self.ow * (self.ic // self.groups) * self.fh * self.fw

    def min_bytes(self):
        e = 1 if self.dtype == "qsi8" else 4
        return (int(np.prod(self.src_shape())) * e + int(np.prod(self.flt_shape())) * e +
                self.oc * 4 + int(np.prod(self.dst_shape())) * e)


class PoolCase:
    def __init__(self, fmt, mode, n, c, ih, iw, window, stride, pad, scale=0.05):
        self.fmt, self.mode, self.n, self.c, self.ih, self.iw = fmt, mode, n, c, ih, iw
        self.window, self.stride, self.pad, self.scale = window, stride, pad, scale
        self.oh = (ih + 2 * pad - window) // stride + 1
        self.ow = (iw + 2 * pad - window) // stride + 1

    def __repr__(self):
        return "%s[n%d c%d %dx%d]" % (self.symbol(), self.n, self.c, self.ih, self.iw)

    def src_shape(self):
        return ((self.n, self.c // 4, self.ih, self.iw, 4) if self.fmt == abi.FMT_NCHW44
                else (self.n, self.c, self.ih, self.iw))

    def dst_shape(self):
        return ((self.n, self.c // 4, self.oh, self.ow, 4) if self.fmt == abi.FMT_NCHW44
                else (self.n, self.c, self.oh, self.ow))

    def symbol(self):
        """PoolingImpl::GetKernelSymbol (BareMetal/Pooling.cpp:31-44); the NCHW44 kernel comes
        from GI with its extra io-string and _fallback suffix
        (GeneralIntrinsic/PoolingKernel/QInt8PoolingNCHW44.cpp:25-31)."""
        s = "kernel_pooling_%s_%s_p%dx%d_s%dx%d_w%dx%d_qsi8qsi8" % (
            abi.POOL_NAMES[self.mode], FMT_NAME[self.fmt], self.pad, self.pad, self.stride,
            self.stride, self.window, self.window)
        if self.fmt == abi.FMT_NCHW44:
            s = "GI_" + s + "_qsi8qsi8_fallback"
        return s

    def spec_line(self):
        return " ".join([
            "PoolingKernel", "format=s:" + FMT_NAME[self.fmt], "mode=s:" + abi.POOL_NAMES[self.mode],
            "window_h=u:%d" % self.window, "window_w=u:%d" % self.window,
            "stride_h=u:%d" % self.stride, "stride_w=u:%d" % self.stride,
            "pad_h=u:%d" % self.pad, "pad_w=u:%d" % self.pad, "nr_operands=i:2",
            "operand:0=" + _op(self.src_shape(), "qsi8", self.scale),
            "operand:1=" + _op(self.dst_shape(), "qsi8", self.scale)])

    def attr(self):
        return abi.PoolAttr(self.window, self.window, self.stride, self.stride, self.pad, self.pad,
                            self.fmt, self.mode)

    def gen(self, seed=0):
        return {"src": rng(seed).integers(-128, 128, self.src_shape()).astype(np.int8)}

    def specs(self, arrays):
        return ([TensorSpec(b"src", self.src_shape(), abi.QINT8, self.scale, arrays["src"])],
                [TensorSpec(b"dst", self.dst_shape(), abi.QINT8, self.scale)])

    def run_port(self, arrays):
        return port.pool_q8(arrays["src"], self.fmt, self.mode, (self.window,) * 2,
                            (self.stride,) * 2, (self.pad,) * 2)


class MultiTypeCase:
    def __init__(self, mode, shape, scales=(0.05, 0.01, 0.05), bshape=None):
        self.mode, self.shape, self.scales = mode, tuple(shape), scales
        self.bshape = tuple(bshape) if bshape is not None else self.shape

    def __repr__(self):
        return "%s%s%s" % (self.symbol(), list(self.shape), list(self.bshape))

    def symbol(self):
        """BareMetal/ElemwiseMultiType.cpp:94-100"""
        io = "qsi8qsi8" if self.mode == abi.Q_RELU else "qsi8qsi8qsi8"
        return "kernel_elementwise_multitype_%s_%s" % (abi.MULTITYPE_NAMES[self.mode], io)

    def spec_line(self):
        ops = [_op(self.shape, "qsi8", self.scales[0])]
        if self.mode != abi.Q_RELU:
            ops.append(_op(self.bshape, "qsi8", self.scales[1]))
        ops.append(_op(self.shape, "qsi8", self.scales[2]))
        return " ".join(["ElemwiseMultiKernel", "mode=s:" + abi.MULTITYPE_NAMES[self.mode],
                         "nr_operands=i:%d" % len(ops)] +
                        ["operand:%d=%s" % (i, o) for i, o in enumerate(ops)])

    def gen(self, seed=0):
        r = rng(seed)
        a = r.integers(-128, 128, self.shape).astype(np.int8)
        b = None if self.mode == abi.Q_RELU else r.integers(-128, 128, self.bshape).astype(np.int8)
        return {"a": a, "b": b}

    def specs(self, arrays):
        ins = [TensorSpec(b"a", self.shape, abi.QINT8, self.scales[0], arrays["a"])]
        if self.mode != abi.Q_RELU:
            ins.append(TensorSpec(b"b", self.bshape, abi.QINT8, self.scales[1], arrays["b"]))
        return ins, [TensorSpec(b"dst", self.shape, abi.QINT8, self.scales[2])]

    def run_port(self, arrays):
        return port.multitype_q8(arrays["a"], arrays["b"], self.mode, *self.scales)


_KIND_ENUM = {"f32": abi.FLOAT, "qsi8": abi.QINT8, "qsi32": abi.QINT32}


class TypeCvtCase:
    def __init__(self, src_kind, dst_kind, shape, src_scale=1.0, dst_scale=1.0, span=None):
        self.src_kind, self.dst_kind, self.shape = src_kind, dst_kind, tuple(shape)
        self.src_scale, self.dst_scale, self.span = src_scale, dst_scale, span

    def __repr__(self):
        return "%s%s" % (self.symbol(), list(self.shape))

    def symbol(self):
        """GI for q8<->f32 and q8->q8 (GeneralIntrinsic/Typecvt.cpp:36-41), BareMetal otherwise
        (BareMetal/Typecvt.cpp:36-41)."""
        gi = (self.src_kind, self.dst_kind) != ("qsi32", "qsi8")
        return ("GI_" if gi else "") + "kernel_typecvt_%s%s" % (self.src_kind, self.dst_kind)

    def spec_line(self):
        return " ".join([
            "TypeCvtKernel", "nr_operands=i:2",
            "operand:0=" + _op(self.shape, self.src_kind,
                               None if self.src_kind == "f32" else self.src_scale),
            "operand:1=" + _op(self.shape, self.dst_kind,
                               None if self.dst_kind == "f32" else self.dst_scale)])

    def gen(self, seed=0):
        r = rng(seed)
        if self.src_kind == "f32":
            span = self.span or 140 * self.dst_scale
            src = r.uniform(-span, span, self.shape).astype(np.float32)
            # exact .5 ties, which round half away from zero
            flat = src.reshape(-1)
            k = min(flat.size, 64)
            flat[:k] = (np.arange(k, dtype=np.float32) - k // 2 + 0.5) * np.float32(self.dst_scale)
        elif self.src_kind == "qsi8":
            src = r.integers(-128, 128, self.shape).astype(np.int8)
        else:
            span = int(self.span or 140 * self.dst_scale / self.src_scale)
            src = r.integers(-span, span + 1, self.shape).astype(np.int32)
        return {"src": src}

    def specs(self, arrays):
        return ([TensorSpec(b"src", self.shape, _KIND_ENUM[self.src_kind], self.src_scale,
                            arrays["src"])],
                [TensorSpec(b"dst", self.shape, _KIND_ENUM[self.dst_kind], self.dst_scale)])

    def run_port(self, arrays):
        return port.typecvt(arrays["src"], self.src_kind, self.dst_kind, self.src_scale,
                            self.dst_scale)


class MatMulCase:
    def __init__(self, m, k, n, trans_a=False, trans_b=False):
        self.m, self.k, self.n, self.trans_a, self.trans_b = m, k, n, trans_a, trans_b

    def __repr__(self):
        return "%s[%dx%dx%d]" % (self.symbol(), self.m, self.k, self.n)

    def ops(self):
        return 2 * self.m * self.n * self.k

    def symbol(self):
        """GeneralIntrinsic/MatMulKernel/Fp32Gevm.cpp:109-135 (M<=4, A not transposed) else
        Fp32MatMulM4N12.cpp:9-45"""
        t = ("t" if self.trans_a else "n") + ("t" if self.trans_b else "n")
        if self.m <= 4 and not self.trans_a:
            return "GI_kernel_gevm_" + t
        return "GI_kernel_fp32_matmul_4x12_" + t

    def spec_line(self):
        ashape = (self.k, self.m) if self.trans_a else (self.m, self.k)
        bshape = (self.n, self.k) if self.trans_b else (self.k, self.n)
        return " ".join([
            "MatrixMulKernel", "transposeA=b:%d" % self.trans_a, "transposeB=b:%d" % self.trans_b,
            "format=s:DEFAULT", "compute_mode=s:DEFAULT", "nr_operands=i:3",
            "operand:0=" + _op(ashape, "f32"), "operand:1=" + _op(bshape, "f32"),
            "operand:2=" + _op((self.m, self.n), "f32")])

    def attr(self):
        return abi.MatMulAttr(int(self.trans_a), int(self.trans_b))

    def gen(self, seed=0):
        r = rng(seed)
        ashape = (self.k, self.m) if self.trans_a else (self.m, self.k)
        bshape = (self.n, self.k) if self.trans_b else (self.k, self.n)
        return {"a": r.uniform(-1, 1, ashape).astype(np.float32),
                "b": r.uniform(-1, 1, bshape).astype(np.float32)}

    def specs(self, arrays):
        return ([TensorSpec(b"a", arrays["a"].shape, abi.FLOAT, 1.0, arrays["a"]),
                 TensorSpec(b"b", arrays["b"].shape, abi.FLOAT, 1.0, arrays["b"])],
                [TensorSpec(b"c", (self.m, self.n), abi.FLOAT)])

    def run_port(self, arrays):
        return port.matmul_f32(arrays["a"], arrays["b"], self.trans_a, self.trans_b)


def _nelem(shape):
    return int(np.prod(shape, dtype=np.int64))


def binary_bcast_type(s0, s1):
    """GetBinaryBcastType, Common/ElemwiseCommon.cpp:47-127: the name the reference gives the way
    two operand shapes meet (part of the GI kernel's symbol)."""
    s0, s1 = tuple(s0), tuple(s1)
    n0, n1 = _nelem(s0), _nelem(s1)
    if n0 == n1:
        return "VEC_VEC"
    if n0 == 1:
        return "SCALAR_VEC"
    if n1 == 1:
        return "VEC_SCALAR"
    if (n0 == s0[-1] or n1 == s1[-1]) and s0[-1] == s1[-1]:
        return "BCAST111C_VEC" if n0 == s0[-1] else "VEC_BCAST111C"
    assert len(s0) == len(s1)
    small, big = (s0, s1) if n0 < n1 else (s1, s0)
    names = (lambda a, b: a + "_VEC" if n0 < n1 else "VEC_" + a)
    if all(sm == 1 for sm, bg in zip(small, big) if bg == 1):
        if len(small) == 4 and small[0] == small[2] == small[3] == 1:
            return names("BCAST101", None)
        if len(small) == 5 and small[0] == small[2] == small[3] == 1 and small[4] in (4, 8):
            return names("BCAST101xX", None)
        # CalBroadcastElemwise: runs of broadcast / elementwise dims
        runs, bc = [1], True
        for sm, bg in zip(small, big):
            if not bc and sm != bg:
                bc = True
                runs.append(1)
            elif bc and sm != 1:
                bc = False
                runs.append(1)
            runs[-1] *= bg
        if len(runs) == 2:
            return names("BV", None)
        if small[:-1] == big[:-1] and small[-1] == 1 and big[-1] > 1:
            return names("BCAST110", None)
    return "NAIVE"


class ElemwiseCase:
    """f32 Elemwise: unary (one shape) or binary over the broadcast of two shapes (right-aligned,
    extent 1 stretches: megdnn's rule, which is numpy's). `span` = range of the drawn values."""

    GI_MODES = {"RELU", "EXP", "SIGMOID", "H_SWISH", "ADD", "SUB", "MUL", "TRUE_DIV",
                "FUSE_ADD_RELU", "MAX", "MIN"}

    def __init__(self, mode, shapes, span=(-4.0, 4.0)):
        self.mode, self.shapes, self.span = mode, [tuple(s) for s in shapes], span
        assert len(self.shapes) == (2 if abi.EW_MODES[mode] >= abi.EW_ADD else 1)
        self.out_shape = tuple(np.broadcast_shapes(*self.shapes))

    def __repr__(self):
        return "elemwise_%s[%s]" % (self.mode, " ".join("x".join(map(str, s)) for s in self.shapes))

    def symbol(self):
        """GeneralIntrinsic/Elemwise/Elemwise.cpp:38-63 for the modes GI knows (:17-20), else
        BareMetal/ElemwiseKernel.cpp:433-439"""
        io = "f32" * (len(self.shapes) + 1)
        if self.mode not in self.GI_MODES:
            return "kernel_elementwise_%s_%s" % (self.mode, io)
        kind = "unary_vec_vec" if len(self.shapes) == 1 else \
            "binary_" + binary_bcast_type(*self.shapes)
        return "GI_kernel_elementwise_%s_f32_%s_%s" % (self.mode, kind, io)

    def spec_line(self):
        ops = [_op(s, "f32") for s in self.shapes] + [_op(self.out_shape, "f32")]
        return " ".join(["ElemwiseKernel", "mode=s:" + self.mode, "nr_operands=i:%d" % len(ops)] +
                        ["operand:%d=%s" % (i, o) for i, o in enumerate(ops)])

    def gen(self, seed=0):
        r = rng(seed)
        out = {"a": r.uniform(self.span[0], self.span[1], self.shapes[0]).astype(np.float32)}
        out["b"] = (r.uniform(self.span[0], self.span[1], self.shapes[1]).astype(np.float32)
                    if len(self.shapes) == 2 else None)
        return out

    def specs(self, arrays):
        ins = [TensorSpec(b"a", self.shapes[0], abi.FLOAT, 1.0, arrays["a"])]
        if len(self.shapes) == 2:
            ins.append(TensorSpec(b"b", self.shapes[1], abi.FLOAT, 1.0, arrays["b"]))
        return ins, [TensorSpec(b"dst", self.out_shape, abi.FLOAT, 1.0)]

    def run_port(self, arrays):
        return port.elemwise_f32(arrays["a"], arrays["b"], abi.EW_MODES[self.mode])

    def min_bytes(self):
        return 4 * (sum(_nelem(s) for s in self.shapes) + _nelem(self.out_shape))


class ReduceCase:
    """f32 Reduce over one axis (kept with extent 1 in the output, as megdnn deduces it)"""

    def __init__(self, mode, shape, axis):
        self.mode, self.shape, self.axis = mode, tuple(shape), axis
        self.out_shape = tuple(1 if i == axis else d for i, d in enumerate(self.shape))

    def __repr__(self):
        return "reduce_%s_a%d[%s]" % (self.mode, self.axis, "x".join(map(str, self.shape)))

    def symbol(self):
        """GeneralIntrinsic/Reduce.cpp:615-623 (f32 always resolves to the GI kernel)"""
        return "GI_kernel_reduce_%s_DEFAULT_f32_a%d" % (self.mode, self.axis)

    def spec_line(self):
        return " ".join(["ReduceKernel", "mode=s:" + self.mode, "axis=i:%d" % self.axis,
                         "data_type=s:DEFAULT", "nr_operands=i:2",
                         "operand:0=" + _op(self.shape, "f32"),
                         "operand:1=" + _op(self.out_shape, "f32")])

    def attr(self):
        return abi.ReduceAttr(abi.REDUCE_MODES[self.mode], self.axis)

    def gen(self, seed=0):
        lo, hi = (0.6, 1.5) if self.mode == "PRODUCT" else (-3.0, 3.0)
        return {"src": rng(seed).uniform(lo, hi, self.shape).astype(np.float32)}

    def specs(self, arrays):
        return ([TensorSpec(b"src", self.shape, abi.FLOAT, 1.0, arrays["src"])],
                [TensorSpec(b"dst", self.out_shape, abi.FLOAT, 1.0)])

    def run_port(self, arrays):
        return port.reduce_f32(arrays["src"], abi.REDUCE_MODES[self.mode], self.axis)


POISON = 0x5A  # byte every output buffer holds before a kernel runs


def poisoned(shape, dtype):
    return np.full(int(np.prod(shape, dtype=np.int64)) * np.dtype(dtype).itemsize, POISON,
                   np.uint8).view(dtype).reshape(shape)


DTYPES = {"f32": (abi.FLOAT, np.float32), "qsi8": (abi.QINT8, np.int8),
          "qsi32": (abi.QINT32, np.int32)}


def dense_strides(shape):
    st, s = [], 1
    for d in reversed(shape):
        st.append(s)
        s *= int(d)
    return tuple(reversed(st))


def view_of(buf, shape, strides, offset):
    """numpy view of the flat array `buf`: element strides, first element at `offset`"""
    return np.lib.stride_tricks.as_strided(
        buf.reshape(-1)[offset:], shape, [s * buf.itemsize for s in strides], writeable=True)


def span_of(shape, strides):
    """(lowest, highest) element offset a view touches relative to its first element"""
    lo = sum((d - 1) * s for d, s in zip(shape, strides) if s < 0)
    hi = sum((d - 1) * s for d, s in zip(shape, strides) if s > 0)
    return lo, hi


class RelayoutCase:
    """dst view <- src view, both strided views (element strides, None = dense) over dense
    buffers sized to the views' spans (+ `slack` untouched elements either side)."""

    def __init__(self, dtype, src_shape, src_strides=None, dst_shape=None, dst_strides=None,
                 slack=3):
        self.dtype = dtype
        self.src_shape = tuple(src_shape)
        self.dst_shape = tuple(dst_shape) if dst_shape is not None else self.src_shape
        self.src_strides = tuple(src_strides) if src_strides is not None else None
        self.dst_strides = tuple(dst_strides) if dst_strides is not None else None
        self.slack = slack

    def __repr__(self):
        return "relayout_%s%s_%s%s_to_%s%s" % (
            self.dtype, "" if self.slack == 3 else "_slack%d" % self.slack, "x".join(map(str, self.src_shape)),
            "" if self.src_strides is None else "s" + ".".join(map(str, self.src_strides)),
            "x".join(map(str, self.dst_shape)),
            "" if self.dst_strides is None else "s" + ".".join(map(str, self.dst_strides)))

    def symbol(self):
        # (GeneralIntrinsic/Relayout.cpp:43-48 comes first in the registry's candidate list;
        #  BareMetal's kernel_relayout_<dtype> is the same operator)
        return "GI_kernel_relayout_" + self.dtype

    def spec_line(self):
        sc = None if self.dtype == "f32" else 0.05
        return "RelayoutKernel operand:0=%s operand:1=%s" % (
            _op(self.src_shape, self.dtype, sc), _op(self.dst_shape, self.dtype, sc))

    def _place(self, shape, strides):
        """(strides, offset, storage elements) of a view inside its buffer"""
        if strides is None:
            return None, 0, int(np.prod(shape, dtype=np.int64))
        lo, hi = span_of(shape, strides)
        return strides, self.slack - lo, hi - lo + 1 + 2 * self.slack

    def gen(self, seed=0):
        r = rng(seed)
        _, _, n = self._place(self.src_shape, self.src_strides)
        np_dt = DTYPES[self.dtype][1]
        if self.dtype == "f32":
            src = r.standard_normal(n).astype(np.float32)
        else:
            info = np.iinfo(np_dt)
            src = r.integers(info.min, info.max, n, endpoint=True).astype(np_dt)
        return {"src": src}

    def specs(self, arrays):
        te = DTYPES[self.dtype][0]
        sc = 1.0 if self.dtype == "f32" else 0.05
        ss, so, _ = self._place(self.src_shape, self.src_strides)
        ds, do, dn = self._place(self.dst_shape, self.dst_strides)
        return ([TensorSpec(b"src", self.src_shape, te, sc, arrays["src"], ss, so)],
                [TensorSpec(b"dst", self.dst_shape, te, sc, None, ds, do,
                            storage=(dn,) if ds is not None else None)])

    def run_port(self, arrays):
        ss, so, _ = self._place(self.src_shape, self.src_strides)
        ds, do, dn = self._place(self.dst_shape, self.dst_strides)
        np_dt = DTYPES[self.dtype][1]
        if ds is None:
            out = np.zeros(self.dst_shape, np_dt)
            port.relayout(arrays["src"], so, self.src_shape, ss or dense_strides(self.src_shape),
                          out, 0, self.dst_shape, dense_strides(self.dst_shape))
            return out
        out = poisoned((dn,), np_dt)
        port.relayout(arrays["src"], so, self.src_shape, ss or dense_strides(self.src_shape),
                      out, do, self.dst_shape, ds)
        return out


class ConcatCase:
    """dense inputs of `shapes` joined along `axis`"""

    def __init__(self, dtype, shapes, axis):
        self.dtype, self.shapes, self.axis = dtype, [tuple(s) for s in shapes], axis

    def __repr__(self):
        return "concat_%s_a%d_%s" % (self.dtype, self.axis,
                                     "_".join("x".join(map(str, s)) for s in self.shapes))

    def out_shape(self):
        o = list(self.shapes[0])
        o[self.axis] = sum(s[self.axis] for s in self.shapes)
        return tuple(o)

    def symbol(self):
        return "kernel_concat_byte_%d_axis_%d" % (np.dtype(DTYPES[self.dtype][1]).itemsize,
                                                  self.axis)

    def spec_line(self):
        sc = None if self.dtype == "f32" else 0.05
        ops = ["operand:%d=%s" % (i, _op(s, self.dtype, sc)) for i, s in enumerate(self.shapes)]
        ops.append("operand:%d=%s" % (len(self.shapes), _op(self.out_shape(), self.dtype, sc)))
        return "ConcatKernel axis=i:%d nr_operands=i:%d %s" % (
            self.axis, len(self.shapes) + 1, " ".join(ops))

    def gen(self, seed=0):
        r = rng(seed)
        np_dt = DTYPES[self.dtype][1]
        out = {}
        for i, s in enumerate(self.shapes):
            if self.dtype == "f32":
                out["in%d" % i] = r.standard_normal(s).astype(np.float32)
            else:
                info = np.iinfo(np_dt)
                out["in%d" % i] = r.integers(info.min, info.max, s, endpoint=True).astype(np_dt)
        return out

    def specs(self, arrays):
        te = DTYPES[self.dtype][0]
        sc = 1.0 if self.dtype == "f32" else 0.05
        ins = [TensorSpec(b"in%d" % i, s, te, sc, arrays["in%d" % i])
               for i, s in enumerate(self.shapes)]
        return ins, [TensorSpec(b"dst", self.out_shape(), te, sc)]

    def run_port(self, arrays):
        return port.concat([arrays["in%d" % i] for i in range(len(self.shapes))], self.axis)


class ResizeCase:
    """f32 Resize [N,C,IH,IW] -> [N,C,OH,OW] (NCHW; `c` counts blocks of 4 for NCHW44).
    NEAREST reads its source through the tensor's strides (Common/Resize.h:158-175):
    `src_strides` (elements, positive) makes the source a view of a larger dense buffer."""

    def __init__(self, fmt, imode, n, c, ih, iw, oh, ow, src_strides=None):
        assert fmt in (abi.FMT_NCHW, abi.FMT_NCHW44) and imode in ("LINEAR", "NEAREST")
        assert src_strides is None or (imode == "NEAREST" and fmt == abi.FMT_NCHW)
        self.fmt, self.imode = fmt, imode
        self.n, self.c, self.ih, self.iw, self.oh, self.ow = n, c, ih, iw, oh, ow
        self.src_strides = None if src_strides is None else tuple(src_strides)

    def _fmt(self):
        return "NCHW44" if self.fmt == abi.FMT_NCHW44 else "NCHW"

    def __repr__(self):
        return "resize_%s_%s[n%d c%d %dx%d->%dx%d%s]" % (
            self._fmt(), self.imode, self.n, self.c, self.ih, self.iw, self.oh, self.ow,
            "" if self.src_strides is None else " strides " + "x".join(map(str, self.src_strides)))

    def src_shape(self):
        tail = (4,) if self.fmt == abi.FMT_NCHW44 else ()
        return (self.n, self.c, self.ih, self.iw) + tail

    def dst_shape(self):
        tail = (4,) if self.fmt == abi.FMT_NCHW44 else ()
        return (self.n, self.c, self.oh, self.ow) + tail

    def symbol(self):
        # GeneralIntrinsic/Resize.cpp:13-33 takes LINEAR, BareMetal/Resize.cpp:15-35 NEAREST
        return "%skernel_resize_linear_%s_%s_f32" % ("GI_" if self.imode == "LINEAR" else "",
                                                      self._fmt(), self.imode)

    def spec_line(self):
        return "ResizeKernel imode=s:%s format=s:%s nr_operands=i:2 operand:0=%s operand:1=%s" % (
            self.imode, self._fmt(), _op(self.src_shape(), "f32"), _op(self.dst_shape(), "f32"))

    def gen(self, seed=0):
        r = rng(seed)
        if self.src_strides is None:
            return {"src": r.uniform(-30, 30, self.src_shape()).astype(np.float32)}
        _, hi = span_of(self.src_shape(), self.src_strides)
        return {"src": r.uniform(-30, 30, hi + 1 + 3).astype(np.float32)}

    def specs(self, arrays):
        return ([TensorSpec(b"src", self.src_shape(), abi.FLOAT, 1.0, arrays["src"],
                            self.src_strides, 0)],
                [TensorSpec(b"dst", self.dst_shape(), abi.FLOAT, 1.0)])

    def run_port(self, arrays):
        return port.resize(arrays["src"], (self.oh, self.ow), self.imode,
                           self.fmt == abi.FMT_NCHW44, self.src_strides,
                           self.src_shape() if self.src_strides is not None else None)


class FusedCase:
    """a fused chain of f32 elementwise steps (`modes` as the compiler writes them: "I0,I1,ADD,O0",
    ..., compiler/test/kernel/opr/common/fused_elemwise.cpp:67-112) over inputs of `shapes`; the
    output has the shape of the largest input. Inputs are small integers as in the reference's
    test (UniformIntRNG(-10, 10), fused_elemwise.cpp:132), or positive where `positive` says so
    (LOG, divisors)."""

    GI_MODES = {"RELU", "SIGMOID", "EXP", "H_SWISH", "NEGATE", "ADD", "SUB", "MUL", "MAX", "MIN",
                "TRUE_DIV", "FUSE_ADD_RELU", "FUSE_ADD_SIGMOID", "FUSE_MUL_ADD3", "FUSE_MUL_ADD4"}

    def __init__(self, modes, shapes, positive=()):
        self.modes, self.shapes = list(modes), [tuple(s) for s in shapes]
        self.positive = set(positive)
        self.out_shape = max(self.shapes, key=lambda sh: int(np.prod(sh)))
        self.prog = abi.parse_fused_modes(self.modes, len(self.shapes))

    def __repr__(self):
        return "fused[%s | %s]" % (" ".join(m.split(",")[-2] for m in self.modes),
                                   " ".join("x".join(map(str, s)) for s in self.shapes))

    def types(self):
        """Common/ElemwiseCommon.cpp:7-45"""
        n = int(np.prod(self.out_shape))
        out = []
        for sh in self.shapes:
            ne = int(np.prod(sh))
            if ne == n:
                out.append(0)
            elif ne == 1:
                out.append(1)
            elif len(sh) == 4 and sh[0] == 1 and sh[2] == 1 and sh[3] == 1:
                out.append(2)
            else:
                assert len(sh) == 5 and sh[0] == 1 and sh[2] == 1 and sh[3] == 1 and sh[4] == 4, sh
                out.append(3)
        return out

    def symbol(self):
        # GeneralIntrinsic/FusedElemwiseKernel.cpp:680-726 when it knows every mode, else
        # BareMetal/FusedElemwiseKernel.cpp:270-317; the output counts as one more VECTOR operand
        names = [m.split(",")[-2] for m in self.modes]
        # (both availability checks keep only their verdict on the last step)
        head = "kernel_gi_fused_elementwise" if names[-1] in self.GI_MODES \
            else "kernel_naive_fused_elementwise"
        return "%s_%s_%s_%s" % (head, "_".join(names),
                                "_".join("tensortype%d" % t for t in self.types() + [0]),
                                "f32" * (len(self.shapes) + 1))

    def spec_line(self):
        ops = ["operand:%d=%s" % (i, _op(s, "f32")) for i, s in enumerate(self.shapes)]
        ops.append("operand:%d=%s" % (len(self.shapes), _op(self.out_shape, "f32")))
        ms = ["modes:%d=s:%s" % (i, m) for i, m in enumerate(self.modes)]
        return "FusedElemwiseKernel modes:size=i:%d %s nr_operands=i:%d %s" % (
            len(self.modes), " ".join(ms), len(self.shapes) + 1, " ".join(ops))

    def gen(self, seed=0):
        r = rng(seed)
        out = {}
        for i, sh in enumerate(self.shapes):
            lo = 1 if i in self.positive else -10
            out["in%d" % i] = r.integers(lo, 10, sh, endpoint=True).astype(np.float32)
        return out

    def specs(self, arrays):
        ins = [TensorSpec(b"in%d" % i, s, abi.FLOAT, 1.0, arrays["in%d" % i])
               for i, s in enumerate(self.shapes)]
        return ins, [TensorSpec(b"dst", self.out_shape, abi.FLOAT, 1.0)]

    def desc(self):
        d = abi.KernelDesc()
        d.kind = abi.KERN_FUSED_ELEMWISE
        d.attr.fused = abi.fused_attr(self.prog, len(self.shapes))
        return d

    def run_port(self, arrays):
        return port.fused_elemwise(self.prog, [arrays["in%d" % i] for i in range(len(self.shapes))],
                                   self.types(), self.out_shape)


class SoftmaxCase:
    """soft-max over the last axis in one kernel (megcc_gfx950_softmax): what the importer's
    decomposition Reduce MAX -> SUB -> EXP -> Reduce SUM -> TRUE_DIV computes
    (compiler/lib/Target/MGB/importer.cpp:987-1016), optionally from qsi8 logits that
    GI_kernel_typecvt_qsi8f32 would dequantise first. The oracle is that chain of oracle calls."""

    def __init__(self, shape, quantised=False, scale=0.1, span=(-8.0, 8.0)):
        self.shape, self.quantised, self.scale, self.span = tuple(shape), quantised, scale, span

    def __repr__(self):
        return "softmax%s[%s]" % ("_q8" if self.quantised else "", "x".join(map(str, self.shape)))

    def symbol(self):
        return None  # no reference symbol: the kernel is addressed by a descriptor

    def desc(self):
        d = abi.KernelDesc()
        d.kind = abi.KERN_SOFTMAX
        return d

    def gen(self, seed=0):
        r = rng(seed)
        if self.quantised:
            return {"src": r.integers(-128, 128, self.shape).astype(np.int8)}
        return {"src": r.uniform(self.span[0], self.span[1], self.shape).astype(np.float32)}

    def specs(self, arrays):
        if self.quantised:
            ins = [TensorSpec(b"src", self.shape, abi.QINT8, self.scale, arrays["src"])]
        else:
            ins = [TensorSpec(b"src", self.shape, abi.FLOAT, 1.0, arrays["src"])]
        return ins, [TensorSpec(b"dst", self.shape, abi.FLOAT, 1.0)]

    def run_port(self, arrays):
        x = arrays["src"]
        if self.quantised:
            x = port.typecvt(np.ascontiguousarray(x), "qsi8", "f32", self.scale, 1.0)
        x2 = np.ascontiguousarray(x.reshape(-1, self.shape[-1]))
        mx = port.reduce_f32(x2, abi.REDUCE_MAX, 1)
        e = port.elemwise_f32(port.elemwise_f32(x2, mx, abi.EW_SUB), None, abi.EW_EXP)
        return port.elemwise_f32(e, port.reduce_f32(e, abi.REDUCE_SUM, 1), abi.EW_TRUE_DIV).reshape(self.shape)


def run_ref(case, arrays, symbol=None):
    """Evaluate `case` with the reference's generated C kernel; returns the output array."""
    ins, outs = case.specs(arrays)
    o = outs[0]
    strided = o.strides is not None
    out_arr = (poisoned if strided else np.zeros)(o.storage, abi.np_dtype(o.type_enum))
    tin = [abi.host_tensor(s.array, s.type_enum, s.scale, s.name,
                           s.shape if s.strides is not None else None, s.strides, s.offset)
           for s in ins]
    tout = [abi.host_tensor(out_arr, o.type_enum, o.scale, o.name, o.shape if strided else None,
                            o.strides, o.offset)]
    ref.run(symbol or case.symbol(), tin, tout)
    return out_arr


def max_rel_err(got, want):
    """|a-b| / max(1, min(|a|,|b|)): the reference's model-level metric (ci/compare_output_bin.py)."""
    got = got.astype(np.float64)
    want = want.astype(np.float64)
    d = np.abs(got - want) / np.maximum(1.0, np.minimum(np.abs(got), np.abs(want)))
    return float(d.max()) if d.size else 0.0
