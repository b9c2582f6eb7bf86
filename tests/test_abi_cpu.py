"""CPU-only checks of the boundary: the library loads, exports every entry point the header
declares, and the host-side logic that needs no GPU (symbol parsing, workspace size, argument
validation) behaves like the reference's."""
import ctypes as C
import json
import os
import re

import pytest

from megcc_amd import abi, runtime

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)


def header_functions():
    text = open(os.path.join(ROOT, "include", "megcc_gfx950.h")).read()
    return sorted(set(re.findall(r"\b(megcc_gfx950_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    L = runtime.lib()
    declared = header_functions()
    assert len(declared) >= 20
    for name in declared:
        assert hasattr(L, name), name
    assert sorted(runtime.EXPORTS) == declared


def test_struct_sizes_match_the_c_abi():
    # x86-64 layout of runtime/src/data_struct.h: Layout = 4 + 28 + 28 + 4, Tensor = 8 + 12 + 64 + ...
    assert C.sizeof(abi.Layout) == 64
    assert C.sizeof(abi.DType) == 12
    assert C.sizeof(abi.Tensor) == 136
    assert C.sizeof(abi.Workspace) == 24
    assert C.sizeof(abi.Device) == 24


with open(os.path.join(HERE, "golden", "symbols.json")) as f:
    SYMBOLS = json.load(f)


@pytest.mark.parametrize("symbol", sorted(set(SYMBOLS.values())))
def test_every_reference_symbol_parses(symbol):
    if "fused_elementwise" in symbol:
        # the reference names a fused chain by its modes and operand kinds only; which value feeds
        # which step is not in the name, so the library refuses to guess (the shim carries it)
        with pytest.raises(runtime.MegccError):
            runtime.parse_symbol(symbol)
        return
    desc = runtime.parse_symbol(symbol)
    assert desc.kind in range(1, 11)


def test_parse_conv_symbol_fields():
    d = runtime.parse_symbol(
        "kernel_conv2d_3x3_NCHW44_DENSE_p1x1_s2x2_d1x1_qsi8qsi8qsi32qsi8_bias_H_SWISH")
    a = d.attr.conv
    assert d.kind == abi.KERN_CONV
    assert (a.kernel_h, a.kernel_w, a.pad_h, a.pad_w, a.stride_h, a.stride_w) == (3, 3, 1, 1, 2, 2)
    assert (a.format, a.sparse, a.nonline, a.with_bias) == (abi.FMT_NCHW44, abi.DENSE, abi.H_SWISH, 1)
    d = runtime.parse_symbol("kernel_conv2d_3x3_NCHW_NCHW44_DENSE_p1x1_s2x2_d1x1_qsi8qsi8qsi32qsi8_bias_RELU")
    assert d.attr.conv.format == abi.FMT_NCHW_NCHW44 and d.attr.conv.nonline == abi.RELU
    d = runtime.parse_symbol("GI_kernel_conv2d_im2col_3x3_NCHW_DENSE_p1x1_s1x1_d1x1_bias_RELUf32")
    assert (d.attr.conv.format, d.attr.conv.with_bias, d.attr.conv.nonline) == (abi.FMT_NCHW, 1, abi.RELU)
    d = runtime.parse_symbol("GI_kernel_conv2d_im2col_3x3_NCHW_DENSE_p1x1_s1x1_d1x1f32")
    assert (d.attr.conv.with_bias, d.attr.conv.nonline) == (0, abi.IDENTITY)


def test_parse_f32_nchw44_symbols_of_the_general_intrinsic_pack():
    """the names MegCC's GI pack gives the f32 NCHW44 layers: all three Winograd variants (F63 is
    the first choice of a 3x3 stride-1 layer, GeneralIntrinsic/KernelPack.cpp:54-56; F43 and F63
    end in _fp32, Fp32WinogradNchw44.cpp:157,231), the NCHW -> NCHW44 first layer
    (Fp32ConvNchwNchw44.cpp:37-55) and the channel-wise kernel (ConvKernel.h:63-65)"""
    base = "GI_kernel_conv2d_3x3_NCHW44_DENSE_p1x1_s1x1_d1x1_f32f32f32f32_bias_RELU"
    for tail in ("_winograd_f23", "_winograd_f43_fp32", "_winograd_f63_fp32"):
        a = runtime.parse_symbol(base + tail).attr.conv
        assert (a.format, a.sparse, a.kernel_h, a.with_bias, a.nonline) == (abi.FMT_NCHW44, abi.DENSE, 3, 1, abi.RELU)
    for bad in ("_winograd_f43", "_winograd_f63", "_winograd_f23_fp32"):
        with pytest.raises(runtime.MegccError):
            runtime.parse_symbol(base + bad)
    a = runtime.parse_symbol(
        "GI_kernel_conv2d_3x3_NCHW_NCHW44_DENSE_p1x1_s2x2_d1x1_f32f32f32f32_bias_H_SWISH_nchw_nchw44_oc32_ic3").attr.conv
    assert (a.format, a.stride_h, a.pad_w, a.nonline, a.with_bias) == (abi.FMT_NCHW_NCHW44, 2, 1, abi.H_SWISH, 1)
    a = runtime.parse_symbol("GI_kernel_conv2d_5x5_NCHW_NCHW44_DENSE_p2x2_s1x1_d1x1_f32f32f32_nchw_nchw44_oc8_ic1").attr.conv
    assert (a.format, a.kernel_w, a.with_bias, a.nonline) == (abi.FMT_NCHW_NCHW44, 5, 0, abi.IDENTITY)
    a = runtime.parse_symbol("GI_chanwise_kernel_conv2d_5x5_NCHW44_GROUP_p2x2_s2x2_d1x1_f32f32f32f32_bias_RELU").attr.conv
    assert (a.format, a.sparse, a.kernel_h, a.stride_w, a.nonline) == (abi.FMT_NCHW44, abi.GROUP, 5, 2, abi.RELU)
    for bad in ("GI_chanwise_kernel_conv2d_3x3_NCHW44_DENSE_p1x1_s1x1_d1x1_f32f32f32f32",
                "kernel_conv2d_3x3_NCHW44_DENSE_p1x1_s2x2_d1x1_f32f32f32f32_nchw_nchw44_oc32_ic3",
                "GI_kernel_conv2d_3x3_NCHW_DENSE_p1x1_s2x2_d1x1_f32f32f32f32_nchw_nchw44_oc32_ic3"):
        with pytest.raises(runtime.MegccError):
            runtime.parse_symbol(bad)


def test_parse_other_symbols():
    d = runtime.parse_symbol("kernel_pooling_AVERAGE_COUNT_EXCLUDE_PADDING_NCHW_p1x1_s2x2_w3x3_qsi8qsi8")
    assert d.kind == abi.KERN_POOLING and d.attr.pool.mode == abi.POOL_AVERAGE_COUNT_EXCLUDE_PADDING
    assert (d.attr.pool.window_h, d.attr.pool.stride_w, d.attr.pool.pad_h) == (3, 2, 1)
    d = runtime.parse_symbol("GI_kernel_pooling_MAX_NCHW44_p0x0_s2x2_w2x2_qsi8qsi8_qsi8qsi8_fallback")
    assert d.attr.pool.format == abi.FMT_NCHW44 and d.attr.pool.mode == abi.POOL_MAX
    d = runtime.parse_symbol("kernel_elementwise_multitype_QFUSE_ADD_RELU_qsi8qsi8qsi8")
    assert d.kind == abi.KERN_ELEMWISE_MULTITYPE and d.attr.multitype == abi.Q_FUSE_ADD_RELU
    d = runtime.parse_symbol("GI_kernel_elementwise_TRUE_DIV_f32_binary_VEC_VEC_f32f32f32")
    assert d.kind == abi.KERN_ELEMWISE and d.attr.elemwise == abi.EW_TRUE_DIV
    d = runtime.parse_symbol("GI_kernel_reduce_MAX_DEFAULT_f32_a1")
    assert d.kind == abi.KERN_REDUCE and (d.attr.reduce.mode, d.attr.reduce.axis) == (abi.REDUCE_MAX, 1)
    d = runtime.parse_symbol("GI_kernel_gevm_nn")
    assert d.kind == abi.KERN_MATMUL and d.attr.matmul.transpose_b == 0
    d = runtime.parse_symbol("GI_kernel_fp32_matmul_4x12_nt")
    assert d.attr.matmul.transpose_b == 1
    for sym in ("kernel_relayout_f32", "GI_kernel_relayout_qsi8", "kernel_relayout_ui8"):
        assert runtime.parse_symbol(sym).kind == abi.KERN_RELAYOUT
    d = runtime.parse_symbol("kernel_concat_byte_4_axis_2")
    assert d.kind == abi.KERN_CONCAT and d.attr.concat_axis == 2
    d = runtime.parse_symbol("GI_kernel_resize_linear_NCHW44_LINEAR_f32")
    assert d.kind == abi.KERN_RESIZE
    assert (d.attr.resize.format, d.attr.resize.imode) == (abi.FMT_NCHW44, abi.IMODE_LINEAR)
    d = runtime.parse_symbol("kernel_resize_linear_NCHW_NEAREST_f32")
    assert (d.attr.resize.format, d.attr.resize.imode) == (abi.FMT_NCHW, abi.IMODE_NEAREST)


def test_copy_kernels_reject_bad_arguments_before_any_launch():
    """the checks of Relayout / Concat need no GPU: nothing is launched on a mismatch"""
    L = runtime.lib()
    fake = 0x1000  # never dereferenced
    t = lambda shape, te=abi.FLOAT, strides=None: abi.make_tensor(fake, shape, te, strides=strides)
    call = lambda fn, ins, out, *pre: fn(*pre, abi.tensor_array(ins), len(ins),
                                         abi.tensor_array([out]), 1, None, None)
    assert call(L.megcc_gfx950_relayout, [t((2, 3))], t((2, 3), abi.QINT8)) == \
        abi.ERROR_UNSUPPORTED_DTYPE_TYPE
    assert call(L.megcc_gfx950_relayout, [t((2, 3))], t((2, 4))) == abi.ERROR_INVALID_LAYOUT
    assert call(L.megcc_gfx950_relayout, [t((2, 3))], t((2, 3), strides=(0, 1))) == \
        abi.ERROR_INVALID_LAYOUT  # two rows written to the same place
    assert call(L.megcc_gfx950_relayout, [t((0, 3))], t((0, 3))) == 0  # empty: nothing to do
    axis = C.c_int(1)
    assert call(L.megcc_gfx950_concat, [t((2, 3)), t((2, 4))], t((2, 8)), C.byref(axis)) == \
        abi.ERROR_INVALID_LAYOUT
    assert call(L.megcc_gfx950_concat, [t((2, 3)), t((3, 4))], t((2, 7)), C.byref(axis)) == \
        abi.ERROR_INVALID_LAYOUT
    assert call(L.megcc_gfx950_concat, [t((2, 3)), t((2, 4), abi.QINT8)], t((2, 7)),
                C.byref(axis)) == abi.ERROR_UNSUPPORTED_DTYPE_TYPE
    axis = C.c_int(2)
    assert call(L.megcc_gfx950_concat, [t((2, 3))], t((2, 3)), C.byref(axis)) == \
        abi.ERROR_OUT_OF_RANGE
    assert L.megcc_gfx950_concat(None, None, 0, None, 0, None, None) == abi.ERROR_NULL_PTR
    lin = abi.ResizeAttr(abi.FMT_NCHW, abi.IMODE_LINEAR)
    assert call(L.megcc_gfx950_resize, [t((1, 2, 4, 4))], t((1, 3, 8, 8)), C.byref(lin)) == \
        abi.ERROR_INVALID_LAYOUT  # channels differ
    assert call(L.megcc_gfx950_resize, [t((1, 2, 4, 4), strides=(64, 32, 8, 2))], t((1, 2, 8, 8)),
                C.byref(lin)) == abi.ERROR_INVALID_LAYOUT  # LINEAR reads dense tensors only
    assert call(L.megcc_gfx950_resize, [t((1, 2, 4, 4), abi.QINT8)], t((1, 2, 8, 8), abi.QINT8),
                C.byref(lin)) == abi.ERROR_UNSUPPORTED_DTYPE_TYPE
    assert call(L.megcc_gfx950_resize, [t((1, 2, 4, 4))], t((1, 2, 0, 8)), C.byref(lin)) == 0
    near44 = abi.ResizeAttr(abi.FMT_NCHW44, abi.IMODE_NEAREST)
    assert call(L.megcc_gfx950_resize, [t((1, 2, 4, 4, 4))], t((1, 2, 8, 8, 4)),
                C.byref(near44)) == abi.ERROR_OUT_OF_RANGE  # no such kernel in the reference
    assert L.megcc_gfx950_resize(None, None, 0, None, 0, None, None) == abi.ERROR_NULL_PTR
    # fused elementwise: the program is checked before anything is launched
    prog = abi.parse_fused_modes(["I0,I1,ADD,O0", "O0,RELU,D"], 2)
    ok = abi.fused_attr(prog, 2)
    x = t((2, 3, 4, 5))
    assert call(L.megcc_gfx950_fused_elemwise, [x, t((1, 3, 1, 1))], t((0, 3, 4, 5)), C.byref(ok)) == 0
    assert call(L.megcc_gfx950_fused_elemwise, [x, t((1, 4, 1, 1))], x, C.byref(ok)) == \
        abi.ERROR_INVALID_LAYOUT  # neither the output's size, a scalar nor [1,C,1,1]
    assert call(L.megcc_gfx950_fused_elemwise, [x], x, C.byref(ok)) == \
        abi.ERROR_OUT_OF_RANGE  # 1 input, the program wants 2
    late = abi.fused_attr([(abi.EW_ADD, [0, 3]), (abi.EW_RELU, [2])], 2)  # reads step 1's result in step 0
    assert call(L.megcc_gfx950_fused_elemwise, [x, x], x, C.byref(late)) == abi.ERROR_OUT_OF_RANGE
    arity = abi.fused_attr([(abi.EW_ADD, [0])], 2)
    assert call(L.megcc_gfx950_fused_elemwise, [x, x], x, C.byref(arity)) == abi.ERROR_OUT_OF_RANGE
    assert call(L.megcc_gfx950_fused_elemwise, [x, t((2, 3, 4, 5), abi.QINT8)], x, C.byref(ok)) == \
        abi.ERROR_UNSUPPORTED_DTYPE_TYPE


def test_unknown_symbol_is_reported_not_guessed():
    desc = abi.KernelDesc()
    for bad in ("kernel_argsort_f32", "kernel_relayout_f64", "kernel_concat_byte_8_axis_0",
                "kernel_concat_byte_4_axis_1x", "kernel_resize_linear_NCHW44_NEAREST_f32",
                "GI_kernel_resize_linear_NHWC_LINEAR_f32",
                "kernel_gi_fused_elementwise_ADD_RELU_tensortype0_tensortype0_tensortype0_f32f32f32", "kernel_resize_linear_NCHW_LINEAR_f16", "kernel_conv2d_3x3_NHWC_DENSE_p1x1_s1x1_d1x1_f32f32f32",
                "kernel_typecvt_f16f32", ""):
        st = runtime.lib().megcc_gfx950_parse_symbol(bad.encode(), C.byref(desc))
        assert st == abi.ERROR_NO_FOUND
        assert b"not a kernel" in runtime.lib().megcc_gfx950_last_error()


def test_null_arguments_are_rejected():
    L = runtime.lib()
    attr = abi.ConvAttr(3, 3, 1, 1, 1, 1, 1, 1, abi.FMT_NCHW44, abi.DENSE, abi.RELU, 1)
    assert L.megcc_gfx950_conv2d(C.byref(attr), None, 0, None, 0, None, None) == abi.ERROR_NULL_PTR
    assert L.megcc_gfx950_conv2d(None, None, 0, None, 0, None, None) == abi.ERROR_NULL_PTR
    size = C.c_size_t(123)
    assert L.megcc_gfx950_conv2d_workspace(C.byref(attr), None, 0, 1, C.byref(size)) == 0
    assert size.value == 0
