"""The small cases whose reference outputs are committed under tests/golden/ (see
tests/golden/make_golden.py). Shapes follow the reference's own kernel tests
(compiler/test/kernel/opr/naive/conv.cpp:53-264, pool.cpp:6-66, elemwise_multitype.cpp:6-64,
typecvt.cpp:5-70): odd sizes, k in {1,3}, stride in {1,2}, pad in {0,k/2}, every activation, the
small-magnitude tie case and the 30..50 overflow case."""
from megcc_amd import abi
from cases import (ConcatCase, ConvCase, ElemwiseCase, FusedCase, MatMulCase, MultiTypeCase, PoolCase,
                   ReduceCase, RelayoutCase, ResizeCase, TypeCvtCase)

A = abi


def unsat(k_taps):
    """dst scale that keeps outputs inside [-128,127] for full-range int8 data: the accumulator's
    std is about 74*73*sqrt(K); put 3 sigma near 100."""
    return 0.02 * 0.01 * 5.4e3 * (k_taps ** 0.5) / 35.0


def golden_cases():
    c = {}
    # --- qsi8 dense NCHW44 3x3 (headline kernel), every activation, saturating and not
    for act in (A.IDENTITY, A.RELU, A.H_SWISH, A.SIGMOID):
        c["conv44_3x3_s1_%s" % A.NONLINE_NAMES[act]] = ConvCase(
            A.FMT_NCHW44, A.DENSE, 2, 8, 7, 9, 12, 3, 1, 1, act, scales=(0.02, 0.01, unsat(72)))
    c["conv44_3x3_s1_RELU_baseline_scales"] = ConvCase(
        A.FMT_NCHW44, A.DENSE, 1, 16, 9, 11, 16, 3, 1, 1, A.RELU, scales=(0.02, 0.01, 0.05))
    # rounding ties: acc * 0.5 * 0.5 / 0.5 = acc / 2 -> every odd accumulator is an exact .5
    c["conv44_3x3_s1_ties"] = ConvCase(
        A.FMT_NCHW44, A.DENSE, 1, 8, 6, 5, 8, 3, 1, 1, A.IDENTITY, scales=(0.5, 0.5, 0.5),
        src_range=(-3, 3), flt_range=(-3, 3), bias_range=(-3, 3))
    # overflow case of the reference tests: all-positive 30..50 -> clamps at 127
    c["conv44_3x3_s1_overflow"] = ConvCase(
        A.FMT_NCHW44, A.DENSE, 1, 8, 6, 5, 8, 3, 1, 1, A.IDENTITY, scales=(1.0, 1.0, 1.0),
        src_range=(30, 50), flt_range=(30, 50), bias_range=(30, 50))
    c["conv44_3x3_s2_RELU"] = ConvCase(
        A.FMT_NCHW44, A.DENSE, 2, 8, 9, 8, 8, 3, 2, 1, A.RELU, scales=(0.02, 0.01, unsat(72)))
    c["conv44_3x3_s1_p0"] = ConvCase(
        A.FMT_NCHW44, A.DENSE, 1, 8, 7, 7, 8, 3, 1, 0, A.IDENTITY, scales=(0.02, 0.01, unsat(72)))
    c["conv44_1x1_RELU"] = ConvCase(
        A.FMT_NCHW44, A.DENSE, 2, 16, 5, 7, 24, 1, 1, 0, A.RELU, scales=(0.02, 0.01, unsat(16)))
    c["conv44_1x1_s2_RELU"] = ConvCase(
        A.FMT_NCHW44, A.DENSE, 2, 16, 9, 8, 24, 1, 2, 0, A.RELU, scales=(0.02, 0.01, unsat(16)))
    # (a qsi8 conv without bias does not exist in the reference: ConvGeneral::IsAvailable wants
    #  operand:2 to be qsi32, BareMetal/ConvKernel.cpp:25-29)
    # --- qsi8 NCHW dense: FullyConnected (1x1 on [M,K,1,1]) and 3x3
    c["fc_q8_5x40x13"] = ConvCase(
        A.FMT_NCHW, A.DENSE, 5, 40, 1, 1, 13, 1, 1, 0, A.IDENTITY, scales=(0.01, 0.01, unsat(40) / 2))
    c["fc_q8_1x64x10_RELU"] = ConvCase(
        A.FMT_NCHW, A.DENSE, 1, 64, 1, 1, 10, 1, 1, 0, A.RELU, scales=(0.01, 0.01, 0.1))
    c["conv_nchw_3x3_s1"] = ConvCase(
        A.FMT_NCHW, A.DENSE, 2, 5, 7, 6, 7, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(45)))
    c["conv_nchw_3x3_s2"] = ConvCase(
        A.FMT_NCHW, A.DENSE, 1, 5, 9, 9, 6, 3, 2, 1, A.IDENTITY, scales=(0.02, 0.01, unsat(45)))
    # --- depthwise
    for s in (1, 2):
        c["dw44_3x3_s%d_RELU" % s] = ConvCase(
            A.FMT_NCHW44, A.GROUP, 2, 8, 9, 7, 8, 3, s, 1, A.RELU, scales=(0.02, 0.01, unsat(9)))
        c["dw_nchw_3x3_s%d_RELU" % s] = ConvCase(
            A.FMT_NCHW, A.GROUP, 2, 6, 9, 7, 6, 3, s, 1, A.RELU, scales=(0.02, 0.01, unsat(9)))
    c["dw44_3x3_s1_IDENTITY_baseline_scales"] = ConvCase(
        A.FMT_NCHW44, A.GROUP, 1, 8, 6, 6, 8, 3, 1, 1, A.IDENTITY, scales=(0.02, 0.01, 0.05))
    # --- first layer NCHW -> NCHW44
    c["conv_hybrid_3x3_s2_RELU"] = ConvCase(
        A.FMT_NCHW_NCHW44, A.DENSE, 2, 3, 11, 9, 8, 3, 2, 1, A.RELU, scales=(0.02, 0.01, unsat(27)))
    # --- f32 (tolerance-based)
    c["conv_f32_3x3_RELU"] = ConvCase(A.FMT_NCHW, A.DENSE, 1, 6, 9, 8, 5, 3, 1, 1, A.RELU, dtype="f32")
    c["matmul_f32_11x8x13"] = MatMulCase(11, 8, 13)
    c["gevm_f32_1x37x29"] = MatMulCase(1, 37, 29)
    # --- pooling
    c["pool_max_nchw_2x2"] = PoolCase(A.FMT_NCHW, A.POOL_MAX, 2, 3, 8, 6, 2, 2, 0)
    c["pool_max_nchw44_2x2"] = PoolCase(A.FMT_NCHW44, A.POOL_MAX, 2, 8, 8, 6, 2, 2, 0)
    c["pool_max_nchw_3x3_p1"] = PoolCase(A.FMT_NCHW, A.POOL_MAX, 1, 3, 9, 7, 3, 2, 1)
    c["pool_max_nchw44_3x3_p1"] = PoolCase(A.FMT_NCHW44, A.POOL_MAX, 1, 8, 9, 7, 3, 2, 1)
    c["pool_avg_nchw_7x7"] = PoolCase(A.FMT_NCHW, A.POOL_AVERAGE, 2, 5, 7, 7, 7, 7, 0)
    c["pool_avg_nchw44_7x7"] = PoolCase(A.FMT_NCHW44, A.POOL_AVERAGE, 2, 8, 7, 7, 7, 7, 0)
    c["pool_avg_nchw_3x3_p1"] = PoolCase(A.FMT_NCHW, A.POOL_AVERAGE, 1, 3, 9, 7, 3, 2, 1)
    c["pool_avgx_nchw_3x3_p1"] = PoolCase(
        A.FMT_NCHW, A.POOL_AVERAGE_COUNT_EXCLUDE_PADDING, 1, 3, 9, 7, 3, 2, 1)
    # --- quantized elemwise: three broadcast modes
    for mode in (A.Q_ADD, A.Q_FUSE_ADD_RELU, A.Q_MUL):
        nm = A.MULTITYPE_NAMES[mode]
        sc = (0.05, 0.01, 0.05) if mode != A.Q_MUL else (0.05, 0.04, 0.3)
        c["%s_vec" % nm] = MultiTypeCase(mode, (2, 3, 5, 7), sc)
        c["%s_chan" % nm] = MultiTypeCase(mode, (2, 3, 5, 7), sc, bshape=(1, 3, 1, 1))
        c["%s_scalar" % nm] = MultiTypeCase(mode, (2, 3, 5, 7), sc, bshape=(1,))
    c["QRELU"] = MultiTypeCase(A.Q_RELU, (2, 3, 5, 7), (0.05, 0.01, 0.03))
    c["QADD_ties"] = MultiTypeCase(A.Q_ADD, (4, 1, 8, 8), (0.5, 0.5, 1.0))
    # --- typecvt (37 elements: SIMD body of 16 + scalar tail)
    c["cvt_f32_q8"] = TypeCvtCase("f32", "qsi8", (3, 37), dst_scale=0.02)
    c["cvt_q8_f32"] = TypeCvtCase("qsi8", "f32", (3, 37), src_scale=0.05)
    c["cvt_q8_q8"] = TypeCvtCase("qsi8", "qsi8", (3, 37), src_scale=0.05, dst_scale=0.02)
    c["cvt_q32_q8"] = TypeCvtCase("qsi32", "qsi8", (3, 37), src_scale=0.0002, dst_scale=0.05)
    # --- relayout: the layouts of compiler/test/kernel/opr/naive/relayout.cpp:7-131 (NCHW <->
    # NCHW4, negative strides, the transposes of RelayoutFast both ways, a strided destination)
    for dt in ("f32", "qsi8"):
        n, ch, hw = 3, 8, 5
        nchw4_as_nchw = (ch * hw * hw, hw * hw * 4, hw, 1, hw * hw)
        c["relayout_%s_nchw_to_nchw4" % dt] = RelayoutCase(
            dt, (n, ch // 4, hw, hw, 4), nchw4_as_nchw)
        c["relayout_%s_nchw4_to_nchw" % dt] = RelayoutCase(
            dt, (n, ch // 4, hw, hw, 4), None, None, nchw4_as_nchw)
        c["relayout_%s_neg_w" % dt] = RelayoutCase(dt, (1, 2, 3, 4), (24, 12, 4, -1))
        c["relayout_%s_neg_h" % dt] = RelayoutCase(dt, (1, 2, 3, 4), (24, 12, -4, 1))
        n, ch, h, w = 2, 8, 2, 3
        fast = [
            ((n, h, w, ch), (ch * h * w, w, 1, h * w), (n, ch, h, w)),
            ((n, ch, h, w), (ch * h * w, 1, ch * w, ch), (n, h, w, ch)),
            ((n, ch // 4, h, w, 4), (ch * h * w, h * w * 4, w, 1, h * w), (n, ch // 4, 4, h, w)),
            ((n, ch // 4, 4, h, w), (ch * h * w, h * w * 4, 1, w * 4, 4), (n, ch // 4, h, w, 4)),
        ]
        for i, (shape, strides, other) in enumerate(fast):
            c["relayout_%s_fast%d" % (dt, i)] = RelayoutCase(dt, shape, strides, other)
            c["relayout_%s_fast%d_back" % (dt, i)] = RelayoutCase(dt, other, None, shape, strides)
        c["relayout_%s_into_slice" % dt] = RelayoutCase(
            dt, (n, ch, h, w), None, None, (ch * 3 * h * w, 3 * h * w, w, 1))
        c["relayout_%s_step2" % dt] = RelayoutCase(dt, (3, 5, 7), (140, 14, 2), None, (70, 7, 1))
        c["relayout_%s_views" % dt] = RelayoutCase(dt, (6, 4), (9, 2), (2, 12), (31, 2))
        c["relayout_%s_broadcast" % dt] = RelayoutCase(dt, (4, 5, 6), (6, 0, 1))
    # --- concat: compiler/test/kernel/opr/naive/concat.cpp:5-28 (4 inputs, extent i+1 along axis)
    for dt in ("f32", "qsi8"):
        for axis in range(4):
            shapes = []
            for i in range(4):
                sh = [3, 4, 5, 6]
                sh[axis] = i + 1
                shapes.append(tuple(sh))
            c["concat_%s_axis%d" % (dt, axis)] = ConcatCase(dt, shapes, axis)
    # --- resize: the shapes of compiler/test/kernel/opr/naive/resize.cpp:7-35 (up and down, both
    # at once), then the corners of get_coord: extent 1 in and out, same size, a strided source
    for i, (n, ch, ih, iw, oh, ow) in enumerate(((1, 1, 5, 6, 7, 13), (1, 4, 5, 6, 9, 12),
                                                  (2, 3, 15, 16, 9, 12))):
        c["resize_linear_nchw_%d" % i] = ResizeCase(A.FMT_NCHW, "LINEAR", n, ch, ih, iw, oh, ow)
        c["resize_linear_nchw44_%d" % i] = ResizeCase(A.FMT_NCHW44, "LINEAR", n, ch, ih, iw, oh, ow)
        c["resize_nearest_nchw_%d" % i] = ResizeCase(A.FMT_NCHW, "NEAREST", n, ch, ih, iw, oh, ow)
    c["resize_linear_nchw_from_1x1"] = ResizeCase(A.FMT_NCHW, "LINEAR", 2, 3, 1, 1, 4, 5)
    c["resize_linear_nchw_row"] = ResizeCase(A.FMT_NCHW, "LINEAR", 1, 2, 1, 7, 3, 10)
    c["resize_linear_nchw_to_1x1"] = ResizeCase(A.FMT_NCHW, "LINEAR", 1, 2, 6, 9, 1, 1)
    c["resize_linear_nchw44_same"] = ResizeCase(A.FMT_NCHW44, "LINEAR", 1, 2, 6, 5, 6, 5)
    c["resize_linear_nchw_x2"] = ResizeCase(A.FMT_NCHW, "LINEAR", 1, 3, 8, 10, 16, 20)
    c["resize_nearest_nchw_x2"] = ResizeCase(A.FMT_NCHW, "NEAREST", 1, 3, 8, 10, 16, 20)
    # --- fused elementwise: the chains and shapes of compiler/test/kernel/opr/naive/fused_elemwise.cpp
    # (the reference names a kernel by its modes and operand kinds only, so every case here has a
    # name of its own), then the modes only the BareMetal generator knows
    two_x_plus = ["I0,I1,ADD,O0", "I2,O0,MUL,O1", "O0,I3,SUB,D"]
    c["fused_2xy_vec"] = FusedCase(two_x_plus, [(4, 6, 9, 2), (4, 6, 9, 2), (1,), (4, 6, 9, 2)])
    c["fused_2xy_bcast101"] = FusedCase(two_x_plus, [(1, 6, 1, 1), (4, 6, 9, 2), (1,), (4, 6, 9, 2)])
    more = ["I0,I1,ADD,O0", "O0,SIGMOID,O1", "O1,I2,MAX,O2", "O2,I2,TRUE_DIV,D"]
    c["fused_more_101x4_scalar"] = FusedCase(more, [(3, 10, 10, 5, 4), (1, 10, 1, 1, 4), (1,)], positive=(2,))
    c["fused_more_vec"] = FusedCase(more, [(3, 10, 10, 5, 4)] * 3, positive=(2,))
    c["fused_more_101x4_twice"] = FusedCase(more, [(3, 10, 10, 5, 4), (1, 10, 1, 1, 4), (1, 10, 1, 1, 4)],
                                            positive=(2,))
    c["fused_relu_exp"] = FusedCase(["I0,RELU,O0", "I1,EXP,O1", "O0,O1,FUSE_ADD_RELU,D"],
                                    [(3, 10, 10, 5, 4), (1, 10, 1, 1, 4)])
    c["fused_neg_hswish"] = FusedCase(["I0,NEGATE,O0", "I1,H_SWISH,O1", "O0,O1,FUSE_ADD_SIGMOID,D"],
                                      [(3, 10, 10, 5, 4), (1, 10, 1, 1, 4)])
    c["fused_mul_add3"] = FusedCase(["I0,I1,I2,FUSE_MUL_ADD3,O0", "O0,RELU,D"],
                                    [(2, 5, 7, 3), (2, 5, 7, 3), (1, 5, 1, 1)])
    c["fused_mul_add4"] = FusedCase(["I0,I1,I2,I3,FUSE_MUL_ADD4,O0", "O0,I0,MIN,D"],
                                    [(2, 5, 7, 3), (1,), (2, 5, 7, 3), (1, 5, 1, 1)])
    # (the reference's availability checks read operand:<i> for every step i and keep only the
    # verdict on the last step - BareMetal/FusedElemwiseKernel.cpp:270-290 and the GI twin - so a
    # chain for the BareMetal generator has no more steps than operands and ends in a mode only
    # that generator knows)
    c["fused_naive_unary"] = FusedCase(["I0,I1,I2,FUSE_MUL_ADD3,O0", "O0,SILU,O1", "O1,ABS,O2", "O2,LOG,D"],
                                       [(2, 3, 4, 5), (2, 3, 4, 5), (1, 3, 1, 1)], positive=(0, 1, 2))
    c["fused_naive_round"] = FusedCase(["I0,I1,TRUE_DIV,O0", "O0,ROUND,D"], [(2, 3, 4, 5), (1,)],
                                       positive=(1,))
    c["fused_naive_compare"] = FusedCase(["I0,I1,LT,O0", "I0,I2,LEQ,O1", "O0,O1,ADD,O2", "O2,I2,FUSE_ADD_TANH,D"],
                                         [(2, 3, 4, 5), (1, 3, 1, 1), (2, 3, 4, 5)])
    c["fused_naive_eq_floordiv"] = FusedCase(["I0,I1,EQ,O0", "O0,I0,ADD,O1", "O1,I1,FLOOR_DIV,D"],
                                             [(2, 3, 4, 5), (2, 3, 4, 5)], positive=(1,))
    c["resize_nearest_nchw_view"] = ResizeCase(A.FMT_NCHW, "NEAREST", 2, 3, 6, 5, 9, 11,
                                               src_strides=(400, 120, 20, 2))
    # --- f32 elementwise: the shapes of compiler/test/kernel/opr/generalIntrinsic/elementwise.cpp
    # :7-80 (every way two operands meet: same shape, scalar either side, [1,C,1,1] either side,
    # a trailing vector either side, a leading run, a kept last axis of extent 1; {2,100,3,96}
    # cut to {2,10,3,96}), then the NCHW44 channel vector, a general broadcast and the
    # FullyConnected bias [M,N] + [1,N]
    for mode in ("RELU", "SIGMOID", "EXP", "H_SWISH", "NEGATE"):
        c["ew_%s_4d" % mode] = ElemwiseCase(mode, [(1, 10, 12, 13)])
    c["ew_RELU_1"] = ElemwiseCase("RELU", [(1,)])
    pairs = [((1,), (1,)), ((1, 10), (1, 10)), ((1, 10), (1, 1)), ((2, 3, 4, 5), (2, 3, 4, 5)),
             ((2, 3, 4, 5), (1, 3, 1, 1)), ((1, 3, 1, 1), (2, 3, 4, 5)), ((13,), (3, 9, 13)),
             ((3, 9, 13), (13,)), ((1, 1, 1, 13), (2, 3, 4, 13)), ((2, 10, 3, 96), (1, 1, 1, 96)),
             ((3, 6, 9, 5), (3, 6, 9, 1)), ((5, 32, 1), (5, 32, 13)),
             ((2, 3, 4, 5, 4), (1, 3, 1, 1, 4)), ((1, 3, 1, 1, 4), (2, 3, 4, 5, 4)),
             ((2, 3, 4, 5), (1, 1, 4, 5)), ((2, 3, 4, 5), (2, 1, 4, 1)), ((5, 40), (1, 40))]
    for i, (s0, s1) in enumerate(pairs):
        c["ew_ADD_%d" % i] = ElemwiseCase("ADD", [s0, s1])
    others = ["SUB", "MUL", "FUSE_ADD_RELU", "MAX", "MIN"]
    for i, (s0, s1) in enumerate(pairs):  # every pairing under two more modes
        for j in (0, 1):
            mode = others[(2 * i + j) % len(others)]
            c["ew_%s_%d" % (mode, i)] = ElemwiseCase(mode, [s0, s1])
    for i, (s0, s1) in enumerate(pairs + [((2, 3, 4), (1,)), ((1,), (2, 3, 4))]):
        c["ew_TRUE_DIV_%d" % i] = ElemwiseCase("TRUE_DIV", [s0, s1], span=(3.0, 12.0))
    # --- f32 reduce: compiler/test/kernel/opr/generalIntrinsic/reduce.cpp:7-27 (every mode, every
    # axis of a 2-, 3- and 4-d tensor)
    for mode in ("SUM", "MEAN", "MAX", "MIN", "PRODUCT", "SUM_SQR"):
        for shape in ((2, 3), (3, 4, 5), (4, 5, 6, 7)):
            for axis in range(len(shape)):
                c["reduce_%s_%dd_a%d" % (mode, len(shape), axis)] = ReduceCase(mode, shape, axis)
    # --- later additions (appended: the seed of a case is its position in this dictionary)
    # f32 dense layers in NCHW44, depthwise 5x5 / 7x7, H_SWISH on a dense 5x5 layer
    c["conv44_f32_3x3_RELU"] = ConvCase(A.FMT_NCHW44, A.DENSE, 2, 8, 9, 7, 12, 3, 1, 1, A.RELU, dtype="f32")
    c["conv44_f32_1x1_IDENTITY"] = ConvCase(A.FMT_NCHW44, A.DENSE, 1, 12, 6, 5, 8, 1, 1, 0, A.IDENTITY, dtype="f32")
    c["dw44_5x5_s1_H_SWISH"] = ConvCase(
        A.FMT_NCHW44, A.GROUP, 2, 8, 9, 11, 8, 5, 1, 2, A.H_SWISH, scales=(0.02, 0.01, unsat(25)))
    c["dw44_5x5_s2_RELU"] = ConvCase(
        A.FMT_NCHW44, A.GROUP, 2, 8, 9, 11, 8, 5, 2, 2, A.RELU, scales=(0.02, 0.01, unsat(25)))
    c["dw44_7x7_s1_IDENTITY"] = ConvCase(
        A.FMT_NCHW44, A.GROUP, 1, 4, 10, 9, 4, 7, 1, 3, A.IDENTITY, scales=(0.02, 0.01, unsat(49)))
    c["conv44_5x5_H_SWISH"] = ConvCase(
        A.FMT_NCHW44, A.DENSE, 2, 8, 9, 7, 8, 5, 1, 2, A.H_SWISH, scales=(0.02, 0.01, unsat(200)))
    # f32 first layers (NCHW source, NCHW44 result: GeneralIntrinsic/ConvKernel/Fp32ConvNchwNchw44.cpp)
    # and f32 channel-wise layers in NCHW44 (Fp32ChannelWiseMk4.cpp: 3x3 and 5x5, stride 1 and 2)
    c["conv_hybrid_f32_3x3_s2_RELU"] = ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 2, 3, 11, 9, 8, 3, 2, 1, A.RELU, dtype="f32")
    c["conv_hybrid_f32_3x3_s1_H_SWISH"] = ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 1, 3, 9, 8, 12, 3, 1, 1, A.H_SWISH,
                                                   dtype="f32")
    c["conv_hybrid_f32_5x5_s2_IDENTITY"] = ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 2, 1, 12, 10, 4, 5, 2, 2, A.IDENTITY,
                                                    dtype="f32")
    c["conv_hybrid_f32_7x7_s2_RELU_nobias"] = ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 1, 3, 17, 15, 8, 7, 2, 3, A.RELU,
                                                       dtype="f32", bias=False)
    c["dw44_f32_3x3_s1_RELU"] = ConvCase(A.FMT_NCHW44, A.GROUP, 2, 8, 9, 7, 8, 3, 1, 1, A.RELU, dtype="f32")
    c["dw44_f32_3x3_s2_IDENTITY"] = ConvCase(A.FMT_NCHW44, A.GROUP, 2, 8, 9, 7, 8, 3, 2, 1, A.IDENTITY, dtype="f32")
    c["dw44_f32_5x5_s1_H_SWISH"] = ConvCase(A.FMT_NCHW44, A.GROUP, 1, 12, 10, 11, 12, 5, 1, 2, A.H_SWISH, dtype="f32")
    c["dw44_f32_5x5_s2_RELU_nobias"] = ConvCase(A.FMT_NCHW44, A.GROUP, 2, 4, 11, 13, 4, 5, 2, 2, A.RELU, dtype="f32",
                                                bias=False)
    return c
