"""megcc_gfx950_pw_dw: a pointwise 1x1 convolution and the channel-wise 3x3 convolution of its result
in one kernel, against the oracle's two convolutions run one after the other, bit for bit; and the
model runtime's use of it."""
import ctypes as C

import numpy as np
import pytest

import cases
from cases import ConvCase
from megcc_amd import abi, runtime
from megcc_amd import abi as A

pytestmark = pytest.mark.gpu

TIES = (0.02, 0.01)        # source and filter scale whose product over the output scale has exact ties
GENERIC = (0.0213, 0.0097)  # ... and without: IDENTITY / RELU requantise by the proven multiply-add

PAIRS = [
    # (n, ic, oc, h, w, stride of the 3x3, pointwise act, channel-wise act, pw bias, dw bias, scales)
    # the pairs of a MobileNetV1 at 224 x 224 from 28 x 28 down, at a small batch ...
    (2, 128, 256, 28, 28, 1, A.RELU, A.RELU, True, True, GENERIC),
    (2, 256, 256, 28, 28, 2, A.RELU, A.RELU, True, True, TIES),
    (3, 256, 512, 14, 14, 1, A.RELU, A.RELU, True, True, GENERIC),
    (2, 512, 512, 14, 14, 1, A.RELU, A.RELU, True, True, TIES),
    (3, 512, 512, 14, 14, 2, A.RELU, A.RELU, True, True, GENERIC),
    (2, 512, 1024, 7, 7, 1, A.RELU, A.RELU, True, True, GENERIC),
    # ... and at the batches of the benchmark (14 x 14: 64 channels per workgroup, 7 x 7: 128)
    (64, 512, 512, 14, 14, 1, A.RELU, A.RELU, True, True, GENERIC),
    (32, 512, 1024, 7, 7, 1, A.RELU, A.IDENTITY, True, True, TIES),
    # rows of 4, 5, 13, 31 pixels, one row, more rows than pixels a row, IDENTITY on either side, no bias
    (2, 128, 64, 9, 5, 1, A.IDENTITY, A.RELU, False, True, GENERIC),
    (1, 128, 128, 6, 13, 2, A.RELU, A.IDENTITY, True, False, TIES),
    (2, 256, 64, 3, 31, 1, A.IDENTITY, A.IDENTITY, False, False, GENERIC),
    (3, 128, 192, 5, 4, 2, A.RELU, A.RELU, True, True, GENERIC),
    (2, 128, 64, 1, 8, 1, A.RELU, A.RELU, True, True, TIES),
    (1, 128, 64, 33, 7, 2, A.RELU, A.RELU, True, True, GENERIC),
    (5, 256, 320, 8, 16, 1, A.RELU, A.RELU, True, True, TIES),
    (5, 512, 128, 7, 7, 2, A.RELU, A.IDENTITY, True, True, GENERIC),
    (3, 256, 64, 4, 6, 1, A.IDENTITY, A.RELU, True, True, TIES),
    (1, 512, 1024, 7, 7, 1, A.RELU, A.RELU, True, True, GENERIC),
    # small batches run 32 channels per workgroup, batches that fill the chip 64: the latter with every
    # K, both strides, and an image of few tiles
    (64, 128, 256, 14, 14, 2, A.RELU, A.RELU, True, True, TIES),
    (32, 256, 512, 14, 14, 1, A.RELU, A.IDENTITY, True, True, GENERIC),
    (128, 128, 192, 5, 4, 2, A.IDENTITY, A.RELU, True, True, GENERIC),
]


def pair_cases(n, ic, oc, h, w, stride, act0, act1, bias0, bias1, scales):
    mid = 0.0371 if scales is GENERIC else 0.05
    pw = ConvCase(A.FMT_NCHW44, A.DENSE, n, ic, h, w, oc, 1, 1, 0, act0, scales=scales + (mid,), bias=bias0)
    # (filter values of the 3x3 small enough that its output uses the whole int8 range without saturating everywhere)
    dw = ConvCase(A.FMT_NCHW44, A.GROUP, n, oc, h, w, oc, 3, stride, 1, act1,
                  scales=(mid, 0.0131 if scales is GENERIC else 0.01, 0.0689 if scales is GENERIC else 0.05),
                  bias=bias1, flt_range=(-40, 40))
    return pw, dw


def ident(cfg):
    return "n%d_c%d-%d_%dx%d_s%d_%s_%s%s%s_%s" % (
        cfg[0], cfg[1], cfg[2], cfg[3], cfg[4], cfg[5], A.NONLINE_NAMES[cfg[6]], A.NONLINE_NAMES[cfg[7]],
        "" if cfg[8] else "_nopwbias", "" if cfg[9] else "_nodwbias", "ties" if cfg[10] is TIES else "generic")


def fused_call(pw, dw, a0, a1):
    """-> (status, result or None, `supported` answer) of the pair through megcc_gfx950_call"""
    L = runtime.lib()
    # the pointwise operator's own init protocol packs its filter
    ins0, outs0 = pw.specs(a0)
    op0 = runtime.PreparedOp(runtime.parse_symbol(pw.symbol()), ins0, outs0)
    assert op0.n_processed == 1
    ins1, outs1 = dw.specs(a1)
    bufs = [runtime.DeviceBuffer.from_array(s.array) for s in ins1[1:]]
    tin = list(op0.in_tensors) + [
        abi.make_tensor(b.ptr, s.shape, s.type_enum, s.scale, s.name) for b, s in zip(bufs, ins1[1:])]
    out = runtime.DeviceBuffer(int(np.prod(dw.dst_shape())))
    out.fill(cases.POISON)
    tout = [abi.make_tensor(out.ptr, dw.dst_shape(), abi.QINT8, dw.scales[2], b"dst")]
    desc = abi.KernelDesc()
    desc.kind = abi.KERN_PW_DW
    desc.attr.pw_dw.pw = pw.attr()
    desc.attr.pw_dw.dw = dw.attr()
    desc.attr.pw_dw.mid_scale = pw.scales[2]
    L.megcc_gfx950_pw_dw_supported.argtypes = [
        C.POINTER(abi.PwDwAttr), C.POINTER(C.POINTER(abi.Tensor)), C.c_int, C.POINTER(C.POINTER(abi.Tensor)), C.c_int]
    ok = L.megcc_gfx950_pw_dw_supported(
        C.byref(desc.attr.pw_dw), abi.tensor_array(tin), len(tin), abi.tensor_array(tout), 1)
    st = L.megcc_gfx950_call(C.byref(desc), abi.tensor_array(tin), len(tin), abi.tensor_array(tout), 1, None, None)
    got = None
    if st == abi.SUCCESS:
        runtime.wait()
        got = out.to_array(dw.dst_shape(), np.int8)
    for b in bufs + [out]:
        b.free()
    return st, got, ok


def oracle_pair(pw, dw, a0, a1):
    mid = pw.run_port(a0)
    return mid, dw.run_port({"src": mid, "flt": a1["flt"], "bias": a1["bias"]})


@pytest.mark.parametrize("cfg", PAIRS, ids=[ident(c) for c in PAIRS])
def test_pointwise_and_depthwise_in_one_kernel_equal_the_two_layers(cfg):
    pw, dw = pair_cases(*cfg)
    print("GPU case:", repr(pw), repr(dw), flush=True)
    a0, a1 = pw.gen(31), dw.gen(32)
    mid, want = oracle_pair(pw, dw, a0, a1)
    # the data must exercise both layers: the tensor in between and the result use most of their range
    assert len(np.unique(mid)) > (100 if cfg[6] == A.RELU else 200), len(np.unique(mid))
    assert len(np.unique(want)) > (60 if cfg[7] == A.RELU else 120), len(np.unique(want))
    st, got, ok = fused_call(pw, dw, a0, a1)
    assert ok == 1 and st == abi.SUCCESS, runtime.lib().megcc_gfx950_last_error().decode()
    kernel = runtime.last_kernel()
    assert kernel.startswith("conv_pw_dw:"), kernel
    assert kernel.endswith("+affine") == (cfg[10] is GENERIC), kernel
    bad = np.flatnonzero(got.reshape(-1) != want.reshape(-1))
    assert bad.size == 0, "%r: %d of %d differ, first at %d: got %d want %d" % (
        cfg, bad.size, got.size, bad[0], got.reshape(-1)[bad[0]], want.reshape(-1)[bad[0]])


@pytest.mark.parametrize("cfg,why", [
    ((2, 128, 64, 8, 32, 1, A.RELU, A.RELU, True, True, GENERIC), "rows of 32 pixels"),
    ((2, 64, 64, 8, 8, 1, A.RELU, A.RELU, True, True, GENERIC), "64 input channels"),
    ((2, 128, 32, 8, 8, 1, A.RELU, A.RELU, True, True, GENERIC), "32 output channels"),
    ((2, 128, 64, 8, 8, 1, A.H_SWISH, A.RELU, True, True, GENERIC), "H_SWISH"),
    ((2, 128, 64, 8, 8, 1, A.RELU, A.SIGMOID, True, True, GENERIC), "SIGMOID"),
    ((1, 128, 64, 65, 8, 1, A.RELU, A.RELU, True, True, GENERIC), "65 rows"),
], ids=lambda v: v.replace(" ", "_") if isinstance(v, str) else "")
def test_what_the_entry_point_refuses(cfg, why):
    pw, dw = pair_cases(*cfg)
    st, got, ok = fused_call(pw, dw, pw.gen(1), dw.gen(2))
    assert ok == 0 and st == abi.ERROR_INVALID_LAYOUT and got is None, why


def _pair_model(cfg, fused, second_reader=False):
    pw, dw = pair_cases(*cfg)
    a0, a1 = pw.gen(31), dw.gen(32)
    # (left alone the runtime times both forms and keeps the faster one: the two switches pin it)
    runtime.set_option("nofusepwdw", 0 if fused else 1)
    runtime.set_option("fusepwdw", 1 if fused else 0)
    try:
        m = runtime.Model()
        x = m.tensor("x", pw.src_shape(), abi.QINT8, pw.scales[0])
        m.mark_input(x)
        ins = [x, m.weight("pw.w", a0["flt"], abi.QINT8, pw.scales[1])]
        if pw.bias:
            ins.append(m.weight("pw.b", a0["bias"], abi.QINT32, float(np.float32(pw.scales[0]) * np.float32(pw.scales[1]))))
        t1 = m.tensor("mid", pw.dst_shape(), abi.QINT8, pw.scales[2])
        m.opr(pw.symbol(), ins, [t1])
        ins = [t1, m.weight("dw.w", a1["flt"], abi.QINT8, dw.scales[1])]
        if dw.bias:
            ins.append(m.weight("dw.b", a1["bias"], abi.QINT32, float(np.float32(dw.scales[0]) * np.float32(dw.scales[1]))))
        t2 = m.tensor("out", dw.dst_shape(), abi.QINT8, dw.scales[2])
        m.opr(dw.symbol(), ins, [t2])
        m.mark_output(t2)
        if second_reader:
            m.mark_output(t1)
        m.finalize()
    finally:
        runtime.set_option("nofusepwdw", 0)
        runtime.set_option("fusepwdw", 0)
    m.set_input(x, a0["src"])
    outs = []
    for _ in range(3):  # eager, captured, replayed
        m.forward()
        runtime.wait()
        outs.append(m.get(t2).copy())
    mid = m.get(t1).copy() if second_reader else None
    return outs, m.nr_kernel, oracle_pair(pw, dw, a0, a1), mid


@pytest.mark.parametrize("cfg", [PAIRS[2], PAIRS[4], PAIRS[5], PAIRS[9]], ids=[ident(c) for c in (PAIRS[2], PAIRS[4], PAIRS[5], PAIRS[9])])
def test_model_runtime_runs_the_pair_as_one_kernel(cfg):
    fused, nk, (_, want), _ = _pair_model(cfg, True)
    assert nk == 1, nk
    plain, nk, _, _ = _pair_model(cfg, False)
    assert nk == 2, nk
    for o in fused + plain:
        assert np.array_equal(o, want), cfg


def test_large_image_at_a_large_batch():
    """64 planes of 60 x 31 pixels and 512 x 64 filter bytes do not fit the LDS: 32 channels per
    workgroup although the batch would fill the chip at 64. Against the two kernels (which the other
    tests hold against the oracle) - the oracle would take a minute here."""
    cfg = (16, 512, 1024, 60, 31, 1, A.RELU, A.RELU, True, True, GENERIC)
    pw, dw = pair_cases(*cfg)
    a0, a1 = pw.gen(31), dw.gen(32)
    outs = []
    for fused in (True, False):
        runtime.set_option("nofusepwdw", 0 if fused else 1)
        runtime.set_option("fusepwdw", 1 if fused else 0)
        try:
            m = runtime.Model()
            x = m.tensor("x", pw.src_shape(), abi.QINT8, pw.scales[0])
            m.mark_input(x)
            bias_scale = lambda c: float(np.float32(c.scales[0]) * np.float32(c.scales[1]))
            t1 = m.tensor("mid", pw.dst_shape(), abi.QINT8, pw.scales[2])
            m.opr(pw.symbol(), [x, m.weight("pw.w", a0["flt"], abi.QINT8, pw.scales[1]),
                                m.weight("pw.b", a0["bias"], abi.QINT32, bias_scale(pw))], [t1])
            t2 = m.tensor("out", dw.dst_shape(), abi.QINT8, dw.scales[2])
            m.opr(dw.symbol(), [t1, m.weight("dw.w", a1["flt"], abi.QINT8, dw.scales[1]),
                                m.weight("dw.b", a1["bias"], abi.QINT32, bias_scale(dw))], [t2])
            m.mark_output(t2)
            m.finalize()
        finally:
            runtime.set_option("nofusepwdw", 0)
            runtime.set_option("fusepwdw", 0)
        assert m.nr_kernel == (1 if fused else 2)
        m.set_input(x, a0["src"])
        m.forward()
        runtime.wait()
        outs.append(m.get(t2).copy())
        m.close()
    assert len(np.unique(outs[0])) > 100 and np.array_equal(outs[0], outs[1])


def test_model_runtime_keeps_the_pair_apart_when_the_tensor_between_is_read_elsewhere():
    outs, nk, (mid_want, want), mid = _pair_model(PAIRS[2], True, second_reader=True)
    assert nk == 2, nk
    assert np.array_equal(mid, mid_want)
    for o in outs:
        assert np.array_equal(o, want)


def test_model_runtime_left_alone_keeps_whichever_form_it_measures_faster():
    """no switch: one kernel or two, and the same bytes either way"""
    pw, dw = pair_cases(*PAIRS[2])
    a0, a1 = pw.gen(31), dw.gen(32)
    m = runtime.Model()
    x0 = m.tensor("x0", pw.src_shape(), abi.QINT8, 0.03)
    m.mark_input(x0)
    # (the pair's source is an arena tensor, like inside a network)
    pre = cases.MultiTypeCase(A.Q_RELU, pw.src_shape(), (0.03, 0.01, pw.scales[0]))
    x = m.tensor("x", pw.src_shape(), abi.QINT8, pw.scales[0])
    m.opr(pre.symbol(), [x0], [x])
    bias_scale = lambda c: float(np.float32(c.scales[0]) * np.float32(c.scales[1]))
    t1 = m.tensor("mid", pw.dst_shape(), abi.QINT8, pw.scales[2])
    m.opr(pw.symbol(), [x, m.weight("pw.w", a0["flt"], abi.QINT8, pw.scales[1]),
                        m.weight("pw.b", a0["bias"], abi.QINT32, bias_scale(pw))], [t1])
    t2 = m.tensor("out", dw.dst_shape(), abi.QINT8, dw.scales[2])
    m.opr(dw.symbol(), [t1, m.weight("dw.w", a1["flt"], abi.QINT8, dw.scales[1]),
                        m.weight("dw.b", a1["bias"], abi.QINT32, bias_scale(dw))], [t2])
    m.mark_output(t2)
    m.finalize()
    assert m.nr_kernel in (2, 3), m.nr_kernel
    src0 = np.random.default_rng(5).integers(-128, 128, pw.src_shape()).astype(np.int8)
    m.set_input(x0, src0)
    m.forward()
    runtime.wait()
    a0["src"] = pre.run_port({"a": src0, "b": None})
    _, want = oracle_pair(pw, dw, a0, a1)
    assert np.array_equal(m.get(t2), want)


# A memory plan made for the two operators gives the depthwise result the bytes of the pointwise
# layer's source (dead after the pointwise layer). The one kernel reads that source while other
# workgroups already write the result, so under such a plan the pair must stay two kernels.
def _planned_pair(out_offset):
    cfg = (3, 256, 128, 9, 12, 1, A.RELU, A.RELU, True, True, GENERIC)
    pw, dw = pair_cases(*cfg)
    a0, a1 = pw.gen(41), dw.gen(42)
    x0 = np.random.default_rng(43).integers(-128, 128, pw.src_shape()).astype(np.int8)
    pre = cases.MultiTypeCase(A.Q_RELU, pw.src_shape(), (0.03, 0.01, pw.scales[0]))
    bias_scale = lambda c: float(np.float32(c.scales[0]) * np.float32(c.scales[1]))
    runtime.set_option("fusepwdw", 1)  # (no timing: the one kernel wherever it may run)
    try:
        m = runtime.Model()
        t_in = m.tensor("x0", pw.src_shape(), abi.QINT8, 0.03)
        m.mark_input(t_in)
        t_x = m.tensor("x", pw.src_shape(), abi.QINT8, pw.scales[0])  # an arena tensor that dies at the pointwise layer
        m.opr(pre.symbol(), [t_in], [t_x])
        w0 = m.weight("pw.w", a0["flt"], abi.QINT8, pw.scales[1])
        b0 = m.weight("pw.b", a0["bias"], abi.QINT32, bias_scale(pw))
        t1 = m.tensor("mid", pw.dst_shape(), abi.QINT8, pw.scales[2])
        m.opr(pw.symbol(), [t_x, w0, b0], [t1])
        w1 = m.weight("dw.w", a1["flt"], abi.QINT8, dw.scales[1])
        b1 = m.weight("dw.b", a1["bias"], abi.QINT32, bias_scale(dw))
        t2 = m.tensor("out", dw.dst_shape(), abi.QINT8, dw.scales[2])
        m.opr(dw.symbol(), [t1, w1, b1], [t2])
        m.mark_output(t2)
        up = lambda v: (v + 255) // 256 * 256
        nx, nmid, nout = (int(np.prod(s)) for s in (pw.src_shape(), pw.dst_shape(), dw.dst_shape()))
        offs = [0] * (t2 + 1)
        offs[t_x], offs[t1] = 0, up(nx)
        offs[t2] = out_offset if out_offset is not None else offs[t1] + up(nmid)
        m.set_plan(offs, offs[t1] + up(nmid) + up(nout))
        m.finalize()
    finally:
        runtime.set_option("fusepwdw", 0)
    m.set_input(t_in, x0)
    outs = []
    for _ in range(3):
        m.forward()
        runtime.wait()
        outs.append(m.get(t2).copy())
    nk = m.nr_kernel
    m.close()
    a0["src"] = pre.run_port({"a": x0, "b": None})
    return outs, nk, oracle_pair(pw, dw, a0, a1)[1]


@pytest.mark.parametrize("out_offset,kernels", [(None, 2), (0, 3), (256, 3), (41472, 3)],
                         ids=["apart", "result_on_the_source", "result_256_bytes_into_the_source", "result_over_the_source_tail"])
def test_pair_is_one_kernel_only_when_its_result_shares_no_byte_with_its_source(out_offset, kernels):
    outs, nk, want = _planned_pair(out_offset)
    assert nk == kernels
    for o in outs:
        assert np.array_equal(o, want)


@pytest.mark.parametrize("w", range(4, 32))
def test_every_row_width(w):
    """the planes' pitch is the power of two above the width and a pixel group's window reaches one
    dword past either end of a row: every width the entry point takes, both strides, odd heights"""
    for stride, h in ((1, 3 + w % 4), (2, 2 + w % 5)):
        cfg = (2, 128, 64, h, w, stride, A.RELU, A.IDENTITY, True, True, GENERIC if w & 1 else TIES)
        pw, dw = pair_cases(*cfg)
        a0, a1 = pw.gen(100 + w), dw.gen(200 + w)
        _, want = oracle_pair(pw, dw, a0, a1)
        st, got, ok = fused_call(pw, dw, a0, a1)
        assert ok == 1 and st == abi.SUCCESS, runtime.lib().megcc_gfx950_last_error().decode()
        assert np.array_equal(got, want), cfg
