"""CPU tests of the checker itself: the C restatement (oracle/oracle_port.c) against
(1) the committed fixtures produced by the reference's own generated kernels (tests/golden/),
(2) the same generated kernels run live where oracle/_ref has been built, on larger seeded cases,
(3) what the mathematics fixes independently of either (exact integer correlation via numpy,
    zero-weight and identity-weight closed forms)."""
import json
import os

import numpy as np
import pytest

import cases
from cases import ConvCase, MultiTypeCase, PoolCase, TypeCvtCase, MatMulCase
from golden_cases import golden_cases, unsat
from megcc_amd import abi
from oracle import port, ref

HERE = os.path.dirname(os.path.abspath(__file__))
GOLD = np.load(os.path.join(HERE, "golden", "golden.npz"))
with open(os.path.join(HERE, "golden", "symbols.json")) as f:
    SYMBOLS = json.load(f)
CASES = golden_cases()
F32_TOL = 1e-4  # max |a-b| / max(1, min(|a|,|b|)), the north star's fp32 bar


def golden_arrays(name):
    out = {}
    for key in GOLD.files:
        if key.startswith(name + "/"):
            out[key.split("/", 1)[1]] = GOLD[key]
    return out


def is_float_case(case):
    _, outs = case.specs(case.gen(0))
    return outs[0].type_enum == abi.FLOAT


@pytest.mark.parametrize("name", sorted(CASES))
def test_port_matches_golden(name):
    case = CASES[name]
    g = golden_arrays(name)
    arrays = {k: g.get(k) for k in case.gen(0).keys()}
    got = case.run_port(arrays)
    if got.dtype == np.float32:
        assert cases.max_rel_err(got, g["expect"]) <= F32_TOL
    else:
        np.testing.assert_array_equal(got, g["expect"])


@pytest.mark.parametrize("name", sorted(CASES))
def test_symbol_mirror(name):
    """our reading of the reference's symbol scheme against what its registry actually chose"""
    case = CASES[name]
    if isinstance(case, ConvCase) and case.dtype == "f32" and case.fmt == abi.FMT_NCHW_NCHW44:
        # the GI first-layer kernel: our reading of the name + its own suffix
        assert SYMBOLS[name] == "GI_%s_nchw_nchw44_oc%d_ic%d" % (case.symbol(), case.oc, case.ic)
    elif isinstance(case, ConvCase) and case.dtype == "f32" and case.sparse == abi.GROUP:
        assert SYMBOLS[name] == "GI_chanwise_" + case.symbol()
    elif isinstance(case, ConvCase) and case.dtype == "f32" and case.fmt == abi.FMT_NCHW44:
        # the registry's first choice for f32 NCHW44: Winograd F(2,3) for 3x3, the 1x1 kernel
        assert SYMBOLS[name].startswith(("GI_kernel_conv2d_3x3_NCHW44_DENSE", "GI_kernel_conv2d_conv1x1_NCHW44"))
    elif isinstance(case, ConvCase) and case.dtype == "f32":
        assert SYMBOLS[name].startswith("GI_kernel_conv2d_im2col_3x3_NCHW_DENSE")
    else:
        assert case.symbol() == SYMBOLS[name]


def test_golden_not_degenerate():
    """the fixtures must exercise rounding, not just the clamps"""
    for name in ("conv44_3x3_s1_IDENTITY", "conv44_1x1_RELU", "fc_q8_5x40x13", "dw44_3x3_s1_RELU"):
        e = GOLD[name + "/expect"]
        sat = np.mean((e == 127) | (e == -128))
        assert sat < 0.2, (name, sat)
        assert len(np.unique(e)) > 40, name
    e = GOLD["conv44_3x3_s1_overflow/expect"]
    assert (e == 127).all()


LIVE = [
    ConvCase(abi.FMT_NCHW44, abi.DENSE, 2, 64, 14, 14, 64, 3, 1, 1, abi.RELU, scales=(0.02, 0.01, unsat(576))),
    ConvCase(abi.FMT_NCHW44, abi.DENSE, 1, 32, 12, 13, 48, 3, 1, 1, abi.IDENTITY, scales=(0.02, 0.01, 0.05)),
    ConvCase(abi.FMT_NCHW44, abi.DENSE, 1, 32, 9, 9, 32, 3, 1, 1, abi.H_SWISH, scales=(0.02, 0.01, unsat(288))),
    ConvCase(abi.FMT_NCHW44, abi.DENSE, 1, 32, 9, 9, 32, 3, 1, 1, abi.SIGMOID, scales=(0.02, 0.01, unsat(288) * 40)),
    ConvCase(abi.FMT_NCHW44, abi.DENSE, 2, 64, 7, 7, 128, 1, 1, 0, abi.RELU, scales=(0.02, 0.01, unsat(64))),
    ConvCase(abi.FMT_NCHW, abi.DENSE, 16, 256, 1, 1, 100, 1, 1, 0, abi.IDENTITY, scales=(0.01, 0.01, unsat(256) / 2)),
    ConvCase(abi.FMT_NCHW44, abi.GROUP, 2, 32, 20, 18, 32, 3, 1, 1, abi.RELU, scales=(0.02, 0.01, unsat(9))),
    ConvCase(abi.FMT_NCHW44, abi.GROUP, 2, 32, 20, 18, 32, 3, 2, 1, abi.RELU, scales=(0.02, 0.01, unsat(9))),
    ConvCase(abi.FMT_NCHW_NCHW44, abi.DENSE, 1, 3, 32, 32, 32, 3, 2, 1, abi.RELU, scales=(0.02, 0.01, unsat(27))),
    PoolCase(abi.FMT_NCHW44, abi.POOL_MAX, 2, 16, 14, 14, 2, 2, 0),
    PoolCase(abi.FMT_NCHW44, abi.POOL_AVERAGE, 3, 64, 7, 7, 7, 7, 0),
    PoolCase(abi.FMT_NCHW, abi.POOL_AVERAGE, 3, 64, 7, 7, 7, 7, 0),
    MultiTypeCase(abi.Q_FUSE_ADD_RELU, (4, 32, 14, 14), (0.05, 0.01, 0.05)),
    MultiTypeCase(abi.Q_ADD, (4, 32, 14, 14), (0.031, 0.017, 0.023)),
    TypeCvtCase("f32", "qsi8", (5, 1001), dst_scale=0.0173),
    TypeCvtCase("qsi8", "qsi8", (5, 1001), src_scale=0.0173, dst_scale=0.0291),
]


@pytest.mark.skipif(not ref.available(), reason="oracle/_ref not built (needs /root/reference)")
@pytest.mark.parametrize("case", LIVE, ids=[repr(c) for c in LIVE])
def test_port_matches_reference_live(case):
    if not ref.has(case.symbol()):
        pytest.skip("symbol not in this _ref build")
    arrays = case.gen(seed=7)
    want = cases.run_ref(case, arrays)
    got = case.run_port(arrays)
    np.testing.assert_array_equal(got, want)


# ---- checks that do not involve the reference at all ----------------------------------------
@pytest.mark.parametrize("name", sorted(n for n in CASES if n.startswith("relayout_")))
def test_port_relayout_vs_numpy_views(name):
    """numpy's own strided views (as_strided + reshape) define the same copy"""
    case = CASES[name]
    arrays = case.gen(3)
    ins, outs = case.specs(arrays)
    s, o = ins[0], outs[0]
    src_view = cases.view_of(arrays["src"], s.shape, s.strides or cases.dense_strides(s.shape),
                             s.offset)
    want = cases.poisoned(o.storage, arrays["src"].dtype) if o.strides else \
        np.zeros(o.storage, arrays["src"].dtype)
    dst_view = cases.view_of(want, o.shape, o.strides or cases.dense_strides(o.shape), o.offset)
    dst_view[...] = np.ascontiguousarray(src_view).reshape(o.shape)
    np.testing.assert_array_equal(case.run_port(arrays), want)


def test_port_relayout_known_answers():
    """transpose, flip and NCHW -> NCHW4 written with numpy's own operators"""
    x = np.arange(2 * 8 * 3 * 5, dtype=np.int32).reshape(2, 8, 3, 5)
    out = np.zeros((2, 2, 3, 5, 4), np.int32)
    port.relayout(x, 0, (2, 2, 3, 5, 4), (120, 60, 5, 1, 15), out, 0, out.shape,
                  cases.dense_strides(out.shape))
    np.testing.assert_array_equal(out, x.reshape(2, 2, 4, 3, 5).transpose(0, 1, 3, 4, 2))
    m = np.arange(35, dtype=np.int8).reshape(5, 7)
    out = np.zeros((7, 5), np.int8)
    port.relayout(m, 0, (7, 5), (1, 7), out, 0, (7, 5), (5, 1))
    np.testing.assert_array_equal(out, m.T)
    out = np.zeros((5, 7), np.int8)
    port.relayout(m, 6, (5, 7), (7, -1), out, 0, (5, 7), (7, 1))
    np.testing.assert_array_equal(out, m[:, ::-1])


@pytest.mark.parametrize("name", sorted(n for n in CASES if n.startswith("concat_")))
def test_port_concat_vs_numpy(name):
    case = CASES[name]
    arrays = case.gen(3)
    want = np.concatenate([arrays["in%d" % i] for i in range(len(case.shapes))], case.axis)
    np.testing.assert_array_equal(case.run_port(arrays), want)


def _acc_numpy_nchw44_dense(src, flt, bias, pad, stride):
    """exact int64 correlation, written against the layout definition (not the port's loops)"""
    n, c4, ih, iw, _ = src.shape
    oc4 = flt.shape[0]
    x = src.transpose(0, 1, 4, 2, 3).reshape(n, c4 * 4, ih, iw).astype(np.int64)
    # flt[oc/4, ic/4, fh, fw, ic%4, oc%4] -> w[oc, ic, fh, fw]
    w = flt.transpose(0, 5, 1, 4, 2, 3).reshape(oc4 * 4, c4 * 4, flt.shape[2], flt.shape[3]).astype(np.int64)
    xp = np.pad(x, ((0, 0), (0, 0), (pad, pad), (pad, pad)))
    fh, fw = w.shape[2:]
    oh = (ih + 2 * pad - fh) // stride + 1
    ow = (iw + 2 * pad - fw) // stride + 1
    acc = np.zeros((n, oc4 * 4, oh, ow), np.int64)
    for a in range(fh):
        for b in range(fw):
            win = xp[:, :, a:a + stride * oh:stride, b:b + stride * ow:stride]
            acc += np.einsum("nchw,oc->nohw", win, w[:, :, a, b])
    acc += bias.reshape(1, -1, 1, 1)
    return acc


def _requant_numpy(acc, s0, s1, s2, relu):
    v = acc.astype(np.int32).astype(np.float32) * np.float32(s0) * np.float32(s1) / np.float32(s2)
    if relu:
        v = np.where(v > 0, v, np.float32(0))
    r = np.sign(v) * np.floor(np.abs(v) + np.float32(0.5))  # half away from zero
    # floor(|v|+0.5) in fp32 can differ from roundf for |v| just below .5: compare via float64
    r = np.sign(v) * np.floor(np.abs(v.astype(np.float64)) + 0.5)
    return np.clip(r, -128, 127).astype(np.int8)


@pytest.mark.parametrize("stride,relu", [(1, False), (1, True), (2, True)])
def test_port_conv_vs_numpy_closed_form(stride, relu):
    case = ConvCase(abi.FMT_NCHW44, abi.DENSE, 2, 16, 10, 9, 24, 3, stride, 1,
                    abi.RELU if relu else abi.IDENTITY, scales=(0.02, 0.01, unsat(144)))
    a = case.gen(3)
    acc = _acc_numpy_nchw44_dense(a["src"], a["flt"], a["bias"].reshape(-1), 1, stride)
    want = _requant_numpy(acc, *case.scales, relu)
    want44 = want.reshape(2, 6, 4, case.oh, case.ow).transpose(0, 1, 3, 4, 2)
    np.testing.assert_array_equal(case.run_port(a), want44)


def test_port_conv_zero_weight_gives_bias_only():
    case = ConvCase(abi.FMT_NCHW44, abi.DENSE, 1, 8, 5, 5, 8, 3, 1, 1, abi.IDENTITY,
                    scales=(0.5, 0.5, 0.25), bias_range=(-100, 100))
    a = case.gen(1)
    a["flt"][:] = 0
    got = case.run_port(a)
    want = np.clip(a["bias"].reshape(1, 2, 1, 1, 4), -128, 127).astype(np.int8)  # 0.5*0.5/0.25 = 1
    np.testing.assert_array_equal(got, np.broadcast_to(want, got.shape))


def test_port_fc_identity_weight():
    k = 16
    case = ConvCase(abi.FMT_NCHW, abi.DENSE, 7, k, 1, 1, k, 1, 1, 0, abi.IDENTITY,
                    scales=(1.0, 1.0, 1.0), bias_range=(0, 0))
    a = case.gen(2)
    a["flt"][:] = np.eye(k, dtype=np.int8).reshape(k, k, 1, 1)
    np.testing.assert_array_equal(case.run_port(a), a["src"])


def test_port_maxpool_vs_numpy():
    case = PoolCase(abi.FMT_NCHW, abi.POOL_MAX, 2, 3, 8, 6, 2, 2, 0)
    a = case.gen(5)
    want = a["src"].reshape(2, 3, 4, 2, 3, 2).max(axis=(3, 5))
    np.testing.assert_array_equal(case.run_port(a), want)


def test_port_matmul_vs_float64():
    case = MatMulCase(9, 33, 17)
    a = case.gen(4)
    want = a["a"].astype(np.float64) @ a["b"].astype(np.float64)
    assert cases.max_rel_err(case.run_port(a), want) <= 1e-5


def test_port_resize_closed_forms():
    """what the mathematics fixes for Resize: same size = copy; a constant image stays constant; a
    plane that is affine in (h, w) is reproduced exactly by bilinear weights wherever the
    half-pixel source coordinate lies inside the image (no edge clamping); NEAREST equals
    numpy indexing with floor(o * I / O) for integer ratios."""
    r = np.random.default_rng(5)
    x = r.uniform(-30, 30, (2, 3, 6, 5)).astype(np.float32)
    assert np.array_equal(port.resize(x, (6, 5), "LINEAR"), x)
    x4 = r.uniform(-30, 30, (1, 2, 6, 5, 4)).astype(np.float32)
    assert np.array_equal(port.resize(x4, (6, 5), "LINEAR", nchw44=True), x4)
    const = np.full((1, 2, 4, 7), 3.25, np.float32)
    # (dyadic weights at ratio 2: no rounding at all; any ratio: within rounding)
    assert np.array_equal(port.resize(const, (8, 14), "LINEAR"), np.full((1, 2, 8, 14), 3.25, np.float32))
    np.testing.assert_allclose(port.resize(const, (9, 3), "LINEAR"), 3.25, rtol=1e-6)
    # affine plane, exactly representable values: 2x upscale of f(h, w) = 8 h + w
    ih, iw = 8, 8
    hh, ww = np.meshgrid(np.arange(ih), np.arange(iw), indexing="ij")
    plane = (8.0 * hh + ww).astype(np.float32)[None, None]
    got = port.resize(plane, (16, 16), "LINEAR")[0, 0]
    oh = (np.arange(16) + 0.5) / 2 - 0.5
    want = 8.0 * oh[:, None] + oh[None, :]
    inside = (oh >= 0) & (oh <= ih - 1)
    assert np.array_equal(got[np.ix_(inside, inside)], want[np.ix_(inside, inside)].astype(np.float32))
    # edges clamp to the border rows / columns
    assert got[0, 5] == got[0, 5] and np.array_equal(got[0, inside], (8.0 * 0 + oh[inside]).astype(np.float32))
    # NCHW44 is the same function on interleaved channels
    y = r.uniform(-30, 30, (2, 8, 5, 6)).astype(np.float32)
    y44 = np.ascontiguousarray(y.reshape(2, 2, 4, 5, 6).transpose(0, 1, 3, 4, 2))
    a = port.resize(y, (7, 13), "LINEAR")
    b = port.resize(y44, (7, 13), "LINEAR", nchw44=True)
    assert np.array_equal(b.transpose(0, 1, 4, 2, 3).reshape(2, 8, 7, 13), a)
    # NEAREST, integer ratios up and down
    z = r.uniform(-30, 30, (1, 2, 6, 8)).astype(np.float32)
    assert np.array_equal(port.resize(z, (12, 24), "NEAREST"),
                          z[:, :, np.arange(12) // 2][:, :, :, np.arange(24) // 3])
    assert np.array_equal(port.resize(z, (3, 4), "NEAREST"), z[:, :, ::2, ::2])
    # strided source = the same result as on a dense copy of the view
    buf = r.uniform(-30, 30, 2 * 400 + 8).astype(np.float32)
    view = np.lib.stride_tricks.as_strided(buf, (2, 3, 6, 5), [4 * s for s in (400, 120, 20, 2)])
    assert np.array_equal(
        port.resize(buf, (9, 11), "NEAREST", src_strides=(400, 120, 20, 2), src_shape=(2, 3, 6, 5)),
        port.resize(np.ascontiguousarray(view), (9, 11), "NEAREST"))


def test_port_fused_elemwise_vs_numpy():
    """the chain interpreter against numpy written out by hand: operand kinds (same size, scalar,
    [1,C,1,1], [1,C,1,1,4]), reuse of an intermediate value, 3- and 4-operand steps"""
    from megcc_amd import abi
    r = np.random.default_rng(9)
    x = r.integers(-10, 10, (3, 10, 10, 5, 4), endpoint=True).astype(np.float32)
    b = r.integers(-10, 10, (1, 10, 1, 1, 4), endpoint=True).astype(np.float32)
    z = np.array([3.0], np.float32)
    prog = abi.parse_fused_modes(["I0,I1,ADD,O0", "O0,SIGMOID,O1", "O1,I2,MAX,O2", "O2,I2,TRUE_DIV,D"], 3)
    got = port.fused_elemwise(prog, [x, b, z], [0, 3, 1], x.shape)
    sig = np.float32(1) / (np.float32(1) + np.exp(-(x + b), dtype=np.float32))
    np.testing.assert_allclose(got, np.maximum(sig, z) / z, rtol=1e-6)
    y = r.integers(-10, 10, (4, 6, 9, 2), endpoint=True).astype(np.float32)
    c = r.integers(-10, 10, (1, 6, 1, 1), endpoint=True).astype(np.float32)
    prog = abi.parse_fused_modes(["I0,I1,ADD,O0", "I2,O0,MUL,O1", "O0,I3,SUB,D"], 4)
    got = port.fused_elemwise(prog, [c, y, np.array([2.0], np.float32), y], [2, 0, 1, 0], y.shape)
    assert np.array_equal(got, (c + y) - y)  # step 1's result is computed and not used
    prog = abi.parse_fused_modes(["I0,I1,I2,I1,FUSE_MUL_ADD4,O0", "O0,I0,LT,O1", "O1,O0,FLOOR_DIV,D"], 3)
    w = r.integers(1, 10, (4, 6, 9, 2), endpoint=True).astype(np.float32)
    got = port.fused_elemwise(prog, [y, w, c], [0, 0, 2], y.shape)
    t0 = y * w + c * w
    with np.errstate(divide="ignore", invalid="ignore"):
        want = np.floor((t0 < y).astype(np.float32) / t0)
    assert np.array_equal(got, want, equal_nan=True)


# ---- f32 elementwise and reduce: what numpy fixes without the reference --------------------------
EW_PAIRS = [((7, 40), (40,)), ((7, 40), (1, 40)), ((2, 3, 4, 5), (1, 3, 1, 1)), ((1, 3, 1, 1), (2, 3, 4, 5)),
            ((2, 3, 4, 5), (2, 1, 4, 1)), ((5, 32, 1), (5, 32, 13)), ((6,), (1,)), ((1,), (2, 3, 4)),
            ((2, 3, 4, 5, 4), (1, 3, 1, 1, 4)), ((9, 11), (9, 11))]


@pytest.mark.parametrize("shapes", EW_PAIRS, ids=lambda s: "%sx%s" % s)
def test_port_elemwise_binary_vs_numpy(shapes):
    """single IEEE operations under numpy's own broadcasting: results must be identical, bit for
    bit (a wrong operand order, a transposed broadcast or a dropped operand all show)"""
    from cases import ElemwiseCase
    r = np.random.default_rng(11)
    a = r.uniform(-4, 4, shapes[0]).astype(np.float32)
    b = r.uniform(0.5, 4, shapes[1]).astype(np.float32)
    f32 = np.float32
    want = {"ADD": a + b, "SUB": a - b, "MUL": a * b, "TRUE_DIV": a / b, "MAX": np.maximum(a, b),
            "MIN": np.minimum(a, b), "FUSE_ADD_RELU": np.maximum(a + b, f32(0))}
    for mode, w in want.items():
        got = ElemwiseCase(mode, list(shapes)).run_port({"a": a, "b": b})
        assert got.dtype == np.float32 and np.array_equal(got, w), mode
    # not commutative: the operands must not be swapped
    assert not np.array_equal(ElemwiseCase("SUB", list(shapes)).run_port({"a": a, "b": b}), b - a)


def test_port_elemwise_unary_vs_numpy():
    from cases import ElemwiseCase
    x = np.random.default_rng(12).uniform(-8, 8, (3, 5, 7)).astype(np.float32)
    x[0, 0, :4] = [0.0, -3.0, 3.0, -0.0]
    run = lambda m: ElemwiseCase(m, [x.shape]).run_port({"a": x, "b": None})
    assert np.array_equal(run("RELU"), np.maximum(x, np.float32(0)))
    assert np.array_equal(run("NEGATE"), -x)
    x64 = x.astype(np.float64)
    np.testing.assert_allclose(run("EXP"), np.exp(x64), rtol=3e-7)
    np.testing.assert_allclose(run("SIGMOID"), 1 / (1 + np.exp(-x64)), rtol=5e-7)
    np.testing.assert_allclose(run("H_SWISH"), x64 * np.clip(x64 + 3, 0, 6) / 6, rtol=5e-7, atol=1e-7)
    # H_SWISH is zero at and below -3 and the identity at and above 3
    hs = run("H_SWISH")
    assert hs[0, 0, 1] == 0 and hs[0, 0, 2] == 3.0


@pytest.mark.parametrize("shape,axis", [((2, 3), 0), ((2, 3), 1), ((3, 4, 5), 0), ((3, 4, 5), 1),
                                        ((3, 4, 5), 2), ((4, 5, 6, 7), 2), ((64, 1000), 1)])
def test_port_reduce_vs_numpy(shape, axis):
    """MAX / MIN are exact; the sums are the float32 running sum in ascending order along the
    axis (numpy's accumulate does exactly that), MEAN divides it once by the extent; fp64 numpy
    bounds all of them"""
    from cases import ReduceCase
    x = np.random.default_rng(13).uniform(-3, 3, shape).astype(np.float32)
    run = lambda m: ReduceCase(m, shape, axis).run_port({"src": x})
    keep = lambda v: np.expand_dims(v, axis)
    assert np.array_equal(run("MAX"), keep(x.max(axis)))
    assert np.array_equal(run("MIN"), keep(x.min(axis)))
    last = lambda acc: keep(np.take(acc, -1, axis=axis))
    seq = last(np.add.accumulate(x, axis=axis, dtype=np.float32))
    assert np.array_equal(run("SUM"), seq)
    assert np.array_equal(run("MEAN"), seq / np.float32(shape[axis]))
    assert np.array_equal(run("SUM_SQR"), last(np.add.accumulate(x * x, axis=axis, dtype=np.float32)))
    assert np.array_equal(run("PRODUCT"), last(np.multiply.accumulate(x, axis=axis, dtype=np.float32)))
    np.testing.assert_allclose(run("SUM"), keep(x.astype(np.float64).sum(axis)), rtol=1e-4, atol=1e-4)
    assert run("SUM").shape == tuple(1 if i == axis else d for i, d in enumerate(shape))


LIVE_F32 = None


def _live_f32():
    from cases import ElemwiseCase, ReduceCase
    return [ElemwiseCase("ADD", [(64, 4096), (1, 4096)]), ElemwiseCase("ADD", [(33, 1000), (1000,)]),
            ElemwiseCase("SUB", [(64, 1000), (64, 1)]), ElemwiseCase("TRUE_DIV", [(64, 1000), (64, 1)], span=(1.0, 9.0)),
            ElemwiseCase("MUL", [(4, 32, 14, 14), (1, 32, 1, 1)]), ElemwiseCase("EXP", [(64, 1000)], span=(-20.0, 0.0)),
            ElemwiseCase("SIGMOID", [(5, 1001)]), ElemwiseCase("H_SWISH", [(5, 1001)], span=(-6.0, 6.0)),
            ElemwiseCase("MAX", [(3, 1, 5, 1), (3, 4, 5, 6)]),
            ReduceCase("MAX", (64, 1000), 1), ReduceCase("SUM", (64, 1000), 1),
            ReduceCase("MEAN", (8, 1024, 49), 2), ReduceCase("MEAN", (6, 50, 33), 1),
            ReduceCase("MIN", (50, 7, 9), 0)]


@pytest.mark.skipif(not ref.available(), reason="oracle/_ref not built (needs /root/reference)")
@pytest.mark.parametrize("idx", range(14))
def test_port_f32_elemwise_reduce_match_reference_live(idx):
    """larger shapes through the reference's generated GI kernels (SIMD bodies + scalar tails;
    their exp is a polynomial, hence the tolerance)"""
    case = _live_f32()[idx]
    if not ref.has(case.symbol()):
        pytest.skip("symbol not in this _ref build")
    arrays = case.gen(seed=7)
    want = cases.run_ref(case, arrays)
    got = case.run_port(arrays)
    assert got.shape == want.shape
    tol = 1e-4 if type(case).__name__ == "ReduceCase" else 1e-5  # (SIMD partial sums: another order)
    assert cases.max_rel_err(got, want) <= tol, repr(case)
