"""Parity at the full sizes the benchmark configurations name, one test per configuration.

The reference's kernels treat batch images (rows of a FullyConnected) independently
(BareMetal/ConvKernel.cpp:305 is the outermost loop), so the oracle evaluated on a few images of
the batch is exact for those images: the GPU runs the whole configuration, the oracle a subset,
and the matching slices are compared - bit for bit for qsi8, within 1e-4 for f32. Each test also
records which kernel variant ran, so that the kernel a benchmark times is the one checked here."""
import numpy as np
import pytest

import cases
import mobilenet
from cases import ConvCase, ElemwiseCase, MatMulCase, MultiTypeCase, PoolCase
from golden_cases import unsat
from megcc_amd import abi, runtime
from oracle import port

pytestmark = pytest.mark.gpu
A = abi


def run_gpu(case, arrays):
    print("GPU case:", repr(case), flush=True)
    ins, outs = case.specs(arrays)
    got = runtime.run_symbol(case.symbol(), ins, outs)
    print("   kernel:", runtime.last_kernel(), flush=True)
    return got


def same_bytes(got, want, what):
    assert got.shape == want.shape and got.dtype == want.dtype, what
    bad = np.flatnonzero(got.reshape(-1) != want.reshape(-1))
    assert bad.size == 0, "%s: %d of %d differ, first at %d: got %d want %d" % (
        what, bad.size, got.size, bad[0], got.reshape(-1)[bad[0]], want.reshape(-1)[bad[0]])


def f32_close(got, want, what, tol=1e-4):
    """|a-b| / max(1, min(|a|,|b|)) <= tol (the reference's model-level metric,
    ci/compare_output_bin.py) AND the plain relative error wherever |want| >= 1e-3"""
    assert got.shape == want.shape, what
    err = cases.max_rel_err(got, want)
    assert err <= tol, "%s: max err %g" % (what, err)
    w = want.astype(np.float64)
    big = np.abs(w) >= 1e-3
    rel = np.abs(got.astype(np.float64)[big] - w[big]) / np.abs(w[big])
    print("   %s: max |a-b|/max(1,.) = %.3g, max relative error on |ref| >= 1e-3 = %.3g" % (
        what, err, rel.max() if rel.size else 0.0), flush=True)
    # (relative error of a sum of K products of uniform[-1,1] values: the condition number of the
    #  sum bounds it, not the kernel; 1e-3 leaves room for |ref| close to 1e-3)
    assert rel.size == 0 or np.median(rel) <= 1e-5, "%s: median relative error %g" % (what, np.median(rel))


# ---- configs[1]: qsi8 3x3 NCHW44 at N = 32 -----------------------------------------------------
CFG2 = [(c, hw, act, sc) for c in (64, 256) for hw in (56, 28)
        for act, sc in ((A.RELU, 0.05), (A.IDENTITY, 0.05), (A.IDENTITY, None))]


@pytest.mark.parametrize("c,hw,act,dst_scale", CFG2, ids=[
    "c%d_%dx%d_%s_%s" % (c, hw, hw, A.NONLINE_NAMES[act], "baseline_scales" if sc else "unsaturated")
    for c, hw, act, sc in CFG2])
def test_cfg2_conv3x3_n32(c, hw, act, dst_scale):
    """N = 32 (the benchmarked shape is c256 56x56 RELU with the mandated scales 0.02/0.01/0.05,
    where most outputs saturate; the unsaturated variant exercises the rounding)"""
    port.set_threads(16)
    scales = (0.02, 0.01, dst_scale if dst_scale else unsat(9 * c))
    case = ConvCase(A.FMT_NCHW44, A.DENSE, 32, c, hw, hw, c, 3, 1, 1, act, scales=scales)
    arrays = case.gen(seed=3)
    got = run_gpu(case, arrays)
    kernel = runtime.last_kernel()
    assert kernel.startswith("conv_mfma_i8_dma"), kernel
    if c == 256 and hw == 56:
        # the instantiation bench.py times: plane-major patch of 1024 slots, 128 oc x 512 px
        assert kernel.split("+")[0] == "conv_mfma_i8_dma:3,128,512,1024,1", kernel
    one = ConvCase(A.FMT_NCHW44, A.DENSE, 1, c, hw, hw, c, 3, 1, 1, act, scales=scales)
    for i in (0, 17, 31):
        want = one.run_port({"src": arrays["src"][i:i + 1], "flt": arrays["flt"], "bias": arrays["bias"]})
        same_bytes(got[i:i + 1], want, "%r image %d" % (case, i))
    if dst_scale is None:
        sat = np.mean((got == 127) | (got == -128))
        assert sat < 0.2 and len(np.unique(got)) > 100, "unsaturated variant saturates: %g" % sat


def test_cfg2_conv3x3_n1():
    """the four N = 1 shapes in full"""
    port.set_threads(16)
    for c in (64, 256):
        for hw in (56, 28):
            for act, sc in ((A.RELU, 0.05), (A.IDENTITY, unsat(9 * c))):
                case = ConvCase(A.FMT_NCHW44, A.DENSE, 1, c, hw, hw, c, 3, 1, 1, act, scales=(0.02, 0.01, sc))
                arrays = case.gen(seed=4)
                same_bytes(run_gpu(case, arrays), case.run_port(arrays), repr(case))


# ---- configs[2]: MatMul / FullyConnected ---------------------------------------------------------
FC_SCALES = [("baseline_scales", 0.1), ("unsaturated", None)]


def fc_rows(m, k, n, scale_name, dst_scale, rows):
    port.set_threads(16)
    sc = (0.01, 0.01, dst_scale if dst_scale else unsat(k) / 2)
    case = ConvCase(A.FMT_NCHW, A.DENSE, m, k, 1, 1, n, 1, 1, 0, A.IDENTITY, scales=sc)
    arrays = case.gen(seed=5)
    got = run_gpu(case, arrays)
    sub = ConvCase(A.FMT_NCHW, A.DENSE, len(rows), k, 1, 1, n, 1, 1, 0, A.IDENTITY, scales=sc)
    want = sub.run_port({"src": np.ascontiguousarray(arrays["src"][rows]), "flt": arrays["flt"],
                         "bias": arrays["bias"]})
    same_bytes(np.ascontiguousarray(got[rows]), want, repr(case))
    if dst_scale is None:
        assert np.mean((got == 127) | (got == -128)) < 0.2
    return runtime.last_kernel()


@pytest.mark.parametrize("scale_name,dst_scale", FC_SCALES, ids=[s for s, _ in FC_SCALES])
def test_cfg3_fc_q8_1x1024x1000(scale_name, dst_scale):
    assert fc_rows(1, 1024, 1000, scale_name, dst_scale, [0]) == "fc_gevm_q8"


@pytest.mark.parametrize("scale_name,dst_scale", FC_SCALES, ids=[s for s, _ in FC_SCALES])
def test_cfg3_fc_q8_64x4096x4096(scale_name, dst_scale):
    assert fc_rows(64, 4096, 4096, scale_name, dst_scale, list(range(64))) == "fc_one:32,4"


@pytest.mark.parametrize("scale_name,dst_scale", FC_SCALES, ids=[s for s, _ in FC_SCALES])
def test_cfg3_fc_q8_4096x4096x4096(scale_name, dst_scale):
    rows = sorted(set(range(64)) | set(np.random.default_rng(8).integers(64, 4096, 64).tolist()) | {4095})
    kernel = fc_rows(4096, 4096, 4096, scale_name, dst_scale, rows)
    assert kernel.split("+")[0] == "conv_mfma_i8_dma_xo:1,256,256,256,4", kernel  # the 256 x 256 FullyConnected tile, XCD-aware tile order


def matmul_rows(m, k, n, rows):
    """GPU against the fp64 product (the truth) at 1e-4, and against the oracle's float32 running
    sum (k ascending per output, the order of the reference's gevm / 4x12 kernels). At K = 4096
    that running sum is itself further than 1e-4 from the fp64 result on some outputs; the bound
    for the GPU-oracle distance is then the oracle's own distance from fp64 (the GPU's tiled sums
    are the more accurate of the two), never less than 1e-4."""
    case = MatMulCase(m, k, n)
    arrays = case.gen(seed=6)
    got = run_gpu(case, arrays)
    got_rows = np.ascontiguousarray(got[rows])
    want64 = arrays["a"][rows].astype(np.float64) @ arrays["b"].astype(np.float64)
    f32_close(got_rows, want64.astype(np.float32), repr(case) + " vs fp64")
    sub = port.matmul_f32(np.ascontiguousarray(arrays["a"][rows]), arrays["b"])
    oracle_own = cases.max_rel_err(sub, want64)
    print("   oracle (float32 running sum) vs fp64: %.3g" % oracle_own, flush=True)
    f32_close(got_rows, sub, repr(case) + " vs the port", tol=max(1e-4, 1.5 * oracle_own))
    return got, arrays


def test_cfg3_matmul_f32_1x1024x1000_with_bias():
    got, _ = matmul_rows(1, 1024, 1000, [0])
    assert runtime.last_kernel() == "gevm_f32"
    add = ElemwiseCase("ADD", [(1, 1000), (1000,)])
    bias = cases.rng(9).uniform(-1, 1, (1000,)).astype(np.float32)
    out = run_gpu(add, {"a": got, "b": bias})
    assert np.array_equal(out, got + bias)


def test_cfg3_matmul_f32_64x4096x4096_with_bias():
    got, _ = matmul_rows(64, 4096, 4096, list(range(64)))
    add = ElemwiseCase("ADD", [(64, 4096), (4096,)])
    bias = cases.rng(9).uniform(-1, 1, (4096,)).astype(np.float32)
    out = run_gpu(add, {"a": got, "b": bias})
    assert np.array_equal(out, got + bias)  # one IEEE addition per element: exact


def test_cfg3_matmul_f32_4096x4096x4096_with_bias():
    rows = sorted(set(range(64)) | set(np.random.default_rng(8).integers(64, 4096, 64).tolist()) | {4095})
    got, _ = matmul_rows(4096, 4096, 4096, rows)
    add = ElemwiseCase("ADD", [(4096, 4096), (4096,)])
    bias = cases.rng(9).uniform(-1, 1, (4096,)).astype(np.float32)
    out = run_gpu(add, {"a": got, "b": bias})
    assert np.array_equal(out, got + bias)


# ---- configs[0]: f32 conv at its real size -------------------------------------------------------
def test_cfg1_conv_f32():
    case = ConvCase(A.FMT_NCHW, A.DENSE, 1, 32, 56, 56, 32, 3, 1, 1, A.RELU, dtype="f32")
    arrays = case.gen(seed=0)
    got = run_gpu(case, arrays)
    f32_close(got, case.run_port(arrays), repr(case))
    # fp64 referee: correlation written with numpy on the padded image
    x = np.pad(arrays["src"].astype(np.float64), ((0, 0), (0, 0), (1, 1), (1, 1)))
    w = arrays["flt"].astype(np.float64)
    acc = np.zeros((1, 32, 56, 56))
    for a in range(3):
        for b in range(3):
            acc += np.einsum("nchw,oc->nohw", x[:, :, a:a + 56, b:b + 56], w[:, :, a, b])
    acc += arrays["bias"].astype(np.float64)
    f32_close(got, np.maximum(acc, 0).astype(np.float32), repr(case) + " vs fp64")


# ---- configs[3]: the bandwidth-bound chain at N = 64 ---------------------------------------------
CFG4 = [(32, 112, 1), (32, 112, 2), (512, 14, 1), (512, 14, 2), (512, 112, 1), (512, 112, 2), (32, 14, 1), (32, 14, 2)]


@pytest.mark.parametrize("c,hw,stride", CFG4, ids=["c%d_%dx%d_s%d" % (c, hw, hw, st) for c, hw, st in CFG4])
def test_cfg4_chain_n64(c, hw, stride):
    """depthwise 3x3 -> max-pool 2x2 s2 -> add + ReLU with requantisation, N = 64, each stage fed
    with the GPU's output of the stage before; the oracle checks images 0, 31 and 63 of every
    stage (and the whole tensor for the pooling and the add, which are cheap)"""
    port.set_threads(16)
    n = 64
    dw = ConvCase(A.FMT_NCHW44, A.GROUP, n, c, hw, hw, c, 3, stride, 1, A.RELU, scales=(0.02, 0.01, 0.05))
    arrays = dw.gen(seed=7)
    y = run_gpu(dw, arrays)
    assert runtime.last_kernel().startswith("dwconv44")
    one = ConvCase(A.FMT_NCHW44, A.GROUP, 1, c, hw, hw, c, 3, stride, 1, A.RELU, scales=(0.02, 0.01, 0.05))
    for i in (0, 31, 63):
        want = one.run_port({"src": arrays["src"][i:i + 1], "flt": arrays["flt"], "bias": arrays["bias"]})
        same_bytes(y[i:i + 1], want, "%r image %d" % (dw, i))
    # the mandated scales saturate most outputs of a 3x3 window; the unsaturated twin rounds
    dwu = ConvCase(A.FMT_NCHW44, A.GROUP, n, c, hw, hw, c, 3, stride, 1, A.RELU, scales=(0.02, 0.01, unsat(9)))
    yu = run_gpu(dwu, arrays)
    oneu = ConvCase(A.FMT_NCHW44, A.GROUP, 1, c, hw, hw, c, 3, stride, 1, A.RELU, scales=(0.02, 0.01, unsat(9)))
    for i in (0, 63):
        want = oneu.run_port({"src": arrays["src"][i:i + 1], "flt": arrays["flt"], "bias": arrays["bias"]})
        same_bytes(yu[i:i + 1], want, "%r image %d" % (dwu, i))
    pool = PoolCase(A.FMT_NCHW44, A.POOL_MAX, n, c, dw.oh, dw.ow, 2, 2, 0, scale=0.05)
    z = run_gpu(pool, {"src": yu})
    same_bytes(z, pool.run_port({"src": yu}), repr(pool))
    add = MultiTypeCase(A.Q_FUSE_ADD_RELU, z.shape, (0.05, 0.01, 0.05))
    other = cases.rng(8).integers(-128, 128, z.shape).astype(np.int8)
    out = run_gpu(add, {"a": z, "b": other})
    same_bytes(out, add.run_port({"a": z, "b": other}), repr(add))


# ---- configs[4]: MobileNetV1-int8 end to end at batch 1, 64, 256 ---------------------------------
@pytest.mark.parametrize("batch", [1, 64, 256])
def test_cfg5_mobilenet(batch):
    """every layer of the batch-B forward, on the first, middle and last image, against the
    oracle's forward of just those images (image i of a batch does not depend on the others)"""
    picks = sorted({0, batch // 2, batch - 1})
    net = mobilenet.Net(batch)
    image = mobilenet.draw_input(batch, seed=5)
    model, ids = net.build_gpu(keep_all=True)
    model.set_input(ids["image"], image)
    model.forward()
    small = mobilenet.Net(len(picks))
    want, trace = small.run_oracle(np.ascontiguousarray(image[picks]), keep=True)
    for name, tid in ids.items():
        if name in ("image", "softmax", "dequant"):
            continue
        got = model.get(tid)[picks]
        exp = trace[name].reshape(got.shape)
        bad = int((got != exp).sum())
        assert bad == 0, "batch %d, %s: %d of %d elements differ" % (batch, name, bad, got.size)
    got = model.get(ids["softmax"])
    assert cases.max_rel_err(got[picks], want) <= 1e-4
    assert np.allclose(got.sum(axis=1), 1.0, atol=1e-4)
    assert want.max() < 0.999
    if batch >= 64:
        # the images must not collapse to one answer: their logits differ in most classes (with
        # random weights the bias picks the arg-max class, so that one may well coincide)
        fc = model.get(ids["fc"]).reshape(batch, 1000)
        assert np.mean(fc[0] != fc[-1]) > 0.5 and len(np.unique(fc)) > 50
    # second and third forward: the HIP-graph replay must give the same bytes
    first = model.get(ids["pw13"]).copy()
    for _ in range(2):
        model.forward()
        assert np.array_equal(model.get(ids["pw13"]), first)
    model.close()
