"""The reference's own TinyNN runtime driving this library: oracle/_ref/ref_lite_run is MegCC's
runtime/src (parse.c, init.c, vm.c, vm/op.c, lite/network.c, ...) compiled from the reference tree
with megcc_amd/upstream/runtime_device_gfx950.patch applied, linked with the kernel tables that
the reference's KernelGen registry - with megcc_amd/upstream/kernelgen_arch_gfx950.patch applied -
exported for Arch::GFX950, and with libmegcc_gfx950.so. A caller that only knows the LITE C API
(host buffers in, host buffers out) loads a `.tiny` file and gets, bit for bit, what the model
runtime of this library computes for the same file, and what the CPU oracle computes."""
import os
import subprocess

import numpy as np
import pytest

import cases
import mobilenet
from cases import ConvCase, MultiTypeCase, PoolCase
from megcc_amd import abi, runtime, tiny

HERE = os.path.dirname(os.path.abspath(__file__))
REF_DIR = os.path.join(os.path.dirname(HERE), "oracle", "_ref")
RUNNER = os.path.join(REF_DIR, "ref_lite_run")
IDS = os.path.join(REF_DIR, "lite_kernel_ids.txt")

pytestmark = pytest.mark.skipif(
    not (os.path.exists(RUNNER) and os.path.exists(IDS)),
    reason="oracle/_ref/ref_lite_run is built by `make -C oracle ref` where the reference tree exists")


def kernel_table():
    table = {}
    with open(IDS) as f:
        for line in f:
            sym, k, i, w = line.split()
            table[sym] = (int(k), int(i), int(w))
    return table


def test_every_mobilenet_operator_has_a_kernel_in_the_exported_tables():
    table = kernel_table()
    assert len({ids for ids in table.values()}) == len(table)
    net = mobilenet.Net(1)
    for _, name, case, _ in net.steps:
        assert case.symbol() in table or name in ("quant", "dequant") or \
            any(s.endswith(case.symbol().split("kernel_", 1)[1]) for s in table), (name, case.symbol())


def run_lite(tmp_path, model_bytes, inputs, out_specs, forwards=1):
    """inputs: arrays in the model's input order; out_specs: [(shape, dtype)] in output order"""
    model_path = tmp_path / "model.tiny"
    model_path.write_bytes(model_bytes)
    in_paths, out_paths = [], []
    for i, a in enumerate(inputs):
        p = tmp_path / ("in_%d.bin" % i)
        np.ascontiguousarray(a).tofile(p)
        in_paths.append(str(p))
    for i in range(len(out_specs)):
        out_paths.append(str(tmp_path / ("out_%d.bin" % i)))
    r = subprocess.run([RUNNER, str(model_path), str(forwards)] + in_paths + ["--"] + out_paths,
                       capture_output=True, text=True, timeout=240)
    assert r.returncode == 0, "ref_lite_run failed (%d):\n%s\n%s" % (r.returncode, r.stdout[-2000:], r.stderr[-4000:])
    return [np.fromfile(p, dtype=dt).reshape(shape) for p, (shape, dt) in zip(out_paths, out_specs)]


def mobilenet_builder(batch):
    net = mobilenet.Net(batch)
    b = tiny.ModelBuilder("mobilenet_v1_int8", device=tiny.DEVICE_GFX950, alignment=256,
                          kernel_table=kernel_table())
    ids = {}
    real_tensor = b.tensor

    def named(name, shape, type_enum, scale=1.0):
        ids[name] = real_tensor(name, shape, type_enum, scale)
        return ids[name]

    b.tensor = named
    net.build_gpu(model=b)
    return net, b, ids


@pytest.mark.gpu
@pytest.mark.parametrize("batch,forwards", [(1, 1), (4, 3)])
def test_lite_forward_of_the_reference_runtime_equals_the_model_runtime(tmp_path, batch, forwards):
    net, b, ids = mobilenet_builder(batch)
    data = b.to_bytes()
    image = mobilenet.draw_input(batch, seed=40 + batch)
    # the reference's VM: LITE_load_model_from_path ... LITE_forward ... LITE_get_tensor_memory
    (lite_out,) = run_lite(tmp_path, data, [image], [((batch, 1000), np.float32)], forwards)
    # this library's model runtime on the very same file
    shapes = {ids["image"]: ((batch, 3, 224, 224), abi.FLOAT), ids["softmax"]: ((batch, 1000), abi.FLOAT)}
    runtime.set_option("nofusesoftmax", 1)  # the VM runs the five soft-max operators one by one
    try:
        model = runtime.Model.load(data, shapes)
    finally:
        runtime.set_option("nofusesoftmax", 0)
    model.set_input(ids["image"], image)
    model.forward()
    ours = model.get(ids["softmax"])
    model.close()
    assert np.array_equal(lite_out, ours), "LITE_forward differs from model_forward in %d of %d values" % (
        int((lite_out != ours).sum()), ours.size)
    want, _ = net.run_oracle(image)
    assert cases.max_rel_err(lite_out, want) <= 1e-4
    assert np.allclose(lite_out.sum(axis=1), 1.0, atol=1e-4)


@pytest.mark.gpu
def test_lite_forward_runs_layers_that_need_their_workspace(tmp_path):
    """FullyConnected with 64 rows and a long K under few output channels asks for K-slice partial
    sums: the file carries the size the kernel's _workspace function gives and an offset in the
    arena, the reference's init_model_memory points Opr.workspace there"""
    fc = ConvCase(abi.FMT_NCHW, abi.DENSE, 64, 16384, 1, 1, 256, 1, 1, 0, abi.IDENTITY,
                  scales=(0.01, 0.01, 0.02 * 0.01 * 5.4e3 * 128 / 70.0))
    table = dict(kernel_table())
    arrays = fc.gen(5)
    b = tiny.ModelBuilder("fc", device=tiny.DEVICE_GFX950, alignment=256, kernel_table=table)
    x = b.tensor("x", fc.src_shape(), abi.QINT8, fc.scales[0])
    b.mark_input(x)
    w = b.weight("w", arrays["flt"], abi.QINT8, fc.scales[1])
    bias = b.weight("b", arrays["bias"], abi.QINT32, float(np.float32(fc.scales[0]) * np.float32(fc.scales[1])))
    y = b.tensor("y", fc.dst_shape(), abi.QINT8, fc.scales[2])
    b.opr(fc.symbol(), [x, w, bias], [y])
    b.mark_output(y)
    d = b.to_dict()
    opr = [f for k, f in d["device_models"][0]["instructions"] if k == "Opr"][0]
    assert opr["workspace_size"] > 0 and d["device_models"][0]["tensor_memory"] >= opr["workspace_size"]
    (got,) = run_lite(tmp_path, tiny.write_model(d), [arrays["src"]], [(fc.dst_shape(), np.int8)])
    want = fc.run_port(arrays)
    assert np.array_equal(got, want)


@pytest.mark.gpu
def test_lite_forward_of_the_bandwidth_chain(tmp_path):
    """depthwise 3x3 -> max-pool 2x2 -> add + ReLU, two model inputs, three Opr instructions"""
    n, c, hw = 3, 32, 28
    dw = ConvCase(abi.FMT_NCHW44, abi.GROUP, n, c, hw, hw, c, 3, 1, 1, abi.RELU, scales=(0.02, 0.01, 0.02 * 0.01 * 5.4e3 * 3 / 35.0))
    pool = PoolCase(abi.FMT_NCHW44, abi.POOL_MAX, n, c, dw.oh, dw.ow, 2, 2, 0, scale=dw.scales[2])
    add = MultiTypeCase(abi.Q_FUSE_ADD_RELU, pool.dst_shape(), (dw.scales[2], 0.013, 0.9 * dw.scales[2]))
    arrays = dw.gen(9)
    other = np.random.default_rng(10).integers(-128, 128, pool.dst_shape()).astype(np.int8)
    b = tiny.ModelBuilder("chain", device=tiny.DEVICE_GFX950, alignment=256, kernel_table=kernel_table())
    x = b.tensor("x", dw.src_shape(), abi.QINT8, dw.scales[0])
    o = b.tensor("other", pool.dst_shape(), abi.QINT8, add.scales[1])
    b.mark_input(x)
    b.mark_input(o)
    w = b.weight("dw.w", arrays["flt"], abi.QINT8, dw.scales[1])
    bias = b.weight("dw.b", arrays["bias"], abi.QINT32, float(np.float32(dw.scales[0]) * np.float32(dw.scales[1])))
    t1 = b.tensor("dw", dw.dst_shape(), abi.QINT8, dw.scales[2])
    b.opr(dw.symbol(), [x, w, bias], [t1])
    t2 = b.tensor("pool", pool.dst_shape(), abi.QINT8, dw.scales[2])
    b.opr(pool.symbol(), [t1], [t2])
    t3 = b.tensor("out", pool.dst_shape(), abi.QINT8, add.scales[2])
    b.opr(add.symbol(), [t2, o], [t3])
    b.mark_output(t3)
    (got,) = run_lite(tmp_path, b.to_bytes(), [arrays["src"], other], [(pool.dst_shape(), np.int8)], forwards=2)
    want = add.run_port({"a": pool.run_port({"src": dw.run_port(arrays)}), "b": other})
    assert np.array_equal(got, want)
