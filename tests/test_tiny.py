"""`.tiny` model files: writer (megcc_amd/tiny.py), reader (megcc_gfx950_tiny_describe, host code)
and loader (megcc_gfx950_model_load, GPU).

The referee for the file format is the reference's own generated FlatBuffers reader
(runtime/src/cheader/model_reader.h - the accessors runtime/src/parse.c uses), compiled into
oracle/_ref/ref_tiny_dump: golden/small.tiny.txt is what it prints for golden/small.tiny, and where
the reference tree is at hand it is also run on a freshly written MobileNetV1 file."""
import os

import numpy as np
import pytest

import cases
import mobilenet
import tiny_cases
from megcc_amd import abi, runtime, tiny
from oracle import ref

HERE = os.path.dirname(os.path.abspath(__file__))
SMALL = os.path.join(HERE, "golden", "small.tiny")


def small_bytes():
    with open(SMALL, "rb") as f:
        return f.read()


def test_reader_sees_what_the_reference_reader_saw():
    with open(SMALL + ".txt") as f:
        want = f.read()
    assert runtime.tiny_describe(small_bytes()) == want


def test_writer_is_deterministic_and_matches_the_stored_file():
    assert tiny.write_model(tiny_cases.small_model()) == small_bytes()


def test_defaults_left_out_of_the_file_are_applied():
    text = runtime.tiny_describe(small_bytes())
    line = [l for l in text.splitlines() if l.startswith("inst 0 Opr")][0]
    # the writer drops fields equal to their schema default: init_id, workspace_id, deduce_id = -1
    assert "init_id=-1 kernel_id=0 workspace_id=-1 deduce_id=-1" in line
    assert "weight 2 name=w.f16 dtype=0 scale=1 " in text  # no DTypeParam table at all


@pytest.mark.skipif(not ref.tiny_dump_available(), reason="oracle/_ref not built (needs the reference tree)")
def test_mobilenet_file_reads_the_same_with_the_reference_reader(tmp_path):
    net = mobilenet.Net(1)
    b = tiny.ModelBuilder("mobilenet_v1_int8")
    net.build_gpu(model=b)
    data = b.to_bytes()
    path = tmp_path / "mobilenet.tiny"
    path.write_bytes(data)
    mine = runtime.tiny_describe(data)
    assert mine == ref.tiny_dump(str(path))
    assert mine.count("\ninst ") == 37  # 36 kernels + the view in front of the FullyConnected


def test_truncated_files_are_rejected_not_read_past_the_end():
    data = small_bytes()
    for n in list(range(0, 64)) + list(range(64, len(data), 7)):
        with pytest.raises(runtime.MegccError):
            runtime.tiny_describe(data[:n])


def test_corrupted_files_never_crash_the_reader():
    data = bytearray(small_bytes())
    rng = np.random.default_rng(11)
    rejected = 0
    for _ in range(600):
        bad = bytearray(data)
        for _ in range(int(rng.integers(1, 4))):
            bad[int(rng.integers(0, len(bad)))] = int(rng.integers(0, 256))
        try:
            runtime.tiny_describe(bytes(bad))
        except runtime.MegccError:
            rejected += 1
    assert rejected > 0


# ---- loader (GPU) ------------------------------------------------------------------------------

def mobilenet_file(batch, device=tiny.DEVICE_BARE_METAL):
    net = mobilenet.Net(batch)
    b = tiny.ModelBuilder("mobilenet_v1_int8", device=device, alignment=256)
    ids = {}
    real_tensor = b.tensor

    def named(name, shape, type_enum, scale=1.0):
        ids[name] = real_tensor(name, shape, type_enum, scale)
        return ids[name]

    b.tensor = named
    net.build_gpu(model=b)
    return net, b, ids


@pytest.mark.gpu
@pytest.mark.parametrize("device", [tiny.DEVICE_BARE_METAL, tiny.DEVICE_GFX950])
def test_loaded_mobilenet_equals_the_model_built_in_memory(device):
    batch = 2
    net, b, ids = mobilenet_file(batch, device)
    image = mobilenet.draw_input(batch, seed=4)
    want, _ = net.run_oracle(image)
    direct, direct_ids = net.build_gpu()
    direct.set_input(direct_ids["image"], image)
    direct.forward()
    ref_out = direct.get(direct_ids["softmax"])

    shapes = {ids["image"]: ((batch, 3, 224, 224), abi.FLOAT),
              ids["softmax"]: ((batch, 1000), abi.FLOAT)}
    model = runtime.Model.load(b.to_bytes(), shapes)
    assert model.arena_bytes == b.to_dict()["device_models"][0]["tensor_memory"]
    assert model.nr_opr == 36
    for _ in range(3):  # eager, captured, replayed
        model.set_input(ids["image"], image)
        model.forward()
        got = model.get(ids["softmax"])
        assert np.array_equal(got, ref_out)
    assert cases.max_rel_err(got, want) <= 1e-4
    model.close()
    direct.close()


@pytest.mark.gpu
def test_loader_refuses_what_it_cannot_run():
    d = tiny_cases.small_model()  # dynamic tensor, DevMemAlloc, no kernel for half the symbols
    with pytest.raises(runtime.MegccError, match="dynamic"):
        runtime.Model.load(tiny.write_model(d))
    dm = d["device_models"][0]
    dm["tensors"] = dm["tensors"][:4]
    with pytest.raises(runtime.MegccError, match="instruction 3 has type 2"):
        runtime.Model.load(tiny.write_model(d))
    dm["instructions"] = [i for i in dm["instructions"] if i[0] in ("Opr", "MemForward")][:3]
    dm["tensors"][2]["offset"] = 4500  # 200 bytes at 4500 do not fit a 4608 byte arena
    with pytest.raises(runtime.MegccError, match="arena"):
        runtime.Model.load(tiny.write_model(d))
    d["device_models"] = [d["device_models"][1]]  # ARM64 only
    with pytest.raises(runtime.MegccError, match="none for gfx950 or BARE_METAL"):
        runtime.Model.load(tiny.write_model(d))
    with pytest.raises(runtime.MegccError, match="model_load"):
        runtime.Model.load(small_bytes()[:100])


# ---- strided views (SUBTENSOR / DIMSHUFFLE MemForward) + Relayout + Concat ----------------------
def test_view_file_carries_strides_and_byte_offsets():
    b = tiny.ModelBuilder("views")
    net = tiny_cases.ViewNet()
    ids = net.build(b)
    text = runtime.tiny_describe(b.to_bytes())
    lines = text.splitlines()
    view = [l for l in lines if "name=image.as_nchw4" in l][0]
    assert "dims=[2,2,6,6,4]" in view and "stride=[288,144,6,1,36]" in view
    tail = [l for l in lines if "name=cat.tail" in l][0]
    assert "stride=[144,36,12,4,1]" in tail
    fwd = [l for l in lines if " MemForward " in l]
    assert len(fwd) == 2 and "offset=0" in fwd[0] and "offset=72" in fwd[1]
    assert ids["out"] == 7


@pytest.mark.skipif(not ref.tiny_dump_available(), reason="oracle/_ref not built (needs the reference tree)")
def test_view_file_reads_the_same_with_the_reference_reader(tmp_path):
    b = tiny.ModelBuilder("views")
    tiny_cases.ViewNet().build(b)
    path = tmp_path / "views.tiny"
    path.write_bytes(b.to_bytes())
    assert runtime.tiny_describe(b.to_bytes()) == ref.tiny_dump(str(path))


@pytest.mark.gpu
@pytest.mark.parametrize("how", ["built", "loaded"])
def test_views_relayout_and_concat_inside_a_model(how):
    net = tiny_cases.ViewNet()
    if how == "built":
        model = runtime.Model()
        ids = net.build(model)
    else:
        b = tiny.ModelBuilder("views")
        ids = net.build(b)
        half = (net.N, net.C // 4, net.H // 2, net.W // 2, 4)
        both = (net.N, net.C // 2, net.H // 2, net.W // 2, 4)
        model = runtime.Model.load(b.to_bytes(), {
            ids["image"]: ((net.N, net.C, net.H, net.W), abi.QINT8),
            ids["cat"]: (both, abi.QINT8), ids["out"]: (half, abi.QINT8)})
    assert model.nr_opr == 5
    for seed in (1, 2, 3):  # eager, captured, replayed
        image = net.draw_input(seed)
        cat, out = net.run_oracle(image)
        model.set_input(ids["image"], image)
        model.forward()
        assert np.array_equal(model.get(ids["cat"]), cat)
        assert np.array_equal(model.get(ids["out"]), out)
    model.close()


@pytest.mark.gpu
def test_views_that_leave_their_tensor_are_refused():
    m = runtime.Model()
    x = m.tensor("x", (4, 6), abi.QINT8, 0.05)
    m.view("ok", x, (6, 4), (1, 6))
    m.view("ok.reversed", x, (4, 6), (6, -1), offset=5)
    with pytest.raises(runtime.MegccError, match="leaves"):
        m.view("long", x, (4, 7), (6, 1))
    with pytest.raises(runtime.MegccError, match="leaves"):
        m.view("before", x, (4, 6), (6, -1), offset=4)
    m.close()
    b = tiny.ModelBuilder("bad")
    x = b.tensor("x", (4, 6), abi.QINT8, 0.05)
    b.mark_input(x)
    v = b.view("long", x, (4, 7), (6, 1))
    y = b.tensor("y", (4, 7), abi.QINT8, 0.05)
    b.opr("kernel_relayout_qsi8", [v], [y])
    b.mark_output(y)
    with pytest.raises(runtime.MegccError, match="views bytes 0..25 of tensor 0"):
        runtime.Model.load(b.to_bytes())
    d = b.to_dict()
    d["device_models"][0]["tensors"][2]["stride"] = [1, 4]  # an owning tensor must be dense
    d["device_models"][0]["tensors"][1]["dims"] = [4, 6]
    with pytest.raises(runtime.MegccError, match="not dense"):
        runtime.Model.load(tiny.write_model(d))


@pytest.mark.gpu
def test_dense_relayout_is_a_copy_that_replays_in_the_graph():
    """a Relayout between two dense tensors is a device-to-device copy node of the captured graph:
    every replay must move the current input"""
    m = runtime.Model()
    x = m.tensor("x", (3, 5, 7), abi.QINT8, 0.05)
    m.mark_input(x)
    y = m.tensor("y", (3, 5, 7), abi.QINT8, 0.05)
    m.opr("kernel_relayout_qsi8", [x], [y])
    z = m.tensor("z", (3, 5, 7), abi.QINT8, 0.05)
    m.opr("kernel_elementwise_multitype_QRELU_qsi8qsi8", [y], [z])
    m.mark_output(z)
    m.finalize()
    r = np.random.default_rng(3)
    for _ in range(4):  # eager, captured, replayed twice
        a = r.integers(-128, 128, (3, 5, 7)).astype(np.int8)
        m.set_input(x, a)
        m.forward()
        assert np.array_equal(m.get(z), np.maximum(a, 0))
    m.close()


@pytest.mark.gpu
def test_model_with_resize_and_a_fused_chain_replays():
    """an up-sampling neck in one model: Resize x2 (by symbol), then a fused chain given as a
    descriptor (its symbol does not determine it): SiLU(up) * scale[c] + skip. Every forward -
    eager, captured, replayed - must use the current input."""
    from oracle import port
    m = runtime.Model()
    x = m.tensor("x", (2, 6, 9, 11), abi.FLOAT, 1.0)
    skip = m.tensor("skip", (2, 6, 18, 22), abi.FLOAT, 1.0)
    m.mark_input(x)
    m.mark_input(skip)
    scale = np.linspace(0.5, 1.5, 6, dtype=np.float32).reshape(1, 6, 1, 1)
    w = m.weight("scale", scale, abi.FLOAT, 1.0)
    up = m.tensor("up", (2, 6, 18, 22), abi.FLOAT, 1.0)
    m.opr("GI_kernel_resize_linear_NCHW_LINEAR_f32", [x], [up])
    out = m.tensor("out", (2, 6, 18, 22), abi.FLOAT, 1.0)
    prog = abi.parse_fused_modes(["I0,SILU,O0", "O0,I1,I2,FUSE_MUL_ADD3,D"], 3)
    desc = abi.KernelDesc()
    desc.kind = abi.KERN_FUSED_ELEMWISE
    desc.attr.fused = abi.fused_attr(prog, 3)
    m.opr_desc(desc, "silu_scale_skip", [up, w, skip], [out])
    m.mark_output(out)
    m.finalize()
    r = np.random.default_rng(11)
    for _ in range(4):
        a = r.uniform(-4, 4, (2, 6, 9, 11)).astype(np.float32)
        s = r.uniform(-4, 4, (2, 6, 18, 22)).astype(np.float32)
        m.set_input(x, a)
        m.set_input(skip, s)
        m.forward()
        want = port.fused_elemwise(prog, [port.resize(a, (18, 22), "LINEAR"), scale, s], [0, 2, 0],
                                   (2, 6, 18, 22))
        assert cases.max_rel_err(m.get(out), want) <= 1e-4
    m.close()
