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
