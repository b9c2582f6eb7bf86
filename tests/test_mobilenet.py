"""End-to-end MobileNetV1-int8 through the model runtime (static memory plan on one HBM arena)
against the CPU oracle evaluated layer by layer."""
import numpy as np
import pytest

import cases
import mobilenet
from megcc_amd import abi, runtime


def test_layer_table_matches_the_standard_topology():
    layers = mobilenet.conv_layers(1)
    assert len(layers) == 1 + 26 + 1
    assert mobilenet.macs_per_image() == 568740352  # 568.74 MMAC per image
    weights = mobilenet.draw_weights(0)
    assert sum(w[0].size for w in weights.values()) == 4209088  # int8 weight bytes


def test_scales_cover_every_layer():
    scales = mobilenet.load_scales()
    for name, _ in mobilenet.conv_layers(1):
        assert scales[name]["filter"] > 0 and scales[name]["dst"] > 0


@pytest.mark.gpu
def test_every_layer_is_bit_exact_batch2():
    net = mobilenet.Net(2)
    image = mobilenet.draw_input(2, seed=5)
    want, trace = net.run_oracle(image, keep=True)
    model, ids = net.build_gpu(keep_all=True)
    model.set_input(ids["image"], image)
    model.forward()
    for name, tid in ids.items():
        if name in ("image", "softmax", "dequant"):
            continue
        got = model.get(tid)
        exp = trace[name].reshape(got.shape)
        bad = int((got != exp).sum())
        assert bad == 0, "%s: %d of %d elements differ" % (name, bad, got.size)
    got = model.get(ids["softmax"])
    assert cases.max_rel_err(got, want) <= 1e-4
    assert np.allclose(got.sum(axis=1), 1.0, atol=1e-4)
    # the test images must not collapse to a constant prediction
    # (with random weights the bias picks the arg-max class; the logits of the two images differ)
    fc = trace["fc"].reshape(2, 1000)
    assert np.mean(fc[0] != fc[1]) > 0.5 and len(np.unique(fc)) > 50 and want.max() < 0.999
    model.close()


@pytest.mark.gpu
def test_memory_plan_reuses_the_arena_and_keeps_results():
    net = mobilenet.Net(3)
    image = mobilenet.draw_input(3, seed=9)
    want, _ = net.run_oracle(image)
    # (with consecutive forwards overlapping, the runtime's plan also gives the last operators' tensors
    #  bytes of their own - tests/test_pipeline.py; here the plan of the operators as they are)
    runtime.set_option("nopipeline", 1)
    try:
        model, ids = net.build_gpu()
    finally:
        runtime.set_option("nopipeline", 0)
    total = sum(c.n * c.oc * c.oh * c.ow for k, _, c, _ in net.steps if k == "conv")
    assert model.arena_bytes < total / 3, "tensors with disjoint lifetimes must share memory"
    # the arena is the reference allocator's plan for this model's lifetimes (stored answer for
    # batch 1 and 64 in golden/memplan.json; here the same planner on batch 3)
    # (... plus the one rule the runtime's own plan adds: see Lifetimes)
    lt = mobilenet.Lifetimes(keep_pointwise_sources=True)
    net.build_gpu(model=lt)
    tids, begin, end, size = lt.requests()
    off, arena, _ = runtime.plan_memory(begin, end, size, 256)
    assert model.arena_bytes == arena
    ptrs = [runtime.lib().megcc_gfx950_model_tensor_ptr(model.h, t) for t in tids]
    lowest = min(ptrs)
    assert [p - lowest for p in ptrs] == (off - off.min()).tolist()
    for _ in range(2):  # a second forward must not depend on leftovers of the first
        model.set_input(ids["image"], image)
        model.forward()
        got = model.get(ids["softmax"])
        assert cases.max_rel_err(got, want) <= 1e-4
    model.close()


@pytest.mark.gpu
def test_graph_replays_equal_eager_forwards():
    """The model runtime captures its operator sequence into a HIP graph on the fourth forward, replays
    it on the fifth and sixth, ninth and tenth (plain launches again in between) and then keeps
    whichever of eager launches and replays it measured faster. Every forward, with new inputs, host copies and synchronisations in between, must give
    what an eager forward gives (bit for bit: same kernels, same order)."""
    net = mobilenet.Net(2)
    eager, ids = net.build_gpu(keep_all=True)
    graph, _ = net.build_gpu(keep_all=True)
    names = ["conv0", "pw1", "pw13", "fc", "softmax"]
    for it in range(13):
        image = mobilenet.draw_input(2, seed=20 + it)
        runtime.set_option("no_graph", 1)
        try:
            eager.set_input(ids["image"], image)
            eager.forward()
        finally:
            runtime.set_option("no_graph", 0)
        want = {k: eager.get(ids[k]).copy() for k in names}
        graph.set_input(ids["image"], image)
        graph.forward()  # it 0-2: eager, 3: capture + first launch, 4-5: replays, 6-7: eager, 8-9: replays, then the faster way
        for k in names:
            np.testing.assert_array_equal(graph.get(ids[k]), want[k], err_msg="%s, forward %d" % (k, it))
    eager.close()
    graph.close()


@pytest.mark.gpu
def test_softmax_chain_runs_as_one_kernel_and_gives_the_same_result():
    """forward() replaces Reduce MAX -> SUB -> EXP -> Reduce SUM -> TRUE_DIV (and the typecvt in
    front) by one kernel when nothing else reads the intermediates; with every layer's result kept
    as an output the typecvt stays an operator of its own, with the option off all of them do. Same
    probabilities either way, on eager forwards and on graph replays."""
    net = mobilenet.Net(3)
    image = mobilenet.draw_input(3, seed=33)
    want, _ = net.run_oracle(image)
    fused, ids = net.build_gpu()
    runtime.set_option("nofusesoftmax", 1)
    try:
        plain, _ = net.build_gpu()
    finally:
        runtime.set_option("nofusesoftmax", 0)
    kept, kids = net.build_gpu(keep_all=True)
    results = []
    for model, mids, last in ((fused, ids, "softmax_rows:1"), (plain, ids, "elemwise_f32_bcast"),
                              (kept, kids, "softmax_rows:4")):
        model.set_input(mids["image"], image)
        for it in range(3):  # eager, capture, replay
            model.forward()
            out = model.get(mids["softmax"])
            assert cases.max_rel_err(out, want) <= 1e-4
            if it == 0:
                assert runtime.last_kernel().startswith(last), runtime.last_kernel()
        results.append(out.copy())
        assert model.nr_opr == 36
    assert cases.max_rel_err(results[0], results[1]) <= 1e-6
    np.testing.assert_array_equal(results[0], results[2])
    for m in (fused, plain, kept):
        m.close()
