"""Consecutive forwards overlap: with plain launches the model runtime runs the last, small operators
of a forward on a second stream, so that the next forward's first operators need not wait for them.
The results must be those of forwards run strictly one after the other: under the runtime's own memory
plan (which gives what those operators touch bytes of its own) and under a plan that does not (the
reference planner's, where their tensors share bytes with early layers' and the next forward has to
wait for them)."""
import numpy as np
import pytest

import cases
import mobilenet
from megcc_amd import abi, runtime

pytestmark = pytest.mark.gpu

BATCH = 32  # (kernels must average 6 us or more for the runtime to use two streams)


class PlannedModel(runtime.Model):
    """runtime.Model that installs the reference planner's offsets for the operators' own lifetimes
    (no operator chains, no overlap: what a compiled model file carries) before it finalizes"""

    def __init__(self, net):
        super().__init__()
        lt = mobilenet.Lifetimes()
        net.build_gpu(model=lt)
        tids, begin, end, size = lt.requests()
        off, arena, _ = runtime.plan_memory(begin, end, size, 256)
        self.offsets = [0] * len(lt.sizes)
        for t, o in zip(tids, off):
            self.offsets[t] = int(o)
        self.arena = int(arena)

    def finalize(self):
        self.set_plan(self.offsets, self.arena)
        super().finalize()


def build(net, planned, keep_all=False, **options):
    for k, v in options.items():
        runtime.set_option(k, v)
    try:
        return net.build_gpu(keep_all=keep_all, model=PlannedModel(net) if planned else None)
    finally:
        for k in options:
            runtime.set_option(k, 0)


@pytest.mark.parametrize("planned", [False, True], ids=["own_plan", "reference_plan"])
def test_overlapped_forwards_equal_forwards_run_one_after_the_other(planned):
    net = mobilenet.Net(BATCH)
    images = [mobilenet.draw_input(BATCH, seed=s) for s in (1, 2, 3, 4, 5)]
    # (no_graph: plain launches from the first forward on, no measuring phase)
    pipe, ids = build(net, planned, no_graph=1)
    serial, _ = build(net, planned, no_graph=1, nopipeline=1)
    assert pipe.nr_tail_kernel >= 2 and serial.nr_tail_kernel == 0
    assert pipe.nr_kernel - pipe.nr_tail_kernel >= 4
    if not planned:
        assert pipe.arena_bytes > serial.arena_bytes  # the tail's tensors have bytes of their own
    else:
        assert pipe.arena_bytes == serial.arena_bytes
    want = []
    for img in images:
        serial.set_input(ids["image"], img)
        serial.forward()
        want.append(serial.get(ids["softmax"]).copy())
    assert not np.array_equal(want[0], want[1])
    # forward, copy of its result and the next input enqueued without the host waiting for anything
    outs = [np.zeros((BATCH, 1000), np.float32) for _ in images]
    for img, out in zip(images, outs):
        pipe.set_input(ids["image"], img)
        pipe.forward()
        pipe.get_async(ids["softmax"], out)
    runtime.wait()
    for k, (o, w) in enumerate(zip(outs, want)):
        np.testing.assert_array_equal(o, w, err_msg="forward %d" % k)
    # forwards with nothing read in between, then the blocking read; and a forward read at once
    for _ in range(3):
        for img in images:
            pipe.set_input(ids["image"], img)
            pipe.forward()
    np.testing.assert_array_equal(pipe.get(ids["softmax"]), want[-1])
    pipe.set_input(ids["image"], images[0])
    pipe.forward()
    np.testing.assert_array_equal(pipe.get(ids["softmax"]), want[0])
    # the serial results themselves against the oracle (first input)
    ref, _ = mobilenet.Net(2).run_oracle(images[0][:2])  # (same weights: they do not depend on the batch)
    assert cases.max_rel_err(want[0][:2], ref) <= 1e-4
    pipe.close()
    serial.close()


def test_asynchronous_read_of_a_tensor_the_first_stream_writes():
    """every layer's result kept as an output: a layer far from the end is read between two forwards
    (that copy goes to the library stream, between this forward's operators and the next one's), the
    last layer's behind the second stream"""
    net = mobilenet.Net(BATCH)
    images = [mobilenet.draw_input(BATCH, seed=s) for s in (7, 8)]
    pipe, ids = build(net, False, keep_all=True, no_graph=1)
    serial, _ = build(net, False, keep_all=True, no_graph=1, nopipeline=1)
    assert pipe.nr_tail_kernel >= 2
    mid = np.zeros(pipe.shapes[ids["pw3"]][0], np.int8)
    last = np.zeros((BATCH, 1000), np.float32)
    pipe.set_input(ids["image"], images[0])
    pipe.forward()  # (the first forward of a model runs on one stream)
    for img in images:
        pipe.set_input(ids["image"], img)
        pipe.forward()
        if img is images[0]:
            pipe.get_async(ids["pw3"], mid)
            pipe.get_async(ids["softmax"], last)
    runtime.wait()
    serial.set_input(ids["image"], images[0])
    serial.forward()
    np.testing.assert_array_equal(mid, serial.get(ids["pw3"]))
    np.testing.assert_array_equal(last, serial.get(ids["softmax"]))
    serial.set_input(ids["image"], images[1])
    serial.forward()
    np.testing.assert_array_equal(pipe.get(ids["softmax"]), serial.get(ids["softmax"]))
    pipe.close()
    serial.close()


def test_a_network_of_a_few_operators_keeps_one_stream():
    """fewer than four operators in front and two behind: nothing to overlap"""
    from cases import MultiTypeCase
    m = runtime.Model()
    x = m.tensor("x", (4, 64, 56, 56), abi.QINT8, 0.05)
    m.mark_input(x)
    t = x
    for k in range(5):
        y = m.tensor("relu%d" % k, (4, 64, 56, 56), abi.QINT8, 0.05)
        m.opr(MultiTypeCase(abi.Q_RELU, (4, 64, 56, 56), (0.05, 0.01, 0.05)).symbol(), [t], [y])
        t = y
    m.mark_output(t)
    runtime.set_option("no_graph", 1)
    try:
        m.finalize()
    finally:
        runtime.set_option("no_graph", 0)
    assert m.nr_kernel == 5 and m.nr_tail_kernel == 0
    m.close()


def test_the_measuring_forwards_of_a_two_stream_model():
    """default options: forwards 2 + 3 and 7 + 8 are plain launches on two streams, 4 captures a graph
    (the tail of forward 3 still pending when the capture begins), 5 + 6 and 9 + 10 replay it, then the
    faster way runs. Same bytes throughout."""
    net = mobilenet.Net(BATCH)
    images = [mobilenet.draw_input(BATCH, seed=s) for s in (11, 12)]
    model, ids = build(net, False)
    serial, _ = build(net, False, no_graph=1, nopipeline=1)
    assert model.nr_tail_kernel >= 2
    want = []
    for img in images:
        serial.set_input(ids["image"], img)
        serial.forward()
        want.append(serial.get(ids["softmax"]).copy())
    model.set_input(ids["image"], images[0])
    for k in range(1, 13):
        model.forward()
        if k >= 4 and k % 2 == 0:
            np.testing.assert_array_equal(model.get(ids["softmax"]), want[0], err_msg="forward %d" % k)
    assert model.launch_mode()[0] in (1, -1)
    for img, w in zip(images[::-1], want[::-1]):
        model.set_input(ids["image"], img)
        model.forward()
        model.forward()
        np.testing.assert_array_equal(model.get(ids["softmax"]), w)
    model.close()
    serial.close()


@pytest.mark.parametrize("planned", [False, True], ids=["own_plan", "reference_plan"])
def test_two_hundred_overlapped_forwards(planned):
    """three inputs in rotation, every result copied out asynchronously, the host waits once at the
    end: each of the 200 results is the one of its input"""
    net = mobilenet.Net(BATCH)
    images = [mobilenet.draw_input(BATCH, seed=s) for s in (21, 22, 23)]
    pipe, ids = build(net, planned, no_graph=1)
    serial, _ = build(net, planned, no_graph=1, nopipeline=1)
    assert pipe.nr_tail_kernel >= 2
    want = []
    for img in images:
        serial.set_input(ids["image"], img)
        serial.forward()
        want.append(serial.get(ids["softmax"]).copy())
    outs = [np.zeros((BATCH, 1000), np.float32) for _ in range(200)]
    for k, out in enumerate(outs):
        pipe.set_input(ids["image"], images[k % 3])
        pipe.forward()
        pipe.get_async(ids["softmax"], out)
    runtime.wait()
    bad = [k for k, out in enumerate(outs) if not np.array_equal(out, want[k % 3])]
    assert not bad, bad[:10]
    pipe.close()
    serial.close()
