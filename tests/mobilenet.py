"""MobileNetV1 (width 1.0, 224x224x3, 13 depthwise-separable blocks, global average pool,
FC-1000, softmax) as the list of operators MegCC would emit for it with the NCHW44 layout enabled
(compiler/lib/Target/MGB/importer.cpp:1337-1352: nchw44 + fused conv-bias-activation; softmax
decomposed into Reduce-MAX, SUB, EXP, Reduce-SUM, TRUE_DIV, importer.cpp:987-1016; global average
pooling as a 7x7 stride-7 AVERAGE Pooling, importer.cpp:691-713).

No MobileNetV1 weights exist in the reference tree: weights are random int8 drawn from a seed and
the per-tensor scales come from tests/golden/mobilenet_scales.json, calibrated once from the same
seed so that activations use the int8 range instead of saturating (tests/golden/make_mobilenet_scales.py).

The same description drives (a) the GPU model runtime (megcc_gfx950_model_*), and (b) a layer by
layer evaluation with the CPU oracle.
"""
import json
import os

import numpy as np

from cases import ConvCase, PoolCase, TypeCvtCase
from megcc_amd import abi
from oracle import port

HERE = os.path.dirname(os.path.abspath(__file__))
SCALES_PATH = os.path.join(HERE, "golden", "mobilenet_scales.json")

# (stride of the depthwise conv, output channels of the pointwise conv)
BLOCKS = [(1, 64), (2, 128), (1, 128), (2, 256), (1, 256), (2, 512),
          (1, 512), (1, 512), (1, 512), (1, 512), (1, 512), (2, 1024), (1, 1024)]
IN_SCALE = 1.0 / 127.0


def conv_layers(batch):
    """[(name, ConvCase without scales)] in execution order"""
    layers = [("conv0", ConvCase(abi.FMT_NCHW_NCHW44, abi.DENSE, batch, 3, 224, 224, 32, 3, 2, 1, abi.RELU))]
    c, hw = 32, 112
    for i, (s, oc) in enumerate(BLOCKS, 1):
        layers.append(("dw%d" % i, ConvCase(abi.FMT_NCHW44, abi.GROUP, batch, c, hw, hw, c, 3, s, 1, abi.RELU)))
        hw //= s
        layers.append(("pw%d" % i, ConvCase(abi.FMT_NCHW44, abi.DENSE, batch, c, hw, hw, oc, 1, 1, 0, abi.RELU)))
        c = oc
    layers.append(("fc", ConvCase(abi.FMT_NCHW, abi.DENSE, batch, 1024, 1, 1, 1000, 1, 1, 0, abi.IDENTITY)))
    return layers


def macs_per_image():
    return sum(c.ops() // 2 for _, c in conv_layers(1))


def algorithmic_bytes(batch):
    """bytes one forward must move when every operator reads its inputs and writes its result once
    (activations in, weights, bias, activations out; the f32 image, the typecvts, the pooling and
    the five soft-max operators included): the figure a bandwidth roofline of the whole network is
    priced against"""
    n = lambda shape: int(np.prod(shape))
    total = batch * 3 * 224 * 224 * (4 + 1)  # quantise the f32 image
    for _, c in conv_layers(batch):
        total += n(c.src_shape()) + n(c.flt_shape()) + 4 * n(c.bias_shape()) + n(c.dst_shape())
    total += batch * 1024 * (49 + 1)  # global average pooling
    total += batch * 1000 * (1 + 4)  # dequantise the logits
    total += batch * 1000 * 4 * (1 + 2 + 2 + 1 + 2) + batch * 4 * (1 + 1 + 1 + 1)  # max, sub, exp, sum, div
    return total


def draw_weights(seed=0):
    """{layer: (filter int8, bias int32, filter scale)} -- independent of the batch size"""
    r = np.random.Generator(np.random.PCG64(seed))
    out = {}
    for name, case in conv_layers(1):
        flt = r.integers(-127, 128, case.flt_shape()).astype(np.int8)
        bias = r.integers(-1000, 1001, case.bias_shape()).astype(np.int32)
        out[name] = (flt, bias, 0.01)  # provisional filter scale, see make_mobilenet_scales.py
    return out


def load_scales():
    with open(SCALES_PATH) as f:
        return json.load(f)


def draw_input(batch, seed=0):
    r = np.random.Generator(np.random.PCG64(1000 + seed))
    return r.uniform(-1, 1, (batch, 3, 224, 224)).astype(np.float32)


class Lifetimes:
    """Stands in for runtime.Model on a machine without a GPU: records tensors and operators and
    derives the memory-plan requests the model runtime makes from them - time step = operator
    index; a tensor is alive from the operator that writes it to one past the last operator that
    touches it (outputs: one past the last operator + 1); views share their root's request;
    weights and model inputs (the caller's memory) are not planned."""

    def __init__(self, keep_pointwise_sources=False):
        """keep_pointwise_sources: what the model runtime's own plan adds to the reference's rule - the
        source of a pointwise convolution whose result feeds a channel-wise 3x3 convolution lives one
        operator longer (the pair may run as one kernel that reads it while it writes the result)"""
        self.sizes, self.root, self.first, self.last = [], [], [], []
        self.is_weight, self.is_output, self.is_input, self.dtype = [], [], [], []
        self.nr_opr = 0
        self.keep, self.prev, self.shapes = keep_pointwise_sources, None, []

    def _add(self, shape, type_enum, root=-1, weight=False):
        self.shapes.append(tuple(shape))
        self.sizes.append(int(np.prod(shape)) * abi.np_dtype(type_enum).itemsize)
        self.root.append(root)
        self.first.append(-1)
        self.last.append(-1)
        self.is_weight.append(weight)
        self.is_output.append(False)
        self.is_input.append(False)
        self.dtype.append(type_enum)
        return len(self.sizes) - 1

    def _root(self, t):
        while self.root[t] >= 0:
            t = self.root[t]
        return t

    def tensor(self, name, shape, type_enum, scale=1.0):
        return self._add(shape, type_enum)

    def weight(self, name, array, type_enum, scale=1.0):
        return self._add(array.shape, type_enum, weight=True)

    def alias(self, name, of, shape):
        return self._add(shape, self.dtype[of], root=of)

    def opr(self, symbol, inputs, outputs):
        k = self.nr_opr
        for t in inputs:
            r = self._root(t)
            self.last[r] = max(self.last[r], k)
        for t in outputs:
            r = self._root(t)
            if self.first[r] < 0:
                self.first[r] = k
            self.last[r] = max(self.last[r], k)
        if (self.keep and self.prev and "_conv2d_1x1_NCHW44_DENSE_p0x0_s1x1_" in self.prev[0]
                and "_conv2d_3x3_NCHW44_GROUP_p1x1_" in symbol and inputs[0] == self.prev[2][0]):
            n, ic4, _, w, _ = self.shapes[self.prev[1][0]]
            oc4 = self.shapes[self.prev[2][0]][1]
            if ic4 * 4 in (128, 256, 512) and oc4 % 16 == 0 and 4 <= w <= 31 and n * (oc4 // 16) <= 512:
                r = self._root(self.prev[1][0])
                self.last[r] = max(self.last[r], k)
        self.prev = (symbol, list(inputs), list(outputs))
        self.nr_opr += 1

    def mark_input(self, t):
        r = self._root(t)
        self.is_input[r] = True
        self.first[r] = 0
        self.last[r] = max(self.last[r], 0)

    def mark_output(self, t):
        self.is_output[self._root(t)] = True

    def finalize(self):
        pass

    def requests(self):
        """(tensor ids, begin, end, size) in tensor-id order"""
        ids = [t for t in range(len(self.sizes))
               if not self.is_weight[t] and not self.is_input[t] and self.root[t] < 0
               and self.first[t] >= 0]
        begin = [self.first[t] for t in ids]
        end = [self.nr_opr + 1 if self.is_output[t] else self.last[t] + 1 for t in ids]
        return ids, begin, end, [self.sizes[t] for t in ids]


class Net:
    """The operator list with all scales resolved: steps = [(kind, name, case, extra)]"""

    def __init__(self, batch, seed=0, scales=None):
        self.batch = batch
        self.weights = draw_weights(seed)
        self.scales = scales if scales is not None else load_scales()
        self.steps = []
        s_in = IN_SCALE
        self.steps.append(("typecvt", "quant", TypeCvtCase("f32", "qsi8", (batch, 3, 224, 224), dst_scale=s_in), None))
        for name, case in conv_layers(batch):
            if name == "fc":
                pool = PoolCase(abi.FMT_NCHW44, abi.POOL_AVERAGE, batch, 1024, 7, 7, 7, 7, 0, scale=s_in)
                self.steps.append(("pool", "avgpool", pool, None))
            wscale = float(self.scales[name]["filter"])
            case.scales = (s_in, wscale, float(self.scales[name]["dst"]))
            self.steps.append(("conv", name, case, None))
            s_in = case.scales[2]
        self.fc_scale = s_in
        self.steps.append(("typecvt", "dequant", TypeCvtCase("qsi8", "f32", (batch, 1000), src_scale=s_in), None))

    # ---- CPU oracle, layer by layer ------------------------------------------------------------
    def run_oracle(self, image, keep=False):
        port.set_threads(8)
        x = image
        trace = {}
        for kind, name, case, _ in self.steps:
            if kind == "typecvt":
                x = case.run_port({"src": np.ascontiguousarray(x.reshape(case.shape))})
            elif kind == "pool":
                x = case.run_port({"src": x})
            else:
                flt, bias, _ = self.weights[name]
                if name == "fc":
                    x = np.ascontiguousarray(x.reshape(self.batch, 1024, 1, 1))
                x = case.run_port({"src": x, "flt": flt, "bias": bias})
            if keep:
                trace[name] = x
        logits = x.reshape(self.batch, 1000)
        mx = port.reduce_f32(logits, abi.REDUCE_MAX, 1)
        e = port.elemwise_f32(port.elemwise_f32(logits, mx, abi.EW_SUB), None, abi.EW_EXP)
        sm = port.elemwise_f32(e, port.reduce_f32(e, abi.REDUCE_SUM, 1), abi.EW_TRUE_DIV)
        trace["softmax"] = sm
        return sm, trace

    def run_cpu_timed(self, image, threads=1):
        """One forward on host cores for the reported CPU baseline: every operator through the
        reference's own generated kernel when oracle/_ref has it, else through the C restatement.
        Returns (seconds, {operators run by reference kernels, by the port})."""
        import time
        import cases
        from oracle import ref
        port.set_threads(threads)
        x = image
        used = {"reference": 0, "port": 0}
        t0 = time.perf_counter()
        for kind, name, case, _ in self.steps:
            if kind == "typecvt":
                arrays = {"src": np.ascontiguousarray(x.reshape(case.shape))}
            elif kind == "pool":
                arrays = {"src": x}
            else:
                flt, bias, _ = self.weights[name]
                if name == "fc":
                    x = np.ascontiguousarray(x.reshape(self.batch, 1024, 1, 1))
                arrays = {"src": x, "flt": flt, "bias": bias}
            if ref.available() and ref.has(case.symbol()):
                x = cases.run_ref(case, arrays)
                used["reference"] += 1
            else:
                x = case.run_port(arrays)
                used["port"] += 1
        logits = x.reshape(self.batch, 1000)
        mx = port.reduce_f32(logits, abi.REDUCE_MAX, 1)
        e = port.elemwise_f32(port.elemwise_f32(logits, mx, abi.EW_SUB), None, abi.EW_EXP)
        port.elemwise_f32(e, port.reduce_f32(e, abi.REDUCE_SUM, 1), abi.EW_TRUE_DIV)
        return time.perf_counter() - t0, used

    # ---- GPU model -----------------------------------------------------------------------------
    def build_gpu(self, keep_all=False, model=None):
        """Describes the network to a runtime.Model (or to anything with the same methods, e.g.
        the Lifetimes recorder below) and finalizes it."""
        if model is None:
            from megcc_amd import runtime
            model = runtime.Model()
        m = model
        ids = {}
        b = self.batch
        x = m.tensor("image", (b, 3, 224, 224), abi.FLOAT)
        m.mark_input(x)
        ids["image"] = x
        for kind, name, case, _ in self.steps:
            if kind == "typecvt" and name == "quant":
                y = m.tensor(name, case.shape, abi.QINT8, case.dst_scale)
                m.opr(case.symbol(), [x], [y])
            elif kind == "typecvt":
                y = m.tensor(name, case.shape, abi.FLOAT)
                m.opr(case.symbol(), [x], [y])
            elif kind == "pool":
                y = m.tensor(name, case.dst_shape(), abi.QINT8, case.scale)
                m.opr(case.symbol(), [x], [y])
            else:
                flt, bias, _ = self.weights[name]
                wscale = case.scales[1]
                if name == "fc":  # MemForward: [B,256,1,1,4] and [B,1024,1,1] are the same bytes
                    x = m.alias("fc_in", x, (b, 1024, 1, 1))
                w = m.weight(name + ".w", flt, abi.QINT8, wscale)
                bi = m.weight(name + ".b", bias, abi.QINT32,
                              float(np.float32(case.scales[0]) * np.float32(wscale)))
                y = m.tensor(name, case.dst_shape(), abi.QINT8, case.scales[2])
                m.opr(case.symbol(), [x, w, bi], [y])
            ids[name] = y
            x = y
        logits = x
        mx = m.tensor("sm.max", (b, 1), abi.FLOAT)
        m.opr("kernel_reduce_MAX_DEFAULT_a1_f32f32", [logits], [mx])
        sub = m.tensor("sm.sub", (b, 1000), abi.FLOAT)
        m.opr("kernel_elementwise_SUB_f32f32f32", [logits, mx], [sub])
        ex = m.tensor("sm.exp", (b, 1000), abi.FLOAT)
        m.opr("kernel_elementwise_EXP_f32f32", [sub], [ex])
        sm_sum = m.tensor("sm.sum", (b, 1), abi.FLOAT)
        m.opr("kernel_reduce_SUM_DEFAULT_a1_f32f32", [ex], [sm_sum])
        out = m.tensor("softmax", (b, 1000), abi.FLOAT)
        m.opr("kernel_elementwise_TRUE_DIV_f32f32f32", [ex, sm_sum], [out])
        ids["softmax"] = out
        m.mark_output(out)
        if keep_all:
            for tid in ids.values():
                m.mark_output(tid)
        m.finalize()
        return m, ids
