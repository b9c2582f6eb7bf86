#!/usr/bin/env python3
"""bench.py -- one JSON line for the headline metric of the generated-kernel hot path.

Default workload: the qsi8 3x3 stride-1 pad-1 NCHW44 convolution of BASELINE.json configs[1] at
its largest single-GPU shape (N=32, Cin=Cout=256, 56x56, int32 bias, fused ReLU, scales
0.02/0.01 -> 0.05), called through the C ABI exactly as the TinyNN VM would: init protocol once,
then one kernel call per step with all operands resident in HBM.

  value      whole-job int8 throughput, ops = 2*N*OC*OH*OW*IC*FH*FW  (the reference's own workload
             formula, compiler/test/kernel/common/src/workload_proxy.cpp:69), wall clock around
             the K timed steps with a stream sync on both sides
  roofline   the same ops over the average kernel duration measured with HIP events on the
             library's stream, against the 5.0 POP/s dense int8 MFMA peak of MI355X
  cpu_baseline  the reference's own generated C kernel (oracle/_ref, kind "reference") or our C
             restatement (kind "port") on ONE host core, on a bounded slice of the same layer

  checked    after the timed region the output of the LAST timed launch is fetched and compared
             with the CPU oracle (bit for bit for qsi8): images 0, middle and last of a batched
             convolution (the reference's kernels treat images independently, so the oracle on one
             image is exact for that image), the whole tensor for small workloads. A mismatch
             aborts the run: no metric line is printed for wrong results.

Before the W warm-up steps the same operator is launched untimed for --preheat-ms (default 300 ms):
a cold MI355X takes a few hundred 60 us launches to leave its idle clocks, and 5 warm-up launches
(1/3 ms) measure that ramp rather than the kernel. The line says how many launches that was.

Other workloads (--workload dw|fc|chain|mobilenet ...) report the other configurations; the driver
uses the default.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

PEAK_INT8_TOPS = 5000.0  # dense int8 MFMA, MI355X
PEAK_HBM_GBS = 8000.0
# HBM bytes per launch of a workload's dominant kernel come from the committed rocprofv3 --pmc
# summaries (FETCH_SIZE / WRITE_SIZE in KiB per dispatch, scaled by what a 256 MiB copy reads on
# the same counters); a summary holds one line "TRAFFIC_BYTES_PER_LAUNCH[<workload>]=<n>" per
# workload it covers.
TRAFFIC_FILES = ["profiles/conv_mfma_i8_dma__conv3x3_n32_c256_56x56.txt",
                 "profiles/cfg3_fc_matmul__all_shapes.txt", "profiles/cfg4_dw_pool_add__n64.txt"]


def measured_traffic(workload):
    """(bytes read per launch, bytes written per launch, file) from the committed counter summaries,
    or (None, None, None). A summary holds "TRAFFIC_READ_BYTES_PER_LAUNCH[<workload>]=<n>" and
    "TRAFFIC_WRITE_BYTES_PER_LAUNCH[<workload>]=<n>" (older ones one line with the sum:
    "TRAFFIC_BYTES_PER_LAUNCH[...]", returned as reads with writes unknown)."""
    keys = ["TRAFFIC_%sBYTES_PER_LAUNCH[%s]=" % (k, workload) for k in ("READ_", "WRITE_", "")]
    for rel in TRAFFIC_FILES:
        found = {}
        try:
            with open(os.path.join(ROOT, rel)) as f:
                for line in f:
                    for k in keys:
                        if line.startswith(k):
                            found[k] = int(line.split("=", 1)[1])
        except OSError:
            continue
        if keys[0] in found:
            return found[keys[0]], found.get(keys[1]), rel
        if keys[2] in found:
            return found[keys[2]], None, rel
    return None, None, None


def traffic_fields(workload, algorithmic_bytes, output_bytes):
    """roofline.traffic and what it is made of. WRITE_SIZE reads (close to) nothing for some kernels
    that do write - their dirty lines are still in L2 when the dispatch ends and leave it during the
    next one - so where the counter shows less than half of the bytes the kernel must write, the
    output bytes are counted instead and the line says so."""
    rd, wr, rel = measured_traffic(workload)
    if rd is None:
        return {"traffic": None}
    out = {"traffic_source": rel, "traffic_read": rd}
    if wr is None:
        out.update(traffic=rd, traffic_note="reads and writes as summed in the summary")
    elif wr < 0.5 * output_bytes:
        out.update(traffic=rd + output_bytes, traffic_write=output_bytes,
                   traffic_note="WRITE_SIZE showed %d bytes for a kernel that writes %d (dirty lines still in L2 "
                                "at dispatch end): the output bytes are counted instead" % (wr, output_bytes))
    else:
        out.update(traffic=rd + wr, traffic_write=wr)
    out["traffic_over_algorithmic"] = round(out["traffic"] / algorithmic_bytes, 3)
    return out


class HipEvents:
    def __init__(self, stream):
        self.hip = C.CDLL("libamdhip64.so")
        self.stream = C.c_void_p(stream)
        self.hip.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        self.hip.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        self.hip.hipEventSynchronize.argtypes = [C.c_void_p]
        self.hip.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]

    def new(self):
        e = C.c_void_p()
        assert self.hip.hipEventCreate(C.byref(e)) == 0
        return e

    def record(self, e):
        assert self.hip.hipEventRecord(e, self.stream) == 0

    def elapsed_ms(self, a, b):
        assert self.hip.hipEventSynchronize(b) == 0
        ms = C.c_float()
        assert self.hip.hipEventElapsedTime(C.byref(ms), a, b) == 0
        return ms.value


def headline_case(n=32, c=256, hw=56, scales=(0.02, 0.01, 0.05)):
    from cases import ConvCase
    from megcc_amd import abi
    return ConvCase(abi.FMT_NCHW44, abi.DENSE, n, c, hw, hw, c, 3, 1, 1, abi.RELU, scales=scales)


def make_workload(name):
    """-> (case, description, bound, algorithmic units per launch)"""
    from cases import (ConcatCase, ConvCase, FusedCase, MatMulCase, MultiTypeCase, PoolCase,
                       RelayoutCase, ResizeCase, TypeCvtCase)
    from megcc_amd import abi
    if name == "stem7x7":
        case = ConvCase(abi.FMT_NCHW_NCHW44, abi.DENSE, 64, 3, 224, 224, 64, 7, 2, 3, abi.RELU,
                        scales=(0.02, 0.01, 0.05))
        return case, "qsi8 first layer NCHW->NCHW44 7x7 s2 p3 N=64 3->64 224x224", "hbm"
    if name == "conv5x5":
        case = ConvCase(abi.FMT_NCHW44, abi.DENSE, 64, 32, 28, 28, 64, 5, 1, 2, abi.RELU,
                        scales=(0.02, 0.01, 0.05))
        return case, "qsi8 conv5x5 s1 p2 NCHW44 N=64 32->64 28x28", "mfma"
    if name.startswith("conv_s2:"):  # conv_s2:N,C,HW - 3x3 stride 2 pad 1, Cin = Cout (down-sampling layers)
        n, c, hw = (int(v) for v in name[8:].split(","))
        case = ConvCase(abi.FMT_NCHW44, abi.DENSE, n, c, hw, hw, c, 3, 2, 1, abi.RELU, scales=(0.02, 0.01, 0.05))
        return case, "qsi8 conv3x3 s2 p1 NCHW44 N=%d Cin=Cout=%d %dx%d +bias +ReLU requant" % (n, c, hw, hw), "mfma"
    if name == "pw_s2":
        case = ConvCase(abi.FMT_NCHW44, abi.DENSE, 64, 256, 56, 56, 512, 1, 2, 0, abi.IDENTITY,
                        scales=(0.02, 0.01, 0.05))
        return case, "qsi8 conv1x1 s2 NCHW44 N=64 256->512 56x56 -> 28x28", "mfma"
    if name == "fused":
        return (FusedCase(["I0,SILU,O0", "O0,I1,MUL,O1", "O1,I2,ADD,D"],
                          [(8, 256, 80, 80), (1, 256, 1, 1), (1, 256, 1, 1)]),
                "f32 fused SiLU(x) * scale[c] + shift[c], N=8 C=256 80x80", "hbm")
    if name in ("resize_linear", "resize_linear44", "resize_nearest"):
        fmt = abi.FMT_NCHW44 if name == "resize_linear44" else abi.FMT_NCHW
        c = 64 if name == "resize_linear44" else 256
        return (ResizeCase(fmt, "NEAREST" if name == "resize_nearest" else "LINEAR", 8, c, 40, 40, 80, 80),
                "f32 %s x2 N=8 C=256 40x40 -> 80x80" % name, "hbm")
    if name in ("to_nchw4", "from_nchw4"):
        hw = 56 * 56
        nchw = (256 * hw, 4 * hw, 56, 1, hw)  # a [N, C/4, H, W, 4] view of NCHW memory
        shape = (32, 64, 56, 56, 4)
        if name == "to_nchw4":
            return (RelayoutCase("qsi8", shape, nchw, slack=0),
                    "qsi8 relayout NCHW -> NCHW4 N=32 C=256 56x56", "hbm")
        return (RelayoutCase("qsi8", shape, None, None, nchw, slack=0),
                "qsi8 relayout NCHW4 -> NCHW N=32 C=256 56x56", "hbm")
    if name == "transpose":
        return RelayoutCase("f32", (4096, 4096), (1, 4096), slack=0), "f32 transpose 4096x4096", "hbm"
    if name == "concat":
        return (ConcatCase("qsi8", [(32, 32, 56, 56, 4), (32, 32, 56, 56, 4)], 1),
                "qsi8 concat of two N=32 C=128 56x56 NCHW44 maps along C", "hbm")
    if name.startswith("conv:"):  # conv:N,C,HW - any shape of the qsi8 3x3 configuration
        n, c, hw = (int(v) for v in name[5:].split(","))
        return (headline_case(n, c, hw),
                "qsi8 conv3x3 s1 p1 NCHW44 N=%d Cin=Cout=%d %dx%d +bias +ReLU requant" % (n, c, hw, hw), "mfma")
    if name == "conv":
        case = headline_case()
        return case, "qsi8 conv3x3 s1 p1 NCHW44 N=32 Cin=Cout=256 56x56 +bias +ReLU requant", "mfma"
    if name == "conv_cal":
        # The default scales (0.02 * 0.01 / 0.05 = 1 / 250) make every 125th accumulator an exact tie, the
        # worst case for the requantisation (threshold table). Scales without ties, as a calibrated
        # network has them, requantise by one multiply-add; the output then also uses the whole range.
        return (headline_case(scales=(0.0213, 0.0097, 0.517)),
                "qsi8 conv3x3 s1 p1 NCHW44 N=32 Cin=Cout=256 56x56 +bias +ReLU requant, scales without exact ties", "mfma")
    if name == "conv_c64":
        return headline_case(32, 64, 56), "qsi8 conv3x3 NCHW44 N=32 C=64 56x56", "mfma"
    if name == "conv_c256_28":
        return headline_case(32, 256, 28), "qsi8 conv3x3 NCHW44 N=32 C=256 28x28", "mfma"
    if name == "conv_n1":
        return headline_case(1, 64, 56), "qsi8 conv3x3 NCHW44 N=1 C=64 56x56", "mfma"
    if name == "pw":
        case = ConvCase(abi.FMT_NCHW44, abi.DENSE, 64, 512, 14, 14, 512, 1, 1, 0, abi.RELU,
                        scales=(0.02, 0.01, 0.05))
        return case, "qsi8 conv1x1 NCHW44 N=64 C=512 14x14", "mfma"
    if name in ("pw1", "pw2", "pw3", "pw4", "pw5", "pw6", "pw7", "pw12", "pw13"):
        # MobileNetV1 pointwise layers, batch 64
        ic, oc, hw = {"pw1": (32, 64, 112), "pw2": (64, 128, 56), "pw3": (128, 128, 56),
                      "pw4": (128, 256, 28), "pw5": (256, 256, 28), "pw6": (256, 512, 14),
                      "pw7": (512, 512, 14), "pw12": (512, 1024, 7), "pw13": (1024, 1024, 7)}[name]
        case = ConvCase(abi.FMT_NCHW44, abi.DENSE, 64, ic, hw, hw, oc, 1, 1, 0, abi.RELU,
                        scales=(0.02, 0.01, 0.05))
        return case, "qsi8 conv1x1 NCHW44 N=64 %d->%d %dx%d" % (ic, oc, hw, hw), "hbm"
    if name.startswith("mb:"):  # mb:<layer> - a convolution of MobileNetV1 at batch 64 with its calibrated scales
        import mobilenet
        for kind, lname, case, _ in mobilenet.Net(64).steps:
            if kind == "conv" and lname == name[3:]:
                return case, "MobileNetV1 batch 64, layer %s: %s" % (lname, case.symbol()), "hbm"
        raise SystemExit("bench.py: MobileNetV1 has no convolution called %r" % name[3:])
    if name == "fc":
        case = ConvCase(abi.FMT_NCHW, abi.DENSE, 4096, 4096, 1, 1, 4096, 1, 1, 0, abi.IDENTITY,
                        scales=(0.01, 0.01, 0.1))
        return case, "qsi8 FullyConnected 4096x4096x4096", "mfma"
    if name == "fc1":
        case = ConvCase(abi.FMT_NCHW, abi.DENSE, 1, 1024, 1, 1, 1000, 1, 1, 0, abi.IDENTITY,
                        scales=(0.01, 0.01, 0.1))
        return case, "qsi8 FullyConnected 1x1024x1000", "hbm"
    if name == "fc64":
        case = ConvCase(abi.FMT_NCHW, abi.DENSE, 64, 4096, 1, 1, 4096, 1, 1, 0, abi.IDENTITY,
                        scales=(0.01, 0.01, 0.1))
        return case, "qsi8 FullyConnected 64x4096x4096", "hbm"
    if name in ("dw_nchw", "dw_nchw_s2"):  # the depthwise layer of configs[3] on plain NCHW tensors
        s = 2 if name.endswith("s2") else 1
        case = ConvCase(abi.FMT_NCHW, abi.GROUP, 64, 32, 112, 112, 32, 3, s, 1, abi.RELU, scales=(0.02, 0.01, 0.05))
        return case, "qsi8 depthwise 3x3 s%d NCHW N=64 C=32 112x112" % s, "hbm"
    if name in ("dw5x5", "dw5x5_s2", "dw7x7", "dw_hswish"):  # depthwise layers of MobileNetV3 / EfficientNet style blocks
        c, hw, k, s, act = {"dw5x5": (240, 28, 5, 1, abi.RELU), "dw5x5_s2": (96, 56, 5, 2, abi.RELU),
                            "dw7x7": (96, 28, 7, 1, abi.RELU), "dw_hswish": (144, 56, 3, 1, abi.H_SWISH)}[name]
        case = ConvCase(abi.FMT_NCHW44, abi.GROUP, 64, c, hw, hw, c, k, s, k // 2, act, scales=(0.02, 0.01, 0.05))
        return case, "qsi8 depthwise %dx%d s%d NCHW44 N=64 C=%d %dx%d %s" % (
            k, k, s, c, hw, hw, abi.NONLINE_NAMES[act]), "hbm"
    if name in ("pw_24_144", "pw_144_24"):  # pointwise layers whose channel counts are no multiples of 32
        ic, oc = (24, 144) if name == "pw_24_144" else (144, 24)
        case = ConvCase(abi.FMT_NCHW44, abi.DENSE, 64, ic, 56, 56, oc, 1, 1, 0, abi.RELU, scales=(0.02, 0.01, 0.05))
        return case, "qsi8 conv1x1 NCHW44 N=64 %d->%d 56x56" % (ic, oc), "hbm"
    if name.startswith("dw"):  # dw:C,HW,S - any shape of the depthwise layer of configs[3]
        c, hw, s = [int(v) for v in name[3:].split(",")] if name.startswith("dw:") else {
            "dw": (32, 112, 1), "dw_s2": (32, 112, 2), "dw512": (512, 14, 1), "dw512_s2": (512, 14, 2)}[name]
        case = ConvCase(abi.FMT_NCHW44, abi.GROUP, 64, c, hw, hw, c, 3, s, 1, abi.RELU,
                        scales=(0.02, 0.01, 0.05))
        return case, "qsi8 depthwise 3x3 s%d NCHW44 N=64 C=%d %dx%d" % (s, c, hw, hw), "hbm"
    if name == "pool":
        return (PoolCase(abi.FMT_NCHW44, abi.POOL_MAX, 64, 32, 112, 112, 2, 2, 0),
                "qsi8 maxpool 2x2 s2 NCHW44 N=64 C=32 112x112", "hbm")
    if name == "pool44_s2":  # the same stem pooling in NCHW44
        return (PoolCase(abi.FMT_NCHW44, abi.POOL_MAX, 64, 64, 112, 112, 3, 2, 1),
                "qsi8 maxpool 3x3 s2 p1 NCHW44 N=64 C=64 112x112", "hbm")
    if name in ("pool_nchw", "pool_nchw_s1"):  # the stem pooling of a ResNet-like model kept in NCHW
        w, s = (3, 2) if name == "pool_nchw" else (3, 1)
        return (PoolCase(abi.FMT_NCHW, abi.POOL_MAX, 64, 64, 112, 112, w, s, 1),
                "qsi8 maxpool %dx%d s%d p1 NCHW N=64 C=64 112x112" % (w, w, s), "hbm")
    if name == "add":
        return (MultiTypeCase(abi.Q_FUSE_ADD_RELU, (64, 32, 56, 56), (0.05, 0.01, 0.05)),
                "qsi8 QFUSE_ADD_RELU 64x32x56x56", "hbm")
    if name in ("mm", "mm64", "mm1"):
        m, k, n = {"mm": (4096, 4096, 4096), "mm64": (64, 4096, 4096), "mm1": (1, 1024, 1000)}[name]
        return MatMulCase(m, k, n), "f32 MatMul %dx%dx%d" % (m, k, n), "mfma_f32"
    if name == "conv_f32":
        case = ConvCase(abi.FMT_NCHW, abi.DENSE, 1, 32, 56, 56, 32, 3, 1, 1, abi.RELU, dtype="f32")
        return case, "f32 conv3x3 NCHW N=1 C=32 56x56 +bias +ReLU", "mfma_f32"
    if name in ("bias64", "bias4096", "bias1"):  # the f32 FullyConnected bias: [M,N] + [N]
        from cases import ElemwiseCase
        m, n = {"bias64": (64, 4096), "bias4096": (4096, 4096), "bias1": (1, 1000)}[name]
        return ElemwiseCase("ADD", [(m, n), (n,)]), "f32 elementwise ADD [%d,%d] + [%d]" % (m, n, n), "hbm"
    if name == "softmax_max":
        from cases import ReduceCase
        return ReduceCase("MAX", (64, 1000), 1), "f32 reduce MAX [64,1000] axis 1", "hbm"
    if name == "copy":  # same-scale requantise = a plain copy: the counter calibration kernel
        return (TypeCvtCase("qsi8", "qsi8", (256, 1024, 1024), src_scale=0.05, dst_scale=0.05),
                "qsi8->qsi8 typecvt, equal scales, 256 MiB in + 256 MiB out", "hbm")
    if name == "copy_dw":  # a plain copy of the depthwise workload's size: what that size allows
        return (TypeCvtCase("qsi8", "qsi8", (64, 32, 112 * 112), src_scale=0.05, dst_scale=0.05),
                "qsi8->qsi8 typecvt, equal scales, 25.7 MB in + 25.7 MB out", "hbm")
    raise SystemExit("unknown workload " + name)


def bench_mobilenet(batch, steps, warmup, per_layer=False):
    """MobileNetV1-int8 end to end through the model runtime: images/s, inputs resident in HBM."""
    import mobilenet
    from megcc_amd import runtime
    net = mobilenet.Net(batch)
    model, ids = net.build_gpu()
    model.set_input(ids["image"], mobilenet.draw_input(batch, seed=1))
    ev = HipEvents(runtime.lib().megcc_gfx950_stream())
    for _ in range(warmup):
        model.forward()
    runtime.wait()
    e0, e1 = ev.new(), ev.new()
    t0 = time.perf_counter()
    ev.record(e0)
    for _ in range(steps):
        model.forward()
    model.join()  # (the last operators of a forward may be on the runtime's second stream)
    ev.record(e1)
    runtime.wait()
    wall = time.perf_counter() - t0
    dev_ms = ev.elapsed_ms(e0, e1) / steps
    out = {"batch": batch, "images_per_s": round(batch * steps / wall, 1),
           "ms_per_forward": round(wall * 1e3 / steps, 4), "device_ms_per_forward": round(dev_ms, 4),
           "arena_bytes": model.arena_bytes, "nr_opr": model.nr_opr,
           "int8_tops": round(2 * mobilenet.macs_per_image() * batch / (dev_ms * 1e-3) / 1e12, 2)}
    # the network is bandwidth-bound at these batches (1.14 GOP against 11 MB of activations and
    # weights per image): priced against HBM on the bytes its operators read and write once each
    moved = mobilenet.algorithmic_bytes(batch)
    out["nr_kernel"] = model.nr_kernel
    out["nr_tail_kernel"] = model.nr_tail_kernel  # of those, on the second stream (they overlap the next forward's first kernels)
    mode, eager_ms, graph_ms = model.launch_mode()
    out["launch_mode"] = {1: "graph", -1: "eager", 0: "undecided"}[mode]
    out["launch_mode_measured_ms"] = {"eager": round(eager_ms, 4), "graph": round(graph_ms, 4)}
    out["roofline"] = {"bound": "hbm", "achieved": round(moved / (dev_ms * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBS,
                       "unit": "GB/s", "frac": round(moved / (dev_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                       "traffic": None, "algorithmic_per_launch": moved,
                       "mfma_frac": round(out["int8_tops"] / PEAK_INT8_TOPS, 4)}
    if per_layer:
        names = [n for _, n, _, _ in net.steps] + ["sm.max", "sm.sub", "sm.exp", "sm.sum", "softmax"]
        layers = []
        for i in range(model.nr_opr):
            for _ in range(3):
                model.run_opr(i)
            runtime.wait()
            a, b = ev.new(), ev.new()
            ev.record(a)
            for _ in range(10):
                model.run_opr(i)
            ev.record(b)
            runtime.wait()
            layers.append((names[i], round(ev.elapsed_ms(a, b) / 10 * 1e3, 1)))
        out["layer_us"] = layers
    model.close()
    return out


def check_output(case, arrays, got):
    """Compares the output the timed launches left behind with the CPU oracle. Returns a short
    description of what was compared; raises SystemExit on a mismatch."""
    import numpy as np
    import cases
    from cases import ConvCase
    from oracle import port
    port.set_threads(os.cpu_count() or 8)

    def same(a, b, what):
        if a.dtype == np.float32:
            err = cases.max_rel_err(a, b)
            if err > 1e-4:
                raise SystemExit("bench.py: %s differs from the oracle (max err %g)" % (what, err))
        elif not np.array_equal(a, b):
            raise SystemExit("bench.py: %s differs from the oracle in %d of %d elements" % (
                what, int((a != b).sum()), a.size))

    if isinstance(case, ConvCase) and case.n > 3 and case.ops() > 4e9:
        picks = sorted({0, case.n // 2, case.n - 1})
        import copy
        one = copy.copy(case)
        one.n = 1
        for i in picks:
            want = one.run_port({"src": arrays["src"][i:i + 1], "flt": arrays["flt"], "bias": arrays["bias"]})
            same(got[i:i + 1], want, "image / row %d of the output" % i)
        return "%s %s of %d against the oracle, bit for bit" % (
            "rows" if case.ih == 1 and case.fmt == 0 else "images", picks, case.n)
    from cases import MatMulCase
    if isinstance(case, MatMulCase):
        # f32 MatMul: against the fp64 product of the first 64 rows. (The oracle's float32 running
        # sum over K = 4096 is itself up to 1.2e-4 from the fp64 result, further than the GPU's
        # tiled sums; tests/test_full_size.py compares all three.)
        rows = min(case.m, 64)
        a = arrays["a"].T if case.trans_a else arrays["a"]
        b = arrays["b"].T if case.trans_b else arrays["b"]
        want = (a[:rows].astype(np.float64) @ b.astype(np.float64)).astype(np.float32)
        same(got[:rows], want, "rows 0..%d of the product" % (rows - 1))
        return "rows 0..%d of %d against the fp64 product, 1e-4" % (rows - 1, case.m)
    if hasattr(case, "ops") and case.ops() > 4e10:
        return None  # (too large for the oracle in a benchmark run; covered by tests/test_full_size.py)
    same(got, case.run_port(arrays), "the output")
    return "whole output against the oracle"


def bench_chain(c, hw, stride, steps, warmup, batch=64, cpu=False):
    """BASELINE configs[3]: depthwise 3x3 -> max-pool 2x2 s2 -> add + ReLU with requantisation,
    three operators of one model on the static arena (the model runtime runs the chain as one kernel
    when nothing else reads the tensors in between). Bytes = what each operator must read and write
    once (the pooled map's partner tensor included)."""
    import numpy as np
    from cases import ConvCase, MultiTypeCase, PoolCase
    from megcc_amd import abi, runtime
    dw = ConvCase(abi.FMT_NCHW44, abi.GROUP, batch, c, hw, hw, c, 3, stride, 1, abi.RELU,
                  scales=(0.02, 0.01, 0.05))
    pool = PoolCase(abi.FMT_NCHW44, abi.POOL_MAX, batch, c, dw.oh, dw.ow, 2, 2, 0, scale=0.05)
    add = MultiTypeCase(abi.Q_FUSE_ADD_RELU, pool.dst_shape(), (0.05, 0.01, 0.05))
    arrays = dw.gen(0)
    other = np.random.default_rng(1).integers(-128, 128, pool.dst_shape()).astype(np.int8)
    m = runtime.Model()
    x = m.tensor("x", dw.src_shape(), abi.QINT8, 0.02)
    y = m.tensor("other", pool.dst_shape(), abi.QINT8, 0.01)
    m.mark_input(x)
    m.mark_input(y)
    w = m.weight("dw.w", arrays["flt"], abi.QINT8, 0.01)
    b = m.weight("dw.b", arrays["bias"], abi.QINT32, float(np.float32(0.02) * np.float32(0.01)))
    t1 = m.tensor("dw", dw.dst_shape(), abi.QINT8, 0.05)
    m.opr(dw.symbol(), [x, w, b], [t1])
    t2 = m.tensor("pool", pool.dst_shape(), abi.QINT8, 0.05)
    m.opr(pool.symbol(), [t1], [t2])
    t3 = m.tensor("out", pool.dst_shape(), abi.QINT8, 0.05)
    m.opr(add.symbol(), [t2, y], [t3])
    m.mark_output(t3)
    m.finalize()
    m.set_input(x, arrays["src"])
    m.set_input(y, other)
    ev = HipEvents(runtime.lib().megcc_gfx950_stream())
    for _ in range(max(warmup, 3)):
        m.forward()
    runtime.wait()
    e0, e1 = ev.new(), ev.new()
    ev.record(e0)
    for _ in range(steps):
        m.forward()
    m.join()
    ev.record(e1)
    runtime.wait()
    ms = ev.elapsed_ms(e0, e1) / steps
    n_in, n_dw, n_pool = (int(np.prod(sh)) for sh in (dw.src_shape(), dw.dst_shape(), pool.dst_shape()))
    nbytes = (n_in + n_dw) + (n_dw + n_pool) + 3 * n_pool  # the three operators, each reading and writing once
    # the model runtime runs the chain as one kernel when it can: then the two tensors in between never
    # reach memory and what must move is the input, the addition's other operand and the result
    fused = runtime.last_kernel().startswith("dwconv44_chain")
    moved = n_in + 2 * n_pool if fused else nbytes
    # what came out, against the oracle on image 0 and the last one
    from oracle import port
    port.set_threads(os.cpu_count() or 8)
    got = m.get(t3)
    one = ConvCase(abi.FMT_NCHW44, abi.GROUP, 1, c, hw, hw, c, 3, stride, 1, abi.RELU, scales=(0.02, 0.01, 0.05))
    for i in (0, batch - 1):
        d = one.run_port({"src": arrays["src"][i:i + 1], "flt": arrays["flt"], "bias": arrays["bias"]})
        p = port.pool_q8(d, abi.FMT_NCHW44, abi.POOL_MAX, (2, 2), (2, 2), (0, 0))
        want = port.multitype_q8(p, other[i:i + 1], abi.Q_FUSE_ADD_RELU, 0.05, 0.01, 0.05)
        if not np.array_equal(got[i:i + 1], want):
            raise SystemExit("bench.py: chain output of image %d differs from the oracle" % i)
    m.close()
    cpu_leg = {}
    if cpu:
        # the three operators through the C restatement on ONE host core, image 0 only
        port.set_threads(1)
        t0 = time.perf_counter()
        d = one.run_port({"src": arrays["src"][:1], "flt": arrays["flt"], "bias": arrays["bias"]})
        p = port.pool_q8(d, abi.FMT_NCHW44, abi.POOL_MAX, (2, 2), (2, 2), (0, 0))
        port.multitype_q8(p, other[:1], abi.Q_FUSE_ADD_RELU, 0.05, 0.01, 0.05)
        dt = time.perf_counter() - t0
        cpu_leg = {"cpu_baseline": {
            "value": round(nbytes / batch / dt / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "batch 1 of %d, timed once in %.5f s (the whole workload at that rate: %.4g s); "
                      "oracle/oracle_port.c built with -O2" % (batch, dt, dt * batch),
            "host_cores": os.cpu_count()}}
    return {**cpu_leg, "metric": "hbm_gbps", "value": round(nbytes / (ms * 1e-3) / 1e9, 1), "unit": "GB/s",
            "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": round(ms, 5),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int8",
            "data": "synthetic",
            "config": {"workload": "qsi8 depthwise 3x3 s%d -> maxpool 2x2 s2 -> add+ReLU requant, N=%d C=%d %dx%d NCHW44"
                       % (stride, batch, c, hw, hw), "one_kernel": fused,
                       "value_counts": "the bytes the three operators read and write when each runs on its own"},
            "roofline": {"bound": "hbm", "achieved": round(moved / (ms * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBS,
                         "unit": "GB/s", "frac": round(moved / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                         "traffic": None, "algorithmic_per_launch": moved},
            "checked": True, "checked_what": "images 0 and %d of the chain's output, bit for bit" % (batch - 1)}


def bench_pwdw(batch, ic, oc, hw, stride, steps, warmup):
    """A pointwise 1x1 layer and the channel-wise 3x3 layer behind it as a two-operator model on the
    static arena, three ways: as the model runtime decides (it times both forms at finalize), as one
    kernel (megcc_gfx950_pw_dw) and as the two kernels. Scales with an exact multiply-add
    requantisation, like a calibrated network's."""
    import numpy as np
    from cases import ConvCase, MultiTypeCase
    from megcc_amd import abi, runtime
    pw = ConvCase(abi.FMT_NCHW44, abi.DENSE, batch, ic, hw, hw, oc, 1, 1, 0, abi.RELU, scales=(0.0213, 0.0097, 0.0371))
    dw = ConvCase(abi.FMT_NCHW44, abi.GROUP, batch, oc, hw, hw, oc, 3, stride, 1, abi.RELU,
                  scales=(0.0371, 0.0131, 0.0689), flt_range=(-40, 40))
    a0, a1 = pw.gen(31), dw.gen(32)
    src0 = np.random.default_rng(5).integers(-128, 128, pw.src_shape()).astype(np.int8)
    pre = MultiTypeCase(abi.Q_RELU, pw.src_shape(), (0.03, 0.01, pw.scales[0]))
    bias_scale = lambda c: float(np.float32(c.scales[0]) * np.float32(c.scales[1]))
    ev = HipEvents(runtime.lib().megcc_gfx950_stream())
    out, results = {}, {}
    for mode in ("runtime", "one", "two"):
        runtime.set_option("nofusepwdw", 1 if mode == "two" else 0)
        runtime.set_option("fusepwdw", 1 if mode == "one" else 0)
        m = runtime.Model()
        x0 = m.tensor("x0", pw.src_shape(), abi.QINT8, 0.03)
        m.mark_input(x0)
        # (the pair's source is an arena tensor, as inside a network; it is an output as well, so that
        #  no memory plan lays the pair's result over it and the one kernel can run at every batch)
        x = m.tensor("x", pw.src_shape(), abi.QINT8, pw.scales[0])
        m.opr(pre.symbol(), [x0], [x])
        m.mark_output(x)
        t1 = m.tensor("mid", pw.dst_shape(), abi.QINT8, pw.scales[2])
        m.opr(pw.symbol(), [x, m.weight("pw.w", a0["flt"], abi.QINT8, pw.scales[1]),
                            m.weight("pw.b", a0["bias"], abi.QINT32, bias_scale(pw))], [t1])
        t2 = m.tensor("out", dw.dst_shape(), abi.QINT8, dw.scales[2])
        m.opr(dw.symbol(), [t1, m.weight("dw.w", a1["flt"], abi.QINT8, dw.scales[1]),
                            m.weight("dw.b", a1["bias"], abi.QINT32, bias_scale(dw))], [t2])
        m.mark_output(t2)
        m.finalize()
        runtime.set_option("nofusepwdw", 0)
        runtime.set_option("fusepwdw", 0)
        m.set_input(x0, src0)
        m.forward()
        runtime.wait()
        results[mode] = m.get(t2).copy()
        # the pair alone: operators 1.. of the schedule cannot be run apart from operator 0 through
        # forward(), so the ReLU in front is timed too and subtracted (its own model below)
        for _ in range(max(warmup, 3)):
            m.forward()
        runtime.wait()
        e0, e1 = ev.new(), ev.new()
        ev.record(e0)
        for _ in range(steps):
            m.forward()
        m.join()
        ev.record(e1)
        runtime.wait()
        out[mode] = {"us_per_forward": round(ev.elapsed_ms(e0, e1) / steps * 1e3, 2), "nr_kernel": m.nr_kernel}
        m.close()
    if not (np.array_equal(results["one"], results["two"]) and np.array_equal(results["runtime"], results["two"])):
        raise SystemExit("bench.py: the one-kernel pair and the two kernels differ")
    # image 0 against the oracle
    from oracle import port
    port.set_threads(os.cpu_count() or 8)
    one0 = ConvCase(abi.FMT_NCHW44, abi.DENSE, 1, ic, hw, hw, oc, 1, 1, 0, abi.RELU, scales=pw.scales)
    one1 = ConvCase(abi.FMT_NCHW44, abi.GROUP, 1, oc, hw, hw, oc, 3, stride, 1, abi.RELU, scales=dw.scales)
    mid = one0.run_port({"src": pre.run_port({"a": src0[:1], "b": None}), "flt": a0["flt"], "bias": a0["bias"]})
    want = one1.run_port({"src": mid, "flt": a1["flt"], "bias": a1["bias"]})
    if not np.array_equal(results["one"][:1], want):
        raise SystemExit("bench.py: pair output of image 0 differs from the oracle")
    n_in, n_mid, n_out = (int(np.prod(sh)) for sh in (pw.src_shape(), pw.dst_shape(), dw.dst_shape()))
    ms = out["runtime"]["us_per_forward"] * 1e-3
    moved = 2 * n_in + n_in + n_out + ic * oc + (0 if out["runtime"]["nr_kernel"] == 2 else 2 * n_mid)
    return {"metric": "hbm_gbps", "value": round(moved / (ms * 1e-3) / 1e9, 1), "unit": "GB/s", "n_gpus": 1,
            "steps": steps, "warmup": warmup, "ms_per_step": round(ms, 5), "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "int8", "data": "synthetic",
            "config": {"workload": "qsi8 ReLU -> pointwise %d->%d -> depthwise 3x3 s%d, N=%d %dx%d NCHW44 (three "
                                   "operators; the last two are the pair)" % (ic, oc, stride, batch, hw, hw)},
            "forms": out,
            "roofline": {"bound": "hbm", "achieved": round(moved / (ms * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBS,
                         "unit": "GB/s", "frac": round(moved / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4), "traffic": None,
                         "algorithmic_per_launch": moved},
            "checked": True, "checked_what": "one kernel == two kernels on every image; image 0 == oracle"}


def case_bytes(case):
    ins, outs = case.specs(case.gen(0))
    return sum(s.nbytes for s in ins) + sum(s.nbytes for s in outs)


MFMA_OPS = 2 * 32 * 32 * 32  # one v_mfma_i32_32x32x32_i8


def bench_mfma_only(mfma_per_simd, launches):
    """Launches that issue nothing but v_mfma_i32_32x32x32_i8 (operands in registers), timed by the
    library with HIP events, for three operand distributions: the board is power-limited and the
    rate depends on the operand values."""
    import ctypes
    import megcc_amd
    path = os.path.join(megcc_amd.PKG_DIR, "libmegcc_bench_probe.so")  # bench-only, not the product library
    if not os.path.exists(path):
        raise SystemExit("%s is missing: run __graft_entry__.build()" % path)
    lib = ctypes.CDLL(path)
    lib.megcc_bench_probe_mfma_i8.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                              ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double)]
    lib.megcc_bench_probe_mfma_i8.restype = ctypes.c_int
    res = {}
    for kind, name in ((1, "uniform_int8"), (0, "zeros"), (2, "relu_activations_normal_weights")):
        us, n = ctypes.c_double(), ctypes.c_double()
        st = lib.megcc_bench_probe_mfma_i8(kind, mfma_per_simd, launches, ctypes.byref(us), ctypes.byref(n))
        if st != 0:
            raise SystemExit("megcc_bench_probe_mfma_i8: status %d" % st)
        res[name] = {"us_per_launch": round(us.value, 2), "tops": round(n.value * MFMA_OPS / us.value / 1e6, 1)}
    v = res["uniform_int8"]
    return {"metric": "int8_mfma_only_tops", "value": v["tops"], "unit": "TOP/s", "n_gpus": 1, "steps": launches,
            "warmup": launches, "ms_per_step": round(v["us_per_launch"] * 1e-3, 5), "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "int8", "data": "synthetic",
            "config": {"workload": "v_mfma_i32_32x32x32_i8 only, %d per SIMD per launch (the default "
                       "workload's count), operands in registers" % mfma_per_simd,
                       "abi": "megcc_bench_probe_mfma_i8 (libmegcc_bench_probe.so, not the product library)"},
            "roofline": {"bound": "mfma", "achieved": v["tops"], "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
                         "frac": round(v["tops"] / PEAK_INT8_TOPS, 4), "traffic": None},
            **res}


def cpu_baseline(full_case, unit="TOP/s"):
    """One host core on a bounded sample of the same workload, through the reference's own
    generated kernel where oracle/_ref has it: batch 1 of a batched convolution, 64 rows of a
    FullyConnected / MatMul with more (images and rows are independent in the reference's loops,
    so the time of the whole workload is the sample's time times the stated factor)."""
    import copy
    from oracle import port, ref
    import cases
    import config_cases
    from cases import ConvCase, MatMulCase
    sample, factor, what = full_case, 1, "the whole workload"
    if isinstance(full_case, ConvCase):
        fc = full_case.fmt == 0 and full_case.fh == 1 and full_case.ih == 1
        keep = 64 if fc else 1
        if full_case.n > keep:
            sample = copy.copy(full_case)
            sample.n = keep
            factor = full_case.n / keep
            what = "%s %d of %d" % ("rows" if fc else "batch", keep, full_case.n)
    elif isinstance(full_case, MatMulCase) and full_case.m > 64:
        sample = MatMulCase(64, full_case.k, full_case.n, full_case.trans_a, full_case.trans_b)
        factor = full_case.m / 64
        what = "rows 64 of %d" % full_case.m
    arrays = sample.gen(seed=0)
    try:
        symbol = config_cases.ref_symbol(sample)
    except AssertionError:
        symbol = sample.symbol()
    use_ref = ref.available() and ref.has(symbol)
    port.set_threads(1)
    t0 = time.perf_counter()
    if use_ref:
        cases.run_ref(sample, arrays, symbol)
    else:
        sample.run_port(arrays)
    dt = time.perf_counter() - t0
    work = sample.ops() if unit != "GB/s" and hasattr(sample, "ops") else case_bytes(sample)
    return {
        "value": round(work / dt / (1e9 if unit == "GB/s" else 1e12), 6), "unit": unit, "cores": 1,
        "kind": "reference" if use_ref else "port",
        "sample": "%s, timed once in %.5f s (the whole workload at that rate: %.4g s); %s" % (
            what, dt, dt * factor,
            "MegCC's generated kernel %s built with -O3 -fno-finite-math-only" % symbol
            if use_ref else "oracle/oracle_port.c built with -O2"),
        "host_cores": os.cpu_count(),
    }


def bench_sustained(op, seconds):
    """Back-to-back launches for `seconds`, 2000 per interval: time per launch of each interval next
    to the GPU clock and board power the driver reports meanwhile (pp_dpm_sclk's current level,
    hwmon power1_average / power1_input, sampled every 0.2 s from sysfs; None where the files are
    not readable). Says whether a kernel's rate is held back by the power cap."""
    import glob
    import threading
    from megcc_amd import runtime
    samples, stop = [], [False]

    def read(path):
        try:
            with open(path) as f:
                return f.read().strip()
        except OSError:
            return None

    def sampler():
        cards = glob.glob("/sys/class/drm/card*/device")
        t0 = time.perf_counter()
        while not stop[0]:
            mhz, watts = None, None
            for c in cards:
                levels = read(c + "/pp_dpm_sclk")
                cur = [l for l in (levels or "").splitlines() if l.endswith("*")]
                if cur:
                    mhz = max(mhz or 0, int("".join(ch for ch in cur[0].split(":")[1] if ch.isdigit())))
                for h in glob.glob(c + "/hwmon/hwmon*/power1_average") + glob.glob(c + "/hwmon/hwmon*/power1_input"):
                    v = read(h)
                    if v and v.isdigit():
                        watts = max(watts or 0, int(v) / 1e6)
            samples.append((time.perf_counter() - t0, mhz, watts))
            time.sleep(0.2)

    th = threading.Thread(target=sampler)
    th.start()
    ev = HipEvents(runtime.lib().megcc_gfx950_stream())
    rows, t0 = [], time.perf_counter()
    try:
        while time.perf_counter() - t0 < seconds:
            e0, e1 = ev.new(), ev.new()
            ev.record(e0)
            for _ in range(2000):
                op.launch()
            ev.record(e1)
            runtime.wait()
            t = time.perf_counter() - t0
            near = [x for x in samples if abs(x[0] - t) < 0.3]
            rows.append({"t_s": round(t, 2), "us_per_launch": round(ev.elapsed_ms(e0, e1) / 2, 2),
                         "sclk_mhz": near[-1][1] if near else None,
                         "power_w": round(near[-1][2], 0) if near and near[-1][2] else None})
    finally:
        stop[0] = True
        th.join()
    return rows


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=500,
                    help="untimed launches first (the GPU takes a few hundred 70 us launches to "
                         "reach its sustained clocks)")
    ap.add_argument("--preheat-ms", type=float, default=300.0,
                    help="untimed launches of the same operator before the warm-up steps, for this long")
    ap.add_argument("--workload", default="conv")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--cpu", action="store_true",
                    help="time the CPU baseline for this workload too (the default workload always does)")
    ap.add_argument("--batch", type=int, default=64, help="batch of the mobilenet workload")
    ap.add_argument("--per-layer", action="store_true")
    ap.add_argument("--sustain", type=float, default=0.0,
                    help="instead of the timed steps: launch the workload back to back for this many "
                         "seconds and print time per launch, GPU clock and board power over time")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py: this build runs on ONE GPU (the path shards over the batch "
                         "dimension with no exchange step); --gpus %d is not supported" % args.gpus)

    from megcc_amd import runtime
    import numpy as np

    if args.workload == "mobilenet":
        print(json.dumps(bench_mobilenet(args.batch, args.steps, args.warmup, args.per_layer)))
        return
    if args.workload.startswith("pwdw:"):  # pwdw:N,IC,OC,HW,S
        n, ic, oc, hw, st = [int(v) for v in args.workload[5:].split(",")]
        print(json.dumps(bench_pwdw(n, ic, oc, hw, st, args.steps, args.warmup)))
        return
    if args.workload.startswith("chain"):  # chain, chain_s2, chain512, chain512_s2, chain:C,HW,S
        c, hw, st = [int(v) for v in args.workload[6:].split(",")] if args.workload.startswith("chain:") else {
            "chain": (32, 112, 1), "chain_s2": (32, 112, 2), "chain512": (512, 14, 1),
            "chain512_s2": (512, 14, 2)}[args.workload]
        print(json.dumps(bench_chain(c, hw, st, args.steps, args.warmup, cpu=args.cpu)))
        return
    if args.workload == "mfma_only":
        # as many MFMAs per SIMD as the default workload's launch has, spread evenly over 256 CUs
        print(json.dumps(bench_mfma_only(int(make_workload("conv")[0].ops() / MFMA_OPS / (4 * 256)), args.steps)))
        return
    case, desc, bound = make_workload(args.workload)
    arrays = case.gen(seed=0)
    ins, outs = case.specs(arrays)
    kdesc = case.desc() if hasattr(case, "desc") else runtime.parse_symbol(case.symbol())
    op = runtime.PreparedOp(kdesc, ins, outs)
    ev = HipEvents(runtime.lib().megcc_gfx950_stream())
    if args.sustain > 0:
        print(json.dumps({"workload": desc, "kernel": None, "sustained": bench_sustained(op, args.sustain)}))
        return

    preheat = 0
    t_heat = time.perf_counter() + args.preheat_ms * 1e-3
    while time.perf_counter() < t_heat:
        for _ in range(50):
            op.launch()
        runtime.wait()
        preheat += 50
    for _ in range(args.warmup):
        op.launch()
    runtime.wait()
    e0, e1 = ev.new(), ev.new()
    t0 = time.perf_counter()
    ev.record(e0)
    for _ in range(args.steps):
        op.launch()
    ev.record(e1)
    runtime.wait()
    wall = time.perf_counter() - t0
    kern_ms = ev.elapsed_ms(e0, e1) / args.steps
    kernel_name = runtime.last_kernel()

    # outside the timed region: what the timed launches computed, against the CPU oracle
    checked = check_output(case, arrays, op.result())
    ops = case.ops() if hasattr(case, "ops") else 0
    nbytes = case_bytes(case)
    ms = wall * 1e3 / args.steps
    if bound == "mfma_f32":
        bound = "mfma"
        value, unit, metric = ops / (wall / args.steps) / 1e12, "TFLOP/s", "f32_tflops"
        roof = {"bound": "mfma", "achieved": round(ops / (kern_ms * 1e-3) / 1e12, 3),
                "peak": 157.3, "unit": "TFLOP/s", "traffic": None}
    elif bound == "mfma":
        value, unit, metric = ops / (wall / args.steps) / 1e12, "TOP/s", "int8_conv_tops"
        roof = {"bound": "mfma", "achieved": round(ops / (kern_ms * 1e-3) / 1e12, 3),
                "peak": PEAK_INT8_TOPS, "unit": "TOP/s", "traffic": None}
    else:
        value, unit, metric = nbytes / (wall / args.steps) / 1e9, "GB/s", "hbm_gbps"
        roof = {"bound": "hbm", "achieved": round(nbytes / (kern_ms * 1e-3) / 1e9, 2),
                "peak": PEAK_HBM_GBS, "unit": "GB/s", "traffic": None}
    roof.update(traffic_fields(args.workload, nbytes, sum(sp.nbytes for sp in outs)))
    roof["frac"] = round(roof["achieved"] / roof["peak"], 4)
    roof["kernel_ms"] = round(kern_ms, 5)
    roof["algorithmic_per_launch"] = ops if bound == "mfma" else nbytes
    if args.workload == "conv":
        # what the matrix cores alone deliver on this board for the same number of MFMAs per SIMD and
        # the same operand distribution (uniform random int8): no loads, no LDS, no epilogue
        mo = bench_mfma_only(int(ops / MFMA_OPS / (4 * 256)), 300)
        roof["mfma_only_same_operands"] = {k: mo[k] for k in ("uniform_int8", "zeros")}

    out = {
        "metric": metric, "value": round(value, 3), "unit": unit, "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32" if unit == "TFLOP/s" else "int8", "data": "synthetic",
        "config": {"workload": desc, "symbol": case.symbol(), "abi": "megcc_gfx950_call",
                   "kernel": kernel_name},
        "roofline": roof,
        "checked": checked is not None, "checked_what": checked,
        "preheat_launches": preheat,
    }
    if args.cpu and args.workload != "conv":
        out["cpu_baseline"] = cpu_baseline(case, unit)
    if not args.no_cpu and args.workload == "conv":
        out["cpu_baseline"] = cpu_baseline(case)
        op = None
        mb = bench_mobilenet(64, 200, 100)
        mb1 = bench_mobilenet(1, 300, 100)
        mb256 = bench_mobilenet(256, 60, 30)
        import mobilenet
        cpu_s, used = mobilenet.Net(1).run_cpu_timed(mobilenet.draw_input(1, seed=1), threads=1)
        out["mobilenet_roofline"] = dict(mb["roofline"], workload="MobileNetV1-int8 batch 64, one forward = %d kernels (%s)" % (
            mb["nr_kernel"], mb["launch_mode"]), images_per_s=mb["images_per_s"])
        out["extra"] = {"mobilenet_v1_int8_images_per_s_batch64": mb["images_per_s"],
                        "mobilenet_v1_int8_ms_per_forward_batch64": mb["ms_per_forward"],
                        "mobilenet_v1_int8_images_per_s_batch1": mb1["images_per_s"],
                        "mobilenet_v1_int8_images_per_s_batch256": mb256["images_per_s"],
                        "mobilenet_v1_int8_cpu_images_per_s": round(1.0 / cpu_s, 4),
                        "mobilenet_v1_int8_cpu_note": "1 host core, batch 1, one forward in %.2f s: "
                        "%d operators by MegCC's generated x86 kernels, %d by the C restatement" % (
                            cpu_s, used["reference"], used["port"])}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
