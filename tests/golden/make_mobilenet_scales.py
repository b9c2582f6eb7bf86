#!/usr/bin/env python3
"""Writes tests/golden/mobilenet_scales.json: the output scale of every conv / FC layer of the
random-weight MobileNetV1 of tests/mobilenet.py (weights from seed 0), chosen layer by layer on
one seeded image so that the 99.9th percentile of the layer's output lands near 110 of 127 -- the
activations then exercise the requantisation instead of saturating to a constant. Uses the CPU
oracle only."""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import mobilenet  # noqa: E402
from megcc_amd import abi  # noqa: E402
from oracle import port  # noqa: E402


def main():
    port.set_threads(8)
    weights = mobilenet.draw_weights(0)
    x = mobilenet.draw_input(1, 0)
    x = port.typecvt(x, "f32", "qsi8", dst_scale=mobilenet.IN_SCALE)
    s_in = mobilenet.IN_SCALE
    scales = {}
    for name, case in mobilenet.conv_layers(1):
        flt, bias, wscale = weights[name]
        if name == "fc":
            x = port.pool_q8(x, abi.FMT_NCHW44, abi.POOL_AVERAGE, (7, 7), (7, 7), (0, 0))
            x = np.ascontiguousarray(x.reshape(1, 1024, 1, 1))
        k = (case.ic // case.groups) * 9 if case.fh == 3 else case.ic
        probe = s_in * wscale * 40.0 * 74.0 * (k ** 0.5) * 4 / 127
        for _ in range(12):
            case.scales = (s_in, wscale, probe)
            y = case.run_port({"src": x, "flt": flt, "bias": bias})
            a = np.abs(y.astype(np.int32)).reshape(-1)
            p = float(np.percentile(a, 99.9))
            if a.max() >= 127 and p >= 120:
                probe *= 3
            elif p < 40:
                probe *= max(p, 1.0) / 110.0
            else:
                break
        final = probe * p / 110.0
        # keep the activation scales of the whole net in the same decade: rescale the filter scale
        # (and with it the output scale) so that the output scale is near the input scale
        jitter = 0.7 + 0.7 * ((sum(map(ord, name)) * 31 % 97) / 96.0)
        wnew = float(np.float32(wscale * s_in / final * jitter))
        final = float(np.float32(final * wnew / wscale))
        wscale = wnew
        case.scales = (s_in, wscale, final)
        x = case.run_port({"src": x, "flt": flt, "bias": bias})
        print("%-6s k=%5d scale %.6g  max %d  nonzero %.2f" % (
            name, k, final, np.abs(x.astype(np.int32)).max(), float((x != 0).mean())))
        scales[name] = {"filter": wscale, "dst": final}
        s_in = final
    with open(mobilenet.SCALES_PATH, "w") as f:
        json.dump(scales, f, indent=1)


if __name__ == "__main__":
    main()
