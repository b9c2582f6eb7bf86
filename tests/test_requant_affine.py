"""The one-multiply-add requantisation the library uses where its host search proves it exact:
out = clamp(floor(fma((float)acc, c, d)), lowest output, 127). The search's answer is checked
here from outside, on the CPU: the reference's literal float sequence (the oracle's convolution with
zero input, so that the accumulator is the bias) against the fused multiply-add evaluated in Python
for every accumulator around the 255 steps and on a dense range. No GPU involved."""
import json
import os

import numpy as np
import pytest

import mobilenet
from megcc_amd import abi, runtime
from oracle import port

HERE = os.path.dirname(os.path.abspath(__file__))


def literal(acc, act, scales):
    """fp32_to_int8(act(acc * s_src * s_flt / s_dst)) by the oracle's convolution: zero input,
    one output channel per accumulator, the accumulator as its bias"""
    acc = np.ascontiguousarray(acc, np.int32)
    src = np.zeros((1, 1, 1, 1), np.int8)
    flt = np.zeros((acc.size, 1, 1, 1), np.int8)
    out = port.conv(src, flt, acc, abi.FMT_NCHW, 1, acc.size, 1, 1, (1, 1), (0, 0), (1, 1), act, scales)
    return out.reshape(-1).astype(np.int32)


def affine(acc, c, d, lo):
    """the device's sequence: v_cvt_f32_i32, v_fma_f32, v_cvt_flr_i32_f32, v_med3_i32. The product of
    two float32 is exact in float64 and so is its sum with d while |product| < 4096; one rounding to
    float32 then is the fused multiply-add. Beyond that both sides clamp."""
    a32 = np.asarray(acc, np.int64).astype(np.float32)
    exact = a32.astype(np.float64) * np.float64(np.float32(c)) + np.float64(np.float32(d))
    g = np.floor(exact.astype(np.float32).astype(np.float64))
    return np.clip(g, lo, 127).astype(np.int32)


def check_pair(act, scales):
    """-> True when the library has a pair for these scales (and it is exact), False when it has none"""
    scales = tuple(float(np.float32(s)) for s in scales)
    pair = runtime.requant_affine(act, *scales)
    if pair is None:
        return False
    c, d = pair
    lo = 0 if act == abi.RELU else -128
    assert 0.0 < d < 1.0 and c > 0
    span = int(min(140.0 / c, 2.0e9))  # accumulators beyond +-span clamp on both sides
    rng = np.random.default_rng(int(c * 1e9) & 0xFFFF)
    # (the reference converts the scaled value with `int r = roundf(x)`, which is undefined from
    #  2^31 on - x86 returns INT_MIN there, the device saturates - so the range stops short of it)
    top = int(min(2**31 - 1, 2.1e9 / c))
    parts = [np.arange(-min(span, 200000), min(span, 200000) + 1, dtype=np.int64),
             rng.integers(-span, span, 200000),
             rng.integers(-top, top, 20000),
             np.array([-top, -top + 1, top - 1, top, 0, 1, -1])]
    # every accumulator within 3 of where the output changes (found on the literal sequence)
    for j in range(lo, 128):
        est = (j - 0.5) / c
        if abs(est) < 2.0e9:
            parts.append(np.arange(int(est) - 3, int(est) + 4, dtype=np.int64))
    acc = np.unique(np.clip(np.concatenate(parts), -top, top)).astype(np.int32)
    want = literal(acc, act, scales)
    got = affine(acc, c, d, lo)
    bad = np.nonzero(want != got)[0]
    assert bad.size == 0, "acc %d: literal %d, fma %d (c=%r d=%r scales=%r)" % (
        acc[bad[0]], want[bad[0]], got[bad[0]], c, d, scales)
    return True


def test_every_relu_layer_of_mobilenet_has_an_exact_pair():
    net = mobilenet.Net(1)
    found = 0
    convs = [(name, case) for kind, name, case, _ in net.steps if kind == "conv" and case.act == abi.RELU]
    for name, case in convs:
        found += check_pair(case.act, case.scales)
    assert len(convs) == 27 and found == 27, found


@pytest.mark.parametrize("act", [abi.RELU, abi.IDENTITY])
def test_random_scales_either_have_an_exact_pair_or_none(act):
    rng = np.random.default_rng(7 + act)
    found = 0
    for _ in range(60):
        scales = (rng.uniform(0.004, 0.05), rng.uniform(0.0005, 0.02), rng.uniform(0.004, 0.12))
        found += check_pair(act, scales)
    assert found >= 40, found  # (calibrated scales almost always have one)


def test_scales_with_exact_ties_on_both_sides_have_no_pair():
    """0.02 * 0.01 / 0.05: every 125th accumulator is an exact tie and the reference's three roundings
    send some of them up and some down, which no single multiply-add reproduces: such layers keep the
    threshold table. The other activations never get a pair."""
    assert runtime.requant_affine(abi.RELU, 0.02, 0.01, 0.05) is None
    assert runtime.requant_affine(abi.IDENTITY, 0.02, 0.01, 0.05) is None
    assert runtime.requant_affine(abi.H_SWISH, 0.0123, 0.0045, 0.0317) is None
    assert runtime.requant_affine(abi.SIGMOID, 0.0123, 0.0045, 0.0317) is None
    # extreme scales: the table itself is off for them
    assert runtime.requant_affine(abi.RELU, 1e-35, 0.01, 0.05) is None


def test_large_and_small_ratios():
    """ratios above 1 (several output levels per accumulator step) and tiny ones (accumulators in the
    millions): whatever the library answers must be exact"""
    for scales in [(0.5, 0.5, 0.1), (0.11, 0.73, 0.019), (0.001, 0.0007, 0.9), (0.013, 0.0021, 0.37),
                   (0.02, 0.01, 0.0371234), (1.0, 1.0, 1.0), (0.25, 0.5, 0.125)]:
        for act in (abi.RELU, abi.IDENTITY):
            check_pair(act, scales)
