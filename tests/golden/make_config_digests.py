#!/usr/bin/env python3
"""Writes tests/golden/config_digests.json and tests/golden/config_samples.npz.

Every case of tests/config_cases.py (the benchmark configurations at their own sizes) and every
layer of the batch-1 MobileNetV1-int8 forward is evaluated by the REFERENCE'S OWN generated C
kernels (oracle/_ref/libmegcc_ref.so, see oracle/Makefile); a SHA-256 of each qsi8 output and a
strided sample of each f32 output are stored. Only runs where /root/reference exists
(`make -C oracle ref` first); the committed files are what the tests use everywhere else."""
import json
import os
import sys
import time

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))

import cases  # noqa: E402
import config_cases as cc  # noqa: E402
import mobilenet  # noqa: E402
from oracle import ref  # noqa: E402


def run_ref(case, arrays):
    sym = cc.ref_symbol(case)
    assert ref.has(sym), "oracle/_ref lacks " + sym
    return cases.run_ref(case, arrays, sym)


def main():
    assert ref.available(), "build oracle/_ref first: make -C oracle ref"
    digests, samples = {}, {}

    def record(name, out, symbol):
        entry = {"shape": list(out.shape), "dtype": str(out.dtype), "kernel": symbol}
        if out.dtype == np.float32:
            samples[name] = cc.sample(out)
        else:
            entry["sha256"] = cc.digest(out)
        digests[name] = entry

    for name, (case, seed) in cc.single_cases().items():
        t0 = time.time()
        out = run_ref(case, case.gen(seed=seed))
        record(name, out, cc.ref_symbol(case))
        print("%-50s %6.1f s" % (name, time.time() - t0), flush=True)
    for c, hw, st in cc.CHAINS:
        kernels = []

        def run(case, arrays):
            kernels.append(cc.ref_symbol(case))
            return run_ref(case, arrays)

        for stage, out in cc.chain_stages(c, hw, st, run):
            record("%s/%s" % (cc.chain_name(c, hw, st), stage), out, kernels[-1])
        print(cc.chain_name(c, hw, st), flush=True)
    # MobileNetV1-int8, batch 1: every operator's output
    net = mobilenet.Net(1)
    x = mobilenet.draw_input(1, seed=5)
    for kind, name, case, _ in net.steps:
        if kind == "typecvt":
            arrays = {"src": np.ascontiguousarray(x.reshape(case.shape))}
        elif kind == "pool":
            arrays = {"src": x}
        else:
            flt, bias, _ = net.weights[name]
            if name == "fc":
                x = np.ascontiguousarray(x.reshape(1, 1024, 1, 1))
            arrays = {"src": x, "flt": flt, "bias": bias}
        x = run_ref(case, arrays)
        record("cfg5_mobilenet_b1/" + name, x, cc.ref_symbol(case))
    print("mobilenet batch 1", flush=True)
    with open(os.path.join(HERE, "config_digests.json"), "w") as f:
        json.dump(digests, f, indent=1, sort_keys=True)
    np.savez_compressed(os.path.join(HERE, "config_samples.npz"), **samples)
    print("wrote %d digests, %d f32 samples" % (len(digests), len(samples)))


if __name__ == "__main__":
    main()
