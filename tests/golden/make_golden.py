#!/usr/bin/env python3
"""Writes tests/golden/golden.npz and tests/golden/symbols.json.

For every case of tests/golden_cases.py the seeded inputs are run through the REFERENCE'S OWN
generated C kernel (oracle/_ref/libmegcc_ref.so: MegCC's KernelGen compiled from /root/reference,
its Arch::BAREMETAL kernel emitted and built with the reference's kernel-test flags
`-O3 -fno-finite-math-only`, no -march / -msse4.2; see oracle/Makefile) and inputs + outputs are
stored. symbols.json records which generated kernel MegCC's registry picked for each case.

Only runs where /root/reference exists (`make -C oracle ref` first); the committed files are what
the tests use everywhere else.
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))

import cases  # noqa: E402
from golden_cases import golden_cases  # noqa: E402
from oracle import ref  # noqa: E402


def main():
    assert ref.available(), "build oracle/_ref first: make -C oracle ref"
    manifest = {}
    with open(os.path.join(os.path.dirname(ref._PATH), "gen", "manifest.txt")) as f:
        for line in f:
            label, sym = line.split()
            manifest[label] = sym
    blobs, symbols = {}, {}
    for idx, (name, case) in enumerate(golden_cases().items()):
        arrays = case.gen(seed=1000 + idx)
        sym = manifest[name]
        out = cases.run_ref(case, arrays, sym)
        for k, v in arrays.items():
            if v is not None:
                blobs["%s/%s" % (name, k)] = v
        blobs["%s/expect" % name] = out
        symbols[name] = sym
    np.savez_compressed(os.path.join(HERE, "golden.npz"), **blobs)
    with open(os.path.join(HERE, "symbols.json"), "w") as f:
        json.dump(symbols, f, indent=1, sort_keys=True)
    print("wrote %d cases, %d arrays" % (len(symbols), len(blobs)))


if __name__ == "__main__":
    main()
