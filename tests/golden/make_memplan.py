"""Writes tests/golden/memplan.json: memory-plan requests with the offsets, arena size and lower
bound the REFERENCE's allocator gives for them (its sources compiled into
oracle/_ref/libmegcc_ref_memplan.so by `make -C oracle ref`; runs only where /root/reference is).
The fixture is what the planner tests compare with on a machine without the reference.

    python tests/golden/make_memplan.py
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, os.path.dirname(HERE))

from oracle import ref  # noqa: E402
import memplan_cases  # noqa: E402


def main():
    out = []
    for name, alignment, begin, end, size in memplan_cases.fixture_cases():
        off, arena, bound = ref.plan_memory(begin, end, size, alignment)
        out.append(dict(name=name, alignment=alignment, begin=list(map(int, begin)),
                        end=list(map(int, end)), size=list(map(int, size)),
                        offset=off.tolist(), arena=arena, lower_bound=bound))
    path = os.path.join(HERE, "memplan.json")
    with open(path, "w") as f:
        json.dump(out, f, separators=(",", ":"))
    print("%d cases -> %s (%d bytes)" % (len(out), path, os.path.getsize(path)))


if __name__ == "__main__":
    main()
