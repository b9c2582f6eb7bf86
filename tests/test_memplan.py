"""Static memory plan (megcc_gfx950_plan_memory, host code): the same offsets and arena size as the
reference's PUSHDOWN allocator (compiler/lib/Dialect/Kernel/Transforms/migrate/static_mem_alloc.h,
driven as in Transforms/StaticMemoryPlanning.cpp:34-127).

Three independent anchors: plans worked out by hand, the stored answers of the reference's own
allocator (golden/memplan.json, written by golden/make_memplan.py), and - where the reference tree
is at hand - that allocator itself on fresh random requests. On top, what any valid plan must
satisfy."""
import json
import os

import numpy as np
import pytest

import memplan_cases
from megcc_amd import runtime
from oracle import ref

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "memplan.json")) as f:
    GOLDEN = json.load(f)


def check_valid(begin, end, size, alignment, off, arena, bound):
    begin, end, size = (np.asarray(a, np.int64) for a in (begin, end, size))
    n = len(begin)
    assert (off % alignment == 0).all()
    assert arena % alignment == 0
    if n:
        assert arena >= (off + size).max()
        assert arena == -(-(off + size).max() // alignment) * alignment
    assert bound <= arena
    # alive together -> no shared byte
    for i in range(n):
        together = (begin < end[i]) & (begin[i] < end)
        together[i] = False
        clash = together & (off < off[i] + size[i]) & (off[i] < off + size)
        assert not clash.any(), (i, np.nonzero(clash)[0])
    # the bound is the busiest time step
    steps = np.unique(np.concatenate([begin, end])) if n else []
    busiest = 0
    for t in steps:
        alive = (begin <= t) & (t < end)
        busiest = max(busiest, int((-(-size[alive] // alignment) * alignment).sum()))
    assert bound == busiest


@pytest.mark.parametrize("case", memplan_cases.HAND, ids=[c[0] for c in memplan_cases.HAND])
def test_plans_worked_out_by_hand(case):
    _, alignment, begin, end, size, want_off, want_arena = case
    off, arena, bound = runtime.plan_memory(begin, end, size, alignment)
    assert off.tolist() == want_off
    assert arena == want_arena
    check_valid(begin, end, size, alignment, off, arena, bound)


@pytest.mark.parametrize("case", GOLDEN, ids=[c["name"] for c in GOLDEN])
def test_same_plan_as_the_reference_allocator_stored(case):
    off, arena, bound = runtime.plan_memory(case["begin"], case["end"], case["size"], case["alignment"])
    assert off.tolist() == case["offset"]
    assert arena == case["arena"]
    assert bound == case["lower_bound"]
    check_valid(case["begin"], case["end"], case["size"], case["alignment"], off, arena, bound)


def test_fixture_covers_the_cases_it_is_made_from():
    assert [c["name"] for c in GOLDEN] == [c[0] for c in memplan_cases.fixture_cases()]


@pytest.mark.skipif(not ref.memplan_available(), reason="oracle/_ref not built (needs the reference tree)")
def test_same_plan_as_the_reference_allocator_live():
    for seed in range(1000, 1600):
        alignment, begin, end, size = memplan_cases.random_requests(seed)
        got = runtime.plan_memory(begin, end, size, alignment)
        want = ref.plan_memory(begin, end, size, alignment)
        assert got[0].tolist() == want[0].tolist(), seed
        assert got[1:] == want[1:], seed


def test_large_random_plan_is_valid():
    rng = np.random.default_rng(7)
    n = 3000
    begin = rng.integers(0, 800, n)
    end = begin + rng.integers(1, 30, n)
    size = rng.integers(1, 1 << 22, n)
    off, arena, bound = runtime.plan_memory(begin, end, size, 256)
    check_valid(begin, end, size, 256, off, arena, bound)


def test_mobilenet_chain_needs_no_more_than_its_busiest_step():
    for batch in (1, 64):
        begin, end, size = memplan_cases.mobilenet_requests(batch)
        off, arena, bound = runtime.plan_memory(begin, end, size, 256)
        assert arena == bound


def test_rejects_what_the_reference_asserts_on():
    with pytest.raises(runtime.MegccError):
        runtime.plan_memory([0], [1], [8], alignment=3)
    with pytest.raises(runtime.MegccError):
        runtime.plan_memory([2], [2], [8], alignment=1)
    off, arena, bound = runtime.plan_memory([], [], [], 64)
    assert len(off) == 0 and arena == 0 and bound == 0
