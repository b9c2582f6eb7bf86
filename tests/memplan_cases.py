"""Memory-plan requests for the planner tests: hand-made ones whose answer can be worked out on
paper, the MobileNetV1 model's, and seeded random ones."""
import numpy as np


def random_requests(seed, n_max=60, t_max=40):
    """(alignment, begin, end, size); three size regimes so that ties between equal holes, byte
    sizes that never line up and tensor-like sizes all occur. Sizes are >= 1: the reference's
    self-check aborts on some plans with empty requests."""
    rng = np.random.default_rng(seed)
    n = int(rng.integers(0, n_max))
    t = int(rng.integers(1, t_max))
    begin = rng.integers(0, t, n)
    end = begin + rng.integers(1, 8, n)
    kind = seed % 3
    if kind == 0:
        size = rng.integers(1, 5, n)
    elif kind == 1:
        size = rng.integers(1, 100000, n)
    else:
        size = rng.choice([64, 128, 256, 1000, 4096], n)
    alignment = int(rng.choice([1, 4, 64, 256]))
    return alignment, begin, end, size


# name, alignment, begin, end, size, expected offsets, expected arena: small enough to follow the
# best-fit / stretch / push-down steps by hand
HAND = [
    # nothing alive together: everything at 0
    ("disjoint", 1, [0, 1, 2], [1, 2, 3], [10, 30, 20], [0, 0, 0], 30),
    # all alive together: stacked in the order added
    ("stack", 1, [0, 0, 0], [5, 5, 5], [10, 30, 20], [0, 10, 40], 60),
    # alignment rounds every offset and the arena up
    ("stack_aligned", 16, [0, 0, 0], [5, 5, 5], [10, 30, 20], [0, 16, 48], 80),
    # a chain a->b->c: a dies when c is born, c (larger than a) stretches a's hole below b, so b is
    # pushed up to c's end
    ("chain_stretch", 1, [0, 1, 2], [2, 3, 4], [10, 20, 15], [0, 15, 0], 35),
    # chain where c fits into a's hole: b stays where a ended
    ("chain_fit", 1, [0, 1, 2], [2, 3, 4], [10, 20, 5], [0, 10, 0], 30),
    # best fit: two holes (8 under, 4 between), a 3-byte request takes the 4-byte one
    ("best_fit", 1, [0, 0, 0, 0, 1], [1, 9, 1, 9, 9], [8, 2, 4, 2, 3], [0, 8, 10, 14, 10], 16),
]


def mobilenet_requests(batch):
    import mobilenet
    net = mobilenet.Net(batch)
    lt = mobilenet.Lifetimes()
    net.build_gpu(model=lt)
    _, begin, end, size = lt.requests()
    return begin, end, size


def fixture_cases():
    """(name, alignment, begin, end, size) of every case stored in golden/memplan.json"""
    for name, alignment, begin, end, size, _, _ in HAND:
        yield name, alignment, begin, end, size
    for batch in (1, 64):
        begin, end, size = mobilenet_requests(batch)
        for alignment in (1, 256):
            yield "mobilenet_b%d_a%d" % (batch, alignment), alignment, begin, end, size
    for seed in range(48):
        alignment, begin, end, size = random_requests(seed, n_max=40)
        yield "random_%d" % seed, alignment, begin, end, size
