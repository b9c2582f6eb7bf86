"""megcc_gfx950_conv2d_noalloc against megcc_gfx950_conv2d: same layer, same device tensors, the
library's static scratch array in place of the caller's workspace. Each pair of layers runs back
to back, the second smaller than the first, so the second finds the first one's partial sums (or
gathered pixels, or NCHW44 copies) still in the array."""
import ctypes as C

import numpy as np
import pytest

from cases import ConvCase
from golden_cases import unsat
from megcc_amd import abi, runtime

pytestmark = pytest.mark.gpu
A = abi
SCRATCH = 32 << 20

PAIRS = [
    # FullyConnected with 64 rows and a long K under few output channels: K slices in separate
    # workgroups, 1 MiB of int32 partial sums; then a smaller one
    ("fc_stream",
     ConvCase(A.FMT_NCHW, A.DENSE, 64, 16384, 1, 1, 256, 1, 1, 0, A.IDENTITY, scales=(0.01, 0.01, unsat(16384) / 2)),
     ConvCase(A.FMT_NCHW, A.DENSE, 64, 1024, 1, 1, 1000, 1, 1, 0, A.RELU, scales=(0.01, 0.01, unsat(1024) / 2))),
    # split-K of the one-stage kernel (few pixels, long K)
    ("conv_mfma_i8",
     ConvCase(A.FMT_NCHW44, A.DENSE, 2, 512, 14, 14, 512, 3, 2, 1, A.RELU, scales=(0.02, 0.01, unsat(4608))),
     ConvCase(A.FMT_NCHW44, A.DENSE, 1, 256, 7, 7, 256, 3, 1, 1, A.IDENTITY, scales=(0.02, 0.01, unsat(2304)))),
    # 1x1 with a stride: the gathered pixels (without scratch this layer is an error)
    ("conv_pw_stream",
     ConvCase(A.FMT_NCHW44, A.DENSE, 4, 64, 56, 56, 128, 1, 2, 0, A.IDENTITY, scales=(0.02, 0.01, unsat(64))),
     ConvCase(A.FMT_NCHW44, A.DENSE, 2, 16, 9, 9, 8, 1, 2, 0, A.RELU, scales=(0.02, 0.01, unsat(16)))),
    # dense layer on plain NCHW tensors: two NCHW44 copies around the matrix-core kernel
    ("conv_mfma_i8_dma",
     ConvCase(A.FMT_NCHW, A.DENSE, 8, 64, 56, 56, 64, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(576))),
     ConvCase(A.FMT_NCHW, A.DENSE, 2, 16, 20, 24, 12, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(144)))),
    # channel-wise layer on plain NCHW tensors whose rows are no multiple of 4 pixels
    ("dwconv44 between NCHW relayouts",
     ConvCase(A.FMT_NCHW, A.GROUP, 4, 32, 56, 54, 32, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(9))),
     ConvCase(A.FMT_NCHW, A.GROUP, 3, 16, 29, 31, 16, 3, 2, 1, A.IDENTITY, scales=(0.02, 0.01, unsat(9)))),
    # f32 layer in NCHW44: NCHW copies of input, output and filter around the implicit GEMM
    ("conv_f32_gemm between NCHW44 relayouts",
     ConvCase(A.FMT_NCHW44, A.DENSE, 2, 64, 28, 28, 64, 3, 1, 1, A.RELU, dtype="f32"),
     ConvCase(A.FMT_NCHW44, A.DENSE, 1, 16, 9, 7, 8, 1, 1, 0, A.IDENTITY, dtype="f32")),
    # f32 layer with few tiles: f32 partial sums of a split of K
    ("conv_f32_gemm",
     ConvCase(A.FMT_NCHW, A.DENSE, 4, 64, 56, 56, 64, 3, 1, 1, A.RELU, dtype="f32"),
     ConvCase(A.FMT_NCHW, A.DENSE, 3, 40, 57, 55, 72, 3, 2, 1, A.H_SWISH, dtype="f32")),
]


def prepared(case, seed):
    arrays = case.gen(seed)
    ins, outs = case.specs(arrays)
    return runtime.PreparedOp(runtime.parse_symbol(case.symbol()), ins, outs)


@pytest.mark.parametrize("kernel,big,small", PAIRS, ids=[p[0].replace(" ", "_") for p in PAIRS])
def test_noalloc_equals_conv2d_on_two_calls_in_a_row(kernel, big, small):
    ops = [prepared(big, 71), prepared(small, 72)]
    want = []
    picked = []
    for op in ops:  # the existing entry point, with the workspace its _workspace call asked for
        op.launch()
        want.append(op.result().copy())
        picked.append(runtime.last_kernel())
        assert 0 < op.ws.size <= SCRATCH, "the layer must use scratch memory that fits the array"
        op.poison_outputs()
    assert picked[0].startswith(kernel), picked  # (the kernel the larger layer is meant to reach)
    for op, same in zip(ops, picked):  # back to back, no synchronisation in between
        op.launch_noalloc()
        assert runtime.last_kernel() == same, (runtime.last_kernel(), same)
    for op, w, case in zip(ops, want, (big, small)):
        got = op.result()
        assert got.dtype == w.dtype and np.array_equal(got, w), repr(case)
    # and once more the other way round (small first): the array now holds the big layer's bytes
    for op in reversed(ops):
        op.poison_outputs()
        op.launch_noalloc()
    for op, w in zip(ops, want):
        assert np.array_equal(op.result(), w)


def test_noalloc_rejects_layers_beyond_the_array():
    # N=64 C=128 56x56 on plain NCHW tensors: two 25.7 MB copies do not fit 32 MiB
    case = ConvCase(A.FMT_NCHW, A.DENSE, 64, 128, 56, 56, 128, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(1152)))
    op = prepared(case, 73)
    assert op.ws.size > SCRATCH
    with pytest.raises(runtime.MegccError) as err:
        op.launch_noalloc()
    assert "TinyNNStatus %d" % abi.ERROR_OUT_OF_RANGE in str(err.value) and "scratch" in str(err.value)
    op.launch()  # the entry point with a workspace still takes it
    runtime.wait()


def test_noalloc_runs_layers_whose_optional_scratch_exceeds_the_array_without_it():
    """scratch that only buys speed (relayout detour of a channel-wise NCHW layer, split-K partial
    sums of a skinny f32 layer) is done without when it does not fit, like megcc_gfx950_conv2d does
    when it gets no workspace"""
    # rows of 110 pixels: the detour would need two 18.9 MB NCHW44 copies
    case = ConvCase(A.FMT_NCHW, A.GROUP, 48, 32, 112, 110, 32, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(9)))
    op = prepared(case, 75)
    assert op.ws.size > SCRATCH
    op.launch()
    want = op.result().copy()
    op.poison_outputs()
    op.launch_noalloc()
    assert np.array_equal(op.result(), want)
    # 9 tiles x 57 K slices x 64 KiB of f32 partial sums = 33.6 MB
    case = ConvCase(A.FMT_NCHW, A.DENSE, 1, 512, 8, 16, 1152, 3, 1, 1, A.RELU, dtype="f32")
    op = prepared(case, 76)
    assert op.ws.size > SCRATCH
    op.launch()
    want = op.result().copy()
    op.poison_outputs()
    op.launch_noalloc()
    import cases
    assert cases.max_rel_err(op.result(), want) <= 1e-4


def test_noalloc_layers_without_scratch_run_as_before():
    case = ConvCase(A.FMT_NCHW44, A.DENSE, 8, 64, 56, 56, 128, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(576)))
    op = prepared(case, 74)
    assert op.ws.size == 0
    op.launch()
    want = op.result().copy()
    op.poison_outputs()
    op.launch_noalloc()
    assert np.array_equal(op.result(), want)
