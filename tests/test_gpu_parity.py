"""GPU parity tests: every operator is called through the C ABI (megcc_gfx950_call on the
reference's own kernel symbol, after the workspace / three-phase-init protocol) and compared with
  * the committed outputs of the reference's generated C kernels (tests/golden/),
  * the CPU oracle on larger seeded cases,
bit-exact for qsi8, max |a-b|/max(1,min(|a|,|b|)) <= 1e-4 for f32."""
import json
import os

import numpy as np
import pytest

import cases
from cases import (ConcatCase, ConvCase, ElemwiseCase, FusedCase, MatMulCase, MultiTypeCase, PoolCase,
                   ReduceCase, RelayoutCase, ResizeCase, TypeCvtCase)
from golden_cases import golden_cases, unsat
from megcc_amd import abi, runtime
from oracle import port

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
F32_TOL = 1e-4
CASES = golden_cases()


@pytest.fixture(scope="module")
def golden():
    gold = np.load(os.path.join(HERE, "golden", "golden.npz"))
    with open(os.path.join(HERE, "golden", "symbols.json")) as f:
        return gold, json.load(f)


def compare(got, want, what):
    assert got.shape == want.shape and got.dtype == want.dtype, what
    if got.dtype == np.float32:
        err = cases.max_rel_err(got, want)
        assert err <= F32_TOL, "%s: max rel err %g" % (what, err)
    else:
        bad = np.flatnonzero(got.reshape(-1) != want.reshape(-1))
        assert bad.size == 0, "%s: %d of %d differ, first at %d: got %d want %d" % (
            what, bad.size, got.size, bad[0], got.reshape(-1)[bad[0]], want.reshape(-1)[bad[0]])


def run_gpu(case, arrays, symbol=None):
    print("GPU case:", repr(case), flush=True)
    ins, outs = case.specs(arrays)
    if hasattr(case, "desc"):  # fused elementwise: the symbol does not say which value feeds which step
        op = runtime.PreparedOp(case.desc(), ins, outs)
        op.launch()
        return op.result()
    return runtime.run_symbol(symbol or case.symbol(), ins, outs)


@pytest.mark.parametrize("name", sorted(CASES))
def test_matches_reference_golden(name, golden):
    gold, symbols = golden
    case = CASES[name]
    arrays = {k: (gold["%s/%s" % (name, k)] if "%s/%s" % (name, k) in gold.files else None)
              for k in case.gen(0).keys()}
    got = run_gpu(case, arrays, symbols[name])
    compare(got, gold[name + "/expect"], name)


A = abi
LIVE = [
    # FullyConnected on the LDS-direct kernel, row-major output in 16-byte pieces: the 256 x 256 tile whose
    # rows leave through LDS (ragged rows, a partial channel tile of 32), the 128-channel tile, and a K
    # that is no multiple of 128 (dword activation loads); 2040 outputs (no multiple of 32): dword stores
    ConvCase(A.FMT_NCHW, A.DENSE, 2100, 256, 1, 1, 288, 1, 1, 0, A.RELU, scales=(0.02, 0.01, unsat(256))),
    ConvCase(A.FMT_NCHW, A.DENSE, 2100, 256, 1, 1, 160, 1, 1, 0, A.IDENTITY, scales=(0.0213, 0.0097, unsat(256) * 1.0371)),
    ConvCase(A.FMT_NCHW, A.DENSE, 2100, 160, 1, 1, 320, 1, 1, 0, A.IDENTITY, scales=(0.02, 0.01, unsat(160))),
    ConvCase(A.FMT_NCHW, A.DENSE, 2100, 256, 1, 1, 2040, 1, 1, 0, A.H_SWISH, scales=(0.02, 0.01, unsat(256))),
    # 512-pixel sub-tiles of the plane-major 3x3 kernel: ragged channel tile, three chunks of input
    # channels, rows of 60 pixels; one channel tile (512-pixel sub-tiles from 57 600 pixels on)
    ConvCase(A.FMT_NCHW44, A.DENSE, 9, 96, 56, 60, 200, 3, 1, 1, A.H_SWISH, scales=(0.02, 0.01, unsat(864))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 20, 32, 56, 56, 128, 3, 1, 1, A.IDENTITY, scales=(0.02, 0.01, unsat(288))),
    # headline kernel at its real channel counts (spatial size cut so the oracle stays fast)
    ConvCase(A.FMT_NCHW44, A.DENSE, 2, 64, 56, 56, 64, 3, 1, 1, A.RELU, scales=(0.02, 0.01, 0.05)),
    ConvCase(A.FMT_NCHW44, A.DENSE, 2, 64, 56, 56, 64, 3, 1, 1, A.IDENTITY, scales=(0.02, 0.01, unsat(576))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 1, 256, 28, 28, 256, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(2304))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 3, 256, 14, 14, 256, 3, 1, 1, A.IDENTITY, scales=(0.02, 0.01, 0.05)),
    # ragged: pixel count not a multiple of the 128-pixel tile, oc not a multiple of 64, ic % 32 != 0
    ConvCase(A.FMT_NCHW44, A.DENSE, 3, 40, 13, 17, 72, 3, 1, 1, A.H_SWISH, scales=(0.02, 0.01, unsat(360))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 2, 36, 15, 9, 200, 3, 2, 1, A.RELU, scales=(0.02, 0.01, unsat(324))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 5, 24, 7, 7, 32, 3, 1, 1, A.SIGMOID, scales=(0.02, 0.01, unsat(216) * 40)),
    ConvCase(A.FMT_NCHW44, A.DENSE, 1, 8, 30, 31, 8, 3, 1, 0, A.IDENTITY, scales=(0.02, 0.01, unsat(72))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 1, 16, 20, 20, 16, 3, 1, 2, A.RELU, scales=(0.02, 0.01, unsat(144)), dilate=2),
    # large enough for the software-pipelined kernel (256x256 and 128x256 tiles), ragged edges
    ConvCase(A.FMT_NCHW44, A.DENSE, 6, 32, 56, 56, 160, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(288))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 6, 64, 55, 57, 256, 3, 1, 1, A.IDENTITY, scales=(0.02, 0.01, unsat(576))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 11, 36, 56, 56, 128, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(324))),
    # several 256-pixel sub-tiles per workgroup and three channel stages (pipelined across sub-tiles)
    ConvCase(A.FMT_NCHW44, A.DENSE, 24, 96, 56, 56, 128, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(864))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 21, 32, 60, 52, 136, 3, 1, 1, A.H_SWISH, scales=(0.02, 0.01, unsat(288))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 6, 136, 56, 56, 264, 1, 1, 0, A.RELU, scales=(0.02, 0.01, unsat(136))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 11, 64, 56, 56, 128, 1, 1, 0, A.IDENTITY, scales=(0.02, 0.01, unsat(64))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 70, 256, 14, 14, 512, 1, 1, 0, A.RELU, scales=(0.02, 0.01, unsat(256))),
    ConvCase(A.FMT_NCHW, A.DENSE, 16500, 96, 1, 1, 200, 1, 1, 0, A.RELU, scales=(0.01, 0.01, unsat(96) / 2)),
    # FullyConnected with an output width that is not a multiple of 4 (byte stores) and K % 128 != 0
    ConvCase(A.FMT_NCHW, A.DENSE, 9000, 160, 1, 1, 130, 1, 1, 0, A.IDENTITY, scales=(0.01, 0.01, unsat(160) / 2)),
    ConvCase(A.FMT_NCHW, A.DENSE, 8300, 260, 1, 1, 256, 1, 1, 0, A.SIGMOID, scales=(0.01, 0.01, unsat(260) / 2)),
    # few images at 56x56: between the small-layer tiles and a full grid (half-filled 256-pixel tiles)
    ConvCase(A.FMT_NCHW44, A.DENSE, 3, 64, 56, 56, 128, 1, 1, 0, A.RELU, scales=(0.02, 0.01, unsat(64))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 3, 32, 56, 56, 128, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(288))),
    # MobileNet pointwise shapes
    ConvCase(A.FMT_NCHW44, A.DENSE, 2, 32, 112, 112, 64, 1, 1, 0, A.RELU, scales=(0.02, 0.01, unsat(32))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 4, 512, 14, 14, 512, 1, 1, 0, A.RELU, scales=(0.02, 0.01, unsat(512))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 16, 512, 14, 14, 1024, 1, 1, 0, A.RELU, scales=(0.02, 0.01, unsat(512))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 5, 32, 56, 56, 64, 1, 1, 0, A.IDENTITY, scales=(0.02, 0.01, unsat(32))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 3, 1024, 7, 7, 1024, 1, 1, 0, A.RELU, scales=(0.02, 0.01, unsat(1024))),
    # FullyConnected = 1x1 NCHW conv on [M,K,1,1]
    ConvCase(A.FMT_NCHW, A.DENSE, 64, 1024, 1, 1, 1000, 1, 1, 0, A.IDENTITY, scales=(0.01, 0.01, unsat(1024) / 2)),
    ConvCase(A.FMT_NCHW, A.DENSE, 1, 1024, 1, 1, 1000, 1, 1, 0, A.IDENTITY, scales=(0.01, 0.01, 0.1)),
    ConvCase(A.FMT_NCHW, A.DENSE, 200, 512, 1, 1, 333, 1, 1, 0, A.RELU, scales=(0.01, 0.01, unsat(512) / 2)),
    # at most 64 rows, K a multiple of 128: one launch, eight K slices per workgroup (one block of
    # K: seven idle waves; 8192: the ring of filter chunks is refilled; rows short of 32 / 64;
    # channel counts that are no multiple of 4 or 32; every activation; no bias)
    ConvCase(A.FMT_NCHW, A.DENSE, 5, 128, 1, 1, 37, 1, 1, 0, A.RELU, scales=(0.01, 0.01, unsat(128) / 2)),
    ConvCase(A.FMT_NCHW, A.DENSE, 33, 384, 1, 1, 290, 1, 1, 0, A.H_SWISH, scales=(0.01, 0.01, unsat(384) / 2)),
    ConvCase(A.FMT_NCHW, A.DENSE, 32, 1152, 1, 1, 64, 1, 1, 0, A.SIGMOID, scales=(0.01, 0.01, unsat(1152) / 2)),
    ConvCase(A.FMT_NCHW, A.DENSE, 61, 8192, 1, 1, 96, 1, 1, 0, A.IDENTITY, scales=(0.01, 0.01, unsat(8192) / 2),
             bias=False),
    ConvCase(A.FMT_NCHW, A.DENSE, 17, 2048, 1, 1, 1001, 1, 1, 0, A.IDENTITY, scales=(0.01, 0.01, unsat(2048) / 2)),
    # (more channel tiles than half the CUs: one workgroup of 64 rows per tile instead of two of 32)
    ConvCase(A.FMT_NCHW, A.DENSE, 40, 256, 1, 1, 4200, 1, 1, 0, A.RELU, scales=(0.01, 0.01, unsat(256) / 2)),
    # 3x3 layers with 64..127 output channels on the LDS-direct kernel (64-channel tiles, one of them ragged)
    ConvCase(A.FMT_NCHW44, A.DENSE, 2, 64, 40, 40, 64, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(576))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 9, 32, 31, 29, 96, 3, 1, 1, A.IDENTITY, scales=(0.02, 0.01, unsat(288))),
    # 3x3 stride 2 on the LDS-direct kernel: 128-pixel sub-tiles (ragged rows, sub-tiles that cross
    # images), 256-pixel sub-tiles on a large layer, a ragged last channel tile, the literal epilogue
    ConvCase(A.FMT_NCHW44, A.DENSE, 11, 64, 30, 27, 128, 3, 2, 1, A.RELU, scales=(0.02, 0.01, unsat(576))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 40, 32, 57, 60, 160, 3, 2, 1, A.IDENTITY, scales=(0.02, 0.01, unsat(288))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 16, 96, 28, 28, 136, 3, 2, 1, A.H_SWISH, scales=(0.02, 0.01, unsat(864))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 64, 128, 14, 14, 128, 3, 2, 1, A.RELU, scales=(0.02, 0.01, 0.05)),
    # split-K of the one-stage kernel where the stages do not divide by the split asked for
    # (8 stages, 100 tiles -> 6 slices asked, 4 slices of 2 stages run)
    ConvCase(A.FMT_NCHW44, A.DENSE, 1, 256, 56, 56, 256, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(2304))),
    # small pointwise layers on the streaming kernel: fewer pixels than one tile per wave, ragged tile
    ConvCase(A.FMT_NCHW44, A.DENSE, 1, 256, 7, 7, 512, 1, 1, 0, A.RELU, scales=(0.02, 0.01, unsat(256))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 3, 64, 5, 9, 192, 1, 1, 0, A.IDENTITY, scales=(0.02, 0.01, unsat(64))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 2, 512, 14, 14, 64, 1, 1, 0, A.RELU, scales=(0.02, 0.01, unsat(512))),
    # FullyConnected with K % 128 == 0: 16-byte activation loads, swizzled LDS rows, ragged M and N
    ConvCase(A.FMT_NCHW, A.DENSE, 2500, 384, 1, 1, 200, 1, 1, 0, A.RELU, scales=(0.01, 0.01, unsat(384) / 2)),
    ConvCase(A.FMT_NCHW, A.DENSE, 4099, 256, 1, 1, 131, 1, 1, 0, A.IDENTITY, scales=(0.01, 0.01, unsat(256) / 2)),
    ConvCase(A.FMT_NCHW, A.DENSE, 2600, 256, 1, 1, 300, 1, 1, 0, A.RELU, scales=(0.01, 0.01, unsat(256) / 2)),  # 256-row tiles
    # depthwise, pooling, elemwise chain of the bandwidth-bound config
    ConvCase(A.FMT_NCHW44, A.GROUP, 2, 32, 112, 112, 32, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(9))),
    ConvCase(A.FMT_NCHW44, A.GROUP, 2, 32, 112, 112, 32, 3, 2, 1, A.RELU, scales=(0.02, 0.01, 0.05)),
    ConvCase(A.FMT_NCHW44, A.GROUP, 3, 512, 14, 14, 512, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(9))),
    ConvCase(A.FMT_NCHW44, A.GROUP, 3, 512, 14, 14, 512, 3, 2, 1, A.IDENTITY, scales=(0.02, 0.01, unsat(9))),
    ConvCase(A.FMT_NCHW, A.GROUP, 2, 32, 28, 28, 32, 3, 2, 1, A.RELU, scales=(0.02, 0.01, unsat(9))),
    # dot4 depthwise kernel: ragged rows (OW % 4 != 0), odd heights, every activation
    ConvCase(A.FMT_NCHW44, A.GROUP, 3, 16, 9, 28, 16, 3, 1, 1, A.IDENTITY, scales=(0.02, 0.01, unsat(9))),
    ConvCase(A.FMT_NCHW44, A.GROUP, 2, 8, 11, 20, 8, 3, 2, 1, A.H_SWISH, scales=(0.02, 0.01, unsat(9))),
    ConvCase(A.FMT_NCHW44, A.GROUP, 2, 24, 13, 12, 24, 3, 2, 1, A.RELU, scales=(0.02, 0.01, unsat(9))),
    ConvCase(A.FMT_NCHW44, A.GROUP, 1, 4, 5, 4, 4, 3, 1, 1, A.SIGMOID, scales=(0.02, 0.01, unsat(9) * 40)),
    ConvCase(A.FMT_NCHW44, A.GROUP, 5, 12, 7, 7, 12, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(9))),
    # stride 1 on the matrix cores: rows that are not a multiple of 4 / 8 pixels (masked loads,
    # dword stores), an odd number of plane sets, one pixel group per row, no bias, the literal
    # epilogue, 13 rows x 3 groups x 2 images = 78 columns (a ragged last tile)
    ConvCase(A.FMT_NCHW44, A.GROUP, 2, 20, 13, 18, 20, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(9))),
    ConvCase(A.FMT_NCHW44, A.GROUP, 3, 12, 6, 5, 12, 3, 1, 1, A.IDENTITY, scales=(0.02, 0.01, unsat(9)), bias=False),
    ConvCase(A.FMT_NCHW44, A.GROUP, 1, 36, 17, 33, 36, 3, 1, 1, A.H_SWISH, scales=(0.02, 0.01, unsat(9))),
    ConvCase(A.FMT_NCHW44, A.GROUP, 7, 4, 3, 1, 4, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(9))),
    ConvCase(A.FMT_NCHW44, A.GROUP, 2, 8, 1, 40, 8, 3, 1, 1, A.IDENTITY, scales=(0.5, 0.5, 0.5)),
    # pointwise layers with any channel counts on the streaming kernel: input channels below the next
    # power of two of 32-channel chunks (planes beyond IC are not fetched), output channels that do
    # not fill the last wave's 64 / 32, one channel group in and out, with a stride (gathered pixels)
    ConvCase(A.FMT_NCHW44, A.DENSE, 3, 24, 28, 28, 144, 1, 1, 0, A.RELU, scales=(0.02, 0.01, unsat(24))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 3, 144, 28, 28, 24, 1, 1, 0, A.IDENTITY, scales=(0.02, 0.01, unsat(144))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 2, 16, 19, 23, 96, 1, 1, 0, A.H_SWISH, scales=(0.02, 0.01, unsat(16))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 2, 160, 7, 7, 960, 1, 1, 0, A.RELU, scales=(0.02, 0.01, unsat(160))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 2, 384, 14, 14, 68, 1, 1, 0, A.IDENTITY, scales=(0.02, 0.01, unsat(384)), bias=False),
    ConvCase(A.FMT_NCHW44, A.DENSE, 5, 4, 9, 11, 4, 1, 1, 0, A.SIGMOID, scales=(0.02, 0.01, unsat(4) * 40)),
    ConvCase(A.FMT_NCHW44, A.DENSE, 2, 40, 31, 29, 80, 1, 2, 0, A.RELU, scales=(0.02, 0.01, unsat(40))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 1, 320, 10, 10, 1024, 1, 1, 0, A.RELU, scales=(0.02, 0.01, unsat(320))),
    # dense 5x5 / 7x7 in NCHW44, one filter row per stage of the LDS-direct kernel: half a chunk of
    # input channels, two chunks with a ragged second one, stride 2 (128-pixel sub-tiles), dilation,
    # 64- and 128-channel tiles with ragged channel counts, every activation, no bias
    ConvCase(A.FMT_NCHW44, A.DENSE, 6, 32, 28, 28, 64, 5, 1, 2, A.RELU, scales=(0.02, 0.01, unsat(800))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 6, 16, 56, 56, 128, 5, 2, 2, A.IDENTITY, scales=(0.02, 0.01, unsat(400))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 5, 40, 30, 34, 136, 7, 1, 3, A.H_SWISH, scales=(0.02, 0.01, unsat(1960))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 6, 64, 57, 55, 72, 7, 2, 3, A.RELU, scales=(0.02, 0.01, unsat(3136)), bias=False),
    ConvCase(A.FMT_NCHW44, A.DENSE, 5, 32, 31, 33, 36, 5, 1, 4, A.SIGMOID, scales=(0.02, 0.01, unsat(800) * 40), dilate=2),
    ConvCase(A.FMT_NCHW44, A.DENSE, 3, 8, 40, 300, 32, 5, 1, 2, A.IDENTITY, scales=(0.02, 0.01, unsat(200))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 17, 32, 28, 28, 64, 5, 1, 0, A.RELU, scales=(0.02, 0.01, unsat(800))),
    # H_SWISH through the threshold table in the pointwise kernels (streaming: 64 and 256 input
    # channels; workgroup-shared: 512) and the plane-major 3x3 kernel
    ConvCase(A.FMT_NCHW44, A.DENSE, 3, 64, 28, 28, 128, 1, 1, 0, A.H_SWISH, scales=(0.02, 0.01, unsat(64))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 2, 256, 14, 14, 64, 1, 1, 0, A.H_SWISH, scales=(0.02, 0.01, unsat(256))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 24, 512, 14, 14, 512, 1, 1, 0, A.H_SWISH, scales=(0.02, 0.01, unsat(512))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 4, 64, 56, 56, 128, 3, 1, 1, A.H_SWISH, scales=(0.02, 0.01, unsat(576))),
    # 5x5 (pad 2) and 7x7 (pad 3) on the matrix cores, stride 1 and 2: rows of whole pixel groups,
    # ragged rows (masked loads, dword stores), images smaller than the filter, every activation,
    # no bias, an odd number of plane sets
    ConvCase(A.FMT_NCHW44, A.GROUP, 2, 24, 28, 28, 24, 5, 1, 2, A.RELU, scales=(0.02, 0.01, unsat(25))),
    ConvCase(A.FMT_NCHW44, A.GROUP, 2, 16, 56, 56, 16, 5, 2, 2, A.RELU, scales=(0.02, 0.01, 0.05)),
    ConvCase(A.FMT_NCHW44, A.GROUP, 3, 12, 14, 14, 12, 5, 1, 2, A.H_SWISH, scales=(0.02, 0.01, unsat(25))),
    ConvCase(A.FMT_NCHW44, A.GROUP, 2, 20, 13, 19, 20, 5, 1, 2, A.IDENTITY, scales=(0.02, 0.01, unsat(25))),
    ConvCase(A.FMT_NCHW44, A.GROUP, 2, 8, 17, 21, 8, 5, 2, 2, A.IDENTITY, scales=(0.02, 0.01, unsat(25)), bias=False),
    ConvCase(A.FMT_NCHW44, A.GROUP, 3, 4, 3, 2, 4, 5, 1, 2, A.RELU, scales=(0.02, 0.01, unsat(25))),
    ConvCase(A.FMT_NCHW44, A.GROUP, 1, 4, 2, 3, 4, 5, 2, 2, A.SIGMOID, scales=(0.02, 0.01, unsat(25) * 40)),
    ConvCase(A.FMT_NCHW44, A.GROUP, 2, 16, 28, 28, 16, 7, 1, 3, A.RELU, scales=(0.02, 0.01, unsat(49))),
    ConvCase(A.FMT_NCHW44, A.GROUP, 2, 12, 30, 36, 12, 7, 2, 3, A.IDENTITY, scales=(0.02, 0.01, unsat(49))),
    ConvCase(A.FMT_NCHW44, A.GROUP, 2, 8, 11, 13, 8, 7, 1, 3, A.H_SWISH, scales=(0.02, 0.01, unsat(49))),
    ConvCase(A.FMT_NCHW44, A.GROUP, 1, 4, 9, 7, 4, 7, 2, 3, A.RELU, scales=(0.02, 0.01, unsat(49)), bias=False),
    ConvCase(A.FMT_NCHW44, A.GROUP, 4, 8, 1, 9, 8, 7, 1, 3, A.IDENTITY, scales=(0.5, 0.5, 0.5)),
    # ... and what keeps the one-output-per-thread kernel: other paddings, dilation
    ConvCase(A.FMT_NCHW44, A.GROUP, 2, 8, 12, 16, 8, 5, 1, 0, A.RELU, scales=(0.02, 0.01, unsat(25))),
    ConvCase(A.FMT_NCHW44, A.GROUP, 2, 8, 12, 16, 8, 3, 1, 2, A.RELU, scales=(0.02, 0.01, unsat(9)), dilate=2),
    ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 2, 3, 224, 224, 32, 3, 2, 1, A.RELU, scales=(0.02, 0.01, unsat(27))),
    ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 3, 3, 64, 48, 24, 3, 2, 1, A.IDENTITY, scales=(0.02, 0.01, unsat(27))),
    # the matrix-core form (32 / 64 output channels): ragged last tile, rows of 4 and 8 columns (first
    # and last column next to each other), H_SWISH, no bias
    ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 3, 3, 18, 28, 64, 3, 2, 1, A.IDENTITY, scales=(0.02, 0.01, unsat(27))),
    ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 5, 3, 6, 4, 32, 3, 2, 1, A.RELU, scales=(0.02, 0.01, 0.05)),
    ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 2, 3, 10, 8, 32, 3, 2, 1, A.H_SWISH, scales=(0.02, 0.01, unsat(27))),
    ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 1, 3, 224, 224, 32, 3, 2, 1, A.RELU, scales=(0.02, 0.01, unsat(27)), bias=False),
    ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 1, 3, 32, 36, 8, 3, 2, 1, A.H_SWISH, scales=(0.02, 0.01, unsat(27))),
    ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 2, 3, 30, 34, 8, 3, 2, 1, A.RELU, scales=(0.02, 0.01, unsat(27))),  # generic path (IW % 4 != 0)
    PoolCase(A.FMT_NCHW44, A.POOL_MAX, 2, 32, 112, 112, 2, 2, 0),
    # the 2x2 stride-2 maximum on packed halves (rows of 8, 16 pixels), and rows it does not take
    # dense NCHW layers whose channel counts are no multiple of 4: padded copies around the NCHW44
    # kernel (input lanes, output lanes and the bias padded independently)
    ConvCase(A.FMT_NCHW, A.DENSE, 2, 6, 20, 24, 10, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(54))),
    ConvCase(A.FMT_NCHW, A.DENSE, 3, 3, 31, 17, 8, 3, 2, 1, A.IDENTITY, scales=(0.02, 0.01, unsat(27))),
    ConvCase(A.FMT_NCHW, A.DENSE, 2, 16, 14, 14, 7, 1, 1, 0, A.RELU, scales=(0.02, 0.01, unsat(16))),
    ConvCase(A.FMT_NCHW, A.DENSE, 5, 1, 12, 12, 1, 3, 1, 1, A.H_SWISH, scales=(0.02, 0.01, unsat(9))),
    ConvCase(A.FMT_NCHW, A.DENSE, 4, 33, 28, 28, 65, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(297)), bias=False),
    # 1x1 with 1024 input channels between 2048 and 4096 pixels: the workgroup-shared pointwise
    # kernel (1024 -> 512), half-filled tiles of the LDS-direct kernel (1024 -> 256)
    ConvCase(A.FMT_NCHW44, A.DENSE, 64, 1024, 7, 7, 512, 1, 1, 0, A.RELU, scales=(0.02, 0.01, unsat(1024))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 50, 1024, 7, 7, 256, 1, 1, 0, A.IDENTITY, scales=(0.02, 0.01, unsat(1024))),
    PoolCase(A.FMT_NCHW44, A.POOL_MAX, 3, 12, 6, 8, 2, 2, 0),
    PoolCase(A.FMT_NCHW44, A.POOL_MAX, 1, 4, 2, 16, 2, 2, 0),
    PoolCase(A.FMT_NCHW44, A.POOL_MAX, 2, 8, 6, 12, 2, 2, 0),
    PoolCase(A.FMT_NCHW44, A.POOL_MAX, 2, 8, 7, 16, 2, 2, 0),
    PoolCase(A.FMT_NCHW, A.POOL_MAX, 2, 32, 112, 112, 2, 2, 0),
    PoolCase(A.FMT_NCHW, A.POOL_MAX, 3, 5, 10, 24, 2, 2, 0),   # 8-byte row pieces, odd plane count
    PoolCase(A.FMT_NCHW, A.POOL_MAX, 3, 5, 11, 24, 2, 2, 0),   # odd height: the generic kernel
    PoolCase(A.FMT_NCHW, A.POOL_MAX, 2, 7, 10, 20, 2, 2, 0),   # IW % 8 != 0: the generic kernel
    # four output pixels of a row per thread (NCHW44)
    PoolCase(A.FMT_NCHW44, A.POOL_MAX, 2, 16, 57, 44, 3, 2, 1),
    PoolCase(A.FMT_NCHW44, A.POOL_MAX, 2, 64, 112, 112, 3, 2, 1),
    PoolCase(A.FMT_NCHW44, A.POOL_AVERAGE, 2, 8, 14, 16, 3, 1, 1),
    PoolCase(A.FMT_NCHW44, A.POOL_AVERAGE_COUNT_EXCLUDE_PADDING, 3, 8, 15, 24, 3, 2, 1),
    PoolCase(A.FMT_NCHW44, A.POOL_AVERAGE_COUNT_EXCLUDE_PADDING, 1, 4, 9, 12, 2, 1, 0),
    PoolCase(A.FMT_NCHW44, A.POOL_MAX, 3, 12, 10, 20, 2, 2, 1),
    PoolCase(A.FMT_NCHW44, A.POOL_MAX, 2, 16, 57, 43, 3, 2, 1),  # rows of 43 pixels: the generic kernel
    # four outputs of a row per thread (NCHW): padded and unpadded borders, rows of every alignment
    # (odd widths), output rows that are no multiple of 4, all three modes, window height != width
    # is not expressible here but the height is a run-time loop
    PoolCase(A.FMT_NCHW, A.POOL_MAX, 2, 16, 112, 112, 3, 2, 1),
    PoolCase(A.FMT_NCHW, A.POOL_MAX, 3, 5, 57, 113, 3, 2, 1),
    PoolCase(A.FMT_NCHW, A.POOL_MAX, 2, 3, 30, 41, 3, 2, 0),
    PoolCase(A.FMT_NCHW, A.POOL_AVERAGE, 2, 7, 28, 35, 3, 1, 1),
    PoolCase(A.FMT_NCHW, A.POOL_AVERAGE_COUNT_EXCLUDE_PADDING, 2, 7, 28, 35, 3, 1, 1),
    PoolCase(A.FMT_NCHW, A.POOL_AVERAGE_COUNT_EXCLUDE_PADDING, 3, 4, 19, 50, 2, 2, 1),
    PoolCase(A.FMT_NCHW, A.POOL_AVERAGE, 1, 9, 33, 47, 2, 1, 0),
    PoolCase(A.FMT_NCHW, A.POOL_MAX, 2, 6, 20, 37, 5, 1, 2),
    PoolCase(A.FMT_NCHW44, A.POOL_AVERAGE, 5, 1024, 7, 7, 7, 7, 0),
    PoolCase(A.FMT_NCHW, A.POOL_AVERAGE, 5, 1024, 7, 7, 7, 7, 0),
    PoolCase(A.FMT_NCHW44, A.POOL_MAX, 3, 64, 13, 13, 13, 13, 0),  # one output pixel per plane
    PoolCase(A.FMT_NCHW44, A.POOL_AVERAGE_COUNT_EXCLUDE_PADDING, 3, 64, 13, 13, 13, 13, 0),
    PoolCase(A.FMT_NCHW44, A.POOL_AVERAGE, 2, 8, 4, 4, 4, 4, 0),
    MultiTypeCase(A.Q_FUSE_ADD_RELU, (2, 32, 56, 56), (0.05, 0.01, 0.05)),
    MultiTypeCase(A.Q_ADD, (3, 7, 13, 5), (0.031, 0.017, 0.023)),
    MultiTypeCase(A.Q_MUL, (2, 32, 56, 56), (0.05, 0.04, 0.3)),
    MultiTypeCase(A.Q_RELU, (1, 1, 1, 100003), (0.05, 0.01, 0.03)),
    TypeCvtCase("f32", "qsi8", (2, 3, 224, 224), dst_scale=0.0173),
    TypeCvtCase("qsi8", "f32", (64, 1000), src_scale=0.0173),
    TypeCvtCase("qsi8", "qsi8", (5, 1001), src_scale=0.0173, dst_scale=0.0291),
    TypeCvtCase("qsi32", "qsi8", (5, 1001), src_scale=0.0002, dst_scale=0.05),
    # relayout: NCHW <-> NCHW4 at a model's size, plain and batched transposes, every permutation
    # class of a 4-d tensor, ragged tiles, views with negative / zero / non-unit strides, rows
    # that can and cannot be widened to 16-byte elements
    RelayoutCase("qsi8", (8, 16, 56, 56, 4), (64 * 3136, 4 * 3136, 56, 1, 3136)),
    RelayoutCase("qsi8", (8, 16, 56, 56, 4), None, None, (64 * 3136, 4 * 3136, 56, 1, 3136)),
    RelayoutCase("f32", (4, 8, 28, 28, 4), (32 * 784, 4 * 784, 28, 1, 784)),
    RelayoutCase("f32", (1000, 1023), (1, 1000)),
    RelayoutCase("f32", (1023, 1000), None, None, (1, 1023)),
    RelayoutCase("qsi8", (3, 517, 259), (517 * 259, 1, 517)),
    RelayoutCase("qsi32", (5, 70, 3, 66), (70 * 3 * 66, 1, 70 * 66, 70)),
    RelayoutCase("f32", (6, 10, 14, 18), (1, 6, 60, 840)),
    RelayoutCase("f32", (6, 10, 14, 18), (18, 108, 1080, 1)),
    RelayoutCase("qsi8", (6, 10, 14, 18), (140, 14, 1, 840)),
    RelayoutCase("qsi8", (2, 3, 1, 2, 3, 2, 5), (180, 5, 7, 30, 60, 15, 1)),
    RelayoutCase("f32", (7, 9, 33), (9 * 33, -33, 1)),
    RelayoutCase("qsi8", (7, 9, 33), (9 * 33, 33, -1)),
    RelayoutCase("f32", (40, 50), (-50, -1), None, (1, 40)),
    RelayoutCase("f32", (16, 3, 64), (64, 0, 1)),
    RelayoutCase("qsi8", (5, 1000), (0, 1)),
    RelayoutCase("qsi8", (64, 4096), (8192, 1), slack=0),
    RelayoutCase("qsi8", (64, 4096), (8192, 1), slack=5),
    RelayoutCase("qsi8", (64, 4090), (8190, 1), slack=0),
    RelayoutCase("f32", (32, 100, 64), None, None, (100 * 192, 192, 1), slack=4),
    RelayoutCase("f32", (32, 100, 64), (2 * 6400, 2 * 64, 2), None, (7000, 70, 1)),
    RelayoutCase("qsi8", (60, 40), (90, 2), (20, 120), (310, 2)),
    RelayoutCase("f32", (1, 1, 1), None),
    RelayoutCase("f32", (2, 3, 1, 5), (1, 2, 77, 6)),
    # concat: compiler/test/kernel/opr/naive/concat.cpp:5-28 and the channel join of NCHW44 maps
    ConcatCase("f32", [(12, 13, i + 1, 15) for i in range(4)], 2),
    ConcatCase("qsi8", [(12, i + 1, 14, 15) for i in range(4)], 1),
    ConcatCase("qsi8", [(i + 1, 13, 14, 15) for i in range(4)], 0),
    ConcatCase("qsi32", [(12, 13, 14, i + 1) for i in range(4)], 3),
    ConcatCase("qsi8", [(8, 16, 28, 28, 4), (8, 8, 28, 28, 4), (8, 24, 28, 28, 4)], 1),
    ConcatCase("f32", [(64, 1000)], 1),
    # f32
    ConvCase(A.FMT_NCHW, A.DENSE, 1, 32, 56, 56, 32, 3, 1, 1, A.RELU, dtype="f32"),
    ConvCase(A.FMT_NCHW, A.DENSE, 2, 5, 19, 23, 37, 3, 2, 1, A.IDENTITY, dtype="f32"),
    # above 2^27 multiply-adds: the implicit GEMM on the matrix cores
    ConvCase(A.FMT_NCHW, A.DENSE, 4, 64, 56, 56, 64, 3, 1, 1, A.RELU, dtype="f32"),
    ConvCase(A.FMT_NCHW, A.DENSE, 3, 40, 57, 55, 72, 3, 2, 1, A.H_SWISH, dtype="f32"),
    # f32 dense layers in NCHW44: NCHW copies of input, output and filter around the implicit GEMM
    # (with and without a split of K), stride 2, 1x1, no bias, every activation
    ConvCase(A.FMT_NCHW44, A.DENSE, 2, 64, 28, 28, 64, 3, 1, 1, A.RELU, dtype="f32"),
    ConvCase(A.FMT_NCHW44, A.DENSE, 3, 40, 29, 31, 72, 3, 2, 1, A.H_SWISH, dtype="f32"),
    ConvCase(A.FMT_NCHW44, A.DENSE, 2, 16, 14, 12, 128, 1, 1, 0, A.IDENTITY, dtype="f32", bias=False),
    ConvCase(A.FMT_NCHW44, A.DENSE, 1, 256, 7, 7, 32, 3, 1, 1, A.SIGMOID, dtype="f32"),
    ConvCase(A.FMT_NCHW44, A.DENSE, 2, 8, 12, 10, 8, 5, 1, 2, A.RELU, dtype="f32", dilate=1),
    # the last tile of output pixels is ragged (1584 = 12 x 128 + 48): its surplus columns must
    # gather inside the tensor; padding wider than half the filter, no bias, split K
    ConvCase(A.FMT_NCHW, A.DENSE, 3, 86, 45, 42, 117, 5, 2, 3, A.SIGMOID, dtype="f32", bias=False),
    ConvCase(A.FMT_NCHW, A.DENSE, 1, 40, 9, 11, 30, 3, 1, 1, A.RELU, dtype="f32", dilate=2),
    MatMulCase(1, 1024, 1000),
    MatMulCase(64, 512, 384),
    MatMulCase(130, 77, 259),
    MatMulCase(33, 65, 70, trans_a=True),
    MatMulCase(33, 65, 70, trans_b=True),
    MatMulCase(33, 65, 70, trans_a=True, trans_b=True),
    # at most 4 rows (the one-pass kernels): B as it lies and transposed, sizes that allow 16-byte
    # loads and sizes that do not, K short of a whole step
    MatMulCase(2, 130, 45),
    MatMulCase(3, 301, 79, trans_b=True),
    MatMulCase(4, 1024, 1000, trans_b=True),
    MatMulCase(4, 100, 64),
    # whole tiles are staged with 16-byte loads, tiles at the edges and the last stage of K element
    # by element: both in one product, every transposition; then the 64-row tile with split K
    MatMulCase(192, 100, 320),
    MatMulCase(192, 100, 320, trans_a=True),
    MatMulCase(192, 100, 320, trans_b=True),
    MatMulCase(192, 100, 320, trans_a=True, trans_b=True),
    MatMulCase(64, 1024, 2048),
    MatMulCase(64, 1024, 2048, trans_a=True),
    MatMulCase(64, 1024, 2048, trans_b=True),
    MatMulCase(64, 1024, 2048, trans_a=True, trans_b=True),
]


@pytest.mark.parametrize("case", LIVE, ids=[repr(c) for c in LIVE])
def test_matches_oracle(case):
    port.set_threads(8)
    arrays = case.gen(seed=11)
    want = case.run_port(arrays)
    got = run_gpu(case, arrays)
    compare(got, want, repr(case))


F32_NCHW44 = [
    # f32 channel-wise layers in NCHW44 (the reference's GI_chanwise kernels: 3x3 / 5x5, stride 1 / 2):
    # tiles of 4 x 64 pixels - extents below, at and above a tile, padding 0 .. k/2 + 1, every activation
    ("dwconv44_f32", ConvCase(A.FMT_NCHW44, A.GROUP, 3, 32, 56, 56, 32, 3, 1, 1, A.RELU, dtype="f32")),
    ("dwconv44_f32", ConvCase(A.FMT_NCHW44, A.GROUP, 2, 16, 57, 131, 16, 3, 2, 1, A.IDENTITY, dtype="f32")),
    ("dwconv44_f32", ConvCase(A.FMT_NCHW44, A.GROUP, 2, 24, 28, 28, 24, 5, 1, 2, A.H_SWISH, dtype="f32")),
    ("dwconv44_f32", ConvCase(A.FMT_NCHW44, A.GROUP, 1, 8, 30, 65, 8, 5, 2, 2, A.SIGMOID, dtype="f32", bias=False)),
    ("dwconv44_f32", ConvCase(A.FMT_NCHW44, A.GROUP, 5, 4, 3, 2, 4, 3, 1, 1, A.RELU, dtype="f32")),
    ("dwconv44_f32", ConvCase(A.FMT_NCHW44, A.GROUP, 2, 12, 9, 70, 12, 3, 1, 0, A.RELU, dtype="f32")),
    ("dwconv44_f32", ConvCase(A.FMT_NCHW44, A.GROUP, 2, 12, 13, 64, 12, 5, 1, 3, A.IDENTITY, dtype="f32")),
    ("dwconv44_f32", ConvCase(A.FMT_NCHW44, A.GROUP, 1, 8, 1, 1, 8, 3, 2, 1, A.RELU, dtype="f32")),
    # (a 7x7 window is none of the reference's four variants: the one-output-per-thread kernel)
    ("conv_direct", ConvCase(A.FMT_NCHW44, A.GROUP, 1, 8, 12, 11, 8, 7, 1, 3, A.RELU, dtype="f32")),
    # f32 first layers, NCHW source -> NCHW44 result (the reference's GI nchw_nchw44 kernel)
    ("conv_first_f32", ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 2, 3, 64, 64, 32, 3, 2, 1, A.RELU, dtype="f32")),
    ("conv_first_f32", ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 2, 3, 37, 41, 64, 7, 2, 3, A.RELU, dtype="f32")),
    ("conv_first_f32", ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 1, 1, 30, 29, 8, 5, 1, 2, A.H_SWISH, dtype="f32")),
    ("conv_first_f32", ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 3, 4, 17, 300, 40, 3, 1, 0, A.IDENTITY, dtype="f32",
                                bias=False)),
    ("conv_first_f32", ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 1, 2, 5, 4, 4, 3, 2, 2, A.SIGMOID, dtype="f32")),
    ("conv_first_f32", ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 2, 3, 20, 20, 36, 3, 1, 1, A.RELU, dtype="f32")),
]


@pytest.mark.parametrize("kernel,case", F32_NCHW44, ids=[repr(c) for _, c in F32_NCHW44])
def test_f32_channel_wise_and_first_layers_in_nchw44(kernel, case):
    port.set_threads(8)
    arrays = case.gen(seed=13)
    got = run_gpu(case, arrays)
    assert runtime.last_kernel().startswith(kernel), runtime.last_kernel()
    compare(got, case.run_port(arrays), repr(case))


F32_POINTWISE = [
    # f32 elementwise: the FullyConnected bias [M,N] + [N] / [1,N] at the sizes of the MatMul
    # configurations, the softmax steps ([A,N] op [A,1]), every other way two operands meet
    # (scalar and [1,C,1,1] either side, NCHW44 channel vector, leading run, general broadcast),
    # ragged sizes that take the one-element-per-thread path, every mode
    ElemwiseCase("ADD", [(64, 4096), (4096,)]),
    ElemwiseCase("ADD", [(64, 4096), (1, 4096)]),
    ElemwiseCase("ADD", [(1, 1000), (1000,)]),
    ElemwiseCase("ADD", [(4096, 4096), (1, 4096)]),
    ElemwiseCase("ADD", [(1, 4096), (4096, 4096)]),
    ElemwiseCase("SUB", [(64, 1000), (64, 1)]),
    ElemwiseCase("TRUE_DIV", [(64, 1000), (64, 1)], span=(1.0, 9.0)),
    ElemwiseCase("TRUE_DIV", [(1,), (5, 1001)], span=(1.0, 9.0)),
    ElemwiseCase("MUL", [(4, 32, 14, 14), (1, 32, 1, 1)]),
    ElemwiseCase("MUL", [(1, 32, 1, 1), (4, 32, 14, 14)]),
    ElemwiseCase("MUL", [(4, 32, 7, 9), (1, 32, 1, 1)]),
    ElemwiseCase("MAX", [(4, 8, 14, 14, 4), (1, 8, 1, 1, 4)]),
    ElemwiseCase("MIN", [(3, 1, 5, 1), (3, 4, 5, 6)]),
    ElemwiseCase("MIN", [(3, 4, 5, 8), (3, 1, 5, 1)]),
    ElemwiseCase("FUSE_ADD_RELU", [(2, 3, 4, 5), (1, 1, 4, 5)]),
    ElemwiseCase("FUSE_ADD_RELU", [(64, 1000), (64, 1000)]),
    ElemwiseCase("SUB", [(100003,), (1,)]),
    ElemwiseCase("ADD", [(7, 1, 9, 1, 5, 1, 4), (1, 6, 1, 3, 1, 2, 4)]),
    ElemwiseCase("RELU", [(64, 1000)]),
    ElemwiseCase("NEGATE", [(5, 1001)]),
    ElemwiseCase("EXP", [(64, 1000)], span=(-20.0, 0.0)),
    ElemwiseCase("SIGMOID", [(5, 1001)]),
    ElemwiseCase("H_SWISH", [(3, 16, 28, 28)], span=(-6.0, 6.0)),
    # f32 reduce: the softmax steps, a global average written as MEAN, every mode, every position
    # of the axis (first: C > 1 with A = 1; middle; last: C = 1)
    ReduceCase("MAX", (64, 1000), 1),
    ReduceCase("SUM", (64, 1000), 1),
    ReduceCase("MEAN", (8, 1024, 49), 2),
    ReduceCase("MEAN", (6, 50, 33), 1),
    ReduceCase("MIN", (50, 7, 9), 0),
    ReduceCase("SUM", (3000, 5), 0),
    ReduceCase("SUM_SQR", (4, 5, 6, 7), 2),
    ReduceCase("PRODUCT", (3, 40, 5), 1),
    ReduceCase("MAX", (1, 100003), 1),
]


@pytest.mark.parametrize("case", F32_POINTWISE, ids=[repr(c) for c in F32_POINTWISE])
def test_f32_elemwise_and_reduce(case):
    arrays = case.gen(seed=67)
    compare(run_gpu(case, arrays), case.run_port(arrays), repr(case))


def _random_views():
    """seeded random strided views: permuted dims, steps of 2, reversed dims, both sides or one"""
    r = np.random.Generator(np.random.PCG64(77))

    def view(shape):
        nd = len(shape)
        perm = r.permutation(nd)
        step = [int(r.integers(1, 3)) if r.random() < 0.3 else 1 for _ in range(nd)]
        # dense strides of the permuted, stepped storage
        st = [0] * nd
        acc = 1
        for ax in reversed(perm):
            st[ax] = acc * step[ax]
            acc *= shape[ax] * step[ax]
        if r.random() < 0.25:
            ax = int(r.integers(0, nd))
            st[ax] = -st[ax]
        return tuple(st)

    out = []
    for i in range(36):
        nd = int(r.integers(1, 6))
        big = r.random() < 0.4
        shape = tuple(int(r.integers(1, 40 if big else 9)) for _ in range(nd))
        if int(np.prod(shape)) > 300000:
            shape = shape[:3]
        dt = ["f32", "qsi8", "qsi32"][i % 3]
        kind = i % 4
        src = view(shape) if kind != 1 else None
        dst = view(shape) if kind in (1, 2) else None
        out.append(RelayoutCase(dt, shape, src, None, dst, slack=int(r.integers(0, 5))))
    return out


VIEWS = _random_views()


@pytest.mark.parametrize("case", VIEWS, ids=["%d-%r" % (i, c) for i, c in enumerate(VIEWS)])
def test_relayout_random_views(case):
    arrays = case.gen(seed=31)
    compare(run_gpu(case, arrays), case.run_port(arrays), repr(case))


HYBRID = [
    # NCHW -> NCHW44 first layers beyond 3x3 stride 2: the matrix-core kernel with the reduction
    # re-ordered to (ic, fh, fw padded to 8); 1..4 input channels, strips of 128 pixels (one and
    # several per row), partial channel tiles, every activation
    ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 2, 3, 64, 64, 64, 7, 2, 3, A.RELU, scales=(0.02, 0.01, unsat(147))),
    ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 1, 3, 224, 224, 64, 7, 2, 3, A.RELU, scales=(0.02, 0.01, unsat(147))),
    ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 1, 3, 57, 61, 24, 5, 2, 2, A.IDENTITY, scales=(0.02, 0.01, unsat(75))),
    ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 2, 3, 33, 47, 32, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(27))),
    ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 3, 1, 40, 40, 8, 3, 2, 0, A.H_SWISH, scales=(0.02, 0.01, unsat(9))),
    ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 1, 4, 30, 150, 96, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(36))),
    ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 1, 3, 40, 300, 12, 8, 2, 3, A.SIGMOID, scales=(0.02, 0.01, unsat(192) * 30)),
    ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 2, 2, 19, 23, 128, 1, 1, 0, A.IDENTITY, scales=(0.02, 0.01, unsat(2))),
    ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 1, 3, 9, 9, 4, 5, 1, 2, A.RELU, scales=(0.02, 0.01, unsat(75))),
    # enough rows that a workgroup takes 4 / 2 output rows per strip and shares their input rows
    # in LDS; the last group of rows is incomplete (62 = 15 * 4 + 2, 63 = 31 * 2 + 1)
    ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 66, 3, 124, 60, 16, 7, 2, 3, A.RELU, scales=(0.02, 0.01, unsat(147))),
    ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 34, 3, 126, 50, 8, 7, 2, 3, A.IDENTITY, scales=(0.02, 0.01, unsat(147))),
    ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 40, 2, 30, 140, 8, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(18))),
]


@pytest.mark.parametrize("case", HYBRID, ids=[repr(c) for c in HYBRID])
def test_first_layer_shapes(case):
    port.set_threads(8)
    arrays = case.gen(seed=37)
    compare(run_gpu(case, arrays), case.run_port(arrays), repr(case))


STRIDED_1X1 = [
    # projection shortcuts: 1x1 with a stride = the pointwise kernels on the gathered pixels
    ConvCase(A.FMT_NCHW44, A.DENSE, 4, 64, 56, 56, 128, 1, 2, 0, A.IDENTITY, scales=(0.02, 0.01, unsat(64))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 2, 256, 14, 14, 512, 1, 2, 0, A.RELU, scales=(0.02, 0.01, unsat(256))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 3, 32, 15, 17, 24, 1, 2, 0, A.IDENTITY, scales=(0.02, 0.01, unsat(32))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 1, 1024, 7, 7, 64, 1, 3, 0, A.H_SWISH, scales=(0.02, 0.01, unsat(1024))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 2, 16, 9, 9, 8, 1, 2, 0, A.RELU, scales=(0.02, 0.01, unsat(16))),
]


@pytest.mark.parametrize("case", STRIDED_1X1, ids=[repr(c) for c in STRIDED_1X1])
def test_strided_pointwise(case):
    port.set_threads(8)
    arrays = case.gen(seed=47)
    compare(run_gpu(case, arrays), case.run_port(arrays), repr(case))


DOT4 = [
    # dense NCHW44 layers the matrix-core kernels do not take (more than 9 taps): the dot-product
    # kernel; both channel-group widths, an odd number of channel groups, stride, dilation,
    # padding wider than the image edge, every activation
    ConvCase(A.FMT_NCHW44, A.DENSE, 4, 32, 28, 28, 64, 5, 1, 2, A.RELU, scales=(0.02, 0.01, unsat(800))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 1, 8, 9, 11, 12, 5, 2, 2, A.IDENTITY, scales=(0.02, 0.01, unsat(200))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 2, 16, 23, 19, 20, 7, 2, 3, A.H_SWISH, scales=(0.02, 0.01, unsat(784))),
    ConvCase(A.FMT_NCHW44, A.DENSE, 3, 4, 30, 30, 4, 5, 1, 0, A.SIGMOID, scales=(0.02, 0.01, unsat(100) * 30)),
    ConvCase(A.FMT_NCHW44, A.DENSE, 2, 12, 17, 17, 28, 4, 1, 3, A.RELU, scales=(0.02, 0.01, unsat(192)), dilate=2),
    ConvCase(A.FMT_NCHW44, A.DENSE, 40, 8, 20, 20, 40, 6, 3, 1, A.RELU, scales=(0.02, 0.01, unsat(288))),
]


@pytest.mark.parametrize("case", DOT4, ids=[repr(c) for c in DOT4])
def test_many_tap_dense_conv(case):
    port.set_threads(8)
    arrays = case.gen(seed=53)
    compare(run_gpu(case, arrays), case.run_port(arrays), repr(case))


NCHW_SPATIAL = [
    # dense qsi8 convolutions on plain NCHW tensors (no NCHW44 layout pass): relayout, the NCHW44
    # matrix-core kernel, relayout back; channel counts that are no multiple of 4 stay on the
    # one-output-per-thread kernel
    ConvCase(A.FMT_NCHW, A.DENSE, 2, 16, 20, 24, 12, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(144))),
    ConvCase(A.FMT_NCHW, A.DENSE, 3, 64, 28, 28, 64, 3, 2, 1, A.IDENTITY, scales=(0.02, 0.01, unsat(576))),
    ConvCase(A.FMT_NCHW, A.DENSE, 1, 32, 17, 13, 40, 1, 1, 0, A.H_SWISH, scales=(0.02, 0.01, unsat(32))),
    ConvCase(A.FMT_NCHW, A.DENSE, 2, 8, 15, 15, 8, 3, 1, 2, A.RELU, scales=(0.02, 0.01, unsat(72)), dilate=2),
    ConvCase(A.FMT_NCHW, A.DENSE, 2, 6, 11, 9, 10, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(54))),
]


@pytest.mark.parametrize("case", NCHW_SPATIAL, ids=[repr(c) for c in NCHW_SPATIAL])
def test_nchw_spatial_conv(case):
    port.set_threads(8)
    arrays = case.gen(seed=59)
    compare(run_gpu(case, arrays), case.run_port(arrays), repr(case))


NCHW_DW = [
    # channel-wise qsi8 convolution on plain NCHW tensors: the NCHW44 depthwise kernel between
    # relayouts (channel counts that are multiples of 4; the others stay on the generic kernel)
    ConvCase(A.FMT_NCHW, A.GROUP, 4, 32, 56, 56, 32, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(9))),
    ConvCase(A.FMT_NCHW, A.GROUP, 3, 16, 29, 31, 16, 3, 2, 1, A.IDENTITY, scales=(0.02, 0.01, unsat(9))),
    ConvCase(A.FMT_NCHW, A.GROUP, 2, 8, 13, 17, 8, 5, 1, 2, A.H_SWISH, scales=(0.02, 0.01, unsat(25))),
    ConvCase(A.FMT_NCHW, A.GROUP, 2, 6, 9, 7, 6, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(9))),
    # native NCHW kernel (rows of a multiple of 4 pixels): channel counts that are no multiple of 4,
    # one group per row, output rows that are no multiple of 4 (byte stores), no bias, literal epilogue
    ConvCase(A.FMT_NCHW, A.GROUP, 2, 6, 9, 8, 6, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(9))),
    ConvCase(A.FMT_NCHW, A.GROUP, 3, 5, 11, 12, 5, 3, 2, 1, A.IDENTITY, scales=(0.02, 0.01, unsat(9))),
    ConvCase(A.FMT_NCHW, A.GROUP, 1, 3, 4, 4, 3, 3, 1, 1, A.IDENTITY, scales=(0.5, 0.5, 0.5), bias=False),
    ConvCase(A.FMT_NCHW, A.GROUP, 2, 7, 17, 28, 7, 3, 2, 1, A.H_SWISH, scales=(0.02, 0.01, unsat(9))),
    ConvCase(A.FMT_NCHW, A.GROUP, 2, 33, 30, 44, 33, 3, 1, 1, A.RELU, scales=(0.02, 0.01, 0.05)),
    ConvCase(A.FMT_NCHW, A.GROUP, 1, 2, 1, 4, 2, 3, 2, 1, A.RELU, scales=(0.02, 0.01, unsat(9))),
]


@pytest.mark.parametrize("case", NCHW_DW, ids=[repr(c) for c in NCHW_DW])
def test_nchw_depthwise_conv(case):
    port.set_threads(8)
    arrays = case.gen(seed=61)
    compare(run_gpu(case, arrays), case.run_port(arrays), repr(case))


RESIZE = [
    # the 2x upsampling of detection necks, a camera frame scaled down to a network input, odd
    # ratios, extent 1 either side, a channel slice with a column step as NEAREST source
    ResizeCase(A.FMT_NCHW, "LINEAR", 2, 16, 40, 52, 80, 104),
    ResizeCase(A.FMT_NCHW44, "LINEAR", 2, 8, 40, 52, 80, 104),
    ResizeCase(A.FMT_NCHW, "NEAREST", 2, 16, 40, 52, 80, 104),
    ResizeCase(A.FMT_NCHW, "LINEAR", 1, 3, 480, 640, 224, 224),
    ResizeCase(A.FMT_NCHW44, "LINEAR", 3, 2, 37, 53, 111, 29),
    ResizeCase(A.FMT_NCHW, "LINEAR", 3, 5, 17, 1, 33, 7),
    ResizeCase(A.FMT_NCHW, "LINEAR", 2, 3, 1, 19, 1, 300),
    ResizeCase(A.FMT_NCHW, "LINEAR", 1, 2, 5, 700, 3, 2500),  # rows longer than the column table
    ResizeCase(A.FMT_NCHW, "NEAREST", 3, 7, 31, 45, 17, 101),
    ResizeCase(A.FMT_NCHW, "NEAREST", 2, 5, 33, 47, 100, 31, src_strides=(40000, 3300, 100, 2)),
]


@pytest.mark.parametrize("case", RESIZE, ids=[repr(c) for c in RESIZE])
def test_resize(case):
    arrays = case.gen(seed=41)
    got, want = run_gpu(case, arrays), case.run_port(arrays)
    compare(got, want, repr(case))
    # the kernels keep the reference's order of operations: equal bit for bit
    assert np.array_equal(got, want), repr(case)


FUSED = [
    # chains at the sizes of a detection head (SiLU gating, residual scale + shift, clipped
    # activations), every operand kind, a chain of the maximum length, a length that is no
    # multiple of the workgroup
    FusedCase(["I0,SILU,O0", "O0,I1,MUL,O1", "O1,I2,ADD,D"], [(8, 64, 40, 40), (1, 64, 1, 1), (1, 64, 1, 1)]),
    FusedCase(["I0,I1,I2,FUSE_MUL_ADD3,O0", "O0,H_SWISH,O1", "O1,I3,FUSE_ADD_RELU,D"],
              [(4, 16, 28, 28, 4), (1, 16, 1, 1, 4), (1, 16, 1, 1, 4), (4, 16, 28, 28, 4)]),
    FusedCase(["I0,I1,SUB,O0", "O0,EXP,O1", "O1,I2,TRUE_DIV,D"], [(64, 1000), (1,), (1,)], positive=(2,)),
    FusedCase(["I0,I1,ADD,O0"] + ["O%d,I1,%s,O%d" % (j, m, j + 1) for j, m in enumerate(
        ["MUL", "SUB", "MAX", "MIN", "ADD", "MUL", "SUB", "FUSE_ADD_RELU", "ADD", "MAX", "MIN", "SUB", "ADD", "MUL"])]
        + ["O14,SIGMOID,D"], [(3, 5, 7, 11), (3, 5, 7, 11)]),
    FusedCase(["I0,ABS,O0", "O0,LOG,O1", "O1,I1,LT,O2", "O2,O1,I0,I1,FUSE_MUL_ADD4,D"],
              [(1, 3, 1, 331), (1, 3, 1, 1)], positive=(0,)),
]


@pytest.mark.parametrize("case", FUSED, ids=[repr(c) for c in FUSED])
def test_fused_elemwise(case):
    arrays = case.gen(seed=43)
    compare(run_gpu(case, arrays), case.run_port(arrays), repr(case))


OLDER = [
    # shapes the newer kernels take, forced back (megcc_gfx950_set_option) onto the
    # kernels that still serve other shapes: one-stage kernel with split-K (slices of 2 stages out
    # of 8: a sixth slice would start past the packed filter), dword activation loads, the
    # 256-pixel variant, the tiled FullyConnected
    ("nosmall", ConvCase(A.FMT_NCHW44, A.DENSE, 1, 256, 56, 56, 256, 3, 1, 1, A.RELU,
                               scales=(0.02, 0.01, unsat(2304)))),
    ("nosmall", ConvCase(A.FMT_NCHW44, A.DENSE, 3, 256, 14, 14, 256, 3, 1, 1, A.IDENTITY,
                               scales=(0.02, 0.01, 0.05))),
    ("nopm", ConvCase(A.FMT_NCHW44, A.DENSE, 6, 32, 56, 56, 160, 3, 1, 1, A.RELU,
                            scales=(0.02, 0.01, unsat(288)))),
    # the plain tile order of the tiled GEMMs (the default gives each XCD a compact rectangle of
    # tiles): f32 MatMul with a ragged 9 x 8 grid of 128 x 128 tiles, all four transpositions,
    # FullyConnected with 256 x 256 tiles (8 x 8)
    ("noxcdorder", MatMulCase(1100, 40, 1000)),
    ("noxcdorder", MatMulCase(1024, 24, 1030, trans_a=True)),
    ("noxcdorder", MatMulCase(1024, 24, 1030, trans_b=True)),
    ("noxcdorder", MatMulCase(1030, 24, 1024, trans_a=True, trans_b=True)),
    ("noxcdorder", ConvCase(A.FMT_NCHW, A.DENSE, 2048, 128, 1, 1, 2040, 1, 1, 0, A.IDENTITY,
                            scales=(0.02, 0.01, unsat(128)))),
    # the threshold table where the default is the one-multiply-add requantisation the host proved
    # exact for the layer's scales (scales without exact ties; "+affine" in the kernel's name):
    # pointwise streaming and workgroup-shared kernels, depthwise on the matrix cores and by v_dot4,
    # the matrix-core first layer, the LDS-direct 3x3 kernel with 256- and 512-pixel sub-tiles
    ("noaffine", ConvCase(A.FMT_NCHW44, A.DENSE, 4, 32, 56, 56, 64, 1, 1, 0, A.RELU,
                          scales=(0.0213, 0.0097, unsat(32) * 1.0371))),
    ("noaffine", ConvCase(A.FMT_NCHW44, A.DENSE, 64, 512, 14, 14, 512, 1, 1, 0, A.RELU,
                          scales=(0.015522320754826069, 0.0012519484153017402, 0.015279783867299557),
                          src_range=(-40, 40), flt_range=(-40, 40))),
    ("noaffine", ConvCase(A.FMT_NCHW44, A.GROUP, 3, 64, 28, 28, 64, 3, 1, 1, A.RELU,
                          scales=(0.0213, 0.0097, unsat(9) * 1.0371))),
    ("noaffine", ConvCase(A.FMT_NCHW44, A.GROUP, 3, 64, 28, 28, 64, 3, 2, 1, A.IDENTITY,
                          scales=(0.0213, 0.0097, unsat(9) * 1.0371))),
    ("noaffine", ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 2, 3, 64, 64, 32, 3, 2, 1, A.RELU,
                          scales=(0.0213, 0.0097, unsat(27) * 1.0371))),
    ("noaffine", ConvCase(A.FMT_NCHW44, A.DENSE, 6, 32, 56, 56, 160, 3, 1, 1, A.RELU,
                          scales=(0.0213, 0.0097, unsat(288) * 1.0371))),
    ("noaffine", ConvCase(A.FMT_NCHW44, A.DENSE, 20, 32, 56, 56, 128, 3, 1, 1, A.RELU,
                          scales=(0.0213, 0.0097, unsat(288) * 1.0371))),
    ("nodma512", ConvCase(A.FMT_NCHW44, A.DENSE, 22, 64, 54, 57, 128, 3, 1, 1, A.RELU,
                                scales=(0.02, 0.01, unsat(576)))),
    ("nogevm", ConvCase(A.FMT_NCHW, A.DENSE, 1, 1024, 1, 1, 1000, 1, 1, 0, A.IDENTITY,
                              scales=(0.01, 0.01, unsat(1024) / 2))),
    ("nogevm", MatMulCase(3, 301, 79, trans_b=True)),
    # FullyConnected with few rows as K slices in separate workgroups + the split-K reduction
    ("nofcone", ConvCase(A.FMT_NCHW, A.DENSE, 40, 1024, 1, 1, 200, 1, 1, 0, A.RELU,
                         scales=(0.01, 0.01, unsat(1024) / 2))),
    ("nof32small", ConvCase(A.FMT_NCHW, A.DENSE, 1, 32, 56, 56, 32, 3, 1, 1, A.RELU, dtype="f32")),
    ("nopwshare", ConvCase(A.FMT_NCHW44, A.DENSE, 70, 512, 14, 14, 512, 1, 1, 0, A.RELU,
                                 scales=(0.02, 0.01, unsat(512)))),
    ("nopws", ConvCase(A.FMT_NCHW44, A.DENSE, 11, 64, 56, 56, 128, 1, 1, 0, A.IDENTITY,
                             scales=(0.02, 0.01, unsat(64)))),
    ("nopws", ConvCase(A.FMT_NCHW44, A.DENSE, 3, 24, 28, 28, 144, 1, 1, 0, A.RELU,
                             scales=(0.02, 0.01, unsat(24)))),
    # stride-1 depthwise on the v_dot4 kernels (two rows per thread on large planes, one on small)
    ("nodwmfma", ConvCase(A.FMT_NCHW44, A.GROUP, 2, 32, 112, 112, 32, 3, 1, 1, A.RELU,
                          scales=(0.02, 0.01, unsat(9)))),
    ("nodwmfma", ConvCase(A.FMT_NCHW44, A.GROUP, 3, 16, 9, 28, 16, 3, 1, 1, A.IDENTITY,
                          scales=(0.02, 0.01, unsat(9)))),
    ("nodwmfma", ConvCase(A.FMT_NCHW44, A.GROUP, 5, 12, 7, 7, 12, 3, 1, 1, A.H_SWISH,
                          scales=(0.02, 0.01, unsat(9)))),
    ("nodwmfma", ConvCase(A.FMT_NCHW44, A.GROUP, 2, 24, 28, 28, 24, 5, 1, 2, A.RELU,
                          scales=(0.02, 0.01, unsat(25)))),
    # dense 5x5 on the v_dot4 kernel (what layers under 2048 pixels still use)
    ("norowsplit", ConvCase(A.FMT_NCHW44, A.DENSE, 6, 32, 28, 28, 64, 5, 1, 2, A.RELU,
                            scales=(0.02, 0.01, unsat(800)))),
    # channel-wise NCHW through the NCHW44 detour (what rows that are no multiple of 4 still use)
    ("nodwnchw", ConvCase(A.FMT_NCHW, A.GROUP, 4, 32, 56, 56, 32, 3, 1, 1, A.RELU,
                          scales=(0.02, 0.01, unsat(9)))),
    # NCHW pooling one output per thread (what windows wider than 5 or non-square ones still use)
    ("nofirstmfma", ConvCase(A.FMT_NCHW_NCHW44, A.DENSE, 2, 3, 224, 224, 32, 3, 2, 1, A.RELU,
                             scales=(0.02, 0.01, unsat(27)))),
    ("nopoolrows", PoolCase(A.FMT_NCHW, A.POOL_AVERAGE_COUNT_EXCLUDE_PADDING, 2, 5, 29, 37, 3, 2, 1)),
    ("nopoolrows", PoolCase(A.FMT_NCHW44, A.POOL_MAX, 2, 16, 57, 44, 3, 2, 1)),
]


SOFTMAX = [
    cases.SoftmaxCase((64, 1000)), cases.SoftmaxCase((64, 1000), quantised=True, scale=0.13),
    cases.SoftmaxCase((1, 1000), quantised=True, scale=0.05), cases.SoftmaxCase((3, 7, 4096)),
    cases.SoftmaxCase((5, 1)), cases.SoftmaxCase((2, 3, 257), span=(-60.0, 60.0)),
    cases.SoftmaxCase((300, 10), quantised=True, scale=1.0),
]


@pytest.mark.parametrize("case", SOFTMAX, ids=[repr(c) for c in SOFTMAX])
def test_softmax_in_one_kernel_equals_the_five_operator_chain(case):
    """the fused soft-max against the oracle's chain of the five operators it replaces"""
    arrays = case.gen(seed=41)
    ins, outs = case.specs(arrays)
    got = runtime.PreparedOp(case.desc(), ins, outs)
    got.launch()
    out = got.result()
    want = case.run_port(arrays)
    assert cases.max_rel_err(out, want) <= 1e-5, repr(case)
    assert np.allclose(out.reshape(-1, case.shape[-1]).sum(axis=1), 1.0, atol=1e-5)


def test_softmax_refuses_rows_beyond_its_limit():
    case = cases.SoftmaxCase((2, 4097))
    ins, outs = case.specs(case.gen(seed=1))
    with pytest.raises(runtime.MegccError):
        runtime.PreparedOp(case.desc(), ins, outs).launch()


@pytest.mark.parametrize("src_off,dst_off", [(1, 0), (2, 3), (3, 1)])
@pytest.mark.parametrize("mode", [A.POOL_MAX, A.POOL_AVERAGE_COUNT_EXCLUDE_PADDING])
def test_nchw_pooling_on_unaligned_tensors(mode, src_off, dst_off):
    """the row kernel fetches aligned dwords around a window and shifts: tensors that start at any
    byte, outputs stored byte by byte when their rows cannot be stored as dwords, and not a byte
    written outside the destination"""
    case = PoolCase(A.FMT_NCHW, mode, 2, 3, 21, 32, 3, 2, 1)
    arrays = case.gen(seed=3)
    want = case.run_port(arrays)
    src = arrays["src"]
    flat = np.zeros(src.size + 8, np.int8)
    flat[src_off:src_off + src.size] = src.ravel()
    ins = [cases.TensorSpec(b"src", src.shape, A.QINT8, case.scale, flat, offset=src_off)]
    outs = [cases.TensorSpec(b"dst", want.shape, A.QINT8, case.scale, offset=dst_off,
                             storage=(want.size + 8,))]
    got = runtime.run_symbol(case.symbol(), ins, outs)
    assert runtime.last_kernel().startswith("pool_nchw_rows")
    np.testing.assert_array_equal(got[dst_off:dst_off + want.size].reshape(want.shape), want)
    assert (got[:dst_off] == 0x5A).all() and (got[dst_off + want.size:] == 0x5A).all()


@pytest.mark.parametrize("switch,case", OLDER, ids=["%s-%r" % (s, c) for s, c in OLDER])
def test_older_kernels_still_agree(switch, case):
    port.set_threads(8)
    arrays = case.gen(seed=29)
    want = case.run_port(arrays)
    normally = None
    try:
        runtime.set_option(switch, 1)
        got = run_gpu(case, arrays)
        forced = runtime.last_kernel()
    finally:
        runtime.set_option(switch, 0)
    compare(got, want, repr(case))
    # the switch must have changed which kernel ran
    run_gpu(case, arrays)
    normally = runtime.last_kernel()
    assert forced != normally, "%s did not change the kernel (%s)" % (switch, forced)


def _plane_major_sweep():
    """seeded random 3x3 stride-1 layers whose rows are a multiple of 4 pixels and that are large
    enough for the LDS-direct kernels: batches whose sub-tiles cross image borders, ragged last
    sub-tiles, padding 0 / 1 / 2 (with dilation 2), channel counts that leave partial tiles"""
    r = np.random.Generator(np.random.PCG64(2024))
    out = []
    while len(out) < 14:
        iw = int(r.integers(2, 17)) * 4
        ih = int(r.integers(6, 70))
        pad, dil = [(1, 1), (0, 1), (2, 2), (1, 1)][int(r.integers(0, 4))]
        oh, ow = ih + 2 * pad - 2 * dil, iw + 2 * pad - 2 * dil
        if oh < 1 or ow < 1:
            continue
        n = int(r.integers(1, 9))
        if n * oh * ow < 2048 or n * oh * ow > 60000:
            continue
        ic = int(r.choice([32, 64, 96, 128]))
        oc = int(r.choice([64, 96, 128, 192, 256]))
        act = [A.RELU, A.IDENTITY][int(r.integers(0, 2))]
        out.append(ConvCase(A.FMT_NCHW44, A.DENSE, n, ic, ih, iw, oc, 3, 1, pad, act,
                            scales=(0.02, 0.01, unsat(9 * ic)), dilate=dil))
    return out


SWEEP = _plane_major_sweep()


@pytest.mark.parametrize("case", SWEEP, ids=[repr(c) for c in SWEEP])
def test_plane_major_patch_sweep(case):
    port.set_threads(8)
    arrays = case.gen(seed=23)
    compare(run_gpu(case, arrays), case.run_port(arrays), repr(case))


def _new_kernel_sweep():
    """seeded random layers for the pointwise kernel with any channel counts, the depthwise 5x5 / 7x7
    kernels and the dense 5x5 / 7x7 layers with one filter row per stage: random image sizes (rows
    that are no multiple of 4 or 8 pixels), strides, batches, channel counts, the three activations
    that go through the threshold table and SIGMOID"""
    r = np.random.Generator(np.random.PCG64(77))
    acts = [A.RELU, A.IDENTITY, A.H_SWISH, A.SIGMOID]
    out = []
    for _ in range(10):  # pointwise
        ic, oc = int(r.integers(1, 129)) * 4, int(r.integers(1, 97)) * 4
        ih, iw, n = int(r.integers(3, 40)), int(r.integers(3, 40)), int(r.integers(1, 6))
        act = acts[int(r.integers(0, 4))]
        sc = unsat(ic) * (40 if act == A.SIGMOID else 1)
        out.append(ConvCase(A.FMT_NCHW44, A.DENSE, n, ic, ih, iw, oc, 1, 1, 0, act, scales=(0.02, 0.01, sc)))
    for _ in range(10):  # depthwise 5x5 / 7x7
        k, s = int(r.choice([5, 7])), int(r.integers(1, 3))
        c = int(r.integers(1, 25)) * 4
        ih, iw, n = int(r.integers(1, 45)), int(r.integers(1, 45)), int(r.integers(1, 5))
        act = acts[int(r.integers(0, 4))]
        sc = unsat(k * k) * (40 if act == A.SIGMOID else 1)
        out.append(ConvCase(A.FMT_NCHW44, A.GROUP, n, c, ih, iw, c, k, s, k // 2, act, scales=(0.02, 0.01, sc),
                            bias=bool(r.integers(0, 2))))
    while len(out) < 28:  # dense 5x5 / 7x7 of at least 4096 pixels
        k, s = int(r.choice([5, 7])), int(r.integers(1, 3))
        ic, oc = int(r.integers(1, 13)) * 4, int(r.integers(8, 41)) * 4
        ih, iw, n = int(r.integers(20, 70)), int(r.integers(20, 70)), int(r.integers(2, 9))
        pad = int(r.integers(0, k // 2 + 1))
        oh, ow = (ih + 2 * pad - k) // s + 1, (iw + 2 * pad - k) // s + 1
        if n * oh * ow < 4096 or n * oh * ow > 30000:
            continue
        act = acts[int(r.integers(0, 4))]
        sc = unsat(k * k * ic) * (40 if act == A.SIGMOID else 1)
        out.append(ConvCase(A.FMT_NCHW44, A.DENSE, n, ic, ih, iw, oc, k, s, pad, act, scales=(0.02, 0.01, sc)))
    return out


NEW_SWEEP = _new_kernel_sweep()


@pytest.mark.parametrize("case", NEW_SWEEP, ids=[repr(c) for c in NEW_SWEEP])
def test_pointwise_depthwise_and_row_split_sweep(case):
    port.set_threads(8)
    arrays = case.gen(seed=29)
    got = run_gpu(case, arrays)
    kernel = runtime.last_kernel()
    if case.sparse == A.GROUP:
        assert kernel.startswith("dwconv44_mfma"), kernel
    elif case.fh == 1 and case.ic <= 512:
        assert kernel.startswith("conv_pw_stream"), kernel
    elif case.fh >= 5:
        assert kernel.startswith("conv_mfma_i8_dma:8") or kernel.startswith("conv_mfma_i8_dma:9"), kernel
    compare(got, case.run_port(arrays), repr(case))


def _fully_connected_sweep():
    """seeded random FullyConnected layers of at most 64 rows (K a multiple of 128: 1..4 blocks of K
    per wave, more than 4096, long K under few channels) and f32 products of at most 4 rows with B
    as it lies and transposed"""
    r = np.random.Generator(np.random.PCG64(77))
    acts = [A.IDENTITY, A.RELU, A.H_SWISH, A.SIGMOID]
    out = []
    for i in range(18):
        m, k, oc = int(r.integers(1, 65)), int(r.integers(1, 33)) * 128, int(r.integers(1, 500))
        if i % 6 == 0:
            k, oc = int(r.choice([8192, 12288])), int(r.integers(1, 160))
        act = acts[int(r.integers(0, 4))]
        sc = unsat(k) / 2 * (40 if act == A.SIGMOID else 1)
        out.append(ConvCase(A.FMT_NCHW, A.DENSE, m, k, 1, 1, oc, 1, 1, 0, act, scales=(0.01, 0.01, sc),
                            bias=bool(r.integers(0, 2))))
    for _ in range(8):
        out.append(MatMulCase(int(r.integers(1, 5)), int(r.integers(1, 1500)), int(r.integers(1, 1200)),
                              trans_b=bool(r.integers(0, 2))))
    return out


FC_SWEEP = _fully_connected_sweep()


@pytest.mark.parametrize("case", FC_SWEEP, ids=[repr(c) for c in FC_SWEEP])
def test_fully_connected_sweep(case):
    port.set_threads(8)
    arrays = case.gen(seed=31)
    got = run_gpu(case, arrays)
    kernel = runtime.last_kernel()
    if isinstance(case, MatMulCase):
        assert kernel == "gevm_f32", kernel
    elif case.n <= 4:
        assert kernel == "fc_gevm_q8", kernel
    elif case.ic > 8192:
        assert kernel.startswith("fc_stream"), kernel
    else:
        assert kernel.startswith("fc_one"), kernel
    compare(got, case.run_port(arrays), repr(case))


def _f32_sweep():
    """seeded random f32 convolutions (NCHW and NCHW44; 1x1, 3x3 with and without dilation, 5x5;
    stride 1 / 2; any padding up to k/2 + 1; ragged channel counts and pixel counts, so that the
    implicit GEMM's edge tiles, its last partial stage of K and the small-layer kernel's clamped
    taps all occur) and f32 products of 5..300 rows in all four transpositions, a third of them
    with at most 64 rows and K, N multiples of 64 / 256 (the 64 x 256 tiles with split K)"""
    r = np.random.Generator(np.random.PCG64(99))
    acts = [A.IDENTITY, A.RELU, A.H_SWISH, A.SIGMOID]
    out = []
    for i in range(50):
        k = int(r.choice([1, 3, 3, 5]))
        s = int(r.integers(1, 3))
        dil = int(r.integers(1, 3)) if k == 3 else 1
        ic, oc = int(r.integers(1, 90)), int(r.integers(1, 200))
        ih, iw, n = int(r.integers(5, 60)), int(r.integers(5, 60)), int(r.integers(1, 9))
        pad = int(r.integers(0, k // 2 + 2))
        eh = dil * (k - 1) + 1
        if ih + 2 * pad < eh or iw + 2 * pad < eh:
            continue
        fmt = A.FMT_NCHW
        if i % 5 == 0:
            ic, oc, fmt = (ic + 3) // 4 * 4, (oc + 3) // 4 * 4, A.FMT_NCHW44
        act, bias = acts[int(r.integers(0, 4))], bool(r.integers(0, 2))
        out.append((500 + i, ConvCase(fmt, A.DENSE, n, ic, ih, iw, oc, k, s, pad, act, dtype="f32", bias=bias,
                                      dilate=dil)))
    for i in range(30):
        m, k, n = int(r.integers(5, 300)), int(r.integers(1, 700)), int(r.integers(1, 700))
        if i % 3 == 0:
            m, k, n = int(r.integers(5, 65)), int(r.integers(1, 40)) * 64, int(r.integers(1, 20)) * 256
        out.append((700 + i, MatMulCase(m, k, n, trans_a=bool(r.integers(0, 2)), trans_b=bool(r.integers(0, 2)))))
    return out


F32_SWEEP = _f32_sweep()


@pytest.mark.parametrize("seed,case", F32_SWEEP, ids=["%d_%r" % (s, c) for s, c in F32_SWEEP])
def test_f32_convolution_and_matmul_sweep(seed, case):
    port.set_threads(16)
    arrays = case.gen(seed=seed)
    compare(run_gpu(case, arrays), case.run_port(arrays), repr(case))


def test_direct_kernel_when_filter_was_not_packed():
    """a caller that skips the init protocol still gets the right answer (generic kernel)"""
    import ctypes as C
    case = ConvCase(A.FMT_NCHW44, A.DENSE, 2, 16, 9, 11, 24, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(144)))
    arrays = case.gen(5)
    ins, outs = case.specs(arrays)
    bufs = [runtime.DeviceBuffer.from_array(s.array) for s in ins]
    out = runtime.DeviceBuffer(outs[0].nbytes)
    tin = [abi.make_tensor(b.ptr, s.shape, s.type_enum, s.scale, s.name) for b, s in zip(bufs, ins)]
    tout = [abi.make_tensor(out.ptr, outs[0].shape, outs[0].type_enum, outs[0].scale)]
    attr = case.attr()
    runtime.check(runtime.lib().megcc_gfx950_conv2d(
        C.byref(attr), abi.tensor_array(tin), len(tin), abi.tensor_array(tout), 1, None, None), "conv2d")
    compare(out.to_array(outs[0].shape, np.int8), case.run_port(arrays), "direct")


def test_errors_do_not_launch():
    import ctypes as C
    case = ConvCase(A.FMT_NCHW44, A.DENSE, 1, 8, 6, 6, 8, 3, 1, 1, A.RELU)
    arrays = case.gen(5)
    ins, outs = case.specs(arrays)
    bufs = [runtime.DeviceBuffer.from_array(s.array) for s in ins]
    out = runtime.DeviceBuffer(outs[0].nbytes)
    tin = [abi.make_tensor(b.ptr, s.shape, s.type_enum, s.scale, s.name) for b, s in zip(bufs, ins)]
    bad_shape = list(outs[0].shape)
    bad_shape[2] += 1
    tout = [abi.make_tensor(out.ptr, bad_shape, outs[0].type_enum, outs[0].scale)]
    attr = case.attr()
    st = runtime.lib().megcc_gfx950_conv2d(
        C.byref(attr), abi.tensor_array(tin), len(tin), abi.tensor_array(tout), 1, None, None)
    assert st == abi.ERROR_INVALID_LAYOUT
    # bias scale must equal src*flt scale (ConvGeneral::IsAvailable)
    tin[2].dtype.param.scale = 0.5
    tout = [abi.make_tensor(out.ptr, outs[0].shape, outs[0].type_enum, outs[0].scale)]
    st = runtime.lib().megcc_gfx950_conv2d(
        C.byref(attr), abi.tensor_array(tin), len(tin), abi.tensor_array(tout), 1, None, None)
    assert st == abi.ERROR_UNSUPPORTED_DTYPE_TYPE


@pytest.mark.parametrize("case", [
    ConvCase(A.FMT_NCHW44, A.DENSE, 2, 16, 9, 9, 8, 1, 2, 0, A.RELU, scales=(0.02, 0.01, unsat(16))),
    ConvCase(A.FMT_NCHW, A.DENSE, 2, 16, 20, 24, 12, 3, 1, 1, A.RELU, scales=(0.02, 0.01, unsat(144))),
], ids=["strided_1x1", "dense_nchw"])
def test_layers_that_require_their_workspace_say_so(case):
    """a strided 1x1 NCHW44 layer and a dense layer on plain NCHW tensors run on copies in the
    workspace; once the init protocol has packed the filter for that, a call without the
    workspace (or with a short one) must fail with TinyNN_ERROR_OUT_OF_RANGE and launch nothing"""
    import ctypes as C
    arrays = case.gen(5)
    ins, outs = case.specs(arrays)
    op = runtime.PreparedOp(runtime.parse_symbol(case.symbol()), ins, outs)
    assert op.n_processed == 1 and op.ws.size > 0
    for ws in (None, abi.Workspace(op.ws.ptr, op.ws.size - 1, 0)):
        st = runtime.lib().megcc_gfx950_call(
            C.byref(op.desc), op.ins, len(op.in_tensors), op.outs, len(op.out_tensors),
            C.byref(ws) if ws is not None else None, None)
        assert st == abi.ERROR_OUT_OF_RANGE
        assert b"workspace" in runtime.lib().megcc_gfx950_last_error()
    assert (op.result().view(np.uint8) == cases.POISON).all(), "nothing may have been written"
    op.launch()
    compare(op.result(), case.run_port(arrays), repr(case))


def test_mfma_only_probe_reports_a_plausible_rate():
    """the measurement aid behind bench.py's mfma_only figures: argument checks, the MFMA count of
    a launch, and a rate between a tenth of the published int8 peak and the peak itself"""
    import ctypes as C
    import megcc_amd
    lib = C.CDLL(os.path.join(megcc_amd.PKG_DIR, "libmegcc_bench_probe.so"))
    lib.megcc_bench_probe_mfma_i8.argtypes = [C.c_int, C.c_int, C.c_int, C.POINTER(C.c_double),
                                              C.POINTER(C.c_double)]
    us, n = C.c_double(), C.c_double()
    assert lib.megcc_bench_probe_mfma_i8(3, 256, 10, C.byref(us), C.byref(n)) == 1
    assert lib.megcc_bench_probe_mfma_i8(1, 256, 0, C.byref(us), C.byref(n)) == 1
    assert lib.megcc_bench_probe_mfma_i8(1, 256, 10, None, C.byref(n)) == 1
    for kind in (0, 1, 2):
        assert lib.megcc_bench_probe_mfma_i8(kind, 1024, 20, C.byref(us), C.byref(n)) == 0
        assert n.value == 256 * 4 * 1024, "256 CUs x 4 SIMDs x 1024 MFMAs"
        tops = n.value * 65536 / us.value / 1e6
        assert 500 < tops <= 5000, (kind, us.value, tops)


@pytest.mark.parametrize("scales", [(0.02, 0.01, 0.025), (0.02, 0.01, 0.05), (0.5, 0.5, 64.0)],
                         ids=["c0.008", "c0.004_exact_ties", "c_2^-8_exact_ties"])
@pytest.mark.parametrize("act", [A.IDENTITY, A.RELU, A.H_SWISH], ids=["IDENTITY", "RELU", "H_SWISH"])
def test_every_accumulator_value_requantises_like_the_literal_sequence(act, scales):
    """the threshold-table requantisation over a contiguous range of accumulators: a 1x1 layer whose
    accumulator is 127 * (y - 128) + (x - 128) + bias at pixel (y, x), i.e. every integer in
    [-16384, 16383] (plus 64 different bias offsets), against the literal float sequence of the
    oracle - all 127 / 255 thresholds of the first scale triple lie inside that range, the other
    two put an exact tie at every 125th / 128th accumulator"""
    case = ConvCase(A.FMT_NCHW44, A.DENSE, 1, 32, 256, 256, 64, 1, 1, 0, act, scales=scales)
    arrays = case.gen(3)
    arrays["src"][...] = 0
    arrays["flt"][...] = 0
    ramp = np.arange(-128, 128, dtype=np.int8)
    arrays["src"][0, 0, :, :, 0] = ramp[:, None]
    arrays["src"][0, 0, :, :, 1] = ramp[None, :]
    arrays["flt"][:, 0, 0, 0, 0, :] = 127
    arrays["flt"][:, 0, 0, 0, 1, :] = 1
    arrays["bias"][...] = (np.arange(64, dtype=np.int32) * 37 - 1000).reshape(arrays["bias"].shape)
    ins, outs = case.specs(arrays)
    op = runtime.PreparedOp(runtime.parse_symbol(case.symbol()), ins, outs)
    op.launch()
    got, want = op.result(), case.run_port(arrays)
    if scales[2] == 0.025:
        assert len(np.unique(want)) == (128 if act != A.IDENTITY else 256), "the range must cover every threshold"
    compare(got, want, repr(case))


# ---- depthwise 3x3 -> max-pool 2x2 s2 -> QADD / QFUSE_ADD_RELU in one kernel ------------------------
CHAINS = [
    # (n, c, ih, iw, stride, conv activation, add mode, bias): the four shapes of the bandwidth-bound
    # configuration at a small batch, odd extents (the pooling drops the last row / column), rows that
    # are no multiple of 4 / 8 pixels, one pooled pixel, every activation, both additions, no bias
    (2, 32, 112, 112, 1, A.RELU, A.Q_FUSE_ADD_RELU, True), (2, 32, 112, 112, 2, A.RELU, A.Q_FUSE_ADD_RELU, True),
    (3, 512, 14, 14, 1, A.RELU, A.Q_FUSE_ADD_RELU, True), (3, 512, 14, 14, 2, A.RELU, A.Q_FUSE_ADD_RELU, True),
    (2, 8, 13, 19, 1, A.IDENTITY, A.Q_ADD, True), (2, 12, 21, 30, 2, A.H_SWISH, A.Q_ADD, False),
    (1, 4, 2, 2, 1, A.SIGMOID, A.Q_FUSE_ADD_RELU, True), (3, 20, 9, 6, 1, A.RELU, A.Q_ADD, False),
    (2, 16, 11, 37, 2, A.IDENTITY, A.Q_FUSE_ADD_RELU, True), (1, 8, 5, 3, 1, A.RELU, A.Q_FUSE_ADD_RELU, True),
]


def _chain_cases(n, c, ih, iw, stride, act, mode, bias):
    sc = unsat(9) * (40 if act == A.SIGMOID else 1)
    s_src, s_flt = 0.02, 0.01
    if n % 2 == 0:
        # scales without exact ties: IDENTITY / RELU then requantise by the proven multiply-add, the
        # odd batches (0.02 * 0.01 / ...: ties at every 125th accumulator or so) by threshold table
        s_src, s_flt, sc = 0.0213, 0.0097, sc * 1.0371
    dw = ConvCase(A.FMT_NCHW44, A.GROUP, n, c, ih, iw, c, 3, stride, 1, act, scales=(s_src, s_flt, sc), bias=bias)
    pool = PoolCase(A.FMT_NCHW44, A.POOL_MAX, n, c, dw.oh, dw.ow, 2, 2, 0, scale=sc)
    add = MultiTypeCase(mode, pool.dst_shape(), (sc, 0.013, 0.9 * sc))
    return dw, pool, add


@pytest.mark.parametrize("cfg", CHAINS, ids=["n%d_c%d_%dx%d_s%d_%s_%s%s" % (
    c[0], c[1], c[2], c[3], c[4], A.NONLINE_NAMES[c[5]], A.MULTITYPE_NAMES[c[6]], "" if c[7] else "_nobias")
    for c in CHAINS])
def test_depthwise_pool_add_in_one_kernel_equals_the_three_operator_chain(cfg):
    """megcc_gfx950_dw_pool_add against the oracle's depthwise convolution, pooling and addition run
    one after the other, bit for bit"""
    import ctypes as C
    dw, pool, add = _chain_cases(*cfg)
    arrays = dw.gen(11)
    other = np.random.default_rng(12).integers(-128, 128, pool.dst_shape()).astype(np.int8)
    want = add.run_port({"a": pool.run_port({"src": dw.run_port(arrays)}), "b": other})
    attr = abi.DwPoolAddAttr()
    attr.conv = dw.attr()
    attr.pool = abi.PoolAttr(2, 2, 2, 2, 0, 0, A.FMT_NCHW44, A.POOL_MAX)
    attr.mode = cfg[6]
    attr.mid_scale = dw.scales[2]
    ins, _ = dw.specs(arrays)
    bufs = [runtime.DeviceBuffer.from_array(s.array) for s in ins] + [runtime.DeviceBuffer.from_array(other)]
    out = runtime.DeviceBuffer(want.nbytes)
    out.fill(cases.POISON)
    tin = [abi.make_tensor(b.ptr, s.shape, s.type_enum, s.scale, s.name) for b, s in zip(bufs, ins)]
    tin.append(abi.make_tensor(bufs[-1].ptr, pool.dst_shape(), abi.QINT8, add.scales[1], b"other"))
    tout = [abi.make_tensor(out.ptr, pool.dst_shape(), abi.QINT8, add.scales[2], b"dst")]
    L = runtime.lib()
    L.megcc_gfx950_dw_pool_add_supported.argtypes = [
        C.POINTER(abi.DwPoolAddAttr), C.POINTER(C.POINTER(abi.Tensor)), C.c_int, C.POINTER(C.POINTER(abi.Tensor)), C.c_int]
    L.megcc_gfx950_dw_pool_add.argtypes = L.megcc_gfx950_dw_pool_add_supported.argtypes + [C.c_void_p, C.c_void_p]
    assert L.megcc_gfx950_dw_pool_add_supported(C.byref(attr), abi.tensor_array(tin), len(tin), abi.tensor_array(tout), 1) == 1
    runtime.check(L.megcc_gfx950_dw_pool_add(C.byref(attr), abi.tensor_array(tin), len(tin), abi.tensor_array(tout), 1,
                                             None, None), "dw_pool_add")
    runtime.wait()
    got = out.to_array(want.shape, np.int8)
    compare(got, want, repr(dw))
    # what the entry point refuses: a 5x5 window, average pooling, a second operand of another shape
    attr.pool.mode = A.POOL_AVERAGE
    assert L.megcc_gfx950_dw_pool_add_supported(C.byref(attr), abi.tensor_array(tin), len(tin), abi.tensor_array(tout), 1) == 0
    assert L.megcc_gfx950_dw_pool_add(C.byref(attr), abi.tensor_array(tin), len(tin), abi.tensor_array(tout), 1,
                                      None, None) == abi.ERROR_INVALID_LAYOUT
    for b in bufs + [out]:
        b.free()


def _chain_model(cfg, fused):
    dw, pool, add = _chain_cases(*cfg)
    arrays = dw.gen(11)
    other = np.random.default_rng(12).integers(-128, 128, pool.dst_shape()).astype(np.int8)
    runtime.set_option("nofusechain", 0 if fused else 1)
    try:
        m = runtime.Model()
        x = m.tensor("x", dw.src_shape(), abi.QINT8, dw.scales[0])
        y = m.tensor("other", pool.dst_shape(), abi.QINT8, add.scales[1])
        m.mark_input(x)
        m.mark_input(y)
        ins = [x, m.weight("dw.w", arrays["flt"], abi.QINT8, dw.scales[1])]
        if dw.bias:
            ins.append(m.weight("dw.b", arrays["bias"], abi.QINT32, float(np.float32(dw.scales[0]) * np.float32(dw.scales[1]))))
        t1 = m.tensor("dw", dw.dst_shape(), abi.QINT8, dw.scales[2])
        m.opr(dw.symbol(), ins, [t1])
        t2 = m.tensor("pool", pool.dst_shape(), abi.QINT8, dw.scales[2])
        m.opr(pool.symbol(), [t1], [t2])
        t3 = m.tensor("out", pool.dst_shape(), abi.QINT8, add.scales[2])
        m.opr(add.symbol(), [y, t2] if cfg[0] & 1 else [t2, y], [t3])  # (the pooled tensor on either side)
        m.mark_output(t3)
        m.finalize()
    finally:
        runtime.set_option("nofusechain", 0)
    m.set_input(x, arrays["src"])
    m.set_input(y, other)
    outs = []
    for _ in range(3):  # eager, captured, replayed
        m.forward()
        runtime.wait()
        outs.append(m.get(t3).copy())
    kernel = runtime.last_kernel()
    want = add.run_port({"a": pool.run_port({"src": dw.run_port(arrays)}), "b": other})
    return outs, kernel, want


@pytest.mark.parametrize("cfg", CHAINS[:6], ids=[str(i) for i in range(6)])
def test_model_runtime_fuses_the_depthwise_pool_add_chain(cfg):
    fused, kernel, want = _chain_model(cfg, True)
    assert kernel.startswith("dwconv44_chain"), kernel
    plain, kernel, _ = _chain_model(cfg, False)
    assert not kernel.startswith("dwconv44_chain"), kernel
    for o in fused + plain:
        compare(o, want, "chain %r" % (cfg,))


# ---- operator chains that run as one kernel, under memory plans made for the separate operators ----
# A static plan gives a tensor's bytes to the next tensor born after its last reader. For the chain
# depthwise -> pool -> add that is the add's result over the depthwise INPUT (dead after operator i,
# result born at i + 2); for the soft-max chain the result over the logits. The one-kernel forms read
# those inputs while they write the result, so the model runtime must keep the operators apart when
# the plan it was given overlaps them.
def _planned_chain(out_offset):
    n, c, hw = 2, 16, 12
    dw, pool, add = _chain_cases(n, c, hw, hw, 1, A.RELU, A.Q_FUSE_ADD_RELU, True)
    arrays = dw.gen(21)
    x0 = np.random.default_rng(22).integers(-128, 128, dw.src_shape()).astype(np.int8)
    other = np.random.default_rng(23).integers(-128, 128, pool.dst_shape()).astype(np.int8)
    pre = MultiTypeCase(A.Q_RELU, dw.src_shape(), (0.03, 0.01, dw.scales[0]))
    m = runtime.Model()
    t_in = m.tensor("x0", dw.src_shape(), abi.QINT8, 0.03)
    t_other = m.tensor("other", pool.dst_shape(), abi.QINT8, add.scales[1])
    m.mark_input(t_in)
    m.mark_input(t_other)
    t_x = m.tensor("x", dw.src_shape(), abi.QINT8, dw.scales[0])  # an arena tensor that dies at the depthwise layer
    m.opr(pre.symbol(), [t_in], [t_x])
    w = m.weight("dw.w", arrays["flt"], abi.QINT8, dw.scales[1])
    b = m.weight("dw.b", arrays["bias"], abi.QINT32, float(np.float32(dw.scales[0]) * np.float32(dw.scales[1])))
    t1 = m.tensor("dw", dw.dst_shape(), abi.QINT8, dw.scales[2])
    m.opr(dw.symbol(), [t_x, w, b], [t1])
    t2 = m.tensor("pool", pool.dst_shape(), abi.QINT8, dw.scales[2])
    m.opr(pool.symbol(), [t1], [t2])
    t3 = m.tensor("out", pool.dst_shape(), abi.QINT8, add.scales[2])
    m.opr(add.symbol(), [t2, t_other], [t3])
    m.mark_output(t3)
    nx = int(np.prod(dw.src_shape()))
    up = lambda v: (v + 255) // 256 * 256
    offs = [0] * 8
    offs[t_x], offs[t1] = 0, up(nx)
    offs[t2] = offs[t1] + up(nx)
    offs[t3] = out_offset if out_offset is not None else offs[t2] + up(nx)
    m.set_plan(offs[:t3 + 1], offs[t2] + 2 * up(nx))
    m.finalize()
    m.set_input(t_in, x0)
    m.set_input(t_other, other)
    outs = []
    for _ in range(3):
        m.forward()
        runtime.wait()
        outs.append(m.get(t3).copy())
    x = pre.run_port({"a": x0, "b": None})
    arrays["src"] = x
    want = add.run_port({"a": pool.run_port({"src": dw.run_port(arrays)}), "b": other})
    nk = m.nr_kernel
    m.close()
    return outs, nk, want


@pytest.mark.parametrize("out_offset,kernels", [(None, 2), (0, 4), (256, 4), (4352, 4)],
                         ids=["apart", "result_on_the_input", "result_256_bytes_into_the_input", "result_over_the_input_tail"])
def test_chain_is_one_kernel_only_when_its_result_shares_no_byte_with_its_inputs(out_offset, kernels):
    outs, nk, want = _planned_chain(out_offset)
    assert nk == kernels
    for o in outs:
        compare(o, want, "planned chain, result at %r" % (out_offset,))


def _planned_softmax(front, y_on):
    """soft-max chain behind `front`: "cvt" = f32 -> qsi8 -> f32 typecvts (the dequantising one can join
    the one-kernel form, which then reads the qsi8 logits), "neg" = an f32 NEGATE (the kernel reads
    the f32 logits x); the result y is planned apart, or over q / x"""
    rows, cols = 8, 1000
    rng = np.random.default_rng(31)
    logits = (rng.standard_normal((rows, cols)) * 3).astype(np.float32)
    big = 32768  # rows * cols * 4 rounded up to 256
    m = runtime.Model()
    t_in = m.tensor("in", (rows, cols), abi.FLOAT)
    m.mark_input(t_in)
    place = {}
    if front == "cvt":
        q = m.tensor("q", (rows, cols), abi.QINT8, 0.1)
        m.opr("GI_kernel_typecvt_f32qsi8", [t_in], [q])
        x = m.tensor("x", (rows, cols), abi.FLOAT)
        m.opr("GI_kernel_typecvt_qsi8f32", [q], [x])
        place[q] = 0
        xv = np.clip(np.round(logits / np.float32(0.1)), -128, 127).astype(np.float32) * np.float32(0.1)
    else:
        x = m.tensor("x", (rows, cols), abi.FLOAT)
        m.opr("kernel_elementwise_NEGATE_f32f32", [t_in], [x])
        xv = -logits
    mx = m.tensor("sm.max", (rows, 1), abi.FLOAT)
    m.opr("kernel_reduce_MAX_DEFAULT_a1_f32f32", [x], [mx])
    sub = m.tensor("sm.sub", (rows, cols), abi.FLOAT)
    m.opr("kernel_elementwise_SUB_f32f32f32", [x, mx], [sub])
    ex = m.tensor("sm.exp", (rows, cols), abi.FLOAT)
    m.opr("kernel_elementwise_EXP_f32f32", [sub], [ex])
    sm = m.tensor("sm.sum", (rows, 1), abi.FLOAT)
    m.opr("kernel_reduce_SUM_DEFAULT_a1_f32f32", [ex], [sm])
    y = m.tensor("softmax", (rows, cols), abi.FLOAT)
    m.opr("kernel_elementwise_TRUE_DIV_f32f32f32", [ex, sm], [y])
    m.mark_output(y)
    place.update({x: big, mx: 2 * big, sub: 3 * big, ex: 4 * big, sm: 5 * big})
    place[y] = {"apart": 6 * big, "q_shifted": 256, "x_exact": big, "x_shifted": big + 4096}[y_on]
    m.set_plan([place.get(t, 0) for t in range(y + 1)], 8 * big)
    m.finalize()
    m.set_input(t_in, logits)
    outs = []
    for _ in range(3):
        m.forward()
        runtime.wait()
        outs.append(m.get(y).copy())
    nk = m.nr_kernel
    m.close()
    e = np.exp(xv.astype(np.float64) - xv.max(axis=1, keepdims=True))
    return outs, nk, (e / e.sum(axis=1, keepdims=True)).astype(np.float32)


@pytest.mark.parametrize("front,y_on,kernels", [
    ("cvt", "apart", 2), ("cvt", "q_shifted", 3), ("cvt", "x_shifted", 2),
    ("neg", "apart", 2), ("neg", "x_exact", 2), ("neg", "x_shifted", 6)])
def test_softmax_is_one_kernel_only_when_its_result_cannot_overwrite_unread_logits(front, y_on, kernels):
    """cvt/apart: the dequantising typecvt and the five operators are one kernel reading the qsi8
    logits; result over the qsi8 logits: that typecvt stays an operator and the kernel reads the f32
    logits; result over the f32 logits while the kernel reads the qsi8 ones: nothing it reads is
    touched. neg: the kernel reads the f32 logits x; a result exactly on x is fine (a row is read
    whole before it is written), a result shifted into x is not: the five operators run one by one"""
    outs, nk, want = _planned_softmax(front, y_on)
    assert nk == kernels
    for o in outs:
        assert cases.max_rel_err(o, want) <= 1e-5, (front, y_on)
