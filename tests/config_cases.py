"""The benchmark configurations at their own sizes (batch 1 where the full batch would take the
reference's scalar CPU kernels minutes), as cases whose expected outputs come from the
reference's generated kernels: tests/golden/make_config_digests.py runs them through
oracle/_ref and stores a SHA-256 of every qsi8 output and a strided sample of every f32 output;
tests/test_config_digests.py holds the C restatement (CPU) and the HIP library (GPU) to them.

Inputs are not stored: they are drawn from the seeded generator of each case, the same way on
every machine (numpy's PCG64 stream is specified bit for bit)."""
import hashlib

import numpy as np

import cases
from cases import ConvCase, MatMulCase, MultiTypeCase, PoolCase
from golden_cases import unsat
from megcc_amd import abi

A = abi
F32_SAMPLES = 4096


def digest(a):
    a = np.ascontiguousarray(a)
    return hashlib.sha256(a.tobytes()).hexdigest()


def sample(a):
    """every k-th element of the flattened array, at most F32_SAMPLES + 1 of them, plus the last"""
    flat = np.ascontiguousarray(a).reshape(-1)
    step = max(1, flat.size // F32_SAMPLES)
    return np.concatenate([flat[::step], flat[-1:]])


def ref_symbol(case):
    """the kernel MegCC's x86 registry selects for the case (the names tests/golden/symbols.json
    records for the small cases of the same operators)"""
    if isinstance(case, ConvCase) and case.dtype == "f32":
        assert (case.fmt, case.fh, case.sh, case.ph, case.act) == (A.FMT_NCHW, 3, 1, 1, A.RELU)
        return "GI_kernel_conv2d_im2col_3x3_NCHW_DENSE_p1x1_s1x1_d1x1_bias_RELUf32"
    if isinstance(case, MatMulCase):
        return "GI_kernel_gevm_nn" if case.m <= 4 else "GI_kernel_fp32_matmul_4x12_nn"
    return case.symbol()


def single_cases():
    """name -> (case, seed): operators evaluated on their own seeded inputs"""
    out = {}
    out["cfg1_conv_f32_n1_c32_56x56"] = (
        ConvCase(A.FMT_NCHW, A.DENSE, 1, 32, 56, 56, 32, 3, 1, 1, A.RELU, dtype="f32"), 0)
    for c in (64, 256):
        for hw in (56, 28):
            for act, ds, tag in ((A.RELU, 0.05, "baseline"), (A.IDENTITY, unsat(9 * c), "unsat")):
                out["cfg2_conv3x3_n1_c%d_%dx%d_%s_%s" % (c, hw, hw, A.NONLINE_NAMES[act], tag)] = (
                    ConvCase(A.FMT_NCHW44, A.DENSE, 1, c, hw, hw, c, 3, 1, 1, act,
                             scales=(0.02, 0.01, ds)), 100 + c + hw)
    for m, k, n in ((1, 1024, 1000), (64, 4096, 4096)):
        for ds, tag in ((0.1, "baseline"), (unsat(k) / 2, "unsat")):
            out["cfg3_fc_q8_%dx%dx%d_%s" % (m, k, n, tag)] = (
                ConvCase(A.FMT_NCHW, A.DENSE, m, k, 1, 1, n, 1, 1, 0, A.IDENTITY,
                         scales=(0.01, 0.01, ds)), 200 + m)
        out["cfg3_matmul_f32_%dx%dx%d" % (m, k, n)] = (MatMulCase(m, k, n), 300 + m)
    return out


CHAINS = [(32, 112, 1), (32, 112, 2), (512, 14, 1), (512, 14, 2)]


def chain_stages(c, hw, stride, run):
    """configs[3] at N=1: depthwise 3x3 (baseline scales, and the unsaturated twin that feeds the
    rest) -> max-pool 2x2 s2 -> add + ReLU requantised. `run(case, arrays)` evaluates one operator;
    yields (stage name, output)."""
    dw = ConvCase(A.FMT_NCHW44, A.GROUP, 1, c, hw, hw, c, 3, stride, 1, A.RELU, scales=(0.02, 0.01, 0.05))
    arrays = dw.gen(seed=400 + c + hw + stride)
    yield "dw_baseline", run(dw, arrays)
    dwu = ConvCase(A.FMT_NCHW44, A.GROUP, 1, c, hw, hw, c, 3, stride, 1, A.RELU,
                   scales=(0.02, 0.01, unsat(9)))
    y = run(dwu, arrays)
    yield "dw_unsat", y
    pool = PoolCase(A.FMT_NCHW44, A.POOL_MAX, 1, c, dwu.oh, dwu.ow, 2, 2, 0, scale=dwu.scales[2])
    z = run(pool, {"src": y})
    yield "pool", z
    add = MultiTypeCase(A.Q_FUSE_ADD_RELU, z.shape, (dwu.scales[2], 0.01, 0.05))
    other = cases.rng(500 + c + hw + stride).integers(-128, 128, z.shape).astype(np.int8)
    yield "add_relu", run(add, {"a": z, "b": other})


def chain_name(c, hw, stride):
    return "cfg4_chain_n1_c%d_%dx%d_s%d" % (c, hw, hw, stride)
