"""Host-side bounds audit of the kernels that issue their loads unconditionally from clamped
indices (gemm_f32: all four transpositions and the implicit-GEMM gather; gevm_f32; conv_f32_small; the
f32 NCHW44 channel-wise and first-layer kernels; fc_one32 / fc_one; fc_gevm_q8). tests/host_audit/audit.cpp links the library's own kernel sources,
compiled as host C++ against a stand-in HIP header that runs every thread of every workgroup on
the CPU, and fences each operand buffer with inaccessible pages: one element outside a tensor ends
the run. No GPU involved; the shapes are every case of the GPU sweeps plus a seeded sweep of ragged
shapes aimed at the tile edges."""
import ctypes as C
import os
import shutil
import subprocess

import numpy as np
import pytest

from cases import ConvCase, MatMulCase
from megcc_amd import abi, runtime

HERE = os.path.dirname(os.path.abspath(__file__))
AUDIT_DIR = os.path.join(HERE, "host_audit")
CSRC = os.path.join(os.path.dirname(HERE), "megcc_amd", "csrc")
CLANG = "/opt/rocm/llvm/bin/clang++"
SOURCES = ["gemm_f32", "gevm_f32", "conv_f32_small", "conv_f32_nchw44", "fc_stream", "fc_gevm_q8"]

pytestmark = pytest.mark.skipif(not os.path.exists(CLANG), reason="needs ROCm's clang++ for the kernels' vector types")


def compile_audit(out_dir, replace=None):
    """replace: {source name: path of another file to compile in its place}"""
    os.makedirs(out_dir, exist_ok=True)
    flags = ["-x", "c++", "-std=c++17", "-O1", "-g", "-I" + AUDIT_DIR, "-I" + CSRC,
             "-I" + os.path.join(os.path.dirname(HERE), "include"), "-ffp-contract=off", "-Wno-unknown-attributes"]
    objs = []
    jobs = []
    for name in SOURCES + ["audit"]:
        src = os.path.join(AUDIT_DIR, "audit.cpp") if name == "audit" else os.path.join(CSRC, name + ".hip")
        if replace and name in replace:
            src = replace[name]
        obj = os.path.join(out_dir, name + ".o")
        objs.append(obj)
        jobs.append(subprocess.Popen([CLANG] + flags + ["-c", src, "-o", obj], stderr=subprocess.PIPE, text=True))
    for j in jobs:
        err = j.communicate()[1]
        assert j.returncode == 0, err[-4000:]
    exe = os.path.join(out_dir, "audit")
    subprocess.check_call([CLANG, "-o", exe] + objs)
    return exe


@pytest.fixture(scope="module")
def audit_exe(tmp_path_factory):
    return compile_audit(str(tmp_path_factory.mktemp("host_audit")))


def packed_bytes(case):
    """size of the packed filter the layer's init step produces (host code of the library)"""
    arrays = {"src": None}
    desc = runtime.parse_symbol(case.symbol())
    tin = [abi.make_tensor(None, case.src_shape(), abi.QINT8, case.scales[0], b"src"),
           abi.make_tensor(None, case.flt_shape(), abi.QINT8, case.scales[1], b"flt")]
    if case.bias:
        tin.append(abi.make_tensor(None, case.bias_shape(), abi.QINT32, case.scales[0] * case.scales[1], b"bias"))
    w = abi.Tensor()
    runtime.check(runtime.lib().megcc_gfx950_call_init(C.byref(desc), abi.tensor_array(tin), len(tin), C.byref(w),
                                                       None, None), "init(describe)")
    n = 1
    for i in range(w.layout.nr_dim):
        n *= w.layout.dims[i]
    return n


def line_of(case, with_ws=1):
    if isinstance(case, MatMulCase):
        return "mm %d %d %d %d %d 0 0 %d" % (case.m, case.k, case.n, case.trans_a, case.trans_b, with_ws)
    assert isinstance(case, ConvCase)
    if case.dtype == "f32":
        macs = case.n * case.oh * case.ow * case.oc * case.ic * case.fh * case.fw
        small = case.fh in (1, 3) and case.fh == case.fw and macs <= 2 ** 27
        kind = "small" if small else "conv"
        tail = "" if small else " %d" % with_ws
        return "%s %d %d %d %d %d %d %d %d %d %d%s" % (kind, case.n, case.ic, case.ih, case.iw, case.oc, case.fh,
                                                       case.sh, case.ph, case.dh, int(case.bias), tail)
    kind = "fcgevm" if case.n <= 4 else "fcone"
    return "%s %d %d %d %d %d" % (kind, case.n, case.ic, case.oc, packed_bytes(case), int(case.bias))


def audit_lines():
    import test_gpu_parity as gp
    lines = []
    for _, case in gp.F32_SWEEP:
        if isinstance(case, ConvCase) and case.fmt != abi.FMT_NCHW:
            continue  # (NCHW44 layers reach the same kernel through relayouts of dense copies)
        lines.append(line_of(case))
    for case in gp.FC_SWEEP:
        if isinstance(case, ConvCase) and case.ic > 8192:
            continue  # (fc_stream: loads under range tests, not audited here)
        lines.append(line_of(case))
    r = np.random.Generator(np.random.PCG64(2024))
    # MatMul: every transposition x {inside, ragged} x {with, without split-K room}, padded rows, skinny tiles
    for i in range(40):
        m = int(r.choice([1, 2, 3, 4, 5, 31, 64, 65, 127, 128, 129, 200]))
        k = int(r.choice([1, 2, 15, 16, 17, 64, 100, 128, 513, 1040, 2049]))
        n = int(r.choice([1, 3, 4, 5, 63, 127, 128, 129, 255, 256, 257, 1000, 1024]))
        lines.append("mm %d %d %d %d %d %d %d %d" % (m, k, n, r.integers(0, 2), r.integers(0, 2),
                                                       r.choice([0, 1, 4, 7]), r.choice([0, 1, 4, 7]), r.integers(0, 2)))
    # implicit GEMM: pixel counts around multiples of the 128 / 256 pixel tiles, ragged K, few channels
    for i in range(24):
        k = int(r.choice([1, 3, 5]))
        s, d = int(r.integers(1, 3)), int(r.integers(1, 3)) if k == 3 else 1
        p = int(r.integers(0, k // 2 + 2))
        ic, oc = int(r.choice([1, 3, 16, 33, 64, 100])), int(r.choice([1, 5, 63, 64, 65, 128, 130]))
        ih, iw, n = int(r.integers(6, 40)), int(r.integers(6, 40)), int(r.integers(1, 6))
        if ih + 2 * p < d * (k - 1) + 1 or iw + 2 * p < d * (k - 1) + 1:
            continue
        lines.append("conv %d %d %d %d %d %d %d %d %d %d %d" % (n, ic, ih, iw, oc, k, s, p, d, r.integers(0, 2),
                                                               r.integers(0, 2)))
    lines.append("conv 3 86 45 42 117 5 2 3 1 1 1")  # 1584 = 12 x 128 + 48 pixels: the ragged last tile once read past the tensor
    # small layers: one pixel, one channel, rows shorter than the window, strides, dilation
    for (n, ic, ih, iw, oc, k, s, p, d) in [(1, 1, 1, 1, 1, 1, 1, 0, 1), (1, 1, 3, 3, 1, 3, 1, 1, 1), (2, 3, 5, 7, 5, 3, 2, 1, 1),
                                            (1, 32, 56, 56, 32, 3, 1, 1, 1), (3, 7, 9, 11, 13, 3, 1, 2, 2), (1, 5, 2, 2, 3, 3, 1, 1, 1),
                                            (4, 9, 17, 3, 6, 1, 2, 0, 1), (1, 64, 13, 13, 66, 3, 1, 0, 1), (5, 2, 8, 64, 3, 3, 2, 1, 2)]:
        lines.append("small %d %d %d %d %d %d %d %d %d 1" % (n, ic, ih, iw, oc, k, s, p, d))
    # f32 NCHW44: channel-wise tiles of 4 x 64 pixels with halos, first layers of 256-pixel blocks
    for _, case in gp.F32_NCHW44:
        if case.sparse == abi.GROUP and case.fh in (3, 5):
            lines.append("dwf32 %d %d %d %d %d %d %d %d" % (case.n, case.ic, case.ih, case.iw, case.fh, case.sh,
                                                          case.ph, int(case.bias)))
        elif case.fmt == abi.FMT_NCHW_NCHW44:
            lines.append("first %d %d %d %d %d %d %d %d %d" % (case.n, case.ic, case.ih, case.iw, case.oc, case.fh,
                                                             case.sh, case.ph, int(case.bias)))
    for i in range(16):
        k, s = int(r.choice([3, 5])), int(r.integers(1, 3))
        ih, iw = int(r.integers(1, 20)), int(r.choice([1, 2, 63, 64, 65, 127, 129, 200]))
        p = int(r.integers(0, k // 2 + 2))
        if ih + 2 * p < k or iw + 2 * p < k:
            continue
        lines.append("dwf32 %d %d %d %d %d %d %d %d" % (r.integers(1, 4), 4 * r.integers(1, 5), ih, iw, k, s, p,
                                                      r.integers(0, 2)))
    for i in range(12):
        k, s = int(r.choice([3, 5, 7])), int(r.integers(1, 3))
        ih, iw = int(r.integers(3, 40)), int(r.integers(3, 70))
        p = int(r.integers(0, k // 2 + 2))
        if ih + 2 * p < k or iw + 2 * p < k:
            continue
        lines.append("first %d %d %d %d %d %d %d %d %d" % (r.integers(1, 4), r.integers(1, 5), ih, iw,
                                                         4 * r.choice([1, 2, 8, 9, 16]), k, s, p, r.integers(0, 2)))
    # qsi8 FullyConnected: 1..64 rows, K = 1..32 blocks of 128 (and beyond 4096), channel counts off every tile size
    for i in range(24):
        m = int(r.choice([1, 2, 3, 4, 5, 31, 32, 33, 63, 64]))
        k = int(r.choice([128, 256, 384, 512, 1024, 2048, 4096, 4224, 8192])) if m > 4 else int(r.choice([1, 31, 32, 33, 100, 1024, 4095]))
        oc = int(r.choice([1, 3, 31, 32, 33, 63, 64, 65, 255, 256, 257, 1000]))
        case = ConvCase(abi.FMT_NCHW, abi.DENSE, m, k, 1, 1, oc, 1, 1, 0, abi.RELU, scales=(0.01, 0.01, 0.1),
                        bias=bool(r.integers(0, 2)))
        lines.append(line_of(case))
    return lines


def test_every_load_and_store_of_the_clamped_kernels_stays_inside_its_tensor(audit_exe):
    lines = audit_lines()
    assert len(lines) > 150
    r = subprocess.run([audit_exe], input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=1500)
    assert r.returncode == 0, "bounds audit failed:\n%s\n%s" % (r.stdout[-1500:], r.stderr[-3000:])
    assert "audited %d cases" % len(lines) in r.stdout


def test_the_audit_sees_the_out_of_bounds_read_a_missing_clamp_causes(audit_exe, tmp_path):
    """the audit itself, pinned by a mutation: without the clamp of the gather's column the surplus
    columns of a ragged last pixel tile read up to one image past the tensor; the audit must die on it"""
    src = open(os.path.join(CSRC, "gemm_f32.hip")).read()
    clamp = "const int cn = min(n0 + tid % BN, q.N - 1);"
    assert src.count(clamp) == 1
    mutated = tmp_path / "gemm_f32.hip"
    mutated.write_text(src.replace(clamp, "const int cn = n0 + tid % BN;"))
    exe = compile_audit(str(tmp_path / "build"), replace={"gemm_f32": str(mutated)})
    r = subprocess.run([exe], input="conv 3 86 45 42 117 5 2 3 1 1 1\n", capture_output=True, text=True, timeout=300)
    assert r.returncode == 3 and "OUT OF BOUNDS" in r.stderr, (r.returncode, r.stderr[-500:])
