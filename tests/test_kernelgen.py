"""The compile-time half of the boundary: the gfx950 KernelGen target (megcc_amd/kernelgen) must
pick a kernel for every operator of the path, name it as MegCC's own registry does, and emit C
shims that compile against the public header and link against the library."""
import ctypes as C
import json
import os
import subprocess

import numpy as np
import pytest

import cases
from golden_cases import golden_cases, unsat
from megcc_amd import abi, runtime

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
KG = os.path.join(ROOT, "megcc_amd", "kernelgen")


@pytest.fixture(scope="module")
def emitted(tmp_path_factory):
    out = tmp_path_factory.mktemp("shims")
    subprocess.check_call(["make", "-s", "-C", KG])
    subprocess.check_call([os.path.join(KG, "kernelgen_tool"),
                           os.path.join(ROOT, "oracle", "ref_kernels.spec"), str(out)])
    manifest = dict(line.split() for line in open(out / "manifest.txt"))
    return out, manifest


def test_every_operator_of_the_path_has_a_kernel(emitted):
    _, manifest = emitted
    assert len(manifest) >= 50
    assert "NONE" not in manifest.values()


def test_quantized_symbols_equal_the_reference_registry(emitted):
    _, manifest = emitted
    with open(os.path.join(HERE, "golden", "symbols.json")) as f:
        ref = json.load(f)
    checked = 0
    for label, sym in ref.items():
        if "qsi" in sym:  # f32 kernels use the BAREMETAL template's name, see Gfx950Kernels.cpp
            assert manifest[label] == sym, label
            checked += 1
    assert checked >= 35


REFERENCE = "/root/reference"


@pytest.mark.skipif(not os.path.isdir(os.path.join(REFERENCE, "compiler", "lib", "KernelGen")),
                    reason="needs the reference tree (its headers and its KernelGen registry)")
def test_target_builds_against_the_reference_headers_and_agrees_with_its_registry():
    """Gfx950Kernels.cpp compiled with -DMEGCC_GFX950_IN_TREE derives from the reference's own
    KernelFunc and reads its TContext; oracle/ref_intree_check.cpp then asks both registries for
    every operator of the spec: each gfx950 symbol must be the symbol of an available
    Arch::BAREMETAL kernel for the same context, the texts must be produced from the reference's
    attribute bag without a missing key, the workspace text must be self-contained C, and
    GetKernelSymbol(nullptr) must return for every kernel."""
    oracle = os.path.join(ROOT, "oracle")
    subprocess.check_call(["make", "-s", "-C", oracle, "REF=" + REFERENCE, "_ref/intree_check"])
    r = subprocess.run([os.path.join(oracle, "_ref", "intree_check"),
                        os.path.join(oracle, "ref_kernels.spec")], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-1000:]
    summary = dict(kv.split("=") for kv in r.stdout.strip().splitlines()[-1].split()[1:])
    assert int(summary["failed"]) == 0
    assert int(summary["lines"]) >= 250
    # every quantised operator is named exactly as the x86 build's first choice
    for line in r.stdout.splitlines():
        f = line.split()
        if f[0] == "ok" and "qsi" in f[2]:
            assert f[3] == "first", line


def test_symbol_without_a_context(emitted):
    """The exporter filters kernels by name with a null context (KernelGen.cpp:49-53)."""
    r = subprocess.run([os.path.join(KG, "kernelgen_tool"), "--null-symbols"],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    names = r.stdout.split()
    assert len(names) >= 11 and all(n.startswith(("kernel_", "GI_kernel_")) for n in names)


def test_library_resolves_every_emitted_symbol(emitted):
    _, manifest = emitted
    for sym in set(manifest.values()):
        if "fused_elementwise" in sym:
            # named by modes and operand kinds only (as in the reference): the shim carries the
            # program, the library cannot rebuild it from the name
            with pytest.raises(runtime.MegccError):
                runtime.parse_symbol(sym)
            continue
        runtime.parse_symbol(sym)


def test_fused_elemwise_shim_carries_the_program(emitted):
    out, manifest = emitted
    text = open(out / (manifest["fused_2xy_bcast101"] + ".c")).read()
    assert "MegccFusedElemwiseAttr attr = {4, 3, {" in text
    assert "{MEGCC_EW_ADD, 2, {0, 1, 0, 0}}" in text
    assert "{MEGCC_EW_MUL, 2, {2, 4, 0, 0}}" in text  # I2 * O0: value 4 is the result of step 0
    assert "{MEGCC_EW_SUB, 2, {4, 3, 0, 0}}" in text


def test_shim_attributes_round_trip(emitted):
    """the constant struct in the shim must equal what the library parses from the symbol"""
    out, manifest = emitted
    sym = manifest["conv44_3x3_s2_RELU"]
    text = open(out / (sym + ".c")).read()
    assert "MegccConvAttr attr = {3, 3, 2, 2, 1, 1, 1, 1, MEGCC_FMT_NCHW44, MEGCC_SPARSE_DENSE, MEGCC_NONLINE_RELU, 1}" in text
    a = runtime.parse_symbol(sym).attr.conv
    assert (a.kernel_h, a.stride_h, a.pad_h, a.format, a.nonline, a.with_bias) == (3, 2, 1, abi.FMT_NCHW44, abi.RELU, 1)
    sym = manifest["conv_hybrid_3x3_s2_RELU"]
    assert "MEGCC_FMT_NCHW_NCHW44" in open(out / (sym + ".c")).read()


@pytest.fixture(scope="module")
def shim_library(emitted):
    out, manifest = emitted
    so = out / "libshims.so"
    srcs = sorted(str(p) for p in out.glob("*.c"))
    subprocess.check_call(["gcc", "-shared", "-fPIC", "-Wall", "-Werror", "-o", str(so)] + srcs +
                          ["-I" + os.path.join(ROOT, "include"),
                           "-L" + os.path.dirname(runtime.LIB_PATH) if hasattr(runtime, "LIB_PATH") else "-L.",
                           "-L" + os.path.join(ROOT, "megcc_amd"), "-lmegcc_gfx950",
                           "-Wl,-rpath," + os.path.join(ROOT, "megcc_amd")])
    return C.CDLL(str(so)), manifest


def test_shims_compile_and_link(shim_library):
    lib, manifest = shim_library
    for sym in set(manifest.values()):
        assert hasattr(lib, sym)
        assert hasattr(lib, sym + "_init")
        assert hasattr(lib, sym + "_workspace")


def test_generated_workspace_functions_agree_with_the_library(shim_library):
    """the shims compute workspace sizes in plain C (the compiler may run them at compile time);
    they must ask for exactly what the kernels expect"""
    lib, manifest = shim_library
    L = runtime.lib()
    checked = 0
    for sym in sorted(set(manifest.values())):
        if "fused_elementwise" in sym:  # no workspace; not reachable by name (see above)
            continue
        desc = runtime.parse_symbol(sym)
        if desc.kind == 2:  # MatrixMul
            ta, tb = desc.attr.matmul.transpose_a, desc.attr.matmul.transpose_b
            shapes = [(1, 1024, 1000), (64, 4096, 4096), (4096, 4096, 4096), (5, 100, 7), (300, 64, 200)]
            cases_ = [[((k, m) if ta else (m, k)), ((n, k) if tb else (k, n))] for m, k, n in shapes]
        elif desc.kind == 1 and "f32" in sym and "_NCHW_DENSE_" in sym:
            k = desc.attr.conv.kernel_h
            cases_ = [[(1, 32, 56, 56), (32, 32, k, k)], [(2, 5, 19, 23), (37, 5, k, k)],
                      [(8, 64, 56, 56), (128, 64, k, k)]]
        elif desc.kind == 1 and "f32" in sym and "_NCHW44_DENSE_" in sym:
            # relayout -> NCHW implicit GEMM -> relayout: the GEMM's room plus three NCHW copies
            k = desc.attr.conv.kernel_h
            cases_ = [[(2, 2, 9, 7, 4), (3, 2, k, k, 4, 4)], [(8, 16, 56, 56, 4), (16, 16, k, k, 4, 4)],
                      [(1, 128, 7, 7, 4), (128, 128, k, k, 4, 4)]]
        elif desc.kind == 1 and "qsi8" in sym and "_NCHW44_DENSE_" in sym:
            k = desc.attr.conv.kernel_h
            cases_ = [[(64, 256, 7, 7, 4), (256, 256, k, k, 4, 4)], [(2, 8, 20, 24, 4), (12, 8, k, k, 4, 4)],
                      [(1, 128, 14, 14, 4), (32, 128, k, k, 4, 4)], [(8, 64, 56, 56, 4), (128, 64, k, k, 4, 4)]]
        elif desc.kind == 1 and "qsi8" in sym and "_NCHW_GROUP_" in sym:
            k = desc.attr.conv.kernel_h
            cases_ = [[(64, 32, 112, 112), (32, 1, 1, k, k)], [(2, 8, 9, 7), (8, 1, 1, k, k)],
                      [(2, 6, 9, 7), (6, 1, 1, k, k)]]
        elif desc.kind == 1 and "qsi8" in sym and "_3x3_NCHW_DENSE_" in sym:
            # plain NCHW with spatial extent: both NCHW44 copies live in the workspace
            cases_ = [[(2, 8, 20, 24), (12, 8, 3, 3)], [(16, 64, 56, 56), (64, 64, 3, 3)],
                      [(1, 256, 14, 14), (32, 256, 3, 3)], [(2, 5, 9, 9), (7, 5, 3, 3)]]
        elif desc.kind == 1 and "qsi8" in sym and "_1x1_NCHW_DENSE_p0x0_s1x1" in sym:
            cases_ = [[(64, 1024, 1, 1), (1000, 1024, 1, 1)], [(64, 4096, 1, 1), (4096, 4096, 1, 1)],
                      [(1, 1024, 1, 1), (1000, 1024, 1, 1)], [(4096, 4096, 1, 1), (4096, 4096, 1, 1)]]
        else:
            continue
        fn = getattr(lib, sym + "_workspace")
        fn.argtypes = abi.WORKSPACE_ARGS
        dt = abi.FLOAT if "f32" in sym else abi.QINT8
        for shapes_ in cases_:
            tin = [abi.make_tensor(None, s, dt, 1.0) for s in shapes_]
            a, b = C.c_size_t(7), C.c_size_t(9)
            assert fn(abi.tensor_array(tin), len(tin), 1, C.byref(a)) == 0
            assert L.megcc_gfx950_call_workspace(C.byref(desc), abi.tensor_array(tin), len(tin), 1,
                                                 C.byref(b)) == 0
            assert a.value == b.value, (sym, shapes_, a.value, b.value)
            checked += 1
    assert checked >= 20


@pytest.mark.gpu
def test_conv_through_the_generated_shim(shim_library):
    """call the kernel the way the TinyNN runtime would: by its generated symbol"""
    lib, manifest = shim_library
    case = cases.ConvCase(abi.FMT_NCHW44, abi.DENSE, 2, 32, 20, 24, 48, 3, 1, 1, abi.RELU,
                          scales=(0.02, 0.01, unsat(288)))
    sym = case.symbol()
    assert sym in manifest.values()
    arrays = case.gen(3)
    ins, outs = case.specs(arrays)
    bufs = [runtime.DeviceBuffer.from_array(s.array) for s in ins]
    out = runtime.DeviceBuffer(outs[0].nbytes)
    tin = [abi.make_tensor(b.ptr, s.shape, s.type_enum, s.scale, s.name) for b, s in zip(bufs, ins)]
    tout = [abi.make_tensor(out.ptr, outs[0].shape, outs[0].type_enum, outs[0].scale)]
    kern, init, ws = getattr(lib, sym), getattr(lib, sym + "_init"), getattr(lib, sym + "_workspace")
    kern.argtypes, init.argtypes, ws.argtypes = abi.KERNEL_ARGS, abi.INIT_ARGS, abi.WORKSPACE_ARGS
    size = C.c_size_t(1)
    assert ws(abi.tensor_array(tin), len(tin), 1, C.byref(size)) == 0 and size.value == 0
    n = C.c_int(0)
    assert init(abi.tensor_array(tin), len(tin), None, C.byref(n), None) == 0 and n.value == 1
    w = abi.Tensor()
    assert init(abi.tensor_array(tin), len(tin), C.byref(w), None, None) == 0
    assert w.name == tin[1].name
    wbuf = runtime.DeviceBuffer(w.layout.dims[0])
    w.ptr = wbuf.ptr
    assert init(abi.tensor_array(tin), len(tin), C.byref(w), C.byref(n), None) == 0
    tin[1] = w
    assert kern(abi.tensor_array(tin), len(tin), abi.tensor_array(tout), 1, None, None) == 0
    got = out.to_array(outs[0].shape, np.int8)
    np.testing.assert_array_equal(got, case.run_port(arrays))
