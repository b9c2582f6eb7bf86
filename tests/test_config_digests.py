"""The benchmark configurations at their own sizes against outputs of the reference's generated
kernels (tests/golden/config_digests.json, config_samples.npz; written by
tests/golden/make_config_digests.py): SHA-256 of every qsi8 output, a strided sample of every f32
output within 1e-4. Without a GPU the C restatement is held to them, on a GPU the HIP library."""
import json
import os

import numpy as np
import pytest

import cases
import config_cases as cc
import mobilenet
from megcc_amd import runtime
from oracle import port

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "config_digests.json")) as f:
    DIGESTS = json.load(f)
SAMPLES = np.load(os.path.join(HERE, "golden", "config_samples.npz"))
SINGLE = cc.single_cases()
F32_TOL = 1e-4


def check(name, out):
    want = DIGESTS[name]
    assert list(out.shape) == want["shape"] and str(out.dtype) == want["dtype"], name
    if out.dtype == np.float32:
        err = cases.max_rel_err(cc.sample(out), SAMPLES[name])
        assert err <= F32_TOL, "%s: max err %g against the reference kernel %s" % (name, err, want["kernel"])
    else:
        assert cc.digest(out) == want["sha256"], "%s differs from the reference kernel %s" % (name, want["kernel"])


def run_port(case, arrays):
    return case.run_port(arrays)


def run_gpu(case, arrays):
    print("GPU case:", repr(case), flush=True)
    ins, outs = case.specs(arrays)
    return runtime.run_symbol(case.symbol(), ins, outs)


def test_fixture_covers_every_case():
    names = set(SINGLE) | {"%s/%s" % (cc.chain_name(*t), s) for t in cc.CHAINS
                           for s in ("dw_baseline", "dw_unsat", "pool", "add_relu")}
    names |= {"cfg5_mobilenet_b1/" + n for _, n, _, _ in mobilenet.Net(1).steps}
    assert names == set(DIGESTS)
    assert {n for n, d in DIGESTS.items() if d["dtype"] == "float32"} == set(SAMPLES.files)


# ---- the C restatement at configuration sizes (no GPU) ------------------------------------------
@pytest.mark.parametrize("name", sorted(SINGLE))
def test_port_matches_the_reference_kernel(name):
    port.set_threads(8)
    case, seed = SINGLE[name]
    check(name, run_port(case, case.gen(seed=seed)))


@pytest.mark.parametrize("c,hw,stride", cc.CHAINS, ids=[cc.chain_name(*t) for t in cc.CHAINS])
def test_port_chain_matches_the_reference_kernels(c, hw, stride):
    port.set_threads(8)
    for stage, out in cc.chain_stages(c, hw, stride, run_port):
        check("%s/%s" % (cc.chain_name(c, hw, stride), stage), out)


def test_port_mobilenet_batch1_matches_the_reference_kernels():
    net = mobilenet.Net(1)
    _, trace = net.run_oracle(mobilenet.draw_input(1, seed=5), keep=True)
    for _, name, _, _ in net.steps:
        check("cfg5_mobilenet_b1/" + name, trace[name].reshape(DIGESTS["cfg5_mobilenet_b1/" + name]["shape"]))


# ---- the HIP library at configuration sizes ------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(SINGLE))
def test_gpu_matches_the_reference_kernel(name):
    case, seed = SINGLE[name]
    check(name, run_gpu(case, case.gen(seed=seed)))


@pytest.mark.gpu
@pytest.mark.parametrize("c,hw,stride", cc.CHAINS, ids=[cc.chain_name(*t) for t in cc.CHAINS])
def test_gpu_chain_matches_the_reference_kernels(c, hw, stride):
    for stage, out in cc.chain_stages(c, hw, stride, run_gpu):
        check("%s/%s" % (cc.chain_name(c, hw, stride), stage), out)


@pytest.mark.gpu
def test_gpu_mobilenet_batch1_matches_the_reference_kernels():
    net = mobilenet.Net(1)
    model, ids = net.build_gpu(keep_all=True)
    model.set_input(ids["image"], mobilenet.draw_input(1, seed=5))
    model.forward()
    for _, name, _, _ in net.steps:
        want = DIGESTS["cfg5_mobilenet_b1/" + name]
        check("cfg5_mobilenet_b1/" + name, model.get(ids[name]).reshape(want["shape"]))
    model.close()
