"""The committed golden vectors (tests/golden/tiny_unet_128.npz, written by
tests/golden/make_tiny_unet_golden.py from torch.nn.functional in fp32) against the
oracle on the CPU and against the HIP path on the GPU."""
import os

import numpy as np
import pytest

import denox_amd as dx
from util import assert_conv_close

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "tiny_unet_128.npz")


def build_from_fixture(g):
    m = dx.Model()
    x = m.input("input", "W", "H", 3)
    e0 = m.relu(m.conv2d(x, g["w0"], g["b0"]))
    e1 = m.relu(m.conv2d(m.pool(e0), g["w1"], g["b1"]))
    d0 = m.relu(m.conv2d(m.concat(m.upsample(e1), e0), g["w2"], g["b2"]))
    out = m.conv2d(d0, g["w3"], g["b3"])
    m.output(out, "output")
    return m, e0, out


def test_oracle_reproduces_golden_tiny_unet(oracle):
    g = np.load(GOLD)
    m, e0, out = build_from_fixture(g)
    env = oracle.run_graph(m.to_ops({"H": 128, "W": 128}), {"input": g["input"]}, "fp32")
    # fp32 against fp32: only the summation order differs
    np.testing.assert_allclose(env[out.name], g["output_fp32"], rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(env[e0.name][::8, ::8], g["e0_fp32"], rtol=1e-5, atol=1e-6)
    # storing fp16 between layers stays inside the parity bar as well
    f16 = oracle.run_graph(m.to_ops({"H": 128, "W": 128}), {"input": g["input"]}, "f16")[out.name]
    assert_conv_close(f16, g["output_fp32"], "oracle f16 mode vs golden")


@pytest.mark.gpu
@pytest.mark.parametrize("features", [{}, {"upsample_fusion": False, "concat_conv_fusion": False, "conv_relu_fusion": False}])
def test_hip_reproduces_golden_tiny_unet(features):
    g = np.load(GOLD)
    m, _, _ = build_from_fixture(g)
    mod = dx.Module.compile(m, features=features)
    got = mod.instance(H=128, W=128).infer(g["input"])[0]
    assert_conv_close(got, g["output_fp32"], f"HIP vs golden {features}")
