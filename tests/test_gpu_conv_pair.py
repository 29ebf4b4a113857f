"""conv -> conv in one dispatch (conv3x3_pair.hip): the tensor between two 3x3 convolutions stays in LDS.

Checked against the oracle's fp32 evaluation of the two layers (the conv tolerance), against the two-dispatch schedule
of the same model, and -- where fp16 holds every intermediate value exactly -- bit for bit against integer arithmetic,
at extents that exercise one and many strips, one and many row segments, segments that end inside a step, and the
benchmark's full frame."""
import numpy as np
import pytest

import denox_amd as dx
from util import assert_bits_equal, assert_conv_close, fill_lds_with_nans, he_weights, small_bias

pytestmark = pytest.mark.gpu

PAIR_CONFIGS = ["x8r2k16", "x4r4k16", "x4r2k16", "x4r2k32", "y4r2k32", "z4r2k64", "v4r2k64", "v4r2k16", "u4r2k32", "d4r2k64", "t4r2k32"]


def build(rng, C, K1, K2, tail, pad=False, act1=True, bias=True):
    m = dx.Model()
    t = m.input("input", "W", "H", C)
    x = m.pad_to_multiple(t, 16) if pad else t
    y = m.conv2d(x, he_weights(rng, K1, C), small_bias(rng, K1) if bias else None)
    if act1:
        y = m.relu(y)
    z = m.conv2d(y, he_weights(rng, K2, K1), small_bias(rng, K2) if bias else None)
    if tail in ("relu", "pool"):
        z = m.relu(z)
    if tail == "pool":
        z = m.pool(z)
    if tail == "crop":
        z = m.slice(z, 0, t.width, 0, t.height)
    m.output(z)
    return m, z


def entry_points(mod, **extents):
    return [d["entry_point"] for d in dx.describe(mod.dnx, **extents)["dispatches"]]


@pytest.mark.parametrize("config", PAIR_CONFIGS)
@pytest.mark.parametrize("C,K1,K2,tail,pad", [(9, 32, 32, "pool", True), (64, 32, 3, "crop", True), (16, 32, 32, "relu", False), (8, 16, 8, "none", False),
                                                (24, 24, 32, "pool", False), (3, 32, 16, "relu", False), (16, 32, 5, "relu", False), (32, 8, 1, "none", False),
                                                (16, 16, 4, "pool", False)])
def test_pair_against_oracle_and_two_dispatches(oracle, config, C, K1, K2, tail, pad):
    rng = np.random.default_rng(C * 1000 + K1 * 10 + K2)
    m, z = build(rng, C, K1, K2, tail, pad)
    try:
        mod = dx.Module.compile(m, conv_config=config)
    except dx.DenoxHipError as e:
        assert e.status == 5
        pytest.skip(str(e))
    two = dx.Module.compile(m, features={"conv_conv_fusion": False})
    for H, W in [(37, 70), (16, 30), (1, 1), (45, 333), (300, 61)]:
        if tail == "pool" and (H < 2 or W < 2):
            continue
        if not any(e.startswith("convpair_") and e.endswith(config) for e in entry_points(mod, H=H, W=W)):
            pytest.skip(f"{config} does not fit this layer")  # (LDS): the single-convolution schedule was selected
        x = rng.standard_normal((H, W, C)).astype(np.float16)
        fill_lds_with_nans()
        got = mod.instance(H=H, W=W).infer(x)[0]
        want = oracle.run_graph(m.to_ops({"H": H, "W": W}), {"input": x}, "fp32")[z.name]
        assert_conv_close(got, want, f"pair {config} {H}x{W}")
        ref = two.instance(H=H, W=W).infer(x)[0].astype(np.float32)
        assert np.abs(got.astype(np.float32) - ref).max() <= 2e-2 * max(1.0, float(np.abs(ref).max())), "fused against two dispatches"


def test_every_pair_configuration_runs_somewhere():
    """Each configuration of the table fits at least one of the layer shapes above (none is tested by skips alone)."""
    rng = np.random.default_rng(1)
    for config in PAIR_CONFIGS:
        hit = False
        for C, K1, K2, tail in [(9, 32, 32, "relu"), (16, 32, 32, "relu"), (64, 32, 3, "none")]:
            m, _ = build(rng, C, K1, K2, tail)
            hit |= any(e.endswith(config) for e in entry_points(dx.Module.compile(m, conv_config=config), H=64, W=64))
        assert hit, config


def test_pair_with_concat_and_upsample_sources(oracle):
    rng = np.random.default_rng(3)
    H, W = 52, 90
    m = dx.Model()
    a = m.input("low", "W2", "H2", 16)
    b = m.input("skip", "W", "H", 9)
    y = m.relu(m.conv2d(m.concat(m.upsample(a), b), he_weights(rng, 32, 25), small_bias(rng, 32)))
    z = m.relu(m.conv2d(y, he_weights(rng, 24, 32), small_bias(rng, 24)))
    m.output(z)
    mod = dx.Module.compile(m, conv_config="x8r2k16")
    ext = dict(H=H, W=W, H2=H // 2, W2=W // 2)
    assert any(e.startswith("convpair_c16up9") for e in entry_points(mod, **ext)), entry_points(mod, **ext)
    xa = rng.standard_normal((H // 2, W // 2, 16)).astype(np.float16)
    xb = rng.standard_normal((H, W, 9)).astype(np.float16)
    got = mod.instance(**ext).infer(xa, xb)[0]
    want = oracle.run_graph(m.to_ops(ext), {"low": xa, "skip": xb}, "fp32")[z.name]
    assert_conv_close(got, want, "pair with upsample + concat sources")


def integer_pair(x, K1, K2):
    """Both convolutions with all-ones weights, no bias, no activation, in integer arithmetic."""
    H, W, C = x.shape
    xi = np.pad(x.astype(np.int64).sum(axis=2), 1)
    mid = sum(xi[r:r + H, s:s + W] for r in range(3) for s in range(3))  # every channel of the K1 alike
    mp = np.pad(mid * K1, 1)
    out = sum(mp[r:r + H, s:s + W] for r in range(3) for s in range(3))
    return np.repeat(out[:, :, None], K2, axis=2)


@pytest.mark.parametrize("config,C,density", [("x8r2k16", 8, 0.15), ("y4r2k32", 32, 0.04), ("z4r2k64", 64, 0.02), ("v4r2k64", 64, 0.02), ("v4r2k16", 8, 0.15), ("u4r2k32", 32, 0.04),
                                              ("d4r2k64", 64, 0.02), ("t4r2k32", 32, 0.04)])
@pytest.mark.parametrize("H,W", [(33, 47), (288, 31), (1080, 1920), (24, 9000)])  # the last: more strips than workgroups
def test_pair_exact_on_small_integers(H, W, config, C, density):
    """Inputs in {0, 1}, all weights one: every intermediate and final value is an integer below 2048, which binary16
    holds exactly, so the fused kernel must reproduce integer arithmetic bit for bit -- at every strip and segment
    border of the benchmark's frame as well."""
    rng = np.random.default_rng(H)
    K1, K2 = 2, 3
    x = (rng.random((H, W, C)) < density).astype(np.float16)
    m = dx.Model()
    y = m.conv2d(m.input("input", "W", "H", C), np.ones((K1, C, 3, 3), np.float16))
    z = m.conv2d(y, np.ones((K2, K1, 3, 3), np.float16))
    m.output(z)
    mod = dx.Module.compile(m, conv_config=config, assume={"H": H, "W": W})
    assert any(e.startswith("convpair_") and e.endswith(config) for e in entry_points(mod, H=H, W=W))
    want = integer_pair(x, K1, K2)
    assert want.max() < 2048
    fill_lds_with_nans()
    assert_bits_equal(mod.instance(H=H, W=W).infer(x)[0], want.astype(np.float16), f"integer pair {H}x{W}")


def test_pair_pool_and_crop_exact_at_full_size():
    """The two layer pairs of the benchmark network's full-resolution ends, with integer data: replicate pad in front,
    2x2 max pool behind (1088 x 1920 -> 544 x 960), and the crop back to 1080 rows."""
    rng = np.random.default_rng(9)
    H, W, C, K1 = 1080, 1920, 9, 2
    x = (rng.random((H, W, C)) < 0.12).astype(np.float16)
    xp = np.pad(x, ((0, 8), (0, 0), (0, 0)), mode="edge")
    for tail, K2 in (("pool", 32), ("crop", 3)):
        m = dx.Model()
        t = m.input("input", "W", "H", C)
        y = m.conv2d(m.pad_to_multiple(t, 16), np.ones((K1, C, 3, 3), np.float16))
        z = m.conv2d(y, np.ones((K2, K1, 3, 3), np.float16))
        z = m.pool(z) if tail == "pool" else m.slice(z, 0, t.width, 0, t.height)
        m.output(z)
        mod = dx.Module.compile(m, conv_config="x8r2k16", assume={"H": H, "W": W})
        assert any(e.startswith("convpair_c9e") for e in entry_points(mod, H=H, W=W))
        want = integer_pair(xp, K1, K2)
        assert want.max() < 2048
        want = want.reshape(544, 2, 960, 2, K2).max(axis=(1, 3)) if tail == "pool" else want[:H, :W]
        assert_bits_equal(mod.instance(H=H, W=W).infer(x)[0], want.astype(np.float16), f"integer pair + {tail} at full size")
