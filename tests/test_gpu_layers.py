"""GPU parity of single layers and small fused patterns against the CPU oracle.

Every case goes builder -> compile -> runtime -> infer through the C ABI
(libdenox_hip.so); the oracle evaluates the same layer records in fp32.
Conv layers: max-abs <= 2e-2, mean-abs <= 2e-3 on the fp16 output against the
fp32 evaluation.  Pool / upsample / concat / pad / slice / relu: bit-exact.
Shapes follow the reference's system tests (test/system/test_conv.py:126-501:
channel counts 3, 9, 24, 67, 80, 112, 160 ...; 100 x 100 random inputs)."""
import numpy as np
import pytest

import denox_amd as dx
from denox_amd import networks
from util import assert_bits_equal, assert_conv_close, he_weights, small_bias

pytestmark = pytest.mark.gpu


def run(model, x, **kw):
    mod = dx.Module.compile(model, **kw)
    H, W = x.shape[:2]
    return mod, mod.instance(H=H, W=W).infer(x)[0]


CONV_CASES = [
    # C, K, H, W
    (3, 16, 100, 100), (9, 32, 100, 100), (16, 16, 64, 64), (32, 32, 37, 53), (64, 64, 100, 100),
    (24, 48, 33, 70), (67, 80, 40, 40), (80, 112, 31, 33), (112, 96, 16, 40), (160, 112, 24, 32),
    (32, 3, 100, 100), (73, 64, 64, 96), (48, 16, 8, 8), (8, 8, 1, 1), (16, 32, 5, 200),
]


@pytest.mark.parametrize("C,K,H,W", CONV_CASES)
@pytest.mark.parametrize("act", ["none", "relu"])
def test_conv3x3(oracle, C, K, H, W, act):
    rng = np.random.default_rng(C * 1000 + K)
    x = rng.random((H, W, C)).astype(np.float16)
    w, b = he_weights(rng, K, C), small_bias(rng, K)
    m = dx.Model()
    t = m.conv2d(m.input("input", "W", "H", C), w, b)
    if act == "relu":
        t = m.relu(t)
    m.output(t)
    _, got = run(m, x)
    want = oracle.run_graph(m.to_ops({"H": H, "W": W}), {"input": x}, "fp32")[t.name]
    assert_conv_close(got, want, f"conv {C}->{K} {H}x{W} {act}")


ALL_CONFIGS = ["w4r2k16", "w4r2k32", "w4r4k16", "w4r4k32", "w8r2k16", "w8r2k32", "w4r2k64", "w8r1k16", "w4r1k16", "w4r1k32",
               "w4r1k32n", "w4r2k32n", "w2r2k32n", "w2r2k32", "p8r1k16", "p8r1k32", "p16r1k16", "p16r1k32", "p8r2k16", "p8r2k32",
               "p16r2k16", "p4r2k32", "p8r4k16", "p4r4k16", "p4r4k32", "p4r1k32", "p4r2k32n", "p4r1k32n", "s8r2k16", "s12r1k16",
               "w4r1kfn", "w4r1khn", "w4r2kfn", "w2r2kfn", "w4r1kfm", "w4r2khn"]
# the 16x16x32 matrix shape: output channels in blocks of 16, tiles 16 or 32 pixels wide
M16_CONFIGS = ["m4r2k32x2", "m4r2k64x2", "m4r1k32x2", "m4r2k32x1", "m4r4k32x1", "m8r2k32x2", "m4r2kfx1", "m4r1kfx2", "m4r2k32x2n",
               "m4r2kfx1n", "m4r1kfx1n", "m4r2k32x1n", "q8r2k32x2", "q8r1k32x2", "q4r2k32x2", "q8r2k32x1", "q4r2k32x1n"]
ALL_CONFIGS += M16_CONFIGS
# two-phase schedule of the persistent kernel
ALL_CONFIGS += ["t16r1k16", "t16r1k32", "t16r2k16", "t8r2k16", "t8r2k32", "t8r4k16", "t8r1k16", "u8r2k32x2", "u16r1k32x2"]
# staging waves that also store the result (through LDS, whole pixels per store instruction)
OSTAGE_CONFIGS = ["r4r2k16", "r4r2k16n", "r8r1k16n", "r4r2k32n", "r4r1k16n"]
# ... with the matrix loop's fragment reads pipelined (`m`), and the staged halo unpadded with rotated slots (`c`: 32-channel steps)
OSTAGE_CONFIGS += ["c4r2k32n", "c4r2k16n", "c4r2k16m"]
ALL_CONFIGS += OSTAGE_CONFIGS
# the pipelined matrix loop / the rotated halo layout in the streaming, the staging-wave and the plain persistent kernel
PIPELINED_CONFIGS = ["w4r2k16s", "w4r2k32s", "s8r2k16s", "s8r2k32s", "p8r2k32s"]
ALL_CONFIGS += PIPELINED_CONFIGS


# (tests/test_host.py checks on the CPU that every configuration of the library's table is in one of the lists of this file and
# compiles for at least one of the layer shapes it is tested on here: a configuration must not be covered by skips alone)
EVERY_CONFIG_SHAPES = [(80, 64, 45, 70), (73, 96, 130, 300), (16, 32, 300, 530)]
FOLD_CONFIGS = ["f8r1", "f4r2", "f4r1", "g4r1", "g4r1k32", "g4r1n", "g4r1k32n", "h4r2", "h4r2n", "h4r2k32n", "h4r2p", "g4r1p", "h4r2k32p"]
FOLD_SHAPES = [(64, 9, 64, 36, 70, False), (16, 0, 32, 18, 34, False), (32, 24, 40, 62, 130, False), (8, 3, 3, 2, 2, False), (24, 9, 16, 40, 52, True),
               (96, 32, 64, 34, 66, False), (32, 16, 32, 50, 70, True), (48, 12, 96, 22, 134, False), (64, 8, 64, 2, 2, False), (16, 9, 32, 8, 64, False), (128, 9, 128, 20, 70, True)]
STRIDED_ONLY_CONFIGS = ["m2r1k32x1n", "w2r2k16n", "w2r1k16n"]  # offered to strided layers only


@pytest.mark.parametrize("config", ALL_CONFIGS)
@pytest.mark.parametrize("C,K,H,W", EVERY_CONFIG_SHAPES)
def test_conv_every_configuration(oracle, config, C, K, H, W):
    rng = np.random.default_rng(7)
    x = rng.standard_normal((H, W, C)).astype(np.float16)
    w, b = he_weights(rng, K, C), small_bias(rng, K)
    m = dx.Model()
    t = m.relu(m.conv2d(m.input("input", "W", "H", C), w, b))
    m.output(t)
    try:
        _, got = run(m, x, conv_config=config)
    except dx.DenoxHipError as e:
        assert e.status == 5  # this configuration does not exist for this layer shape
        pytest.skip(str(e))
    assert config in dx.last_compile_report()
    want = oracle.run_graph(m.to_ops({"H": H, "W": W}), {"input": x}, "fp32")[t.name]
    assert_conv_close(got, want, config)


@pytest.mark.parametrize("config", M16_CONFIGS)
@pytest.mark.parametrize("CA,CB,K,H,W", [(48, 0, 48, 34, 50), (64, 48, 80, 36, 40), (96, 9, 112, 20, 70), (32, 0, 3, 33, 47), (9, 0, 16, 40, 36)])
def test_conv_16x16_shape_odd_channel_counts(oracle, config, CA, CB, K, H, W):
    """Output-channel counts that are multiples of 16 but not of 32 (paired and unpaired 16-blocks), K = 3,
    with the upsample + concat prologue and the pool epilogue."""
    rng = np.random.default_rng(CA + K)
    w, b = he_weights(rng, K, CA + CB), small_bias(rng, K)
    m = dx.Model()
    if CB:
        lo = rng.standard_normal((H // 2, W // 2, CA)).astype(np.float16)
        x = rng.standard_normal((H, W, CB)).astype(np.float16)
        t = m.pool(m.relu(m.conv2d(m.concat(m.upsample(m.input("lo", m.sym("W") // 2, m.sym("H") // 2, CA)), m.input("x", "W", "H", CB)), w, b)))
        feeds, args = {"lo": lo, "x": x}, (lo, x)
    else:
        x = rng.standard_normal((H, W, CA)).astype(np.float16)
        t = m.relu(m.conv2d(m.input("x", "W", "H", CA), w, b))
        feeds, args = {"x": x}, (x,)
    m.output(t)
    try:
        mod = dx.Module.compile(m, conv_config=config)
    except dx.DenoxHipError as e:
        assert e.status == 5
        pytest.skip(str(e))
    assert config in dx.last_compile_report()
    got = mod.instance(H=H, W=W).infer(*args)[0]
    want = oracle.run_graph(m.to_ops({"H": H, "W": W}), feeds, "fp32")[t.name]
    assert_conv_close(got, want, config)


@pytest.mark.parametrize("config", [None, "w4r2k16", "p8r1k16", "m4r2k32x2", "t8r2k16", "s8r2k16"])
@pytest.mark.parametrize("R,S", [(1, 1), (5, 5), (1, 3), (3, 1), (7, 7), (5, 3)])
def test_odd_filter_extents(oracle, R, S, config):
    """R x S filters with "same" zero padding (the reference's direct_conv.comp takes any extent), bare and with the
    upsample + concat prologue and the pool epilogue."""
    rng = np.random.default_rng(R * 10 + S)
    H, W, CA, CB, K = 26, 44, 24, 9, 40
    pad = ((R - 1) // 2, (S - 1) // 2)
    lo = rng.standard_normal((H // 2, W // 2, CA)).astype(np.float16)
    x = rng.standard_normal((H, W, CB)).astype(np.float16)
    w1 = (rng.standard_normal((K, CA + CB, R, S)) * np.sqrt(2.0 / (R * S * (CA + CB)))).astype(np.float16)
    w2 = (rng.standard_normal((16, CB, R, S)) * np.sqrt(2.0 / (R * S * CB))).astype(np.float16)
    m = dx.Model()
    a = m.input("lo", m.sym("W") // 2, m.sym("H") // 2, CA)
    b = m.input("x", "W", "H", CB)
    o1 = m.pool(m.relu(m.conv2d(m.concat(m.upsample(a), b), w1, small_bias(rng, K), padding=pad)))
    o2 = m.conv2d(b, w2, None, padding=pad)
    m.output(o1, "o1")
    m.output(o2, "o2")
    try:
        mod = dx.Module.compile(m, conv_config=config)
    except dx.DenoxHipError as e:
        assert e.status == 5
        pytest.skip(str(e))
    assert f"conv{R}x{S}" in dx.last_compile_report() and mod.runtime_model.dispatch_count == 2
    got1, got2 = mod.instance(H=H, W=W).infer(lo, x)
    env = oracle.run_graph(m.to_ops({"H": H, "W": W}), {"lo": lo, "x": x}, "fp32")
    assert_conv_close(got1, env[o1.name], f"{R}x{S} fused {config}")
    assert_conv_close(got2, env[o2.name], f"{R}x{S} bare {config}")


@pytest.mark.parametrize("config", FOLD_CONFIGS)
@pytest.mark.parametrize("CA,CB,K,H,W,padb", FOLD_SHAPES)
def test_upsample_folded_into_weights(oracle, config, CA, CB, K, H, W, padb):
    """conv(concat(upsample(A), B)) with the upsample folded into 2x2-tap weights per output parity: the same tensor
    as the layer-by-layer evaluation, within the conv tolerance (the summed weights are rounded to binary16 once)."""
    rng = np.random.default_rng(CA + CB + K)
    w, b = he_weights(rng, K, CA + CB), small_bias(rng, K)
    m = dx.Model()
    lo = rng.standard_normal((H // 2, W // 2, CA)).astype(np.float16)
    feeds = {"lo": lo}
    t = m.upsample(m.input("lo", m.sym("W") // 2, m.sym("H") // 2, CA))
    if CB:
        if padb:  # the skip source is stored 3 rows / 5 columns short and replicate-padded
            x = rng.standard_normal((H - 3, W - 5, CB)).astype(np.float16)
            t = m.concat(t, m.pad(m.input("x", m.sym("W") - 5, m.sym("H") - 3, CB), 2, 3, 1, 2))
        else:
            x = rng.standard_normal((H, W, CB)).astype(np.float16)
            t = m.concat(t, m.input("x", "W", "H", CB))
        feeds["x"] = x
    t = m.activation(m.conv2d(t, w, b), "leaky_relu", 0.25)
    m.output(t)
    try:
        mod = dx.Module.compile(m, conv_config=config)
    except dx.DenoxHipError as e:
        assert e.status == 5
        pytest.skip(str(e))
    assert config in dx.last_compile_report() and mod.runtime_model.dispatch_count == 1
    got = mod.instance(H=H, W=W).infer(*[feeds[k] for k in ("lo", "x") if k in feeds])[0]
    want = oracle.run_graph(m.to_ops({"H": H, "W": W}), feeds, "fp32")[t.name]
    assert_conv_close(got, want, f"fold {config}")


def test_full_size_fold_equals_the_unfolded_kernel_bit_for_bit():
    """The dominant layer of the 1080p U-Net (upsampled 64 channels + 9 replicate-padded input channels -> 64) at its real
    extent, with small integers for inputs and weights: every product and sum is exact in binary16 / fp32, so the
    upsample-folded kernels (weights summed per output parity) must give the unfolded kernel's bits."""
    rng = np.random.default_rng(11)
    H, W, CA, CB, K = 1088, 1920, 64, 9, 64
    w = rng.integers(-1, 2, (K, CA + CB, 3, 3)).astype(np.float16)
    b = rng.integers(-3, 4, K).astype(np.float16)
    m = dx.Model()
    lo = m.input("lo", m.sym("W") // 2, m.sym("H") // 2, CA)
    x = m.input("x", "W", m.sym("H") - 8, CB)
    t = m.relu(m.conv2d(m.concat(m.upsample(lo), m.pad(x, 0, 0, 4, 4)), w, b))
    m.output(t)
    xa = rng.integers(0, 3, (H // 2, W // 2, CA)).astype(np.float16)
    xb = rng.integers(0, 3, (H - 8, W, CB)).astype(np.float16)
    outs = {}
    for config in ("s8r2k16", "g4r1", "g4r1k32", "g4r1n", "h4r2n", "h4r2k32n", "h4r2p", "g4r1p", "h4r2k32p", "f8r1", "r4r2k16n", "c4r2k32n", "w4r2k32s"):
        mod = dx.Module.compile(m, conv_config=config, assume={"H": H, "W": W})
        assert config in dx.last_compile_report() and mod.runtime_model.dispatch_count == 1
        outs[config] = mod.instance(H=H, W=W).infer(xa, xb)[0]
    assert outs["s8r2k16"].max() > 100 and np.array_equal(outs["s8r2k16"], np.round(outs["s8r2k16"]))
    for config in ("g4r1", "g4r1k32", "g4r1n", "h4r2n", "h4r2k32n", "h4r2p", "g4r1p", "h4r2k32p", "f8r1", "r4r2k16n", "c4r2k32n", "w4r2k32s"):
        assert_bits_equal(outs[config], outs["s8r2k16"], config)
    # and the unfolded kernel against the definition, on the four corners and a centre patch (float64 on the host)
    up = np.repeat(np.repeat(xa.astype(np.float64), 2, 0), 2, 1)
    xp = np.pad(xb.astype(np.float64), ((4, 4), (0, 0), (0, 0)), mode="edge")
    src = np.pad(np.concatenate([up, xp], 2), ((1, 1), (1, 1), (0, 0)))
    wf = w.astype(np.float64)
    for y0, x0 in [(0, 0), (0, W - 24), (H - 24, 0), (H - 24, W - 24), (500, 900)]:
        acc = np.zeros((24, 24, K))
        for r in range(3):
            for q in range(3):
                acc += src[y0 + r:y0 + r + 24, x0 + q:x0 + q + 24] @ wf[:, :, r, q].T
        want = np.maximum(acc + b.astype(np.float64), 0)
        assert np.array_equal(outs["s8r2k16"][y0:y0 + 24, x0:x0 + 24].astype(np.float64), want), (y0, x0)


def test_tensor_size_limit_is_reported():
    """Tensors are addressed with 32-bit byte offsets: extents that make one reach 4 GiB are refused when the
    instance is created, before anything is allocated."""
    m = dx.Model()
    m.output(m.relu(m.conv2d(m.input("x", "W", "H", 64), np.zeros((64, 64, 3, 3), np.float16))))
    mod = dx.Module.compile(m)
    with pytest.raises(dx.DenoxHipError) as e:
        mod.instance(H=6000, W=6000)
    assert e.value.status == 5 and "4 GiB" in str(e.value)


def test_conv_closed_forms():
    # centre-tap identity: out == in, bit for bit; all-ones: C * (#taps inside the image)
    C = 16
    rng = np.random.default_rng(1)
    x = rng.standard_normal((20, 40, C)).astype(np.float16)
    w = np.zeros((C, C, 3, 3), np.float16)
    w[np.arange(C), np.arange(C), 1, 1] = 1
    m = dx.Model()
    t = m.conv2d(m.input("input", "W", "H", C), w)
    m.output(t)
    _, got = run(m, x)
    assert_bits_equal(got, x, "identity conv")
    ones = np.ones((9, 35, C), np.float16)
    m = dx.Model()
    t = m.conv2d(m.input("input", "W", "H", C), np.ones((8, C, 3, 3), np.float16))
    m.output(t)
    _, got = run(m, ones)
    assert np.all(got[1:-1, 1:-1] == 9 * C) and np.all(got[0, 1:-1] == 6 * C) and np.all(got[1:-1, -1] == 6 * C)
    assert got[0, 0, 0] == 4 * C and got[-1, -1, 7] == 4 * C


@pytest.mark.parametrize("C,H,W", [(32, 64, 64), (48, 33, 71), (9, 20, 20), (3, 7, 9), (80, 16, 16)])
def test_bandwidth_layers_bit_exact(oracle, C, H, W):
    rng = np.random.default_rng(C + H)
    x = rng.standard_normal((H, W, C)).astype(np.float16)
    for build in ("pool", "upsample", "relu", "leaky", "pad", "slice", "concat"):
        m = dx.Model()
        i = m.input("input", "W", "H", C)
        if build == "pool":
            t = m.pool(i)
        elif build == "upsample":
            t = m.upsample(i)
        elif build == "relu":
            t = m.relu(i)
        elif build == "leaky":
            t = m.activation(i, "leaky_relu", 0.1)
        elif build == "pad":
            t = m.pad_to_multiple(i, 16)
        elif build == "slice":
            t = m.slice(i, 1, i.width - 2, 2, i.height - 1)
        else:
            t = m.concat(m.upsample(m.pool(m.pad_to_multiple(i, 2))), m.pad_to_multiple(i, 2))
        m.output(t)
        _, got = run(m, x)
        want = oracle.run_graph(m.to_ops({"H": H, "W": W}), {"input": x}, "f16")[t.name]
        assert_bits_equal(got, want, f"{build} C={C} {H}x{W}")


FUSION_FLAGS = [
    {},  # everything fused
    {"pool_fusion": False}, {"upsample_fusion": False}, {"concat_conv_fusion": False, "upsample_fusion": False},
    {"conv_relu_fusion": False, "pool_fusion": False, "upsample_fusion": False, "concat_conv_fusion": False},
]


@pytest.mark.parametrize("config", ["w4r2k16", "p8r1k16", "p16r1k16", "w8r2k16", "s8r2k16", "s12r1k16", "t16r1k16", "t8r2k16"])
@pytest.mark.parametrize("features", [{}, {"pad_fusion": False}, {"slice_fusion": False}, {"pad_fusion": False, "slice_fusion": False}])
def test_pad_and_slice_fold_into_the_conv(oracle, features, config):
    """pad -> (upsample, pad) concat -> conv -> relu -> slice, with offsets on every side."""
    rng = np.random.default_rng(3)
    H, W, CA, CB, K = 37, 51, 16, 9, 16
    x = rng.standard_normal((H, W, CB)).astype(np.float16)
    lo = rng.standard_normal((24, 32, CA)).astype(np.float16)  # (H + 3 + 8) / 2, (W + 2 + 11) / 2
    w, b = he_weights(rng, K, CA + CB), small_bias(rng, K)
    w2, b2 = he_weights(rng, 8, CB), small_bias(rng, 8)
    m = dx.Model()
    xi = m.input("x", "W", "H", CB)
    li = m.input("lo", (m.sym("W") + 13) // 2, (m.sym("H") + 11) // 2, CA)
    p = m.pad(xi, 2, 11, 3, 8)
    y = m.relu(m.conv2d(m.concat(m.upsample(li), p), w, b))
    out1 = m.slice(y, 2, 2 + xi.width, 3, 3 + xi.height)
    out2 = m.conv2d(p, w2, b2)  # a second consumer of the padded tensor, padded source as A
    m.output(out1, "out1")
    m.output(out2, "out2")
    mod = dx.Module.compile(m, features=features, conv_config=config)
    got1, got2 = mod.instance(H=H, W=W).infer(x, lo)
    env = oracle.run_graph(m.to_ops({"H": H, "W": W}), {"x": x, "lo": lo}, "fp32")
    assert got1.shape == (H, W, K) and got2.shape == (H + 11, W + 13, 8)
    assert_conv_close(got1, env[out1.name], f"crop {features}")
    assert_conv_close(got2, env[out2.name], f"padA {features}")
    if not features:
        assert mod.runtime_model.dispatch_count == 2


@pytest.mark.parametrize("features", FUSION_FLAGS)
@pytest.mark.parametrize("CA,CB,K,H,W", [(32, 16, 32, 32, 64), (64, 9, 64, 22, 38), (16, 3, 16, 16, 32)])
def test_fused_patterns_agree(oracle, features, CA, CB, K, H, W):
    """upsample -> concat -> conv -> relu -> pool: fused and unfused schedules give the
    same tensor as the oracle's layer-by-layer evaluation."""
    rng = np.random.default_rng(CA + CB)
    lo = rng.random((H // 2, W // 2, CA)).astype(np.float16)
    skip = rng.random((H, W, CB)).astype(np.float16)
    w, b = he_weights(rng, K, CA + CB), small_bias(rng, K)
    m = dx.Model()
    a = m.input("lo", m.sym("W") // 2, m.sym("H") // 2, CA)
    s = m.input("skip", "W", "H", CB)
    t = m.pool(m.relu(m.conv2d(m.concat(m.upsample(a), s), w, b)))
    m.output(t)
    mod = dx.Module.compile(m, features=features)
    got = mod.instance(H=H, W=W).infer(lo, skip)[0]
    env = oracle.run_graph(m.to_ops({"H": H, "W": W}), {"lo": lo, "skip": skip}, "fp32")
    assert_conv_close(got, env[t.name], str(features))
    n = mod.runtime_model.dispatch_count
    assert n == (1 if not features else n)  # the default schedule is a single dispatch


@pytest.mark.parametrize("config", ["s8r2k16", "w4r2k16", "m8r2k32x2", "q8r2k32x2", "t8r2k16", "x8r2k16"])
@pytest.mark.parametrize("act", ["relu", "none"])
def test_pooled_epilogue_equals_conv_then_pool(config, act):
    """The fused epilogue takes the maximum of the four fp32 sums and finishes it once (bias, ReLU and rounding are
    monotonic); the unfused schedule rounds all four and lets the stand-alone pool compare the halves.  Same values,
    element for element (a zero's sign aside), on random data with negative and repeated values."""
    rng = np.random.default_rng(11)
    C, K, H, W = 32, 32, 44, 70
    pair = config.startswith("x")
    x = np.round(rng.standard_normal((H, W, C)) * 4).astype(np.float16) / 4  # a coarse grid: ties inside the windows
    m = dx.Model()
    t = m.input("input", "W", "H", C)
    if pair:
        t = m.relu(m.conv2d(t, he_weights(rng, 32, C), small_bias(rng, 32)))
    y = m.conv2d(t, he_weights(rng, K, 32 if pair else C), small_bias(rng, K))
    y = m.relu(y) if act == "relu" else y
    m.output(m.pool(y))
    fused = dx.Module.compile(m, conv_config=config)
    assert fused.runtime_model.dispatch_count == 1 and config in dx.last_compile_report()
    split = dx.Module.compile(m, conv_config=None if pair else config, features={"pool_fusion": False, "conv_conv_fusion": False})
    assert split.runtime_model.dispatch_count == (3 if pair else 2)
    got = fused.instance(H=H, W=W).infer(x)[0]
    want = split.instance(H=H, W=W).infer(x)[0]
    if pair:  # the fused pair sums the second convolution in another order than the stand-alone kernel: the conv tolerance
        assert np.abs(got.astype(np.float32) - want.astype(np.float32)).max() <= 2e-2 * max(1.0, float(np.abs(want).max()))
    else:
        assert np.array_equal(got, want), f"{int((got != want).sum())} elements differ"


IN_PLACE_CASES = [  # (C, K0, K1, tail): channel range aligned / not aligned to 16 bytes, narrow and wide, a pooled and an activated producer
    (8, 16, 24, "none"), (8, 16, 24, "conv"), (3, 3, 4, "none"), (9, 9, 16, "conv"), (16, 8, 3, "none"), (16, 64, 32, "conv"),
    (8, 16, 16, "pool"), (12, 40, 24, "relu"), (32, 48, 80, "conv")]


@pytest.mark.parametrize("config", [None, "s8r2k16", "m4r2k32x2", "t16r1k16", "q8r2k32x2", "r4r2k16n", "c4r2k32n"])
@pytest.mark.parametrize("C,K0,K1,tail", IN_PLACE_CASES + [(48, 40, 24, "relu"), (64, 64, 32, "none")])
def test_concat_sources_written_in_place(oracle, config, C, K0, K1, tail):
    """concat(conv(x), conv(x)): each conv stores into its channel range of the concat's tensor (pixel pitch K0 + K1),
    no copy runs, and the bits equal those of the schedule that copies."""
    rng = np.random.default_rng(C + K0 + 3 * K1)
    H, W = 37, 70
    x = rng.standard_normal((H, W, C)).astype(np.float16)
    m = dx.Model()
    t = m.input("input", "W", "H", C)

    def branch(K):
        y = m.conv2d(t, he_weights(rng, K, C), small_bias(rng, K))
        if tail == "relu":
            y = m.relu(y)
        if tail == "pool":
            y = m.pool(m.relu(y))
        return y
    c = m.concat(branch(K0), branch(K1))
    out = m.conv2d(c, he_weights(rng, 8, K0 + K1), small_bias(rng, 8)) if tail == "conv" else c
    m.output(out)
    # the consumer conv would otherwise read both sources itself (concat fused into the conv): keep the concat a tensor
    feats = {"concat_conv_fusion": False}
    try:
        mod = dx.Module.compile(m, conv_config=config, features=feats)
        ref = dx.Module.compile(m, conv_config=config, features={**feats, "implicit_concat": False})
    except dx.DenoxHipError as e:
        assert e.status == 5 and config is not None
        pytest.skip(str(e))
    n = 2 + (tail == "conv")
    assert mod.runtime_model.dispatch_count == n and ref.runtime_model.dispatch_count == n + 1
    got = mod.instance(H=H, W=W).infer(x)[0]
    assert_bits_equal(got, ref.instance(H=H, W=W).infer(x)[0], "in place against copied")
    want = oracle.run_graph(m.to_ops({"H": H, "W": W}), {"input": x}, "fp32")[out.name]
    assert_conv_close(got, want, f"in-place concat {config}")


def test_concat_output_written_in_place_follows_external_pointers(oracle):
    """A model output that is a concat whose sources are written in place by their producers: no dispatch binds the
    output tensor itself, only channel ranges inside its buffer.  Caller-supplied output addresses (infer_device) and
    the second set of interface tensors of a frame sequence (infer_many) must reach those dispatches as well."""
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(5)
    H, W, C, K0, K1 = 37, 70, 16, 16, 24
    m = dx.Model()
    t = m.input("input", "W", "H", C)
    c = m.concat(m.relu(m.conv2d(t, he_weights(rng, K0, C), small_bias(rng, K0))), m.relu(m.conv2d(t, he_weights(rng, K1, C), small_bias(rng, K1))))
    m.output(c)
    mod = dx.Module.compile(m)
    assert mod.runtime_model.dispatch_count == 2  # both convs store straight into the output
    xs = [rng.standard_normal((H, W, C)).astype(np.float16) for _ in range(4)]
    inst = mod.instance(H=H, W=W)
    wants = [inst.infer(x)[0] for x in xs]
    for x, want in zip(xs, wants):
        assert_conv_close(want, oracle.run_graph(m.to_ops({"H": H, "W": W}), {"input": x}, "fp32")[c.name], "concat output")
    outs = [torch.full((H, W, K0 + K1), float("nan"), dtype=torch.float16, device="cuda") for _ in range(2)]
    d_in = [torch.from_numpy(x).cuda() for x in xs]
    torch.cuda.synchronize()
    for i in range(4):  # alternating output buffers, as a double-buffering caller would
        inst.infer_device([d_in[i].data_ptr()], [outs[i & 1].data_ptr()])
        inst.synchronize()
        assert_bits_equal(outs[i & 1].cpu().numpy(), wants[i], f"external output, frame {i}")
    many = inst.infer_many([[x] for x in xs])
    for i, want in enumerate(wants):
        assert_bits_equal(many[i][0], want, f"frame sequence, frame {i}")
    assert_bits_equal(inst.infer(xs[0])[0], wants[0], "own buffers afterwards")


def test_graphs_of_recent_interface_addresses_are_kept():
    """More distinct interface address sets than the instance keeps captured graphs for: every one still gives the same bits."""
    torch = pytest.importorskip("torch")
    H, W = 24, 40
    m, _ = networks.build("tiny_unet", seed=8)
    x = networks.synthetic_input("tiny_unet", H, W, seed=8)
    inst = dx.Module.compile(m).instance(H=H, W=W)
    want = inst.infer(x)[0]
    d_in = torch.from_numpy(x).cuda()
    outs = [torch.zeros((H, W, 3), dtype=torch.float16, device="cuda") for _ in range(7)]
    torch.cuda.synchronize()
    for rnd in range(2):
        for o in outs:
            inst.infer_device([d_in.data_ptr()], [o.data_ptr()])  # not synchronised: the eviction has to wait by itself
        inst.synchronize()
        for i, o in enumerate(outs):
            assert_bits_equal(o.cpu().numpy(), want, f"round {rnd}, buffer {i}")
            o.zero_()
        torch.cuda.synchronize()


def test_concat_with_one_source_in_place(oracle):
    """concat(conv(x), x): the model input cannot live inside another tensor, the conv output can -- one copy instead of two."""
    rng = np.random.default_rng(11)
    H, W = 20, 33
    x = rng.standard_normal((H, W, 8)).astype(np.float16)
    m = dx.Model()
    t = m.input("input", "W", "H", 8)
    c = m.concat(t, m.relu(m.conv2d(t, he_weights(rng, 24, 8), small_bias(rng, 24))))
    m.output(c)
    mod = dx.Module.compile(m)
    rep = dx.last_compile_report()
    assert mod.runtime_model.dispatch_count == 2 and "copy/in-place" in rep
    got = mod.instance(H=H, W=W).infer(x)[0]
    assert_bits_equal(got[:, :, :8], x, "copied source")
    want = oracle.run_graph(m.to_ops({"H": H, "W": W}), {"input": x}, "fp32")[c.name]
    assert_conv_close(got, want, "half in-place concat")


def test_timing_table_runs_in_place_candidates(tmp_path):
    """The candidates that store with a foreign pixel pitch are benchmarked like any other: their scratch buffers span
    the wider tensor, and a schedule compiled against the table still gives the same bits."""
    rng = np.random.default_rng(2)
    m = dx.Model()
    t = m.input("input", "W", "H", 8)
    c = m.concat(m.conv2d(t, he_weights(rng, 16, 8)), m.conv2d(t, he_weights(rng, 9, 8)))
    m.output(c)
    db = dx.Db(str(tmp_path / "t.db"))
    assert db.populate(m, assume={"H": 48, "W": 64}, conv_config="w4r2k16") >= 6
    r = db.bench(min_samples=2, max_relative_error=1.0)
    assert r["failed"] == 0 and r["benchmarked"] >= 6
    x = rng.standard_normal((48, 64, 8)).astype(np.float16)
    got = dx.Module.load(dx.compile_model(m, assume={"H": 48, "W": 64}, conv_config="w4r2k16", db=db)).instance(H=48, W=64).infer(x)[0]
    ref = dx.Module.compile(m, conv_config="w4r2k16", features={"implicit_concat": False}).instance(H=48, W=64).infer(x)[0]
    assert_bits_equal(got, ref, "table-driven schedule")


GEOMETRY_CASES = [  # (R, S, (pad_y, pad_x), (stride_y, stride_x))
    (3, 3, (0, 0), (1, 1)),   # "valid"
    (3, 3, (1, 1), (2, 2)),   # the usual strided downsampling
    (3, 3, (0, 0), (2, 2)),
    (2, 2, (0, 0), (2, 2)),   # even filter, patch embedding style
    (4, 4, (1, 1), (2, 2)),
    (1, 1, (0, 0), (2, 2)),   # stride larger than the filter: halo rows and columns nobody reads
    (5, 3, (2, 0), (1, 2)),   # everything different in y and x
    (3, 3, (2, 2), (1, 1)),   # more padding than "same": the output is larger than the input
    (2, 3, (1, 1), (1, 1)),   # even rows
    (7, 7, (3, 3), (4, 4)),
    (3, 3, (1, 1), (3, 1)),
]


@pytest.mark.parametrize("config", [None, "w4r2k16", "s8r2k16", "m4r2k32x2", "p8r2k16", "t16r1k16", "p4r1k32", "q4r2k32x2"] + STRIDED_ONLY_CONFIGS)
@pytest.mark.parametrize("R,S,pad,stride", GEOMETRY_CASES)
def test_conv_padding_and_stride(oracle, config, R, S, pad, stride):
    """Filter extents 1..7 (even ones too), any zero padding, strides up to 4: out[y, x] reads in[y*sy + r - py, x*sx + s - px]."""
    rng = np.random.default_rng(R * 100 + S * 10 + pad[0] + stride[1])
    H, W, C, K = 45, 70, 24, 40
    x = rng.standard_normal((H, W, C)).astype(np.float16)
    m = dx.Model()
    t = m.relu(m.conv2d(m.input("input", "W", "H", C), he_weights(rng, K, C, R, S), small_bias(rng, K), stride=stride, padding=pad))
    m.output(t)
    try:
        mod = dx.Module.compile(m, conv_config=config)
    except dx.DenoxHipError as e:
        assert e.status == 5 and config is not None
        pytest.skip(str(e))
    assert mod.runtime_model.dispatch_count == 1
    inst = mod.instance(H=H, W=W)
    got = inst.infer(x)[0]
    want = oracle.run_graph(m.to_ops({"H": H, "W": W}), {"input": x}, "fp32")[t.name]
    assert got.shape == want.shape == ((H + 2 * pad[0] - R) // stride[0] + 1, (W + 2 * pad[1] - S) // stride[1] + 1, K)
    assert_conv_close(got, want, f"conv {R}x{S} pad {pad} stride {stride} {config}")


@pytest.mark.parametrize("config", [None, "p8r2k16", "m4r2k32x2"])
def test_strided_conv_with_fused_neighbours(oracle, config):
    """A stride-2 valid conv between a fused upsample + concat in front and a fused ReLU + 2x2 max pool behind, odd
    extents everywhere, channel counts that are not multiples of 8."""
    rng = np.random.default_rng(5)
    H, W = 38, 54
    lo = rng.standard_normal((H // 2, W // 2, 16)).astype(np.float16)
    x = rng.standard_normal((H, W, 9)).astype(np.float16)
    m = dx.Model()
    t = m.concat(m.upsample(m.input("lo", m.sym("W") // 2, m.sym("H") // 2, 16)), m.input("x", "W", "H", 9))
    t = m.pool(m.relu(m.conv2d(t, he_weights(rng, 19, 25), small_bias(rng, 19), stride=(2, 2), padding=(0, 0))))
    m.output(t)
    try:
        mod = dx.Module.compile(m, conv_config=config)
    except dx.DenoxHipError as e:
        assert e.status == 5 and config is not None
        pytest.skip(str(e))
    assert mod.runtime_model.dispatch_count == 1
    got = mod.instance(H=H, W=W).infer(lo, x)[0]
    want = oracle.run_graph(m.to_ops({"H": H, "W": W}), {"lo": lo, "x": x}, "fp32")[t.name]
    assert got.shape == want.shape == (9, 13, 19)
    assert_conv_close(got, want, f"strided conv with fused neighbours {config}")


@pytest.mark.parametrize("C0,C1", [(8, 16), (16, 8), (3, 9), (8, 9), (24, 40)])
def test_bandwidth_kernels_store_in_place(oracle, C0, C1):
    """Pool, upsample, activation, pad and slice as producers of concat sources: each stores into its channel range of
    the concat's tensor (16-byte stores when the range is aligned, element stores otherwise); bit-exact against the
    oracle and against the schedule with copies."""
    rng = np.random.default_rng(C0 * 7 + C1)
    H, W = 22, 36
    feeds = {"a": rng.standard_normal((H // 2, W // 2, C0)), "b": rng.standard_normal((H, W, C1)), "c": rng.standard_normal((2 * H, 2 * W, C0)),
             "d": rng.standard_normal((H - 3, W - 5, C1)), "e": rng.standard_normal((H + 4, W + 6, C0))}
    feeds = {k: v.astype(np.float16) for k, v in feeds.items()}
    m = dx.Model()
    a = m.input("a", m.sym("W") // 2, m.sym("H") // 2, C0)
    b = m.input("b", "W", "H", C1)
    c = m.input("c", m.sym("W") * 2, m.sym("H") * 2, C0)
    d = m.input("d", m.sym("W") - 5, m.sym("H") - 3, C1)
    e = m.input("e", m.sym("W") + 6, m.sym("H") + 4, C0)
    o1 = m.concat(m.upsample(a), m.relu(b))
    o2 = m.concat(m.pool(c), m.pad(d, 2, 3, 1, 2))
    o3 = m.concat(m.slice(e, 1, m.sym("W") + 1, 3, m.sym("H") + 3), m.activation(b, "leaky_relu", 0.25))
    for t in (o1, o2, o3):
        m.output(t)
    mod = dx.Module.compile(m)
    ref = dx.Module.compile(m, features={"implicit_concat": False})
    assert mod.runtime_model.dispatch_count == 6 and ref.runtime_model.dispatch_count == 9
    order = ["a", "b", "c", "d", "e"]
    got = mod.instance(H=H, W=W).infer(*[feeds[k] for k in order])
    cop = ref.instance(H=H, W=W).infer(*[feeds[k] for k in order])
    want = oracle.run_graph(m.to_ops({"H": H, "W": W}), feeds, "f16")
    for g, r, t in zip(got, cop, (o1, o2, o3)):
        assert_bits_equal(g, r, "in place against copied")
        assert_bits_equal(g, want[t.name], "in place against the oracle")


@pytest.mark.parametrize("C", [1, 2, 4, 5, 6, 7, 10, 11, 13, 14, 15, 23, 31, 41])
def test_every_channel_remainder(oracle, C):
    """Channel counts with every remainder modulo 8, below and above 8: the bandwidth kernels move a pixel's full chunks of 8
    channels as 16-byte accesses and the remainder as 8 + 4 + 2 bytes.  Each op alone and stored in place into a concat whose
    other half is written by another dispatch -- a store one element too wide would damage the neighbour's channels."""
    rng = np.random.default_rng(C)
    H, W = 10, 27
    x = rng.standard_normal((H, W, C)).astype(np.float16)
    m = dx.Model()
    inp = m.input("input", "W", "H", C)
    singles = [m.relu(inp), m.activation(inp, "leaky_relu", 0.125), m.pool(inp), m.pool(inp, func="avg"), m.upsample(inp),
               m.pad(inp, 1, 2, 3, 0), m.pad(inp, 2, 1, 0, 3, mode="zero"), m.slice(inp, 1, m.sym("W") - 2, 2, m.sym("H") - 1)]
    pairs = [m.concat(m.relu(inp), m.activation(inp, "leaky_relu", 0.5)),
             m.concat(m.pad(m.pool(inp), 0, m.sym("W") - m.sym("W") // 2, 0, m.sym("H") - m.sym("H") // 2), m.relu(inp)),
             m.concat(m.upsample(inp), m.pad(inp, 0, m.sym("W"), m.sym("H"), 0))]
    for t in singles + pairs:
        m.output(t)
    mod = dx.Module.compile(m)
    names = [d_["name"] for d_ in dx.describe(mod.dnx, H=H, W=W)["dispatches"]]
    assert sum(n.endswith("+concat") for n in names) >= 5, names
    got = mod.instance(H=H, W=W).infer(x)
    want = oracle.run_graph(m.to_ops({"H": H, "W": W}), {"input": x}, "f16")
    for t, g in zip(singles + pairs, got):
        assert_bits_equal(g, want[t.name], f"C={C} {t.name}")


@pytest.mark.parametrize("H,W,C", [(7, 24, 9), (6, 25, 9), (5, 32, 73), (9, 31, 73), (4, 16, 12), (3, 5, 15), (1, 1, 9), (2, 3, 11), (33, 130, 10)])
def test_rows_moved_as_runs_of_aligned_vectors(H, W, C):
    """Channel counts that are not multiples of 8: activation, pad, slice and upsample move a row as one run of halves in
    aligned 16-byte vectors (the first and last vector of a run element by element, an upsampled vector from one or two
    source pieces).  Extents whose runs start at every offset from a 16-byte boundary, runs shorter than a vector, rows
    whose replicas share an alignment and rows that do not; checked against numpy, bit for bit."""
    rng = np.random.default_rng(H * 1000 + W * 10 + C)
    x = rng.standard_normal((H, W, C)).astype(np.float16)
    m = dx.Model()
    inp = m.input("input", "W", "H", C)
    outs = [m.relu(inp), m.pad(inp, 0, 0, 2, 3), m.pad(inp, 0, 0, 1, 0, mode="zero"), m.pad(inp, 1, 2, 0, 1), m.slice(inp, 0, "W", 0, m.sym("H") - 0),
            m.upsample(inp)]
    if H > 2 and W > 2:
        outs += [m.slice(inp, 0, "W", 1, m.sym("H") - 1), m.slice(inp, 1, m.sym("W") - 1, 1, "H")]
    for t in outs:
        m.output(t)
    mod = dx.Module.compile(m)
    names = [d_["entry_point"] for d_ in dx.describe(mod.dnx, H=H, W=W)["dispatches"]]
    assert all(n.endswith("f") for n in names), names
    got = mod.instance(H=H, W=W).infer(x)
    want = [np.maximum(x, np.float16(0)), np.pad(x, ((2, 3), (0, 0), (0, 0)), mode="edge"), np.pad(x, ((1, 0), (0, 0), (0, 0))),
            np.pad(x, ((0, 1), (1, 2), (0, 0)), mode="edge"), x, np.repeat(np.repeat(x, 2, 0), 2, 1)]
    if H > 2 and W > 2:
        want += [x[1:H - 1], x[1:, 1:W - 1]]
    for t, g, w in zip(outs, got, want):
        assert_bits_equal(g, w, f"{t.name} {H}x{W}x{C}")


@pytest.mark.parametrize("CA,CB", [(3, 3), (9, 64), (64, 9), (8, 8), (12, 20), (73, 7), (16, 24), (1, 1), (5, 17)])
def test_concat_copy_of_two_sources(oracle, CA, CB):
    """Both sources copied by one launch that writes whole pixels (model inputs cannot be written in place, so neither source
    moves): bit-exact for aligned and odd channel counts, image heights that are not a multiple of the rows a thread covers,
    and for the same tensor on both sides."""
    rng = np.random.default_rng(CA * 100 + CB)
    m = dx.Model()
    ta, tb = m.input("a", "W", "H", CA), m.input("b", "W", "H", CB)
    cat, twice = m.concat(ta, tb), m.concat(tb, tb)
    m.output(cat)
    m.output(twice)
    mod = dx.Module.compile(m)
    # (21 x 37: a few workgroups; 67 x 129 and 1 x 1: pixel counts that are not a multiple of what a workgroup takes,
    # and a last 16-byte vector of the result that is only partly inside it)
    for H, W in [(21, 37), (67, 129), (1, 1), (3, 5)]:
        a = rng.standard_normal((H, W, CA)).astype(np.float16)
        b = rng.standard_normal((H, W, CB)).astype(np.float16)
        d = dx.describe(mod.dnx, H=H, W=W)
        assert [x["name"] for x in d["dispatches"]] == ["concat-copy", "concat-copy"]
        got_cat, got_twice = mod.instance(H=H, W=W).infer(a, b)
        assert_bits_equal(got_cat, np.concatenate([a, b], axis=2), "concat of two inputs")
        assert_bits_equal(got_twice, np.concatenate([b, b], axis=2), "concat of a tensor with itself")
        assert_bits_equal(got_cat, oracle.concat(a, b), "concat against the oracle")


@pytest.mark.parametrize("C,k", [(3, (2, 2)), (8, (2, 2)), (64, (2, 2)), (16, (3, 3)), (9, (2, 3)), (32, (4, 4))])
def test_average_pool(oracle, C, k):
    """Average pool (sum in fp32 in window order, times 1/(ky*kx), one rounding): bit-exact against the oracle routine alone,
    behind a conv (whose epilogue folds only the maximum, so the pool stays a dispatch) and written in place into a concat."""
    rng = np.random.default_rng(C + k[0])
    H, W = 37, 50
    x = rng.standard_normal((H, W, C)).astype(np.float16)
    m = dx.Model()
    inp = m.input("input", "W", "H", C)
    a = m.pool(inp, k, func="avg")
    c = m.relu(m.conv2d(inp, he_weights(rng, 16, C), small_bias(rng, 16)))
    q = m.pool(c, k, func="avg")
    cat = m.concat(m.pool(inp, k, func="avg"), m.pool(inp, k, func="max"))
    for t in (a, q, cat):
        m.output(t)
    mod = dx.Module.compile(m)
    names = [d_["name"] for d_ in dx.describe(mod.dnx, H=H, W=W)["dispatches"]]
    assert "conv3x3+relu" in names and "conv3x3+relu+maxpool" not in names and names.count("avgpool") + names.count("avgpool+concat") == 3
    got_a, got_q, got_cat = mod.instance(H=H, W=W).infer(x)
    ops = m.to_ops({"H": H, "W": W})
    want = oracle.run_graph(ops, {"input": x}, "f16")
    assert got_a.shape == (H // k[0], W // k[1], C)
    assert_bits_equal(got_a, want[a.name], "average pool")
    assert_bits_equal(got_cat, want[cat.name], "average pool into a concat")
    # behind the conv: the mean of the fp32-evaluated conv outputs, within the conv tolerance
    assert_conv_close(got_q, oracle.run_graph(ops, {"input": x}, "fp32")[q.name], "average pool behind a conv")


@pytest.mark.parametrize("C", [3, 8, 9, 64])
def test_zero_padding(oracle, C):
    """Pad with zeros (F.pad mode="constant"): a dispatch of its own (the conv loaders fold only the replicate mode), bit-exact
    alone and in front of a conv, whose own zero padding then sees zeros twice."""
    rng = np.random.default_rng(C)
    H, W = 23, 41
    x = rng.standard_normal((H, W, C)).astype(np.float16)
    m = dx.Model()
    p = m.pad(m.input("input", "W", "H", C), 2, 5, 1, 3, mode="zero")
    y = m.relu(m.conv2d(p, he_weights(rng, 16, C), small_bias(rng, 16)))
    m.output(p)
    m.output(y)
    mod = dx.Module.compile(m)
    names = [d_["name"] for d_ in dx.describe(mod.dnx, H=H, W=W)["dispatches"]]
    assert names == ["pad", "conv3x3+relu"]
    got_p, got_y = mod.instance(H=H, W=W).infer(x)
    want = oracle.run_graph(m.to_ops({"H": H, "W": W}), {"input": x}, "f16")
    assert_bits_equal(got_p, want[p.name], "zero pad")
    assert got_p.shape == (H + 4, W + 7, C) and not got_p[0].any() and not got_p[:, :2].any()
    assert_conv_close(got_y, oracle.run_graph(m.to_ops({"H": H, "W": W}), {"input": x}, "fp32")[y.name], "conv behind a zero pad")
