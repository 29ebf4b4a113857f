"""Internal tensors in the channel-block-major layout (CHWC8) as an alternative to HWC.

Every internal tensor whose channel count is a multiple of 8 has two nodes in the graph the schedule is selected from, one
per layout, as in the reference (compiler/src/denox/compiler/specialization/specialization.cpp:13-16,282-306); convolutions
read either layout and write either, pool / upsample / activation run plane by plane, and a concat of two block-major
tensors that nobody else reads needs no dispatch (placement/placement.cpp:232-255).  With `layout_preference=1` every
candidate that touches a CHWC8 tensor counts half its cost, which forces that path here; results must equal the pixel-major
schedule's: bit for bit where only data moves, within the conv tolerance against the oracle otherwise."""
import numpy as np
import pytest

import denox_amd as dx
from denox_amd import networks
from util import assert_bits_equal, assert_conv_close, fill_lds_with_nans, he_weights, small_bias

pytestmark = pytest.mark.gpu

BLOCKED = dict(layout_preference=1)
BLOCKED_CONFIGS = ["w4r2k16", "w8r2k32", "w4r1kfn", "p16r2k16", "s8r2k16", "t8r2k32", "t16r1k32", "m4r2k32x1", "m8r2k32x2", "m4r2kfx1", "q8r2k32x2", "s12r1k16", "s8r2k32s"]


def entries(mod, **ext):
    return [d["entry_point"] for d in dx.describe(mod.dnx, **ext)["dispatches"]]


def internal_formats(mod, **ext):
    d = dx.describe(mod.dnx, **ext)
    return [t["format"] for t in d["tensors"] if not t["param"]]


@pytest.mark.parametrize("config", BLOCKED_CONFIGS)
@pytest.mark.parametrize("C,K,tail", [(64, 64, "relu"), (48, 80, "pool"), (96, 112, "none"), (32, 32, "pool"), (16, 40, "relu")])
def test_conv_reads_and_writes_either_layout(oracle, config, C, K, tail):
    """conv(64 -> C) writes CHWC8, conv(C -> K) reads and writes it, conv(K -> 64) reads it and writes HWC."""
    rng = np.random.default_rng(C + K)
    m = dx.Model()
    t = m.input("input", "W", "H", 64)
    a = m.relu(m.conv2d(t, he_weights(rng, C, 64), small_bias(rng, C)))
    b = m.conv2d(a, he_weights(rng, K, C), small_bias(rng, K))
    if tail in ("relu", "pool"):
        b = m.relu(b)
    if tail == "pool":
        b = m.pool(b)
    c = m.conv2d(b, he_weights(rng, 64, K), small_bias(rng, 64))
    m.output(c)
    try:
        mod = dx.Module.compile(m, conv_config=config, features=dict(BLOCKED, conv_conv_fusion=False))
    except dx.DenoxHipError as e:
        assert e.status == 5
        pytest.skip(str(e))
    for H, W in [(37, 70), (16, 32), (130, 45)]:
        names = entries(mod, H=H, W=W)
        if not ("_bo_" in names[0] and "_bi_bo_" in names[1] and "_bi_" in names[2]):
            pytest.skip(f"{config} does not exist in the blocked form for this layer: {names}")
        x = rng.standard_normal((H, W, 64)).astype(np.float16)
        fill_lds_with_nans()
        got = mod.instance(H=H, W=W).infer(x)[0]
        want = oracle.run_graph(m.to_ops({"H": H, "W": W}), {"input": x}, "fp32")[c.name]
        assert_conv_close(got, want, f"blocked {config} {C}->{K} {H}x{W}")


@pytest.mark.parametrize("staged", ["r4r2k16n", "c4r2k32n"])
def test_staged_result_kernel_reads_block_major_sources(oracle, tmp_path, staged):
    """r4r2k16n / c4r2k32n (the result goes to memory through LDS, pixel-major only) reading a CHWC8 tensor: no forced configuration
    reaches that combination, because the producer must write CHWC8 with another configuration, so the selection is
    steered to it through a timing table with made-up samples for exactly the wanted candidates."""
    import re
    rng = np.random.default_rng(21)
    m = dx.Model()
    t = m.input("input", "W", "H", 64)
    a = m.relu(m.conv2d(t, he_weights(rng, 48, 64), small_bias(rng, 48)))
    b = m.relu(m.conv2d(a, he_weights(rng, 80, 48), small_bias(rng, 80)))
    c = m.conv2d(b, he_weights(rng, 64, 80), small_bias(rng, 64))
    m.output(c)
    wanted = {"conv3x3_c64_k48_relu_bo_w4r2k16", "conv3x3_c48_k80_relu_bi_" + staged, "conv3x3_c80_k64_" + staged}
    feats = dict(conv_conv_fusion=False)
    db = dx.Db(str(tmp_path / "steer.db"))
    db.populate(m, features=feats)
    for i, row in enumerate(db.dump_csv().splitlines()[1:]):
        if re.search(r"KERNEL_NAME=(\S+)", row).group(1) in wanted:
            for _ in range(3):
                db.add_sample(i, 1000.0)
    mod = dx.Module.compile(m, db=db, features=feats)
    for H, W in [(37, 70), (16, 32), (130, 45)]:
        assert set(entries(mod, H=H, W=W)) == wanted
        x = rng.standard_normal((H, W, 64)).astype(np.float16)
        fill_lds_with_nans()
        got = mod.instance(H=H, W=W).infer(x)[0]
        want = oracle.run_graph(m.to_ops({"H": H, "W": W}), {"input": x}, "fp32")[c.name]
        assert_conv_close(got, want, f"staged result, block-major source {H}x{W}")


def test_every_blocked_configuration_runs_somewhere():
    rng = np.random.default_rng(0)
    for config in BLOCKED_CONFIGS:
        hit = False
        for C, K in [(64, 64), (48, 80), (96, 112), (32, 32), (16, 40)]:
            m = dx.Model()
            a = m.relu(m.conv2d(m.input("input", "W", "H", 64), he_weights(rng, C, 64), small_bias(rng, C)))
            m.output(m.conv2d(m.conv2d(a, he_weights(rng, K, C), small_bias(rng, K)), he_weights(rng, 64, K), small_bias(rng, 64)))
            try:
                mod = dx.Module.compile(m, conv_config=config, features=dict(BLOCKED, conv_conv_fusion=False))
            except dx.DenoxHipError:
                continue
            hit |= "_bi_bo_" in entries(mod, H=64, W=64)[1]
        assert hit, config


def test_data_movement_on_blocked_tensors_is_bit_exact(oracle):
    """relu, max pool, upsample as dispatches of their own on CHWC8 tensors (plane by plane), and a concat of two such tensors
    that is pure aliasing: the same bits as the pixel-major schedule of the same model."""
    rng = np.random.default_rng(4)
    H, W = 38, 52
    m = dx.Model()
    t = m.input("input", "W", "H", 8)
    a = m.conv2d(t, he_weights(rng, 24, 8), small_bias(rng, 24))
    u = m.upsample(m.pool(m.relu(a)))
    b = m.activation(m.conv2d(t, he_weights(rng, 16, 8), small_bias(rng, 16)), "leaky_relu", 0.25)
    cat = m.concat(u, b)
    out = m.conv2d(cat, he_weights(rng, 8, 40), small_bias(rng, 8))
    m.output(out)
    off = dict(conv_relu_fusion=False, concat_conv_fusion=False, upsample_fusion=False, pool_fusion=False, conv_conv_fusion=False)
    blocked = dx.Module.compile(m, conv_config="w4r2k16", features=dict(off, **BLOCKED))
    plain = dx.Module.compile(m, conv_config="w4r2k16", features=dict(off, blocked_layout=False))
    names = [d["name"] + ":" + d["debug_info"].split(" | ")[0] for d in dx.describe(blocked.dnx, H=H, W=W)["dispatches"]]
    assert sum("chwc8" in n for n in names) >= 6, names
    assert not any(n.startswith("concat") for n in names), names  # the concat of two blocked tensors is aliasing, no dispatch
    assert 3 in internal_formats(blocked, H=H, W=W) and 3 not in internal_formats(plain, H=H, W=W)
    x = rng.standard_normal((H, W, 8)).astype(np.float16)
    got = blocked.instance(H=H, W=W).infer(x)[0]
    assert_conv_close(got, oracle.run_graph(m.to_ops({"H": H, "W": W}), {"input": x}, "fp32")[out.name], "blocked data movement")
    # the same conv configuration on both sides accumulates in the same order whatever the layout, and everything between
    # the convs only moves data: identical bits
    assert_bits_equal(got, plain.instance(H=H, W=W).infer(x)[0], "blocked vs pixel-major")


@pytest.mark.parametrize("widths", [(16, 24, 8), (64, 64, 64), (8, 24, 16, 40)])
@pytest.mark.parametrize("features", [{}, BLOCKED], ids=["default", "blocked"])
def test_concat_of_concats(oracle, widths, features):
    """concat(concat(a, b), c) and a three-deep nest with channel counts that are multiples of 8: when the concats are
    aliasing only, every leaf must land inside the outermost result.  Bit for bit against the schedule without block-major
    tensors (which copies or writes in place per pixel), and against the oracle."""
    from test_host import _nested_concat_model
    m, _, out = _nested_concat_model(widths)
    feats = dict(conv_conv_fusion=False)
    mod = dx.Module.compile(m, conv_config="w4r2k16", features=dict(feats, **features))
    plain = dx.Module.compile(m, conv_config="w4r2k16", features=dict(feats, blocked_layout=False))
    rng = np.random.default_rng(5)
    for H, W in [(32, 32), (19, 45)]:
        x = rng.standard_normal((H, W, 16)).astype(np.float16)
        got = mod.instance(H=H, W=W).infer(x)[0]
        want = oracle.run_graph(m.to_ops({"H": H, "W": W}), {"input": x}, "fp32")[out.name]
        assert_conv_close(got, want, f"nested concat {widths} {H}x{W}")
        assert_bits_equal(got, plain.instance(H=H, W=W).infer(x)[0], f"nested concat {widths}: blocked vs pixel-major")
    if features:
        assert not any(n.startswith("concat") or n.startswith("copy") for n in entries(mod, H=32, W=32)), entries(mod, H=32, W=32)


@pytest.mark.parametrize("H,W", [(64, 96), (75, 101), (16, 16), (33, 250)])
def test_oidn_unet_with_blocked_internal_tensors(oracle, H, W):
    m, _ = networks.build("oidn_unet", seed=6)
    x = networks.synthetic_input("oidn_unet", H, W, seed=6)
    mod = dx.Module.compile(m, assume={"H": H, "W": W}, features=BLOCKED)
    fmts = internal_formats(mod, H=H, W=W)
    assert fmts.count(3) >= 5, fmts
    got = mod.instance(H=H, W=W).infer(x)[0]
    from test_gpu_unet import check_net
    check_net(oracle, m, x, got, H, W, f"oidn blocked {H}x{W}")


def test_full_size_oidn_unet_blocked(oracle):
    from test_gpu_unet import check_crops
    H, W = 1080, 1920
    m, _ = networks.build("oidn_unet", seed=0)
    x = networks.synthetic_input("oidn_unet", H, W, seed=0)
    mod = dx.Module.compile(m, assume={"H": H, "W": W}, features=BLOCKED)
    assert internal_formats(mod, H=H, W=W).count(3) >= 5
    got = mod.instance(H=H, W=W).infer(x)[0]
    check_crops(oracle, m, x, got, H, W, [(0, 0), (400, 800), (H - 272 + 8, W - 272)], "blocked 1080p")


@pytest.mark.parametrize("config", ["x8r2k16", "x4r2k32", "x4r4k16", "x4r2k16", "y4r2k32", "z4r2k64", "v4r2k64", "v4r2k16", "u4r2k32", "d4r2k64", "t4r2k32"])
@pytest.mark.parametrize("C,K1,K2,tail", [(64, 32, 32, "pool"), (40, 32, 16, "relu"), (48, 16, 24, "none")])
def test_conv_pair_reads_and_writes_either_layout(oracle, config, C, K1, K2, tail):
    """conv -> conv in one dispatch between two block-major tensors."""
    rng = np.random.default_rng(C + K1 + K2)
    m = dx.Model()
    t = m.input("input", "W", "H", 16)
    a = m.relu(m.conv2d(t, he_weights(rng, C, 16), small_bias(rng, C)))
    b = m.relu(m.conv2d(a, he_weights(rng, K1, C), small_bias(rng, K1)))
    c = m.conv2d(b, he_weights(rng, K2, K1), small_bias(rng, K2))
    if tail in ("relu", "pool"):
        c = m.relu(c)
    if tail == "pool":
        c = m.pool(c)
    d = m.conv2d(c, he_weights(rng, 40, K2), small_bias(rng, 40))  # more than 32 output channels: never the second half of a pair
    m.output(d)
    try:
        mod = dx.Module.compile(m, conv_config=config, features=BLOCKED)
    except dx.DenoxHipError as e:
        assert e.status == 5
        pytest.skip(str(e))
    for H, W in [(38, 70), (16, 32), (130, 44)]:
        names = entries(mod, H=H, W=W)
        pair = [n for n in names if n.startswith("convpair")]
        if not (pair and "_bi_bo_" in pair[0]):
            pytest.skip(f"{config}: no blocked pair for this layer: {names}")
        x = rng.standard_normal((H, W, 16)).astype(np.float16)
        fill_lds_with_nans()
        got = mod.instance(H=H, W=W).infer(x)[0]
        want = oracle.run_graph(m.to_ops({"H": H, "W": W}), {"input": x}, "fp32")[d.name]
        assert_conv_close(got, want, f"blocked pair {config} {C}->{K1}->{K2} {H}x{W}")
