"""Seeded random layer graphs on the GPU against the CPU oracle: channel counts, extents, pad / crop offsets, fusion
switches and kernel configurations drawn at random, so that combinations nobody listed by hand get exercised
(odd extents down to 1 x 1, channel counts around the 8 / 16 / 32 vector and block boundaries, every prologue and
epilogue of the conv kernels in one dispatch).  Each case prints its parameters before it runs."""
import numpy as np
import pytest

import denox_amd as dx
from util import assert_conv_close, fill_lds_with_nans, he_weights, small_bias

pytestmark = pytest.mark.gpu


CONFIGS = [None, None, None, "w4r2k16", "w4r1k32", "w8r2k32", "w2r2kfn", "w4r1kfm", "p8r1k16", "p16r1k16", "p8r2k32", "p4r4k16", "p4r2k32n",
           "s8r2k16", "m4r2k32x2", "m4r1kfx2", "m4r2kfx1n", "q8r2k32x2", "q4r2k32x1n", "t16r1k16", "t8r2k16", "u8r2k32x2", "f8r1", "f4r2", "f4r1"]
CHANNELS = [1, 2, 3, 7, 8, 9, 15, 16, 17, 24, 31, 32, 33, 40, 48, 64, 73, 80]


def one_case(oracle, seed):
    rng = np.random.default_rng(seed)
    H, W = int(rng.integers(1, 48)), int(rng.integers(1, 72))
    up, cat = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    pool, crop, pad = bool(rng.integers(0, 2)), bool(rng.integers(0, 3) == 0), bool(rng.integers(0, 3) == 0)
    act = ["none", "relu", "leaky"][int(rng.integers(0, 3))]
    CA, CB, K = (int(rng.choice(CHANNELS)) for _ in range(3))
    config = CONFIGS[int(rng.integers(0, len(CONFIGS)))]
    feats = {k: bool(rng.integers(0, 4)) for k in ("conv_relu_fusion", "concat_conv_fusion", "upsample_fusion", "pool_fusion", "pad_fusion", "slice_fusion")}
    if up:
        H, W = 2 * max(1, H // 2), 2 * max(1, W // 2)
    pl, pr, pt, pb = (int(v) for v in rng.integers(0, 5, 4)) if pad else (0, 0, 0, 0)
    print(f"fuzz seed={seed} H={H} W={W} CA={CA} CB={CB if cat else 0} K={K} up={up} pool={pool} pad={(pl, pr, pt, pb)} crop={crop} act={act} config={config} feats={feats}", flush=True)

    m = dx.Model()
    feeds = {}
    Hs, Ws = H - pt - pb, W - pl - pr  # extents of the stored (un-padded) full-resolution source
    if pad and (Hs < 1 or Ws < 1):
        pad, (pl, pr, pt, pb), Hs, Ws = False, (0, 0, 0, 0), H, W
    if up:
        a = m.input("a", m.sym("W") // 2, m.sym("H") // 2, CA)
        feeds["a"] = rng.standard_normal((H // 2, W // 2, CA)).astype(np.float16)
        t = m.upsample(a)
    else:
        a = m.input("a", m.sym("W") - (pl + pr), m.sym("H") - (pt + pb), CA)
        feeds["a"] = rng.standard_normal((Hs, Ws, CA)).astype(np.float16)
        t = m.pad(a, pl, pr, pt, pb) if pad else a
    C = CA
    if cat:
        b = m.input("b", m.sym("W") - (pl + pr), m.sym("H") - (pt + pb), CB)
        feeds["b"] = rng.standard_normal((Hs, Ws, CB)).astype(np.float16)
        t = m.concat(t, m.pad(b, pl, pr, pt, pb) if pad else b)
        C += CB
    t = m.conv2d(t, he_weights(rng, K, C), small_bias(rng, K) if rng.integers(0, 4) else None)
    if act == "relu":
        t = m.relu(t)
    elif act == "leaky":
        t = m.activation(t, "leaky_relu", 0.125)
    if pool and H >= 2 and W >= 2:
        t = m.pool(t)
    elif crop and H >= 3 and W >= 3:
        l, tp = int(rng.integers(0, W // 2)), int(rng.integers(0, H // 2))
        t = m.slice(t, l, int(rng.integers(l + 1, W + 1)), tp, int(rng.integers(tp + 1, H + 1)))
    m.output(t)
    try:
        mod = dx.Module.compile(m, features=feats, conv_config=config)
    except dx.DenoxHipError as e:
        assert e.status == 5, str(e)  # this configuration does not exist for this layer
        mod = dx.Module.compile(m, features=feats)
    inst = mod.instance(H=H, W=W)
    fill_lds_with_nans()
    got = inst.infer(*[feeds[k] for k in ("a", "b") if k in feeds])[0]
    want = oracle.run_graph(m.to_ops({"H": H, "W": W}), feeds, "fp32")[t.name]
    assert_conv_close(got, want, f"fuzz seed {seed}")


@pytest.mark.parametrize("block", range(8))
def test_random_fused_conv_graphs(oracle, block):
    for seed in range(block * 25, block * 25 + 25):
        one_case(oracle, seed)


GEOMETRY_CONFIGS = [None, None, "w4r2k16", "w4r1k32", "w2r2kfn", "p8r1k16", "p4r2k32n", "m4r2k32x2", "m4r2kfx1n", "q4r2k32x1n", "t8r1k16", "w2r1k16n", "m2r1k32x1n", "w2r2k16n"]


def one_geometry_case(oracle, seed):
    """A conv with a random filter extent, padding and stride; half of the time twice, concatenated (each branch then
    stores straight into the concat's tensor), with a pool, a crop or another conv behind."""
    rng = np.random.default_rng(10_000 + seed)
    H, W = int(rng.integers(6, 41)), int(rng.integers(6, 61))
    C, K0, K1 = (int(rng.choice(CHANNELS[:14])) for _ in range(3))
    R, S = int(rng.integers(1, 6)), int(rng.integers(1, 6))
    py, px = int(rng.integers(0, 4)), int(rng.integers(0, 4))
    sy, sx = int(rng.integers(1, 4)), int(rng.integers(1, 4))
    Ho, Wo = (H + 2 * py - R) // sy + 1, (W + 2 * px - S) // sx + 1
    two, act, tail = bool(rng.integers(0, 2)), ["none", "relu", "leaky"][int(rng.integers(0, 3))], ["none", "pool", "crop", "conv"][int(rng.integers(0, 4))]
    config = GEOMETRY_CONFIGS[int(rng.integers(0, len(GEOMETRY_CONFIGS)))]
    feats = {k: bool(rng.integers(0, 4)) for k in ("conv_relu_fusion", "concat_conv_fusion", "pool_fusion", "slice_fusion", "implicit_concat")}
    print(f"geometry seed={seed} H={H} W={W} C={C} K={K0},{K1 if two else 0} filter={R}x{S} pad={(py, px)} stride={(sy, sx)} act={act} tail={tail} config={config} feats={feats}", flush=True)
    assert Ho >= 1 and Wo >= 1
    m = dx.Model()
    x = m.input("a", "W", "H", C)
    feeds = {"a": rng.standard_normal((H, W, C)).astype(np.float16)}

    def branch(K):
        y = m.conv2d(x, he_weights(rng, K, C, R, S), small_bias(rng, K) if rng.integers(0, 4) else None, stride=(sy, sx), padding=(py, px))
        return m.relu(y) if act == "relu" else m.activation(y, "leaky_relu", 0.125) if act == "leaky" else y
    t = branch(K0)
    Kt = K0
    if two:
        t = m.concat(t, branch(K1))
        Kt += K1
    if tail == "pool" and Ho >= 2 and Wo >= 2:
        t = m.pool(t)
    elif tail == "crop" and Ho >= 2 and Wo >= 2:
        l, tp = int(rng.integers(0, Wo // 2)), int(rng.integers(0, Ho // 2))
        t = m.slice(t, l, int(rng.integers(l + 1, Wo + 1)), tp, int(rng.integers(tp + 1, Ho + 1)))
    elif tail == "conv":
        t = m.conv2d(t, he_weights(rng, 8, Kt), small_bias(rng, 8))
    m.output(t)
    try:
        mod = dx.Module.compile(m, features=feats, conv_config=config)
    except dx.DenoxHipError as e:
        assert e.status == 5, str(e)
        mod = dx.Module.compile(m, features=feats)
    inst = mod.instance(H=H, W=W)
    fill_lds_with_nans()
    got = inst.infer(feeds["a"])[0]
    want = oracle.run_graph(m.to_ops({"H": H, "W": W}), feeds, "fp32")[t.name]
    assert_conv_close(got, want, f"geometry seed {seed}")


@pytest.mark.parametrize("block", range(6))
def test_random_conv_geometry(oracle, block):
    for seed in range(block * 25, block * 25 + 25):
        one_geometry_case(oracle, seed)


@pytest.mark.parametrize("CA,CB", [(8, 33), (24, 0), (40, 17), (32, 33)])
def test_stale_lds_contents_do_not_reach_the_result(oracle, CA, CB):
    """The upsample-folding kernel stages its sources padded to 16 channels and multiplies the padding with zero weights:
    the padding must be stored as zeros, not left as whatever the previous kernel had in LDS (0 * NaN is NaN).  A conv of
    NaNs runs first so that LDS is full of them, then layers whose channel counts leave 8 padded channels."""
    rng = np.random.default_rng(CA + CB)
    H, W = 36, 44
    m = dx.Model()
    a = m.input("a", m.sym("W") // 2, m.sym("H") // 2, CA)
    feeds = {"a": rng.standard_normal((H // 2, W // 2, CA)).astype(np.float16)}
    t = m.upsample(a)
    if CB:
        t = m.concat(t, m.input("b", "W", "H", CB))
        feeds["b"] = rng.standard_normal((H, W, CB)).astype(np.float16)
    t = m.conv2d(t, he_weights(rng, 16, CA + CB), small_bias(rng, 16))
    m.output(t)
    want = oracle.run_graph(m.to_ops({"H": H, "W": W}), feeds, "fp32")[t.name]
    for config in ("f4r1", "f8r1", "f4r2"):
        try:
            inst = dx.Module.compile(m, conv_config=config).instance(H=H, W=W)
        except dx.DenoxHipError as e:
            assert e.status == 5, str(e)
            continue
        for _ in range(3):
            fill_lds_with_nans()
            got = inst.infer(*[feeds[k] for k in ("a", "b") if k in feeds])[0]
            assert_conv_close(got, want, f"{config} after a kernel that left NaNs in LDS")
