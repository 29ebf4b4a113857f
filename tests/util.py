"""Helpers shared by the GPU parity tests: seeded tensors and the parity bar."""
import numpy as np

# north-star tolerance for conv outputs, on the final fp16 output against an fp32 evaluation
CONV_MAX_ABS = 2e-2
CONV_MEAN_ABS = 2e-3


def he_weights(rng, K, C, R=3, S=3):
    return (rng.standard_normal((K, C, R, S)) * np.sqrt(2.0 / (R * S * C))).astype(np.float16)


def small_bias(rng, K):
    return (rng.standard_normal(K) * 0.01).astype(np.float16)


def assert_conv_close(got_f16, want_f32, what=""):
    got = np.asarray(got_f16, np.float32)
    want = np.asarray(want_f32, np.float32)
    assert got.shape == want.shape, (got.shape, want.shape)
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    err = np.abs(got - want)
    # the bar is absolute on outputs of O(1) magnitude; scale it for layers whose outputs are larger
    scale = max(1.0, float(np.abs(want).max()))
    assert err.max() <= CONV_MAX_ABS * scale, f"{what}: max abs err {err.max():.4g} (scale {scale:.3g}) at {np.unravel_index(err.argmax(), err.shape)}"
    assert err.mean() <= CONV_MEAN_ABS * scale, f"{what}: mean abs err {err.mean():.4g}"


def assert_reference_allclose(got_f16, want_f16, what="", rtol=1e-3, atol=1e-2):
    """The reference's own acceptance: torch.allclose(output, expected, rtol=1e-3, atol=1e-2) against a binary16
    evaluation of the same layers (test/__init__.py:45-49,97 of the reference)."""
    got = np.asarray(got_f16, np.float32)
    want = np.asarray(want_f16, np.float32)
    assert got.shape == want.shape, (got.shape, want.shape)
    excess = np.abs(got - want) - (atol + rtol * np.abs(want))
    assert (excess <= 0).all(), f"{what}: |got - want| exceeds atol + rtol |want| by {excess.max():.4g} at {np.unravel_index(excess.argmax(), excess.shape)}"


def assert_bits_equal(got, want, what=""):
    g = np.ascontiguousarray(got, np.float16).view(np.uint16)
    w = np.ascontiguousarray(want, np.float16).view(np.uint16)
    assert g.shape == w.shape, (g.shape, w.shape)
    bad = np.argwhere(g != w)
    assert bad.size == 0, f"{what}: {len(bad)} differing elements, first at {tuple(bad[0])}: got {g[tuple(bad[0])]:#06x} want {w[tuple(bad[0])]:#06x}"


_poison = None


def fill_lds_with_nans():
    """Runs a conv whose image, weights and bias are all NaN on every compute unit, in the configuration that keeps the
    most LDS (resident weights + halo).  What a kernel leaves in LDS is what the next one finds there: a kernel that
    multiplies a staged value it never wrote with a zero weight then produces NaN.  Called in front of fuzzed layers so
    that such a read shows up whatever ran before."""
    global _poison
    import denox_amd as dx
    if _poison is None:
        m = dx.Model()
        nan = np.float16(np.nan)
        m.output(m.conv2d(m.input("x", "W", "H", 64), np.full((64, 64, 3, 3), nan, np.float16), np.full(64, nan, np.float16)))
        _poison = (dx.Module.compile(m, conv_config="s8r2k16").instance(H=256, W=512), np.full((256, 512, 64), nan, np.float16))
    _poison[0].infer(_poison[1])
