"""Helpers shared by the GPU parity tests: seeded tensors and the parity bar."""
import numpy as np

# the bars live beside the checker, which bench.py's parity leg uses as well
from oracle import CONV_MAX_ABS, CONV_MEAN_ABS, FLOOR_FACTOR_MAX, FLOOR_FACTOR_MEAN, conv_parity  # noqa: F401


def he_weights(rng, K, C, R=3, S=3):
    return (rng.standard_normal((K, C, R, S)) * np.sqrt(2.0 / (R * S * C))).astype(np.float16)


def small_bias(rng, K):
    return (rng.standard_normal(K) * 0.01).astype(np.float16)


def assert_conv_close(got_f16, want_f32, what="", floor=None):
    """max abs <= 2e-2 and mean abs <= 2e-3 against the fp32 evaluation; where that is out of reach of binary16 storage, at most
    FLOOR_FACTOR_MAX / FLOOR_FACTOR_MEAN times the error of the oracle's binary16-storage evaluation (`floor`)."""
    r = conv_parity(got_f16, want_f32, floor)
    assert r["finite"], f"{what}: non-finite output"
    note = "" if r["floor_max_abs"] is None else f" (binary16-storage floor {r['floor_max_abs']:.4g} / {r['floor_mean_abs']:.4g})"
    if not r["literal_ok"] and floor is None:
        note = " (no binary16-storage floor was given for this case: the absolute bar applies)"
    assert r["max_abs"] <= r["bar_max_abs"], f"{what}: max abs err {r['max_abs']:.4g} > {r['bar_max_abs']:.4g}{note} at {r['argmax']}"
    assert r["mean_abs"] <= r["bar_mean_abs"], f"{what}: mean abs err {r['mean_abs']:.4g} > {r['bar_mean_abs']:.4g}{note}"


def f16_floor(oracle, ops, inputs, name):
    """The binary16-storage evaluation of a graph, for `assert_conv_close(..., floor=...)`; evaluated only when needed."""
    return lambda: oracle.run_graph(ops, inputs, "f16")[name]


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
