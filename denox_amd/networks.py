"""The benchmark networks as builder programs, with seeded synthetic weights and inputs.

Topologies: the reference's OIDN-style U-Net (oidn_model.py:231-347: encoder
9->32->32 | 48 | 64 | 80 | 96->96, decoder (96+64)->112->112, (112+48)->96->96,
(96+32)->64->64, (64+9)->64->32->3, replicate-pad to a multiple of 16 and crop)
and a two-level miniature of it.  Weights are He-normal, biases N(0, 0.01),
all drawn from a numpy Generator seeded by the caller.
"""
from __future__ import annotations

import numpy as np

from .graph import Model


def _he(rng, K, C):
    return (rng.standard_normal((K, C, 3, 3)) * np.sqrt(2.0 / (9 * C))).astype(np.float16)


def _bias(rng, K):
    return (rng.standard_normal(K) * 0.01).astype(np.float16)


def tiny_unet(seed=0, channels=3):
    """conv 3->16+ReLU; pool; conv 16->32+ReLU; upsample; concat with the 16-ch skip; conv 48->16+ReLU; conv 16->3."""
    rng = np.random.default_rng(seed)
    m = Model()
    x = m.input("input", "W", "H", channels)
    e0 = m.relu(m.conv2d(x, _he(rng, 16, channels), _bias(rng, 16)))
    p = m.pool(e0)
    e1 = m.relu(m.conv2d(p, _he(rng, 32, 16), _bias(rng, 32)))
    u = m.upsample(e1)
    c = m.concat(u, e0)
    d0 = m.relu(m.conv2d(c, _he(rng, 16, 48), _bias(rng, 16)))
    out = m.conv2d(d0, _he(rng, channels, 16), _bias(rng, channels))
    m.output(out, "output")
    return m


def single_conv(seed=0, C=64, K=64):
    """conv3x3 C->K + bias + ReLU."""
    rng = np.random.default_rng(seed)
    m = Model()
    x = m.input("input", "W", "H", C)
    m.output(m.relu(m.conv2d(x, _he(rng, K, C), _bias(rng, K))), "output")
    return m


def oidn_unet(seed=0, ic=9, oc=3, width_mult=1, align=True):
    """OIDN-style U-Net; `align` wraps it in replicate-pad to a multiple of 16 and a crop back."""
    rng = np.random.default_rng(seed)
    k = width_mult
    ec1, ec2, ec3, ec4, ec5 = 32 * k, 48 * k, 64 * k, 80 * k, 96 * k
    dc4, dc3, dc2a, dc2b, dc1a, dc1b = 112 * k, 96 * k, 64 * k, 64 * k, 64 * k, 32 * k
    m = Model()
    inp = m.input("input", "W", "H", ic)
    x0 = m.pad_to_multiple(inp, 16) if align else inp

    def conv(t, K, relu=True):
        y = m.conv2d(t, _he(rng, K, t.channels), _bias(rng, K))
        return m.relu(y) if relu else y

    x = conv(x0, ec1)
    x = conv(x, ec1)
    x = pool1 = m.pool(x)
    x = conv(x, ec2)
    x = pool2 = m.pool(x)
    x = conv(x, ec3)
    x = pool3 = m.pool(x)
    x = conv(x, ec4)
    x = m.pool(x)
    x = conv(x, ec5)
    x = conv(x, ec5)
    x = m.concat(m.upsample(x), pool3)
    x = conv(x, dc4)
    x = conv(x, dc4)
    x = m.concat(m.upsample(x), pool2)
    x = conv(x, dc3)
    x = conv(x, dc3)
    x = m.concat(m.upsample(x), pool1)
    x = conv(x, dc2a)
    x = conv(x, dc2b)
    x = m.concat(m.upsample(x), x0)
    x = conv(x, dc1a)
    x = conv(x, dc1b)
    x = conv(x, oc, relu=False)
    if align:
        x = m.slice(x, 0, inp.width, 0, inp.height)
    m.output(x, "output")
    return m


def build(name: str, **kw):
    fn = {"tiny_unet": tiny_unet, "single_conv": single_conv, "oidn_unet": oidn_unet}[name]
    m = fn(**kw)
    return m, m.inputs


def synthetic_input(name: str, H: int, W: int, seed: int = 0, C: int | None = None) -> np.ndarray:
    """Seeded synthetic frames (float16, HWC).

    tiny_unet:   uniform [0, 1)
    single_conv: |N(0, 1)|
    oidn_unet:   9 channels = colour lognormal(0,1) clamped to [0,64], albedo uniform[0,1], unit normals
    """
    rng = np.random.default_rng(seed)
    if name == "tiny_unet":
        return rng.random((H, W, C or 3), dtype=np.float32).astype(np.float16)
    if name == "single_conv":
        return np.abs(rng.standard_normal((H, W, C or 64), dtype=np.float32)).astype(np.float16)
    if name == "oidn_unet":
        color = np.clip(rng.lognormal(0.0, 1.0, (H, W, 3)), 0.0, 64.0)
        albedo = rng.random((H, W, 3))
        n = rng.uniform(-1.0, 1.0, (H, W, 3))
        n /= np.maximum(np.linalg.norm(n, axis=2, keepdims=True), 1e-6)
        return np.concatenate([color, albedo, n], axis=2).astype(np.float16)
    raise KeyError(name)


# Compile features that keep every pool, upsample, concat, pad and slice a dispatch of its own (conv + activation stay
# fused): the schedule in which the stand-alone bandwidth kernels can be timed on a whole network.
UNFUSED_FEATURES = dict(conv_relu_fusion=True, concat_conv_fusion=False, upsample_fusion=False, pool_fusion=False, pad_fusion=False,
                        slice_fusion=False, implicit_concat=False, conv_conv_fusion=False)

# networks whose code objects __graft_entry__.build() compiles ahead of time
CACHE_WARM_CONFIGS = [
    ("tiny_unet", {}),
    ("single_conv", {}),
    ("oidn_unet", {}),
    ("oidn_unet", {"width_mult": 2}),
]
