"""Filter and bias parameter blobs of compiled models: the packing is a permutation of the ONNX-order weights plus zero fill.

The reference defines its packed filter layouts by index formulas (common/src/denox/memory/tensor/FilterLayout.hpp:49-116,
BiasLayout.hpp:30-45) and converts KCRS weights into them when a dispatch is built (FilterTensor.cpp:19-29).  The kernels
here have layouts of their own -- [channel tile][reduction chunk][tap][weight row][channel], the rows of a tile permuted so
that a lane of the matrix instruction ends up with consecutive output channels -- and what has to hold is the same: every
weight W[k][c][r][s] appears exactly once, at the position the layout assigns to it, everything else is zero, and the
bias is the bias followed by zeros.  Checked on the bytes of compiled models (read with the FlatBuffers decoder of
test_flatbuf.py), with the inverse of the layout restated here from its description, for both matrix shapes, streamed
and resident weights, paired and unpaired 16-row blocks, and the two-convolution kernel's three parameter forms."""
import re

import numpy as np
import pytest

import denox_amd as dx
from test_flatbuf import _FB
from util import he_weights


def row_channel(mf, kt, row):
    """Output channel (within a tile of kt channels) that weight row `row` computes."""
    if mf == 32:  # 32x32x16: a lane ends up with 16 consecutive channels of a 32-block
        rho = row % 32
        return row - rho + 16 * ((rho >> 2) & 1) + 4 * (rho >> 3) + (rho & 3)
    kb, rho = divmod(row, 16)  # 16x16x32: blocks are paired so that a lane ends up with 8 consecutive channels
    paired = 2 * (kb // 2) + 1 < kt // 16
    return 32 * (kb // 2) + 8 * (rho // 4) + 4 * (kb % 2) + rho % 4 if paired else 16 * kb + rho


def parameters(blob, dispatch=0, **extents):
    """(defines of the dispatch, [parameter blobs as uint16 arrays in binding order])."""
    d = dx.describe(blob, **extents)
    fb = _FB(blob)
    data = {}
    for i in fb.tables(fb.root(), 4):
        pos, n = fb.vector(i, 1)
        data[fb.scalar(i, 0, "I")] = np.frombuffer(blob, np.uint16, n // 2, pos)
    disp = d["dispatches"][dispatch]
    defines = dict(kv.split("=", 1) for kv in disp["debug_info"].split(" | ")[-1].split())
    return defines, [data[b["tensor"]] for b in disp["bindings"] if d["tensors"][b["tensor"]]["param"]]


def check_filter(packed, w, mf, kt, ck, resident):
    K, C, R, S = w.shape
    kstep = 16 if mf == 32 else 32
    cpad, koutp = -(-C // kstep) * kstep, -(-K // mf) * mf
    chunk = cpad if resident else ck
    assert packed.size == koutp * R * S * cpad
    wi = w.view(np.uint16)
    seen = np.zeros(w.shape, np.int32)
    pos = 0
    for t in range(koutp // kt):
        for c0 in range(0, cpad, chunk):
            n = min(chunk, cpad - c0)
            block = packed[pos:pos + R * S * kt * n].reshape(R * S, kt, n)
            pos += block.size
            for row in range(kt):
                k = t * kt + row_channel(mf, kt, row)
                for tap in range(R * S):
                    for e in range(n):
                        c = c0 + e
                        if k < K and c < C:
                            assert block[tap, row, e] == wi[k, c, tap // S, tap % S], (t, c0, tap, row, e)
                            seen[k, c, tap // S, tap % S] += 1
                        else:
                            assert block[tap, row, e] == 0, "padding must be zero"
    assert pos == packed.size and (seen == 1).all()


@pytest.mark.parametrize("config,C,K", [("w4r2k16", 24, 40), ("w4r2k32", 73, 64), ("p8r2k16", 9, 32), ("s8r2k16", 73, 64), ("m4r2k32x2", 48, 48), ("m4r2k32x1", 32, 3),
                                        ("q8r2k32x2", 40, 80), ("m4r2kfx1", 64, 112), ("w4r1kfn", 80, 96)])
def test_filter_and_bias_blobs_are_a_permutation_plus_zeros(config, C, K):
    rng = np.random.default_rng(C + K)
    w = he_weights(rng, K, C)
    w[w == 0] = np.float16(0.5)  # every weight distinguishable from padding
    b = (rng.standard_normal(K) + 3).astype(np.float16)
    m = dx.Model()
    m.output(m.relu(m.conv2d(m.input("input", "W", "H", C), w, b)))
    blob = dx.compile_model(m, conv_config=config)
    assert config in dx.last_compile_report()
    defines, (filt, bias) = parameters(blob, H=64, W=64)
    mf, kt, ck = int(defines.get("MF", 32)), int(defines["KT"]), int(defines["CK"])
    check_filter(filt, w, mf, kt, ck, resident="SLOTS" in defines)
    koutp = -(-K // mf) * mf
    assert bias.size == koutp and (bias[:K] == b.view(np.uint16)).all() and (bias[K:] == 0).all()


@pytest.mark.parametrize("K2", [32, 3])
def test_conv_pair_parameter_blobs(K2):
    """conv3x3_pair.hip: both filters as one resident 32-row tile; a second convolution with at most 5 output channels
    keeps [filter row r][32 rows][32 channels] with row (s, k) = W[k][:][r][s]."""
    rng = np.random.default_rng(K2)
    C, K1 = 24, 20
    w1, w2 = he_weights(rng, K1, C), he_weights(rng, K2, K1)
    w1[w1 == 0] = w2[w2 == 0] = np.float16(0.5)
    b1, b2 = (rng.standard_normal(K1) + 3).astype(np.float16), (rng.standard_normal(K2) + 3).astype(np.float16)
    m = dx.Model()
    m.output(m.conv2d(m.relu(m.conv2d(m.input("input", "W", "H", C), w1, b1)), w2, b2))
    blob = dx.compile_model(m, conv_config="x8r2k16")
    defines, (f1, bias1, f2, bias2) = parameters(blob, H=64, W=64)
    assert re.match(r"convpair_", defines["KERNEL_NAME"])
    check_filter(f1, w1, 32, 32, 32, resident=True)
    for bias, b in ((bias1, b1), (bias2, b2)):
        assert bias.size == 32 and (bias[:b.size] == b.view(np.uint16)).all() and (bias[b.size:] == 0).all()
    if K2 > 5:
        assert "TAPM" not in defines
        padded = np.zeros((K2, 32, 3, 3), np.float16)  # the second convolution reduces over the first one's 32 padded channels
        padded[:, :K1] = w2
        packed = f2.reshape(9, 32, 32)
        for row in range(32):
            k = row_channel(32, 32, row)
            want = padded.view(np.uint16)[k].transpose(1, 2, 0).reshape(9, 32) if k < K2 else np.zeros((9, 32), np.uint16)
            assert (packed[:, row, :] == want).all()
    else:
        assert defines["TAPM"] == "1" and f2.size == 3 * 32 * 32
        packed = f2.reshape(3, 32, 32)
        seen = np.zeros(w2.shape, np.int32)
        for row in range(32):
            lam = row_channel(32, 32, row)
            for r in range(3):
                if lam < 3 * K2:
                    s, k = divmod(lam, K2)
                    assert (packed[r, row, :K1] == w2.view(np.uint16)[k, :, r, s]).all() and (packed[r, row, K1:] == 0).all()
                    seen[k, :, r, s] += 1
                else:
                    assert (packed[r, row] == 0).all()
        assert (seen == 1).all()
