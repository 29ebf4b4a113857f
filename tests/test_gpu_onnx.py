"""ONNX files written by torch.onnx.export, imported, compiled and run on the GPU, against what torch itself computed
for them in fp32 on the CPU (tests/golden/onnx_golden.npz, written by tests/golden/make_onnx_golden.py).  The
reference checks its ONNX path the same way, against torch at run time (test/system)."""
import os

import numpy as np
import pytest

import denox_amd as dx
from util import assert_conv_close

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.fixture(scope="module")
def gold():
    return np.load(os.path.join(GOLD, "onnx_golden.npz"))


@pytest.mark.parametrize("layout", ["CHW", "HWC"])
def test_dynamic_unet_matches_torch_at_two_sizes(gold, layout):
    m = dx.Model.from_onnx(os.path.join(GOLD, "onnx_unet_dynamic.onnx"))
    lay = dx.Layout[layout]
    mod = dx.Module.load(dx.compile_model(m, input_layout=lay, output_layout=lay))
    for tag in ("a", "b"):  # 40 x 56 (the export size) and 33 x 47 (pads to 48 x 48)
        x, want = gold[f"unet_dynamic_{tag}_x"][0], gold[f"unet_dynamic_{tag}_y"][0]
        H, W = x.shape[1:]
        feed = x if layout == "CHW" else np.ascontiguousarray(x.transpose(1, 2, 0))
        got = mod.instance(H=H, W=W).infer(feed)[0]
        got = got if layout == "CHW" else got.transpose(2, 0, 1)
        assert got.shape == want.shape
        assert_conv_close(got, want, f"onnx unet {tag} {layout}")


def test_static_leaky_model_matches_torch(gold):
    m = dx.Model.from_onnx(os.path.join(GOLD, "onnx_leaky_static.onnx"))
    mod = dx.Module.load(dx.compile_model(m, input_layout=dx.Layout.CHW, output_layout=dx.Layout.CHW))
    got = mod.instance().infer(gold["leaky_static_x"][0])[0]
    assert_conv_close(got, gold["leaky_static_y"][0], "onnx leaky static")
