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


def test_oidn_unet_exported_by_torch_at_test_time():
    """The 16-conv OIDN U-Net (the reference's oidn_model.py:206-330 architecture, `padding="same"` convs), wrapped
    in replicate-pad to a multiple of 16 and crop, exported with torch.onnx.export here and now, imported, and
    compared with the exporting module's own fp32 output."""
    torch = pytest.importorskip("torch")
    import io
    import warnings
    import torch.nn as nn
    import torch.nn.functional as F
    try:
        from torch.onnx._internal.torchscript_exporter import onnx_proto_utils
    except ImportError:
        pytest.skip("this torch has no TorchScript ONNX exporter")
    onnx_proto_utils._add_onnxscript_fn = lambda proto, custom_opsets: proto  # needs the onnx package only for onnxscript functions

    class UNet(nn.Module):
        def __init__(self, ic=9, oc=3):
            super().__init__()
            c = lambda i, o: nn.Conv2d(i, o, 3, padding="same")
            self.enc_conv0, self.enc_conv1, self.enc_conv2, self.enc_conv3, self.enc_conv4 = c(ic, 32), c(32, 32), c(32, 48), c(48, 64), c(64, 80)
            self.enc_conv5a, self.enc_conv5b = c(80, 96), c(96, 96)
            self.dec_conv4a, self.dec_conv4b, self.dec_conv3a, self.dec_conv3b = c(96 + 64, 112), c(112, 112), c(112 + 48, 96), c(96, 96)
            self.dec_conv2a, self.dec_conv2b, self.dec_conv1a, self.dec_conv1b, self.dec_conv0 = c(96 + 32, 64), c(64, 64), c(64 + ic, 64), c(64, 32), c(32, oc)

        def forward(self, inp):
            H, W = inp.shape[2], inp.shape[3]
            inp = F.pad(inp, (0, (16 - W % 16) % 16, 0, (16 - H % 16) % 16), mode="replicate")
            up = lambda t: F.interpolate(t, scale_factor=2, mode="nearest")
            x = F.relu(self.enc_conv0(inp))
            x = pool1 = F.max_pool2d(F.relu(self.enc_conv1(x)), 2, 2)
            x = pool2 = F.max_pool2d(F.relu(self.enc_conv2(x)), 2, 2)
            x = pool3 = F.max_pool2d(F.relu(self.enc_conv3(x)), 2, 2)
            x = F.max_pool2d(F.relu(self.enc_conv4(x)), 2, 2)
            x = F.relu(self.enc_conv5b(F.relu(self.enc_conv5a(x))))
            x = F.relu(self.dec_conv4b(F.relu(self.dec_conv4a(torch.cat((up(x), pool3), 1)))))
            x = F.relu(self.dec_conv3b(F.relu(self.dec_conv3a(torch.cat((up(x), pool2), 1)))))
            x = F.relu(self.dec_conv2b(F.relu(self.dec_conv2a(torch.cat((up(x), pool1), 1)))))
            x = F.relu(self.dec_conv1b(F.relu(self.dec_conv1a(torch.cat((up(x), inp), 1)))))
            return self.dec_conv0(x)[:, :, :H, :W]

    torch.manual_seed(3)
    net = UNet().eval()
    with torch.no_grad():
        for p in net.parameters():
            if p.dim() == 4:
                nn.init.kaiming_normal_(p, nonlinearity="relu")
            else:
                p.normal_(0, 0.01)
            p.copy_(p.half().float())
    rng = np.random.default_rng(8)
    x = rng.random((1, 9, 70, 100), dtype=np.float32).astype(np.float16)
    buf = io.BytesIO()
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        torch.onnx.export(net, (torch.from_numpy(x.astype(np.float32)),), buf, input_names=["input"], output_names=["output"],
                          dynamic_axes={"input": {2: "H", 3: "W"}, "output": {2: "H", 3: "W"}}, opset_version=17, dynamo=False)
    with torch.no_grad():
        want = net(torch.from_numpy(x.astype(np.float32))).numpy()[0]
    m = dx.Model.from_onnx(buf.getvalue())
    blob = dx.compile_model(m, input_layout=dx.Layout.CHW, output_layout=dx.Layout.CHW)
    rep = dx.last_compile_report()  # everything else folded into the 16 convs, the thin full-resolution pairs at either end joined
    assert rep.count("conv3x3_mfma") == 12 and rep.count("conv3x3_pair") == 2
    got = dx.Module.load(blob).instance(H=70, W=100).infer(x[0])[0]
    assert_conv_close(got, want, "onnx oidn unet")
