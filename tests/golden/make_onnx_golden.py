#!/usr/bin/env python3
"""Writes the ONNX fixtures of the import tests and what PyTorch computes for them:

  tests/golden/onnx_unet_dynamic.onnx   tiny U-Net, opset 17, dynamic H x W, replicate pad to a multiple of 16 and
                                        crop back (the Shape / Gather / Mod / Sub / ConstantOfShape / Reshape / Slice /
                                        Transpose / Cast chain PyTorch emits for that), MaxPool, Resize, Concat
  tests/golden/onnx_leaky_static.onnx   opset 11, static shape, Conv without bias, LeakyRelu, MaxPool, Resize, Conv
  tests/golden/onnx_golden.npz          per model: the input (binary16 values, NCHW) and torch's fp32 CPU output at
                                        one or two input sizes

The .onnx files are produced by torch.onnx.export (the TorchScript exporter's own serialiser), i.e. by a third party
to the importer under test.  The exporter's last step wants the `onnx` Python package only to splice in onnxscript
functions, of which these models have none; that step is replaced by the identity here.  Weights are rounded to
binary16 values before export, so that the fp32 evaluation differs from the fp16 pipeline only by the rounding of
activations.

Run from the repository root:  python tests/golden/make_onnx_golden.py
"""
import os
import warnings

import numpy as np
import torch
import torch.nn as nn
import torch.nn.functional as F
from torch.onnx._internal.torchscript_exporter import onnx_proto_utils

HERE = os.path.dirname(os.path.abspath(__file__))
onnx_proto_utils._add_onnxscript_fn = lambda proto, custom_opsets: proto


class UNetDynamic(nn.Module):
    def __init__(self):
        super().__init__()
        self.c1 = nn.Conv2d(3, 16, 3, padding=1)
        self.c2 = nn.Conv2d(16, 32, 3, padding=1)
        self.c3 = nn.Conv2d(48, 16, 3, padding=1)
        self.c4 = nn.Conv2d(16, 3, 3, padding=1)

    def forward(self, x):
        H, W = x.shape[2], x.shape[3]
        ph, pw = (16 - H % 16) % 16, (16 - W % 16) % 16
        x = F.pad(x, (0, pw, 0, ph), mode="replicate")
        a = F.relu(self.c1(x))
        b = F.relu(self.c2(F.max_pool2d(a, 2)))
        u = F.interpolate(b, scale_factor=2, mode="nearest")
        d = F.relu(self.c3(torch.cat([u, a], 1)))
        return self.c4(d)[:, :, :H, :W]


class LeakyStatic(nn.Module):
    def __init__(self):
        super().__init__()
        self.c1 = nn.Conv2d(8, 16, 3, padding=1, bias=False)
        self.c2 = nn.Conv2d(16, 8, 3, padding=1)

    def forward(self, x):
        a = F.leaky_relu(self.c1(x), 0.1)
        u = F.interpolate(F.max_pool2d(a, 2), scale_factor=2, mode="nearest")
        return self.c2(u)


def half_weights(m):
    with torch.no_grad():
        for p in m.parameters():
            p.copy_(p.half().float())
    return m.eval()


def main():
    torch.manual_seed(1234)
    rng = np.random.default_rng(77)
    out = {}
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        m = half_weights(UNetDynamic())
        x = torch.from_numpy(rng.random((1, 3, 40, 56), dtype=np.float32).astype(np.float16).astype(np.float32))
        torch.onnx.export(m, (x,), os.path.join(HERE, "onnx_unet_dynamic.onnx"), input_names=["input"], output_names=["output"],
                          dynamic_axes={"input": {2: "H", 3: "W"}, "output": {2: "H", 3: "W"}}, opset_version=17, dynamo=False)
        for tag, (h, w) in (("a", (40, 56)), ("b", (33, 47))):
            xi = torch.from_numpy(rng.random((1, 3, h, w), dtype=np.float32).astype(np.float16).astype(np.float32))
            with torch.no_grad():
                out[f"unet_dynamic_{tag}_x"] = xi.numpy().astype(np.float16)
                out[f"unet_dynamic_{tag}_y"] = m(xi).numpy()
        m = half_weights(LeakyStatic())
        x = torch.from_numpy(rng.standard_normal((1, 8, 24, 32)).astype(np.float16).astype(np.float32))
        torch.onnx.export(m, (x,), os.path.join(HERE, "onnx_leaky_static.onnx"), input_names=["image"], output_names=["result"],
                          opset_version=11, dynamo=False)
        with torch.no_grad():
            out["leaky_static_x"] = x.numpy().astype(np.float16)
            out["leaky_static_y"] = m(x).numpy()
    np.savez_compressed(os.path.join(HERE, "onnx_golden.npz"), **out)
    for f in ("onnx_unet_dynamic.onnx", "onnx_leaky_static.onnx", "onnx_golden.npz"):
        print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    main()
