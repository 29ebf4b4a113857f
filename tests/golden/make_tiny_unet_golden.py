#!/usr/bin/env python3
"""Writes tests/golden/tiny_unet_128.npz: input, weights and the fp32 result of the
tiny two-level U-Net (conv 3->16+ReLU; maxpool; conv 16->32+ReLU; nearest upsample x2;
concat with the 16-channel skip; conv 48->16+ReLU; conv 16->3), evaluated with
torch.nn.functional on the CPU in fp32 -- a library evaluation that shares no code
with the oracle or the HIP path.  Inputs and weights are binary16 values.

Run from the repository root:  python tests/golden/make_tiny_unet_golden.py
"""
import os
import sys

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    rng = np.random.default_rng(20240)
    H = W = 128

    def he(K, C):
        return (rng.standard_normal((K, C, 3, 3)) * np.sqrt(2.0 / (9 * C))).astype(np.float16)

    def bias(K):
        return (rng.standard_normal(K) * 0.01).astype(np.float16)

    x = rng.random((H, W, 3), dtype=np.float32).astype(np.float16)
    w = [he(16, 3), he(32, 16), he(16, 48), he(3, 16)]
    b = [bias(16), bias(32), bias(16), bias(3)]
    tw = [torch.from_numpy(a.astype(np.float32)) for a in w]
    tb = [torch.from_numpy(a.astype(np.float32)) for a in b]
    t = torch.from_numpy(x.astype(np.float32)).permute(2, 0, 1).unsqueeze(0)
    e0 = F.relu(F.conv2d(t, tw[0], tb[0], padding=1))
    p = F.max_pool2d(e0, 2)
    e1 = F.relu(F.conv2d(p, tw[1], tb[1], padding=1))
    u = F.interpolate(e1, scale_factor=2, mode="nearest")
    c = torch.cat([u, e0], 1)
    d0 = F.relu(F.conv2d(c, tw[2], tb[2], padding=1))
    y = F.conv2d(d0, tw[3], tb[3], padding=1)
    out = y.squeeze(0).permute(1, 2, 0).contiguous().numpy()
    np.savez_compressed(os.path.join(HERE, "tiny_unet_128.npz"), input=x, w0=w[0], w1=w[1], w2=w[2], w3=w[3],
                        b0=b[0], b1=b[1], b2=b[2], b3=b[3], output_fp32=out,
                        e0_fp32=e0.squeeze(0).permute(1, 2, 0).contiguous().numpy()[::8, ::8].copy())
    print("wrote tiny_unet_128.npz", out.shape, float(np.abs(out).max()))


if __name__ == "__main__":
    sys.exit(main())
