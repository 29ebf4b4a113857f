"""Per-kernel bandwidth of the stand-alone data-movement kernels at benchmark extents.

`python -m denox_amd.bandwidth_report [H W [C ...]]` builds one-layer models (max pool, upsample, concat, ReLU, pad, slice,
layout conversion), times each dispatch with hipEvents (Instance.bench) and prints achieved GB/s against the
8 TB/s HBM peak, using the byte counts the dispatches carry (reads + writes of the tensors as stored).
"""
import sys

import numpy as np

import denox_amd as dx

HBM_PEAK_GBPS = 8000.0


def cases(C):
    def pool(m, x): return m.pool(x)
    def up(m, x): return m.upsample(x)
    def relu(m, x): return m.relu(x)
    def pad(m, x): return m.pad(x, 0, 0, 0, 8)
    def crop(m, x): return m.slice(x, 0, x.width, 0, x.height - 8)
    def cat(m, x): return m.concat(x, m.input("other", "W", "H", C))
    return [("maxpool", pool, 1), ("upsample", up, 2), ("relu", relu, 1), ("pad", pad, 1), ("slice", crop, 1), ("concat", cat, 1)]


def main(H=1088, W=1920, channels=(64, 32, 8, 9, 3)):
    rng = np.random.default_rng(0)
    print(f"{'kernel':<28}{'C':>4}{'extent':>12}{'ms':>9}{'GB/s':>8}{'of HBM peak':>13}")
    no_fusion = dict(conv_relu_fusion=False, concat_conv_fusion=False, upsample_fusion=False, pool_fusion=False, pad_fusion=False, slice_fusion=False)
    for C in channels:
        for name, fn, shrink in cases(C):
            h, w = H // shrink, W // shrink
            m = dx.Model()
            m.output(fn(m, m.input("input", "W", "H", C)))
            inst = dx.Module.compile(m, features=no_fusion).instance(H=h, W=w)
            inst.infer(*[rng.standard_normal((h, w, C)).astype(np.float16) for _ in range(inst.input_count)])
            reps = 5
            acc = {}
            for _ in range(reps):
                for t in inst.bench(warmup=3):
                    a = acc.setdefault(t["name"], [0.0, t["memory_reads"] + t["memory_writes"]])
                    a[0] += t["latency_ms"] / reps
            for k, (ms, nbytes) in acc.items():
                gbps = nbytes / ms * 1e-6
                print(f"{k:<28}{C:>4}{f'{w}x{h}':>12}{ms:>9.4f}{gbps:>8.0f}{gbps / HBM_PEAK_GBPS:>12.0%}")
    for C, src, dst in ((9, dx.Layout.CHW, dx.Layout.HWC), (3, dx.Layout.HWC, dx.Layout.CHW), (64, dx.Layout.CHWC8, dx.Layout.HWC)):
        m = dx.Model()
        m.output(m.relu(m.input("input", "W", "H", C)))
        inst = dx.Module.compile(m, input_layout=src, output_layout=dst).instance(H=H, W=W)
        inst.infer(rng.standard_normal(H * W * C).astype(np.float16))
        for t in inst.bench(warmup=3):
            if t["name"] == "relayout":
                gbps = (t["memory_reads"] + t["memory_writes"]) / t["latency_ms"] * 1e-6
                print(f"{'relayout ' + t['input'] + '->' + t['output']:<28}{C:>4}{f'{W}x{H}':>12}{t['latency_ms']:>9.4f}{gbps:>8.0f}{gbps / HBM_PEAK_GBPS:>12.0%}")


if __name__ == "__main__":
    args = [int(a) for a in sys.argv[1:]]
    main(*args[:2], **({"channels": tuple(args[2:])} if len(args) > 2 else {}))
