"""Plain device-to-device copy of a known size through the library's slice kernel.

Used to calibrate profiler byte counters: `rocprofv3 --pmc FETCH_SIZE -- python3 -m denox_amd.calibrate`
reads N bytes and writes N bytes per launch (N is printed), so the counter value per dispatch of the
kernel `memory_slice_c64v8` divided by N is the counter's scale on this machine.
"""
import sys
import time

import numpy as np

import denox_amd as dx


def main(H=1088, W=1920, C=64, reps=10):
    m = dx.Model()
    x = m.input("input", "W", "H", C)
    m.output(m.slice(x, 0, x.width, 0, x.height), "output")  # full window: a plain copy
    inst = dx.Module.compile(m).instance(H=H, W=W)
    rng = np.random.default_rng(0)
    inst.infer(rng.standard_normal((H, W, C)).astype(np.float16))
    inst.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        inst.infer_device(None, None)
    inst.synchronize()
    dt = (time.perf_counter() - t0) / reps
    n = H * W * C * 2
    print(f"memory_slice_c{C}v8 copy: {n} bytes read + {n} bytes written per launch, {dt * 1e3:.4f} ms wall per launch "
          f"({2 * n / dt * 1e-9:.0f} GB/s incl. launch overhead)")


if __name__ == "__main__":
    sys.exit(main())
