"""The allocation-free entry point, denox_hip_instance_infer_device_static, against denox_hip_instance_infer_device.

Both run the same dispatches with the same kernels; the static variant keeps the intermediate tensors in the library's
file-scope device array and launches without a graph.  Data movement and convolutions alike must therefore agree bit
for bit.  Two calls in a row share the array, the second with a smaller image (its tensors cover only the front of what
the first call left there)."""
import numpy as np
import pytest

import denox_amd as dx
from denox_amd import networks
from util import assert_bits_equal

pytestmark = pytest.mark.gpu


def _run_both(torch, inst, x, H, W):
    d_in = torch.from_numpy(x).cuda()
    ref = torch.full((H, W, 3), float("nan"), dtype=torch.float16, device="cuda")
    got = torch.full((H, W, 3), float("nan"), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    inst.infer_device([d_in.data_ptr()], [ref.data_ptr()])
    inst.synchronize()
    inst.infer_device_static([d_in.data_ptr()], [got.data_ptr()])
    inst.synchronize()
    return got.cpu().numpy(), ref.cpu().numpy()


def test_static_scratch_entry_point_matches_infer_device():
    torch = pytest.importorskip("torch")
    m, _ = networks.build("oidn_unet", seed=21)
    mod = dx.Module.compile(m)
    first = None
    for H, W in [(96, 160), (40, 56)]:  # the second, smaller image reuses the array the first call filled
        x = networks.synthetic_input("oidn_unet", H, W, seed=H)
        inst = mod.instance(H=H, W=W)
        got, ref = _run_both(torch, inst, x, H, W)
        assert np.isfinite(ref).all()
        assert_bits_equal(got, ref, f"static scratch {H}x{W}")
        if first is None:
            first = (inst, x, H, W, ref)
    # back to the larger image: whatever the smaller call left in the array does not reach the result
    inst, x, H, W, ref = first
    got, _ = _run_both(torch, inst, x, H, W)
    assert_bits_equal(got, ref, "static scratch, larger image again")
    # the instance's own interface tensors (null pointer arrays) work as in infer_device
    want = inst.infer(x)[0]
    inst.infer_device_static(None, None)
    inst.synchronize()
    out = torch.empty((H, W, 3), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    inst.infer_device_static(None, [out.data_ptr()])  # the input the blocking call above uploaded, the caller's output
    inst.synchronize()
    assert_bits_equal(out.cpu().numpy(), want, "static scratch, own input tensor")


def test_static_scratch_entry_point_refuses_what_does_not_fit():
    m, _ = networks.build("oidn_unet", seed=21)
    inst = dx.Module.compile(m).instance(H=1080, W=1920)  # ~0.5 GB of intermediate tensors
    with pytest.raises(dx.DenoxHipError) as e:
        inst.infer_device_static(None, None)
    assert "static scratch" in str(e.value)


def test_static_scratch_is_not_shared_by_calls_that_overlap():
    """Two contexts of one GPU launch on two streams and share the one array.  While calls made through the first are still
    running, a call through the second is refused (INVALID_ARGUMENT) instead of overwriting their tensors; once the first
    context has been synchronized the second runs and gives the bits of its graph path."""
    torch = pytest.importorskip("torch")
    m, _ = networks.build("oidn_unet", seed=21)
    blob = dx.compile_model(m)
    H, W = 256, 448  # about 30 MiB of intermediate tensors: a call lasts a few hundred microseconds
    a = dx.Module.load(blob, dx.Context(0)).instance(H=H, W=W)
    b = dx.Module.load(blob, dx.Context(0)).instance(H=H, W=W)
    x = networks.synthetic_input("oidn_unet", H, W, seed=3)
    want = b.infer(x)[0]
    a.infer(x)
    d_out = torch.full((H, W, 3), float("nan"), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    for _ in range(40):  # milliseconds of queued work on the first context's stream
        a.infer_device_static(None, None)
    with pytest.raises(dx.DenoxHipError) as e:
        b.infer_device_static(None, [d_out.data_ptr()])
    assert e.value.status == 1 and "another context" in str(e.value)
    a.synchronize()
    b.infer_device_static(None, [d_out.data_ptr()])
    b.synchronize()
    assert_bits_equal(d_out.cpu().numpy(), want, "second context after the first has finished")
    # and back: the first context may take the array again once the second's call is done
    a.infer_device_static(None, None)
    a.synchronize()
