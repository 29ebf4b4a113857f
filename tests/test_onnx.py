"""ONNX import (host side): files written by torch.onnx.export are parsed, the graph they describe is the one the
exporting module computes (checked structurally here, numerically on the GPU in test_gpu_onnx.py), hand-built
protobuf messages pin single operators' semantics and error reporting, and damaged files never crash the parser.
Mirrors what the reference's compiler tests do for its importer (test/compiler, compile smoke tests)."""
import os
import struct

import numpy as np
import pytest

import denox_amd as dx

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


# ---------------------------------------------------------------- a minimal protobuf writer (onnx.proto field numbers)
def _varint(v):
    v &= (1 << 64) - 1
    out = bytearray()
    while True:
        b = v & 0x7F
        v >>= 7
        out.append(b | (0x80 if v else 0))
        if not v:
            return bytes(out)


def _field(num, wire, payload):
    return _varint((num << 3) | wire) + payload


def _len(num, payload):
    return _field(num, 2, _varint(len(payload)) + payload)


def _str(num, s):
    return _len(num, s.encode())


def _int(num, v):
    return _field(num, 0, _varint(v))


def tensor(name, arr):
    arr = np.asarray(arr)
    dt = {np.dtype("float32"): 1, np.dtype("int64"): 7, np.dtype("int32"): 6, np.dtype("float64"): 11}[arr.dtype]
    return b"".join(_int(1, d) for d in arr.shape) + _int(2, dt) + _str(8, name) + _len(9, arr.tobytes())


def attr_ints(name, vals):
    return _str(1, name) + b"".join(_int(8, v) for v in vals) + _int(20, 7)


def attr_int(name, v):
    return _str(1, name) + _int(3, v) + _int(20, 2)


def attr_str(name, s):
    return _str(1, name) + _len(4, s.encode()) + _int(20, 3)


def attr_tensor(name, arr):
    return _str(1, name) + _len(5, tensor("", arr)) + _int(20, 4)


def node(op, ins, outs, *attrs, name=""):
    return b"".join(_str(1, i) for i in ins) + b"".join(_str(2, o) for o in outs) + _str(3, name or op) + _str(4, op) + b"".join(_len(5, a) for a in attrs)


def value_info(name, dims, elem=1):
    shape = b"".join(_len(1, _str(2, d) if isinstance(d, str) else _int(1, d)) for d in dims)
    return _str(1, name) + _len(2, _len(1, _int(1, elem) + _len(2, shape)))


def model(nodes, inputs, outputs, inits=(), opset=17):
    g = b"".join(_len(1, n) for n in nodes) + _str(2, "g") + b"".join(_len(5, t) for t in inits) + \
        b"".join(_len(11, v) for v in inputs) + b"".join(_len(12, v) for v in outputs)
    return _int(1, 8) + _str(2, "test") + _len(7, g) + _len(8, _str(1, "") + _int(2, opset))


def dispatch_names(blob, **ext):
    return [d["name"] for d in dx.describe(blob, **ext)["dispatches"]]


# ---------------------------------------------------------------- files written by torch
def test_torch_exported_unet_imports_and_fuses():
    m = dx.Model.from_onnx(os.path.join(GOLD, "onnx_unet_dynamic.onnx"))
    assert [(t.name, t.channels) for t in m.inputs] == [("input", 3)] and [(t.name, t.channels) for t in m.outputs] == [("output", 3)]
    blob = dx.compile_model(m)
    # pad folds into the first conv, upsample + concat into the third, which runs in one dispatch with the last, and the two
    # crops (one Slice node per axis) fold into that
    assert dispatch_names(blob, H=33, W=47) == ["pad+conv3x3+relu", "maxpool", "conv3x3+relu", "concat+upsample+conv3x3+relu+conv3x3+slice"]
    assert dispatch_names(dx.compile_model(m, features=dict(conv_conv_fusion=False)), H=33, W=47) == ["pad+conv3x3+relu", "maxpool", "conv3x3+relu", "concat+upsample+conv3x3+relu", "conv3x3+slice"]
    d = dx.describe(blob, H=33, W=47)
    t = {x["name"]: x for x in d["tensors"] if x.get("name")}
    assert (t["input"]["height"], t["input"]["width"], t["output"]["height"], t["output"]["width"]) == (33, 47, 33, 47)
    # the padded extent is a function of the dynamic extents: 33 x 47 -> 48 x 48 in the first conv's push constants
    assert d["dispatches"][0]["push_constants"][:2] == [48, 48]
    d = dx.describe(blob, H=64, W=80)
    assert d["dispatches"][0]["push_constants"][:2] == [80, 64]


def test_torch_exported_static_model_imports():
    m = dx.Model.from_onnx(os.path.join(GOLD, "onnx_leaky_static.onnx"))
    assert [(t.name, t.channels) for t in m.inputs] == [("image", 8)]
    assert dispatch_names(dx.compile_model(m)) == ["conv3x3+leaky_relu+maxpool", "upsample+conv3x3"]
    with open(os.path.join(GOLD, "onnx_leaky_static.onnx"), "rb") as f:
        assert dispatch_names(dx.compile_model(dx.Model.from_onnx(f.read()))) == ["conv3x3+leaky_relu+maxpool", "upsample+conv3x3"]


# ---------------------------------------------------------------- hand-built graphs
W8 = np.zeros((8, 8, 3, 3), np.float32)


def conv_model(extra_nodes, out_name, out_dims, inits=(), opset=17, in_dims=(1, 8, "H", "W")):
    nodes = [node("Conv", ["x", "w"], ["c"], attr_ints("kernel_shape", [3, 3]), attr_ints("pads", [1, 1, 1, 1]))] + list(extra_nodes)
    return model(nodes, [value_info("x", in_dims)], [value_info(out_name, out_dims)], [tensor("w", W8)] + list(inits), opset)


def test_slice_with_negative_and_open_ends():
    # c[:, :, 2:-3, 1:]  ->  one Slice layer with ranges [1, W) x [2, H-3)
    nodes = [node("Slice", ["c", "st", "en", "ax"], ["y"])]
    inits = [tensor("st", np.array([2, 1], np.int64)), tensor("en", np.array([-3, np.iinfo(np.int64).max], np.int64)), tensor("ax", np.array([2, 3], np.int64))]
    blob = dx.compile_model(dx.Model.from_onnx(conv_model(nodes, "y", (1, 8, "h", "w"), inits)))
    d = dx.describe(blob, H=20, W=30)
    assert [x["name"] for x in d["dispatches"]] == ["conv3x3+slice"]
    out = [t for t in d["tensors"] if t.get("name") == "y"][0]
    assert (out["height"], out["width"]) == (15, 29)


def test_shape_arithmetic_drives_pad():
    # pads = [0, 0, 0, 0, 0, 0, (8 - H % 8) % 8, 3] built from Shape / Gather / Mod / Sub / Unsqueeze / Concat
    c = lambda name, arr: node("Constant", [], [name], attr_tensor("value", arr), name=name)
    nodes = [
        node("Shape", ["c"], ["shp"]), c("i2", np.array(2, np.int64)), node("Gather", ["shp", "i2"], ["h"], attr_int("axis", 0)),
        c("k8", np.array(8, np.int64)), node("Mod", ["h", "k8"], ["r"]), node("Sub", ["k8", "r"], ["d"]), node("Mod", ["d", "k8"], ["ph"]),
        c("ax0", np.array([0], np.int64)), node("Unsqueeze", ["ph", "ax0"], ["ph1"]),
        c("z6", np.zeros(6, np.int64)), c("three", np.array([3], np.int64)), node("Concat", ["z6", "ph1", "three"], ["pads"], attr_int("axis", 0)),
        node("Pad", ["c", "pads"], ["y"], attr_str("mode", "edge")),
    ]
    blob = dx.compile_model(dx.Model.from_onnx(conv_model(nodes, "y", (1, 8, "h", "w"))))
    for H, W, want in ((13, 10, (16, 13)), (16, 5, (16, 8)), (1, 1, (8, 4))):
        out = [t for t in dx.describe(blob, H=H, W=W)["tensors"] if t.get("name") == "y"][0]
        assert (out["height"], out["width"]) == want


def test_integer_mod_takes_the_sign_of_the_divisor():
    # ONNX Mod (fmod = 0) on constants: (-7) mod 3 = 2; used here as a crop offset
    c = lambda name, arr: node("Constant", [], [name], attr_tensor("value", arr), name=name)
    nodes = [c("a", np.array([-7], np.int64)), c("b", np.array([3], np.int64)), node("Mod", ["a", "b"], ["st"]),
             c("en", np.array([np.iinfo(np.int64).max], np.int64)), c("ax", np.array([3], np.int64)), node("Slice", ["c", "st", "en", "ax"], ["y"])]
    blob = dx.compile_model(dx.Model.from_onnx(conv_model(nodes, "y", (1, 8, "h", "w"))))
    out = [t for t in dx.describe(blob, H=9, W=12)["tensors"] if t.get("name") == "y"][0]
    assert out["width"] == 10


def test_clip_on_shape_arithmetic():
    # crop offset = Clip(W - 20, 0, 3): 0 for narrow images, 3 for wide ones, the symbolic value in between
    c = lambda name, arr: node("Constant", [], [name], attr_tensor("value", arr), name=name)
    nodes = [node("Shape", ["c"], ["shp"]), c("i3", np.array([3], np.int64)), node("Gather", ["shp", "i3"], ["w"], attr_int("axis", 0)),
             c("k20", np.array([20], np.int64)), node("Sub", ["w", "k20"], ["d"]),
             c("lo", np.array(0, np.int64)), c("hi", np.array(3, np.int64)), node("Clip", ["d", "lo", "hi"], ["st"]),
             c("en", np.array([np.iinfo(np.int64).max], np.int64)), c("ax", np.array([3], np.int64)), node("Slice", ["c", "st", "en", "ax"], ["y"])]
    blob = dx.compile_model(dx.Model.from_onnx(conv_model(nodes, "y", (1, 8, "h", "w"))))
    for W, want in ((12, 12), (21, 20), (22, 20), (40, 37)):
        out = [t for t in dx.describe(blob, H=9, W=W)["tensors"] if t.get("name") == "y"][0]
        assert out["width"] == want, W
    # only an upper bound (the lower one omitted with an empty name), on constants
    nodes = [c("a", np.array([7], np.int64)), c("hi", np.array(2, np.int64)), node("Clip", ["a", "", "hi"], ["st"]),
             c("en", np.array([np.iinfo(np.int64).max], np.int64)), c("ax", np.array([2], np.int64)), node("Slice", ["c", "st", "en", "ax"], ["y"])]
    blob = dx.compile_model(dx.Model.from_onnx(conv_model(nodes, "y", (1, 8, "h", "w"))))
    out = [t for t in dx.describe(blob, H=9, W=12)["tensors"] if t.get("name") == "y"][0]
    assert out["height"] == 7


@pytest.mark.parametrize("opset,scales_at", [(10, 1), (13, 2)])
def test_resize_scales_input_position_follows_the_opset(opset, scales_at):
    ins = ["c", "sc"] if scales_at == 1 else ["c", "", "sc"]
    attrs = [attr_str("mode", "nearest")] + ([attr_str("coordinate_transformation_mode", "asymmetric"), attr_str("nearest_mode", "floor")] if opset >= 11 else [])
    nodes = [node("Resize", ins, ["y"], *attrs)]
    blob = dx.compile_model(dx.Model.from_onnx(conv_model(nodes, "y", (1, 8, "h", "w"), [tensor("sc", np.array([1, 1, 2, 2], np.float32))], opset)))
    out = [t for t in dx.describe(blob, H=9, W=12)["tensors"] if t.get("name") == "y"][0]
    assert (out["height"], out["width"]) == (18, 24)


def test_one_by_one_and_five_by_five_convs_import():
    w1, w5 = np.zeros((4, 8, 1, 1), np.float32), np.zeros((8, 4, 5, 5), np.float32)
    nodes = [node("Conv", ["x", "w1"], ["a"], attr_ints("kernel_shape", [1, 1])),
             node("Conv", ["a", "w5"], ["y"], attr_ints("kernel_shape", [5, 5]), attr_ints("pads", [2, 2, 2, 2]))]
    onnx = model(nodes, [value_info("x", (1, 8, "H", "W"))], [value_info("y", (1, 8, "H", "W"))], [tensor("w1", w1), tensor("w5", w5)])
    assert dispatch_names(dx.compile_model(dx.Model.from_onnx(onnx)), H=9, W=9) == ["conv1x1", "conv5x5"]
    # a 5x5 filter without padding and with a stride: the extents follow (H - 5) // 2 + 1
    nodes[1] = node("Conv", ["a", "w5"], ["y"], attr_ints("kernel_shape", [5, 5]), attr_ints("strides", [2, 2]))
    onnx = model(nodes, [value_info("x", (1, 8, "H", "W"))], [value_info("y", (1, 8, "h", "w"))], [tensor("w1", w1), tensor("w5", w5)])
    d = dx.describe(dx.compile_model(dx.Model.from_onnx(onnx)), H=20, W=31)
    out = d["tensors"][d["outputs"][0]]
    assert (out["height"], out["width"], out["channels"]) == (8, 14, 8) and "SY=2" in d["dispatches"][1]["debug_info"]
    # a dilated filter has no kernel
    nodes[1] = node("Conv", ["a", "w5"], ["y"], attr_ints("kernel_shape", [5, 5]), attr_ints("dilations", [2, 2]))
    onnx = model(nodes, [value_info("x", (1, 8, "H", "W"))], [value_info("y", (1, 8, "h", "w"))], [tensor("w1", w1), tensor("w5", w5)])
    with pytest.raises(dx.DenoxHipError) as e:
        dx.compile_model(dx.Model.from_onnx(onnx))
    assert e.value.status == 5


def test_average_pool_imports_as_its_own_dispatch():
    """AveragePool (the reference imports it, frontend/onnx/details/ops/average_pool.cpp:9-156, and then finds no shader):
    a dispatch of its own -- the conv epilogue folds only the 2x2 maximum -- and the attributes the reference refuses
    are refused."""
    ap = lambda *extra: conv_model([node("Relu", ["c"], ["r"]), node("AveragePool", ["r"], ["y"], attr_ints("kernel_shape", [2, 2]), attr_ints("strides", [2, 2]), *extra, name="ap0")],
                                   "y", (1, 8, "h", "w"))
    blob = dx.compile_model(dx.Model.from_onnx(ap()))
    d = dx.describe(blob, H=10, W=21)
    assert [x["name"] for x in d["dispatches"]] == ["conv3x3+relu", "avgpool"] and "AVG=1" in d["dispatches"][1]["debug_info"]
    out = d["tensors"][d["outputs"][0]]
    assert (out["height"], out["width"], out["channels"]) == (5, 10, 8)
    for extra, word in [(attr_int("count_include_pad", 1), "count_include_pad"), (attr_int("ceil_mode", 1), "ceil_mode")]:
        with pytest.raises(dx.DenoxHipError) as e:
            dx.Model.from_onnx(ap(extra))
        assert e.value.status == 5 and word in str(e.value) and "ap0" in str(e.value)


def test_unsupported_and_malformed_models_are_reported():
    with pytest.raises(dx.DenoxHipError) as e:
        dx.Model.from_onnx(conv_model([node("Softmax", ["c"], ["y"], name="sm0")], "y", (1, 8, "h", "w")))
    assert e.value.status == 5 and "Softmax" in str(e.value) and "sm0" in str(e.value)
    # constant-mode Pad: zeros are a layer of their own, any other constant has no kernel
    pads = tensor("p", np.array([0, 0, 1, 2, 0, 0, 3, 4], np.int64))
    blob = dx.compile_model(dx.Model.from_onnx(conv_model([node("Pad", ["c", "p"], ["y"])], "y", (1, 8, "h", "w"), [pads])))
    d = dx.describe(blob, H=10, W=20)
    out = d["tensors"][d["outputs"][0]]
    assert (out["height"], out["width"]) == (14, 26) and "ZERO=1" in d["dispatches"][-1]["debug_info"]
    with pytest.raises(dx.DenoxHipError) as e:
        dx.Model.from_onnx(conv_model([node("Pad", ["c", "p", "v"], ["y"])], "y", (1, 8, "h", "w"), [pads, tensor("v", np.array(1.5, np.float32))]))
    assert e.value.status == 5 and "other than 0" in str(e.value)
    with pytest.raises(dx.DenoxHipError) as e:
        dx.Model.from_onnx(conv_model([node("Pad", ["c", "p"], ["y"], attr_str("mode", "reflect"))], "y", (1, 8, "h", "w"), [pads]))
    assert e.value.status == 5 and "mode" in str(e.value)
    with pytest.raises(dx.DenoxHipError) as e:  # batch of 2
        dx.Model.from_onnx(conv_model([], "c", (2, 8, "h", "w"), in_dims=(2, 8, "H", "W")))
    assert e.value.status == 5 and "batch" in str(e.value)
    with pytest.raises(dx.DenoxHipError) as e:  # channel mismatch
        dx.Model.from_onnx(conv_model([], "c", (1, 8, "h", "w"), in_dims=(1, 5, "H", "W")))
    assert e.value.status == 2 and "channels" in str(e.value)
    with pytest.raises(dx.DenoxHipError) as e:
        dx.Model.from_onnx(conv_model([node("Relu", ["nothing"], ["y"])], "y", (1, 8, "h", "w")))
    assert e.value.status == 2 and "nothing" in str(e.value)
    with pytest.raises(dx.DenoxHipError) as e:
        dx.Model.from_onnx(b"")
    assert e.value.status == 1
    with pytest.raises(dx.DenoxHipError) as e:
        dx.Model.from_onnx(b"\x08\x08")  # an ir_version and nothing else
    assert e.value.status == 2


def test_damaged_files_never_crash_the_parser():
    with open(os.path.join(GOLD, "onnx_leaky_static.onnx"), "rb") as f:
        data = f.read()
    rng = np.random.default_rng(5)
    outcomes = {"ok": 0, "error": 0}
    cases = [data[:n] for n in rng.integers(0, len(data), 150)]
    for _ in range(250):
        b = bytearray(data)
        for pos in rng.integers(0, len(b), rng.integers(1, 4)):
            b[pos] = rng.integers(0, 256)
        cases.append(bytes(b))
    for blob in cases:
        try:
            dx.Model.from_onnx(blob)
            outcomes["ok"] += 1
        except dx.DenoxHipError as e:
            assert e.status in (1, 2, 5), str(e)
            outcomes["error"] += 1
    assert outcomes["error"] > 100  # most truncations and many flips must be noticed
