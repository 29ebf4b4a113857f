"""The command line (python -m denox_amd), verb by verb as README.md:112-199 of the reference walks through them:
populate -> bench -> compile --database -> infer.  Host-side verbs run here; bench and infer need the GPU."""
import os

import numpy as np
import pytest

import denox_amd as dx
from denox_amd.__main__ import main

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
ONNX = os.path.join(GOLD, "onnx_unet_dynamic.onnx")


def test_populate_compile_dumpcsv(tmp_path, capsys):
    db, out = str(tmp_path / "gpu.db"), str(tmp_path / "net.dnx")
    assert main(["populate", db, ONNX, "--assume", "H=40", "W=56", "--format", "input=chw", "output=chw"]) == 0
    assert "new dispatches" in capsys.readouterr().out
    assert main(["populate", db, ONNX, "--assume", "H=40 W=56", "--format", "input=chw output=chw"]) == 0
    assert capsys.readouterr().out.startswith("0 new dispatches")  # same candidates: nothing to add
    assert main(["dumpcsv", db]) == 0
    csv = capsys.readouterr().out.splitlines()
    assert csv[0].startswith("operation,shader,config") and len(csv) > 100
    assert main(["compile", ONNX, "-o", out, "-db", db, "--assume", "H=40", "W=56", "--format", "input=chw", "output=chw"]) == 0
    assert "5 dispatches" not in capsys.readouterr().out  # 5 layers + 2 relayouts for the CHW interface
    with open(out, "rb") as f:
        d = dx.describe(f.read(), H=40, W=56)
    assert [x["name"] for x in d["dispatches"]] == ["relayout", "pad+conv3x3+relu", "maxpool", "conv3x3+relu", "concat+upsample+conv3x3+relu+conv3x3+slice", "relayout"]
    tin = d["tensors"][d["inputs"][0]]
    assert (tin["width_name"], tin["height_name"], tin["format"]) == ("W", "H", 2)
    assert main(["compile", ONNX, "-o", out, "--no-fusion"]) == 0
    with open(out, "rb") as f:
        assert len(dx.describe(f.read())["dispatches"]) > 7


def test_errors_and_version(tmp_path, capsys):
    assert main(["-V"]) == 0 and "denox-hip" in capsys.readouterr().out
    assert main(["compile", __file__, "-o", str(tmp_path / "x.dnx")]) == 2
    assert "ONNX import" in capsys.readouterr().err
    with pytest.raises(SystemExit):
        main(["compile", ONNX, "-o", str(tmp_path / "x.dnx"), "--format", "nosuchtensor=hwc"])
    assert main(["info"]) == 0 and "gfx950" in capsys.readouterr().out


@pytest.mark.gpu
def test_bench_and_infer(tmp_path, capsys):
    gold = np.load(os.path.join(GOLD, "onnx_golden.npz"))
    db, out = str(tmp_path / "gpu.db"), str(tmp_path / "net.dnx")
    assert main(["populate", db, ONNX, "--assume", "H=40", "W=56"]) == 0
    assert main(["bench", db, "--samples", "3", "--relative-error", "0.5"]) == 0
    assert "benchmarked" in capsys.readouterr().out
    assert main(["compile", ONNX, "-o", out, "-db", db, "--assume", "H=40", "W=56"]) == 0
    # npy in the model's HWC interface layout
    x = np.ascontiguousarray(gold["unet_dynamic_b_x"][0].transpose(1, 2, 0))
    np.save(tmp_path / "in.npy", x)
    assert main(["infer", out, "-i", str(tmp_path / "in.npy"), "-o", str(tmp_path / "out.npy")]) == 0
    got = np.load(tmp_path / "out.npy")
    want = gold["unet_dynamic_b_y"][0].transpose(1, 2, 0)
    assert got.shape == want.shape and np.abs(got.astype(np.float32) - want).max() <= 2e-2
    # png: 8-bit in, 8-bit out, the same numbers as the library gives for the decoded image
    Image = pytest.importorskip("PIL.Image")
    rgb = (np.random.default_rng(0).random((33, 47, 3)) * 255).astype(np.uint8)
    Image.fromarray(rgb).save(tmp_path / "in.png")
    assert main(["infer", out, "-i", str(tmp_path / "in.png"), "-o", str(tmp_path / "out.png")]) == 0
    with open(out, "rb") as f:
        y = dx.Module.load(f.read()).instance(H=33, W=47).infer((rgb.astype(np.float32) / 255).astype(np.float16))[0]
    want8 = (np.clip(np.nan_to_num(y.astype(np.float32)), 0, 1) * 255 + 0.5).astype(np.uint8)
    assert np.array_equal(np.asarray(Image.open(tmp_path / "out.png")), want8)
    assert main(["bench", out, "--spec", "H=40", "W=56"]) == 0
    assert "total:" in capsys.readouterr().out
