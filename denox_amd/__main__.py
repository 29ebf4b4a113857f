"""Command line over the C ABI: ``python -m denox_amd <command>``.

The commands and their arguments follow the reference's ``denox`` tool
(cli/src/denox/cli/main.cpp:16-42, help.cpp:4-178, and the workflow of README.md:112-199):

    populate DATABASE ONNX [--assume H=1080 W=1920] [--format input=hwc output=hwc]
    bench    DATABASE|MODEL [--samples N] [--relative-error E] [--spec H=1080 W=1920]
    compile  ONNX -o MODEL [-db DATABASE] [--assume ...] [--format ...] [--no-fusion]
    infer    MODEL -i IMAGE -o IMAGE          (png or npy; the image's size sets the dynamic extents)
    dumpcsv  DATABASE
    info                                       (the device limits the kernels are configured with)

Options of the reference that select Vulkan features (--target-env, --fcoopmat, SPIR-V options, image storage) have
no meaning here and are not accepted.  Nothing is computed in Python: every command is a sequence of C-ABI calls.
"""
from __future__ import annotations

import argparse
import sys
import time

import numpy as np

from . import Db, Layout, Model, Module, _capi, compile_model, describe, device_info, last_compile_report, report

_FORMATS = {"hwc": Layout.HWC, "chw": Layout.CHW, "chwc8": Layout.CHWC8}


def _pairs(items, what):
    out = {}
    for it in items or []:
        for tok in it.split():
            if "=" not in tok:
                raise SystemExit(f"denox: {what} expects NAME=VALUE, got '{tok}'")
            k, v = tok.split("=", 1)
            out[k] = v
    return out


def _assume(args):
    return {k: int(v) for k, v in _pairs(args.assume, "--assume").items()}


def _layouts(args, model):
    fm = _pairs(args.format, "--format")
    names_in, names_out = [t.name for t in model.inputs], [t.name for t in model.outputs]
    lay_in = lay_out = Layout.Undefined
    for name, f in fm.items():
        if f.lower() not in _FORMATS:
            raise SystemExit(f"denox: unknown format '{f}' (hwc | chw | chwc8)")
        if name in names_in:
            lay_in = _FORMATS[f.lower()]
        elif name in names_out:
            lay_out = _FORMATS[f.lower()]
        else:
            raise SystemExit(f"denox: --format names '{name}', which is neither an input ({names_in}) nor an output ({names_out})")
    return lay_in, lay_out


def _features(args):
    if getattr(args, "no_fusion", False):
        return {k: False for k in ("conv_relu_fusion", "concat_conv_fusion", "upsample_fusion", "pool_fusion", "pad_fusion", "slice_fusion", "implicit_concat")}
    return {}


def _read_image(path):
    if path.endswith(".npy"):
        return np.load(path)
    from PIL import Image
    img = np.asarray(Image.open(path))
    if img.ndim == 2:
        img = img[:, :, None]
    scale = 65535.0 if img.dtype == np.uint16 else 255.0
    return (img.astype(np.float32) / scale).astype(np.float16)  # as the reference's PngInputStream: [0, 1] binary16, HWC


def _write_image(path, arr):
    if path.endswith(".npy"):
        np.save(path, arr)
        return
    from PIL import Image
    a = np.clip(np.nan_to_num(arr.astype(np.float32)), 0.0, 1.0)
    a = (a * 255.0 + 0.5).astype(np.uint8)
    if a.shape[2] == 1:
        a = a[:, :, 0]
    elif a.shape[2] not in (3, 4):
        raise SystemExit(f"denox: a png holds 1, 3 or 4 channels, the output has {a.shape[2]} (write .npy instead)")
    Image.fromarray(a).save(path)


def cmd_populate(args):
    model = Model.from_onnx(args.onnx)
    lay_in, lay_out = _layouts(args, model)
    db = Db(args.database)
    n = db.populate(model, assume=_assume(args), input_layout=lay_in, output_layout=lay_out, features=_features(args))
    db.writeback()
    print(f"{n} new dispatches, {len(db)} in {args.database}")


def cmd_bench(args):
    with open(args.target, "rb") as f:
        head = f.read(8)
    if head[4:8] == b"dnxx":  # a compiled model (file identifier of dnx.fbs): per-dispatch report (Instance::bench().report() of the reference)
        with open(args.target, "rb") as f:
            mod = Module.load(f.read())
        spec = {k: int(v) for k, v in _pairs(args.spec, "--spec").items()}
        print(report(mod.instance(**spec).bench(warmup=3)))
        return
    db = Db(args.target)
    t0 = time.perf_counter()
    r = db.bench(min_samples=args.samples, max_relative_error=args.relative_error, save_progress=True)
    db.writeback()
    print(f"benchmarked {r['benchmarked']} dispatches ({r['converged']} converged, {r['skipped']} skipped, {r['failed']} failed) in {time.perf_counter() - t0:.1f} s")


def cmd_compile(args):
    model = Model.from_onnx(args.onnx)
    lay_in, lay_out = _layouts(args, model)
    db = Db(args.database) if args.database else None
    blob = compile_model(model, assume=_assume(args), db=db, input_layout=lay_in, output_layout=lay_out, features=_features(args))
    with open(args.output, "wb") as f:
        f.write(blob)
    if args.verbose:
        print(last_compile_report(), file=sys.stderr)
    d = describe(blob)
    print(f"{args.output}: {len(d['dispatches'])} dispatches, {d['binaries']} kernels, {len(blob)} bytes")


def cmd_infer(args):
    with open(args.model, "rb") as f:
        blob = f.read()
    d = describe(blob)
    tin = d["tensors"][d["inputs"][0]]
    x = _read_image(args.input)
    fmt = tin["format"]  # 1 HWC, 2 CHW, 3 CHWC8 (dnx TensorFormat)
    if fmt == 2:
        x = np.ascontiguousarray(x.transpose(2, 0, 1)) if x.ndim == 3 and x.shape[2] == tin["channels"] else x
        h, w, c = x.shape[1], x.shape[2], x.shape[0]
    else:
        h, w, c = x.shape[0], x.shape[1], x.shape[2]
    if c != tin["channels"]:
        raise SystemExit(f"denox: input has invalid channel count. Expected {tin['channels']}, got {c}")
    spec = {}
    for key, got in (("width", w), ("height", h)):
        if key + "_name" in tin:
            spec[tin[key + "_name"]] = got
        elif tin[key] != got:
            raise SystemExit(f"denox: input has invalid {key}. Expected {tin[key]}, got {got}")
    t0 = time.perf_counter()
    mod = Module.load(blob)
    y = mod.instance(**spec).infer(np.ascontiguousarray(x, np.float16))[0]
    print(f"denox-latency: {(time.perf_counter() - t0) * 1e3:.3f}ms", file=sys.stderr)
    tout = d["tensors"][d["outputs"][0]]
    if tout["format"] == 2:
        y = np.ascontiguousarray(y.transpose(1, 2, 0))
    _write_image(args.output, y)


def cmd_dumpcsv(args):
    sys.stdout.write(Db(args.database).dump_csv())


def cmd_info(args):
    for k, v in device_info(args.device).items():
        print(f"{k}: {v}")


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="denox", description="denox on MI355X: compile ONNX models into dispatch lists and run them")
    ap.add_argument("-V", "--version", action="store_true")
    sub = ap.add_subparsers(dest="command")

    def common(p):
        p.add_argument("--assume", nargs="*", action="extend", help="assumed values of named extents, e.g. H=1080 W=1920")
        p.add_argument("--format", nargs="*", action="extend", help="interface layout of a tensor, e.g. input=chw output=chw")
        p.add_argument("--no-fusion", action="store_true", help="one dispatch per layer (debugging)")

    p = sub.add_parser("populate", help="populate a timing database with every candidate dispatch of an ONNX model")
    p.add_argument("database"); p.add_argument("onnx"); common(p); p.set_defaults(fn=cmd_populate)
    p = sub.add_parser("bench", help="time the dispatches of a database, or of a compiled model, on the GPU")
    p.add_argument("target"); p.add_argument("--samples", type=int, default=10); p.add_argument("--relative-error", type=float, default=0.05)
    p.add_argument("--spec", nargs="*", action="extend", help="values of the named extents of a compiled model, e.g. H=1080 W=1920")
    p.set_defaults(fn=cmd_bench)
    p = sub.add_parser("compile", help="compile an ONNX model into a dispatch list")
    p.add_argument("onnx"); p.add_argument("-o", "--output", required=True); p.add_argument("-db", "--database"); p.add_argument("-v", "--verbose", action="store_true")
    common(p); p.set_defaults(fn=cmd_compile)
    p = sub.add_parser("infer", help="run a compiled model on an image")
    p.add_argument("model"); p.add_argument("-i", "--input", required=True); p.add_argument("-o", "--output", required=True); p.set_defaults(fn=cmd_infer)
    p = sub.add_parser("dumpcsv", help="print a timing database as CSV")
    p.add_argument("database"); p.set_defaults(fn=cmd_dumpcsv)
    p = sub.add_parser("info", help="print the device limits in use")
    p.add_argument("--device", type=int, default=-1, help="GPU index; -1 prints the CDNA4 table without asking a device"); p.set_defaults(fn=cmd_info)

    args = ap.parse_args(argv)
    if args.version:
        print((_capi.lib().denox_hip_version() or b"").decode())
        return 0
    if not args.command:
        ap.print_help()
        return 1
    try:
        args.fn(args)
    except _capi.DenoxHipError as e:
        print(f"denox: {e}", file=sys.stderr)
        return 2
    return 0


if __name__ == "__main__":
    sys.exit(main())
