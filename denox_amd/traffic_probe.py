"""HBM traffic of the benchmark's dominant convolution, per candidate kernel, keyed by the SHA-256 of the code object.

Two steps:

`python3 -m denox_amd.traffic_probe run <map.json> [H W]` compiles the OIDN U-Net once per candidate configuration of its
three longest dispatches (dec_conv1a: concat + replicate pad + 2x upsample + conv 73 -> 64 + ReLU, and the two conv -> conv
dispatches at the network's ends), steering the selection to those candidates through a timing table that holds made-up
samples for them, runs every such schedule a few times, runs the
plain copy kernel of `denox_amd.calibrate`, and writes which entry point belongs to which code object.  Run it under
`rocprofv3 --pmc FETCH_SIZE` and again under `rocprofv3 --pmc WRITE_SIZE` (counters per dispatch, csv).

`python3 -m denox_amd.traffic_probe summarize <map.json> <FETCH_SIZE csv> <WRITE_SIZE csv>` averages the counters per
kernel, scales them by what the same counter read for the copy kernel of known size, and prints the JSON that
bench.py reads (`profiles/dominant_conv_traffic.json`): bytes fetched from and written to memory per launch, per code object.
"""
import csv
import json
import os
import re
import sys
import tempfile

import numpy as np

DOMINANT_OPERATION = "concat+pad+upsample+conv3x3+relu"   # dec_conv1a with everything folded into its loader
LAST_PAIR = "conv3x3+relu+conv3x3+slice"                   # dec_conv1b -> dec_conv0 -> crop in one dispatch
FIRST_PAIR = "pad+conv3x3+relu+conv3x3+relu+maxpool"       # enc_conv0 -> enc_conv1 -> pool in one dispatch
# Schedules to run: {operation: configuration} pairs that the selection is steered to.  The candidates of the three
# longest dispatches that the timing table has been seen to select, in the layouts it combines them in.
STEER = ([{DOMINANT_OPERATION: c} for c in ("h4r2n", "h4r2p", "g4r1p", "h4r2k32n", "h4r2", "g4r1n", "g4r1k32n", "g4r1", "g4r1k32", "s8r2k16", "s12r1k16", "t8r2k16", "p8r2k16", "f8r1")] +
         [{DOMINANT_OPERATION: "h4r2n", LAST_PAIR: c, FIRST_PAIR: f} for c, f in (("v4r2k64", "x8r2k16/hwc>chwc8"), ("d4r2k64", "x8r2k16/hwc>chwc8"), ("z4r2k64", "x8r2k16/hwc>chwc8"), ("y4r2k32", "v4r2k16"), ("u4r2k32", "x8r2k16"), ("x8r2k16", "x8r2k16"))] +
         [{DOMINANT_OPERATION: d + "/hwc>chwc8", LAST_PAIR: c + "/chwc8>hwc"} for d, c in (("s8r2k16", "v4r2k64"), ("s12r1k16", "z4r2k64"), ("s8r2k16", "y4r2k32"), ("s12r1k16", "x8r2k16"))] +
         # the same layers as four dispatches (conv -> conv fusion off, pixel-major), for comparison with the pairs
         [{"features": dict(conv_conv_fusion=False, blocked_layout=False)}])
# dispatches of that last schedule whose traffic is reported beside the pairs': entry point prefixes
UNFUSED_PAIR_LAYERS = ("conv3x3_c9e_k32_", "conv3x3_c32_k32_relu_pool_", "conv3x3_c64_k32_relu_", "conv3x3_c32_k3_crop_")
COPY_KERNEL = "memory_slice_c64v8"


def _norm(config):
    """'s8r2k16/kt64/hwc>chwc8' -> 's8r2k16/hwc>chwc8': the output channels per workgroup follow from the layer."""
    return re.sub(r"/kt\d+", "", config.strip('"'))


def run(map_path, H=1080, W=1920, frames=6):
    import denox_amd as dx
    from denox_amd import calibrate, networks
    model, _ = networks.build("oidn_unet", seed=0)
    x = networks.synthetic_input("oidn_unet", H, W, seed=0)
    kernels = {}
    tmp = tempfile.mkdtemp(prefix="denox_hip_probe_")
    for n, steer in enumerate(STEER):
        steer = dict(steer)
        features = steer.pop("features", {})
        db = dx.Db(os.path.join(tmp, f"steer{n}.db"))
        db.populate(model, assume={"H": H, "W": W}, features=features)
        rows = [r.split('","') for r in db.dump_csv().splitlines()[1:]]
        hits = [i for i, r in enumerate(rows) if steer.get(r[0].strip('"')) == _norm(r[2])]
        for i in hits:
            for _ in range(3):
                db.add_sample(i, 1000.0)  # 1 us: below every estimate, so the selection takes this candidate
        blob = dx.compile_model(model, assume={"H": H, "W": W}, db=db, features=features)
        desc = dx.describe(blob, H=H, W=W)["dispatches"]
        taken = {d["name"]: _norm(d["debug_info"].split(" | ")[0]) for d in desc}
        if any(taken.get(op) != cfg for op, cfg in steer.items()):
            print(f"traffic_probe: the schedule did not follow {steer}: {taken}", file=sys.stderr)
            continue
        inst = dx.Module.load(blob).instance(H=H, W=W)
        inst.infer(x)
        for _ in range(frames):
            inst.infer_device(None, None)
        inst.synchronize()
        times = inst.bench(warmup=1)
        for d, t in zip(desc, times):
            k = kernels.setdefault(d["entry_point"], {"code_sha256": d["code_sha256"], "operation": d["name"], "config": d["debug_info"].split(" | ")[0],
                                                     "algorithmic_read_bytes": t["memory_reads"], "algorithmic_write_bytes": t["memory_writes"], "flops": t["flops"]})
            if k["code_sha256"] != d["code_sha256"]:
                raise RuntimeError(f"two code objects share the entry point {d['entry_point']}")
        del inst
    calibrate.main()
    with open(map_path, "w") as f:
        json.dump({"height": H, "width": W, "dominant_operation": DOMINANT_OPERATION, "copy_kernel": COPY_KERNEL,
                   "copy_kernel_bytes": 1088 * 1920 * 64 * 2, "kernels": kernels}, f, indent=1)
    print(f"traffic_probe: {len(kernels)} kernels -> {map_path}")
    return 0


def per_kernel(csv_path, counter):
    acc = {}
    with open(csv_path) as f:
        for r in csv.DictReader(f):
            if r["Counter_Name"] == counter:
                acc.setdefault(r["Kernel_Name"], []).append(float(r["Counter_Value"]))
    return acc


def summarize(map_path, fetch_csv, write_csv):
    with open(map_path) as f:
        m = json.load(f)
    fetch, write = per_kernel(fetch_csv, "FETCH_SIZE"), per_kernel(write_csv, "WRITE_SIZE")
    n = m["copy_kernel_bytes"]
    cf, cw = fetch[m["copy_kernel"]], write[m["copy_kernel"]]
    # skip the first launch of the copy (cold caches)
    fscale, wscale = n / np.mean(cf[1:]), n / np.mean(cw[1:])
    out = {"height": m["height"], "width": m["width"], "dominant_operation": m["dominant_operation"],
           "source": "rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE runs of `python3 -m denox_amd.traffic_probe run` (see profiles/dominant_conv_traffic.md)",
           "calibration": {"copy_kernel": m["copy_kernel"], "copy_kernel_bytes": n, "fetch_size_per_dispatch": round(float(np.mean(cf[1:])), 1),
                           "write_size_per_dispatch": round(float(np.mean(cw[1:])), 1), "fetch_bytes_per_unit": round(fscale, 1), "write_bytes_per_unit": round(wscale, 1)},
           "kernels": {}}
    for entry, k in sorted(m["kernels"].items()):
        # the dominant layer's candidates and the two conv -> conv dispatches: kernels that run at one extent only
        # (a name like conv3x3_c96_k96_relu_* serves two layers of different size; a mean over both describes neither)
        if entry not in fetch or entry not in write or not (k["operation"] in (DOMINANT_OPERATION, LAST_PAIR, FIRST_PAIR) or entry.startswith(UNFUSED_PAIR_LAYERS)):
            continue
        f_, w_ = fetch[entry], write[entry]
        fb, wb = float(np.mean(f_[1:] if len(f_) > 1 else f_)) * fscale, float(np.mean(w_[1:] if len(w_) > 1 else w_)) * wscale
        alg = k["algorithmic_read_bytes"] + k["algorithmic_write_bytes"]
        out["kernels"][k["code_sha256"]] = {"entry_point": entry, "operation": k["operation"], "config": k["config"], "dispatches": [len(f_), len(w_)],
                                            "fetch_bytes": int(round(fb, -3)), "write_bytes": int(round(wb, -3)),
                                            "algorithmic_read_bytes": k["algorithmic_read_bytes"], "algorithmic_write_bytes": k["algorithmic_write_bytes"],
                                            "traffic_over_algorithmic": round((fb + wb) / alg, 3) if alg else None}
    print(json.dumps(out, indent=1))
    return 0


def main(argv):
    if len(argv) >= 2 and argv[0] == "run":
        return run(argv[1], *[int(a) for a in argv[2:4]])
    if len(argv) == 4 and argv[0] == "summarize":
        return summarize(*argv[1:])
    print(__doc__, file=sys.stderr)
    return 2


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
