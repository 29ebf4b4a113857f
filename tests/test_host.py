"""Host-side tests that need no GPU: the C ABI surface, the serialised model, SymIR,
schedule selection, the timing table and the compile pipeline (hiprtc cross-compiles
gfx950 code objects without a device)."""
import ctypes
import itertools
import os
import re

import numpy as np
import pytest

import denox_amd as dx
from denox_amd import _capi, networks

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ----------------------------------------------------------------------------- C ABI surface
def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "denox_hip.h")).read()
    declared = set(re.findall(r"\b(denox_hip_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 50
    lib = ctypes.CDLL(_capi.LIB_PATH)
    missing = [n for n in sorted(declared) if not hasattr(lib, n)]
    assert not missing, missing
    assert declared == set(_capi.SIGNATURES), declared ^ set(_capi.SIGNATURES)
    assert b"gfx950" in _capi.lib().denox_hip_version()


def test_errors_are_codes_not_exceptions():
    L = _capi.lib()
    assert L.denox_hip_builder_create(None) == 1  # INVALID_ARGUMENT
    assert b"null" in L.denox_hip_last_error()
    m = dx.Model()
    x = m.input("input", "W", "H", 8)
    with pytest.raises(ValueError):
        m.conv2d(x, np.zeros((4, 9, 3, 3), np.float16))  # the Python wrapper checks first
    t = ctypes.c_int()
    w = np.zeros((4, 9, 3, 3), np.float16)
    rc = L.denox_hip_builder_conv2d(m._h, x.handle, 4, 9, 3, 3, w.ctypes.data, None, 1, 1, 1, 1, 1, 1, ctypes.byref(t))
    assert rc == 1 and b"input channels" in L.denox_hip_last_error()
    rc = L.denox_hip_builder_concat(m._h, 77, x.handle, ctypes.byref(t))
    assert rc == 1 and b"invalid tensor handle" in L.denox_hip_last_error()


def test_device_info_table():
    d = dx.device_info(-1)
    assert d["arch"] == "gfx950" and d["subgroup_size"] == 64 and d["compute_units"] == 256 and d["xcd_count"] == 8
    assert d["max_shared_memory"] == 160 * 1024 and d["max_workgroup_invocations"] == 1024
    assert (32, 32, 16) in d["matrix_shapes"] and (16, 16, 32) in d["matrix_shapes"]
    assert d["hbm_bytes_per_second"] == 8e12 and d["fp16_mfma_flops"] == 2.5e15 and not d["from_device"]


# ----------------------------------------------------------------------------- compile pipeline on the CPU
def _dispatch_names(blob, **ext):
    return [d["name"] for d in dx.describe(blob, **ext)["dispatches"]]


def test_tiny_unet_schedule_and_geometry():
    m, _ = networks.build("tiny_unet")
    # by default the last two convolutions (16 channels between them, read by nobody else) are one dispatch
    assert _dispatch_names(dx.compile_model(m), H=128, W=128) == ["conv3x3+relu", "maxpool", "conv3x3+relu", "concat+upsample+conv3x3+relu+conv3x3"]
    d = dx.describe(dx.compile_model(m, features=dict(conv_conv_fusion=False)), H=128, W=128)
    names = [x["name"] for x in d["dispatches"]]
    # e0 feeds both the pool and the skip, so the pool stays its own dispatch; upsample+concat fold into the conv
    assert names == ["conv3x3+relu", "maxpool", "conv3x3+relu", "concat+upsample+conv3x3+relu", "conv3x3"]
    conv0 = d["dispatches"][0]
    # IN_W, IN_H, then the tile-walk flag, which alternates along the schedule
    assert conv0["push_constants"] == [128, 128, 0] and conv0["flops"] == 2 * 9 * 3 * 16 * 128 * 128
    assert [x["push_constants"][-1] for x in d["dispatches"] if "conv3x3" in x["name"]] == [0, 1, 0, 1]
    tx, ty, tz = conv0["workgroup_count"]
    rows = conv0["workgroup_size"][0] // 64 * int(re.search(r"RPW=(\d+)", conv0["debug_info"]).group(1))
    assert tx * 32 >= 128 and ty * rows >= 128 and (tx - 1) * 32 < 128 and (ty - 1) * rows < 128 and tz == 1
    pool = d["dispatches"][1]
    assert pool["memory_reads"] == 128 * 128 * 16 * 2 and pool["memory_writes"] == 64 * 64 * 16 * 2
    # bindings are numbered input < output < parameter (weights, bias)
    b = d["dispatches"][3]["bindings"]
    assert [x["binding"] for x in b] == list(range(len(b))) and [x["access"] for x in b] == [0, 0, 1, 0, 0]
    assert [d["tensors"][x["tensor"]]["param"] for x in b] == [False, False, False, True, True]


def test_fusion_switches_change_the_schedule():
    m, _ = networks.build("tiny_unet")
    none = dict(conv_relu_fusion=False, concat_conv_fusion=False, upsample_fusion=False, pool_fusion=False, conv_conv_fusion=False)
    names = _dispatch_names(dx.compile_model(m, features=dict(none, implicit_concat=False)), H=64, W=64)
    assert names == ["conv3x3", "relu", "maxpool", "conv3x3", "relu", "upsample", "concat-copy", "conv3x3", "relu", "conv3x3"]
    # the upsampled tensor is read by the concat only: the upsample stores straight into the concat's tensor; the skip
    # tensor is also read by the pool and keeps its copy
    names = _dispatch_names(dx.compile_model(m, features=none), H=64, W=64)
    assert names == ["conv3x3", "relu", "maxpool", "conv3x3", "relu", "upsample+concat", "concat-copy-src1", "conv3x3", "relu", "conv3x3"]
    names = _dispatch_names(dx.compile_model(m, features=dict(upsample_fusion=False, conv_conv_fusion=False)), H=64, W=64)
    assert names == ["conv3x3+relu", "maxpool", "conv3x3+relu", "upsample", "concat+conv3x3+relu", "conv3x3"]
    names = _dispatch_names(dx.compile_model(m, features=dict(upsample_fusion=False)), H=64, W=64)
    assert names == ["conv3x3+relu", "maxpool", "conv3x3+relu", "upsample", "concat+conv3x3+relu+conv3x3"]


def test_oidn_unet_schedule_dispatch_geometry_covers_every_pixel():
    m, _ = networks.build("oidn_unet")
    for H, W in [(1080, 1920), (1077, 1917), (16, 16), (17, 33)]:
        Hp, Wp = (H + 15) // 16 * 16, (W + 15) // 16 * 16
        # the default schedule joins the two thin full-resolution layer pairs at either end of the network
        f = dx.describe(dx.compile_model(m, assume={"H": H, "W": W}), H=H, W=W)
        assert f["dispatches"][0]["name"] == "pad+conv3x3+relu+conv3x3+relu+maxpool" and f["dispatches"][-1]["name"] == "conv3x3+relu+conv3x3+slice"
        assert len(f["dispatches"]) == 14 and all("conv3x3" in x["name"] for x in f["dispatches"])
        assert sum(x["flops"] for x in f["dispatches"]) == pytest.approx(523.9e9 * (Hp * Wp) / (1088 * 1920), rel=2e-3)
        for x in (f["dispatches"][0], f["dispatches"][-1]):  # persistent launches of one workgroup per compute unit
            assert x["workgroup_count"] == [256, 1, 1] and x["push_constants"][:2] == [Wp, Hp]
        d = dx.describe(dx.compile_model(m, assume={"H": H, "W": W}, features=dict(conv_conv_fusion=False)), H=H, W=W)
        # pad and crop fold into the first / last conv: IN extent, then source extent + offsets or crop window
        assert d["dispatches"][0]["name"] == "pad+conv3x3+relu" and d["dispatches"][-1]["name"] == "conv3x3+slice"
        assert d["dispatches"][0]["push_constants"] == [Wp, Hp, W, H, 0, 0, 0]
        assert d["dispatches"][-1]["push_constants"] == [Wp, Hp, W, H, 0, 0, 1]
        u = dx.describe(dx.compile_model(m, assume={"H": H, "W": W}, features=dict(pad_fusion=False, slice_fusion=False, conv_conv_fusion=False)), H=H, W=W)
        assert u["dispatches"][0]["name"] == "pad" and u["dispatches"][-1]["name"] == "slice"
        assert u["dispatches"][0]["push_constants"] == [Wp, Hp, 0, Wp - W, 0, Hp - H]
        assert u["dispatches"][-1]["push_constants"] == [0, 0, Wp, Hp, W, H]
        convs = [x for x in d["dispatches"] if "conv3x3" in x["name"]]
        assert len(convs) == 16 == len(d["dispatches"])
        assert sum(x["flops"] for x in convs) == pytest.approx(523.9e9 * (Hp * Wp) / (1088 * 1920), rel=2e-3)
        for x in convs:
            w, h = x["push_constants"][:2]
            rows = int(re.search(r"WAVES=(\d+)", x["debug_info"]).group(1)) * int(re.search(r"RPW=(\d+)", x["debug_info"]).group(1))
            gx, gy, gz = x["workgroup_count"]
            kt = int(re.search(r"KT=(\d+)", x["debug_info"]).group(1))
            kout = int(re.search(r"KOUT=(\d+)", x["debug_info"]).group(1))
            if "SLOTS=" in x["debug_info"]:  # persistent launch: 8 XCDs x channel tiles x slots workgroups
                slots = int(re.search(r"SLOTS=(\d+)", x["debug_info"]).group(1))
                assert (gx, gy, gz) == (8 * ((kout + 31) // 32 * 32 // kt) * slots, 1, 1) and gx <= 256
            else:
                assert gx == -(-w // 32) and gy == -(-h // rows)
                assert gz * kt == (kout + 31) // 32 * 32
        out = d["tensors"][d["outputs"][0]]
        assert (out["height"], out["width"], out["channels"]) == (H, W, 3)


def test_every_conv_configuration_has_a_live_parity_case():
    """The GPU parity tests skip a (configuration, layer shape) pair the compiler refuses (not enough LDS or registers for
    that shape).  Checked here, without a GPU: the tests' lists name exactly the configurations of the library's tables, and
    every configuration compiles for at least one shape of the test that covers it -- none is tested by skips alone."""
    import test_gpu_conv_pair as tp
    import test_gpu_layers as tl
    from util import he_weights, small_bias
    listed = set(tl.ALL_CONFIGS) | set(tl.FOLD_CONFIGS) | set(tl.STRIDED_ONLY_CONFIGS) | set(tp.PAIR_CONFIGS)
    assert listed == set(dx.conv_config_names()), listed ^ set(dx.conv_config_names())
    rng = np.random.default_rng(0)

    def compiles(m, config):
        try:
            dx.compile_model(m, conv_config=config)
        except dx.DenoxHipError as e:
            assert e.status == 5
            return False
        return config in dx.last_compile_report()

    def plain(C, K, stride=(1, 1), pad=(1, 1), R=3, S=3):
        m = dx.Model()
        m.output(m.relu(m.conv2d(m.input("input", "W", "H", C), he_weights(rng, K, C, R, S), small_bias(rng, K), stride=stride, padding=pad)))
        return m

    def folded(CA, CB, K):
        m = dx.Model()
        t = m.upsample(m.input("lo", m.sym("W") // 2, m.sym("H") // 2, CA))
        if CB:
            t = m.concat(t, m.input("x", "W", "H", CB))
        m.output(m.activation(m.conv2d(t, he_weights(rng, K, CA + CB), small_bias(rng, K)), "leaky_relu", 0.25))
        return m

    dead = [c for c in tl.ALL_CONFIGS if not any(compiles(plain(C, K), c) for C, K, _, _ in tl.EVERY_CONFIG_SHAPES)]
    dead += [c for c in tl.FOLD_CONFIGS if not any(compiles(folded(CA, CB, K), c) for CA, CB, K, _, _, _ in tl.FOLD_SHAPES)]
    dead += [c for c in tl.STRIDED_ONLY_CONFIGS if not any(compiles(plain(24, 40, stride, pad, R, S), c) for R, S, pad, stride in tl.GEOMETRY_CASES)]
    for c in tp.PAIR_CONFIGS:
        hit = False
        for C, K1, K2, tail in [(9, 32, 32, "relu"), (16, 32, 32, "relu"), (64, 32, 3, "none")]:
            m, _ = tp.build(rng, C, K1, K2, tail)
            hit |= compiles(m, c)
        if not hit:
            dead.append(c)
    assert not dead, dead


def test_missing_kernel_is_reported():
    m = dx.Model()
    x = m.input("input", "W", "H", 8)
    m.output(m.conv2d(x, np.zeros((8, 8, 3, 3), np.float16), dilation=(2, 2)))  # dilated convolutions have no kernel
    with pytest.raises(dx.DenoxHipError) as e:
        dx.compile_model(m)
    assert e.value.status == 5 and "no kernel implements" in str(e.value)


# ----------------------------------------------------------------------------- concat without copies
def _w(rng, k, c):
    return (rng.standard_normal((k, c, 3, 3)) * 0.1).astype(np.float16)


def test_concat_sources_are_placed_inside_the_result():
    rng = np.random.default_rng(0)
    m = dx.Model()
    x = m.input("input", "W", "H", 8)
    a, b = m.conv2d(x, _w(rng, 16, 8)), m.relu(m.conv2d(x, _w(rng, 24, 8)))
    c = m.concat(a, b)
    m.output(c)
    d = dx.describe(dx.compile_model(m, conv_config="w4r2k16"), H=20, W=30)
    assert [x_["name"] for x_ in d["dispatches"]] == ["conv3x3+concat", "conv3x3+relu+concat"]
    assert all("OPITCH=40" in x_["debug_info"] and "OVEC=1" in x_["debug_info"] for x_ in d["dispatches"])
    out = d["tensors"][d["outputs"][0]]
    views = [t for t in d["tensors"] if not t["param"] and t.get("channels") in (16, 24)]
    assert len(views) == 2 and all(t["buffer"] == out["buffer"] for t in views)
    by_c = {t["channels"]: t for t in views}
    assert (by_c[16]["offset"], by_c[24]["offset"]) == (0, 32)  # channel 16 of pixel 0
    assert by_c[24]["size"] == out["size"] - 32 and out["size"] == 20 * 30 * 40 * 2
    assert len(d["buffers"]) == 2 + 2  # input, result, two weight blobs: no buffer is left for the sources
    # switched off: the convs write tensors of their own and one launch copies both into whole pixels
    d = dx.describe(dx.compile_model(m, conv_config="w4r2k16", features={"implicit_concat": False}), H=20, W=30)
    assert [x_["name"] for x_ in d["dispatches"]] == ["conv3x3", "conv3x3+relu", "concat-copy"]
    cat = d["dispatches"][2]
    assert cat["memory_reads"] == cat["memory_writes"] == out["size"] and len(cat["bindings"]) == 3


def test_concat_sources_that_cannot_move():
    rng = np.random.default_rng(1)
    # a source with a second consumer, a model input, a model output and concat(t, t) keep their own buffers
    m = dx.Model()
    x = m.input("input", "W", "H", 8)
    a = m.conv2d(x, _w(rng, 8, 8))
    c = m.concat(a, x)          # x: model input; a: also read by the conv below
    e = m.conv2d(a, _w(rng, 8, 8))
    f = m.concat(e, e)          # the same tensor twice
    m.output(c)
    m.output(f)
    blob = dx.compile_model(m, conv_config="w4r2k16")
    assert "in-place" not in dx.last_compile_report()
    d = dx.describe(blob, H=16, W=16)
    assert sum(x_["name"] == "concat-copy" for x_ in d["dispatches"]) == 2
    m = dx.Model()
    x = m.input("input", "W", "H", 8)
    a = m.conv2d(x, _w(rng, 8, 8))
    m.output(a)                 # a model output stays a tensor of its own
    m.output(m.concat(a, m.conv2d(x, _w(rng, 16, 8))))
    dx.compile_model(m, conv_config="w4r2k16")
    assert "copy/in-place" in dx.last_compile_report()
    # an unaligned channel range is stored element by element
    m = dx.Model()
    x = m.input("input", "W", "H", 8)
    m.output(m.concat(m.conv2d(x, _w(rng, 3, 8)), m.conv2d(x, _w(rng, 8, 8))))
    d = dx.describe(dx.compile_model(m, conv_config="w4r2k16"), H=16, W=16)
    assert all("OPITCH=11" in x_["debug_info"] and "OVEC=0" in x_["debug_info"] for x_ in d["dispatches"]) and len(d["dispatches"]) == 2


# ----------------------------------------------------------------------------- serialised model
def _nested_concat_model(widths, depth_first=True):
    """convs over one 16-channel input, concatenated pairwise into one tensor, then a conv over the lot."""
    rng = np.random.default_rng(sum(widths))
    m = dx.Model()
    t = m.input("input", "W", "H", 16)
    leaves = [m.relu(m.conv2d(t, (rng.standard_normal((k, 16, 3, 3)) * 0.1).astype(np.float16), (rng.standard_normal(k) * 0.01).astype(np.float16))) for k in widths]
    acc = leaves[0]
    for leaf in leaves[1:]:
        acc = m.concat(acc, leaf) if depth_first else m.concat(leaf, acc)
    total = sum(widths)
    out = m.conv2d(acc, (rng.standard_normal((16, total, 3, 3)) * 0.05).astype(np.float16), np.zeros(16, np.float16))
    m.output(out)
    return m, leaves, out


@pytest.mark.parametrize("widths", [(16, 24, 8), (64, 64, 64), (8, 24, 16, 40)])
@pytest.mark.parametrize("features", [{}, {"layout_preference": 1}])
def test_concat_of_concats_without_dispatches_shares_one_buffer(widths, features):
    """A zero-dispatch (CHWC8) concat whose result is the source of another one: every leaf has to end up inside the
    outermost result, at the sum of the offsets along the chain, not inside a buffer that the inner result has left."""
    m, leaves, out = _nested_concat_model(widths)
    H = W = 32
    d = dx.describe(dx.compile_model(m, features=dict(features, conv_conv_fusion=False)), H=H, W=W)
    names = [x["debug_info"].split(" | ")[0] for x in d["dispatches"]]
    if any("concat" in x["name"] for x in d["dispatches"]):
        pytest.skip(f"this selection copies: {names}")
    act = [t for t in d["tensors"] if not t["param"] and t["format"] == 3]
    by_channels = {}
    for t in act:
        by_channels.setdefault(t["channels"], []).append(t)
    whole = by_channels[sum(widths)][0]
    last = d["dispatches"][-1]
    assert whole["buffer"] in [d["tensors"][b["tensor"]]["buffer"] for b in last["bindings"]], "the last conv reads the outermost concat"
    # leaves, in concat order, tile the outermost tensor without gaps
    leaf_tensors = sorted((t for t in act if t["buffer"] == whole["buffer"] and t["channels"] in widths and t is not whole), key=lambda t: t["offset"])
    assert len(leaf_tensors) == len(widths), (len(leaf_tensors), names)
    off = 0
    for t, k in zip(leaf_tensors, widths):
        assert t["offset"] == off and t["channels"] == k and t["size"] == H * W * k * 2, (t, off)
        off += t["size"]
    assert off == whole["size"]
    # the partial concats start where the outermost one does
    for c in itertools.accumulate(widths):
        for t in by_channels.get(c, []):
            if t["channels"] not in widths:
                assert t["buffer"] == whole["buffer"] and t["offset"] == 0, t


def test_dnx_round_trip_and_corruption():
    m, _ = networks.build("tiny_unet")
    blob = dx.compile_model(m)
    assert blob[4:8] == b"dnxx" and len(blob) % 8 == 0  # file identifier of dnx.fbs:4; size a multiple of the widest scalar
    d = dx.describe(blob, H=32, W=48)
    assert d["producer"] == "denox-hip" and d["value_names"] == ["W", "H"] and d["binaries"] >= 3
    pad = len(blob) - len(blob.rstrip(b"\0"))  # the buffer ends with the first string written and its alignment padding
    for cut in (0, 3, 11, 100, len(blob) // 2, len(blob) - pad - 1):
        with pytest.raises(dx.DenoxHipError) as e:
            dx.describe(blob[:cut])
        assert e.value.status == 2
    with pytest.raises(dx.DenoxHipError):
        dx.describe(blob[:4] + b"XXXX" + blob[8:])
    # flip bytes all over the buffer: every outcome must be a clean error or a successful parse, never a crash
    rng = np.random.default_rng(0)
    head = 20000  # root table, tensor / dispatch tables, vtables; the rest is weights and code objects
    for i in range(600):
        b = bytearray(blob)
        pos = int(rng.integers(0, head if i % 2 else len(b)))
        b[pos] ^= int(rng.integers(1, 256))
        try:
            dx.describe(bytes(b), H=32, W=32)
        except dx.DenoxHipError as e:
            assert e.status in (1, 2)


def test_symir_from_builder_matches_oracle(oracle):
    # extents computed by the builder's symbolic engine agree with direct integer arithmetic
    m = dx.Model()
    x = m.input("input", "W", "H", 8)
    p = m.pad_to_multiple(x, 16)
    q = m.pool(m.pool(p))
    u = m.upsample(q, 4)
    s = m.slice(u, 3, x.width - 1, 0, x.height)
    m.output(s)
    blob = dx.compile_model(m)
    for H, W in [(1080, 1920), (1077, 1917), (5, 9), (16, 32), (33, 47)]:
        d = dx.describe(blob, H=H, W=W)
        Hp, Wp = -(-H // 16) * 16, -(-W // 16) * 16
        o = d["tensors"][d["outputs"][0]]
        assert (o["height"], o["width"]) == (H, W - 4)
        assert d["dispatches"][0]["push_constants"] == [Wp, Hp, 0, Wp - W, 0, Hp - H]
    # the same program evaluated by the oracle's SymIR interpreter: (16 - H % 16) % 16 etc.
    dp = oracle.symir_eval([1077, 1917], [(oracle.SYM_MOD | oracle.SYM_RHSC, 0, 16), (oracle.SYM_SUB | oracle.SYM_LHSC, 16, 2),
                                          (oracle.SYM_MOD | oracle.SYM_RHSC, 3, 16)])
    assert dp[-1] == 11


# ----------------------------------------------------------------------------- schedule selection (exhaustive cross-check)
def _select(n, inputs, edges, costs, outputs):
    L = _capi.lib()
    is_in = np.array([1 if i in inputs else 0 for i in range(n)], np.uint8)
    offs = np.zeros(len(edges) + 1, np.uint32)
    flat = []
    for i, (ins, _) in enumerate(edges):
        flat += list(ins)
        offs[i + 1] = len(flat)
    flat = np.array(flat if flat else [0], np.int32)
    outs_e = np.array([o for _, o in edges], np.int32)
    c = np.array(costs, np.float64)
    outs = np.array(outputs, np.int32)
    chosen = np.zeros(max(1, len(edges)), np.uint32)
    cnt, total = ctypes.c_uint32(), ctypes.c_double()
    _capi.check(L.denox_hip_min_cost_subgraph(n, is_in.ctypes.data, len(edges), offs.ctypes.data, flat.ctypes.data, outs_e.ctypes.data,
                                              c.ctypes.data, len(outputs), outs.ctypes.data, chosen.ctypes.data, ctypes.byref(cnt), ctypes.byref(total)))
    return list(chosen[:cnt.value]), total.value


def _brute(n, inputs, edges, costs, outputs):
    best = float("inf")
    for r in range(len(edges) + 1):
        for sub in itertools.combinations(range(len(edges)), r):
            prod = [edges[e][1] for e in sub]
            if len(set(prod)) != len(prod):
                continue
            have = set(inputs) | set(prod)
            if not all(o in have for o in outputs):
                continue
            if not all(all(i in have for i in edges[e][0]) for e in sub):
                continue
            best = min(best, sum(costs[e] for e in sub))
    return best


def test_min_cost_selection_against_exhaustive_enumeration():
    rng = np.random.default_rng(42)
    for trial in range(120):
        n = int(rng.integers(3, 9))
        n_in = int(rng.integers(1, 3))
        inputs = set(range(n_in))
        edges, costs = [], []
        for out in range(n_in, n):
            for _ in range(int(rng.integers(1, 4))):
                k = int(rng.integers(1, 3))  # one- and two-source edges (a fused concat has two)
                ins = tuple(sorted(set(int(v) for v in rng.integers(0, out, k))))
                edges.append((ins, out))
                costs.append(float(rng.integers(1, 20)))
        outputs = [n - 1] + ([int(rng.integers(n_in, n))] if rng.random() < 0.3 else [])
        chosen, total = _select(n, inputs, edges, costs, outputs)
        want = _brute(n, inputs, edges, costs, outputs)
        assert total == pytest.approx(want), (trial, edges, costs, outputs)
        # the chosen set is itself feasible, in execution order, and costs what it claims
        have = set(inputs)
        for e in chosen:
            assert all(i in have for i in edges[e][0])
            assert edges[e][1] not in have
            have.add(edges[e][1])
        assert all(o in have for o in outputs) and sum(costs[e] for e in chosen) == pytest.approx(total)
    # an output nothing produces
    chosen, total = _select(3, {0}, [((0,), 1)], [1.0], [2])
    assert chosen == [] and total >= 1e300
    # a skip tensor used twice is paid for once: 0 ->1 (5), 1->2 (1), {1,2}->3 (1) vs 0->3 direct (8)
    chosen, total = _select(4, {0}, [((0,), 1), ((1,), 2), ((1, 2), 3), ((0,), 3)], [5, 1, 1, 8], [3])
    assert total == 7 and chosen == [0, 1, 2]


def test_extents_the_graph_needs_are_checked_per_instance():
    """Symbolic extents leave two things open until an instance gets its values: whether the sources of a concat agree in
    width and height, and whether a slice stays inside its source.  Both are recorded in the model file and checked when
    extents are supplied (describe here, instance creation on the GPU), with the layer and the numbers in the message;
    with constant extents the builder refuses at once."""
    m, _ = networks.build("oidn_unet", align=False)  # no pad to a multiple of 16: upsample(pool(x)) only matches x for such extents
    blob = dx.compile_model(m)
    assert len(dx.describe(blob, H=64, W=96)["dispatches"]) > 7
    for H, W, what in [(66, 64, "heights"), (64, 70, "widths"), (16, 64, None), (8, 64, "heights")]:
        if what is None:
            dx.describe(blob, H=H, W=W)  # 16 rows: every one of the four levels still halves evenly
            continue
        with pytest.raises(dx.DenoxHipError) as e:
            dx.describe(blob, H=H, W=W)
        assert e.value.status == 1 and "concat" in str(e.value) and what in str(e.value)
    dx.describe(blob)  # a listing without extents evaluates nothing
    m2 = dx.Model()
    t = m2.input("input", "W", "H", 8)
    m2.output(m2.slice(t, 2, 40, 1, m2.sym("H") - 1))
    b2 = dx.compile_model(m2)
    dx.describe(b2, H=10, W=64)
    for H, W in [(10, 30), (1, 64)]:
        with pytest.raises(dx.DenoxHipError) as e:
            dx.describe(b2, H=H, W=W)
        assert e.value.status == 1 and "slice" in str(e.value)
    # the record survives the file: damaged relation codes are refused by the reader's validation
    assert dx.describe(bytes(blob), H=64, W=96)["dispatches"]
    with pytest.raises(dx.DenoxHipError):
        m3 = dx.Model()
        m3.concat(m3.input("a", 8, 8, 4), m3.input("b", 9, 8, 4))


# ----------------------------------------------------------------------------- timing table
def test_db_running_statistics_and_persistence(tmp_path):
    path = str(tmp_path / "gpu.db")
    db = dx.Db(path)
    m, _ = networks.build("tiny_unet")
    n = db.populate(m, assume={"H": 64, "W": 64}, conv_config="w4r2k16")
    assert n == len(db) and n >= 10
    assert db.populate(m, assume={"H": 64, "W": 64}, conv_config="w4r2k16") == 0  # same dispatches: no new rows
    assert db.populate(m, assume={"H": 128, "W": 64}, conv_config="w4r2k16") > 0  # other extents: other push constants / grids
    rng = np.random.default_rng(3)
    samples = rng.normal(50_000, 4_000, 57)
    for s in samples:
        db.add_sample(2, s)
    cnt, mean, std = db.row_stats(2)
    assert cnt == 57 and mean == pytest.approx(samples.mean(), rel=1e-12) and std == pytest.approx(samples.std(), rel=1e-9)
    db.writeback()
    again = dx.Db(path)
    assert len(again) == len(db)
    c2, m2, s2 = again.row_stats(2)
    assert (c2, m2) == (57, pytest.approx(mean, rel=1e-15)) and s2 == pytest.approx(std, rel=1e-12)
    assert again.row_stats(0)[0] == 0
    csv = again.dump_csv().splitlines()
    assert csv[0].startswith("operation,shader,config") and len(csv) == len(db) + 1
    with pytest.raises(dx.DenoxHipError):
        db.add_sample(10**6, 1.0)
    (tmp_path / "bad.db").write_text("not a db\n")
    with pytest.raises(dx.DenoxHipError):
        dx.Db(str(tmp_path / "bad.db"))


def test_measured_latencies_drive_the_selection(tmp_path):
    # make the unfused upsample + concat + conv look cheaper than the fused kernel: the compiler must follow the table
    m, _ = networks.build("tiny_unet")
    db = dx.Db(str(tmp_path / "t.db"))
    single = dict(conv_conv_fusion=False)  # this test is about one layer's alternatives
    db.populate(m, assume={"H": 64, "W": 64}, conv_config="w4r2k16", features=single)
    rows = db.dump_csv().splitlines()[1:]
    for i, r in enumerate(rows):
        op = r.split('","')[0].strip('"')
        lat = 900_000.0 if ("concat+" in op or "upsample+" in op) else 1_000.0
        for _ in range(3):
            db.add_sample(i, lat)
    names = _dispatch_names(dx.compile_model(m, assume={"H": 64, "W": 64}, conv_config="w4r2k16", db=db, features=single), H=64, W=64)
    # (upsample, then one launch copying both sources) and (upsample stored in place, then a copy of the other source) cost the same here
    assert ("upsample" in names and "concat-copy" in names) or ("upsample+concat" in names and "concat-copy-src1" in names)
    assert not any(n.startswith("concat+") for n in names)
    assert "measured" in dx.last_compile_report()
    # without a table the roofline estimate prefers the fused kernel
    names = _dispatch_names(dx.compile_model(m, assume={"H": 64, "W": 64}, conv_config="w4r2k16", features=single), H=64, W=64)
    assert "concat+upsample+conv3x3+relu" in names


def test_internal_tensors_have_two_layouts_to_choose_from(tmp_path):
    """Every internal tensor with a multiple of 8 channels exists pixel-major and channel-block-major (the reference's
    specialization.cpp:13-16,282-306 clones tensors per format): the table lists candidates for both, the measured cost
    decides between them, and what the schedule picks is recorded per tensor in the model file."""
    m, _ = networks.build("oidn_unet")
    assume = {"H": 64, "W": 64}
    db = dx.Db(str(tmp_path / "t.db"))
    db.populate(m, assume=assume)
    rows = [r.split('","') for r in db.dump_csv().splitlines()[1:]]
    configs = [r[2] for r in rows]
    assert any(c.endswith("/hwc>chwc8") for c in configs) and any(c.endswith("/chwc8>hwc") for c in configs) and any(c.endswith("/chwc8>chwc8") for c in configs)
    assert any(c == "vec8/chwc8" for c in configs) and any(c == "vec8" for c in configs)  # pool / upsample / activation in both layouts
    assert sum("chwc8" in c for c in configs) < sum("chwc8" not in c for c in configs)    # only selected conv configurations exist blocked

    def formats(blob):
        return [t["format"] for t in dx.describe(blob, **assume)["tensors"] if not t["param"]]

    # make every blocked candidate look ten times cheaper than the others, then the other way round
    for cheap_blocked in (True, False):
        d2 = dx.Db(str(tmp_path / f"t{int(cheap_blocked)}.db"))
        d2.populate(m, assume=assume)
        for i, c in enumerate(configs):
            for _ in range(3):
                d2.add_sample(i, 1_000.0 if ("chwc8" in c) == cheap_blocked else 10_000.0)
        f = formats(dx.compile_model(m, assume=assume, db=d2))
        assert (f.count(3) >= 8) if cheap_blocked else (3 not in f), (cheap_blocked, f)
    # switched off: no blocked candidate at all, and the switch alone never changes the interface tensors
    off = dx.Db(str(tmp_path / "off.db"))
    off.populate(m, assume=assume, features=dict(blocked_layout=False))
    assert not any("chwc8" in r for r in off.dump_csv().splitlines())
    f = formats(dx.compile_model(m, assume=assume, features=dict(layout_preference=1)))
    assert f[0] == 1 and f.count(3) >= 8
    d = dx.describe(dx.compile_model(m, assume=assume, features=dict(layout_preference=1)), **assume)
    assert d["tensors"][d["inputs"][0]]["format"] == 1 and d["tensors"][d["outputs"][0]]["format"] == 1


# ----------------------------------------------------------------------------- arena planner (runtime/arena_plan.hpp)
@pytest.fixture(scope="module")
def arena_probe(tmp_path_factory):
    import ctypes
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path_factory.mktemp("arena") / "libarena_probe.so"
    subprocess.run(["g++", "-O1", "-g", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra", "-Werror", os.path.join(root, "tests", "arena_probe.cpp"), "-o", str(out)],
                   check=True)
    lib = ctypes.CDLL(str(out))

    def plan(items, period=0):
        n = len(items)
        U, I = ctypes.c_ulonglong * n, ctypes.c_int * n
        offs, arena = U(), ctypes.c_ulonglong()
        lib.arena_probe_plan(n, U(*[b for b, _, _ in items]), I(*[f for _, f, _ in items]), I(*[l for _, _, l in items]), period, offs, ctypes.byref(arena))
        return list(offs), arena.value
    return plan


def test_arena_plan_never_overlaps_live_buffers(arena_probe):
    """Buffers alive at the same dispatch never share a byte; the arena is never larger than the sum of the buffers nor
    smaller than the largest set alive at one dispatch; a chain of equally sized buffers ping-pongs between two slots."""
    rng = np.random.default_rng(0)
    for trial in range(300):
        n = int(rng.integers(1, 24))
        T = int(rng.integers(1, 20))
        items = []
        for _ in range(n):
            f = int(rng.integers(0, T))
            items.append((int(rng.integers(1, 40)) * 256, f, int(rng.integers(f, T))))
        offs, arena = arena_probe(items)
        for i in range(n):
            assert offs[i] + items[i][0] <= arena
            for j in range(i):
                alive_together = items[i][1] <= items[j][2] and items[j][1] <= items[i][2]
                apart = offs[i] + items[i][0] <= offs[j] or offs[j] + items[j][0] <= offs[i]
                assert apart or not alive_together, (trial, i, j)
        peak = max(sum(b for b, f, l in items if f <= t <= l) for t in range(T))
        assert peak <= arena <= sum(b for b, _, _ in items)
    chain = [(1024, t, t + 1) for t in range(10)]  # each buffer written at t, read at t + 1
    offs, arena = arena_probe(chain)
    assert arena == 2048 and all(offs[t] != offs[t + 1] for t in range(9))
    assert arena_probe([]) == ([], 0)
    # an inference's first dispatch follows the previous inference's last: the buffer written first goes where the buffer
    # read last was, not to the lowest free offset (which holds a buffer that died one dispatch earlier)
    items = [(512, 0, 1), (1024, 13, 14), (512, 14, 15)]
    offs, arena = arena_probe(items, 16)
    assert arena == 1536 and offs == [1024, 0, 1024]
    assert arena_probe(items, -1)[0] == [0, 0, 1024]  # the preference switched off
