"""CPU oracle for the denox hot path -- TEST INFRASTRUCTURE ONLY.

Loads ``oracle/_build/libdenox_oracle.so`` (built by ``oracle/Makefile`` from
``oracle/denox_oracle.c``) and wraps it for numpy.  Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import this package; nothing under ``denox_amd/`` does.

Tensors are numpy arrays in HWC order.  binary16 tensors are ``np.float16``
(their bit patterns are what the C side sees); fp32 tensors are ``np.float32``.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Dict, List, Optional, Sequence

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libdenox_oracle.so")

LAYOUT_HWC, LAYOUT_CHW, LAYOUT_CHWC8 = 0, 1, 2
ACT_NONE, ACT_RELU, ACT_LEAKY_RELU = 0, 1, 2


def build(force: bool = False) -> str:
    """Compile the C restatement (gcc, a second or two)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        i64, f32, u16p = ctypes.c_int64, ctypes.c_float, ctypes.c_void_p
        L.dnxo_f16_to_f32.restype = ctypes.c_float
        L.dnxo_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.dnxo_f32_to_f16.restype = ctypes.c_uint16
        L.dnxo_f32_to_f16.argtypes = [ctypes.c_float]
        L.dnxo_f16_to_f32_array.argtypes = [u16p, u16p, ctypes.c_size_t]
        L.dnxo_f32_to_f16_array.argtypes = [u16p, u16p, ctypes.c_size_t]
        L.dnxo_layout_index.restype = i64
        L.dnxo_layout_index.argtypes = [ctypes.c_int] + [i64] * 6
        L.dnxo_relayout_f16.argtypes = [u16p, ctypes.c_int, u16p, ctypes.c_int, i64, i64, i64]
        L.dnxo_conv2d_hwc.argtypes = [u16p, i64, i64, i64, u16p, u16p, i64, i64, i64,
                                      i64, i64, i64, i64, ctypes.c_int, f32, ctypes.c_int, u16p]
        L.dnxo_maxpool_hwc_f16.argtypes = [u16p, i64, i64, i64, i64, i64, u16p]
        L.dnxo_avgpool_hwc_f16.argtypes = [u16p, i64, i64, i64, i64, i64, u16p]
        L.dnxo_upsample_nearest_hwc_f16.argtypes = [u16p, i64, i64, i64, i64, u16p]
        L.dnxo_copy_channels_hwc_f16.argtypes = [u16p, i64, i64, i64, i64, u16p, i64, i64, i64]
        L.dnxo_concat_hwc_f16.argtypes = [u16p, i64, u16p, i64, i64, i64, u16p]
        L.dnxo_pad_replicate_hwc_f16.argtypes = [u16p, i64, i64, i64, i64, i64, i64, i64, u16p]
        L.dnxo_pad_zero_hwc_f16.argtypes = [u16p, i64, i64, i64, i64, i64, i64, i64, u16p]
        L.dnxo_slice_hwc_f16.argtypes = [u16p, i64, i64, i64, i64, i64, i64, i64, u16p]
        L.dnxo_activation_f16.argtypes = [u16p, ctypes.c_size_t, ctypes.c_int, f32, u16p]
        L.dnxo_symir_eval.argtypes = [i64, u16p, i64, u16p, u16p, u16p, u16p]
        L.dnxo_num_threads.restype = ctypes.c_int
        _lib = L
    return _lib


def _p(a: np.ndarray) -> ctypes.c_void_p:
    return ctypes.c_void_p(a.ctypes.data)


def _c(a, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


def _check(rc: int, what: str) -> None:
    if rc != 0:
        raise ValueError(f"oracle {what} failed with code {rc}")


# --------------------------------------------------------------------------- scalars
def f16_to_f32(bits: np.ndarray) -> np.ndarray:
    src = _c(bits, np.uint16)
    dst = np.empty(src.shape, np.float32)
    lib().dnxo_f16_to_f32_array(_p(src), _p(dst), src.size)
    return dst


def f32_to_f16_bits(x: np.ndarray) -> np.ndarray:
    src = _c(x, np.float32)
    dst = np.empty(src.shape, np.uint16)
    lib().dnxo_f32_to_f16_array(_p(src), _p(dst), src.size)
    return dst


def round_f16(x: np.ndarray) -> np.ndarray:
    """fp32 -> binary16 (RNE) -> np.float16 array."""
    return f32_to_f16_bits(x).view(np.float16)


# --------------------------------------------------------------------------- layouts
def layout_index(layout: int, H: int, W: int, C: int, h: int, w: int, c: int) -> int:
    return int(lib().dnxo_layout_index(layout, H, W, C, h, w, c))


def relayout(x_flat: np.ndarray, src_layout: int, dst_layout: int, H: int, W: int, C: int) -> np.ndarray:
    src = _c(x_flat, np.float16).reshape(-1)
    assert src.size == H * W * C
    dst = np.empty_like(src)
    _check(lib().dnxo_relayout_f16(_p(src), src_layout, _p(dst), dst_layout, H, W, C), "relayout")
    return dst


# --------------------------------------------------------------------------- layers
def conv2d(x: np.ndarray, weight_kcrs: np.ndarray, bias: Optional[np.ndarray] = None,
           stride: Sequence[int] = (1, 1), padding: Sequence[int] = (1, 1),
           act: int = ACT_NONE, alpha: float = 0.0, round_f16_out: bool = False) -> np.ndarray:
    """fp32 conv on an HWC tensor; inputs of any float dtype are widened exactly."""
    xin = _c(x, np.float32)
    w = _c(weight_kcrs, np.float32)
    H, W, C = xin.shape
    K, Cw, R, S = w.shape
    assert Cw == C, (Cw, C)
    b = None if bias is None else _c(bias, np.float32)
    Ho = (H + 2 * padding[0] - R) // stride[0] + 1
    Wo = (W + 2 * padding[1] - S) // stride[1] + 1
    out = np.empty((Ho, Wo, K), np.float32)
    _check(lib().dnxo_conv2d_hwc(_p(xin), H, W, C, _p(w), None if b is None else _p(b), K, R, S,
                                 stride[0], stride[1], padding[0], padding[1], act, float(alpha),
                                 1 if round_f16_out else 0, _p(out)), "conv2d")
    return out


def maxpool(x: np.ndarray, k: Sequence[int] = (2, 2)) -> np.ndarray:
    xin = _c(x, np.float16)
    H, W, C = xin.shape
    out = np.empty((H // k[0], W // k[1], C), np.float16)
    _check(lib().dnxo_maxpool_hwc_f16(_p(xin), H, W, C, k[0], k[1], _p(out)), "maxpool")
    return out


def avgpool(x: np.ndarray, k: Sequence[int] = (2, 2)) -> np.ndarray:
    xin = _c(x, np.float16)
    H, W, C = xin.shape
    out = np.empty((H // k[0], W // k[1], C), np.float16)
    _check(lib().dnxo_avgpool_hwc_f16(_p(xin), H, W, C, k[0], k[1], _p(out)), "avgpool")
    return out


def upsample_nearest(x: np.ndarray, f: int = 2) -> np.ndarray:
    xin = _c(x, np.float16)
    H, W, C = xin.shape
    out = np.empty((H * f, W * f, C), np.float16)
    _check(lib().dnxo_upsample_nearest_hwc_f16(_p(xin), H, W, C, f, _p(out)), "upsample")
    return out


def concat(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    a16, b16 = _c(a, np.float16), _c(b, np.float16)
    H, W, Ca = a16.shape
    assert b16.shape[:2] == (H, W)
    Cb = b16.shape[2]
    out = np.empty((H, W, Ca + Cb), np.float16)
    _check(lib().dnxo_concat_hwc_f16(_p(a16), Ca, _p(b16), Cb, H, W, _p(out)), "concat")
    return out


def copy_channels(src: np.ndarray, src_off: int, dst: np.ndarray, dst_off: int, count: int) -> None:
    assert src.dtype == np.float16 and dst.dtype == np.float16 and dst.flags.c_contiguous
    s = _c(src, np.float16)
    H, W, Cs = s.shape
    _check(lib().dnxo_copy_channels_hwc_f16(_p(s), H, W, Cs, src_off, _p(dst), dst.shape[2], dst_off, count),
           "copy_channels")


def pad_replicate(x: np.ndarray, left: int, right: int, top: int, bottom: int) -> np.ndarray:
    xin = _c(x, np.float16)
    H, W, C = xin.shape
    out = np.empty((H + top + bottom, W + left + right, C), np.float16)
    _check(lib().dnxo_pad_replicate_hwc_f16(_p(xin), H, W, C, left, right, top, bottom, _p(out)), "pad")
    return out


def pad_zero(x: np.ndarray, left: int, right: int, top: int, bottom: int) -> np.ndarray:
    xin = _c(x, np.float16)
    H, W, C = xin.shape
    out = np.empty((H + top + bottom, W + left + right, C), np.float16)
    _check(lib().dnxo_pad_zero_hwc_f16(_p(xin), H, W, C, left, right, top, bottom, _p(out)), "pad")
    return out


def slice_hw(x: np.ndarray, left: int, top: int, out_h: int, out_w: int) -> np.ndarray:
    xin = _c(x, np.float16)
    H, W, C = xin.shape
    out = np.empty((out_h, out_w, C), np.float16)
    _check(lib().dnxo_slice_hwc_f16(_p(xin), H, W, C, left, top, out_h, out_w, _p(out)), "slice")
    return out


def activation(x: np.ndarray, act: int, alpha: float = 0.0) -> np.ndarray:
    xin = _c(x, np.float16)
    out = np.empty_like(xin)
    _check(lib().dnxo_activation_f16(_p(xin), xin.size, act, float(alpha), _p(out)), "activation")
    return out


# --------------------------------------------------------------------------- SymIR
SYM_ADD, SYM_SUB, SYM_MUL, SYM_DIV, SYM_MOD, SYM_MIN, SYM_MAX = 1, 2, 3, 4, 5, 6, 7
SYM_LHSC, SYM_RHSC = 0x8000, 0x4000


def symir_eval(var_values: Sequence[int], ops: Sequence[Sequence[int]]) -> List[int]:
    """ops: (wire_opcode, lhs, rhs) triples; returns the whole value table."""
    vc = len(var_values)
    vv = np.asarray(list(var_values), np.int64).reshape(-1)
    oc = np.asarray([o[0] for o in ops], np.uint16).reshape(-1)
    lhs = np.asarray([o[1] for o in ops], np.int64).reshape(-1)
    rhs = np.asarray([o[2] for o in ops], np.int64).reshape(-1)
    dp = np.zeros(vc + len(ops), np.int64)
    _check(lib().dnxo_symir_eval(vc, _p(vv), len(ops), _p(oc), _p(lhs), _p(rhs), _p(dp)), "symir_eval")
    return [int(v) for v in dp]


def num_threads() -> int:
    return int(lib().dnxo_num_threads())


# --------------------------------------------------------------------------- networks
def run_graph(ops: Sequence[dict], inputs: Dict[str, np.ndarray], mode: str = "fp32") -> Dict[str, np.ndarray]:
    """Evaluate a layer list.

    ``ops`` is a list of dicts ``{"op": ..., "src": name | [names], "dst": name, ...}``
    in execution order (the same records ``denox_amd.Model.to_ops()`` emits).

    mode "fp32": the comparison target of the parity criterion -- inputs and
        weights are the binary16 values, every intermediate stays fp32, nothing
        is rounded between layers.
    mode "f16": every layer output is rounded to binary16, i.e. what a runtime
        that stores fp16 activations holds after each dispatch.
    Returns all named tensors (fp32 arrays in "fp32" mode, float16 in "f16").
    """
    assert mode in ("fp32", "f16")
    f16 = mode == "f16"
    env: Dict[str, np.ndarray] = {}
    for k, v in inputs.items():
        v16 = _c(v, np.float16)
        env[k] = v16 if f16 else v16.astype(np.float32)

    def as16(a):  # exact when values already are binary16 values
        return a if a.dtype == np.float16 else a.astype(np.float16)

    def back(a16, like_f32):
        return a16 if f16 else a16.astype(np.float32)

    for op in ops:
        kind = op["op"]
        src = op["src"]
        if kind == "conv2d":
            x = env[src]
            y = conv2d(x, op["weight"], op.get("bias"), op.get("stride", (1, 1)), op.get("padding", (1, 1)),
                       ACT_NONE, 0.0, round_f16_out=f16)
            env[op["dst"]] = y.astype(np.float16) if f16 else y
        elif kind == "activation":
            x = env[src]
            fn = op["func"]
            if f16:
                env[op["dst"]] = activation(x, ACT_RELU if fn == "relu" else ACT_LEAKY_RELU, op.get("alpha", 0.0))
            else:
                if fn == "relu":
                    env[op["dst"]] = np.maximum(x, np.float32(0))
                else:
                    a = np.float32(op.get("alpha", 0.0))
                    env[op["dst"]] = np.maximum(x, a * x)
        elif kind in ("pool", "upsample", "pad", "slice", "concat"):
            # data movement / comparisons: exact in either precision, so the fp32
            # mode runs them on fp32 arrays with numpy while the f16 mode goes
            # through the bit-exact C routines.
            if kind == "concat":
                a, b = env[src[0]], env[src[1]]
                env[op["dst"]] = concat(a, b) if f16 else np.concatenate([a, b], axis=2)
            elif kind == "pool":
                x = env[src]
                k = op.get("kernel", (2, 2))
                avg = op.get("func", "max") == "avg"
                if f16:
                    env[op["dst"]] = avgpool(x, k) if avg else maxpool(x, k)
                else:
                    H, W, C = x.shape
                    Ho, Wo = H // k[0], W // k[1]
                    win = x[:Ho * k[0], :Wo * k[1]].reshape(Ho, k[0], Wo, k[1], C)
                    env[op["dst"]] = win.mean(axis=(1, 3), dtype=np.float32) if avg else win.max(axis=(1, 3))
            elif kind == "upsample":
                x = env[src]
                f = op.get("factor", 2)
                env[op["dst"]] = upsample_nearest(x, f) if f16 else np.repeat(np.repeat(x, f, axis=0), f, axis=1)
            elif kind == "pad":
                x = env[src]
                l, r, t, b = op["left"], op["right"], op["top"], op["bottom"]
                if op.get("mode", "replicate") == "zero":
                    env[op["dst"]] = pad_zero(x, l, r, t, b) if f16 else np.pad(x, ((t, b), (l, r), (0, 0)), mode="constant")
                else:
                    env[op["dst"]] = pad_replicate(x, l, r, t, b) if f16 else np.pad(x, ((t, b), (l, r), (0, 0)), mode="edge")
            else:
                x = env[src]
                l, t, oh, ow = op["left"], op["top"], op["out_h"], op["out_w"]
                env[op["dst"]] = slice_hw(x, l, t, oh, ow) if f16 else np.ascontiguousarray(x[t:t + oh, l:l + ow])
        else:
            raise ValueError(f"unknown op {kind}")
    return env


# --------------------------------------------------------------------------- the parity bar for conv outputs
# Stated tolerance on the final binary16 output against the fp32 evaluation.
CONV_MAX_ABS = 2e-2
CONV_MEAN_ABS = 2e-3
# When an fp32 evaluation has outputs well above 1, a pipeline that *stores* every tensor as binary16 cannot meet the absolute
# bar however exactly it computes: rounding each layer's result once already leaves an error of that size (the oracle's "f16"
# evaluation -- fp32 accumulation, one round-to-nearest-even per layer -- against its "fp32" evaluation).  That error is the
# floor; the kernels are then held to a small multiple of it instead of to a multiple of the outputs' magnitude.
FLOOR_FACTOR_MAX = 2.0
FLOOR_FACTOR_MEAN = 1.5


def conv_parity(got_f16, want_f32, floor_f16=None):
    """Errors of `got_f16` against the fp32 evaluation and the bars they are held to.  `floor_f16`: the oracle's binary16-storage
    evaluation of the same layers on the same input, or a function returning it (only called when the stated bar is missed)."""
    got = np.asarray(got_f16, np.float32)
    want = np.asarray(want_f32, np.float32)
    assert got.shape == want.shape, (got.shape, want.shape)
    err = np.abs(got - want)
    r = {"max_abs": float(err.max()) if err.size else 0.0, "mean_abs": float(err.mean()) if err.size else 0.0,
         "argmax": tuple(int(i) for i in np.unravel_index(err.argmax(), err.shape)) if err.size else (),
         "finite": bool(np.isfinite(got).all()), "bar_max_abs": CONV_MAX_ABS, "bar_mean_abs": CONV_MEAN_ABS,
         "floor_max_abs": None, "floor_mean_abs": None}
    r["literal_ok"] = r["finite"] and r["max_abs"] <= CONV_MAX_ABS and r["mean_abs"] <= CONV_MEAN_ABS
    if floor_f16 is not None and (not r["literal_ok"] or not callable(floor_f16)):
        floor = np.abs(np.asarray(floor_f16() if callable(floor_f16) else floor_f16, np.float32) - want)
        r["floor_max_abs"], r["floor_mean_abs"] = float(floor.max()), float(floor.mean())
        r["bar_max_abs"] = max(CONV_MAX_ABS, FLOOR_FACTOR_MAX * r["floor_max_abs"])
        r["bar_mean_abs"] = max(CONV_MEAN_ABS, FLOOR_FACTOR_MEAN * r["floor_mean_abs"])
    r["ok"] = r["finite"] and r["max_abs"] <= r["bar_max_abs"] and r["mean_abs"] <= r["bar_mean_abs"]
    return r
