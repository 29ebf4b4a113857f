"""Graph builder: the Python face of ``denox_hip_builder_*``.

Mirrors the reference's ``compiler::Model`` builder
(compiler/src/denox/compiler/frontend/model/Model.hpp:33-62): ``input``,
``conv2d``, ``activation``, ``upsample``, ``pool``, ``concat``, ``pad``,
``slice``, ``output``.  Every call goes straight into the native builder; the
Python object additionally keeps a plain record of the layers (``to_ops()``)
so that a checker can evaluate the same network elsewhere.
"""
from __future__ import annotations

import ctypes
from ctypes import byref, c_int, c_int64, c_void_p
from typing import Dict, List, Optional, Sequence, Union

import numpy as np

from . import _capi

SYM_ADD, SYM_SUB, SYM_MUL, SYM_DIV, SYM_MOD, SYM_MIN, SYM_MAX = 1, 2, 3, 4, 5, 6, 7


class Sym:
    """A symbolic integer owned by a Model (constant or expression over named extents)."""

    def __init__(self, model: "Model", handle: int, text: str):
        self.model, self.handle, self.text = model, handle, text

    def _bin(self, op: int, other, sym: str, swap=False) -> "Sym":
        o = self.model.sym(other)
        a, b = (o, self) if swap else (self, o)
        out = c_int64()
        _capi.check(_capi.lib().denox_hip_builder_sym_op(self.model._h, op, a.handle, b.handle, byref(out)))
        return Sym(self.model, out.value, f"({a.text} {sym} {b.text})")

    def __add__(self, o): return self._bin(SYM_ADD, o, "+")
    def __radd__(self, o): return self._bin(SYM_ADD, o, "+", True)
    def __sub__(self, o): return self._bin(SYM_SUB, o, "-")
    def __rsub__(self, o): return self._bin(SYM_SUB, o, "-", True)
    def __mul__(self, o): return self._bin(SYM_MUL, o, "*")
    def __rmul__(self, o): return self._bin(SYM_MUL, o, "*", True)
    def __floordiv__(self, o): return self._bin(SYM_DIV, o, "//")
    def __mod__(self, o): return self._bin(SYM_MOD, o, "%")
    def __rmod__(self, o): return self._bin(SYM_MOD, o, "%", True)
    def __repr__(self): return f"Sym({self.text})"


class Tensor:
    def __init__(self, model: "Model", handle: int, name: str, width: Sym, height: Sym, channels: int):
        self.model, self.handle, self.name = model, handle, name
        self.width, self.height, self.channels = width, height, channels

    def __repr__(self):
        if self.width is None:
            return f"Tensor({self.name}: C={self.channels})"
        return f"Tensor({self.name}: H={self.height.text} W={self.width.text} C={self.channels})"


def _f16(a, shape=None) -> np.ndarray:
    arr = np.ascontiguousarray(np.asarray(a), dtype=np.float16)
    if shape is not None and tuple(arr.shape) != tuple(shape):
        raise ValueError(f"expected shape {tuple(shape)}, got {tuple(arr.shape)}")
    return arr


class Model:
    def __init__(self):
        h = c_void_p()
        _capi.check(_capi.lib().denox_hip_builder_create(byref(h)))
        self._h = h
        self._ops: List[dict] = []
        self._count = 0
        self.inputs: List[Tensor] = []
        self.outputs: List[Tensor] = []

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            _capi.lib().denox_hip_builder_destroy(h)

    @classmethod
    def from_onnx(cls, source) -> "Model":
        """Build the graph from an ONNX file (path) or its bytes, as the reference's
        ``denox.compile(onnx, ...)`` does (compiler/src/denox/compiler/compile.cpp:21-61).
        Image tensors are NCHW with N = 1; dynamic height / width dimensions keep their
        ``dim_param`` names as extents (give them to ``assume=`` / ``instance(...)``)."""
        if isinstance(source, (bytes, bytearray, memoryview)):
            data = bytes(source)
        else:
            with open(source, "rb") as f:
                data = f.read()
        m = cls()
        m._imported = True
        _capi.check(_capi.lib().denox_hip_builder_import_onnx(m._h, data, len(data)))
        from ctypes import c_uint32, create_string_buffer
        for which, dst in (("input", m.inputs), ("output", m.outputs)):
            n = c_uint32()
            _capi.check(getattr(_capi.lib(), f"denox_hip_builder_{which}_count")(m._h, byref(n)))
            for i in range(n.value):
                name, ch = create_string_buffer(256), c_uint32()
                _capi.check(getattr(_capi.lib(), f"denox_hip_builder_{which}_info")(m._h, i, name, 256, byref(ch)))
                dst.append(Tensor(m, -1, name.value.decode(), None, None, ch.value))
        return m

    # ------------------------------------------------------------- symbols
    def sym(self, v: Union[int, str, Sym]) -> Sym:
        if isinstance(v, Sym):
            return v
        out = c_int64()
        if isinstance(v, str):
            _capi.check(_capi.lib().denox_hip_builder_sym_var(self._h, v.encode(), byref(out)))
            return Sym(self, out.value, v)
        _capi.check(_capi.lib().denox_hip_builder_sym_const(self._h, int(v), byref(out)))
        return Sym(self, out.value, str(int(v)))

    def _name(self, prefix: str) -> str:
        self._count += 1
        return f"{prefix}{self._count}"

    # ------------------------------------------------------------- layers
    def input(self, name: str, width, height, channels: int) -> Tensor:
        w, h = self.sym(width), self.sym(height)
        t = c_int()
        _capi.check(_capi.lib().denox_hip_builder_input(self._h, name.encode(), w.handle, h.handle, channels, byref(t)))
        ten = Tensor(self, t.value, name, w, h, channels)
        self.inputs.append(ten)
        return ten

    def conv2d(self, src: Tensor, weight, bias=None, stride=(1, 1), padding=(1, 1), dilation=(1, 1)) -> Tensor:
        """weight: [K][C][R][S] (ONNX / torch order); stride, padding, dilation as (y, x)."""
        w = _f16(weight)
        if w.ndim != 4 or w.shape[1] != src.channels:
            raise ValueError(f"conv2d weight {w.shape} does not fit {src.channels} input channels")
        K, C, R, S = w.shape
        b = None if bias is None else _f16(bias, (K,))
        t = c_int()
        _capi.check(_capi.lib().denox_hip_builder_conv2d(
            self._h, src.handle, K, C, R, S, w.ctypes.data, None if b is None else b.ctypes.data,
            stride[1], stride[0], padding[1], padding[0], dilation[1], dilation[0], byref(t)))
        ow = (src.width + (2 * padding[1] - dilation[1] * (S - 1) - 1)) // stride[1] + 1
        oh = (src.height + (2 * padding[0] - dilation[0] * (R - 1) - 1)) // stride[0] + 1
        out = Tensor(self, t.value, self._name("conv"), ow, oh, K)
        self._ops.append({"op": "conv2d", "src": src.name, "dst": out.name, "weight": w, "bias": b,
                          "stride": tuple(stride), "padding": tuple(padding)})
        return out

    def activation(self, src: Tensor, func: str = "relu", alpha: float = 0.0) -> Tensor:
        code = {"relu": 1, "leaky_relu": 2}[func]
        t = c_int()
        _capi.check(_capi.lib().denox_hip_builder_activation(self._h, src.handle, code, float(alpha), byref(t)))
        out = Tensor(self, t.value, self._name("act"), src.width, src.height, src.channels)
        self._ops.append({"op": "activation", "src": src.name, "dst": out.name, "func": "relu" if code == 1 else "leaky", "alpha": alpha})
        return out

    def relu(self, src: Tensor) -> Tensor:
        return self.activation(src, "relu")

    def upsample(self, src: Tensor, scale: int = 2) -> Tensor:
        t = c_int()
        _capi.check(_capi.lib().denox_hip_builder_upsample(self._h, src.handle, scale, byref(t)))
        out = Tensor(self, t.value, self._name("up"), src.width * scale, src.height * scale, src.channels)
        self._ops.append({"op": "upsample", "src": src.name, "dst": out.name, "factor": scale})
        return out

    def pool(self, src: Tensor, kernel=(2, 2), padding=(0, 0), stride=None, func: str = "max") -> Tensor:
        """``func`` is ``"max"`` or ``"avg"`` (the window's mean, summed in fp32 and rounded once)."""
        stride = tuple(kernel) if stride is None else tuple(stride)
        if func not in ("max", "avg"):
            raise ValueError(f"pool: unknown function {func!r}")
        t = c_int()
        entry = _capi.lib().denox_hip_builder_pool if func == "max" else _capi.lib().denox_hip_builder_avg_pool
        _capi.check(entry(self._h, src.handle, kernel[1], kernel[0], padding[1], padding[0], stride[1], stride[0], byref(t)))
        ow = (src.width + (2 * padding[1] - kernel[1])) // stride[1] + 1
        oh = (src.height + (2 * padding[0] - kernel[0])) // stride[0] + 1
        out = Tensor(self, t.value, self._name("pool"), ow, oh, src.channels)
        self._ops.append({"op": "pool", "src": src.name, "dst": out.name, "kernel": tuple(kernel), "func": func})
        return out

    def concat(self, a: Tensor, b: Tensor) -> Tensor:
        t = c_int()
        _capi.check(_capi.lib().denox_hip_builder_concat(self._h, a.handle, b.handle, byref(t)))
        out = Tensor(self, t.value, self._name("cat"), a.width, a.height, a.channels + b.channels)
        self._ops.append({"op": "concat", "src": [a.name, b.name], "dst": out.name})
        return out

    def pad(self, src: Tensor, left, right, top, bottom, mode: str = "replicate") -> Tensor:
        """mode "replicate" repeats the border pixels (F.pad mode="replicate"), "zero" fills with zeros (mode="constant")."""
        code = {"replicate": 0, "zero": 1}[mode]
        l, r, tp, bt = (self.sym(v) for v in (left, right, top, bottom))
        t = c_int()
        _capi.check(_capi.lib().denox_hip_builder_pad_mode(self._h, src.handle, l.handle, r.handle, tp.handle, bt.handle, code, byref(t)))
        out = Tensor(self, t.value, self._name("pad"), src.width + l + r, src.height + tp + bt, src.channels)
        self._ops.append({"op": "pad", "src": src.name, "dst": out.name, "left": l, "right": r, "top": tp, "bottom": bt, "mode": mode})
        return out

    def slice(self, src: Tensor, left, right, top, bottom) -> Tensor:
        """Half-open source ranges [left, right) x [top, bottom)."""
        l, r, tp, bt = (self.sym(v) for v in (left, right, top, bottom))
        t = c_int()
        _capi.check(_capi.lib().denox_hip_builder_slice(self._h, src.handle, l.handle, r.handle, tp.handle, bt.handle, byref(t)))
        out = Tensor(self, t.value, self._name("slice"), r - l, bt - tp, src.channels)
        self._ops.append({"op": "slice", "src": src.name, "dst": out.name, "left": l, "right": r, "top": tp, "bottom": bt})
        return out

    def output(self, src: Tensor, name: str = "output") -> None:
        _capi.check(_capi.lib().denox_hip_builder_output(self._h, src.handle, name.encode()))
        self.outputs.append(src)

    def pad_to_multiple(self, src: Tensor, alignment: int) -> Tensor:
        """Replicate-pad right/bottom so both extents become multiples of `alignment`
        (the alignment wrapper every pooled U-Net needs)."""
        pw = (alignment - src.width % alignment) % alignment
        ph = (alignment - src.height % alignment) % alignment
        return self.pad(src, 0, pw, 0, ph)

    # ------------------------------------------------------------- export for checkers
    def to_ops(self, extents: Dict[str, int]) -> List[dict]:
        """Layer records with symbolic pad / slice amounts evaluated at `extents`."""
        if getattr(self, "_imported", False):
            raise ValueError("a model imported from ONNX keeps no Python-side layer record")

        def ev(s):
            if not isinstance(s, Sym):
                return s
            return int(eval(s.text, {"__builtins__": {}}, dict(extents)))
        out = []
        for op in self._ops:
            o = dict(op)
            if o["op"] == "pad":
                for k in ("left", "right", "top", "bottom"):
                    o[k] = ev(o[k])
            elif o["op"] == "slice":
                l, r, t, b = (ev(o[k]) for k in ("left", "right", "top", "bottom"))
                o = {"op": "slice", "src": o["src"], "dst": o["dst"], "left": l, "top": t, "out_h": b - t, "out_w": r - l}
            out.append(o)
        return out
