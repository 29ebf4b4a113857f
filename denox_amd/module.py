"""Compile and run: the Python face of the compile / runtime C ABI.

``Module`` follows the reference's Python binding (bindings/python/denox:
``Module.compile(...)``, ``module(input)``; test harness test/__init__.py:45-101)
and its runtime objects (runtime/src/denox/runtime/instance.hpp:44-63).
"""
from __future__ import annotations

import ctypes
import enum
from ctypes import POINTER, byref, c_char_p, c_int64, c_size_t, c_uint32, c_uint64, c_void_p
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from . import _capi
from .graph import Model


class Layout(enum.IntEnum):
    Undefined = 0
    HWC = 1
    CHW = 2
    CHWC8 = 3


class Shape:
    """Extents of the (single) input: ints for static, strings for dynamic sizes."""

    def __init__(self, H="H", W="W", C=None):
        self.H, self.W, self.C = H, W, C


class Context:
    _default: Dict[int, "Context"] = {}

    def __init__(self, device: int = 0):
        h = c_void_p()
        _capi.check(_capi.lib().denox_hip_context_create(device, byref(h)))
        self._h, self.device = h, device

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            _capi.lib().denox_hip_context_destroy(h)

    @property
    def stream(self) -> int:
        s = c_void_p()
        _capi.check(_capi.lib().denox_hip_context_stream(self._h, byref(s)))
        return s.value or 0

    @classmethod
    def default(cls, device: int = 0) -> "Context":
        if device not in cls._default:
            cls._default[device] = Context(device)
        return cls._default[device]


def device_info(device: int = -1) -> dict:
    """CDNA4 limits table (device < 0) or the table refined by a present GPU."""
    d = _capi.DeviceInfo()
    _capi.check(_capi.lib().denox_hip_query_device_info(device, byref(d)))
    return {
        "name": d.name.decode(), "arch": d.arch.decode(), "subgroup_size": d.subgroup_size,
        "max_workgroup_invocations": d.max_workgroup_invocations, "max_workgroup_size": list(d.max_workgroup_size),
        "max_workgroup_count": list(d.max_workgroup_count), "max_shared_memory": d.max_shared_memory,
        "compute_units": d.compute_units, "xcd_count": d.xcd_count, "hbm_bytes": d.hbm_bytes,
        "hbm_bytes_per_second": d.hbm_bytes_per_second, "fp16_mfma_flops": d.fp16_mfma_flops,
        "matrix_shapes": [tuple(d.matrix_shapes[i]) for i in range(d.matrix_shape_count)], "from_device": bool(d.from_device),
    }


def _options(features: Optional[dict], input_layout, output_layout, assume: Optional[dict], conv_config: Optional[str], device: int):
    o = _capi.CompileOptions()
    _capi.lib().denox_hip_compile_options_default(byref(o))
    f = features or {}
    o.enable_conv_relu_fusion = int(f.get("conv_relu_fusion", True))
    o.enable_concat_conv_fusion = int(f.get("concat_conv_fusion", True))
    o.enable_upsample_fusion = int(f.get("upsample_fusion", True))
    o.enable_pool_fusion = int(f.get("pool_fusion", True))
    o.enable_pad_fusion = int(f.get("pad_fusion", True))
    o.enable_slice_fusion = int(f.get("slice_fusion", True))
    o.enable_alternating_traversal = int(f.get("alternating_traversal", True))
    o.enable_upsample_fold = int(f.get("upsample_fold", True))
    o.enable_implicit_concat = int(f.get("implicit_concat", True))
    o.enable_conv_conv_fusion = int(f.get("conv_conv_fusion", True))
    o.enable_blocked_layout = int(f.get("blocked_layout", True))
    o.layout_preference = int(f.get("layout_preference", 0))
    o.input_format = int(input_layout)
    o.output_format = int(output_layout)
    keep = []
    if assume:
        names = (c_char_p * len(assume))(*[k.encode() for k in assume])
        vals = (c_int64 * len(assume))(*[int(v) for v in assume.values()])
        o.assumption_count = len(assume)
        o.assumption_names = ctypes.cast(names, POINTER(c_char_p))
        o.assumption_values = ctypes.cast(vals, POINTER(c_int64))
        keep += [names, vals]
    if conv_config:
        cc = conv_config.encode()
        o.force_conv_config = cc
        keep.append(cc)
    o.device = device
    return o, keep


def compile_model(model: Model, *, features: Optional[dict] = None, input_layout=Layout.HWC, output_layout=Layout.HWC,
                  assume: Optional[dict] = None, conv_config: Optional[str] = None, db: Optional["Db"] = None,
                  device: int = -1) -> bytes:
    """denox::compile: graph -> serialised model (compiler/src/denox/compiler/compile.cpp:21-61)."""
    o, _keep = _options(features, input_layout or Layout.HWC, output_layout or Layout.HWC, assume, conv_config, device)
    blob, size = c_void_p(), c_size_t()
    _capi.check(_capi.lib().denox_hip_compile(model._h, byref(o), db._h if db is not None else None, byref(blob), byref(size)))
    try:
        return ctypes.string_at(blob.value, size.value)
    finally:
        _capi.lib().denox_hip_free(blob)


def describe(dnx: bytes, **extents: int) -> dict:
    """Decode a compiled model (no GPU needed), symbolic quantities evaluated at `extents`."""
    import json
    names = (c_char_p * len(extents))(*[k.encode() for k in extents])
    vals = (c_int64 * len(extents))(*[int(v) for v in extents.values()])
    p = c_void_p()
    _capi.check(_capi.lib().denox_hip_dnx_describe(dnx, len(dnx), names, vals, len(extents), byref(p)))
    try:
        return json.loads(ctypes.string_at(p.value).decode())
    finally:
        _capi.lib().denox_hip_free(p)


def conv_config_names() -> List[str]:
    """Every name `conv_config=` accepts."""
    return _capi.lib().denox_hip_conv_config_names().decode().split(",")


def last_compile_report() -> str:
    return (_capi.lib().denox_hip_last_compile_report() or b"").decode()


class Db:
    """Dispatch timing table (database/src/denox/db/Db.hpp:15-69)."""

    def __init__(self, path: str):
        h = c_void_p()
        _capi.check(_capi.lib().denox_hip_db_open(path.encode(), byref(h)))
        self._h, self.path = h, path

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            _capi.lib().denox_hip_db_close(h)

    def __len__(self) -> int:
        n = c_uint64()
        _capi.check(_capi.lib().denox_hip_db_row_count(self._h, byref(n)))
        return n.value

    def populate(self, model: Model, **kw) -> int:
        o, _keep = _options(kw.get("features"), kw.get("input_layout", Layout.HWC), kw.get("output_layout", Layout.HWC),
                            kw.get("assume"), kw.get("conv_config"), kw.get("device", -1))
        o.populate_compile_kernels = int(kw.get("compile_kernels", True))
        o.kernel_shard_index, o.kernel_shard_count = kw.get("shard", (0, 1))
        n = c_uint64()
        _capi.check(_capi.lib().denox_hip_db_populate(self._h, model._h, byref(o), byref(n)))
        return n.value

    def bench(self, ctx: Optional[Context] = None, min_samples=10, max_relative_error=0.05, max_samples=200, save_progress=True, filter=None) -> dict:
        ctx = ctx or Context.default()
        o = _capi.DbBenchOptions()
        _capi.lib().denox_hip_db_bench_options_default(byref(o))
        o.min_samples, o.max_relative_error, o.max_samples, o.save_progress = min_samples, max_relative_error, max_samples, int(save_progress)
        f = filter.encode() if filter else None
        o.filter = f
        r = _capi.DbBenchResult()
        _capi.check(_capi.lib().denox_hip_db_bench(self._h, ctx._h, byref(o), byref(r)))
        return {"benchmarked": r.benchmarked, "converged": r.converged, "skipped": r.skipped, "failed": r.failed}

    def add_sample(self, row: int, latency_ns: float) -> None:
        _capi.check(_capi.lib().denox_hip_db_add_sample(self._h, row, float(latency_ns)))

    def row_stats(self, row: int) -> Tuple[int, float, float]:
        n, m, s = c_uint64(), ctypes.c_double(), ctypes.c_double()
        _capi.check(_capi.lib().denox_hip_db_row_stats(self._h, row, byref(n), byref(m), byref(s)))
        return n.value, m.value, s.value

    def writeback(self) -> None:
        _capi.check(_capi.lib().denox_hip_db_writeback(self._h))

    def dump_csv(self) -> str:
        p = c_void_p()
        _capi.check(_capi.lib().denox_hip_db_dump_csv(self._h, byref(p)))
        try:
            return ctypes.string_at(p.value).decode()
        finally:
            _capi.lib().denox_hip_free(p)


class RuntimeModel:
    """runtime::Model (runtime/src/denox/runtime/model.hpp:107-170)."""

    def __init__(self, dnx: bytes, ctx: Optional[Context] = None):
        self.ctx = ctx or Context.default()
        h = c_void_p()
        self._dnx = dnx
        _capi.check(_capi.lib().denox_hip_model_create(self.ctx._h, dnx, len(dnx), byref(h)))
        self._h = h

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            _capi.lib().denox_hip_model_destroy(h)

    @property
    def dispatch_count(self) -> int:
        n = c_uint32()
        _capi.check(_capi.lib().denox_hip_model_dispatch_count(self._h, byref(n)))
        return n.value


class Instance:
    """runtime::Instance (runtime/src/denox/runtime/instance.hpp:44-63)."""

    def __init__(self, model: RuntimeModel, **extents: int):
        self.model = model
        names = (c_char_p * len(extents))(*[k.encode() for k in extents])
        vals = (c_int64 * len(extents))(*[int(v) for v in extents.values()])
        h = c_void_p()
        _capi.check(_capi.lib().denox_hip_instance_create(model._h, names, vals, len(extents), byref(h)))
        self._h = h

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            _capi.lib().denox_hip_instance_destroy(h)

    def _count(self, fn) -> int:
        n = c_uint32()
        _capi.check(fn(self._h, byref(n)))
        return n.value

    @property
    def input_count(self) -> int:
        return self._count(_capi.lib().denox_hip_instance_input_count)

    @property
    def output_count(self) -> int:
        return self._count(_capi.lib().denox_hip_instance_output_count)

    def _desc(self, fn, i) -> dict:
        d = _capi.TensorDesc()
        _capi.check(fn(self._h, i, byref(d)))
        return {"width": d.width, "height": d.height, "channels": d.channels, "layout": Layout(d.format), "dtype": d.dtype,
                "byte_size": d.byte_size, "name": d.name.decode()}

    def input_desc(self, i=0) -> dict:
        return self._desc(_capi.lib().denox_hip_instance_input_desc, i)

    def output_desc(self, i=0) -> dict:
        return self._desc(_capi.lib().denox_hip_instance_output_desc, i)

    @staticmethod
    def _np_shape(d: dict):
        if d["layout"] == Layout.CHW:
            return (d["channels"], d["height"], d["width"])
        if d["layout"] == Layout.CHWC8:
            return (d["channels"] // 8, d["height"], d["width"], 8)
        return (d["height"], d["width"], d["channels"])

    def infer(self, *inputs: np.ndarray) -> List[np.ndarray]:
        """Blocking inference on host arrays (float16, in each tensor's declared layout)."""
        if len(inputs) != self.input_count:
            raise ValueError(f"model takes {self.input_count} inputs")
        ins = []
        for i, a in enumerate(inputs):
            d = self.input_desc(i)
            arr = np.ascontiguousarray(a, dtype=np.float16)
            if arr.nbytes != d["byte_size"]:
                raise ValueError(f"input {i}: expected {d['byte_size']} bytes ({self._np_shape(d)} float16), got {arr.nbytes}")
            ins.append(arr)
        outs = [np.empty(self._np_shape(self.output_desc(i)), np.float16) for i in range(self.output_count)]
        pin = (c_void_p * len(ins))(*[a.ctypes.data for a in ins])
        pout = (c_void_p * len(outs))(*[a.ctypes.data for a in outs])
        _capi.check(_capi.lib().denox_hip_instance_infer(self._h, pin, pout))
        return outs

    def infer_many(self, frames: Sequence[Sequence[np.ndarray]], outputs: Optional[Sequence[Sequence[np.ndarray]]] = None) -> List[List[np.ndarray]]:
        """Blocking inference on a sequence of frames (each a sequence of host arrays, one per model input) with uploads,
        dispatches and downloads of neighbouring frames overlapped.  The overlap needs page-locked arrays (`pinned_empty`)
        on both sides; `outputs` may supply them, else pageable arrays are allocated."""
        nin, nout = self.input_count, self.output_count
        ins = []
        for f, frame in enumerate(frames):
            if len(frame) != nin:
                raise ValueError(f"frame {f}: model takes {nin} inputs")
            for i, a in enumerate(frame):
                arr = a if (isinstance(a, np.ndarray) and a.dtype == np.float16 and a.flags.c_contiguous) else np.ascontiguousarray(a, dtype=np.float16)
                d = self.input_desc(i)
                if arr.nbytes != d["byte_size"]:
                    raise ValueError(f"frame {f} input {i}: expected {d['byte_size']} bytes, got {arr.nbytes}")
                ins.append(arr)
        if outputs is None:
            outs = [[np.empty(self._np_shape(self.output_desc(i)), np.float16) for i in range(nout)] for _ in frames]
        else:
            outs = [list(o) for o in outputs]
            for f, o in enumerate(outs):
                if len(o) != nout or any(a.dtype != np.float16 or not a.flags.c_contiguous or a.nbytes != self.output_desc(i)["byte_size"] for i, a in enumerate(o)):
                    raise ValueError(f"frame {f}: outputs must be contiguous float16 arrays of the model's output sizes")
        if len(outs) != len(frames):
            raise ValueError("one set of outputs per frame expected")
        pin = (c_void_p * max(len(ins), 1))(*[a.ctypes.data for a in ins])
        flat = [a for o in outs for a in o]
        pout = (c_void_p * max(len(flat), 1))(*[a.ctypes.data for a in flat])
        _capi.check(_capi.lib().denox_hip_instance_infer_many(self._h, len(frames), pin, pout))
        return outs

    def infer_device(self, inputs: Optional[Sequence[int]] = None, outputs: Optional[Sequence[int]] = None) -> None:
        """Asynchronous inference on device addresses (ints); None = the instance's own tensors."""
        pin = (c_void_p * self.input_count)(*inputs) if inputs is not None else None
        pout = (c_void_p * self.output_count)(*outputs) if outputs is not None else None
        _capi.check(_capi.lib().denox_hip_instance_infer_device(self._h, pin, pout))

    def infer_device_static(self, inputs: Optional[Sequence[int]] = None, outputs: Optional[Sequence[int]] = None) -> None:
        """`infer_device` without any device allocation: plain launches, intermediates in the library's static scratch array."""
        pin = (c_void_p * self.input_count)(*inputs) if inputs is not None else None
        pout = (c_void_p * self.output_count)(*outputs) if outputs is not None else None
        _capi.check(_capi.lib().denox_hip_instance_infer_device_static(self._h, pin, pout))

    def synchronize(self) -> None:
        _capi.check(_capi.lib().denox_hip_instance_synchronize(self._h))

    def input_device_ptr(self, i=0) -> int:
        p = c_void_p()
        _capi.check(_capi.lib().denox_hip_instance_input_device_ptr(self._h, i, byref(p)))
        return p.value

    def output_device_ptr(self, i=0) -> int:
        p = c_void_p()
        _capi.check(_capi.lib().denox_hip_instance_output_device_ptr(self._h, i, byref(p)))
        return p.value

    @property
    def device_bytes(self) -> int:
        n = c_uint64()
        _capi.check(_capi.lib().denox_hip_instance_device_bytes(self._h, byref(n)))
        return n.value

    def bench(self, warmup: int = 10) -> List[dict]:
        """Per-dispatch latency, GB/s and TFLOP/s (Instance::bench().report(), instance.cpp:432-704)."""
        cap = self.model.dispatch_count
        arr = (_capi.Timing * max(cap, 1))()
        n = c_uint32()
        _capi.check(_capi.lib().denox_hip_instance_bench(self._h, warmup, arr, cap, byref(n)))
        out = []
        for t in arr[:min(n.value, cap)]:
            ms = float(t.latency_ms)
            out.append({"name": t.name.decode(), "input": t.input.decode(), "output": t.output.decode(),
                        "memory_reads": t.memory_reads, "memory_writes": t.memory_writes, "flops": t.flops, "latency_ms": ms,
                        "GBps": (t.memory_reads + t.memory_writes) / ms * 1e-6 if ms > 0 else 0.0,
                        "TFLOPs": t.flops / ms * 1e-9 if ms > 0 else 0.0})
        return out

    def bench_in_frame(self, dispatch: int, frames: int = 50, warmup: int = 5) -> float:
        """Milliseconds of dispatch `dispatch` (an index into bench()'s list) inside whole inferences: events around that
        dispatch only, mean over `frames` frames."""
        ms = ctypes.c_float()
        _capi.check(_capi.lib().denox_hip_instance_bench_in_frame(self._h, dispatch, frames, warmup, byref(ms)))
        return float(ms.value)


class _PinnedBlock:
    """Owner of one hipHostMalloc allocation; the arrays made from it keep it alive through their `base` chain."""

    def __init__(self, nbytes: int):
        p = c_void_p()
        _capi.check(_capi.lib().denox_hip_host_alloc(max(int(nbytes), 1), byref(p)))
        self.ptr, self.nbytes = p.value, int(nbytes)
        self.buffer = (ctypes.c_uint8 * max(self.nbytes, 1)).from_address(self.ptr)
        self.buffer._owner = self  # the ctypes view is what numpy holds on to

    def __del__(self):
        if getattr(self, "ptr", None):
            _capi.lib().denox_hip_host_free(self.ptr)
            self.ptr = None


def pinned_empty(shape, dtype=np.float16) -> np.ndarray:
    """An uninitialised array in page-locked host memory (denox_hip_host_alloc), from and to which `Instance.infer_many`
    copies at bus speed and concurrently with the dispatches.  Needs a GPU."""
    dt = np.dtype(dtype)
    n = int(np.prod(shape)) * dt.itemsize
    block = _PinnedBlock(n)
    return np.frombuffer(block.buffer, dtype=dt, count=int(np.prod(shape))).reshape(shape)


def report(timings: List[dict]) -> str:
    lines, total = [], 0.0
    for t in timings:
        total += t["latency_ms"]
        lines.append(f"{t['input']:>18} --{t['name']:-<36}> {t['output']:<12}: {t['latency_ms']:.4f}ms ({t['GBps']:.0f}GB/s, {t['TFLOPs']:.1f}TFLOPS)")
    lines.append(f"total: {total:.4f}ms")
    return "\n".join(lines)


class Module:
    """Compiled network bound to a device: ``Module.compile(model, ...)`` then ``module(x)``."""

    def __init__(self, dnx: bytes, ctx: Optional[Context] = None):
        self.dnx = dnx
        self.runtime_model = RuntimeModel(dnx, ctx)
        self._instances: Dict[Tuple[Tuple[str, int], ...], Instance] = {}

    @staticmethod
    def compile(model: Model, input_shape: Optional[Shape] = None, input_layout=Layout.Undefined, output_layout=Layout.Undefined,
                ctx: Optional[Context] = None, **kw) -> "Module":
        m = Module(compile_model(model, input_layout=input_layout, output_layout=output_layout, **kw), ctx)
        m._input_shape = input_shape or Shape()
        m._input_layout = Layout(input_layout)
        return m

    @staticmethod
    def load(dnx: bytes, ctx: Optional[Context] = None) -> "Module":
        return Module(dnx, ctx)

    def save(self, path: str) -> None:
        with open(path, "wb") as f:
            f.write(self.dnx)

    def instance(self, **extents: int) -> Instance:
        key = tuple(sorted(extents.items()))
        if key not in self._instances:
            self._instances[key] = Instance(self.runtime_model, **extents)
        return self._instances[key]

    def __call__(self, x: np.ndarray, **extents: int) -> np.ndarray:
        """x: float16 array in the model's input layout -- (H, W, C) for HWC, (C, H, W) for CHW,
        (C/8, H, W, 8) for CHWC8.  Dynamic extents named by the compile-time Shape are read off x."""
        x = np.asarray(x)
        if not extents:
            shp = getattr(self, "_input_shape", Shape())
            lay = getattr(self, "_input_layout", Layout.HWC)
            h_ax, w_ax = (0, 1) if lay in (Layout.HWC, Layout.Undefined) else (1, 2)
            if isinstance(shp.H, str):
                extents[shp.H] = x.shape[h_ax]
            if isinstance(shp.W, str):
                extents[shp.W] = x.shape[w_ax]
        return self.instance(**extents).infer(x)[0]
