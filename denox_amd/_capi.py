"""ctypes binding of ``include/denox_hip.h`` (libdenox_hip.so).

The library is the product; this module only declares its entry points.  It
raises ``ImportError``-like ``DenoxHipError`` loudly when the shared library
has not been built -- there is no Python or CPU fallback for any operation.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import (POINTER, Structure, byref, c_char, c_char_p, c_double, c_float, c_int, c_int32, c_int64, c_size_t,
                    c_uint16, c_uint32, c_uint64, c_void_p)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libdenox_hip.so")
CSRC_DIR = os.path.join(_HERE, "csrc")

STATUS_NAMES = {0: "OK", 1: "INVALID_ARGUMENT", 2: "INVALID_MODEL", 3: "HIP_ERROR", 4: "COMPILE_ERROR", 5: "UNSUPPORTED",
                6: "IO_ERROR", 7: "INTERNAL"}


class DenoxHipError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"[{STATUS_NAMES.get(status, status)}] {message}")
        self.status = status


class DeviceInfo(Structure):
    _fields_ = [("name", c_char * 128), ("arch", c_char * 32), ("subgroup_size", c_uint32),
                ("max_workgroup_invocations", c_uint32), ("max_workgroup_size", c_uint32 * 3),
                ("max_workgroup_count", c_uint32 * 3), ("max_shared_memory", c_uint32), ("compute_units", c_uint32),
                ("xcd_count", c_uint32), ("hbm_bytes", c_uint64), ("hbm_bytes_per_second", c_double),
                ("fp16_mfma_flops", c_double), ("matrix_shape_count", c_uint32), ("matrix_shapes", (c_uint32 * 3) * 4),
                ("from_device", c_int32)]


class CompileOptions(Structure):
    _fields_ = [("enable_conv_relu_fusion", c_int32), ("enable_concat_conv_fusion", c_int32),
                ("enable_upsample_fusion", c_int32), ("enable_pool_fusion", c_int32), ("enable_pad_fusion", c_int32),
                ("enable_slice_fusion", c_int32), ("enable_alternating_traversal", c_int32), ("enable_upsample_fold", c_int32), ("enable_implicit_concat", c_int32), ("input_format", c_int32),
                ("output_format", c_int32), ("assumption_count", c_uint32), ("assumption_names", POINTER(c_char_p)),
                ("assumption_values", POINTER(c_int64)), ("force_conv_config", c_char_p), ("device", c_int32),
                ("populate_compile_kernels", c_int32), ("kernel_shard_index", c_uint32), ("kernel_shard_count", c_uint32),
                ("enable_conv_conv_fusion", c_int32), ("enable_blocked_layout", c_int32), ("layout_preference", c_int32)]


class DbBenchOptions(Structure):
    _fields_ = [("min_samples", c_uint32), ("max_relative_error", c_double), ("max_samples", c_uint32),
                ("save_progress", c_int32), ("filter", c_char_p)]


class DbBenchResult(Structure):
    _fields_ = [("benchmarked", c_uint64), ("converged", c_uint64), ("skipped", c_uint64), ("failed", c_uint64)]


class TensorDesc(Structure):
    _fields_ = [("width", c_int64), ("height", c_int64), ("channels", c_int64), ("format", c_int32), ("dtype", c_int32),
                ("byte_size", c_uint64), ("name", c_char * 64)]


class Timing(Structure):
    _fields_ = [("name", c_char * 64), ("input", c_char * 48), ("output", c_char * 48), ("memory_reads", c_uint64),
                ("memory_writes", c_uint64), ("flops", c_uint64), ("latency_ms", c_float)]


# name -> (restype, argtypes); every function include/denox_hip.h declares
SIGNATURES = {
    "denox_hip_last_error": (c_char_p, []),
    "denox_hip_conv_config_names": (c_char_p, []),
    "denox_hip_version": (c_char_p, []),
    "denox_hip_set_kernel_paths": (c_int, [c_char_p, c_char_p]),
    "denox_hip_query_device_info": (c_int, [c_int, POINTER(DeviceInfo)]),
    "denox_hip_builder_create": (c_int, [POINTER(c_void_p)]),
    "denox_hip_builder_destroy": (None, [c_void_p]),
    "denox_hip_builder_sym_const": (c_int, [c_void_p, c_int64, POINTER(c_int64)]),
    "denox_hip_builder_sym_var": (c_int, [c_void_p, c_char_p, POINTER(c_int64)]),
    "denox_hip_builder_sym_op": (c_int, [c_void_p, c_int, c_int64, c_int64, POINTER(c_int64)]),
    "denox_hip_builder_input": (c_int, [c_void_p, c_char_p, c_int64, c_int64, c_uint32, POINTER(c_int)]),
    "denox_hip_builder_conv2d": (c_int, [c_void_p, c_int, c_uint32, c_uint32, c_uint32, c_uint32, c_void_p, c_void_p,
                                         c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, POINTER(c_int)]),
    "denox_hip_builder_activation": (c_int, [c_void_p, c_int, c_int, c_float, POINTER(c_int)]),
    "denox_hip_builder_upsample": (c_int, [c_void_p, c_int, c_uint32, POINTER(c_int)]),
    "denox_hip_builder_pool": (c_int, [c_void_p, c_int, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, POINTER(c_int)]),
    "denox_hip_builder_avg_pool": (c_int, [c_void_p, c_int, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, POINTER(c_int)]),
    "denox_hip_builder_concat": (c_int, [c_void_p, c_int, c_int, POINTER(c_int)]),
    "denox_hip_builder_pad": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, POINTER(c_int)]),
    "denox_hip_builder_pad_mode": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_int32, POINTER(c_int)]),
    "denox_hip_builder_slice": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, POINTER(c_int)]),
    "denox_hip_builder_output": (c_int, [c_void_p, c_int, c_char_p]),
    "denox_hip_builder_import_onnx": (c_int, [c_void_p, c_char_p, c_size_t]),
    "denox_hip_builder_input_count": (c_int, [c_void_p, POINTER(c_uint32)]),
    "denox_hip_builder_output_count": (c_int, [c_void_p, POINTER(c_uint32)]),
    "denox_hip_builder_input_info": (c_int, [c_void_p, c_uint32, c_char_p, c_size_t, POINTER(c_uint32)]),
    "denox_hip_builder_output_info": (c_int, [c_void_p, c_uint32, c_char_p, c_size_t, POINTER(c_uint32)]),
    "denox_hip_compile_options_default": (None, [POINTER(CompileOptions)]),
    "denox_hip_compile": (c_int, [c_void_p, POINTER(CompileOptions), c_void_p, POINTER(c_void_p), POINTER(c_size_t)]),
    "denox_hip_last_compile_report": (c_char_p, []),
    "denox_hip_free": (None, [c_void_p]),
    "denox_hip_dnx_describe": (c_int, [c_void_p, c_size_t, POINTER(c_char_p), POINTER(c_int64), c_uint32, POINTER(c_void_p)]),
    "denox_hip_min_cost_subgraph": (c_int, [c_uint32, c_void_p, c_uint32, c_void_p, c_void_p, c_void_p, c_void_p, c_uint32, c_void_p,
                                            c_void_p, POINTER(c_uint32), POINTER(c_double)]),
    "denox_hip_db_open": (c_int, [c_char_p, POINTER(c_void_p)]),
    "denox_hip_db_close": (None, [c_void_p]),
    "denox_hip_db_row_count": (c_int, [c_void_p, POINTER(c_uint64)]),
    "denox_hip_db_populate": (c_int, [c_void_p, c_void_p, POINTER(CompileOptions), POINTER(c_uint64)]),
    "denox_hip_db_bench_options_default": (None, [POINTER(DbBenchOptions)]),
    "denox_hip_db_bench": (c_int, [c_void_p, c_void_p, POINTER(DbBenchOptions), POINTER(DbBenchResult)]),
    "denox_hip_db_add_sample": (c_int, [c_void_p, c_uint64, c_double]),
    "denox_hip_db_row_stats": (c_int, [c_void_p, c_uint64, POINTER(c_uint64), POINTER(c_double), POINTER(c_double)]),
    "denox_hip_db_writeback": (c_int, [c_void_p]),
    "denox_hip_db_dump_csv": (c_int, [c_void_p, POINTER(c_void_p)]),
    "denox_hip_context_create": (c_int, [c_int, POINTER(c_void_p)]),
    "denox_hip_context_destroy": (None, [c_void_p]),
    "denox_hip_context_stream": (c_int, [c_void_p, POINTER(c_void_p)]),
    "denox_hip_model_create": (c_int, [c_void_p, c_void_p, c_size_t, POINTER(c_void_p)]),
    "denox_hip_model_destroy": (None, [c_void_p]),
    "denox_hip_model_dispatch_count": (c_int, [c_void_p, POINTER(c_uint32)]),
    "denox_hip_instance_create": (c_int, [c_void_p, POINTER(c_char_p), POINTER(c_int64), c_uint32, POINTER(c_void_p)]),
    "denox_hip_instance_destroy": (None, [c_void_p]),
    "denox_hip_instance_input_count": (c_int, [c_void_p, POINTER(c_uint32)]),
    "denox_hip_instance_output_count": (c_int, [c_void_p, POINTER(c_uint32)]),
    "denox_hip_instance_input_desc": (c_int, [c_void_p, c_uint32, POINTER(TensorDesc)]),
    "denox_hip_instance_output_desc": (c_int, [c_void_p, c_uint32, POINTER(TensorDesc)]),
    "denox_hip_instance_infer": (c_int, [c_void_p, POINTER(c_void_p), POINTER(c_void_p)]),
    "denox_hip_instance_infer_device": (c_int, [c_void_p, POINTER(c_void_p), POINTER(c_void_p)]),
    "denox_hip_instance_infer_many": (c_int, [c_void_p, c_uint32, POINTER(c_void_p), POINTER(c_void_p)]),
    "denox_hip_host_alloc": (c_int, [c_size_t, POINTER(c_void_p)]),
    "denox_hip_host_free": (None, [c_void_p]),
    "denox_hip_instance_infer_device_static": (c_int, [c_void_p, POINTER(c_void_p), POINTER(c_void_p)]),
    "denox_hip_instance_synchronize": (c_int, [c_void_p]),
    "denox_hip_instance_input_device_ptr": (c_int, [c_void_p, c_uint32, POINTER(c_void_p)]),
    "denox_hip_instance_output_device_ptr": (c_int, [c_void_p, c_uint32, POINTER(c_void_p)]),
    "denox_hip_instance_bench": (c_int, [c_void_p, c_uint32, POINTER(Timing), c_uint32, POINTER(c_uint32)]),
    "denox_hip_instance_bench_in_frame": (c_int, [c_void_p, c_uint32, c_uint32, c_uint32, POINTER(c_float)]),
    "denox_hip_instance_device_bytes": (c_int, [c_void_p, POINTER(c_uint64)]),
}

_lib = None


def build(force: bool = False) -> str:
    """Compile libdenox_hip.so in-tree (host C++ only; kernels are built by hiprtc at model-compile time)."""
    import subprocess
    cmd = ["make", "-C", CSRC_DIR, "-j8"]
    if force:
        cmd.append("-B")
    subprocess.check_call(cmd, stdout=subprocess.DEVNULL)
    return LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise DenoxHipError(6, f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                                   f"or `make -C {CSRC_DIR}`; there is no fallback implementation")
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(status: int) -> None:
    if status != 0:
        msg = lib().denox_hip_last_error()
        raise DenoxHipError(status, msg.decode("utf-8", "replace") if msg else "")
