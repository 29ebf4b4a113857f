"""denox_amd: MI355X (gfx950) execution backend for denox-style CNN dispatch schedules.

Host side of ``libdenox_hip.so`` (C ABI in ``include/denox_hip.h``):

* ``Model``  -- graph builder (reference: compiler::Model);
* ``compile_model`` / ``Module`` -- compile to a dispatch list and run it
  (reference: denox::compile, runtime::Model / Instance);
* ``Db`` -- dispatch timing table that drives schedule selection
  (reference: denox::Db, runtime::Db::bench);
* ``device_info`` -- CDNA4 limits (reference: DeviceInfo).

Everything executes in the native library and its HIP kernels; nothing here
computes on the CPU.
"""
from ._capi import DenoxHipError, LIB_PATH, build  # noqa: F401
from .graph import Model, Sym, Tensor  # noqa: F401
from .module import (Context, Db, Instance, Layout, Module, RuntimeModel, Shape, compile_model, describe, device_info, pinned_empty,  # noqa: F401
                     last_compile_report, report, conv_config_names)
