"""morok_amd: MI355X (gfx950) device backend for morok behind its Device boundary.

Importing the package loads morok_amd/libmorok_hip.so; nothing here computes on the CPU.
"""
from ._ffi import MorokHipError, lib, declared_symbols  # noqa: F401
from .device import (  # noqa: F401
    Buffer, CompiledSpec, Device, Event, ExecutionPlan, HardwareQueue, Kernel, Program, ProgramSpec, TimelineSignal,
    benchmark_kernel, benchmark_kernel_with_cutoff, cache_key, compile_spec, device_count, kernel_cache_clear, kernel_cache_size, parse_device,
    time_each_launch, time_launches,
)
from . import ops  # noqa: F401
from . import uop  # noqa: F401
from . import sched  # noqa: F401
