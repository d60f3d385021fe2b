"""Device backend: ctypes binding of libxsmi355.so plus device arrays."""
from .capi import lib, XsmiError, init, is_initialized, device_info, synchronize, library_path, profiling, last_kernel_ms, set_option, get_option
from .array import DeviceArray, to_device, empty, zeros, Event, Workspace, PinnedArray, release_cached_memory, workspace_bytes
from .graph import StepGraph
from . import kernels
