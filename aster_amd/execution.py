"""GPU execution runtime over the C-ABI: buffers, events, streams, code-object
modules, and `execute_hsaco`.

Same API as the reference's python/aster/execution/core.py (RAII wrappers
:59-345, array roles :347-376, `MemoryManager` :384-469, kernel-argument packing
:472-554, `execute_hsaco` :605-717) with the nanobind `hip_*` calls replaced by
the `aster_rt_*` entry points of libastergemm.so.  Any code object built with
`hipcc --genco --offload-arch=gfx950` whose kernels are `extern "C" __global__`
can be launched through it.
"""

from __future__ import annotations

import ctypes
import dataclasses
from typing import Any, Callable, List, Optional, Tuple

from . import _capi


def _rt():
    return _capi.load()


_initialised = False


def hip_init() -> None:
    global _initialised
    if not _initialised:
        _capi.check(_rt().aster_rt_init())
        _initialised = True


class GpuBuffer:
    """Device allocation that frees itself; copies are synchronous."""

    def __init__(self, size_bytes: int) -> None:
        hip_init()
        self._size = int(size_bytes)
        p = ctypes.c_void_p()
        _capi.check(_rt().aster_rt_malloc(ctypes.byref(p), max(self._size, 1)))
        self._ptr: Optional[int] = p.value

    def __del__(self) -> None:
        try:
            self.free()
        except Exception:
            pass

    def free(self) -> None:
        if getattr(self, "_ptr", None) is not None:
            ptr, self._ptr = self._ptr, None
            _capi.check(_rt().aster_rt_free(ctypes.c_void_p(ptr)))

    @property
    def ptr(self) -> ctypes.c_void_p:
        return ctypes.c_void_p(self._ptr)

    @property
    def ptr_value(self) -> int:
        return self._ptr

    @property
    def size_bytes(self) -> int:
        return self._size

    @staticmethod
    def _check_array(array, size: int):
        import numpy as np

        if not isinstance(array, np.ndarray):
            raise TypeError(f"expected numpy array, got {type(array)}")
        if array.nbytes > size:
            raise ValueError(f"array of {array.nbytes} bytes exceeds buffer of {size} bytes")
        if not array.flags["C_CONTIGUOUS"]:
            raise ValueError("array must be C-contiguous")

    def copy_from_host(self, array) -> None:
        self._check_array(array, self._size)
        if array.nbytes:
            _capi.check(_rt().aster_rt_memcpy_h2d(self.ptr, array.ctypes.data, array.nbytes))

    def copy_to_host(self, array) -> None:
        self._check_array(array, self._size)
        if array.nbytes:
            _capi.check(_rt().aster_rt_memcpy_d2h(array.ctypes.data, self.ptr, array.nbytes))


class GpuStream:
    def __init__(self) -> None:
        hip_init()
        h = ctypes.c_void_p()
        _capi.check(_rt().aster_rt_stream_create(ctypes.byref(h)))
        self._h: Optional[int] = h.value

    def __del__(self) -> None:
        try:
            self.destroy()
        except Exception:
            pass

    def destroy(self) -> None:
        if getattr(self, "_h", None) is not None:
            h, self._h = self._h, None
            _capi.check(_rt().aster_rt_stream_destroy(ctypes.c_void_p(h)))

    def synchronize(self) -> None:
        _capi.check(_rt().aster_rt_stream_synchronize(ctypes.c_void_p(self._h)))

    @property
    def handle(self) -> ctypes.c_void_p:
        return ctypes.c_void_p(self._h)


class GpuEvent:
    def __init__(self) -> None:
        hip_init()
        h = ctypes.c_void_p()
        _capi.check(_rt().aster_rt_event_create(ctypes.byref(h)))
        self._h: Optional[int] = h.value

    def __del__(self) -> None:
        try:
            self.destroy()
        except Exception:
            pass

    def destroy(self) -> None:
        if getattr(self, "_h", None) is not None:
            h, self._h = self._h, None
            _capi.check(_rt().aster_rt_event_destroy(ctypes.c_void_p(h)))

    def record(self, stream: Optional[GpuStream] = None) -> None:
        s = stream.handle if stream is not None else None
        _capi.check(_rt().aster_rt_event_record(ctypes.c_void_p(self._h), s))

    def synchronize(self) -> None:
        _capi.check(_rt().aster_rt_event_synchronize(ctypes.c_void_p(self._h)))

    def elapsed_ms(self, start: "GpuEvent") -> float:
        ms = ctypes.c_float()
        _capi.check(_rt().aster_rt_event_elapsed_ms(ctypes.c_void_p(start._h),
                                                    ctypes.c_void_p(self._h), ctypes.byref(ms)))
        return float(ms.value)

    def elapsed_ns(self, start: "GpuEvent") -> int:
        return int(self.elapsed_ms(start) * 1e6)

    @property
    def handle(self) -> ctypes.c_void_p:
        return ctypes.c_void_p(self._h)


@dataclasses.dataclass
class InputArray:
    """Copied host -> device before the first launch only."""
    array: Any


@dataclasses.dataclass
class OutputArray:
    """Allocated on the device, not uploaded; copied back after iteration 0."""
    array: Any


@dataclasses.dataclass
class InOutArray:
    """Uploaded before the first launch and copied back after iteration 0."""
    array: Any


class MemoryManager:
    """Pairs numpy arrays (by identity) with device buffers."""

    def __init__(self) -> None:
        self._buffers: dict = {}  # id(array) -> (GpuBuffer, array); the array ref pins the id

    def register(self, array, upload: bool = True) -> GpuBuffer:
        import numpy as np

        if not isinstance(array, np.ndarray):
            raise TypeError(f"expected numpy array, got {type(array)}")
        hit = self._buffers.get(id(array))
        if hit is not None:
            return hit[0]
        buf = GpuBuffer(array.nbytes)
        if upload:
            buf.copy_from_host(array)
        self._buffers[id(array)] = (buf, array)
        return buf

    def _get_entry(self, array):
        try:
            return self._buffers[id(array)]
        except KeyError:
            raise KeyError("array is not registered with this MemoryManager") from None

    def sync_to_gpu(self, array) -> None:
        self._get_entry(array)[0].copy_from_host(array)

    def sync_from_gpu(self, array) -> None:
        self._get_entry(array)[0].copy_to_host(array)

    def get_buffer(self, array) -> GpuBuffer:
        return self._get_entry(array)[0]

    def release(self, array) -> None:
        buf, _ = self._get_entry(array)
        del self._buffers[id(array)]
        buf.free()

    def release_all(self) -> None:
        for buf, _ in self._buffers.values():
            buf.free()
        self._buffers.clear()


_CTYPES_SCALARS = (ctypes.c_int8, ctypes.c_int16, ctypes.c_int32, ctypes.c_int64, ctypes.c_float,
                   ctypes.c_double, ctypes.c_void_p)


def create_kernel_args(*args: Any):
    """Pack kernel arguments the way the reference does (core.py:472-554):
    GpuBuffer -> device pointer, ndarray -> host pointer, int / numpy integer ->
    int32, float / numpy floating -> float32, ctypes scalars as they are.

    Returns (pointer_array, struct, pointer_array) -- all three must stay alive
    until the launch has been issued; (None, None, None) for no arguments.
    """
    import numpy as np

    values, fields = [], []
    for i, arg in enumerate(args):
        if isinstance(arg, GpuBuffer):
            v: Any = ctypes.c_void_p(arg.ptr_value)
        elif isinstance(arg, np.ndarray):
            v = ctypes.c_void_p(arg.ctypes.data)
        elif isinstance(arg, (int, np.integer)):
            v = ctypes.c_int32(int(arg))
        elif isinstance(arg, (float, np.floating)):
            v = ctypes.c_float(float(arg))
        elif isinstance(arg, _CTYPES_SCALARS):
            v = arg
        else:
            raise TypeError(f"unsupported argument type: {type(arg)}")
        values.append(v)
        fields.append((f"_field{i}", type(v)))
    if not values:
        return None, None, None

    class _Args(ctypes.Structure):
        _fields_ = fields

    packed = _Args()
    for i, v in enumerate(values):
        setattr(packed, f"_field{i}", v)
    base = ctypes.addressof(packed)
    ptrs = (ctypes.c_void_p * len(values))(
        *[base + getattr(_Args, f"_field{i}").offset for i in range(len(values))])
    return ptrs, packed, ptrs


create_kernel_args_capsule = create_kernel_args


class GpuFunction:
    def __init__(self, handle: int, module: "GpuModule") -> None:
        self._h = handle
        self._module = module  # keeps the code object loaded

    def launch(self, grid_dim, block_dim, args, cluster_dim=None, shared_bytes: int = 0,
               stream: Optional[GpuStream] = None) -> None:
        if cluster_dim is not None:
            raise NotImplementedError("cluster launch does not exist on gfx950")
        ptrs, keep, _ = create_kernel_args(*args)
        gx, gy, gz = (int(v) for v in grid_dim)
        bx, by, bz = (int(v) for v in block_dim)
        _capi.check(_rt().aster_rt_module_launch_kernel(
            ctypes.c_void_p(self._h), gx, gy, gz, bx, by, bz, int(shared_bytes),
            stream.handle if stream is not None else None,
            ctypes.cast(ptrs, ctypes.POINTER(ctypes.c_void_p)) if ptrs is not None else None))
        del keep

    @property
    def handle(self) -> ctypes.c_void_p:
        return ctypes.c_void_p(self._h)


class GpuModule:
    """A loaded code object (.hsaco / .co file)."""

    def __init__(self, hsaco_path: str) -> None:
        hip_init()
        with open(hsaco_path, "rb") as f:
            self._image = f.read()
        h = ctypes.c_void_p()
        _capi.check(_rt().aster_rt_module_load_data(self._image, len(self._image), ctypes.byref(h)))
        self._h: Optional[int] = h.value

    def __del__(self) -> None:
        try:
            self.unload()
        except Exception:
            pass

    def unload(self) -> None:
        if getattr(self, "_h", None) is not None:
            h, self._h = self._h, None
            _capi.check(_rt().aster_rt_module_unload(ctypes.c_void_p(h)))

    def get_function(self, name: str) -> GpuFunction:
        f = ctypes.c_void_p()
        _capi.check(_rt().aster_rt_module_get_function(ctypes.c_void_p(self._h), name.encode(),
                                                      ctypes.byref(f)))
        return GpuFunction(f.value, self)


class FlushLLC:
    """Evicts the last-level cache between timed launches by rewriting a scratch
    buffer larger than it (the reference streams 256 MB,
    python/aster/execution/flush_llc.py:25-60; MI355X has 256 MB of Infinity
    Cache, hence the 512 MiB default)."""

    def __init__(self, size_bytes: int = 512 << 20) -> None:
        self.size_bytes = size_bytes
        self._buf: Optional[GpuBuffer] = None
        self._value = 0

    def initialize(self) -> None:
        if self._buf is None:
            self._buf = GpuBuffer(self.size_bytes)

    def flush_llc(self) -> None:
        self._value = (self._value + 1) & 0xFF
        _capi.check(_rt().aster_rt_memset(self._buf.ptr, self._value, self.size_bytes))

    def cleanup(self) -> None:
        if self._buf is not None:
            self._buf.free()
            self._buf = None


def execute_hsaco(hsaco_path: str, kernel_name: str, arguments: list,
                  grid_dim: Tuple[int, int, int] = (1, 1, 1),
                  block_dim: Tuple[int, int, int] = (64, 1, 1),
                  cluster_dim: Optional[Tuple[int, int, int]] = None, num_iterations: int = 1,
                  device_id: Optional[int] = None, flush_llc: Optional[Any] = None,
                  verify_fn: Optional[Callable] = None,
                  memory_manager: Optional[MemoryManager] = None,
                  shared_bytes: int = 0) -> List[int]:
    """Launch `kernel_name` from a code object `num_iterations` times on the null
    stream, one HIP event pair per launch; returns the per-launch times in ns.

    Argument roles and their copies follow the reference (core.py:605-717):
    inputs go up once, outputs come back after iteration 0 only, `verify_fn`
    sees the normalised argument list after that copy.
    """
    import numpy as np

    hip_init()
    if device_id is not None:
        _capi.check(_rt().aster_rt_set_device(int(device_id)))
    _rt().aster_rt_clear_last_error()

    arguments = [InOutArray(a) if isinstance(a, np.ndarray) else a for a in arguments]
    owns_mm = memory_manager is None
    mm = MemoryManager() if owns_mm else memory_manager
    roles = (InputArray, OutputArray, InOutArray)
    try:
        for arg in arguments:
            if isinstance(arg, roles):
                mm.register(arg.array, upload=not isinstance(arg, OutputArray))
        launch_args = [mm.get_buffer(a.array) if isinstance(a, roles) else a for a in arguments]

        module = GpuModule(hsaco_path)
        function = module.get_function(kernel_name)
        start, stop = GpuEvent(), GpuEvent()
        times_ns: List[int] = []
        if flush_llc is not None:
            flush_llc.initialize()
        try:
            for it in range(num_iterations):
                if flush_llc is not None:
                    flush_llc.flush_llc()
                start.record()
                function.launch(grid_dim, block_dim, launch_args, cluster_dim=cluster_dim,
                                shared_bytes=shared_bytes)
                stop.record()
                stop.synchronize()
                times_ns.append(stop.elapsed_ns(start))
                if it == 0:
                    for arg in arguments:
                        if isinstance(arg, (OutputArray, InOutArray)):
                            mm.sync_from_gpu(arg.array)
                    if verify_fn is not None:
                        verify_fn(arguments)
        finally:
            if flush_llc is not None:
                flush_llc.cleanup()
    finally:
        if owns_mm:
            mm.release_all()
    return times_ns


def system_has_gpu(mcpu: str = "gfx950") -> bool:
    """True when a device of architecture `mcpu` is visible (the reference parses
    `rocminfo`, python/aster/execution/utils.py:7-37; here the runtime is asked)."""
    try:
        lib = _rt()
        n = ctypes.c_int(0)
        if lib.aster_rt_get_device_count(ctypes.byref(n)) != 0 or n.value <= 0:
            return False
        props = _capi.DeviceProps()
        if lib.aster_rt_get_device_props(0, ctypes.byref(props)) != 0:
            return False
        return props.gcn_arch_name.decode().split(":")[0] == mcpu
    except (OSError, FileNotFoundError):
        return False
