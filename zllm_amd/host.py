"""The platform layer for the HIP backend: a device and the host that executes
the command stream on it. A twin of the reference's ``gpu.Device`` / ``gpu.Host``
surface (src/gpu/host.zig:48-191) over the C ABI of include/zllm_hip.h, with the
reference's error set (src/agility/host.zig:38).
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

import numpy as np

from . import _lib
from .backend import Backend
from .cmd import Completion, Op
from .kernels import Prefill


class GpuError(Exception):
    pass


class DeviceLost(GpuError):
    pass


class BadCommand(GpuError):
    pass


class BadId(GpuError):
    pass


class Truncated(GpuError):
    pass


class BadLength(GpuError):
    pass


class UnsupportedKernel(GpuError):
    pass


class UnsupportedPrefill(GpuError):
    pass


class OutOfMemory(GpuError):
    pass


class NoDevice(GpuError):
    pass


_ERRORS = {
    -1: GpuError, -2: DeviceLost, -3: BadCommand, -4: BadId, -5: Truncated, -6: BadLength, -7: UnsupportedKernel,
    -8: UnsupportedPrefill, -9: OutOfMemory, -10: NoDevice, -11: ValueError,
}


@dataclass(frozen=True)
class Limits:
    max_binding: int
    offset_align: int


@dataclass(frozen=True)
class Adapter:
    vendor: str
    architecture: str
    device: str
    description: str
    api: str


@dataclass(frozen=True)
class TimingKey:
    pipeline: int
    grid: tuple[int, int, int]


@dataclass
class TimingTotal:
    ns: int = 0
    count: int = 0


@dataclass
class Timings:
    """gpu.Timings (src/gpu/timings.zig:6-27)."""

    totals: dict
    untimed: int
    capacity: int = 4096


class Device:
    """One MI355X (src/gpu/host.zig:48-135)."""

    NO_REPLAY = 1    # ZHIP_OPTION_NO_REPLAY: never replay a repeated submit from a HIP graph
    WIDE_DECODE = 2  # ZHIP_OPTION_WIDE_DECODE: large matvec_bf16 / matvec_f16 matrices read once for all of a step's tokens, at every width

    def __init__(self, index: int = 0, flags: int = 0) -> None:
        self.ctx = C.c_void_p()
        opts = _lib.Options(index, flags)
        r = _lib.lib.zhip_create(C.byref(opts), C.byref(self.ctx))
        if r < 0:
            self.ctx = C.c_void_p()
            raise _ERRORS.get(r, GpuError)(f"zhip_create failed ({r}): no gfx950 device at index {index}")
        self.caps = _lib.Caps()
        self.check(_lib.lib.zhip_get_caps(self.ctx, C.byref(self.caps)))

    @classmethod
    def open(cls, index: int = 0, flags: int = 0) -> "Device":
        return cls(index, flags)

    def deinit(self) -> None:
        if self.ctx:
            _lib.lib.zhip_destroy(self.ctx)
            self.ctx = C.c_void_p()

    def __del__(self) -> None:
        try:
            self.deinit()
        except Exception:
            pass

    def check(self, r: int) -> None:
        if r >= 0:
            return
        raise _ERRORS.get(r, GpuError)(self.error_message())

    def backend(self) -> Backend:
        return Backend.hip

    def supports_prefill(self, rung: Prefill) -> bool:
        return bool(_lib.lib.zhip_supports_prefill(self.ctx, int(rung)))

    def limits(self) -> Limits:
        return Limits(self.caps.max_binding, self.caps.offset_align)

    def memory_budget(self) -> int | None:
        caps = _lib.Caps()
        if _lib.lib.zhip_get_caps(self.ctx, C.byref(caps)) < 0:
            return None
        return caps.memory_bytes or None

    def adapter(self) -> Adapter:
        name = self.caps.name.decode()
        arch = self.caps.arch.decode()
        return Adapter("AMD", arch, name, f"{self.caps.compute_units} CUs, wave{self.caps.wavefront}", "hip")

    def error_message(self) -> str:
        buf = C.create_string_buffer(1024)
        _lib.lib.zhip_last_error(self.ctx, buf, len(buf))
        return buf.value.decode(errors="replace")

    def force_loss(self) -> None:
        _lib.lib.zhip_force_loss(self.ctx)


class Host:
    """Executes command batches on a Device (src/gpu/host.zig:138-191)."""

    def __init__(self, device: Device) -> None:
        self.d = device
        self._file = None
        self._profiling = False

    def deinit(self) -> None:
        pass

    def execute(self, words, completions: list) -> None:
        """Runs one batch, appending one completion per submit and per read."""
        words = np.ascontiguousarray(words, dtype=np.uint32)
        cap = int(np.count_nonzero((words & 0xFF) == Op.submit) + np.count_nonzero((words & 0xFF) == Op.read_buffer)) + 64
        out = (_lib.CCompletion * cap)()
        n = C.c_size_t(0)
        r = _lib.lib.zhip_execute(self.d.ctx, words.ctypes.data, words.size, out, cap, C.byref(n))
        for i in range(n.value):
            completions.append(Completion(out[i].token, out[i].status))
        self.d.check(r)

    def set_file(self, data: np.ndarray | None) -> None:
        self._file = None if data is None else np.ascontiguousarray(data).view(np.uint8)
        if self._file is None:
            self.d.check(_lib.lib.zhip_set_file(self.d.ctx, None, 0))
        else:
            self.d.check(_lib.lib.zhip_set_file(self.d.ctx, self._file.ctypes.data, self._file.size))

    def start_profile(self) -> None:
        self.d.check(_lib.lib.zhip_profile_start(self.d.ctx))
        self._profiling = True

    def stop_profile(self) -> None:
        _lib.lib.zhip_profile_stop(self.d.ctx)
        self._profiling = False

    def timings(self) -> Timings | None:
        if not self._profiling:
            return None
        n = C.c_size_t(0)
        untimed = C.c_uint64(0)
        self.d.check(_lib.lib.zhip_profile_read(self.d.ctx, None, 0, C.byref(n), C.byref(untimed)))
        rows = (_lib.CTiming * max(1, n.value))()
        self.d.check(_lib.lib.zhip_profile_read(self.d.ctx, rows, n.value, C.byref(n), C.byref(untimed)))
        totals = {TimingKey(rows[i].pipeline, tuple(rows[i].grid)): TimingTotal(rows[i].ns, rows[i].count) for i in range(n.value)}
        return Timings(totals, untimed.value)

    def replayed_submits(self) -> int:
        """Submits so far whose dispatches ran from a replayed HIP graph."""
        n = C.c_uint64(0)
        self.d.check(_lib.lib.zhip_replayed_submits(self.d.ctx, C.byref(n)))
        return n.value

    def last_submit(self) -> tuple[int, int]:
        """GPU nanoseconds and dispatch count of the last submit's work."""
        ns, count = C.c_uint64(0), C.c_uint64(0)
        self.d.check(_lib.lib.zhip_last_submit(self.d.ctx, C.byref(ns), C.byref(count)))
        return ns.value, count.value
