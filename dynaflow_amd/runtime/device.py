"""The thin seam between the engine and HIP streams / events.

The engine and the schedulers order device work with exactly three things:
events (``record`` / ``wait``), streams (made current for a ``with`` block) and
profiler ranges.  On an MI355X these are ``torch.cuda`` objects, which are HIP
events, HIP streams and roctx ranges on ROCm.  On a host without a GPU the same
protocol is served by recording objects, so that the host logic (issue order,
event chains, FIFO checks) can be exercised by CPU tests.  The recording
objects never compute anything: tensors that reach them are CPU tensors run by
PyTorch eagerly, which is only ever done by tests.

All streams are created at the default priority.
"""
from __future__ import annotations

import contextlib
import threading
from typing import Any

import torch


class HostEvent:
    """Event stand-in that logs ``record`` / ``wait`` with the stream in use."""

    _counter = 0

    def __init__(self, log: list) -> None:
        HostEvent._counter += 1
        self.uid = HostEvent._counter
        self._log = log
        self.recorded_on: str | None = None

    def record(self, stream: Any = None) -> None:
        self.recorded_on = (stream or _host_state.current).name
        self._log.append(("record", self.uid, self.recorded_on))

    def wait(self, stream: Any = None) -> None:
        self._log.append(("wait", self.uid, (stream or _host_state.current).name))

    def synchronize(self) -> None:
        pass


class HostStream:
    """Stream stand-in; only its name matters."""

    def __init__(self, name: str) -> None:
        self.name = name

    def wait_stream(self, other: "HostStream") -> None:
        pass

    def synchronize(self) -> None:
        pass


class _HostState(threading.local):
    def __init__(self) -> None:
        self.current = HostStream("default")


_host_state = _HostState()


class HostDevice:
    """Recording implementation of the seam (no GPU involved)."""

    is_gpu = False

    def __init__(self) -> None:
        self.log: list = []
        self._stream_count = 0

    def new_event(self) -> HostEvent:
        return HostEvent(self.log)

    def new_stream(self, name: str | None = None, cu_mask: "list[int] | None" = None) -> HostStream:
        self._stream_count += 1
        stream = HostStream(name or f"stream{self._stream_count}")
        stream.cu_mask = cu_mask
        return stream

    def current_stream(self) -> HostStream:
        return _host_state.current

    @contextlib.contextmanager
    def stream(self, stream: HostStream):
        previous = _host_state.current
        _host_state.current = stream
        try:
            yield
        finally:
            _host_state.current = previous

    @contextlib.contextmanager
    def range(self, name: str):
        self.log.append(("range", name, _host_state.current.name))
        yield


def stream_key(stream: "torch.cuda.Stream") -> tuple[int, int]:
    """What identifies a HIP stream in the event log: (device index, stream handle)."""
    return (stream.device_index, stream.cuda_stream)


class HipEvent:
    """A HIP event that knows the stream it was recorded on.

    ``wait`` on that very stream issues nothing: stream order already gives the edge, and under stream capture
    such a wait would make the stream its own child in the runtime's books (see ``capture_plan``).  While the
    device's ``trace`` is a list, every ``record`` / ``wait`` is logged there in the recording seam's format.
    """

    __slots__ = ("_owner", "_event", "_recorded_on", "uid")
    _counter = 0

    def __init__(self, owner: "HipDevice") -> None:
        HipEvent._counter += 1
        self.uid = HipEvent._counter
        self._owner = owner
        self._event = torch.cuda.Event()
        self._recorded_on: tuple[int, int] | None = None

    def record(self, stream: "torch.cuda.Stream | None" = None) -> None:
        stream = stream if stream is not None else torch.cuda.current_stream()
        self._recorded_on = stream_key(stream)
        self._owner.note(("record", self.uid, self._recorded_on), stream)
        self._event.record(stream)

    def wait(self, stream: "torch.cuda.Stream | None" = None) -> None:
        stream = stream if stream is not None else torch.cuda.current_stream()
        key = stream_key(stream)
        self._owner.note(("wait", self.uid, key), stream)
        if self._recorded_on is None or key == self._recorded_on:
            return
        self._event.wait(stream)

    def synchronize(self) -> None:
        self._event.synchronize()

    def query(self) -> bool:
        return self._event.query()


def cu_mask_words(first: int, count: int, total: int) -> list[int]:
    """Mask words for compute units ``first .. first + count - 1`` of ``total``."""
    if not (0 <= first and count >= 1 and first + count <= total):
        raise ValueError(f"compute units {first}..{first + count - 1} of {total}")
    bits = ((1 << count) - 1) << first
    return [(bits >> (32 * i)) & 0xFFFFFFFF for i in range((total + 31) // 32)]


def _loaded_hip_runtime() -> str:
    """Path of the HIP runtime that this process has already mapped (the one torch uses): a second copy loaded by
    its bare name would be another runtime with streams and contexts of its own."""
    with open("/proc/self/maps") as maps:
        for line in maps:
            path = line.rsplit(" ", 1)[-1].strip()
            if "libamdhip64.so" in path:
                return path
    raise RuntimeError("no HIP runtime is loaded in this process")


def _masked_stream(cu_mask: list[int]) -> int:
    """hipExtStreamCreateWithCUMask through the HIP runtime that torch has loaded; returns the stream handle."""
    import ctypes

    hip = ctypes.CDLL(_loaded_hip_runtime())
    words = (ctypes.c_uint32 * len(cu_mask))(*cu_mask)
    stream = ctypes.c_void_p()
    torch.cuda.current_stream()   # the device's context exists before the raw call
    rc = hip.hipExtStreamCreateWithCUMask(ctypes.byref(stream), ctypes.c_uint32(len(cu_mask)), words)
    if rc != 0 or not stream.value:
        raise RuntimeError(f"hipExtStreamCreateWithCUMask failed with {rc}")
    return stream.value


class HipDevice:
    """The real thing: HIP events, streams and roctx ranges through torch."""

    is_gpu = True

    def __init__(self) -> None:
        #: while a list: the (kind, event id, stream key) log of every event operation
        self.trace: list | None = None
        self.streams_seen: dict[tuple[int, int], "torch.cuda.Stream"] = {}

    def note(self, entry: tuple, stream: "torch.cuda.Stream") -> None:
        if self.trace is not None:
            self.trace.append(entry)
            self.streams_seen[entry[2]] = stream

    def new_event(self) -> HipEvent:
        return HipEvent(self)

    def new_stream(self, name: str | None = None, cu_mask: "list[int] | None" = None) -> "torch.cuda.Stream":
        """A stream at the default priority.  ``cu_mask`` (32-bit words, bit i = compute unit i may run this
        stream's work) makes it a stream restricted to those compute units - what the reference does with green
        contexts (examples/ae/up-silu-overlap.cu:236-264).  Such a stream lives until the process ends."""
        if cu_mask is None:
            return torch.cuda.Stream()
        return torch.cuda.ExternalStream(_masked_stream(cu_mask))

    def current_stream(self) -> "torch.cuda.Stream":
        return torch.cuda.current_stream()

    def stream(self, stream: "torch.cuda.Stream"):
        return torch.cuda.stream(stream)

    @contextlib.contextmanager
    def range(self, name: str):
        torch.cuda.nvtx.range_push(name)
        try:
            yield
        finally:
            torch.cuda.nvtx.range_pop()


_device: HostDevice | HipDevice | None = None


def get_device() -> HostDevice | HipDevice:
    """The process-wide seam; picks HIP when a GPU is visible."""
    global _device
    if _device is None:
        _device = HipDevice() if torch.cuda.is_available() else HostDevice()
    return _device


def set_device(device: HostDevice | HipDevice | None) -> None:
    """Install a seam explicitly (tests install a fresh ``HostDevice``)."""
    global _device
    _device = device
