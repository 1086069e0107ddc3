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

    def new_stream(self, name: str | None = None) -> HostStream:
        self._stream_count += 1
        return HostStream(name or f"stream{self._stream_count}")

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


class HipDevice:
    """The real thing: HIP events, streams and roctx ranges through torch."""

    is_gpu = True

    def new_event(self) -> "torch.cuda.Event":
        return torch.cuda.Event()

    def new_stream(self, name: str | None = None) -> "torch.cuda.Stream":
        return torch.cuda.Stream()

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
