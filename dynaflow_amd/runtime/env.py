"""Per-nano-batch value store and the "operator being launched" marker.

Mirrors dynaflow/runtime/env.py: values are kept per FX node with a use count
taken from the graph (``len(node.users)``); each read gives one use back and
the payload is dropped at the last one so activations die as early as the graph
allows (env.py:10-46).  The current operator handle is plain module state, set
by the engine around every launch and read by the execution backends
(env.py:48-70); engine and scheduler share one thread, so no context variable
is needed.
"""
from __future__ import annotations

from collections.abc import Generator
from contextlib import contextmanager
from typing import Any

import torch

from dynaflow_amd.interface import OperatorHandle


class ActivationBuffer:
    """A value plus the number of reads it still owes."""

    __slots__ = ("data", "ref_count")

    def __init__(self, data: Any, ref_count: int) -> None:
        self.data = data
        self.ref_count = ref_count

    def get_ref(self) -> Any:
        value = self.data
        self.ref_count -= 1
        if self.ref_count == 0:
            self.data = None
        return value


class ExecutionEnvironment:
    """``env[b][node]`` -> ``ActivationBuffer`` for each nano-batch ``b``."""

    def __init__(self, num_nano_batches: int) -> None:
        self.env: list[dict[torch.fx.Node, ActivationBuffer]] = [
            dict() for _ in range(num_nano_batches)
        ]

    def put(self, batch_idx: int, node: torch.fx.Node, data: Any) -> None:
        self.env[batch_idx][node] = ActivationBuffer(data, len(node.users))

    def get(self, batch_idx: int, node: torch.fx.Node) -> Any:
        value = self.env[batch_idx][node].get_ref()
        # a value read more often than the graph uses it has already been freed
        assert value is not None, f"{node.name} of nano-batch {batch_idx} was read after its last use"
        return value

    def live_entries(self) -> list[tuple[int, str]]:
        """(batch, node name) of every payload still held; for leak checks."""
        return [
            (b, node.name)
            for b, table in enumerate(self.env)
            for node, buf in table.items()
            if buf.data is not None
        ]


_current_op_handle: OperatorHandle | tuple[OperatorHandle, ...] | None = None


def get_op_handle() -> OperatorHandle | tuple[OperatorHandle, ...]:
    """Handle of the operator being launched; only valid inside a launch."""
    assert _current_op_handle is not None, "no operator is being launched"
    return _current_op_handle


def peek_op_handle() -> OperatorHandle | tuple[OperatorHandle, ...] | None:
    """Like ``get_op_handle`` but returns ``None`` outside a launch."""
    return _current_op_handle


@contextmanager
def set_op_handle(
    handle: OperatorHandle | tuple[OperatorHandle, ...],
) -> Generator[None, None, None]:
    global _current_op_handle
    saved = _current_op_handle
    _current_op_handle = handle
    try:
        yield
    finally:
        _current_op_handle = saved
