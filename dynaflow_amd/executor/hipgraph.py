"""Piecewise hipGraph capture and replay of one sub-graph.

``CUDAGraphWrapper`` keeps the name and behaviour of
dynaflow/executor/cudagraph.py:68-123: one graph per (padded size, nano-batch
index), captured only during a dry-run, replayed whenever the current operator
handle asks for graphs, with an optional check that input addresses did not
move between capture and replay.  On ROCm ``torch.cuda.CUDAGraph`` is a
hipGraph.  Each nano-batch index captures into its own memory pool
(cudagraph.py:11-31) so graphs of different nano-batches never share scratch.

The reference hands out weak references to the captured outputs through a vLLM
operator (cudagraph.py:37-65); that operator does not exist in plain PyTorch, so
the entry simply keeps the output tensors (``weak_ref_output`` is accepted and
has no effect).

Nothing in this package records memset nodes into a captured graph; buffers
that must start at zero are cleared by a fill kernel.
"""
from __future__ import annotations

from collections.abc import Callable
from typing import Any

import torch

from dynaflow_amd.config import CUDAGraphConfig
from dynaflow_amd.interface import OperatorHandle
from dynaflow_amd.runtime.env import get_op_handle


class CUDAGraphPool:
    """One graph memory pool per nano-batch index."""

    def __init__(self) -> None:
        self.pools: dict[int, Any] = {}

    def get_pool(self, key: int) -> Any:
        if key not in self.pools:
            self.pools[key] = torch.cuda.graph_pool_handle()
        return self.pools[key]


_global_pool = CUDAGraphPool()


def _tensor_addresses(args: tuple) -> list[int]:
    return [a.data_ptr() for a in args if isinstance(a, torch.Tensor)]


class CUDAGraphWrapper:
    """Capture-once / replay-many wrapper around a sub-graph callable."""

    def __init__(self, runnable: Callable[..., Any], config: CUDAGraphConfig) -> None:
        self.runnable = runnable
        self.config = config
        self._entries: dict[tuple[Any, ...], dict[str, Any]] = {}

    def __call__(self, *args: Any, **kwargs: Any) -> Any:
        handle = get_op_handle()
        if not isinstance(handle, OperatorHandle) or not handle._use_cudagraph:
            return self.runnable(*args, **kwargs)

        size = handle.batch_size
        key = (size, handle.batch_idx, handle.batch_size)
        entry = self._entries.get(key)
        if entry is None:
            assert handle._is_dryrun, (
                f"CUDA graph capture is required for batch size {size} but not in dry-run mode"
            )
            # one eager call first: lazy one-time set-up (kernel attributes, split-K workspaces) must not
            # happen under capture.  Sub-graphs that write state (a KV-cache append) write the same
            # values again in the capture's replay below.
            self.runnable(*args, **kwargs)
            torch.cuda.current_stream().synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, pool=_global_pool.get_pool(handle.batch_idx)):
                out = self.runnable(*args, **kwargs)
            self._entries[key] = {"graph": graph, "out": out, "inputs": _tensor_addresses(args)}
            # capture records without running; replay once so that the dry-run's result is real
            # (the reference hands back the unexecuted capture outputs, cudagraph.py:100-113)
            graph.replay()
            return out

        if self.config.check_ptr_consistency and _tensor_addresses(args) != entry["inputs"]:
            raise RuntimeError("CUDAGraph input addresses changed between capture and replay")
        entry["graph"].replay()
        return entry["out"]
