"""Public types of the scheduling layer and the scheduler plug-in contract.

This module mirrors the surface of dynaflow/interface.py so that scheduler
policies written for the reference import and run unchanged:

* ``InputInfo``        (dynaflow/interface.py:9-21)   what a policy sees of a batch
* ``SplitConfig``      (dynaflow/interface.py:24-52)  the microbatch split record
* ``OperatorHandle``   (dynaflow/interface.py:55-73)  identity-compared op token
* ``ExecutionContext`` (dynaflow/interface.py:76-127) scheduler <-> engine channel
* ``OpSchedulerBase``  (dynaflow/interface.py:130-156) the plug-in base class

Protocol between a scheduler coroutine and the engine
-----------------------------------------------------
``op = await ctx.pop(b)`` yields the next ready operator of nano-batch ``b``
or ``None`` once that nano-batch has produced its output.  ``await
ctx.execute((op,), func=None)`` asks the engine to launch the operator on
whatever HIP stream is *current on the calling thread* at that moment; it
returns when the work has been enqueued, not when the GPU finished it.
Handles of one nano-batch must be executed in the order they were popped.
"""
from __future__ import annotations

import asyncio
from abc import ABC, abstractmethod
from collections.abc import Callable
from dataclasses import dataclass

from dynaflow_amd.matching import MatchingRule


@dataclass
class InputInfo:
    """Per-forward batch summary handed to ``get_split_config``."""

    batch_size: int  # number of requests
    num_tokens: list[int]  # tokens of each request
    total_num_tokens: int  # sum(num_tokens)


@dataclass
class SplitConfig:
    """How one forward is cut into nano-batches (microbatches) along dim 0.

    ``batch_indices`` are request offsets, ``split_indices`` are token offsets;
    both have ``num_nano_batches + 1`` entries and start at 0.  Nano-batch
    ``b`` owns rows ``split_indices[b]:split_indices[b+1]`` of every
    token-shaped input.  ``num_tokens_padded`` differs from ``num_tokens``
    only when a graph-capture size forces padding.
    """

    num_nano_batches: int
    batch_sizes: list[int]
    batch_indices: list[int]
    num_tokens: list[int]
    num_tokens_padded: list[int]
    split_indices: list[int]
    is_dryrun: bool
    use_cudagraph: bool
    # A single nano-batch normally bypasses the scheduler entirely; policies
    # that substitute operators through ``execute(op, func)`` switch that off.
    allow_fallback: bool = True

    def validate(self) -> None:
        """Check the structural invariants every producer of splits upholds."""
        n = self.num_nano_batches
        if n < 1:
            raise ValueError(f"num_nano_batches must be >= 1, got {n}")
        for name, want in (
            ("batch_sizes", n),
            ("num_tokens", n),
            ("num_tokens_padded", n),
            ("batch_indices", n + 1),
            ("split_indices", n + 1),
        ):
            got = len(getattr(self, name))
            if got != want:
                raise ValueError(f"{name} has {got} entries, expected {want}")
        if self.split_indices[0] != 0 or self.batch_indices[0] != 0:
            raise ValueError("split_indices / batch_indices must start at 0")
        for b in range(n):
            if self.split_indices[b + 1] - self.split_indices[b] != self.num_tokens[b]:
                raise ValueError(f"split_indices disagree with num_tokens at {b}")
            if self.batch_indices[b + 1] - self.batch_indices[b] != self.batch_sizes[b]:
                raise ValueError(f"batch_indices disagree with batch_sizes at {b}")
            if self.num_tokens_padded[b] < self.num_tokens[b]:
                raise ValueError(f"padding shrinks nano-batch {b}")


@dataclass(eq=False, frozen=True)
class OperatorHandle:
    """One (sub-graph, nano-batch) launch the scheduler may place.

    Equality is identity (``eq=False``): the engine checks that the handle a
    scheduler executes *is* the one it popped (dynaflow/runtime/engine.py:388).
    """

    module_name: str  # name of the FX sub-module, e.g. "submod_1"
    batch_idx: int  # which nano-batch
    batch_size: int  # padded token count of that nano-batch
    tag: set[str]  # tags from the scheduler's tag rules

    # consumed by the execution backends, not by policies
    _is_dryrun: bool
    _use_cudagraph: bool
    # which engine issued the handle (not in the reference's record): scratch memory that operators keep per
    # nano-batch is kept per engine as well, so that two engines never share arrival counters
    _owner: int = 0


class ExecutionContext:
    """The two queues a scheduler talks to the engine through."""

    def __init__(
        self,
        split_config: SplitConfig,
        op_queue: dict[int, asyncio.Queue],
        execute_queue: asyncio.Queue,
    ) -> None:
        self._split_config = split_config
        self._op_queue = op_queue
        self._execute_queue = execute_queue

    @property
    def split_config(self) -> SplitConfig:
        return self._split_config

    async def pop(self, batch_idx: int) -> OperatorHandle | None:
        """Next ready operator of ``batch_idx``; ``None`` when it is finished."""
        return await self._op_queue[batch_idx].get()

    async def execute(
        self,
        operator: OperatorHandle | tuple[OperatorHandle, ...],
        func: Callable | None = None,
    ) -> None:
        """Have the engine launch ``operator`` now, on the current stream.

        ``func``, when given, replaces the sub-graph: it is called with the
        operator's materialised positional inputs and must return what the
        sub-graph would.  The reference's callers always pass a 1-tuple
        (dynaflow/runtime/engine.py:296-299); a bare handle is accepted too.
        """
        if isinstance(operator, OperatorHandle):
            operator = (operator,)
        finished = asyncio.Event()
        await self._execute_queue.put((operator, func, finished))
        await finished.wait()


class OpSchedulerBase(ABC):
    """Base class of scheduling policies (constructed as ``Class(config)``)."""

    def __init__(self, policy_name: str | None = None) -> None:
        self.policy_name = policy_name

    @abstractmethod
    def get_split_rules(self) -> list[MatchingRule]:
        """Rules whose matches become sub-graphs of their own."""

    @abstractmethod
    def get_tag_rules(self) -> dict[MatchingRule, set[str]]:
        """Rules that attach tags to the sub-graphs containing a match."""

    @abstractmethod
    def get_split_config(self, input_info: InputInfo, use_cudagraph: bool) -> SplitConfig:
        """Decide the nano-batch split of the next forward."""

    @abstractmethod
    async def schedule(self, context: ExecutionContext) -> None:
        """Pop ready operators and issue them until every nano-batch is done."""
