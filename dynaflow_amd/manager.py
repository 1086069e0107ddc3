"""Front door of the scheduling layer (same surface as dynaflow/manager.py).

``initialize``  (manager.py:37-112)  split + tag the traced graph, pick which
                sub-graphs get the kernel backend / piecewise graphs, install
                the backends, build the engine.
``prepare`` / ``override_split_config`` (manager.py:114-159)  store the
                ``SplitConfig`` of the *next* forward; every forward consumes it.
``get_callable`` (manager.py:161-190) the synchronous forward: one nano-batch
                takes the scheduler-free fast path, otherwise engine and
                scheduler coroutines run side by side in a fresh event loop,
                the caller's stream waits for every nano-batch's tail event and
                the per-nano-batch outputs are concatenated on dim 0
                (manager.py:192-261).

On top of that, ``additional_config["whole_graph"]`` turns on whole-schedule
hipGraph replay: the first forward with a given split runs the complete
multi-stream schedule under stream capture (side streams fork from and join
back into the capturing stream through the engine's event chain) and later
forwards with that split replay the one graph, skipping the event loop, the
scheduler and all launches.
"""
from __future__ import annotations

import asyncio
import logging
import os
import tempfile
from collections.abc import Callable
from dataclasses import replace
from typing import Any

import torch

from dynaflow_amd.config import DynaFlowConfig
from dynaflow_amd.executor.compiler import SubgraphCompiler
from dynaflow_amd.interface import ExecutionContext, InputInfo, OpSchedulerBase, SplitConfig
from dynaflow_amd.matching import split_graph, tag_graph
from dynaflow_amd.runtime import capture_plan
from dynaflow_amd.runtime.device import get_device, stream_key
from dynaflow_amd.runtime.engine import DynaFlowEngine

log = logging.getLogger("dynaflow")
if os.environ.get("DYNAFLOW_VERBOSE"):
    logging.basicConfig(level=logging.INFO)


def trivial_split(batch_size: int, num_tokens: list[int], is_dryrun: bool, use_cudagraph: bool) -> SplitConfig:
    """The single-nano-batch split used before initialisation and for dry-runs."""
    total = sum(num_tokens)
    return SplitConfig(
        num_nano_batches=1,
        batch_sizes=[batch_size],
        batch_indices=[0, batch_size],
        num_tokens=[total],
        num_tokens_padded=[total],
        split_indices=[0, total],
        is_dryrun=is_dryrun,
        use_cudagraph=use_cudagraph,
    )


def _already_joined(parts: list[torch.Tensor], shared_buffer: torch.Tensor | None) -> torch.Tensor | None:
    """The concatenation of ``parts`` on dim 0 without a copy, if they are consecutive row ranges that together
    make up the engine's shared output buffer; else ``None``."""
    base = parts[0]._base
    if shared_buffer is None or base is not shared_buffer or not base.is_contiguous():
        return None
    offset, tail = base.storage_offset(), tuple(parts[0].shape[1:])
    for part in parts:
        if part._base is not base or not part.is_contiguous() or tuple(part.shape[1:]) != tail:
            return None
        if part.storage_offset() != offset:
            return None
        offset += part.numel()
    if offset - base.storage_offset() != base.numel():
        return None
    rows = sum(part.shape[0] for part in parts)
    return base.view(rows, *tail)


def join_results(results: dict[int, Any], num_nano_batches: int, shared_buffer: torch.Tensor | None = None) -> Any:
    """Concatenate per-nano-batch outputs on dim 0 (tuples field by field); outputs that already are the
    consecutive rows of the engine's shared output buffer are returned as that buffer."""
    first = results[0]
    assert all(isinstance(r, type(first)) for r in results.values()), (
        f"Results have different types: {results}"
    )
    ordered = [results[b] for b in range(num_nano_batches)]
    if isinstance(first, torch.Tensor):
        joined = _already_joined(ordered, shared_buffer)
        return joined if joined is not None else torch.cat(ordered, dim=0)
    if isinstance(first, tuple):
        width = len(first)
        assert all(len(r) == width for r in ordered), (
            f"Results have different number of elements: {results}"
        )
        fields = []
        for i in range(width):
            column = [r[i] for r in ordered]
            assert all(isinstance(e, torch.Tensor) for e in column), f"Elements are not tensors: {column}"
            joined = _already_joined(column, shared_buffer)
            fields.append(joined if joined is not None else torch.cat(column, dim=0))
        return tuple(fields)
    return first


class _ScheduleGraph:
    """One captured forward: the graph, the tensors it reads and its output."""

    def __init__(self, graph: Any, inputs: list[Any], token_shaped: list[bool], output: Any) -> None:
        self.graph = graph
        self.inputs = inputs
        self.token_shaped = token_shaped
        self.output = output


class DynaFlowManager:
    """Splits a traced graph and runs it under a programmable scheduler."""

    def __init__(self) -> None:
        self.initialized = False
        self.config: DynaFlowConfig | None = None
        self.graph_module: torch.fx.GraphModule | None = None
        self.cached_config: SplitConfig | None = None
        self.scheduler: OpSchedulerBase | None = None
        self.engine: DynaFlowEngine | None = None
        self.graph_dump_path: str | None = None
        self._schedule_graphs: dict[tuple, _ScheduleGraph] = {}
        #: per captured schedule: "caller" (captured from the caller's side) or "schedule" (from one of its streams)
        self.capture_origins: dict[tuple, str] = {}

    # ------------------------------------------------------------ set-up
    def initialize(
        self,
        graph_module: torch.fx.GraphModule,
        config: DynaFlowConfig,
        scheduler: OpSchedulerBase,
        example_inputs: list[Any],
    ) -> None:
        """Prepare a traced full graph for scheduled execution.

        Must be called from inside the ``torch.compile`` backend that received
        ``graph_module`` (the ambient fake mode is needed), with the token
        dimension of the inputs symbolic so every sub-graph receives the token
        count as a ``SymInt`` argument.
        """
        self.initialized = True
        self.config = config
        self.graph_module = split_graph(graph_module, scheduler.get_split_rules())
        tag_graph(self.graph_module, scheduler.get_tag_rules())

        def tagged_without(word: str) -> list[str]:
            return [
                name
                for name, module in self.graph_module.named_modules()
                if isinstance(tag := getattr(module, "tag", None), set) and word not in tag
            ]

        backend_on = config.inductor_config.enabled and bool(config.knob("hip_backend", True))
        inductor_compile_targets = tagged_without("no-inductor") if backend_on else []
        cudagraph_targets = tagged_without("no-cudagraph") if config.cudagraph_config.enabled else []

        if config.knob("dump_graph", True):
            self.graph_dump_path = os.path.join(tempfile.mkdtemp(), "gm_with_subgraphs.py")
            with open(self.graph_dump_path, "w") as f:
                f.write("# Graph\n")
                f.write(f"# Inductor Compile Targets: {inductor_compile_targets}\n")
                f.write(f"# CUDAGraph Targets: {cudagraph_targets}\n")
                f.write(self.graph_module.print_readable(print_output=False))
            log.info("Graph saved to %s", self.graph_dump_path)

        SubgraphCompiler(
            self.graph_module,
            config,
            inductor_compile_targets=inductor_compile_targets,
            cudagraph_targets=cudagraph_targets,
        ).run(*example_inputs)
        self.engine = DynaFlowEngine(self.graph_module, config)
        self.scheduler = scheduler
        self._schedule_graphs = {}

    # ----------------------------------------------------- split selection
    def prepare(
        self,
        batch_size: int,
        num_tokens: list[int],
        is_dryrun: bool = False,
        use_cudagraph: bool = False,
    ) -> SplitConfig:
        """Choose and remember the split of the next forward."""
        if not self.initialized or is_dryrun:
            self.cached_config = trivial_split(batch_size, num_tokens, is_dryrun, use_cudagraph)
        else:
            assert self.scheduler is not None
            self.cached_config = self.scheduler.get_split_config(
                InputInfo(batch_size, num_tokens, sum(num_tokens)),
                use_cudagraph=use_cudagraph,
            )
        return self.cached_config

    def override_split_config(self, split_config: SplitConfig) -> None:
        self.cached_config = split_config

    # -------------------------------------------------------------- forward
    def get_callable(self) -> Callable:
        """The synchronous callable ``torch.compile`` gets back from the backend."""
        assert self.initialized

        def _forward(*args, **kwargs) -> Any:
            assert (
                self.cached_config is not None
                and self.graph_module is not None
                and self.config is not None
            ), "call prepare() or override_split_config() before every forward"
            split = self.cached_config
            log.info("Executing with SplitConfig: %s", split)
            try:
                if not split.is_dryrun and split.num_nano_batches == 1 and split.allow_fallback:
                    assert self.engine is not None
                    return self.engine.execute_single_batch(split, args, kwargs)
                if self._wants_whole_graph(split):
                    return self._forward_whole_graph(split, args, kwargs)
                return asyncio.run(self._forward_async(args, kwargs))
            finally:
                self.cached_config = None

        return _forward

    async def _forward_async(self, args: tuple, kwargs: dict, split: SplitConfig | None = None) -> Any:
        """Engine and scheduler side by side; join and concatenate at the end."""
        split = split if split is not None else self.cached_config
        assert self.initialized and self.engine is not None and self.scheduler is not None
        assert split is not None
        lanes = split.num_nano_batches
        op_queue = {b: asyncio.Queue(maxsize=10) for b in range(lanes)}
        execute_queue: asyncio.Queue = asyncio.Queue()
        context = ExecutionContext(split, op_queue, execute_queue)

        from dynaflow_amd import ops

        with ops.launch_options(side_by_side=self.launches_side_by_side(split)):
            if split.is_dryrun:
                results, events = self.engine.dryrun(args, kwargs, split)
            else:
                (results, events), _ = await asyncio.gather(
                    self.engine.execute(args, kwargs, op_queue, execute_queue, split),
                    self.scheduler.schedule(context),
                )
        # the caller's stream continues only after every nano-batch's last launch
        for event in events:
            event.wait()
        return join_results(results, len(results), getattr(self.engine, "shared_output_buffer", None))

    def launches_side_by_side(self, split: SplitConfig) -> int:
        """How many nano-batches run the SAME sub-graph at the same time in a forward with this split - what the
        kernel plans are made for (``ops.launch_options``).  It follows from the schedule, not from a promise of
        the user: the shipped schedulers pick a launch's stream from the sub-graph's tag (``streams="by_kind"``,
        the reference's policies, examples/ae/scheduler/hf/nanoflow.py:122-146: launches of one kind queue on one
        stream, so a launch of a kind runs alone) or from the nano-batch (``"by_nano_batch"``: two streams that the
        nano-batches take in turn, so two nano-batches run the same sub-graph side by side); one stream
        (``serialize``), one nano-batch, or a scheduler that does not say how it assigns streams give 1.

        ``additional_config["side_by_side"]`` overrides the derived figure downwards (kernels planned as for
        fewer co-runners, for comparisons); a figure above it contradicts the schedule - launches planned for
        partners that never run - and is refused, except on the one-stream schedule, which is the baseline of
        whichever plan it is given (same kernels, nothing overlapped)."""
        assert self.config is not None and self.scheduler is not None
        lanes = split.num_nano_batches
        if split.is_dryrun:      # a dry-run captures what the scheduled forwards replay: plan as for those
            lanes = int(getattr(self.scheduler, "num_nano_batches", self.config.max_num_splits))
        policy = getattr(self.scheduler, "stream_policy", None)
        main, side = getattr(self.scheduler, "comp_stream", None), getattr(self.scheduler, "comm_stream", None)
        one_stream = main is None or main is side
        derived = min(lanes, 2) if (policy == "by_nano_batch" and not one_stream) else 1
        asked = self.config.knob("side_by_side", None)
        if asked is None or asked == "auto":
            return derived
        asked = int(asked)
        if asked < 1:
            raise ValueError(f"side_by_side={asked}: at least one launch runs")
        if asked > derived and not one_stream:
            raise ValueError(
                f"side_by_side={asked} contradicts the schedule: with streams={policy!r} and {lanes} nano-batch(es) "
                f"{derived} launch(es) of a sub-graph run at the same time; leave the knob out (it is derived) or "
                'use streams="by_nano_batch"')
        return asked

    # ------------------------------------------------- whole-schedule graphs
    def _wants_whole_graph(self, split: SplitConfig) -> bool:
        assert self.config is not None
        return (
            bool(self.config.knob("whole_graph", False))
            and split.use_cudagraph
            and not split.is_dryrun
            and get_device().is_gpu
        )

    def _token_shaped_flags(self, args: tuple) -> list[bool]:
        assert self.engine is not None
        flags = [False] * len(args)
        for node, idx in self.engine.placeholder_node_to_idx.items():
            example = node.meta.get("example_value", None)
            flags[idx] = isinstance(example, torch.Tensor) and isinstance(example.shape[0], torch.SymInt)
        return flags

    def _forward_whole_graph(self, split: SplitConfig, args: tuple, kwargs: dict) -> Any:
        """Replay (or first capture) the complete schedule for this split.

        The graph is captured against the very tensors of the capturing call.
        On replay a token-shaped input that lives elsewhere is copied into the
        captured tensor first; weights must not have moved.  The returned
        tensors belong to the graph and are overwritten by the next replay.
        """
        assert self.config is not None
        assert not kwargs, "whole-schedule graphs take positional graph inputs only"
        assert self.graph_module is not None
        # the whole schedule is captured at its exact size: capture-size padding does not apply
        eager_split = replace(split, use_cudagraph=False, num_tokens_padded=list(split.num_tokens))
        key = (
            tuple(split.split_indices),
            tuple((tuple(a.shape), a.dtype) if isinstance(a, torch.Tensor) else a for a in args),
        )
        entry = self._schedule_graphs.get(key)
        if entry is None:
            # one eager pass first: lazy one-time set-up (kernel attributes, allocator growth) must not
            # happen under capture; its event log says from which stream the schedule can be captured
            device = get_device()
            device.trace = []
            try:
                asyncio.run(self._forward_async(args, kwargs, eager_split))
            finally:
                event_log, device.trace = device.trace, None
            caller = stream_key(torch.cuda.current_stream())
            origin = capture_plan.choose_origin(event_log, caller)
            if origin is None:
                raise NotImplementedError(
                    "this schedule cannot be captured as one graph from any of its streams: streams wait for "
                    f"each other's events in a cycle {capture_plan.join_cycle(event_log, caller, caller)}; use "
                    "per-sub-graph graphs (CUDAGraphConfig(enabled=True)) or the eager schedule"
                )
            torch.cuda.current_stream().synchronize()
            graph = torch.cuda.CUDAGraph()
            # captured from the caller's side (torch's own capture stream) when that is safe, else from the
            # stream of the schedule that the others meet at
            capture_on = {} if origin == caller else {"stream": device.streams_seen[origin]}
            with torch.cuda.graph(graph, **capture_on):
                output = asyncio.run(self._forward_async(args, kwargs, eager_split))
            self.capture_origins[key] = "caller" if origin == caller else "schedule"
            entry = _ScheduleGraph(graph, list(args), self._token_shaped_flags(args), output)
            self._schedule_graphs[key] = entry
        else:
            for captured, given, token_shaped in zip(entry.inputs, args, entry.token_shaped):
                if not isinstance(captured, torch.Tensor):
                    continue
                if captured.data_ptr() == given.data_ptr():
                    continue
                if token_shaped:
                    captured.copy_(given)
                elif self.config.cudagraph_config.check_ptr_consistency:
                    raise RuntimeError("a static graph input (weight) moved between capture and replay")
                else:
                    captured.copy_(given)
        entry.graph.replay()
        return entry.output
