"""The producer side of a forward: walks the split graph once per nano-batch.

Behavioural contract (dynaflow/runtime/engine.py):

* ``execute`` (engine.py:222-424) - for every nano-batch the engine walks the
  top-level node list.  Nodes that are not sub-graph calls (placeholders,
  ``getitem``, ``get_attr`` ...) run inline; placeholders slice token-shaped
  inputs to the nano-batch's rows (engine.py:426-477).  Sub-graph calls are
  published to the scheduler as ``OperatorHandle``s and launched when the
  scheduler asks for them, on the stream that is current at that moment.
  Device ordering inside a nano-batch is a chain of events: every launch waits
  for the nano-batch's previous event and records a new one (engine.py:302-303,
  386).  Nano-batches never depend on one another.
* ``dryrun`` (engine.py:81-177) - priming pass without scheduler, optionally
  over ``max_num_splits`` fake nano-batches so every (size, batch index) graph
  gets captured.
* ``execute_single_batch`` (engine.py:179-220) - scheduler-free fast path.

Deliberate differences from the reference, none of which changes results:
static input buffers are per nano-batch (the reference aliases one dict across
all of them, engine.py:40) and are sized by ``additional_config["max_tokens"]``
instead of a fixed 16384 rows (engine.py:124-126); tensors that cross streams
are registered with the allocator (``record_stream``) before use; a graph with
no sub-graph call finishes instead of waiting for a request that never comes.
"""
from __future__ import annotations

import asyncio
from collections import deque
from collections.abc import Callable
from typing import Any

import torch
import torch.fx

from dynaflow_amd.config import DynaFlowConfig
from dynaflow_amd.interface import OperatorHandle, SplitConfig
from dynaflow_amd.runtime.device import get_device
from dynaflow_amd.runtime.env import ExecutionEnvironment, set_op_handle

_DEFAULT_MAX_TOKENS = 16384


def _is_symbolic(value: Any) -> bool:
    return isinstance(value, torch.SymInt)


class _SharedOutput:
    """Rows of one output buffer handed to the operator that ends each nano-batch (``ops.offer_output_rows``).

    The buffer is allocated when the first operator asks, on the stream of the caller of the forward (whose
    earlier work every nano-batch stream has waited for), with as many rows as the asking nano-batch's share
    of the tokens implies; a nano-batch gets the rows at its token offset.
    """

    def __init__(self, module_name: str, split_config: SplitConfig, device: Any) -> None:
        self.module_name = module_name
        self.split = split_config
        self.origin_stream = device.current_stream()
        self.buffer: torch.Tensor | None = None

    def offer(self, op: OperatorHandle) -> bool:
        if op.module_name != self.module_name:
            return False
        from dynaflow_amd import ops

        b = op.batch_idx
        tokens, total = self.split.num_tokens[b], self.split.split_indices[-1]
        first = self.split.split_indices[b]

        def provider(rows: int, cols: int, dtype: torch.dtype, dev: torch.device) -> torch.Tensor | None:
            if tokens <= 0 or rows % tokens:
                return None
            per_token = rows // tokens
            if self.buffer is None:
                with torch.cuda.stream(self.origin_stream):
                    self.buffer = torch.empty((per_token * total, cols), dtype=dtype, device=dev)
            buf = self.buffer
            if buf.shape[1] != cols or buf.dtype != dtype or buf.shape[0] != per_token * total:
                return None
            buf.record_stream(torch.cuda.current_stream())
            return buf[per_token * first: per_token * first + rows]

        ops.offer_output_rows(provider)
        return True

    @staticmethod
    def withdraw() -> None:
        from dynaflow_amd import ops

        ops.withdraw_output_rows()


class DynaFlowEngine:
    """Runs a split ``GraphModule`` under a scheduler's control."""

    def __init__(self, graph_module: torch.fx.GraphModule, config: DynaFlowConfig) -> None:
        self.graph_module = graph_module
        self.config = config
        #: the buffer that the last forward's nano-batches wrote their output rows into (or None)
        self.shared_output_buffer: torch.Tensor | None = None
        self.max_tokens = int(config.knob("max_tokens", _DEFAULT_MAX_TOKENS))
        # static input buffers for graph replay: [nano-batch][placeholder index]
        self.input_buffers: list[dict[int, torch.Tensor]] = [
            dict() for _ in range(config.max_num_splits)
        ]
        self.nodes: list[torch.fx.Node] = list(graph_module.graph.nodes)
        self.module_name_to_node: dict[str, torch.fx.Node] = {}
        self.placeholder_nodes: list[torch.fx.Node] = []
        self.get_attr_cache: dict[str, Any] = {}
        for node in self.nodes:
            if node.op == "call_module":
                assert isinstance(node.target, str)
                self.module_name_to_node[node.target] = node
            elif node.op == "placeholder":
                self.placeholder_nodes.append(node)
            elif node.op == "get_attr":
                assert isinstance(node.target, str)
                self.get_attr_cache[node.target] = getattr(graph_module, node.target)
        self.placeholder_node_to_idx: dict[torch.fx.Node, int] = {
            node: i for i, node in enumerate(self.placeholder_nodes)
        }
        #: (module name, nano-batch) of every launch of the last ``execute``
        self.issue_trace: list[tuple[str, int]] = []
        self.last_env: ExecutionEnvironment | None = None

    # ------------------------------------------------------------------ inputs
    def allocate_input_buffer(
        self, batch_idx: int, placeholder_idx: int, num_tokens: int, example_value: torch.Tensor
    ) -> None:
        """Create the static buffer of one token-shaped input, once."""
        if self.input_buffers[batch_idx].get(placeholder_idx) is None:
            self.input_buffers[batch_idx][placeholder_idx] = torch.zeros(
                (num_tokens,) + tuple(example_value.shape[1:]),
                dtype=example_value.dtype,
                device=example_value.device,
            )

    def _bind_placeholder(
        self,
        node: torch.fx.Node,
        batch_idx: int,
        args: tuple,
        env: ExecutionEnvironment,
        split_config: SplitConfig,
    ) -> None:
        """Give nano-batch ``batch_idx`` its view of one graph input.

        Token-shaped tensors (symbolic dim 0) are sliced to the nano-batch's
        rows, or copied into its static buffer under graphs; tensors with a
        static dim 0 (weights) pass whole; a symbolic integer equal to the total
        padded token count becomes this nano-batch's padded count
        (engine.py:441-477).
        """
        idx = self.placeholder_node_to_idx[node]
        example = node.meta.get("example_value", None)
        if isinstance(example, torch.Tensor):
            if not _is_symbolic(example.shape[0]):
                env.put(batch_idx, node, args[idx])
                return
            lo = split_config.split_indices[batch_idx]
            hi = split_config.split_indices[batch_idx + 1]
            if not split_config.use_cudagraph:
                env.put(batch_idx, node, args[idx][lo:hi])
                return
            buf = self.input_buffers[batch_idx].get(idx)
            assert buf is not None, "static input buffer missing: run a dry-run with use_cudagraph first"
            n = split_config.num_tokens[batch_idx]
            buf[:n].copy_(args[idx][lo:hi])
            env.put(batch_idx, node, buf[: split_config.num_tokens_padded[batch_idx]])
        elif _is_symbolic(example):
            if args[idx] == sum(split_config.num_tokens_padded):
                env.put(batch_idx, node, split_config.num_tokens_padded[batch_idx])
            else:
                env.put(batch_idx, node, args[idx])
        else:
            raise ValueError(f"Invalid example value type: {type(example)}")

    # --------------------------------------------------------- inline execution
    @staticmethod
    def _load(env: ExecutionEnvironment, batch_idx: int, value: Any) -> Any:
        return env.get(batch_idx, value) if isinstance(value, torch.fx.Node) else value

    def _execute_non_module(
        self,
        node: torch.fx.Node,
        batch_idx: int,
        args: tuple,
        env: ExecutionEnvironment,
        split_config: SplitConfig,
    ) -> None:
        """Run one node that is not a sub-graph call (engine.py:426-510)."""
        kind = node.op
        if kind == "placeholder":
            self._bind_placeholder(node, batch_idx, args, env, split_config)
        elif kind == "call_function":
            fn = node.target
            assert callable(fn)
            pos = [self._load(env, batch_idx, a) for a in node.args]
            kw = {k: self._load(env, batch_idx, v) for k, v in node.kwargs.items()}
            env.put(batch_idx, node, fn(*pos, **kw))
        elif kind == "call_method":
            assert isinstance(node.target, str)
            receiver = env.get(batch_idx, node.args[0])  # type: ignore[arg-type]
            method = getattr(receiver, node.target)
            assert callable(method)
            pos = [self._load(env, batch_idx, a) for a in node.args[1:]]
            kw = {k: self._load(env, batch_idx, v) for k, v in node.kwargs.items()}
            env.put(batch_idx, node, method(*pos, **kw))
        elif kind == "get_attr":
            assert isinstance(node.target, str)
            env.put(batch_idx, node, self.get_attr_cache[node.target])
        else:
            raise ValueError(f"Invalid node operation: {kind}")

    def _collect_output(self, node: torch.fx.Node, batch_idx: int, env: ExecutionEnvironment) -> Any:
        out = node.args[0]
        if isinstance(out, torch.fx.Node):
            return env.get(batch_idx, out)
        if isinstance(out, (tuple, list)):
            return tuple(self._load(env, batch_idx, item) for item in out)
        return out

    def _handle_for(self, node: torch.fx.Node, batch_idx: int, size: int, split_config: SplitConfig):
        assert isinstance(node.target, str)
        module = getattr(self.graph_module, node.target)
        assert isinstance(module.tag, set)
        return OperatorHandle(
            module_name=node.target,
            batch_idx=batch_idx,
            batch_size=size,
            tag=module.tag,
            _is_dryrun=split_config.is_dryrun,
            _use_cudagraph=split_config.use_cudagraph,
            _owner=id(self),
        )

    def _shared_output_for(self, split_config: SplitConfig, device: Any) -> "_SharedOutput | None":
        """One buffer for the model output of all nano-batches, when the graph allows it: the graph returns the
        result of its last sub-graph call as it is, that result is token-shaped, and no per-sub-graph graph or
        capture-size padding stands between the operator and its output."""
        if not device.is_gpu or split_config.is_dryrun or split_config.use_cudagraph:
            return None
        if not self.config.knob("shared_output", True):
            return None
        if list(split_config.num_tokens_padded) != list(split_config.num_tokens):
            return None
        output = self.nodes[-1]
        if output.op != "output":
            return None
        producer = output.args[0]
        if isinstance(producer, (tuple, list)) and len(producer) == 1:
            producer = producer[0]                       # dynamo graphs return a one-element tuple
        if not isinstance(producer, torch.fx.Node) or producer.op != "call_module" or len(producer.users) != 1:
            return None
        # what the sub-graph returns is recorded inside it (the call node itself carries no example value)
        module = getattr(self.graph_module, producer.target)
        inner = getattr(module, "gm", module)
        if not isinstance(inner, torch.fx.GraphModule):
            return None
        returned = next(n for n in inner.graph.nodes if n.op == "output").args[0]
        if not isinstance(returned, torch.fx.Node):
            return None
        example = returned.meta.get("example_value", None)
        if not isinstance(example, torch.Tensor) or example.dim() < 1 or not _is_symbolic(example.shape[0]):
            return None
        return _SharedOutput(producer.target, split_config, device)

    # ------------------------------------------------------------------ dry-run
    def dryrun(
        self, args: tuple, kwargs: dict, split_config: SplitConfig
    ) -> tuple[dict[int, Any], list[Any]]:
        """Prime backends without a scheduler (engine.py:81-177).

        With ``use_cudagraph`` the same inputs are pushed through
        ``max_num_splits`` fake nano-batches one after the other so that each
        (padded size, nano-batch index) pair captures its graphs against that
        nano-batch's static input buffers.  Only nano-batch 0's result is
        returned.
        """
        assert split_config.num_nano_batches == 1 and split_config.is_dryrun
        device = get_device()
        lanes = self.config.max_num_splits if split_config.use_cudagraph else 1
        num_tokens = split_config.num_tokens_padded[0]
        env = ExecutionEnvironment(lanes)
        events = [device.new_event() for _ in range(lanes)]
        results: dict[int, Any] = {}

        for b in range(lanes):
            for node in self.nodes:
                if node.op == "placeholder":
                    idx = self.placeholder_node_to_idx[node]
                    example = node.meta.get("example_value", None)
                    if _is_symbolic(example):
                        assert args[idx] == num_tokens
                        env.put(b, node, num_tokens)
                        continue
                    assert isinstance(example, torch.Tensor)
                    if not _is_symbolic(example.shape[0]) or not split_config.use_cudagraph:
                        env.put(b, node, args[idx])
                        continue
                    assert num_tokens <= self.max_tokens, (
                        f"{num_tokens} tokens exceed the static buffers ({self.max_tokens}); "
                        "raise additional_config['max_tokens']"
                    )
                    self.allocate_input_buffer(b, idx, self.max_tokens, example)
                    buf = self.input_buffers[b][idx]
                    buf[:num_tokens].copy_(args[idx][:num_tokens])
                    env.put(b, node, buf[:num_tokens])
                elif node.op == "call_module":
                    handle = self._handle_for(node, b, num_tokens, split_config)
                    module = getattr(self.graph_module, node.target)
                    pos = [self._load(env, b, a) for a in node.args]
                    kw = {k: self._load(env, b, v) for k, v in node.kwargs.items()}
                    with set_op_handle(handle):
                        env.put(b, node, module(*pos, **kw))
                elif node.op == "output":
                    results[b] = self._collect_output(node, b, env)
                else:
                    self._execute_non_module(node, b, args, env, split_config)
            events[b].record()
        return {0: results[0]}, events

    # ---------------------------------------------------------------- fast path
    def execute_single_batch(self, split_config: SplitConfig, args: tuple, kwargs: dict) -> Any:
        """One nano-batch, no scheduler: call the split graph directly.

        Under graphs the token-shaped inputs are first copied into nano-batch
        0's static buffers, the very tensors the graphs were captured against
        (engine.py:179-220).
        """
        padded = split_config.num_tokens_padded[0]
        call_args = list(args)
        for node in self.placeholder_nodes:
            idx = self.placeholder_node_to_idx[node]
            example = node.meta.get("example_value", None)
            if _is_symbolic(example):
                if args[idx] == padded:
                    call_args[idx] = padded
            elif (
                isinstance(example, torch.Tensor)
                and _is_symbolic(example.shape[0])
                and split_config.use_cudagraph
            ):
                buf = self.input_buffers[0].get(idx)
                if buf is None:
                    raise RuntimeError(
                        "static input buffer missing: graph replay of an unsplit batch needs a dry-run with "
                        "use_cudagraph at this size first"
                    )
                buf[:padded].copy_(args[idx])
                call_args[idx] = buf[:padded]
        handle = OperatorHandle(
            module_name=type(self.graph_module).__name__,
            batch_idx=0,
            batch_size=padded,
            tag=set(),
            _is_dryrun=False,
            _use_cudagraph=split_config.use_cudagraph,
            _owner=id(self),
        )
        with set_op_handle(handle):
            return self.graph_module(*call_args, **kwargs)

    # ---------------------------------------------------------- scheduled path
    async def execute(
        self,
        args: tuple,
        kwargs: dict,
        op_queue: dict[int, asyncio.Queue],
        execute_queue: asyncio.Queue,
        split_config: SplitConfig,
    ) -> tuple[dict[int, Any], list[Any]]:
        """Producer coroutine of one forward; runs beside ``scheduler.schedule``.

        Returns the per-nano-batch results and each nano-batch's tail event,
        which the caller must wait on before touching the results.
        """
        device = get_device()
        lanes = split_config.num_nano_batches
        env = ExecutionEnvironment(lanes)
        self.last_env = env
        self.issue_trace = []
        results: dict[int, Any] = {}
        tail_events = [device.new_event() for _ in range(lanes)]
        todo: dict[int, deque[torch.fx.Node]] = {b: deque(self.nodes) for b in range(lanes)}
        # operators handed to the scheduler and not yet executed, per nano-batch
        outstanding: dict[int, deque[OperatorHandle]] = {b: deque() for b in range(lanes)}

        async def run_inline_until_op(b: int) -> None:
            """Run inline nodes of ``b`` up to its next sub-graph call / the end."""
            queue = todo[b]
            while queue:
                node = queue[0]
                if node.op == "call_module":
                    return
                if node.op == "output":
                    results[b] = self._collect_output(node, b, env)
                    queue.popleft()
                    await op_queue[b].put(None)
                    return
                self._execute_non_module(node, b, args, env, split_config)
                queue.popleft()

        shared_output = self._shared_output_for(split_config, device)

        # Inputs of every nano-batch are bound up front, on the caller's stream.
        for b in range(lanes):
            queue = todo[b]
            while queue and queue[0].op not in ("call_module", "output"):
                self._execute_non_module(queue[0], b, args, env, split_config)
                queue.popleft()
            tail_events[b].record()

        while any(todo.values()):
            # publish every sub-graph call that heads a nano-batch's list
            for b in range(lanes):
                queue = todo[b]
                while queue and queue[0].op == "call_module" and not op_queue[b].full():
                    handle = self._handle_for(
                        queue[0], b, split_config.num_tokens_padded[b], split_config
                    )
                    await op_queue[b].put(handle)
                    outstanding[b].append(handle)
                    queue.popleft()

            if not any(outstanding.values()):
                # nothing for the scheduler to ask for: only inline work is left
                for b in range(lanes):
                    await run_inline_until_op(b)
                continue

            operators, func, finished = await execute_queue.get()
            if isinstance(operators, OperatorHandle):
                operators = (operators,)

            call_pos: list[list[Any]] = []
            call_kw: list[dict[str, Any]] = []
            for op in operators:
                b = op.batch_idx
                node = self.module_name_to_node[op.module_name]
                # chain: this launch starts after the nano-batch's previous work
                tail_events[b].wait()
                tail_events[b] = device.new_event()
                # only node-valued positional inputs are forwarded (engine.py:304-310)
                pos = [env.get(b, a) for a in node.args if isinstance(a, torch.fx.Node)]
                kw = {k: self._load(env, b, v) for k, v in node.kwargs.items()}
                if device.is_gpu:
                    current = device.current_stream()
                    for value in pos:
                        if isinstance(value, torch.Tensor) and value.is_cuda:
                            value.record_stream(current)
                call_pos.append(pos)
                call_kw.append(kw)

            outputs: list[Any] = []
            if func is not None:
                if len(operators) != 1:
                    raise NotImplementedError("Operator batching is not implemented")
                with set_op_handle(operators[0]):
                    outputs.append(func(*call_pos[0], **call_kw[0]))
            elif len(operators) != 1 and all(
                op.module_name == operators[0].module_name for op in operators
            ):
                raise NotImplementedError("Operator batching is not implemented")
            else:
                for i, op in enumerate(operators):
                    with device.range(f"op_{op.module_name}_{op.batch_idx}"), set_op_handle(op):
                        module = getattr(self.graph_module, op.module_name)
                        offered = shared_output.offer(op) if shared_output is not None else False
                        try:
                            outputs.append(module(*call_pos[i], **call_kw[i]))
                        finally:
                            if offered:
                                shared_output.withdraw()

            for op, value in zip(operators, outputs):
                b = op.batch_idx
                tail_events[b].record()
                env.put(b, self.module_name_to_node[op.module_name], value)
                # per-nano-batch FIFO: the executed handle is the oldest published one
                assert outstanding[b] and op is outstanding[b][0], (
                    f"{op.module_name} of nano-batch {b} executed out of order"
                )
                outstanding[b].popleft()
                self.issue_trace.append((op.module_name, b))

            for b in range(lanes):
                if not outstanding[b]:
                    await run_inline_until_op(b)
            finished.set()

        self.shared_output_buffer = shared_output.buffer if shared_output is not None else None
        return results, tail_events
