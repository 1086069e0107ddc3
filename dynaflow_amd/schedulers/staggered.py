"""Staggered N-way scheduler: nano-batch i runs one sub-graph ahead of i+1.

Follows examples/ae/scheduler/megatron/nanoflow.py: an equal N-way split
(megatron/nanoflow.py:42-76) and a schedule that first advances nano-batch 0 by
one operator and then goes round-robin, popping and issuing one operator at a
time (megatron/nanoflow.py:78-102).  With two kinds of sub-graph alternating
along the graph, neighbouring nano-batches are then always in different kinds,
i.e. on different streams - the pairing "sub-graph k+1 of nano-batch i beside
sub-graph k of nano-batch i+1".
"""
from __future__ import annotations

from dynaflow_amd.config import DynaFlowConfig
from dynaflow_amd.interface import ExecutionContext, InputInfo, OpSchedulerBase, SplitConfig
from dynaflow_amd.matching import MatchingRule
from dynaflow_amd.runtime.device import cu_mask_words, get_device
from dynaflow_amd.schedulers.policies import equal_n_way


class StaggeredScheduler(OpSchedulerBase):
    def __init__(
        self,
        config: DynaFlowConfig,
        split_rules: list[MatchingRule] | None = None,
        tag_rules: dict[MatchingRule, set[str]] | None = None,
        side_tag: str = "network",
    ) -> None:
        super().__init__(policy_name="nanoflow_staggered")
        self.min_nano_split_tokens: int = config.knob("min_nano_split_tokens", 64)
        self.num_nano_batches: int = config.knob("num_nano_batches", 2)
        self._split_rules = list(split_rules or [])
        self._tag_rules = dict(tag_rules or {})
        self.side_tag = side_tag
        device = get_device()
        # "cu_split": n - the side stream may use compute units 0 .. n-1 only and the main stream the others
        # (hard partition, the reference's green-context experiment); unset: both streams may use every unit
        cu_split = config.knob("cu_split", None)
        if cu_split:
            total = int(config.knob("compute_units", 256))
            self.comm_stream = device.new_stream("side", cu_mask_words(0, int(cu_split), total))
            self.comp_stream = device.new_stream("main", cu_mask_words(int(cu_split), total - int(cu_split), total))
        else:
            self.comm_stream = device.new_stream("side")
            self.comp_stream = device.new_stream("main")
        # "by_kind": tagged sub-graphs on the side stream, the others on the main one (the reference's policies);
        # "by_nano_batch": every nano-batch keeps one stream for its whole chain, so that sub-graphs of the same
        # kind of different nano-batches can run side by side as well (with the staggered order they are one
        # sub-graph apart)
        self.stream_policy: str = config.knob("streams", "by_kind")
        if self.stream_policy not in ("by_kind", "by_nano_batch"):
            raise ValueError(f"unknown stream policy {self.stream_policy!r}")
        # "staggered": nano-batch 0 starts one sub-graph ahead; "round_robin": all nano-batches in step
        self.order: str = config.knob("schedule", "staggered")

    def get_split_rules(self) -> list[MatchingRule]:
        return self._split_rules

    def get_tag_rules(self) -> dict[MatchingRule, set[str]]:
        return self._tag_rules

    def get_split_config(self, input_info: InputInfo, use_cudagraph: bool = False) -> SplitConfig:
        return equal_n_way(input_info, use_cudagraph, self.num_nano_batches, self.min_nano_split_tokens)

    def _stream_for(self, op):
        if self.stream_policy == "by_nano_batch" and self.comm_stream is not self.comp_stream:
            return self.comm_stream if op.batch_idx % 2 else self.comp_stream
        return self.comm_stream if self.side_tag in op.tag else self.comp_stream

    async def _issue(self, context: ExecutionContext, op) -> None:
        with get_device().stream(self._stream_for(op)):
            await context.execute((op,))

    async def schedule(self, context: ExecutionContext) -> None:
        lanes = context.split_config.num_nano_batches
        live = list(range(lanes))
        if lanes >= 2 and self.order != "round_robin":
            head = await context.pop(0)
            if head is None:
                live.remove(0)
            else:
                await self._issue(context, head)
        while live:
            for b in list(live):
                op = await context.pop(b)
                if op is None:
                    live.remove(b)
                    continue
                await self._issue(context, op)
