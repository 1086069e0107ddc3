"""Round-robin two-stream scheduler (the NanoFlow policy).

Follows examples/ae/scheduler/hf/nanoflow.py: a balanced two-way split
(hf/nanoflow.py:65-120) and a schedule that, round after round, pops one ready
operator from every live nano-batch and then issues them in that order, each on
the stream its tags select (hf/nanoflow.py:122-146).  Which tag goes to the
second stream and which graph nodes are cut out are constructor parameters,
so the class serves any pair of resource classes (network/compute in the
reference, GEMM/elementwise here).
"""
from __future__ import annotations

from dynaflow_amd.config import DynaFlowConfig
from dynaflow_amd.interface import ExecutionContext, InputInfo, OpSchedulerBase, SplitConfig
from dynaflow_amd.matching import MatchingRule
from dynaflow_amd.runtime.device import get_device
from dynaflow_amd.schedulers.policies import balanced_two_way


class NanoFlowScheduler(OpSchedulerBase):
    def __init__(
        self,
        config: DynaFlowConfig,
        split_rules: list[MatchingRule] | None = None,
        tag_rules: dict[MatchingRule, set[str]] | None = None,
        side_tag: str = "network",
    ) -> None:
        super().__init__(policy_name="nanoflow")
        self.min_nano_split_tokens = config.knob("min_nano_split_tokens", 64)
        self.max_num_nano_batches = config.max_num_splits
        self.cudagraph_capture_sizes = config.cudagraph_config.capture_sizes
        self._split_rules = list(split_rules or [])
        self._tag_rules = dict(tag_rules or {})
        self.side_tag = side_tag
        device = get_device()
        self.comm_stream = device.new_stream("side")
        self.comp_stream = device.new_stream("main")

    def get_split_rules(self) -> list[MatchingRule]:
        return self._split_rules

    def get_tag_rules(self) -> dict[MatchingRule, set[str]]:
        return self._tag_rules

    def get_split_config(self, input_info: InputInfo, use_cudagraph: bool) -> SplitConfig:
        assert self.cudagraph_capture_sizes
        return balanced_two_way(
            input_info, use_cudagraph, self.min_nano_split_tokens, self.cudagraph_capture_sizes
        )

    def _stream_for(self, op):
        return self.comm_stream if self.side_tag in op.tag else self.comp_stream

    async def schedule(self, context: ExecutionContext) -> None:
        device = get_device()
        live = list(range(context.split_config.num_nano_batches))
        while live:
            ready = []
            for b in list(live):
                op = await context.pop(b)
                if op is None:
                    live.remove(b)
                else:
                    ready.append(op)
            for op in ready:
                with device.stream(self._stream_for(op)):
                    await context.execute((op,))
