"""Scheduler for one decoder layer: attention of one nano-batch beside the MLP of the other.

The graph of ``dynaflow_amd.decoder.DecoderLayer`` is cut with a single ``Mod`` rule: the run of
nodes traced from the ``MLPBlock`` instance becomes a sub-graph of its own (tag ``mlp``, second
stream), everything in front of it (embedding, attention block) is the other one.  The split is
the balanced two-way cut at a request (sequence) boundary, the order is the staggered one, so the
issue order is  (attn, b0) (mlp, b0) (attn, b1) (mlp, b1)  with (attn, b1) beside (mlp, b0).

``Mod`` is the module-stack condition of dynaflow/matching.py:19-50; the balanced cut is the
split policy of examples/ae/scheduler/hf/nanoflow.py:65-120, the order that of
examples/ae/scheduler/megatron/nanoflow.py:78-102; two sub-graphs with different resource profiles
side by side is the case examples/ae/OVERLAP.md:161-176 argues for.
"""
from __future__ import annotations

from dynaflow_amd.config import DynaFlowConfig
from dynaflow_amd.decoder import MLPBlock
from dynaflow_amd.interface import InputInfo, SplitConfig
from dynaflow_amd.matching import MatchingRule, Mod
from dynaflow_amd.schedulers.policies import balanced_two_way
from dynaflow_amd.schedulers.staggered import StaggeredScheduler

MLP_TAG = "mlp"


def decoder_split_rules() -> list[MatchingRule]:
    return [MatchingRule(condition=Mod(MLPBlock))]


def _starts_at_compute_node(nodes, start: int) -> bool:
    # Inside a sub-graph the placeholder that brings in the previous MLP block's output carries that
    # block's module stack; without this veto the attention sub-graph of the next layer would match
    # the Mod condition on that placeholder and be tagged as well.
    return nodes[start].op != "placeholder"


def decoder_tag_rules() -> dict[MatchingRule, set[str]]:
    return {MatchingRule(condition=Mod(MLPBlock), hook=_starts_at_compute_node): {MLP_TAG}}


class DecoderOverlapScheduler(StaggeredScheduler):
    def __init__(self, config: DynaFlowConfig) -> None:
        super().__init__(config, decoder_split_rules(), decoder_tag_rules(), side_tag=MLP_TAG)
        self.policy_name = "decoder_overlap"
        self.capture_sizes = config.cudagraph_config.capture_sizes
        if config.knob("serialize", False):
            self.comm_stream = self.comp_stream

    def get_split_config(self, input_info: InputInfo, use_cudagraph: bool = False) -> SplitConfig:
        return balanced_two_way(input_info, use_cudagraph, self.min_nano_split_tokens, self.capture_sizes or [0])
