"""Scheduler for the batch-split SwiGLU MLP: GEMM beside SiLU*mul + down-proj.

The graph ``g = gate(x); u = up(x); y = down(silu(g) * u)`` is cut in front of
``silu`` so that every nano-batch consists of two sub-graphs:

    submod_0  gate and up projection          (no tag)         -> stream "main"
    submod_1  SiLU*mul and down projection    (tag "tail")     -> stream "side"

and the staggered order of ``StaggeredScheduler`` issues
``(s0,b0) (s1,b0) (s0,b1) (s1,b1) ...``: nano-batch i+1's gate/up GEMM runs
beside nano-batch i's SiLU*mul and down projection.  ``schedule="round_robin"``
selects the NanoFlow order instead; both give the same per-stream order.

With ``additional_config["fuse_silu_epilogue"]`` the cut moves in front of the down
projection ({gate, up, silu, mul} | {down}) and the lowering turns the first sub-graph into
one GEMM with the SiLU*mul as its epilogue; nano-batch i+1's fused GEMM then runs beside
nano-batch i's down projection.

Split policy: ``additional_config["num_nano_batches"]`` equal chunks (default
``max_num_splits``); with ``split_policy="balanced"`` the two-way balanced cut
at a request boundary.

A policy file in the shape of the reference's own (rules and hooks like
examples/ae/scheduler/hf/nanoflow.py:46-62, streams picked from the tag like :138-146, the
staggered order of examples/ae/scheduler/megatron/nanoflow.py:78-102); which two kinds of work
may share the compute units follows the rule of examples/ae/OVERLAP.md:161-176.
"""
from __future__ import annotations

from dynaflow_amd.config import DynaFlowConfig
from dynaflow_amd.interface import ExecutionContext, InputInfo, SplitConfig
from dynaflow_amd.matching import MatchingRule, Op
from dynaflow_amd.schedulers.nanoflow import NanoFlowScheduler
from dynaflow_amd.schedulers.policies import balanced_two_way, equal_n_way
from dynaflow_amd.schedulers.staggered import StaggeredScheduler

_LINEAR = r"linear(\.default)?"
_SILU = r"silu(\.default)?"
_MUL = r"mul(\.Tensor)?"

TAIL_TAG = "tail"
HEAD_TAG = "head"


def mlp_split_rules() -> list[MatchingRule]:
    return [
        # silu -> mul -> down projection traced back to back
        MatchingRule(condition=(Op(_SILU), Op(_MUL), Op(_LINEAR))),
        # silu traced between the two projections: cut at the product instead
        MatchingRule(condition=(Op(_MUL), Op(_LINEAR))),
        # already fused elementwise operator
        MatchingRule(condition=(Op(r"silu_mul(\.default)?"), Op(_LINEAR))),
        # fp8 block: SiLU*mul + re-quantisation, then the fp8 down projection
        MatchingRule(condition=(Op(r"silu_mul_quant_fp8(\.default)?"), Op(r"linear_fp8(\.default)?"))),
    ]


def _follows_product(node_list, start_idx: int) -> bool:
    """True for a ``linear`` whose input is the SiLU*mul product (the down projection)."""
    node = node_list[start_idx]
    producer = node.args[0] if node.args else None
    name = getattr(getattr(producer, "target", None), "__name__", "")
    if name == "getitem" and getattr(producer, "args", None):     # first output of an operator with two
        producer = producer.args[0]
        name = getattr(getattr(producer, "target", None), "__name__", "")
    return getattr(producer, "op", None) == "call_function" and name.split(".")[0] in (
        "mul", "silu_mul", "gate_up_silu", "gate_up_silu_quant_fp8")


def mlp_split_rules_fused() -> list[MatchingRule]:
    """Cut only in front of the down projection: {gate, up, silu, mul} | {down}, so that the
    SiLU*mul can become the epilogue of the gate/up GEMM."""
    return [MatchingRule(condition=Op(_LINEAR), hook=_follows_product),
            MatchingRule(condition=Op(r"linear_fp8(\.default)?"), hook=_follows_product)]


def mlp_tag_rules_fused() -> dict[MatchingRule, set[str]]:
    # inside the down-projection sub-graph the product is just an input, so the sub-graph that
    # holds the product is the one that gets a tag (and the second stream)
    return {MatchingRule(condition=Op(_MUL)): {HEAD_TAG},
            MatchingRule(condition=Op(r"gate_up_silu_quant_fp8(\.default)?")): {HEAD_TAG}}


def mlp_tag_rules() -> dict[MatchingRule, set[str]]:
    return {
        MatchingRule(condition=Op(_MUL)): {TAIL_TAG},
        MatchingRule(condition=Op(r"silu_mul(\.default)?")): {TAIL_TAG},
        MatchingRule(condition=Op(r"silu_mul_quant_fp8(\.default)?")): {TAIL_TAG},
    }


class MLPOverlapScheduler(StaggeredScheduler):
    def __init__(self, config: DynaFlowConfig) -> None:
        if config.knob("fuse_silu_epilogue", False):
            super().__init__(config, mlp_split_rules_fused(), mlp_tag_rules_fused(), side_tag=HEAD_TAG)
        else:
            super().__init__(config, mlp_split_rules(), mlp_tag_rules(), side_tag=TAIL_TAG)
        self.policy_name = "mlp_overlap"
        self.num_nano_batches = config.knob("num_nano_batches", config.max_num_splits)
        self.split_policy = config.knob("split_policy", "equal")
        self.order = config.knob("schedule", "staggered")
        self.capture_sizes = config.cudagraph_config.capture_sizes
        self.serialize = bool(config.knob("serialize", False))
        if self.serialize:
            # debugging / baseline mode: every launch on one stream
            self.comm_stream = self.comp_stream

    def get_split_config(self, input_info: InputInfo, use_cudagraph: bool = False) -> SplitConfig:
        if self.split_policy == "balanced":
            return balanced_two_way(
                input_info, use_cudagraph, self.min_nano_split_tokens, self.capture_sizes or [0]
            )
        return equal_n_way(input_info, use_cudagraph, self.num_nano_batches, self.min_nano_split_tokens)

    async def schedule(self, context: ExecutionContext) -> None:
        if self.order == "round_robin":
            await NanoFlowScheduler.schedule(self, context)  # type: ignore[arg-type]
        else:
            await super().schedule(context)
