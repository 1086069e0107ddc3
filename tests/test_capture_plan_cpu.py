"""From which stream a schedule can be captured as one graph: the event logs of the shipped schedules on the
recording device, and what the plan makes of them.

A capture dies at its end when a stream other than the one the capture started on waits for an event it
recorded itself, or when two such streams wait for each other's events.  The schedules below are the ones that
were captured successfully on an MI355X (no such cycle from the caller's side) and the ones whose capture
ended in a segmentation fault (each has one)."""
import pytest
import torch

from dynaflow_amd.runtime import capture_plan as plan

from test_decode_cpu import decode_inputs, small_model
from test_engine_cpu import compile_mlp, make_config


def mlp_log(host_device, splits, **knobs):
    cfg = make_config(splits, num_nano_batches=splits, **knobs)
    model, manager, compiled, x = compile_mlp(cfg, tokens=96)
    manager.prepare(96, [96])
    host_device.log.clear()
    with torch.no_grad():
        compiled(x)
    return [e for e in host_device.log if e[0] in ("record", "wait")]


def decode_log(host_device, **knobs):
    from dynaflow_amd.backend import make_backend
    from dynaflow_amd.config import CUDAGraphConfig, DynaFlowConfig, InductorConfig
    from dynaflow_amd.manager import DynaFlowManager

    model, T = small_model(), 6
    inputs = decode_inputs(T)
    cfg = DynaFlowConfig("dynaflow_amd.schedulers:DecoderOverlapScheduler", 2, InductorConfig(enabled=False),
                         CUDAGraphConfig(enabled=False, capture_sizes=[T]),
                         {"min_nano_split_tokens": 1, "dump_graph": False, "hip_backend": False, **knobs})
    manager = DynaFlowManager()
    torch._dynamo.reset()
    for t in inputs:
        torch._dynamo.mark_dynamic(t, 0)
    compiled = torch.compile(model, backend=make_backend(manager, cfg), fullgraph=True)
    with torch.no_grad():
        manager.prepare(T, [1] * T)
        compiled(*inputs)
        manager.prepare(T, [1] * T)
        host_device.log.clear()
        compiled(*inputs)
    return [e for e in host_device.log if e[0] in ("record", "wait")]


def test_hand_made_logs():
    # origin O, streams A and B
    fork_join = [("record", 1, "O"), ("wait", 1, "A"), ("record", 2, "A"), ("wait", 2, "B"), ("record", 3, "B"),
                 ("wait", 3, "O")]
    assert plan.wait_edges(fork_join) == [("O", "A"), ("A", "B"), ("B", "O")]
    assert plan.join_cycle(fork_join, "O", "O") is None and plan.choose_origin(fork_join, "O") == "O"
    # A and B wait for each other: a cycle from O, none when the capture starts on A or on B
    ping_pong = fork_join[:5] + [("wait", 3, "A"), ("record", 4, "A"), ("wait", 4, "O")]
    assert plan.join_cycle(ping_pong, "O", "O") == ["A", "B", "A"]
    assert plan.join_cycle(ping_pong, "O", "A") is None and plan.join_cycle(ping_pong, "O", "B") is None
    assert plan.choose_origin(ping_pong, "O") == "A"
    # a wait on the recording stream is never issued, so it is no edge
    own = [("record", 1, "O"), ("wait", 1, "A"), ("record", 2, "A"), ("wait", 2, "A"), ("record", 3, "A"),
           ("wait", 3, "O")]
    assert plan.join_cycle(own, "O", "O") is None
    # a ring of three streams is cut open by starting on any of them
    ring = [("record", 1, "O"), ("wait", 1, "A"), ("record", 2, "A"), ("wait", 2, "B"), ("record", 3, "B"),
            ("wait", 3, "C"), ("record", 4, "C"), ("wait", 4, "A"), ("record", 5, "A"), ("wait", 5, "O")]
    assert plan.join_cycle(ring, "O", "O") == ["A", "B", "C", "A"] and plan.choose_origin(ring, "O") == "A"
    # two pairs that each wait for each other: whichever stream the capture starts on, one pair remains
    pairs = [("record", 1, "O"), ("wait", 1, "A"), ("wait", 1, "C"),
             ("record", 2, "A"), ("wait", 2, "B"), ("record", 3, "B"), ("wait", 3, "A"),
             ("record", 4, "C"), ("wait", 4, "D"), ("record", 5, "D"), ("wait", 5, "C"),
             ("record", 6, "A"), ("wait", 6, "O"), ("record", 7, "C"), ("wait", 7, "O")]
    assert plan.choose_origin(pairs, "O") is None
    # a wait for an event that was never recorded orders nothing
    assert plan.wait_edges([("wait", 9, "A")]) == []


@pytest.mark.parametrize("splits", [2, 3, 4])
def test_two_segment_schedules_capture_from_the_callers_side(host_device, splits):
    log = mlp_log(host_device, splits)
    assert sorted(set(plan.wait_edges(log))) == [("default", "main"), ("main", "side"), ("side", "default")]
    assert plan.choose_origin(log, "default") == "default"


@pytest.mark.parametrize("knobs", [dict(serialize=True), dict(streams="by_nano_batch")])
def test_schedules_that_keep_a_nano_batch_on_one_stream(host_device, knobs):
    """Their only offence is the wait on the recording stream, which the GPU seam does not issue."""
    log = mlp_log(host_device, 2, **knobs)
    own = [(a, b) for a, b in plan.wait_edges(log) if a == b]
    assert own and all(a != "default" for a, _ in own)
    assert plan.choose_origin(log, "default") == "default"


def test_by_nano_batch_with_four_nano_batches(host_device):
    log = mlp_log(host_device, 4, streams="by_nano_batch")
    assert plan.choose_origin(log, "default") == "default"


def test_multi_layer_schedule_by_kind_is_captured_from_its_main_stream(host_device):
    """Attention sub-graphs on one stream, MLP sub-graphs on the other, layer after layer: the two streams wait
    for each other, so neither may be a bystander of a capture started elsewhere."""
    log = decode_log(host_device)
    edges = set(plan.wait_edges(log))
    assert ("main", "side") in edges and ("side", "main") in edges
    assert plan.join_cycle(log, "default", "default") == ["main", "side", "main"]
    assert plan.choose_origin(log, "default") == "main"


def test_multi_layer_schedule_by_nano_batch(host_device):
    log = decode_log(host_device, streams="by_nano_batch")
    assert plan.choose_origin(log, "default") == "default"
