"""Host logic of a forward on the recording device seam: the engine + shipped
schedulers must produce the launch order and event chain the oracle derives,
and the results of eager PyTorch on the unsplit input."""
import asyncio

import pytest
import torch

from dynaflow_amd.backend import make_backend
from dynaflow_amd.config import CUDAGraphConfig, DynaFlowConfig, InductorConfig
from dynaflow_amd.interface import ExecutionContext, OpSchedulerBase, SplitConfig
from dynaflow_amd.manager import DynaFlowManager
from dynaflow_amd.mlp import SwiGLUMLP
from dynaflow_amd.schedulers import MLPOverlapScheduler
from dynaflow_amd.schedulers.mlp_overlap import mlp_split_rules, mlp_tag_rules
from oracle import schedule_trace as ref


def make_config(splits=2, **extra):
    knobs = {"min_nano_split_tokens": 8, "dump_graph": False}
    knobs.update(extra)
    return DynaFlowConfig("dynaflow_amd.schedulers:MLPOverlapScheduler", splits,
                          InductorConfig(enabled=False), CUDAGraphConfig(enabled=False, capture_sizes=[64, 128]), knobs)


def compile_mlp(cfg, tokens=64, hidden=32, inter=96, scheduler=None):
    torch._dynamo.reset()
    torch.manual_seed(0)
    model = SwiGLUMLP(hidden, inter, dtype=torch.float32)
    manager = DynaFlowManager()
    x = torch.randn(tokens, hidden)
    torch._dynamo.mark_dynamic(x, 0)
    compiled = torch.compile(model, backend=make_backend(manager, cfg, scheduler), fullgraph=True)
    manager.prepare(tokens, [tokens])  # not initialised yet: trivial split, used by the tracing call
    with torch.no_grad():
        compiled(x)
    return model, manager, compiled, x


def top_level(manager):
    top = []
    for node in manager.graph_module.graph.nodes:
        if node.op == "placeholder":
            top.append("in")
        elif node.op == "call_module":
            top.append(("mod", node.target))
        elif node.op == "output":
            top.append("out")
        else:
            top.append("fn")
    return top


@pytest.mark.parametrize("order,splits", [("staggered", 2), ("round_robin", 2), ("staggered", 4), ("round_robin", 3)])
def test_launch_order_and_streams_match_oracle(host_device, order, splits):
    cfg = make_config(splits, schedule=order, num_nano_batches=splits)
    model, manager, compiled, x = compile_mlp(cfg, tokens=96)
    split = manager.prepare(96, [96])
    assert split.num_nano_batches == splits
    host_device.log.clear()
    with torch.no_grad():
        y = compiled(x)
    assert manager.cached_config is None, "the split is consumed by the forward"
    torch.testing.assert_close(y, model(x), rtol=0, atol=0)

    want = ref.simulate(top_level(manager), splits, order,
                        lambda m: "side" if "tail" in getattr(manager.graph_module, m).tag else "main",
                        caller_stream="default")
    ranges = [(e[1], e[2]) for e in host_device.log if e[0] == "range"]
    got_launches = [(name.rsplit("_", 1)[0][3:], int(name.rsplit("_", 1)[1]), stream) for name, stream in ranges]
    assert got_launches == ref.launches(want)
    assert manager.engine.issue_trace == [(m, b) for m, b, _ in ref.launches(want)]

    # the full event chain: map event uids to nano-batches through the order of creation
    kinds = [(e[0], e[2]) for e in host_device.log if e[0] in ("record", "wait")]
    want_kinds = [("record" if e[0] == "record" else "wait", e[2]) for e in want if e[0] in ("record", "wait", "join")]
    assert kinds == want_kinds
    # a wait always refers to the event its nano-batch recorded last
    last_record = {}
    launch_iter = iter(ref.launches(want))
    for e in host_device.log:
        if e[0] == "record":
            last_record[e[1]] = e[2]
        elif e[0] == "wait":
            assert e[1] in last_record, "waited on an event that was never recorded"


def test_environment_is_drained(host_device):
    cfg = make_config(2)
    model, manager, compiled, x = compile_mlp(cfg)
    manager.prepare(64, [64])
    with torch.no_grad():
        compiled(x)
    assert manager.engine.last_env.live_entries() == []


def test_single_batch_takes_fast_path_and_bypasses_scheduler(host_device):
    cfg = make_config(2, min_nano_split_tokens=1000)
    model, manager, compiled, x = compile_mlp(cfg)
    split = manager.prepare(64, [64])
    assert split.num_nano_batches == 1
    host_device.log.clear()
    with torch.no_grad():
        y = compiled(x)
    assert [e for e in host_device.log if e[0] == "range"] == []
    torch.testing.assert_close(y, model(x), rtol=0, atol=0)


def test_single_batch_graph_replay_without_a_capturing_dry_run_is_refused(host_device):
    cfg = make_config(2, min_nano_split_tokens=1000)
    model, manager, compiled, x = compile_mlp(cfg)
    manager.prepare(64, [64], use_cudagraph=True)
    with torch.no_grad(), pytest.raises(RuntimeError, match="static input buffer missing"):
        compiled(x)


def test_single_batch_through_scheduler_when_fallback_disallowed(host_device):
    cfg = make_config(2, min_nano_split_tokens=1000)
    model, manager, compiled, x = compile_mlp(cfg)
    split = manager.prepare(64, [64])
    split.allow_fallback = False
    manager.override_split_config(split)
    with torch.no_grad():
        y = compiled(x)
    assert manager.engine.issue_trace == [("submod_0", 0), ("submod_1", 0)]
    torch.testing.assert_close(y, model(x), rtol=0, atol=0)


def test_forward_without_prepare_fails(host_device):
    cfg = make_config(2)
    model, manager, compiled, x = compile_mlp(cfg)
    with pytest.raises(AssertionError):
        compiled(x)


def test_uneven_split_rows_land_in_order(host_device):
    cfg = make_config(2)
    model, manager, compiled, x = compile_mlp(cfg, tokens=50)
    manager.override_split_config(SplitConfig(2, [13, 37], [0, 13, 50], [13, 37], [13, 37], [0, 13, 50], False, False))
    with torch.no_grad():
        y = compiled(x)
    torch.testing.assert_close(y, model(x), rtol=0, atol=0)


def test_dryrun_returns_whole_batch(host_device):
    cfg = make_config(2)
    model, manager, compiled, x = compile_mlp(cfg)
    split = manager.prepare(64, [64], is_dryrun=True)
    assert split.is_dryrun and split.num_nano_batches == 1
    with torch.no_grad():
        y = compiled(x)
    torch.testing.assert_close(y, model(x), rtol=0, atol=0)


class _OutOfOrder(MLPOverlapScheduler):
    async def schedule(self, context: ExecutionContext) -> None:
        first = await context.pop(0)
        await context.execute((first,))
        second = await context.pop(0)
        # executing the first handle again violates the per-nano-batch FIFO
        await context.execute((first,))


def test_out_of_order_execution_is_caught(host_device):
    cfg = make_config(2)
    model, manager, compiled, x = compile_mlp(cfg, scheduler=_OutOfOrder(cfg))
    manager.prepare(64, [64])
    with pytest.raises((AssertionError, KeyError)):
        compiled(x)


class _Substituting(MLPOverlapScheduler):
    calls = 0

    async def schedule(self, context: ExecutionContext) -> None:
        live = list(range(context.split_config.num_nano_batches))
        while live:
            for b in list(live):
                op = await context.pop(b)
                if op is None:
                    live.remove(b)
                    continue
                if "tail" in op.tag:
                    def tail(gate, size, up, w_down):
                        _Substituting.calls += 1
                        assert isinstance(size, int) and gate.shape[0] == size
                        return torch.nn.functional.linear(torch.nn.functional.silu(gate) * up, w_down)
                    await context.execute((op,), tail)
                else:
                    await context.execute(op)  # a bare handle is accepted too


def test_operator_substitution_gets_node_inputs_in_graph_order(host_device):
    cfg = make_config(2)
    model, manager, compiled, x = compile_mlp(cfg, scheduler=_Substituting(cfg))
    manager.prepare(64, [64])
    _Substituting.calls = 0
    with torch.no_grad():
        y = compiled(x)
    assert _Substituting.calls == 2
    torch.testing.assert_close(y, model(x), rtol=1e-6, atol=1e-6)


class _Quitter(MLPOverlapScheduler):
    async def schedule(self, context: ExecutionContext) -> None:
        op = await context.pop(0)
        await context.execute((op,))


def test_scheduler_that_returns_early_leaves_engine_waiting(host_device):
    """Failure detection on the host: the engine blocks on the execute queue; a
    caller that bounds the forward with a time-out sees it."""
    cfg = make_config(2)
    model, manager, compiled, x = compile_mlp(cfg, scheduler=_Quitter(cfg))
    split = manager.prepare(64, [64])

    async def bounded():
        args = (model.gate_proj.weight, 64, x, model.up_proj.weight, model.down_proj.weight)
        placeholders = [n.name for n in manager.engine.placeholder_nodes]
        assert len(placeholders) == len(args)
        await asyncio.wait_for(manager._forward_async(args, {}, split), timeout=0.5)

    with pytest.raises(asyncio.TimeoutError):
        asyncio.run(bounded())


def test_join_results_skips_the_copy_for_consecutive_rows_of_one_buffer():
    from dynaflow_amd.manager import join_results

    buf = torch.arange(24.0).reshape(6, 4).clone()
    parts = {0: buf[0:2], 1: buf[2:5], 2: buf[5:6]}
    joined = join_results(parts, 3, buf)
    assert joined.data_ptr() == buf.data_ptr() and torch.equal(joined, buf)
    # views with more dimensions (sequences x positions x hidden) of the same rows
    joined3 = join_results({0: buf[0:4].view(2, 2, 4), 1: buf[4:6].view(1, 2, 4)}, 2, buf)
    assert joined3.data_ptr() == buf.data_ptr() and joined3.shape == (3, 2, 4)
    # a one-element tuple per nano-batch (what a dynamo graph returns)
    (field,) = join_results({0: (buf[0:3],), 1: (buf[3:6],)}, 2, buf)
    assert field.data_ptr() == buf.data_ptr()
    # rows of a buffer that is not the engine's own (say, views of an input) are copied like torch.cat does
    assert join_results({0: buf[0:3], 1: buf[3:6]}, 2).data_ptr() != buf.data_ptr()
    # anything else is concatenated: a gap, a wrong order, separate tensors, part of a larger buffer
    for parts in ({0: buf[0:2], 1: buf[3:6]}, {0: buf[3:6], 1: buf[0:3]}, {0: buf[0:3].clone(), 1: buf[3:6].clone()},
                  {0: buf[0:2], 1: buf[2:4]}):
        joined = join_results(parts, 2, buf)
        assert joined.data_ptr() != buf.data_ptr()
        assert torch.equal(joined, torch.cat([parts[0], parts[1]], dim=0))


_REFERENCE_STYLE_POLICY = '''
"""A policy file written against the reference package's import names (not this build's)."""
from typing_extensions import override

from dynaflow.config import DynaFlowConfig
from dynaflow.interface import ExecutionContext, InputInfo, OpSchedulerBase, SplitConfig
from dynaflow.matching import MatchingRule, Op
from dynaflow.utils import pack_tokens


class TwoWay(OpSchedulerBase):
    def __init__(self, config: DynaFlowConfig) -> None:
        super().__init__(policy_name="two_way")
        self.capture_sizes = config.cudagraph_config.capture_sizes

    @override
    def get_split_rules(self) -> list[MatchingRule]:
        return [MatchingRule(condition=(Op("silu"), Op("mul"), Op("linear")))]

    @override
    def get_tag_rules(self) -> dict[MatchingRule, set[str]]:
        return {MatchingRule(condition=Op("mul")): {"tail"}}

    @override
    def get_split_config(self, input_info: InputInfo, use_cudagraph: bool = False) -> SplitConfig:
        total = sum(input_info.num_tokens)
        left = total // 2
        padded, fits = pack_tokens(left, self.capture_sizes)
        assert fits and padded >= left
        return SplitConfig(num_nano_batches=2, batch_sizes=[1, 1], batch_indices=[0, 1, 2],
                           num_tokens=[left, total - left], num_tokens_padded=[left, total - left],
                           split_indices=[0, left, total], is_dryrun=False, use_cudagraph=False)

    @override
    async def schedule(self, context: ExecutionContext) -> None:
        live = [0, 1]
        while live:
            for b in list(live):
                op = await context.pop(b)
                if op is None:
                    live.remove(b)
                    continue
                await context.execute((op,))
'''


def test_policy_file_written_against_the_reference_package_names_runs_unmodified(host_device, tmp_path):
    import sys

    import dynaflow_amd

    path = tmp_path / "two_way_policy.py"
    path.write_text(_REFERENCE_STYLE_POLICY)
    dynaflow_amd.install_as_dynaflow()
    try:
        import dynaflow.executor.cudagraph as graphs  # the reference's module name for the graph wrapper

        assert hasattr(graphs, "CUDAGraphWrapper")
        cfg = DynaFlowConfig(f"{path}:TwoWay", 2, InductorConfig(enabled=False),
                             CUDAGraphConfig(enabled=False, capture_sizes=[64, 128]),
                             {"min_nano_split_tokens": 8, "dump_graph": False})
        model, manager, compiled, x = compile_mlp(cfg, tokens=96)
        assert type(manager.scheduler).__name__ == "TwoWay" and manager.scheduler.policy_name == "two_way"
        split = manager.prepare(96, [96])
        assert split.split_indices == [0, 48, 96]
        with torch.no_grad():
            got = compiled(x)
            want = model(x)
        assert torch.allclose(got, want, atol=1e-6)
        assert manager.engine.issue_trace == [("submod_0", 0), ("submod_0", 1), ("submod_1", 0), ("submod_1", 1)]
    finally:
        for name in [n for n in sys.modules if n == "dynaflow" or n.startswith("dynaflow.")]:
            del sys.modules[name]


def test_one_stream_per_nano_batch_policy(host_device):
    """``streams="by_nano_batch"``: every launch of nano-batch 0 on the main stream, of nano-batch 1 on the side
    stream, whatever the sub-graph's tag; the issue order stays the staggered one and the result the same."""
    cfg = make_config(2, streams="by_nano_batch")
    model, manager, compiled, x = compile_mlp(cfg, tokens=96)
    manager.prepare(96, [96])
    host_device.log.clear()
    with torch.no_grad():
        y = compiled(x)
    torch.testing.assert_close(y, model(x), rtol=0, atol=0)
    ranges = [(e[1], e[2]) for e in host_device.log if e[0] == "range"]
    launches = [(name.rsplit("_", 1)[0][3:], int(name.rsplit("_", 1)[1]), stream) for name, stream in ranges]
    assert launches == [("submod_0", 0, "main"), ("submod_1", 0, "main"), ("submod_0", 1, "side"),
                        ("submod_1", 1, "side")]
    with pytest.raises(ValueError):
        MLPOverlapScheduler(make_config(2, streams="per_kernel"))


def test_compute_unit_split_gives_the_two_streams_disjoint_masks(host_device):
    """``cu_split=n``: the side stream gets compute units 0 .. n-1, the main stream the others (the counterpart of
    the reference's green contexts, examples/ae/up-silu-overlap.cu:236-264); unset, the streams carry no mask."""
    from dynaflow_amd.runtime.device import cu_mask_words

    assert cu_mask_words(0, 32, 256) == [0xFFFFFFFF, 0, 0, 0, 0, 0, 0, 0]
    assert cu_mask_words(40, 24, 256) == [0, 0xFFFFFF00, 0, 0, 0, 0, 0, 0]
    assert cu_mask_words(224, 32, 256)[7] == 0xFFFFFFFF
    with pytest.raises(ValueError):
        cu_mask_words(250, 16, 256)
    plain = MLPOverlapScheduler(make_config(2))
    assert plain.comm_stream.cu_mask is None and plain.comp_stream.cu_mask is None
    split = MLPOverlapScheduler(make_config(2, cu_split=48))
    side, main = split.comm_stream.cu_mask, split.comp_stream.cu_mask
    assert len(side) == len(main) == 8
    as_int = lambda words: sum(w << (32 * i) for i, w in enumerate(words))
    assert as_int(side) == (1 << 48) - 1
    assert as_int(side) & as_int(main) == 0 and as_int(side) | as_int(main) == (1 << 256) - 1


def test_listed_sizes_get_their_own_callable_in_a_dry_run(host_device):
    """``InductorConfig.compile_sizes`` (dynaflow/executor/compiler.py:69-85): a dry-run at a listed size builds
    that size's callable; scheduled forwards whose nano-batches have that size dispatch to it, other sizes go to
    the dynamic callable; outside a dry-run an unbuilt listed size is an error."""
    cfg = make_config(2)
    cfg.inductor_config.compile_sizes = {48}
    model, manager, compiled, x = compile_mlp(cfg, tokens=96)
    backends = [manager.graph_module.__dict__[n.target] for n in manager.graph_module.graph.nodes
                if n.op == "call_module"]
    assert all(b.callables_per_size == {} for b in backends)

    # a scheduled forward with nano-batches of the listed size before any dry-run: refused
    manager.prepare(96, [96])
    with pytest.raises(AssertionError, match="dry-run"):
        with torch.no_grad():
            compiled(x)

    # the dry-run at 48 tokens builds the callable of that size in every sub-graph
    small = x[:48].clone()
    manager.prepare(48, [48], is_dryrun=True)
    with torch.no_grad():
        dry = compiled(small)
    torch.testing.assert_close(dry, model(small), rtol=0, atol=0)
    assert all(sorted(b.callables_per_size) == [48] for b in backends)

    # count the calls each callable gets from now on
    calls = {"sized": 0, "dynamic": 0}
    for b in backends:
        sized, dynamic = b.callables_per_size[48], b.callable_dynamic

        def counted(fn, key):
            def call(*a, **k):
                calls[key] += 1
                return fn(*a, **k)
            return call

        b.callables_per_size[48] = counted(sized, "sized")
        b.callable_dynamic = counted(dynamic, "dynamic")

    split = manager.prepare(96, [96])
    assert split.num_tokens == [48, 48]
    with torch.no_grad():
        y = compiled(x)
    torch.testing.assert_close(y, model(x), rtol=0, atol=0)
    assert calls == {"sized": 2 * len(backends), "dynamic": 0}

    # another split of the same input: sizes that are not listed use the dynamic callable
    calls.update(sized=0, dynamic=0)
    manager.override_split_config(SplitConfig(num_nano_batches=2, batch_sizes=[40, 56], batch_indices=[0, 40, 96],
                                              num_tokens=[40, 56], num_tokens_padded=[40, 56],
                                              split_indices=[0, 40, 96], is_dryrun=False, use_cudagraph=False))
    with torch.no_grad():
        y = compiled(x)
    torch.testing.assert_close(y, model(x), rtol=0, atol=0)
    assert calls == {"sized": 0, "dynamic": 2 * len(backends)}


@pytest.mark.parametrize("knobs,splits,want", [
    ({"streams": "by_nano_batch"}, 2, 2),                        # the same sub-graph of both nano-batches at once
    ({"streams": "by_nano_batch"}, 4, 2),                        # four nano-batches take the two streams in turn
    ({"streams": "by_kind"}, 2, 1),                              # launches of one kind queue on one stream
    ({"streams": "by_nano_batch", "serialize": True}, 2, 1),     # one stream
    ({"streams": "by_nano_batch", "side_by_side": 1}, 2, 1),     # override downwards: planned as lone launches
    ({"streams": "by_kind", "serialize": True, "side_by_side": 2}, 2, 2),   # the one-stream baseline of a pair plan
])
def test_kernel_plans_follow_the_schedule_not_a_promise(host_device, monkeypatch, knobs, splits, want):
    """``side_by_side`` - how many launches of one sub-graph share the GPU, what the GEMM plans are made for - is
    derived from the stream policy and the split of each forward; the knob only overrides it downwards."""
    import contextlib

    from dynaflow_amd import ops

    seen = []
    real = ops.launch_options

    @contextlib.contextmanager
    def recording(side_by_side=1):
        seen.append(side_by_side)
        with real(side_by_side=side_by_side):
            yield

    monkeypatch.setattr(ops, "launch_options", recording)
    cfg = make_config(splits, num_nano_batches=splits, **knobs)
    model, manager, compiled, x = compile_mlp(cfg, tokens=96)
    split = manager.prepare(96, [96])
    assert split.num_nano_batches == splits
    assert manager.launches_side_by_side(split) == want
    seen.clear()
    with torch.no_grad():
        y = compiled(x)
    assert seen == [want]
    torch.testing.assert_close(y, model(x), rtol=0, atol=0)
    # a forward that is not split has nothing beside it, whatever the stream policy
    single = manager.prepare(4, [4])
    assert single.num_nano_batches == 1
    if "side_by_side" not in knobs:
        assert manager.launches_side_by_side(single) == 1


@pytest.mark.parametrize("knobs", [{"streams": "by_kind", "side_by_side": 2},
                                   {"streams": "by_nano_batch", "side_by_side": 3},
                                   {"streams": "by_nano_batch", "side_by_side": 0}])
def test_a_side_by_side_override_that_contradicts_the_schedule_is_refused(host_device, knobs):
    """Streams by sub-graph kind with kernels planned for a pair would queue two half-chip launches on one stream;
    such a configuration raises instead of running slowly."""
    cfg = make_config(2, num_nano_batches=2, **knobs)
    model, manager, compiled, x = compile_mlp(cfg, tokens=96)
    manager.prepare(96, [96])
    with torch.no_grad(), pytest.raises(ValueError, match="side_by_side"):
        compiled(x)
