"""The whole path on an MI355X: torch.compile backend -> manager -> engine ->
scheduler -> HIP operators on two streams, against the CPU oracle."""
import pytest
import torch

from oracle import mlp

pytestmark = pytest.mark.gpu

TOL = {"fp32": 1e-5, "bf16": 2e-2, "fp8": 5e-2}


def rel_err(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    return ((got - want).abs().max() / want.abs().max().clamp_min(1e-30)).item()


def build(tokens, hidden, inter, dtype, splits=2, prenorm=False, **knobs):
    from dynaflow_amd.backend import make_backend
    from dynaflow_amd.config import CUDAGraphConfig, DynaFlowConfig, InductorConfig
    from dynaflow_amd.manager import DynaFlowManager
    from dynaflow_amd.mlp import SwiGLUMLP

    extra = {"min_nano_split_tokens": 1, "num_nano_batches": splits, "dump_graph": False}
    extra.update(knobs)
    cfg = DynaFlowConfig("dynaflow_amd.schedulers:MLPOverlapScheduler", splits, InductorConfig(enabled=True),
                         CUDAGraphConfig(enabled=False, capture_sizes=[tokens]), extra)
    x, wg, wu, wd = mlp.make_inputs(tokens, hidden, inter, dtype, prenorm=prenorm)
    model = SwiGLUMLP(hidden, inter, dtype=dtype, device="cuda")
    with torch.no_grad():
        model.gate_proj.weight.copy_(wg)
        model.up_proj.weight.copy_(wu)
        model.down_proj.weight.copy_(wd)
    manager = DynaFlowManager()
    torch._dynamo.reset()
    xg = x.cuda()
    torch._dynamo.mark_dynamic(xg, 0)
    compiled = torch.compile(model, backend=make_backend(manager, cfg), fullgraph=True)
    manager.prepare(tokens, [tokens])
    with torch.no_grad():
        compiled(xg)  # traces; runs the trivial split through the fast path
    return manager, compiled, xg, (x, wg, wu, wd)


def run(manager, compiled, xg, tokens, use_cudagraph=False):
    split = manager.prepare(tokens, [tokens], use_cudagraph=use_cudagraph)
    with torch.no_grad():
        y = compiled(xg)
    torch.cuda.synchronize()
    return y, split


def test_subgraphs_run_on_hip_operators():
    from dynaflow_amd import ops

    manager, compiled, xg, _ = build(256, 1024, 2816, torch.float32)
    for name in ("submod_0", "submod_1"):
        backend = manager.graph_module.__dict__[name]
        targets = [n.target for n in backend.callable_dynamic.graph.nodes if n.op == "call_function"]
        import operator

        assert all(t in (ops.linear, ops.linear_to_output, ops.silu_mul, operator.getitem) for t in targets), targets


def test_config1_fp32_matches_cpu_reference_path():
    """x[256,1024] fp32, I=2816, 2 x 128 tokens: the reference's CPU-runnable case."""
    manager, compiled, xg, (x, wg, wu, wd) = build(256, 1024, 2816, torch.float32)
    y, split = run(manager, compiled, xg, 256)
    assert split.split_indices == [0, 128, 256]
    want = mlp.mlp_schedule(x, wg, wu, wd, split.split_indices)
    assert rel_err(y, want) < TOL["fp32"]
    assert manager.engine.issue_trace == [("submod_0", 0), ("submod_1", 0), ("submod_0", 1), ("submod_1", 1)]


@pytest.mark.parametrize("tokens,splits", [(512, 2), (500, 2), (384, 3), (96, 4)])
def test_bf16_schedule_small(tokens, splits):
    manager, compiled, xg, (x, wg, wu, wd) = build(tokens, 512, 1408, torch.bfloat16, splits=splits)
    y, split = run(manager, compiled, xg, tokens)
    assert split.num_nano_batches == splits
    want = mlp.mlp_schedule(x, wg, wu, wd, split.split_indices)     # eager bf16 PyTorch on the CPU
    assert rel_err(y.float(), want.float()) < TOL["bf16"]
    exact = mlp.mlp_fp32_from(x, wg, wu, wd)                       # fp32 on the same bf16 operands
    assert rel_err(y.float(), exact) < TOL["bf16"]


def test_config2_full_size_properties():
    """x[4096,4096] bf16 pre-normed, I=14336, 2 x 2048.  The CPU oracle takes too long at this
    size for the whole output, so: (1) sampled rows against the oracle, (2) split == unsplit
    through the HIP path, (3) serialised == overlapped bit for bit."""
    manager, compiled, xg, (x, wg, wu, wd) = build(4096, 4096, 14336, torch.bfloat16, prenorm=True)
    y, split = run(manager, compiled, xg, 4096)
    assert split.split_indices == [0, 2048, 4096]
    rows = torch.tensor([0, 1, 2047, 2048, 3000, 4095])
    want = mlp.mlp_fp32_from(x[rows], wg, wu, wd)
    assert rel_err(y[rows].float(), want) < TOL["bf16"]
    # unsplit through the same kernels (single nano-batch fast path)
    from dynaflow_amd.manager import trivial_split

    manager.override_split_config(trivial_split(4096, [4096], False, False))
    with torch.no_grad():
        whole = compiled(xg)
    torch.cuda.synchronize()
    assert rel_err(y.float(), whole.float()) < 2 ** -6
    # a second overlapped run is bit-identical (no race between the streams)
    y2, _ = run(manager, compiled, xg, 4096)
    assert torch.equal(y, y2)


def test_config2_headline_mode_full_size():
    """The mode that the bench reports, at full size: SiLU*mul as the epilogue of the gate/up GEMM, one stream per
    nano-batch - so the manager plans the kernels for the two launches of a kind that run side by side - and the
    whole schedule as one hipGraph.  (1) sampled rows against the oracle, (2) the same bits as the unfused schedule
    with the same stream policy (separate gate, up and SiLU*mul launches; the same plan for the down projection),
    (3) every replay of the graph equals the eager issue, with eager work between the replays."""
    manager, compiled, xg, (x, wg, wu, wd) = build(4096, 4096, 14336, torch.bfloat16, prenorm=True,
                                                   fuse_silu_epilogue=True, whole_graph=True, streams="by_nano_batch")
    eager, split = run(manager, compiled, xg, 4096)
    eager = eager.clone()
    assert split.split_indices == [0, 2048, 4096]
    rows = torch.tensor([0, 255, 256, 2047, 2048, 3333, 4095])
    want = mlp.mlp_fp32_from(x[rows], wg, wu, wd)
    assert rel_err(eager[rows].float(), want) < TOL["bf16"]
    assert manager.launches_side_by_side(split) == 2
    plain_manager, plain, xp, _ = build(4096, 4096, 14336, torch.bfloat16, prenorm=True, streams="by_nano_batch")
    unfused, _ = run(plain_manager, plain, xp, 4096)
    assert torch.equal(eager, unfused)
    for _ in range(3):
        replay, _ = run(manager, compiled, xg, 4096, use_cudagraph=True)
        assert torch.equal(replay, eager)
        again, _ = run(plain_manager, plain, xp, 4096)          # eager work of another manager in between
        assert torch.equal(again, unfused)


def test_config2_kernels_planned_for_two_nano_batches_side_by_side():
    """``side_by_side=2`` with one stream per nano-batch: the same sub-graph of the two nano-batches runs at the same
    time, and the kernels are planned for the pair.  Each down projection of a 2048-token nano-batch runs one
    workgroup per 256 x 256 tile (128 of them) instead of two that split K; the gate/up/SiLU launches take the
    256 x (128 + 128) tile, whose 2 x 896 tiles are exactly 7 rounds of the 256 compute units.  Sampled rows against
    the oracle; the two-stream issue, the one-stream issue and every replay of the whole-schedule graph have the
    same bits; within a rounding of the form planned for lone launches (K of the down projection split)."""
    knobs = dict(fuse_silu_epilogue=True, whole_graph=True, streams="by_nano_batch", side_by_side=2)
    manager, compiled, xg, (x, wg, wu, wd) = build(4096, 4096, 14336, torch.bfloat16, prenorm=True, **knobs)
    eager, split = run(manager, compiled, xg, 4096)
    eager = eager.clone()
    assert split.split_indices == [0, 2048, 4096]
    rows = torch.tensor([0, 255, 256, 2047, 2048, 3333, 4095])
    assert rel_err(eager[rows].float(), mlp.mlp_fp32_from(x[rows], wg, wu, wd)) < TOL["bf16"]
    for _ in range(3):
        replay, _ = run(manager, compiled, xg, 4096, use_cudagraph=True)
        assert torch.equal(replay, eager)
    serial_manager, serial, xs, _ = build(4096, 4096, 14336, torch.bfloat16, prenorm=True, serialize=True,
                                          fuse_silu_epilogue=True, side_by_side=2)
    one_stream, _ = run(serial_manager, serial, xs, 4096)
    assert torch.equal(one_stream, eager)
    lone_manager, lone, xk, _ = build(4096, 4096, 14336, torch.bfloat16, prenorm=True, fuse_silu_epilogue=True)
    lone_form, _ = run(lone_manager, lone, xk, 4096)
    assert not torch.equal(lone_form, eager)            # other order of the fp32 additions in the down projection ...
    assert rel_err(lone_form.float(), eager.float()) < 2 ** -7   # ... and nothing else


def test_nano_batch_outputs_land_in_one_buffer(monkeypatch):
    """The down projection of every nano-batch writes its rows of one output buffer: the forward ends without a
    concatenation, and the result has the bits of the schedule that allocates per nano-batch and concatenates."""
    manager, compiled, xg, _ = build(512, 512, 1408, torch.bfloat16, splits=2)
    plain_manager, plain, xp, _ = build(512, 512, 1408, torch.bfloat16, splits=2, shared_output=False)
    want, _ = run(plain_manager, plain, xp, 512)
    real_cat = torch.cat

    def no_cat(*args, **kwargs):
        raise AssertionError("the forward concatenated its nano-batch outputs")

    monkeypatch.setattr(torch, "cat", no_cat)
    got, split = run(manager, compiled, xg, 512)
    monkeypatch.setattr(torch, "cat", real_cat)
    assert split.num_nano_batches == 2
    assert got.shape == want.shape and torch.equal(got, want)
    # ragged split (3 nano-batches of 171, 171, 170 tokens)
    manager3, compiled3, x3, (x, wg, wu, wd) = build(512, 512, 1408, torch.bfloat16, splits=3)
    monkeypatch.setattr(torch, "cat", no_cat)
    got3, split3 = run(manager3, compiled3, x3, 512)
    monkeypatch.setattr(torch, "cat", real_cat)
    assert split3.num_nano_batches == 3
    assert rel_err(got3.float(), mlp.mlp_schedule(x, wg, wu, wd, split3.split_indices).float()) < TOL["bf16"]


def test_serialized_schedule_is_bit_identical_to_overlapped():
    m1, c1, xg1, _ = build(1024, 1024, 2816, torch.bfloat16)
    y1, _ = run(m1, c1, xg1, 1024)
    m2, c2, xg2, _ = build(1024, 1024, 2816, torch.bfloat16, serialize=True)
    y2, _ = run(m2, c2, xg2, 1024)
    assert torch.equal(y1, y2)


def test_whole_schedule_graph_replay():
    """One hipGraph for the whole two-stream schedule: every replay must equal the eager result,
    with eager work and synchronisations between the replays."""
    manager, compiled, xg, (x, wg, wu, wd) = build(1024, 1024, 2816, torch.bfloat16, whole_graph=True)
    eager, _ = run(manager, compiled, xg, 1024, use_cudagraph=False)
    eager = eager.clone()
    for i in range(4):
        y, _ = run(manager, compiled, xg, 1024, use_cudagraph=True)
        assert torch.equal(y, eager), f"replay {i}"
        junk = torch.randn(512, 512, device="cuda") @ torch.randn(512, 512, device="cuda")
        torch.cuda.synchronize()
    assert len(manager._schedule_graphs) == 1
    # new input values in the captured tensor are picked up by the replay
    new_x = torch.randn_like(xg)
    xg.copy_(new_x)
    y, _ = run(manager, compiled, xg, 1024, use_cudagraph=True)
    want, _ = run(manager, compiled, xg, 1024, use_cudagraph=False)
    assert torch.equal(y, want)
    # an input living elsewhere is copied into the captured tensor first
    other = torch.randn_like(xg)
    y, _ = run(manager, compiled, other, 1024, use_cudagraph=True)
    want, _ = run(manager, compiled, other, 1024, use_cudagraph=False)
    assert torch.equal(y, want)


def fp8_layer(tokens, hidden, inter, fuse_gate_up=False):
    from dynaflow_amd.fp8_mlp import Fp8SwiGLU

    x, wg, wu, wd = mlp.make_inputs(tokens, hidden, inter, torch.bfloat16)
    quantised = [mlp.quant_e4m3_per_channel(w) for w in (wg, wu, wd)]
    buffers = []
    for codes, scale in quantised:
        buffers += [codes.cuda().view(torch.float8_e4m3fn), scale.cuda()]
    return Fp8SwiGLU(*buffers, fuse_gate_up=fuse_gate_up), x, quantised, (wg, wu, wd)


def test_fp8_layer_against_dequantised_reference():
    """fp8 MLP (per-tensor activation scale, per-channel weight scale), 4 nano-batches issued directly."""
    from dynaflow_amd.fp8_mlp import Fp8SwiGLU

    layer, x, quantised, (wg, wu, wd) = fp8_layer(512, 1024, 2048)
    split = [0, 128, 256, 384, 512]
    y = layer.forward_schedule(x.cuda(), split)
    torch.cuda.synchronize()
    (wg_q, wg_s), (wu_q, wu_s), (wd_q, wd_s) = quantised
    want = mlp.mlp_fp8_dequant_reference(x, wg_q, wg_s, wu_q, wu_s, wd_q, wd_s, split)
    assert rel_err(y.float(), want.float()) < TOL["fp8"]
    # the device-side weight quantiser agrees with the oracle's codec (up to last-bit division effects)
    auto = Fp8SwiGLU.from_weights(wg.cuda(), wu.cuda(), wd.cuda())
    agree = ((auto.w_gate_q.cpu().view(torch.uint8) & 0x7F) == (wg_q & 0x7F)).float().mean()
    assert agree > 0.999 and torch.allclose(auto.w_gate_s.cpu(), wg_s, rtol=1e-6)


def test_fp8_layer_through_the_manager_with_four_nano_batches():
    from dynaflow_amd.backend import make_backend
    from dynaflow_amd.config import CUDAGraphConfig, DynaFlowConfig, InductorConfig
    from dynaflow_amd.manager import DynaFlowManager

    tokens = 512
    layer, x, quantised, _ = fp8_layer(tokens, 1024, 2048)
    cfg = DynaFlowConfig("dynaflow_amd.schedulers:MLPOverlapScheduler", 4, InductorConfig(enabled=True),
                         CUDAGraphConfig(enabled=False, capture_sizes=[tokens]),
                         {"min_nano_split_tokens": 1, "num_nano_batches": 4, "dump_graph": False})
    manager = DynaFlowManager()
    torch._dynamo.reset()
    xg = x.cuda()
    torch._dynamo.mark_dynamic(xg, 0)
    compiled = torch.compile(layer, backend=make_backend(manager, cfg), fullgraph=True)
    with torch.no_grad():
        manager.prepare(tokens, [tokens])
        compiled(xg)
        split = manager.prepare(tokens, [tokens])
        y = compiled(xg)
    torch.cuda.synchronize()
    assert split.split_indices == [0, 128, 256, 384, 512]
    assert manager.engine.issue_trace == [("submod_0", 0), ("submod_1", 0), ("submod_0", 1), ("submod_0", 2),
                                          ("submod_0", 3), ("submod_1", 1), ("submod_1", 2), ("submod_1", 3)]
    (wg_q, wg_s), (wu_q, wu_s), (wd_q, wd_s) = quantised
    want = mlp.mlp_fp8_dequant_reference(x, wg_q, wg_s, wu_q, wu_s, wd_q, wd_s, split.split_indices)
    assert rel_err(y.float(), want.float()) < TOL["fp8"]
    assert torch.equal(y, layer.forward_schedule(xg, split.split_indices))


def test_fp8_layer_with_fused_gate_up_epilogue_through_the_manager():
    """The fp8 block with gate/up/SiLU*mul as one operator, cut in front of the down projection: the fused
    sub-graph of one nano-batch beside the down projection of the previous one; same bits as the unfused block."""
    from dynaflow_amd import ops
    from dynaflow_amd.backend import make_backend
    from dynaflow_amd.config import CUDAGraphConfig, DynaFlowConfig, InductorConfig
    from dynaflow_amd.manager import DynaFlowManager

    tokens = 512
    layer, x, quantised, _ = fp8_layer(tokens, 1024, 2048, fuse_gate_up=True)
    plain, *_ = fp8_layer(tokens, 1024, 2048)
    cfg = DynaFlowConfig("dynaflow_amd.schedulers:MLPOverlapScheduler", 4, InductorConfig(enabled=True),
                         CUDAGraphConfig(enabled=False, capture_sizes=[tokens]),
                         {"min_nano_split_tokens": 1, "num_nano_batches": 4, "dump_graph": False,
                          "fuse_silu_epilogue": True})
    manager = DynaFlowManager()
    torch._dynamo.reset()
    xg = x.cuda()
    torch._dynamo.mark_dynamic(xg, 0)
    compiled = torch.compile(layer, backend=make_backend(manager, cfg), fullgraph=True)
    with torch.no_grad():
        manager.prepare(tokens, [tokens])
        compiled(xg)
        split = manager.prepare(tokens, [tokens])
        y = compiled(xg)
    torch.cuda.synchronize()
    names = [n.target for n in manager.graph_module.graph.nodes if n.op == "call_module"]
    assert len(names) == 2
    head = [n.target for n in manager.graph_module.__dict__[names[0]].callable_dynamic.graph.nodes
            if n.op == "call_function"]
    assert any(getattr(t, "overloadpacket", t) is ops.gate_up_silu_quant_fp8 for t in head)
    assert getattr(manager.graph_module, names[0]).tag == {"head"}
    assert split.split_indices == [0, 128, 256, 384, 512]
    (wg_q, wg_s), (wu_q, wu_s), (wd_q, wd_s) = quantised
    want = mlp.mlp_fp8_dequant_reference(x, wg_q, wg_s, wu_q, wu_s, wd_q, wd_s, split.split_indices)
    assert rel_err(y.float(), want.float()) < TOL["fp8"]
    assert torch.equal(y, plain.forward_schedule(xg, split.split_indices))


def test_piecewise_graphs_capture_in_dryrun_and_replay():
    """Per-sub-graph hipGraphs as in the reference: captured for every (size, nano-batch index) during a
    dry-run over fake nano-batches, replayed by the scheduled forward against per-nano-batch static buffers."""
    from dynaflow_amd.backend import make_backend
    from dynaflow_amd.config import CUDAGraphConfig, DynaFlowConfig, InductorConfig
    from dynaflow_amd.interface import SplitConfig
    from dynaflow_amd.manager import DynaFlowManager
    from dynaflow_amd.mlp import SwiGLUMLP

    tokens, hidden, inter = 512, 512, 1408
    cfg = DynaFlowConfig("dynaflow_amd.schedulers:MLPOverlapScheduler", 2, InductorConfig(enabled=True),
                         CUDAGraphConfig(enabled=True, capture_sizes=[256, 512]),
                         {"min_nano_split_tokens": 1, "num_nano_batches": 2, "dump_graph": False, "max_tokens": 1024})
    x, wg, wu, wd = mlp.make_inputs(tokens, hidden, inter, torch.bfloat16)
    model = SwiGLUMLP(hidden, inter, dtype=torch.bfloat16, device="cuda")
    with torch.no_grad():
        model.gate_proj.weight.copy_(wg)
        model.up_proj.weight.copy_(wu)
        model.down_proj.weight.copy_(wd)
    manager = DynaFlowManager()
    torch._dynamo.reset()
    xg = x.cuda()
    torch._dynamo.mark_dynamic(xg, 0)
    compiled = torch.compile(model, backend=make_backend(manager, cfg), fullgraph=True)
    with torch.no_grad():
        manager.prepare(tokens, [tokens])
        compiled(xg)                                   # trace
        eager = compiled_eager = None
        manager.prepare(tokens, [tokens])
        eager = compiled(xg).clone()                   # scheduled, no graphs
        # dry-run at the nano-batch size: captures (256, 0) and (256, 1) for both sub-graphs
        half = xg[:256].contiguous()
        manager.prepare(256, [256], is_dryrun=True, use_cudagraph=True)
        dry = compiled(half)
        torch.cuda.synchronize()
        assert torch.equal(dry, eager[:256])
        # scheduled forward replaying the captured graphs
        split = SplitConfig(2, [256, 256], [0, 256, 512], [256, 256], [256, 256], [0, 256, 512], False, True)
        for _ in range(3):
            manager.override_split_config(split)
            y = compiled(xg)
            torch.cuda.synchronize()
            assert torch.equal(y, eager)
            torch.randn(256, 256, device="cuda").sum().item()
        # new values flow through the static buffers
        xg2 = torch.randn_like(xg)
        manager.prepare(tokens, [tokens])
        want = compiled(xg2).clone()
        manager.override_split_config(split)
        assert torch.equal(compiled(xg2), want)
        # a size that was never captured cannot be replayed
        bad = SplitConfig(2, [128, 384], [0, 128, 512], [128, 384], [128, 384], [0, 128, 512], False, True)
        manager.override_split_config(bad)
        with pytest.raises(AssertionError):
            compiled(xg)
    for name in ("submod_0", "submod_1"):
        wrapper = manager.graph_module.__dict__[name].callable_dynamic
        assert sorted(k[:2] for k in wrapper._entries) == [(256, 0), (256, 1)]


def test_listed_sizes_dispatch_to_their_own_lowered_callable():
    """``InductorConfig(compile_sizes={256})``: the dry-run at 256 tokens lowers a callable for that size in
    every sub-graph, the scheduled forward with 2 x 256 tokens dispatches to it (never to the dynamic one), and
    the result has the bits of the dynamic callable (dynaflow/executor/compiler.py:69-85)."""
    from dynaflow_amd import ops
    from dynaflow_amd.backend import make_backend
    from dynaflow_amd.config import CUDAGraphConfig, DynaFlowConfig, InductorConfig
    from dynaflow_amd.manager import DynaFlowManager
    from dynaflow_amd.mlp import SwiGLUMLP

    tokens, hidden, inter = 512, 512, 1408
    x, wg, wu, wd = mlp.make_inputs(tokens, hidden, inter, torch.bfloat16)
    model = SwiGLUMLP(hidden, inter, dtype=torch.bfloat16, device="cuda")
    with torch.no_grad():
        model.gate_proj.weight.copy_(wg)
        model.up_proj.weight.copy_(wu)
        model.down_proj.weight.copy_(wd)
    xg = x.cuda()
    outputs = {}
    for sizes in (None, {256}):
        cfg = DynaFlowConfig("dynaflow_amd.schedulers:MLPOverlapScheduler", 2,
                             InductorConfig(enabled=True, compile_sizes=sizes),
                             CUDAGraphConfig(enabled=False, capture_sizes=[tokens]),
                             {"min_nano_split_tokens": 1, "num_nano_batches": 2, "dump_graph": False})
        manager = DynaFlowManager()
        torch._dynamo.reset()
        torch._dynamo.mark_dynamic(xg, 0)
        compiled = torch.compile(model, backend=make_backend(manager, cfg), fullgraph=True)
        with torch.no_grad():
            manager.prepare(tokens, [tokens])
            compiled(xg)                                    # trace (512 is not a listed size)
            backends = [manager.graph_module.__dict__[n.target] for n in manager.graph_module.graph.nodes
                        if n.op == "call_module"]
            calls = {"sized": 0, "dynamic": 0}
            if sizes:
                manager.prepare(256, [256], is_dryrun=True)
                dry = compiled(xg[:256].contiguous())
                torch.cuda.synchronize()
                assert all(sorted(b.callables_per_size) == [256] for b in backends)
                for b in backends:
                    sized_targets = [n.target for n in b.callables_per_size[256].graph.nodes
                                     if n.op == "call_function"]
                    # every sub-graph of this layer holds at least one product or the SiLU*mul, lowered
                    assert any(str(t).startswith("dynaflow_hip.") for t in sized_targets), sized_targets
                    b.callables_per_size[256] = (lambda fn: lambda *a, **k: (calls.__setitem__(
                        "sized", calls["sized"] + 1), fn(*a, **k))[1])(b.callables_per_size[256])
                    b.callable_dynamic = (lambda fn: lambda *a, **k: (calls.__setitem__(
                        "dynamic", calls["dynamic"] + 1), fn(*a, **k))[1])(b.callable_dynamic)
            split = manager.prepare(tokens, [tokens])
            assert split.num_tokens == [256, 256]
            outputs[bool(sizes)] = compiled(xg).clone()
            torch.cuda.synchronize()
            if sizes:
                assert calls == {"sized": 2 * len(backends), "dynamic": 0}
                assert torch.equal(dry, outputs[True][:256])
    assert torch.equal(outputs[False], outputs[True])
    want = mlp.mlp_fp32_from(x, wg, wu, wd)
    assert rel_err(outputs[True].float(), want) < TOL["bf16"]


def test_fp8_config_full_size_properties():
    """fp8 70B-shaped layer at full size (x[8192,8192], I=28672, 4 x 2048), in both lowerings: separate gate / up /
    SiLU*mul launches, and the mode the bench reports - gate, up, SiLU*mul and absmax as ONE launch
    (``fuse_gate_up`` + knob ``fuse_silu_epilogue``).  (1) the scheduled two-stream run equals the nano-batches
    issued one after the other bit for bit, (2) two runs agree, (3) the two lowerings agree bit for bit, (4) sampled
    rows of two nano-batches agree with an evaluation that takes NOTHING from the kernels under test: activations
    quantised with torch's own e4m3 conversion, gate and up of the WHOLE nano-batch as fp32 products of the
    dequantised operands (torch on the GPU), rounded to bf16, the oracle's exact SiLU*mul, its absmax over the whole
    nano-batch (the re-quantisation scale needs every row), the oracle's e4m3 encoder for the sampled rows, fp32
    down projection."""
    from dynaflow_amd.backend import make_backend
    from dynaflow_amd.config import CUDAGraphConfig, DynaFlowConfig, InductorConfig
    from dynaflow_amd.fp8_mlp import Fp8SwiGLU
    from dynaflow_amd.manager import DynaFlowManager

    tokens, hidden, inter = 8192, 8192, 28672
    gen = torch.Generator(device="cuda").manual_seed(0)
    x = torch.randn(tokens, hidden, generator=gen, device="cuda").bfloat16()
    ws = [(torch.randn(s, generator=gen, device="cuda") * 0.02).bfloat16() for s in ((inter, hidden), (inter, hidden), (hidden, inter))]
    layer = Fp8SwiGLU.from_weights(*ws)
    del ws
    outputs = {}
    for fused in (False, True):
        print(f"config 5 at full size: fused gate/up/SiLU launch = {fused}", flush=True)
        layer.fuse_gate_up = fused
        knobs = {"min_nano_split_tokens": 64, "num_nano_batches": 4, "dump_graph": False}
        if fused:
            knobs["fuse_silu_epilogue"] = True
        cfg = DynaFlowConfig("dynaflow_amd.schedulers:MLPOverlapScheduler", 4, InductorConfig(enabled=True),
                             CUDAGraphConfig(enabled=False, capture_sizes=[tokens]), knobs)
        manager = DynaFlowManager()
        torch._dynamo.reset()
        torch._dynamo.mark_dynamic(x, 0)
        compiled = torch.compile(layer, backend=make_backend(manager, cfg), fullgraph=True)
        with torch.no_grad():
            manager.prepare(tokens, [tokens])
            compiled(x)
            split = manager.prepare(tokens, [tokens])
            y = compiled(x)
            manager.prepare(tokens, [tokens])
            y2 = compiled(x)
            direct = layer.forward_schedule(x, split.split_indices)
        torch.cuda.synchronize()
        assert split.split_indices == [0, 2048, 4096, 6144, 8192]
        assert torch.equal(y, y2) and torch.equal(y, direct)
        if fused:
            from dynaflow_amd import ops
            names = [n.target for n in manager.graph_module.graph.nodes if n.op == "call_module"]
            head = manager.graph_module.__dict__[names[0]].callable_dynamic
            assert ops.gate_up_silu_quant_fp8 in [n.target for n in head.graph.nodes if n.op == "call_function"]
        outputs[fused] = y.clone()
        del manager, compiled, direct, y, y2
    assert torch.equal(outputs[False], outputs[True])

    fp8_max = 448.0
    wd = layer.w_down_q.float() * layer.w_down_s[:, None]
    wg = layer.w_gate_q.float() * layer.w_gate_s[:, None]
    wu = layer.w_up_q.float() * layer.w_up_s[:, None]
    for nano_batch, picked in ((0, [0, 1, 777, 2047]), (3, [0, 1024, 2046, 2047])):
        print(f"config 5 at full size: oracle-side evaluation of nano-batch {nano_batch}", flush=True)
        xb = x[nano_batch * 2048:(nano_batch + 1) * 2048].float()
        x_scale = xb.abs().max().clamp_min(1e-12) / fp8_max
        xd = (xb / x_scale).clamp(-fp8_max, fp8_max).to(torch.float8_e4m3fn).float() * x_scale
        g = (xd @ wg.t()).bfloat16()
        u = (xd @ wu.t()).bfloat16()
        act = mlp.silu_mul_exact(g, u)                       # bf16, whole nano-batch
        a_scale = act.float().abs().max().clamp_min(1e-12) / fp8_max
        rows = torch.tensor(picked)
        scaled = (act[rows.cuda()].float() / a_scale).clamp(-fp8_max, fp8_max).cpu()
        codes = torch.from_numpy(mlp.e4m3_encode(scaled.numpy()))
        a_rows = mlp.dequant(codes, a_scale.reshape(1).cpu())
        want = a_rows.cuda() @ wd.t()
        got = outputs[True][nano_batch * 2048 + rows.cuda()]
        err = rel_err(got.float(), want)
        print(f"config 5 at full size: nano-batch {nano_batch}, sampled rows against the oracle-side evaluation: "
              f"{err:.4f}", flush=True)
        assert err < TOL["fp8"]
        del xb, xd, g, u, act


def test_fused_silu_epilogue_schedule():
    """fuse_silu_epilogue: {gate, up, silu, mul} becomes one GEMM with the SiLU*mul as epilogue, the cut
    moves in front of the down projection; same bits as the unfused schedule."""
    from dynaflow_amd import ops

    manager, compiled, xg, (x, wg, wu, wd) = build(1024, 1024, 2816, torch.bfloat16, fuse_silu_epilogue=True)
    head = manager.graph_module.__dict__["submod_0"].callable_dynamic
    tail = manager.graph_module.__dict__["submod_1"].callable_dynamic
    assert [n.target for n in head.graph.nodes if n.op == "call_function"] == [ops.gate_up_silu]
    assert [n.target for n in tail.graph.nodes if n.op == "call_function"] == [ops.linear_to_output]
    y, split = run(manager, compiled, xg, 1024)
    assert manager.engine.issue_trace == [("submod_0", 0), ("submod_1", 0), ("submod_0", 1), ("submod_1", 1)]
    want = mlp.mlp_fp32_from(x, wg, wu, wd)
    assert rel_err(y.float(), want) < TOL["bf16"]
    unfused = build(1024, 1024, 2816, torch.bfloat16)
    y0, _ = run(unfused[0], unfused[1], unfused[2], 1024)
    assert torch.equal(y, y0)   # the epilogue rounds like the separate kernels


def build_decoder(batch, seq_len, hidden, heads, kv_heads, head_dim, inter, vocab, **knobs):
    from dynaflow_amd.backend import make_backend
    from dynaflow_amd.config import CUDAGraphConfig, DynaFlowConfig, InductorConfig
    from dynaflow_amd.decoder import DecoderLayer
    from dynaflow_amd.manager import DynaFlowManager

    layer = DecoderLayer(vocab=vocab, hidden=hidden, heads=heads, kv_heads=kv_heads, head_dim=head_dim, inter=inter,
                         seq_len=seq_len, dtype=torch.bfloat16)
    layer.init_weights(seed=7)
    ids = torch.randint(0, vocab, (batch * seq_len,), generator=torch.Generator().manual_seed(4))
    gpu_layer = DecoderLayer(vocab=vocab, hidden=hidden, heads=heads, kv_heads=kv_heads, head_dim=head_dim,
                             inter=inter, seq_len=seq_len, dtype=torch.bfloat16, device="cuda")
    gpu_layer.load_state_dict(layer.state_dict())
    extra = {"min_nano_split_tokens": 1, "dump_graph": False}
    extra.update(knobs)
    cfg = DynaFlowConfig("dynaflow_amd.schedulers:DecoderOverlapScheduler", 2, InductorConfig(enabled=True),
                         CUDAGraphConfig(enabled=False, capture_sizes=[batch * seq_len]), extra)
    manager = DynaFlowManager()
    torch._dynamo.reset()
    idg = ids.cuda()
    torch._dynamo.mark_dynamic(idg, 0)
    compiled = torch.compile(gpu_layer, backend=make_backend(manager, cfg), fullgraph=True)
    with torch.no_grad():
        manager.prepare(batch, [seq_len] * batch)
        compiled(idg)
    return manager, compiled, idg, layer, ids


def test_decoder_layer_attention_beside_mlp_small():
    """Decoder layer through the manager: attention sub-graph of nano-batch 1 beside the MLP sub-graph of
    nano-batch 0, against the independent float64 oracle (bf16 tolerance)."""
    from dynaflow_amd import ops
    from oracle import decoder as ref

    batch, S = 4, 128
    manager, compiled, idg, layer, ids = build_decoder(batch, S, 512, 8, 2, 64, 1408, 1000)
    names = [n.target for n in manager.graph_module.graph.nodes if n.op == "call_module"]
    mlp_graph = manager.graph_module.__dict__[names[1]].callable_dynamic
    targets = [n.target for n in mlp_graph.graph.nodes if n.op == "call_function"]
    assert ops.rms_norm in targets and ops.silu_mul in targets
    # gate and up as one GEMM against stacked weights; down projection + residual in one launch (as the value
    # the sub-graph returns it may write into offered rows)
    assert targets.count(ops.linear_multi) == 1 and targets.count(ops.linear) == 0
    assert targets.count(ops.linear_add) + targets.count(ops.linear_add_to_output) == 1
    attn_targets = [n.target for n in manager.graph_module.__dict__[names[0]].callable_dynamic.graph.nodes
                    if n.op == "call_function"]
    assert attn_targets.count(ops.linear_multi) == 1 and attn_targets.count(ops.linear) == 0   # q, k, v
    assert attn_targets.count(ops.linear_add) + attn_targets.count(ops.linear_add_to_output) == 1
    assert ops.rms_norm in attn_targets
    assert attn_targets.count(ops.rope_pair) == 1 and attn_targets.count(ops.rope) == 0     # q and k in one launch
    with torch.no_grad():
        split = manager.prepare(batch, [S] * batch)
        y = compiled(idg)
    torch.cuda.synchronize()
    assert split.batch_indices == [0, 2, 4] and split.split_indices == [0, 2 * S, 4 * S]
    assert manager.engine.issue_trace == [(names[0], 0), (names[1], 0), (names[0], 1), (names[1], 1)]
    want = ref.decoder_layer(ids, ref.params_of(layer), S, 8, 2, 64)
    assert rel_err(y.float(), want) < TOL["bf16"]
    # serialised issue gives the same bits
    m2, c2, idg2, _, _ = build_decoder(batch, S, 512, 8, 2, 64, 1408, 1000, serialize=True)
    with torch.no_grad():
        m2.prepare(batch, [S] * batch)
        y2 = c2(idg2)
    assert torch.equal(y, y2)


def sub_graph_targets(manager):
    names = [n.target for n in manager.graph_module.graph.nodes if n.op == "call_module"]
    return names, [[n.target for n in manager.graph_module.__dict__[name].callable_dynamic.graph.nodes
                    if n.op == "call_function"] for name in names]


@pytest.mark.parametrize("batch,S", [(4, 128), (2, 320)])
def test_decoder_layer_head_dim_128_runs_the_attention_kernel_inside_the_schedule(batch, S):
    """head_dim 128 (the Llama-3 shape): the attention sub-graph holds the hand-written prefill attention and
    the paired rotation, fed by column ranges of the stacked q/k/v product, and runs on one stream beside the
    MLP sub-graph of the other nano-batch.  S = 128 and 320 leave the last 256-row query block ragged."""
    from dynaflow_amd import ops
    from oracle import decoder as ref

    shape = dict(hidden=512, heads=4, kv_heads=2, head_dim=128, inter=1408, vocab=1000)
    manager, compiled, idg, layer, ids = build_decoder(batch, S, **shape)
    names, (attn_targets, mlp_targets) = sub_graph_targets(manager)
    assert attn_targets.count(ops.causal_attention) == 1
    assert attn_targets.count(ops.rope_pair) == 1 and attn_targets.count(ops.rope) == 0
    assert attn_targets.count(ops.linear_multi) == 1 and attn_targets.count(ops.linear) == 0
    assert attn_targets.count(ops.linear_add) + attn_targets.count(ops.linear_add_to_output) == 1
    assert not any(getattr(t, "__name__", "") == "causal_gqa_attention" for t in attn_targets)
    assert ops.silu_mul in mlp_targets and ops.rms_norm in mlp_targets
    with torch.no_grad():
        split = manager.prepare(batch, [S] * batch)
        y = compiled(idg)
    torch.cuda.synchronize()
    assert split.split_indices == [0, (batch // 2) * S, batch * S]
    assert manager.engine.issue_trace == [(names[0], 0), (names[1], 0), (names[0], 1), (names[1], 1)]
    want = ref.decoder_layer(ids, ref.params_of(layer), S, 4, 2, 128)
    assert rel_err(y.float(), want) < TOL["bf16"]
    # the same kernels issued on one stream give the same bits, and so does a second overlapped run
    m2, c2, idg2, _, _ = build_decoder(batch, S, serialize=True, **shape)
    with torch.no_grad():
        m2.prepare(batch, [S] * batch)
        y2 = c2(idg2)
        manager.prepare(batch, [S] * batch)
        y3 = compiled(idg)
    torch.cuda.synchronize()
    assert torch.equal(y, y2) and torch.equal(y, y3)


def test_config3_full_size_properties():
    """The Llama-3-8B decoder layer at its real shape: 8 sequences x 2048 tokens, hidden 4096, 32 query / 8 kv
    heads of 128, intermediate 14336, vocabulary 128256; two nano-batches of 4 sequences, attention of one beside
    the MLP of the other.  The float64 oracle takes too long for the whole output at this size, so: (1) sampled
    (sequence, position) rows against the oracle restricted to those rows, (2) the split schedule against the same
    layer run as one batch through the same kernels, (3) run-to-run bit identity, (4) serialized == overlapped."""
    from dynaflow_amd import ops
    from dynaflow_amd.manager import trivial_split
    from oracle import decoder as ref

    batch, S = 8, 2048
    shape = dict(hidden=4096, heads=32, kv_heads=8, head_dim=128, inter=14336, vocab=128256)
    manager, compiled, idg, layer, ids = build_decoder(batch, S, fuse_silu_epilogue=True, **shape)
    names, (attn_targets, mlp_targets) = sub_graph_targets(manager)
    assert attn_targets.count(ops.causal_attention) == 1 and attn_targets.count(ops.rope_pair) == 1
    with torch.no_grad():
        split = manager.prepare(batch, [S] * batch)
        y = compiled(idg)
    torch.cuda.synchronize()
    assert split.batch_indices == [0, 4, 8] and split.split_indices == [0, 4 * S, 8 * S]
    assert manager.engine.issue_trace == [(names[0], 0), (names[1], 0), (names[0], 1), (names[1], 1)]
    assert bool(torch.isfinite(y.float()).all())
    # (1) rows of both nano-batches: first and last position of a sequence, the edges of a 256-row query block
    rows = [0, 255, 2047, 3 * S + 256, 4 * S, 5 * S + 1000, 8 * S - 1]
    want = ref.decoder_layer_rows(ids, ref.params_of(layer), rows, S, 32, 8, 128)
    assert rel_err(y[rows].float(), want) < TOL["bf16"]
    # (2) one batch through the same kernels
    with torch.no_grad():
        manager.override_split_config(trivial_split(batch, [S] * batch, False, False))
        whole = compiled(idg)
    torch.cuda.synchronize()
    assert rel_err(y.float(), whole.float()) < 2 ** -6
    # (3) a second overlapped run has the same bits (no race between the streams)
    with torch.no_grad():
        manager.prepare(batch, [S] * batch)
        y2 = compiled(idg)
    torch.cuda.synchronize()
    assert torch.equal(y, y2)
    # (4) the same launches on one stream
    del whole, y2
    m2, c2, idg2, _, _ = build_decoder(batch, S, fuse_silu_epilogue=True, serialize=True, **shape)
    with torch.no_grad():
        m2.prepare(batch, [S] * batch)
        y3 = c2(idg2)
    torch.cuda.synchronize()
    assert torch.equal(y, y3)


def test_decoder_layer_whole_schedule_graph_with_padded_capture_size():
    """use_cudagraph=True pads the nano-batch sizes to the capture size; the whole-schedule graph
    ignores that padding (it captures the real sizes) and every replay equals the eager run."""
    batch, S = 3, 64      # 128 + 64 tokens, only capture size 192: both nano-batches are padded
    manager, compiled, idg, layer, ids = build_decoder(batch, S, 256, 4, 2, 64, 704, 500, whole_graph=True)
    with torch.no_grad():
        manager.prepare(batch, [S] * batch, use_cudagraph=False)
        eager = compiled(idg).clone()
        for i in range(3):
            split = manager.prepare(batch, [S] * batch, use_cudagraph=True)
            y = compiled(idg)
            torch.cuda.synchronize()
            assert list(split.num_tokens_padded) != list(split.num_tokens)
            assert y.shape == eager.shape and torch.equal(y, eager), f"replay {i}"
            torch.randn(256, 256, device="cuda").sum().item()
    assert len(manager._schedule_graphs) == 1
