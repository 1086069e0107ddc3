"""Whole-schedule graphs of the schedules whose capture used to end in a segmentation fault: one stream for
everything, one stream per nano-batch, and the multi-layer schedule whose two streams wait for each other.
Every replay (with eager work between replays) must have the bits of the eager schedule."""
import pytest
import torch

from test_gpu_decode import build_decode
from test_gpu_schedule import build, build_decoder, fp8_layer, run

pytestmark = pytest.mark.gpu


def replays_equal_eager(manager, call, prepare, eager, origin):
    for i in range(3):
        print(f"whole-schedule graph: forward {i}", flush=True)
        prepare(True)
        y = call()
        torch.cuda.synchronize()
        assert torch.equal(y, eager), f"replay {i}"
        torch.randn(256, 256, device="cuda").sum().item()
    assert len(manager._schedule_graphs) == 1
    assert list(manager.capture_origins.values()) == [origin]


def test_serialized_mlp_schedule_as_one_graph():
    print("case: serialized MLP schedule, whole graph", flush=True)
    manager, compiled, xg, _ = build(512, 512, 1408, torch.bfloat16, serialize=True, whole_graph=True)
    eager, _ = run(manager, compiled, xg, 512)
    eager = eager.clone()
    replays_equal_eager(manager, lambda: torch.no_grad()(compiled)(xg),
                        lambda g: manager.prepare(512, [512], use_cudagraph=g), eager, "caller")


def test_decoder_layer_one_stream_per_nano_batch_as_one_graph():
    print("case: decoder layer, streams=by_nano_batch, whole graph", flush=True)
    batch, S = 4, 128
    manager, compiled, idg, layer, ids = build_decoder(batch, S, 512, 4, 2, 128, 1408, 1000, whole_graph=True,
                                                       streams="by_nano_batch")
    with torch.no_grad():
        manager.prepare(batch, [S] * batch)
        eager = compiled(idg).clone()
    torch.cuda.synchronize()
    replays_equal_eager(manager, lambda: torch.no_grad()(compiled)(idg),
                        lambda g: manager.prepare(batch, [S] * batch, use_cudagraph=g), eager, "caller")


def test_fp8_layer_one_stream_per_nano_batch_as_one_graph():
    print("case: fp8 layer, 4 nano-batches, streams=by_nano_batch, whole graph", flush=True)
    from dynaflow_amd.backend import make_backend
    from dynaflow_amd.config import CUDAGraphConfig, DynaFlowConfig, InductorConfig
    from dynaflow_amd.manager import DynaFlowManager

    tokens = 512
    layer, x, quantised, _ = fp8_layer(tokens, 1024, 2048, fuse_gate_up=True)
    cfg = DynaFlowConfig("dynaflow_amd.schedulers:MLPOverlapScheduler", 4, InductorConfig(enabled=True),
                         CUDAGraphConfig(enabled=False, capture_sizes=[tokens]),
                         {"min_nano_split_tokens": 1, "num_nano_batches": 4, "dump_graph": False,
                          "fuse_silu_epilogue": True, "whole_graph": True, "streams": "by_nano_batch"})
    manager = DynaFlowManager()
    torch._dynamo.reset()
    xg = x.cuda()
    torch._dynamo.mark_dynamic(xg, 0)
    compiled = torch.compile(layer, backend=make_backend(manager, cfg), fullgraph=True)
    with torch.no_grad():
        manager.prepare(tokens, [tokens])
        compiled(xg)
        manager.prepare(tokens, [tokens])
        eager = compiled(xg).clone()
    torch.cuda.synchronize()
    replays_equal_eager(manager, lambda: torch.no_grad()(compiled)(xg),
                        lambda g: manager.prepare(tokens, [tokens], use_cudagraph=g), eager, "caller")


@pytest.mark.parametrize("streams,origin", [("by_kind", "schedule"), ("by_nano_batch", "caller")])
def test_multi_layer_decode_schedule_as_one_graph(streams, origin):
    print(f"case: decode model, 3 layers = 6 sub-graphs per nano-batch, streams={streams}, whole graph", flush=True)
    T = 24
    manager, compiled, dev, host, model, inputs, cm = build_decode(T, whole_graph=True, knobs={"streams": streams})
    with torch.no_grad():
        manager.prepare(T, [1] * T, use_cudagraph=False)
        eager = compiled(*dev).clone()      # a decode step with fixed lengths is idempotent
    torch.cuda.synchronize()
    replays_equal_eager(manager, lambda: torch.no_grad()(compiled)(*dev),
                        lambda g: manager.prepare(T, [1] * T, use_cudagraph=g), eager, origin)
