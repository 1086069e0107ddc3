"""The HIP lowering pass on traced graphs (graph surgery only; nothing runs)."""
import torch

from dynaflow_amd import matching, ops
from dynaflow_amd.executor.hip_lowering import lower_to_hip
from dynaflow_amd.mlp import SwiGLUMLP
from dynaflow_amd.schedulers.mlp_overlap import mlp_split_rules


def traced(dtype, hidden=64, inter=128):
    captured = {}

    def backend(gm, example_inputs):
        captured["gm"] = gm
        return gm

    torch._dynamo.reset()
    x = torch.randn(16, hidden).to(dtype)
    torch._dynamo.mark_dynamic(x, 0)
    torch.compile(SwiGLUMLP(hidden, inter, dtype=dtype), backend=backend, fullgraph=True)(x)
    return matching.split_graph(captured["gm"], mlp_split_rules())


def targets(gm):
    return [n.target for n in gm.graph.nodes if n.op == "call_function"]


def test_bf16_mlp_subgraphs_are_fully_lowered():
    split = traced(torch.bfloat16)
    head, stats0 = lower_to_hip(split.submod_0)
    tail, stats1 = lower_to_hip(split.submod_1)
    assert stats0 == {"linear": 0, "silu_mul": 0, "linear_multi": 1}
    assert stats1 == {"linear": 1, "silu_mul": 1, "to_output": 1}
    # gate and up projection of the same activation: one GEMM against the stacked weights, two column ranges
    import operator
    assert targets(head) == [ops.linear_multi, operator.getitem, operator.getitem]
    multi = next(n for n in head.graph.nodes if n.target is ops.linear_multi)
    assert len(multi.args[1]) == 2 and all(w.op == "placeholder" for w in multi.args[1])
    # the projection that the sub-graph returns may write into output rows offered by the engine
    assert targets(tail) == [ops.silu_mul, ops.linear_to_output]
    silu_mul = next(n for n in tail.graph.nodes if n.target is ops.silu_mul)
    assert silu_mul.args[2] is True  # bf16: silu rounded before the product, like two aten kernels
    # the original sub-graph is untouched
    assert ops.linear not in targets(split.submod_0)


def test_fp32_is_lowered_without_intermediate_rounding_flag():
    split = traced(torch.float32)
    tail, stats = lower_to_hip(split.submod_1)
    assert stats == {"linear": 1, "silu_mul": 1, "to_output": 1}
    silu_mul = next(n for n in tail.graph.nodes if n.target is ops.silu_mul)
    assert silu_mul.args[2] is False


def test_unsupported_shapes_stay_on_aten():
    split = traced(torch.bfloat16, hidden=40, inter=72)  # K % 64 != 0
    head, stats = lower_to_hip(split.submod_0)
    assert stats["linear"] == 0
    assert all(t is not ops.linear for t in targets(head))


def test_lowered_graph_fails_loudly_on_the_host():
    import pytest

    split = traced(torch.bfloat16)
    head, _ = lower_to_hip(split.submod_0)
    x = torch.randn(16, 64).bfloat16()
    w = torch.randn(128, 64).bfloat16()
    with pytest.raises((RuntimeError, NotImplementedError)):
        head(x, 16, w, w)


def test_decoder_layer_rope_and_norms_are_lowered():
    from dynaflow_amd.decoder import DecoderLayer

    captured = {}

    def backend(gm, example_inputs):
        captured["gm"] = gm
        return gm

    torch._dynamo.reset()
    layer = DecoderLayer(vocab=64, hidden=128, heads=4, kv_heads=2, head_dim=32, inter=256, seq_len=8)
    layer.init_weights(0)
    ids = torch.arange(16) % 64
    torch.compile(layer, backend=backend, fullgraph=True)(ids)
    names = [getattr(n.target, "__name__", "") for n in captured["gm"].graph.nodes if n.op == "call_function"]
    assert names.count("apply_rope") == 2          # q and k, each ONE node: dynamo does not trace into it
    lowered, stats = lower_to_hip(captured["gm"])
    assert stats["rope"] == 2 and stats["rms_norm"] == 2
    # 7 projections: q / k / v and gate / up each become one GEMM against stacked weights
    assert stats["linear"] == 2 and stats["linear_multi"] == 2
    multis = [n for n in lowered.graph.nodes if n.target is ops.linear_multi]
    assert sorted(len(n.args[1]) for n in multis) == [2, 3]
    # ... and the two rotations share their tables: one operator for q and k
    assert stats["rope_pair"] == 1 and targets(lowered).count(ops.rope_pair) == 1 and ops.rope not in targets(lowered)


def test_decoder_layer_attention_is_lowered_for_head_dim_128():
    from dynaflow_amd.decoder import DecoderLayer

    captured = {}

    def backend(gm, example_inputs):
        captured["gm"] = gm
        return gm

    torch._dynamo.reset()
    layer = DecoderLayer(vocab=64, hidden=256, heads=4, kv_heads=2, head_dim=128, inter=256, seq_len=64)
    layer.init_weights(0)
    ids = torch.arange(128) % 64
    torch._dynamo.mark_dynamic(ids, 0)
    torch.compile(layer, backend=backend, fullgraph=True)(ids)
    names = [getattr(n.target, "__name__", "") for n in captured["gm"].graph.nodes if n.op == "call_function"]
    assert names.count("causal_gqa_attention") == 1            # one node: dynamo does not trace into it
    lowered, stats = lower_to_hip(captured["gm"])
    assert stats["causal_attention"] == 1 and stats["rope"] == 2
    assert targets(lowered).count(ops.causal_attention) == 1
    # a sequence length the kernel does not take (not a multiple of 64) stays on the tensor operations
    torch._dynamo.reset()
    layer = DecoderLayer(vocab=64, hidden=256, heads=4, kv_heads=2, head_dim=128, inter=256, seq_len=48)
    layer.init_weights(0)
    ids = torch.arange(96) % 64
    torch._dynamo.mark_dynamic(ids, 0)
    torch.compile(layer, backend=backend, fullgraph=True)(ids)
    _, stats = lower_to_hip(captured["gm"])
    assert "causal_attention" not in stats


def test_stacked_weight_cache_keys_and_lifetime():
    """The cache behind ``linear_multi`` on host tensors (the logic has no device part): an entry dies with its
    weights, so an address that the allocator reuses never finds an old concatenation; an in-place write and a
    swapped ``.data`` are seen; a write through ``.data`` needs ``invalidate``."""
    import gc

    from dynaflow_amd.ops import StackedWeightCache

    cache = StackedWeightCache()
    builds = []

    def stack(ws):
        def build():
            builds.append(1)
            return torch.cat([w.detach() for w in ws], dim=0)
        return build

    a, b = torch.randn(8, 16), torch.randn(24, 16)
    s1 = cache.get([a, b], stack([a, b]))
    assert cache.get([a, b], stack([a, b])) is s1 and len(builds) == 1
    assert torch.equal(s1, torch.cat([a, b]))
    # K and the row count are part of the key: a view of the same storage with another shape is another group
    a_wide = a.view(4, 32)
    b_wide = b.view(12, 32)
    assert cache.get([a_wide, b_wide], stack([a_wide, b_wide])).shape == (16, 32) and len(builds) == 2

    # in-place write: new version counter, new entry, the stale one is gone
    a.mul_(2.0)
    s2 = cache.get([a, b], stack([a, b]))
    assert s2 is not s1 and torch.equal(s2[:8], a) and len(cache) == 2

    # .data pointed at another tensor: new address, new entry
    a.data = torch.ones(8, 16)
    s3 = cache.get([a, b], stack([a, b]))
    assert torch.equal(s3[:8], torch.ones(8, 16)) and len(cache) == 2

    # a write THROUGH .data does not touch the version counter: stale until invalidated
    a.data.copy_(torch.full((8, 16), 3.0))
    assert cache.get([a, b], stack([a, b])) is s3 and not torch.equal(s3[:8], a)
    cache.invalidate([a])
    s4 = cache.get([a, b], stack([a, b]))
    assert torch.equal(s4[:8], a)

    # entries die with their weights; a new tensor that lands on a freed weight's address starts from nothing
    address, version = a.data_ptr(), a._version
    del a, a_wide, s1, s2, s3, s4
    gc.collect()
    assert len(cache) == 0
    reused = None
    for _ in range(64):                                   # the host allocator usually hands the block straight back
        t = torch.zeros(8, 16)
        if t.data_ptr() == address:
            reused = t
            break
    if reused is not None:
        n = len(builds)
        s5 = cache.get([reused, b], stack([reused, b]))
        assert len(builds) == n + 1 and torch.equal(s5[:8], reused)

    # build() may decline (under stream capture): nothing is kept
    assert cache.get([b], lambda: None) is None and len(cache) == (1 if reused is not None else 0)
    cache.invalidate()
    assert len(cache) == 0


def test_side_by_side_option_and_the_plan_for_shared_launches():
    """``launch_options(side_by_side=n)`` (knob ``side_by_side``) holds for the launches issued inside the block
    and comes back afterwards, also after an exception.  The plan for launches that share the GPU (host logic of
    the library, no GPU needed): the down projection of a 2048-token nano-batch of the 8B shape - 128 tiles of
    256 x 256 - splits K in two alone and not at all beside a second one; the gate projection keeps its 224-wide
    tiles either way; decode-sized activations keep the weight-streaming kernel and its split."""
    import ctypes
    from dynaflow_amd import _cabi, ops

    assert ops._side_by_side() == 1
    with ops.launch_options(side_by_side=2):
        assert ops._side_by_side() == 2
        with ops.launch_options(side_by_side=1):
            assert ops._side_by_side() == 1
        assert ops._side_by_side() == 2
    try:
        with ops.launch_options(side_by_side=4):
            raise RuntimeError("inside")
    except RuntimeError:
        pass
    assert ops._side_by_side() == 1

    lib = _cabi.load()

    def plan(M, N, K, share):
        v, k = ctypes.c_int(), ctypes.c_int()
        assert lib.dfhip_gemm_bf16_plan_shared(M, N, K, share, ctypes.byref(v), ctypes.byref(k)) == 0
        return v.value, k.value

    def plan_alone(M, N, K):
        v, k = ctypes.c_int(), ctypes.c_int()
        assert lib.dfhip_gemm_bf16_plan(M, N, K, ctypes.byref(v), ctypes.byref(k)) == 0
        return v.value, k.value

    for shape in ((2048, 4096, 14336), (2048, 14336, 4096), (128, 4096, 4096), (8192, 4096, 4096), (300, 264, 512)):
        assert plan(*shape, 1) == plan_alone(*shape)
    assert plan(2048, 4096, 14336, 1) == (0, 2)
    assert plan(2048, 4096, 14336, 2) == (0, 1)
    assert plan(1024, 4096, 14336, 2) == (0, 2)          # 64 tiles, twice: still two parts each
    assert plan(2048, 14336, 4096, 1) == plan(2048, 14336, 4096, 2) == (5, 1)
    # the weight-streaming kernel: one round of workgroups for all the launches that share the GPU
    assert plan(128, 4096, 4096, 1) == (6, 5) and plan(128, 4096, 4096, 2) == (6, 4)
    assert plan(128, 4096, 14336, 1) == (6, 8) and plan(128, 4096, 14336, 2) == (6, 4)
    assert plan(128, 6144, 4096, 2) == (6, 2) and plan(128, 14336, 4096, 2) == (6, 1)
    v, k = ctypes.c_int(), ctypes.c_int()
    assert lib.dfhip_gemm_bf16_plan_shared(2048, 4096, 14336, 0, ctypes.byref(v), ctypes.byref(k)) == -7
