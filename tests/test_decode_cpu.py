"""Decode step on the host: the oracle against special cases and the prefill oracle, the product module
(plain tensor operations) against the oracle, the graph cut and the schedule on the recording device."""
import pytest
import torch

from dynaflow_amd import matching
from dynaflow_amd.decode import DecodeModel, attend_and_append, pack_v_cache, unpack_v_cache
from dynaflow_amd.decoder import MLPBlock
from oracle import decode as ref
from oracle import decoder as ref_prefill

CFG = dict(layers=2, vocab=50, hidden=64, heads=4, kv_heads=2, inter=96, slots=6, capacity=32)
D = 128


def small_model(dtype=torch.float64, **over):
    cfg = dict(CFG, **over)
    model = DecodeModel(**cfg, dtype=dtype)
    model.init_weights(3, std=0.1)
    model.fill_caches(7)
    with torch.no_grad():
        for i, blk in enumerate(model.attn):
            blk.norm_weight.copy_(1 + 0.1 * torch.randn(cfg["hidden"], generator=torch.Generator().manual_seed(i)))
    return model


def test_v_cache_layout_round_trip():
    v = torch.arange(2 * 3 * 16 * D, dtype=torch.float32).view(2, 3, 16, D)
    packed = pack_v_cache(v)
    assert packed.shape == (2, 3, 2, D, 8)
    assert packed[1, 2, 1, 5, 3] == v[1, 2, 8 + 3, 5]       # [slot, head, pos // 8, dim, pos % 8]
    assert torch.equal(unpack_v_cache(packed), v)


def test_oracle_attend_special_cases():
    g = torch.Generator().manual_seed(0)
    q = torch.randn(4, 8, dtype=torch.float64, generator=g)
    k = torch.randn(5, 2, 8, dtype=torch.float64, generator=g)
    v = torch.randn(5, 2, 8, dtype=torch.float64, generator=g)
    one = ref.attend(q, k[:1], v[:1])                           # a single position: its value, per group
    assert torch.allclose(one, v[0].repeat_interleave(2, dim=0))
    const = ref.attend(q, k, torch.full_like(v, 0.25))          # softmax weights sum to 1
    assert torch.allclose(const, torch.full_like(const, 0.25))
    big = k.clone(); big[3] = 50 * q[0]                         # head 0 is dominated by position 3
    assert torch.allclose(ref.attend(q, big, v)[0], v[3, 0], atol=1e-9)
    assert not torch.allclose(ref.attend(q, big, v)[3], v[3, 1], atol=1e-3)   # heads 2, 3 read kv head 1


def test_oracle_rope_at_matches_prefill_rotation():
    t = torch.randn(1, 9, 3, 16, dtype=torch.float64)
    want = ref_prefill.rope(t, 500000.0)[0]
    got = ref.rope_at(t[0], torch.arange(9), 500000.0)
    assert torch.allclose(got, want)
    shuffled = torch.tensor([4, 0, 7])
    assert torch.allclose(ref.rope_at(t[0, shuffled], shuffled, 500000.0), want[shuffled])


def test_oracle_token_by_token_decode_equals_prefill():
    """Causal attention over a whole sequence == decoding it one token at a time into an empty cache."""
    from dynaflow_amd.decoder import DecoderLayer

    S, heads, kv_heads = 7, 2, 1
    layer = DecoderLayer(vocab=40, hidden=32, heads=heads, kv_heads=kv_heads, head_dim=D, inter=48, seq_len=S,
                         dtype=torch.float64)
    layer.init_weights(1, std=0.1)
    ids = torch.randint(0, 40, (2 * S,), generator=torch.Generator().manual_seed(2))
    P = ref_prefill.params_of(layer)
    want = ref_prefill.decoder_layer(ids, P, S, heads, kv_heads, D).view(2, S, -1)
    params = {"embed": P["embed"], "attn_norm.0": P["attn_norm"], "wqkv.0": torch.cat([P["wq"], P["wk"], P["wv"]]),
              "wo.0": P["wo"], "mlp_norm.0": P["mlp_norm"], "w_gate.0": P["w_gate"], "w_up.0": P["w_up"],
              "w_down.0": P["w_down"]}
    kc = [torch.zeros(2, 8, kv_heads, D, dtype=torch.float64)]
    vc = [torch.zeros(2, 8, kv_heads, D, dtype=torch.float64)]
    for step in range(S):
        tok = ids.view(2, S)[:, step]
        out = ref.decode_step(tok, torch.tensor([1, 0]), torch.tensor([step + 1, step + 1]), params, kc, vc,
                              heads, kv_heads)
        assert torch.allclose(out, want[:, step], atol=1e-10), step


def decode_inputs(T, cfg=CFG, seed=11):
    g = torch.Generator().manual_seed(seed)
    ids = torch.randint(0, cfg["vocab"], (T,), generator=g)
    slots = torch.randperm(cfg["slots"], generator=g)[:T].int()
    lengths = torch.randint(1, cfg["capacity"] + 1, (T,), generator=g).int()
    lengths[0] = 1
    lengths[-1] = cfg["capacity"]
    return ids, slots, lengths


def test_product_module_matches_oracle_float64():
    model = small_model()
    ids, slots, lengths = decode_inputs(5)
    params = ref.params_of(model)
    kc, vc = ref.caches_of(model)
    want = ref.decode_step(ids, slots, lengths, params, kc, vc, CFG["heads"], CFG["kv_heads"])
    with torch.no_grad():
        got = model(ids, slots, lengths)
    assert (got - want).abs().max() / want.abs().max() < 1e-6        # the product rotates with fp32 tables
    kc2, vc2 = ref.caches_of(model)                                   # the appended entries agree too
    for a, b in zip(kc + vc, kc2 + vc2):
        assert (a - b).abs().max() < 1e-6


def test_attend_and_append_touches_only_the_new_position():
    model = small_model()
    blk = model.attn[0]
    before_k, before_v = blk.k_cache.clone(), blk.v_cache.clone()
    ids, slots, lengths = decode_inputs(4)
    qkv = torch.randn(4, (CFG["heads"] + 2 * CFG["kv_heads"]) * D, dtype=torch.float64)
    attend_and_append(qkv, blk.k_cache, blk.v_cache, slots, lengths, model.cos, model.sin, CFG["heads"],
                      CFG["kv_heads"])
    changed_k = (blk.k_cache != before_k).any(dim=-1).nonzero()
    assert sorted(set(map(tuple, changed_k[:, [0, 2]].tolist()))) == sorted(
        {(int(s), int(n) - 1) for s, n in zip(slots, lengths)})
    natural_before, natural_after = unpack_v_cache(before_v), unpack_v_cache(blk.v_cache)
    changed_v = (natural_after != natural_before).any(dim=-1).nonzero()
    assert sorted(set(map(tuple, changed_v[:, [0, 2]].tolist()))) == sorted(
        {(int(s), int(n) - 1) for s, n in zip(slots, lengths)})
    want_v = qkv[:, (CFG["heads"] + CFG["kv_heads"]) * D:].view(4, CFG["kv_heads"], D)
    for t in range(4):
        assert torch.equal(natural_after[int(slots[t]), :, int(lengths[t]) - 1], want_v[t])


def traced_decode(model, T):
    captured = {}

    def backend(gm, example_inputs):
        captured["gm"] = gm
        return gm

    torch._dynamo.reset()
    ids, slots, lengths = decode_inputs(T)
    for t in (ids, slots, lengths):
        torch._dynamo.mark_dynamic(t, 0)
    with torch.no_grad():
        torch.compile(model, backend=backend, fullgraph=True)(ids, slots, lengths)
    return captured["gm"]


def test_decode_graph_is_cut_into_attention_and_mlp_per_layer():
    model = small_model()
    gm = traced_decode(model, 4)
    names = [getattr(n.target, "__name__", "").split(".")[0] for n in gm.graph.nodes if n.op == "call_function"]
    assert names.count("attend_and_append") == CFG["layers"]    # one node per layer: an operator of its own
    split = matching.split_graph(gm, [matching.MatchingRule(condition=matching.Mod(MLPBlock))])
    subs = [n.target for n in split.graph.nodes if n.op == "call_module"]
    assert len(subs) == 2 * CFG["layers"]
    for i, name in enumerate(subs):
        inner = [getattr(n.target, "__name__", "").split(".")[0] for n in getattr(split, name).graph.nodes
                 if n.op == "call_function"]
        assert ("attend_and_append" in inner) == (i % 2 == 0)
        assert ("silu" in inner) == (i % 2 == 1)


def test_decode_lowering_replaces_attention_node():
    from dynaflow_amd import ops
    from dynaflow_amd.executor.hip_lowering import lower_to_hip

    model = small_model(dtype=torch.bfloat16)
    gm = traced_decode(model, 4)
    lowered, stats = lower_to_hip(gm)
    assert stats["decode_attention"] == CFG["layers"]
    assert [n.target for n in lowered.graph.nodes if n.op == "call_function"].count(ops.decode_attention) == CFG["layers"]


def test_decode_schedule_on_recording_device(host_device):
    """Through manager, engine and scheduler on the host: two nano-batches of sequences, attention of one
    beside the MLP of the other in every layer, same result as the unsplit module and as the oracle."""
    from dynaflow_amd.backend import make_backend
    from dynaflow_amd.config import CUDAGraphConfig, DynaFlowConfig, InductorConfig
    from dynaflow_amd.manager import DynaFlowManager

    model = small_model()
    twin = small_model()
    T = 6
    ids, slots, lengths = decode_inputs(T)
    with torch.no_grad():
        want = twin(ids, slots, lengths)
    cfg = DynaFlowConfig("dynaflow_amd.schedulers:DecoderOverlapScheduler", 2, InductorConfig(enabled=False),
                         CUDAGraphConfig(enabled=False, capture_sizes=[T]),
                         {"min_nano_split_tokens": 1, "dump_graph": False, "hip_backend": False})
    manager = DynaFlowManager()
    torch._dynamo.reset()
    for t in (ids, slots, lengths):
        torch._dynamo.mark_dynamic(t, 0)
    compiled = torch.compile(model, backend=make_backend(manager, cfg), fullgraph=True)
    with torch.no_grad():
        manager.prepare(T, [1] * T)
        compiled(ids, slots, lengths)
        fresh = small_model()
        for a, b in zip(model.attn, fresh.attn):          # the tracing pass appended already: start over
            a.k_cache.copy_(b.k_cache); a.v_cache.copy_(b.v_cache)
        split = manager.prepare(T, [1] * T)
        got = compiled(ids, slots, lengths)
    assert split.split_indices == [0, 3, 6]
    assert torch.allclose(got, want, atol=1e-12)
    trace = manager.engine.issue_trace
    subs = [n.target for n in manager.graph_module.graph.nodes if n.op == "call_module"]
    assert len(subs) == 2 * CFG["layers"] and len(trace) == 2 * len(subs)
    assert trace[0] == (subs[0], 0) and trace[1] == (subs[1], 0) and trace[2] == (subs[0], 1)
    for b in (0, 1):
        assert [name for name, batch in trace if batch == b] == subs
    # attention sub-graphs on the main stream, MLP sub-graphs on the side stream, in every layer
    streams = {e[1]: e[2] for e in host_device.log if e[0] == "range"}
    for i, name in enumerate(subs):
        for b in (0, 1):
            assert streams[f"op_{name}_{b}"] == ("side" if i % 2 else "main"), (name, b)
