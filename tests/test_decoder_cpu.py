"""Decoder layer (attention-beside-MLP configuration): pins the oracle, checks the product module
against it on the CPU, and the graph partition / schedule on the recording device."""
import math

import pytest
import torch

from dynaflow_amd import matching
from dynaflow_amd.decoder import AttentionBlock, DecoderLayer, MLPBlock, apply_rope, rope_tables
from oracle import decoder as ref

CFG = dict(vocab=97, hidden=64, heads=4, kv_heads=2, head_dim=16, inter=160, seq_len=12, theta=500000.0)


def small_layer(dtype=torch.float64):
    layer = DecoderLayer(**CFG, dtype=dtype)
    layer.init_weights(seed=3, std=0.2)
    with torch.no_grad():
        layer.attn.norm_weight.copy_(1 + 0.1 * torch.randn(CFG["hidden"], generator=torch.Generator().manual_seed(1)))
        layer.mlp.norm_weight.copy_(1 + 0.1 * torch.randn(CFG["hidden"], generator=torch.Generator().manual_seed(2)))
    return layer


def test_oracle_rope_is_a_rotation_with_relative_phase():
    t = torch.randn(1, 9, 2, 16, dtype=torch.float64)
    r = ref.rope(t, 500000.0)
    assert torch.allclose(r.norm(dim=-1), t.norm(dim=-1))
    assert torch.allclose(r[:, 0], t[:, 0])                      # position 0 is not rotated
    # dot products depend only on the position difference
    q = torch.randn(16, dtype=torch.float64); k = torch.randn(16, dtype=torch.float64)
    qs = ref.rope(q.expand(1, 9, 1, 16).clone(), 500000.0)[0, :, 0]
    ks = ref.rope(k.expand(1, 9, 1, 16).clone(), 500000.0)[0, :, 0]
    assert torch.allclose(qs[5] @ ks[2], qs[8] @ ks[5]) and torch.allclose(qs[3] @ ks[3], q @ k)


def test_oracle_attention_is_causal_and_normalised():
    q = torch.randn(1, 7, 4, 8, dtype=torch.float64)
    k = torch.randn(1, 7, 2, 8, dtype=torch.float64)
    v = torch.randn(1, 7, 2, 8, dtype=torch.float64)
    out = ref.attention(q, k, v)
    assert torch.allclose(out[0, 0], v[0, 0].repeat_interleave(2, dim=0))   # first token attends to itself only
    k2, v2 = k.clone(), v.clone()
    k2[0, 5:], v2[0, 5:] = 0.3, -0.7                                         # later tokens do not matter earlier
    assert torch.allclose(ref.attention(q, k2, v2)[0, :5], out[0, :5])
    ones = ref.attention(q, k, torch.ones_like(v))
    assert torch.allclose(ones, torch.ones_like(ones))                        # softmax rows sum to 1


def test_product_module_matches_oracle_float64():
    layer = small_layer()
    ids = torch.randint(0, CFG["vocab"], (3 * CFG["seq_len"],), generator=torch.Generator().manual_seed(4))
    with torch.no_grad():
        got = layer(ids)
    want = ref.decoder_layer(ids, ref.params_of(layer), CFG["seq_len"], CFG["heads"], CFG["kv_heads"], CFG["head_dim"])
    # the product rotates in fp32 (by design, like the bf16 path); everything else is float64 here
    assert (got - want).abs().max() / want.abs().max() < 1e-6


def test_sampled_row_oracle_equals_the_whole_layer_oracle():
    """decoder_layer_rows (what the full-size GPU test compares with) against decoder_layer on every row."""
    layer = small_layer()
    ids = torch.randint(0, CFG["vocab"], (3 * CFG["seq_len"],), generator=torch.Generator().manual_seed(5))
    params = ref.params_of(layer)
    whole = ref.decoder_layer(ids, params, CFG["seq_len"], CFG["heads"], CFG["kv_heads"], CFG["head_dim"])
    rows = list(range(3 * CFG["seq_len"]))
    got = ref.decoder_layer_rows(ids, params, rows, CFG["seq_len"], CFG["heads"], CFG["kv_heads"], CFG["head_dim"])
    assert got.shape == whole.shape
    assert (got - whole).abs().max() / whole.abs().max() < 1e-12


def test_product_rope_matches_oracle():
    cos, sin = rope_tables(12, 16, 500000.0, torch.float64)
    t = torch.randn(2, 12, 3, 16, dtype=torch.float64)
    assert torch.allclose(apply_rope(t, cos, sin), ref.rope(t, 500000.0), atol=1e-6)


def traced(layer, ids):
    captured = {}

    def backend(gm, example_inputs):
        captured["gm"] = gm
        return gm

    torch._dynamo.reset()
    torch._dynamo.mark_dynamic(ids, 0)
    torch.compile(layer, backend=backend, fullgraph=True)(ids)
    return captured["gm"]


def test_mod_rule_cuts_the_layer_into_attention_and_mlp():
    from dynaflow_amd.schedulers.decoder_overlap import decoder_split_rules, decoder_tag_rules

    layer = small_layer(torch.float32)
    ids = torch.randint(0, CFG["vocab"], (4 * CFG["seq_len"],))
    gm = traced(layer, ids)
    nodes = list(gm.graph.nodes)
    ids_map = matching.assign_partition_ids(nodes, decoder_split_rules())
    owners = {}
    for n in nodes:
        if n.op == "call_function":
            info = matching.Mod.get_module_info(n)
            owners.setdefault(ids_map[n], set()).add(info[1].__name__ if info else None)
    # Parameters lifted to placeholders carry their module in the meta data too, so a run of MLP
    # parameters in front of the graph is matched as well (its id is never used: the partitioner
    # ignores placeholder ids).  Of the compute nodes, exactly the MLP ones share one odd id.
    mlp_ids = [i for i, who in owners.items() if who == {"MLPBlock"}]
    assert len(mlp_ids) == 1 and mlp_ids[0] % 2 == 1
    assert all("MLPBlock" not in who for i, who in owners.items() if i != mlp_ids[0])
    # the oracle's restatement numbers the same node list identically
    from oracle import partition as ref_partition
    from test_oracle_partition import to_records, to_ref_rule

    want = ref_partition.partition_ids(to_records(nodes), [to_ref_rule(r) for r in decoder_split_rules()])
    assert [ids_map[n] for n in nodes] == want
    split = matching.split_graph(gm, decoder_split_rules())
    names = [n.target for n in split.graph.nodes if n.op == "call_module"]
    assert len(names) == 2 and names[1] == f"submod_{mlp_ids[0]}"
    matching.tag_graph(split, decoder_tag_rules())
    assert getattr(split, names[0]).tag == set() and getattr(split, names[1]).tag == {"mlp"}


def test_decoder_schedule_on_recording_device(host_device):
    from dynaflow_amd.backend import make_backend
    from dynaflow_amd.config import CUDAGraphConfig, DynaFlowConfig, InductorConfig
    from dynaflow_amd.manager import DynaFlowManager

    layer = small_layer(torch.float32)
    S = CFG["seq_len"]
    ids = torch.randint(0, CFG["vocab"], (6 * S,), generator=torch.Generator().manual_seed(5))
    cfg = DynaFlowConfig("dynaflow_amd.schedulers:DecoderOverlapScheduler", 2, InductorConfig(enabled=False),
                         CUDAGraphConfig(enabled=False, capture_sizes=[6 * S]),
                         {"min_nano_split_tokens": 1, "dump_graph": False})
    manager = DynaFlowManager()
    torch._dynamo.reset()
    torch._dynamo.mark_dynamic(ids, 0)
    compiled = torch.compile(layer, backend=make_backend(manager, cfg), fullgraph=True)
    with torch.no_grad():
        manager.prepare(6, [S] * 6)
        compiled(ids)
        split = manager.prepare(6, [S] * 6)
        y = compiled(ids)
        want = layer(ids)
    assert split.batch_indices == [0, 3, 6] and split.split_indices == [0, 3 * S, 6 * S]
    a, m = [n.target for n in manager.graph_module.graph.nodes if n.op == "call_module"]
    assert manager.engine.issue_trace == [(a, 0), (m, 0), (a, 1), (m, 1)]
    streams = [e[2] for e in host_device.log if e[0] == "range"][-4:]
    assert streams == ["main", "side", "main", "side"]
    torch.testing.assert_close(y, want, rtol=1e-5, atol=1e-5)
