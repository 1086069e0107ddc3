"""Pins oracle/partition.py with hand-derived goldens and invariants, then checks
dynaflow_amd.matching against it on real torch.fx graphs (bit-exact partition ids)."""
import operator
import random

import pytest
import torch
import torch.fx as fx
import torch.nn.functional as F

from conftest import load_golden
from dynaflow_amd import matching
from oracle import partition as ref

CASES = load_golden("partition_cases.json")
_CLASSES: dict = {}


def cls_of(name):
    if name not in _CLASSES:
        _CLASSES[name] = type(name, (torch.nn.Module,), {})
    return _CLASSES[name]


HOOKS = {None: None, "never": lambda nodes, i: False, "always": lambda nodes, i: True,
         "not_first_position": lambda nodes, i: i != 1}


def build_nodes(raw):
    nodes = []
    for op, name, stack in raw:
        node = {"op": op, "name": name}
        if stack is not None:
            node["stack"] = [(q, cls_of(c)) for q, c in stack]
        nodes.append(node)
    return nodes


def build_rule(raw):
    cond = [(k, cls_of(a) if k == "mod" else a) for k, a in raw["cond"]]
    return {"cond": cond, "hook": HOOKS[raw["hook"]]}


@pytest.mark.parametrize("case", CASES["partition"], ids=lambda c: c["name"])
def test_partition_golden(case):
    nodes = build_nodes(case["nodes"])
    rules = [build_rule(r) for r in case["rules"]]
    assert ref.partition_ids(nodes, rules) == case["expect"]


@pytest.mark.parametrize("case", CASES["tags"], ids=lambda c: c["name"])
def test_tags_golden(case):
    nodes = build_nodes(case["nodes"])
    tag_rules = [(build_rule(r), set(t)) for r, t in case["tag_rules"]]
    assert sorted(ref.subgraph_tags(nodes, tag_rules)) == case["expect"]


def test_partition_invariants_random():
    rng = random.Random(3)
    names = ["linear", "silu", "mul", "add", "getitem", "relu"]
    rules = [{"cond": [("op", "silu"), ("op", "mul")], "hook": None}, {"cond": [("op", "relu")], "hook": None}]
    for _ in range(500):
        nodes = [{"op": "placeholder", "name": None}]
        nodes += [{"op": "call_function", "name": rng.choice(names)} for _ in range(rng.randint(1, 15))]
        nodes.append({"op": "output", "name": None})
        ids = ref.partition_ids(nodes, rules)
        assert len(ids) == len(nodes)
        assert all(a <= b for a, b in zip(ids, ids[1:])), "ids never decrease along the node list"
        # a matched span owns its id: ids of matched spans are odd, unmatched stretches even
        for node, pid in zip(nodes, ids):
            if node["name"] in ("relu",):
                assert pid % 2 == 1


# ------------------------------------------------------------------ product vs oracle on fx graphs
def to_records(nodes):
    out = []
    for n in nodes:
        rec = {"op": n.op, "name": getattr(n.target, "__name__", None) if n.op == "call_function" else None}
        if "nn_module_stack" in n.meta:
            rec["stack"] = list(n.meta["nn_module_stack"].values())
        out.append(rec)
    return out


def to_ref_rule(rule):
    conds = rule.condition if isinstance(rule.condition, tuple) else (rule.condition,)
    cond = [("op", c.pattern) if isinstance(c, matching.Op) else ("mod", c.target_cls) for c in conds]
    hook = None
    if rule.hook is not None:
        hook = lambda recs, i, _h=rule.hook, _n=None: _h(_CURRENT_FX_NODES, i)
    return {"cond": cond, "hook": hook}


_CURRENT_FX_NODES: list = []


def assert_same_partition(gm, rules):
    global _CURRENT_FX_NODES
    nodes = list(gm.graph.nodes)
    _CURRENT_FX_NODES = nodes
    got = matching.assign_partition_ids(nodes, rules)
    want = ref.partition_ids(to_records(nodes), [to_ref_rule(r) for r in rules])
    assert [got[n] for n in nodes] == want
    return want


def hand_graph(names):
    """fx graph x -> chain of the named functions (getitem via a tuple producer)."""
    fns = {"linear": F.linear, "silu": F.silu, "mul": operator.mul, "relu": F.relu, "add": operator.add,
           "getitem": operator.getitem}
    g = fx.Graph()
    x = g.placeholder("x")
    cur = x
    for name in names:
        if name in ("linear", "mul", "add"):
            cur = g.call_function(fns[name], (cur, x))
        elif name == "getitem":
            cur = g.call_function(operator.getitem, (cur, 0))
        else:
            cur = g.call_function(fns[name], (cur,))
    g.output(cur)
    return fx.GraphModule(torch.nn.Module(), g)


@pytest.mark.parametrize("names", [
    ["linear", "linear", "silu", "mul", "linear"],
    ["linear", "silu", "linear", "mul", "linear"],
    ["silu", "silu", "linear"],
    ["linear", "getitem", "getitem", "silu", "mul"],
    ["silu", "getitem", "mul", "linear", "relu"],
    ["relu", "add", "relu"],
])
def test_matching_equals_oracle_on_hand_graphs(names):
    rules = [matching.MatchingRule((matching.Op("silu"), matching.Op("mul"), matching.Op("linear"))),
             matching.MatchingRule((matching.Op("silu"), matching.Op("mul"))),
             matching.MatchingRule(matching.Op("relu"), hook=lambda nodes, i: nodes[i].prev.op != "placeholder")]
    assert_same_partition(hand_graph(names), rules)


def test_matching_equals_oracle_on_random_graphs():
    rng = random.Random(7)
    rules = [matching.MatchingRule((matching.Op("silu"), matching.Op("mul"))),
             matching.MatchingRule(matching.Op(r"re.u"))]
    for _ in range(200):
        names = [rng.choice(["linear", "silu", "mul", "add", "getitem", "relu"]) for _ in range(rng.randint(1, 12))]
        assert_same_partition(hand_graph(names), rules)


def dynamo_graph(module, x):
    captured = {}

    def backend(gm, example_inputs):
        captured["gm"] = gm
        return gm

    torch._dynamo.reset()
    torch._dynamo.mark_dynamic(x, 0)
    torch.compile(module, backend=backend, fullgraph=True)(x)
    return captured["gm"]


def test_mlp_graph_partition_and_submodules():
    from dynaflow_amd.mlp import SwiGLUMLP
    from dynaflow_amd.schedulers.mlp_overlap import mlp_split_rules, mlp_tag_rules

    gm = dynamo_graph(SwiGLUMLP(32, 96, dtype=torch.float32), torch.randn(16, 32))
    ids = assert_same_partition(gm, mlp_split_rules())
    compute = [(n.target.__name__, i) for n, i in zip(gm.graph.nodes, ids) if n.op == "call_function"]
    assert compute == [("linear", 0), ("linear", 0), ("silu", 1), ("mul", 1), ("linear", 1)]
    split = matching.split_graph(gm, mlp_split_rules())
    names = [n.target for n in split.graph.nodes if n.op == "call_module"]
    assert names == ["submod_0", "submod_1"]
    matching.tag_graph(split, mlp_tag_rules())
    assert split.submod_0.tag == set() and split.submod_1.tag == {"tail"}
    # the oracle's tagger agrees on the sub-graph node lists
    tag_rules = [(to_ref_rule(r), t) for r, t in mlp_tag_rules().items()]
    assert ref.subgraph_tags(to_records(split.submod_1.graph.nodes), tag_rules) == {"tail"}
    assert ref.subgraph_tags(to_records(split.submod_0.graph.nodes), tag_rules) == set()


def test_mod_condition_on_dynamo_graph():
    class Block(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.a = torch.nn.Linear(8, 8)
            self.b = torch.nn.Linear(8, 8)

        def forward(self, x):
            return self.b(torch.relu(self.a(x)))

    gm = dynamo_graph(Block(), torch.randn(4, 8))
    rules = [matching.MatchingRule(matching.Mod(torch.nn.Linear))]
    ids = assert_same_partition(gm, rules)
    by_name = {n.name: i for n, i in zip(gm.graph.nodes, ids)}
    linears = [n.name for n in gm.graph.nodes if n.op == "call_function" and n.target.__name__ == "linear"]
    assert len(linears) == 2 and by_name[linears[0]] != by_name[linears[1]]
    assert by_name[linears[0]] % 2 == 1 and by_name[linears[1]] % 2 == 1
